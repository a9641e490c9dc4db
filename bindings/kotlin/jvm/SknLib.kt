// Panama FFM (JDK 22+) downcall handles for every entry point of include/skainet_hip.h, one per function, in the
// order of the header.  Lives in a JVM source set of its own compiled for JDK 22 (the reference's other JVM code
// targets 1.8 / 11 bytecode, core/build.gradle.kts:20).  Not compiled in this repository's build image (no JVM).
package sk.ai.net.hip

import java.lang.foreign.Arena
import java.lang.foreign.FunctionDescriptor
import java.lang.foreign.Linker
import java.lang.foreign.SymbolLookup
import java.lang.foreign.ValueLayout.ADDRESS
import java.lang.foreign.ValueLayout.JAVA_FLOAT
import java.lang.foreign.ValueLayout.JAVA_INT
import java.lang.foreign.ValueLayout.JAVA_LONG
import java.lang.invoke.MethodHandle

object SknLib {
    const val ABI_VERSION = 3
    const val OK = 0
    const val ERR_ARG = -1
    const val ERR_TYPE = -2
    const val ERR_SHAPE = -3
    const val ERR_OOM = -4
    const val ERR_HIP = -5
    const val ERR_RANGE = -6
    const val ERR_POOL = -7
    const val ERR_STATE = -8

    private val linker: Linker = Linker.nativeLinker()
    private val lib: SymbolLookup =
        SymbolLookup.libraryLookup(System.getProperty("skainet.hip.library", "libskainet_hip.so"), Arena.global())

    private fun h(name: String, fd: FunctionDescriptor): MethodHandle =
        linker.downcallHandle(lib.find(name).orElseThrow { UnsatisfiedLinkError("libskainet_hip lacks $name") }, fd)

    val abiVersion: MethodHandle = h("skn_abi_version", FunctionDescriptor.of(JAVA_INT))
    val init: MethodHandle = h("skn_init", FunctionDescriptor.of(JAVA_INT, JAVA_INT, ADDRESS))
    val shutdown: MethodHandle = h("skn_shutdown", FunctionDescriptor.ofVoid(ADDRESS))
    val lastError: MethodHandle = h("skn_last_error", FunctionDescriptor.of(ADDRESS, ADDRESS))
    val statusString: MethodHandle = h("skn_status_string", FunctionDescriptor.of(ADDRESS, JAVA_INT))
    val deviceInfo: MethodHandle = h("skn_device_info", FunctionDescriptor.of(JAVA_INT, ADDRESS, ADDRESS, JAVA_LONG, ADDRESS, ADDRESS))
    val typeBlock: MethodHandle = h("skn_type_block", FunctionDescriptor.of(JAVA_INT, JAVA_INT, ADDRESS, ADDRESS))
    val rowBytes: MethodHandle = h("skn_row_bytes", FunctionDescriptor.of(JAVA_LONG, JAVA_INT, JAVA_LONG))
    val malloc: MethodHandle = h("skn_malloc", FunctionDescriptor.of(JAVA_INT, ADDRESS, JAVA_LONG, ADDRESS))
    val free: MethodHandle = h("skn_free", FunctionDescriptor.of(JAVA_INT, ADDRESS, ADDRESS))
    val upload: MethodHandle = h("skn_upload", FunctionDescriptor.of(JAVA_INT, ADDRESS, ADDRESS, ADDRESS, JAVA_LONG))
    val download: MethodHandle = h("skn_download", FunctionDescriptor.of(JAVA_INT, ADDRESS, ADDRESS, ADDRESS, JAVA_LONG))
    val memset: MethodHandle = h("skn_memset", FunctionDescriptor.of(JAVA_INT, ADDRESS, ADDRESS, JAVA_INT, JAVA_LONG))
    val copy: MethodHandle = h("skn_copy", FunctionDescriptor.of(JAVA_INT, ADDRESS, ADDRESS, ADDRESS, JAVA_LONG))
    val sync: MethodHandle = h("skn_sync", FunctionDescriptor.of(JAVA_INT, ADDRESS))
    val setStream: MethodHandle = h("skn_set_stream", FunctionDescriptor.of(JAVA_INT, ADDRESS, ADDRESS))
    val setOption: MethodHandle = h("skn_set_option", FunctionDescriptor.of(JAVA_INT, ADDRESS, ADDRESS, JAVA_INT))
    val getStat: MethodHandle = h("skn_get_stat", FunctionDescriptor.of(JAVA_INT, ADDRESS, ADDRESS, ADDRESS))
    val timerStart: MethodHandle = h("skn_timer_start", FunctionDescriptor.of(JAVA_INT, ADDRESS))
    val timerStop: MethodHandle = h("skn_timer_stop", FunctionDescriptor.of(JAVA_INT, ADDRESS, ADDRESS))
    val profStart: MethodHandle = h("skn_prof_start", FunctionDescriptor.of(JAVA_INT, ADDRESS, JAVA_INT))
    val profStop: MethodHandle = h("skn_prof_stop", FunctionDescriptor.of(JAVA_INT, ADDRESS, ADDRESS, ADDRESS))
    val dequant: MethodHandle = h("skn_dequant", FunctionDescriptor.of(JAVA_INT, ADDRESS, JAVA_INT, ADDRESS, JAVA_LONG, ADDRESS))
    val matvecQ: MethodHandle = h("skn_matvec_q", FunctionDescriptor.of(JAVA_INT, ADDRESS, JAVA_INT, ADDRESS, JAVA_INT, JAVA_INT, ADDRESS, ADDRESS))
    val gemmQ: MethodHandle = h("skn_gemm_q", FunctionDescriptor.of(JAVA_INT, ADDRESS, JAVA_INT, ADDRESS, JAVA_INT, JAVA_INT, ADDRESS, JAVA_INT, ADDRESS))
    val gemmExpandedBytes: MethodHandle = h("skn_gemm_expanded_bytes", FunctionDescriptor.of(JAVA_INT, ADDRESS, JAVA_INT, JAVA_INT, JAVA_INT, ADDRESS))
    val gemmExpand: MethodHandle = h("skn_gemm_expand", FunctionDescriptor.of(JAVA_INT, ADDRESS, JAVA_INT, ADDRESS, JAVA_INT, JAVA_INT, ADDRESS))
    val gemmExpanded: MethodHandle = h("skn_gemm_expanded", FunctionDescriptor.of(JAVA_INT, ADDRESS, ADDRESS, JAVA_INT, JAVA_INT, ADDRESS, JAVA_INT, ADDRESS))
    val kvCreate: MethodHandle = h("skn_kv_create", FunctionDescriptor.of(JAVA_INT, ADDRESS, JAVA_INT, JAVA_INT, JAVA_INT, JAVA_INT, JAVA_INT, ADDRESS))
    val kvFree: MethodHandle = h("skn_kv_free", FunctionDescriptor.of(JAVA_INT, ADDRESS, ADDRESS))
    val kvReset: MethodHandle = h("skn_kv_reset", FunctionDescriptor.of(JAVA_INT, ADDRESS, ADDRESS, JAVA_INT))
    val kvLen: MethodHandle = h("skn_kv_len", FunctionDescriptor.of(JAVA_INT, ADDRESS, ADDRESS, JAVA_INT))
    val kvAppend: MethodHandle = h("skn_kv_append", FunctionDescriptor.of(JAVA_INT, ADDRESS, ADDRESS, ADDRESS, ADDRESS, ADDRESS, JAVA_INT))
    val kvAppendRun: MethodHandle = h("skn_kv_append_run", FunctionDescriptor.of(JAVA_INT, ADDRESS, ADDRESS, JAVA_INT, ADDRESS, ADDRESS, JAVA_INT))
    val kvGather: MethodHandle = h("skn_kv_gather", FunctionDescriptor.of(JAVA_INT, ADDRESS, ADDRESS, JAVA_INT, JAVA_INT, JAVA_INT, ADDRESS, ADDRESS))
    val attnDecode: MethodHandle = h("skn_attn_decode", FunctionDescriptor.of(JAVA_INT, ADDRESS, ADDRESS, ADDRESS, ADDRESS, JAVA_FLOAT, ADDRESS))
    val attnDecodeStatic: MethodHandle = h("skn_attn_decode_static", FunctionDescriptor.of(JAVA_INT, ADDRESS, ADDRESS, ADDRESS, JAVA_FLOAT, ADDRESS))
    val attnPrefill: MethodHandle = h("skn_attn_prefill", FunctionDescriptor.of(JAVA_INT, ADDRESS, ADDRESS, JAVA_INT, ADDRESS, JAVA_INT, JAVA_FLOAT, ADDRESS))
    val rmsnorm: MethodHandle = h("skn_rmsnorm", FunctionDescriptor.of(JAVA_INT, ADDRESS, ADDRESS, ADDRESS, JAVA_INT, JAVA_INT, JAVA_FLOAT, ADDRESS))
    val rope: MethodHandle = h("skn_rope", FunctionDescriptor.of(JAVA_INT, ADDRESS, ADDRESS, JAVA_INT, JAVA_INT, JAVA_INT, JAVA_INT, JAVA_FLOAT))
    val swiglu: MethodHandle = h("skn_swiglu", FunctionDescriptor.of(JAVA_INT, ADDRESS, ADDRESS, ADDRESS, JAVA_LONG, ADDRESS))
    val relu: MethodHandle = h("skn_relu", FunctionDescriptor.of(JAVA_INT, ADDRESS, ADDRESS, JAVA_LONG, ADDRESS))
    val addInplace: MethodHandle = h("skn_add_inplace", FunctionDescriptor.of(JAVA_INT, ADDRESS, ADDRESS, ADDRESS, JAVA_LONG))
    val argmax: MethodHandle = h("skn_argmax", FunctionDescriptor.of(JAVA_INT, ADDRESS, ADDRESS, JAVA_INT, ADDRESS))
    val f32ToF16: MethodHandle = h("skn_f32_to_f16", FunctionDescriptor.of(JAVA_INT, ADDRESS, ADDRESS, JAVA_LONG, ADDRESS))
    val f32ToBf16: MethodHandle = h("skn_f32_to_bf16", FunctionDescriptor.of(JAVA_INT, ADDRESS, ADDRESS, JAVA_LONG, ADDRESS))
    val llamaCreate: MethodHandle = h("skn_llama_create", FunctionDescriptor.of(JAVA_INT, ADDRESS, ADDRESS, ADDRESS, ADDRESS))
    val llamaFree: MethodHandle = h("skn_llama_free", FunctionDescriptor.of(JAVA_INT, ADDRESS, ADDRESS))
    val llamaReset: MethodHandle = h("skn_llama_reset", FunctionDescriptor.of(JAVA_INT, ADDRESS, ADDRESS))
    val llamaPrefill: MethodHandle = h("skn_llama_prefill", FunctionDescriptor.of(JAVA_INT, ADDRESS, ADDRESS, ADDRESS, JAVA_INT, ADDRESS))
    val llamaDecode: MethodHandle = h("skn_llama_decode", FunctionDescriptor.of(JAVA_INT, ADDRESS, ADDRESS, JAVA_INT, JAVA_INT, ADDRESS))
    val llamaLogits: MethodHandle = h("skn_llama_logits", FunctionDescriptor.of(JAVA_INT, ADDRESS, ADDRESS, ADDRESS))
    val synthWeight: MethodHandle = h("skn_synth_weight", FunctionDescriptor.of(JAVA_INT, JAVA_INT, JAVA_LONG, JAVA_LONG, JAVA_LONG, ADDRESS, JAVA_LONG))
    val synthActivationF32: MethodHandle = h("skn_synth_activation_f32", FunctionDescriptor.of(JAVA_INT, JAVA_LONG, JAVA_LONG, ADDRESS))
    val synthActivationBf16: MethodHandle = h("skn_synth_activation_bf16", FunctionDescriptor.of(JAVA_INT, JAVA_LONG, JAVA_LONG, ADDRESS))
    val synthKvF16: MethodHandle = h("skn_synth_kv_f16", FunctionDescriptor.of(JAVA_INT, JAVA_LONG, JAVA_LONG, ADDRESS))
    val synthChecksum: MethodHandle = h("skn_synth_checksum", FunctionDescriptor.of(JAVA_LONG, ADDRESS, JAVA_LONG))
    val testFusedMatvec: MethodHandle = h("skn_test_fused_matvec", FunctionDescriptor.of(JAVA_INT, ADDRESS, JAVA_INT, JAVA_INT, ADDRESS, JAVA_INT, ADDRESS, JAVA_INT, ADDRESS, JAVA_INT, JAVA_INT, ADDRESS, ADDRESS, JAVA_FLOAT, ADDRESS, ADDRESS, ADDRESS, JAVA_FLOAT))
    val testMatvecQ4kStamps: MethodHandle = h("skn_test_matvec_q4k_stamps", FunctionDescriptor.of(JAVA_INT, ADDRESS, ADDRESS, JAVA_INT, JAVA_INT, ADDRESS, ADDRESS, ADDRESS))

    init {
        val v = abiVersion.invokeExact() as Int
        check(v == ABI_VERSION) { "libskainet_hip has ABI version $v, this binding was written for $ABI_VERSION" }
    }
}
