// Kotlin/Native flavour of the context over the cinterop stubs generated from skainet_hip.def: the same calls as the
// JVM flavour, with CPointer handles.  DeviceTensor / QuantizedTensor for linuxX64 are the JVM sources with
// `MemorySegment` read as `COpaquePointer` and `SknLib.x.invokeExact(...)` read as `skn_x(...)`.
package sk.ai.net.hip

import kotlinx.cinterop.ByteVar
import kotlinx.cinterop.COpaquePointer
import kotlinx.cinterop.COpaquePointerVar
import kotlinx.cinterop.CPointer
import kotlinx.cinterop.CPointerVar
import kotlinx.cinterop.ExperimentalForeignApi
import kotlinx.cinterop.FloatVar
import kotlinx.cinterop.addressOf
import kotlinx.cinterop.alloc
import kotlinx.cinterop.memScoped
import kotlinx.cinterop.ptr
import kotlinx.cinterop.toKString
import kotlinx.cinterop.usePinned
import kotlinx.cinterop.value
import sk.ai.net.hip.cinterop.*

@OptIn(ExperimentalForeignApi::class)
class SknNativeContext(device: Int = 0) : AutoCloseable {
    val handle: CPointer<skn_ctx>

    init {
        handle = memScoped {
            val out = alloc<CPointerVar<skn_ctx>>()
            val rc = skn_init(device, out.ptr)
            if (rc != SKN_OK) throw IllegalStateException(skn_last_error(null)?.toKString() ?: "skn_init failed ($rc)")
            out.value!!
        }
    }

    fun check(rc: Int) {
        if (rc == SKN_OK) return
        val msg = skn_last_error(handle)?.toKString() ?: "libskainet_hip error $rc"
        when (rc) {
            SKN_ERR_SHAPE, SKN_ERR_ARG, SKN_ERR_RANGE -> throw IllegalArgumentException(msg)
            SKN_ERR_TYPE -> throw IllegalArgumentException("Invalid quantization type: $msg")
            else -> throw IllegalStateException(msg)
        }
    }

    fun malloc(bytes: Long): COpaquePointer = memScoped {
        val out = alloc<COpaquePointerVar>()
        check(skn_malloc(handle, maxOf(bytes, 16L).toULong(), out.ptr))
        out.value!!
    }

    fun free(dev: COpaquePointer) = check(skn_free(handle, dev))

    fun uploadBytes(bytes: ByteArray): COpaquePointer {
        val dev = malloc(bytes.size.toLong())
        bytes.usePinned { check(skn_upload(handle, dev, it.addressOf(0), bytes.size.toULong())) }
        return dev
    }

    fun uploadFloats(values: FloatArray): COpaquePointer {
        val dev = malloc(4L * values.size)
        values.usePinned { check(skn_upload(handle, dev, it.addressOf(0), (4L * values.size).toULong())) }
        return dev
    }

    fun downloadFloats(dev: COpaquePointer, count: Int): FloatArray {
        val out = FloatArray(count)
        out.usePinned { check(skn_download(handle, it.addressOf(0), dev, (4L * count).toULong())) }
        return out
    }

    /** y = deq(W) . x for an [n, k] weight of `ggmlType` (gguf/Constants.kt:14-46 ids). */
    fun matvec(ggmlType: Int, w: COpaquePointer, n: Int, k: Int, x: COpaquePointer, y: COpaquePointer) =
        check(skn_matvec_q(handle, ggmlType, w, n, k, x.reinterpretFloat(), y.reinterpretFloat()))

    private fun COpaquePointer.reinterpretFloat(): CPointer<FloatVar> = this as CPointer<FloatVar>

    override fun close() = skn_shutdown(handle)
}
