// GGUF block bytes on the device behind the reference's Tensor interface
// (core/src/commonMain/kotlin/sk/ai/net/Tensor.kt:6-92).  The logical shape is Linear's [out, in]
// (nn/Linear.kt:26-28); t() is a view flag -- the reference's t() materialises a transpose on every forward
// (impl/DoublesTensor.kt:362-387).  A weight is read-only and only ever the right-hand operand of a matmul, so the
// arithmetic of the interface is answered on the dequantized values (an explicit, visible copy to the host type).
package sk.ai.net.hip

import sk.ai.net.DataDescriptor
import sk.ai.net.Shape
import sk.ai.net.Tensor
import sk.ai.net.gguf.GGMLQuantizationType
import sk.ai.net.impl.DoublesTensor
import java.lang.foreign.MemorySegment

class QuantizedTensor internal constructor(
    val ctx: SknContext,
    val ggmlType: GGMLQuantizationType,
    private val storedShape: Shape,           // [out, in], as stored
    internal val dev: MemorySegment,
    val transposed: Boolean = false,
    private val owner: Boolean = true,
) : Tensor, AutoCloseable {

    companion object {
        /** From a ReaderTensor's raw bytes and reversed dims (GGUFReader.kt:354-373): [out, in] rows of blocks. */
        fun fromBytes(ctx: SknContext, type: GGMLQuantizationType, out: Int, `in`: Int, bytes: ByteArray): QuantizedTensor {
            val d = QuantDescriptor(type)
            require(bytes.size.toLong() == out * d.rowBytes(`in`)) { "byte count does not match the shape" }
            return QuantizedTensor(ctx, type, Shape(out, `in`), ctx.uploadBytes(bytes))
        }
    }

    private val descriptor = QuantDescriptor(ggmlType)

    init {
        require(storedShape.rank == 2) { "quantized weights are rank-2 [out, in] tensors" }
        descriptor.rowBytes(storedShape.dimensions[1])  // the reference's block-multiple check
    }

    val outFeatures: Int get() = storedShape.dimensions[0]
    val inFeatures: Int get() = storedShape.dimensions[1]

    override val shape: Shape
        get() = if (transposed) Shape(inFeatures, outFeatures) else storedShape
    override val dataDescriptor: DataDescriptor get() = descriptor

    /** The fp16-pair copy that rank-2 products multiply with (skn_gemm_expand); shared by the views t() makes. */
    internal var expanded: MemorySegment? = null

    override fun t(): Tensor =
        QuantizedTensor(ctx, ggmlType, storedShape, dev, !transposed, owner = false).also { it.expanded = expanded }

    /**
     * Keeps the expanded copy of the weights on the device (4 bytes per weight) so that rank-2 products skip the
     * per-call weight pass of the formats other than Q4_K, which has none and is left as it is.
     */
    fun expandForGemm(): QuantizedTensor {
        if (expanded == null && ggmlType != GGMLQuantizationType.Q4_K) {
            val copy = ctx.malloc(ctx.gemmExpandedBytes(ggmlType.value, outFeatures, inFeatures))
            ctx.check(SknLib.gemmExpand.invokeExact(ctx.handle, ggmlType.value, dev, outFeatures, inFeatures, copy) as Int)
            expanded = copy
        }
        return this
    }

    /** skn_dequant: the dequantizer the reference leaves as a TODO (gguf/.../Quants.kt:8), bit-exact ggml values. */
    fun dequantize(): DeviceTensor {
        val outT = ctx.newTensor(storedShape)
        ctx.check(SknLib.dequant.invokeExact(ctx.handle, ggmlType.value, dev, storedShape.volume.toLong(), outT.dev) as Int)
        return outT
    }

    /** The values as the reference's own tensor type, in the logical (possibly transposed) orientation. */
    fun toDoubles(): DoublesTensor {
        val host = dequantize().use { it.toDoubles() }
        return if (transposed) host.t() as DoublesTensor else host
    }

    // A quantized weight is the right-hand operand: x.matmul(W.t()) is DeviceTensor.matmul.  As a receiver it has
    // the reference's semantics on its values.
    override fun matmul(other: Tensor): Tensor = toDoubles().matmul(hostOf(other))

    override fun plus(other: Tensor): Tensor = toDoubles() + hostOf(other)
    override fun plus(other: Double): Tensor = toDoubles() + other
    override fun plus(other: Int): Tensor = toDoubles() + other
    override fun minus(other: Double): Tensor = toDoubles() - other
    override fun minus(other: Int): Tensor = toDoubles() - other
    override fun minus(other: Tensor): Tensor = toDoubles() - hostOf(other)
    override fun relu(): Tensor = toDoubles().relu()
    override fun softmax(dim: Int): Tensor = toDoubles().softmax(dim)
    override fun softmax(): Tensor = toDoubles().softmax()
    override fun pow(tensor: Tensor): Tensor = toDoubles().pow(hostOf(tensor))
    override fun pow(scalar: Double): Tensor = toDoubles().pow(scalar)
    override fun sin(): Tensor = toDoubles().sin()
    override fun cos(): Tensor = toDoubles().cos()
    override fun tan(): Tensor = toDoubles().tan()
    override fun asin(): Tensor = toDoubles().asin()
    override fun acos(): Tensor = toDoubles().acos()
    override fun atan(): Tensor = toDoubles().atan()
    override fun sinh(): Tensor = toDoubles().sinh()
    override fun cosh(): Tensor = toDoubles().cosh()
    override fun tanh(): Tensor = toDoubles().tanh()
    override fun exp(): Tensor = toDoubles().exp()
    override fun log(): Tensor = toDoubles().log()
    override fun sqrt(): Tensor = toDoubles().sqrt()
    override fun cbrt(): Tensor = toDoubles().cbrt()
    override fun sigmoid(): Tensor = toDoubles().sigmoid()
    override fun ln(): Tensor = toDoubles().ln()
    override fun flatten(startDim: Int, endDim: Int): Tensor = toDoubles().flatten(startDim, endDim)

    override fun close() {
        if (owner) {
            expanded?.let { ctx.free(it) }
            ctx.free(dev)
        }
    }
}

/** The host view of any tensor, for the operations that are not on the device path. */
internal fun hostOf(t: Tensor): Tensor = when (t) {
    is DeviceTensor -> t.toDoubles()
    is QuantizedTensor -> t.toDoubles()
    else -> t
}
