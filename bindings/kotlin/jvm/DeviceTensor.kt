// fp32 activations on the device behind the reference's Tensor interface (core/.../Tensor.kt:6-92).
// DoublesTensor.matmul hard-casts its argument (impl/DoublesTensor.kt:235,242,250,260,274), so the device tensor must
// be the receiver: Linear.forward calls input.matmul(weight.t()) + bias (nn/Linear.kt:48), which lands in matmul() and
// plus() below.  matmul with a transposed QuantizedTensor, plus with a device tensor and relu run on the device; every
// other operation of the interface is answered by the reference's own DoublesTensor on downloaded values (these are
// not on the inference path).
package sk.ai.net.hip

import sk.ai.net.DataDescriptor
import sk.ai.net.Shape
import sk.ai.net.Tensor
import sk.ai.net.impl.DoublesTensor
import java.lang.foreign.MemorySegment

class DeviceTensor internal constructor(
    val ctx: SknContext,
    override val shape: Shape,
    internal val dev: MemorySegment,
    private val owner: Boolean = true,   // false: a view of another tensor's buffer (a reshape)
) : Tensor, AutoCloseable {

    companion object {
        fun of(ctx: SknContext, shape: Shape, values: DoubleArray): DeviceTensor {
            require(values.size == shape.volume) { "element count does not match the shape" }
            return DeviceTensor(ctx, shape, ctx.uploadFloats(FloatArray(values.size) { values[it].toFloat() }))
        }

        fun of(ctx: SknContext, host: DoublesTensor): DeviceTensor = of(ctx, host.shape, host.elements)
    }

    override val dataDescriptor: DataDescriptor get() = Float32Descriptor

    fun toFloats(): FloatArray = ctx.downloadFloats(dev, shape.volume)

    fun toDoubles(): DoublesTensor {
        val f = toFloats()
        return DoublesTensor(shape, DoubleArray(f.size) { f[it].toDouble() })
    }

    /**
     * x.matmul(W.t()) with W a quantized [out, in] weight: rank 1 -> skn_matvec_q (DoublesTensor.kt:255-264 semantics),
     * rank 2 -> skn_gemm_q on bf16 rows (DoublesTensor.kt:267-279 semantics); ranks 3 and 4 multiply every [.., in] row
     * (DoublesTensor.kt:281-357), i.e. the same GEMM with the leading dimensions as its rows.  Anything else: the
     * reference's matmul on host values, including its error messages.
     */
    override fun matmul(other: Tensor): Tensor {
        if (other is QuantizedTensor && other.transposed && (rank == 3 || rank == 4)) {
            val k = shape.dimensions.last()
            if (k != other.inFeatures) throw IllegalArgumentException("Shapes do not align.")
            val rows = DeviceTensor(ctx, Shape(shape.volume / k, k), dev, owner = false)
            val out = rows.matmul(other) as DeviceTensor
            val lead = shape.dimensions.dropLast(1).toIntArray()
            return out.reshaped(Shape(*lead, other.outFeatures))  // (out itself is not closed: the result owns its buffer)
        }
        if (other !is QuantizedTensor || !other.transposed || (rank != 1 && rank != 2)) {
            if (other is QuantizedTensor && (rank == 1 || rank == 2))
                throw IllegalArgumentException(
                    "Unsupported tensor shapes for multiplication: ${shape.dimensions.toList()} and ${other.shape.dimensions.toList()}"
                )  // DoublesTensor.kt:359: an untransposed [out, in] weight is no Linear
            return toDoubles().matmul(hostOf(other))
        }
        val n = other.outFeatures
        val k = other.inFeatures
        if (shape.dimensions.last() != k) throw IllegalArgumentException("Shapes do not align.")  // DoublesTensor.kt:256,268
        if (rank == 1) {
            val y = ctx.newTensor(Shape(n))
            ctx.check(SknLib.matvecQ.invokeExact(ctx.handle, other.ggmlType.value, other.dev, n, k, dev, y.dev) as Int)
            return y
        }
        val m = shape.dimensions[0]
        val a16 = ctx.malloc(2L * m * k)
        try {
            ctx.check(SknLib.f32ToBf16.invokeExact(ctx.handle, dev, m.toLong() * k, a16) as Int)
            val c = ctx.newTensor(Shape(m, n))
            val kept = other.expanded
            if (kept != null)
                ctx.check(SknLib.gemmExpanded.invokeExact(ctx.handle, kept, n, k, a16, m, c.dev) as Int)
            else
                ctx.check(SknLib.gemmQ.invokeExact(ctx.handle, other.ggmlType.value, other.dev, n, k, a16, m, c.dev) as Int)
            return c
        } finally {
            ctx.sync()      // the GEMM reads a16 asynchronously
            ctx.free(a16)
        }
    }

    /** Elementwise sum; a lower-rank right operand whose shape is this tensor's trailing shape is added to every row
     *  (the bias of Linear.forward, nn/Linear.kt:48). */
    override fun plus(other: Tensor): Tensor {
        if (other !is DeviceTensor) return toDoubles() + hostOf(other)
        val rows = if (other.shape.volume == 0) 0 else shape.volume / other.shape.volume
        val trailing = shape.dimensions.takeLast(other.rank)
        if (trailing != other.shape.dimensions.toList() || rows * other.shape.volume != shape.volume)
            throw IllegalArgumentException("Shapes do not align.")
        val out = ctx.newTensor(shape)
        ctx.check(SknLib.copy.invokeExact(ctx.handle, out.dev, dev, 4L * shape.volume) as Int)
        for (r in 0 until rows) {
            val row = out.dev.asSlice(4L * r * other.shape.volume)
            ctx.check(SknLib.addInplace.invokeExact(ctx.handle, row, other.dev, other.shape.volume.toLong()) as Int)
        }
        return out
    }

    /** max(x, 0) on the device (skn_relu; impl/DoublesTensor.kt:389-390). */
    override fun relu(): Tensor {
        val out = ctx.newTensor(shape)
        ctx.check(SknLib.relu.invokeExact(ctx.handle, dev, shape.volume.toLong(), out.dev) as Int)
        return out
    }

    // ---- the rest of the interface: the reference's own arithmetic on downloaded values ------------------------
    override fun plus(other: Double): Tensor = toDoubles() + other
    override fun plus(other: Int): Tensor = toDoubles() + other
    override fun minus(other: Double): Tensor = toDoubles() - other
    override fun minus(other: Int): Tensor = toDoubles() - other
    override fun minus(other: Tensor): Tensor = toDoubles() - hostOf(other)
    override fun t(): Tensor = toDoubles().t()
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

    /** The same buffer under another shape of the same volume; the receiver gives up ownership to the result. */
    internal fun reshaped(to: Shape): DeviceTensor {
        require(to.volume == shape.volume) { "a reshape keeps the element count" }
        return DeviceTensor(ctx, to, dev, owner)
    }

    override fun close() {
        if (owner) ctx.free(dev)
    }
}
