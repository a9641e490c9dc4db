// DataDescriptor of a GGUF block format (core/src/commonMain/kotlin/sk/ai/net/DataDescriptor.kt:6-24).  `bits` is an
// Int in the reference, which cannot say 4.5 / 6.5625 / 8.5 bits per weight: it carries the quant's own width and
// `bitsPerWeight` the storage cost including scales (block bytes * 8 / block elements, Constants.kt:58-90).
package sk.ai.net.hip

import sk.ai.net.DataDescriptor
import sk.ai.net.gguf.GGMLQuantizationType
import sk.ai.net.gguf.GGML_QUANT_SIZES

class QuantDescriptor(val type: GGMLQuantizationType) : DataDescriptor {
    private val sizes = GGML_QUANT_SIZES[type] ?: throw IllegalArgumentException("Invalid quantization type")
    val blockElements: Int get() = sizes.first
    val blockBytes: Int get() = sizes.second
    val bitsPerWeight: Double get() = blockBytes * 8.0 / blockElements
    override val name: String get() = type.name
    override val bits: Int
        get() = when (type) {
            GGMLQuantizationType.Q8_0, GGMLQuantizationType.Q8_K -> 8
            GGMLQuantizationType.Q6_K -> 6
            GGMLQuantizationType.Q5_0, GGMLQuantizationType.Q5_1, GGMLQuantizationType.Q5_K -> 5
            GGMLQuantizationType.Q4_0, GGMLQuantizationType.Q4_1, GGMLQuantizationType.Q4_K,
            GGMLQuantizationType.IQ4_NL, GGMLQuantizationType.IQ4_XS -> 4
            GGMLQuantizationType.Q3_K -> 3
            GGMLQuantizationType.Q2_K, GGMLQuantizationType.TQ1_0, GGMLQuantizationType.TQ2_0 -> 2
            GGMLQuantizationType.F16, GGMLQuantizationType.BF16 -> 16
            else -> 32
        }
    override fun isSigned(): Boolean = true
    override val minValue: Double get() = Double.NEGATIVE_INFINITY  // the scale of a block is a free fp16 factor
    override val maxValue: Double get() = Double.POSITIVE_INFINITY
    override val isFloatingPoint: Boolean get() = false

    /** quantShapeToByteShape on the last axis (gguf/.../Quants.kt:10-20). */
    fun rowBytes(k: Int): Long {
        require(k % blockElements == 0) {
            "Quantized tensor row size ($k) is not a multiple of ${type.name} block size ($blockElements)"
        }
        return k.toLong() / blockElements * blockBytes
    }
}

/** Device arithmetic is fp32. */
object Float32Descriptor : DataDescriptor {
    override val name = "Float32"
    override val bits = 32
    override fun isSigned() = true
    override val minValue = -Float.MAX_VALUE.toDouble()
    override val maxValue = Float.MAX_VALUE.toDouble()
    override val isFloatingPoint = true
}
