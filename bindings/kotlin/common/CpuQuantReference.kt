// The quantized path restated for the reference's own CPU backend, in common Kotlin (no native code): block
// dequantization for Q8_0 / Q4_K / Q6_K -- what gguf/src/commonMain/kotlin/sk/ai/net/gguf/Quants.kt:8 leaves as a TODO --
// and Linear's y = x . W^T over such a weight without materialising t() (nn/Linear.kt:48 calls
// impl/DoublesTensor.kt:362-387 on every forward).  Block layouts are ggml's; sizes are the reference's table
// (gguf/Constants.kt:58-90).  Values are formed in Float exactly as ggml forms them (each is the exact real rounded
// once), sums are accumulated in Double like the reference's matmul (impl/DoublesTensor.kt:255-264).
// This is the CPU figure to time beside the device path on a box that has a JVM; it is source only here.
package sk.ai.net.hip

import sk.ai.net.Shape
import sk.ai.net.gguf.GGMLQuantizationType
import sk.ai.net.impl.DoublesTensor

object CpuQuantReference {

    /** IEEE binary16 bits -> Float, subnormals honoured. */
    fun halfToFloat(h: Int): Float {
        val sign = if (h and 0x8000 != 0) -1f else 1f
        val exp = (h shr 10) and 0x1F
        val man = h and 0x3FF
        return when (exp) {
            0 -> sign * man * (1f / 16777216f)                       // man * 2^-24
            31 -> if (man == 0) sign * Float.POSITIVE_INFINITY else Float.NaN
            else -> sign * Float.fromBits(((exp + 112) shl 23) or (man shl 13))
        }
    }

    private fun u8(b: ByteArray, i: Int) = b[i].toInt() and 0xFF
    private fun f16(b: ByteArray, i: Int) = halfToFloat(u8(b, i) or (u8(b, i + 1) shl 8))

    /** One Q8_0 block (34 bytes: f16 d, 32 x int8) at `off` -> out[o .. o+31]. */
    fun dequantQ8_0(b: ByteArray, off: Int, out: FloatArray, o: Int) {
        val d = f16(b, off)
        for (i in 0 until 32) out[o + i] = d * b[off + 2 + i].toInt()
    }

    /** One Q4_K superblock (144 bytes: f16 d, f16 dmin, 12 bytes of 6-bit scales / mins, 128 bytes of nibbles). */
    fun dequantQ4_K(b: ByteArray, off: Int, out: FloatArray, o: Int) {
        val d = f16(b, off)
        val dmin = f16(b, off + 2)
        val s = off + 4
        val q = off + 16
        for (j in 0 until 8) {
            val sc: Int
            val m: Int
            if (j < 4) {
                sc = u8(b, s + j) and 63
                m = u8(b, s + j + 4) and 63
            } else {
                sc = (u8(b, s + j + 4) and 0x0F) or ((u8(b, s + j - 4) shr 6) shl 4)
                m = (u8(b, s + j + 4) shr 4) or ((u8(b, s + j) shr 6) shl 4)
            }
            val ds = d * sc
            val dm = dmin * m
            val chunk = j / 2          // 32 bytes of nibbles per pair of sub-blocks: low nibbles first, then high
            for (l in 0 until 32) {
                val byte = u8(b, q + 32 * chunk + l)
                val nib = if (j % 2 == 0) byte and 0x0F else byte shr 4
                out[o + 32 * j + l] = ds * nib - dm
            }
        }
    }

    /** One Q6_K superblock (210 bytes: ql[128], qh[64], int8 scales[16], f16 d). */
    fun dequantQ6_K(b: ByteArray, off: Int, out: FloatArray, o: Int) {
        val d = f16(b, off + 208)
        for (n in 0 until 2) {
            val ql = off + 64 * n
            val qh = off + 128 + 32 * n
            val sc = off + 192 + 8 * n
            for (l in 0 until 32) {
                val isub = l / 16
                val h = u8(b, qh + l)
                val q1 = ((u8(b, ql + l) and 0x0F) or ((h and 3) shl 4)) - 32
                val q2 = ((u8(b, ql + l + 32) and 0x0F) or (((h shr 2) and 3) shl 4)) - 32
                val q3 = ((u8(b, ql + l) shr 4) or (((h shr 4) and 3) shl 4)) - 32
                val q4 = ((u8(b, ql + l + 32) shr 4) or (((h shr 6) and 3) shl 4)) - 32
                val base = o + 128 * n + l
                out[base] = d * b[sc + isub].toInt() * q1
                out[base + 32] = d * b[sc + isub + 2].toInt() * q2
                out[base + 64] = d * b[sc + isub + 4].toInt() * q3
                out[base + 96] = d * b[sc + isub + 6].toInt() * q4
            }
        }
    }

    /** Block elements and bytes of the three formats (gguf/Constants.kt:65,69,71). */
    private fun sizes(type: GGMLQuantizationType): Pair<Int, Int> = when (type) {
        GGMLQuantizationType.Q8_0 -> 32 to 34
        GGMLQuantizationType.Q4_K -> 256 to 144
        GGMLQuantizationType.Q6_K -> 256 to 210
        else -> throw IllegalArgumentException("Invalid quantization type")
    }

    /** A row of k elements starting at byte `off` -> out[0 .. k-1]. */
    fun dequantRow(type: GGMLQuantizationType, bytes: ByteArray, off: Int, k: Int, out: FloatArray) {
        val (be, bb) = sizes(type)
        require(k % be == 0) { "Quantized tensor row size ($k) is not a multiple of ${type.name} block size ($be)" }
        for (blk in 0 until k / be) when (type) {
            GGMLQuantizationType.Q8_0 -> dequantQ8_0(bytes, off + blk * bb, out, blk * be)
            GGMLQuantizationType.Q4_K -> dequantQ4_K(bytes, off + blk * bb, out, blk * be)
            else -> dequantQ6_K(bytes, off + blk * bb, out, blk * be)
        }
    }

    /** y[n] = sum_k deq(W)[n, k] * x[k]: Linear.forward for a rank-1 input over an [out = n, in = k] weight. */
    fun matvec(type: GGMLQuantizationType, bytes: ByteArray, n: Int, k: Int, x: DoubleArray): DoublesTensor {
        if (x.size != k) throw IllegalArgumentException("Shapes do not align.")
        val (be, bb) = sizes(type)
        val rowBytes = k / be * bb
        val row = FloatArray(k)
        val y = DoubleArray(n)
        for (r in 0 until n) {
            dequantRow(type, bytes, r * rowBytes, k, row)
            var acc = 0.0
            for (i in 0 until k) acc += row[i].toDouble() * x[i]
            y[r] = acc
        }
        return DoublesTensor(Shape(n), y)
    }

    /** C[m, n] = sum_k A[m, k] * deq(W)[n, k] (impl/DoublesTensor.kt:267-279 semantics, rows of A against rows of W). */
    fun matmul(type: GGMLQuantizationType, bytes: ByteArray, n: Int, k: Int, a: DoublesTensor): DoublesTensor {
        require(a.shape.rank == 2) { "Unsupported tensor shapes for multiplication" }
        val m = a.shape.dimensions[0]
        if (a.shape.dimensions[1] != k) throw IllegalArgumentException("Shapes do not align.")
        val (be, bb) = sizes(type)
        val rowBytes = k / be * bb
        val row = FloatArray(k)
        val c = DoubleArray(m * n)
        for (r in 0 until n) {
            dequantRow(type, bytes, r * rowBytes, k, row)
            for (i in 0 until m) {
                var acc = 0.0
                for (j in 0 until k) acc += a.elements[i * k + j] * row[j]
                c[i * n + r] = acc
            }
        }
        return DoublesTensor(Shape(m, n), c)
    }
}
