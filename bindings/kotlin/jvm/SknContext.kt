// The context a device tensor lives in: one HIP stream, opaque handle, AutoCloseable (reference tensors are
// garbage-collected host objects, so an explicit lifetime is new).  JVM flavour over SknLib; the Kotlin/Native flavour
// is the same class over the cinterop stubs (sk.ai.net.hip.cinterop.*), see SknContext.native.kt.
package sk.ai.net.hip

import sk.ai.net.Shape
import java.lang.foreign.Arena
import java.lang.foreign.MemorySegment
import java.lang.foreign.ValueLayout.ADDRESS
import java.lang.foreign.ValueLayout.JAVA_BYTE
import java.lang.foreign.ValueLayout.JAVA_FLOAT
import java.lang.foreign.ValueLayout.JAVA_LONG

class SknException(val code: Int, message: String) : IllegalStateException(message)

class SknContext(device: Int = 0) : AutoCloseable {
    internal val handle: MemorySegment

    init {
        Arena.ofConfined().use { arena ->
            val out = arena.allocate(ADDRESS)
            val rc = SknLib.init.invokeExact(device, out) as Int
            if (rc != SknLib.OK) throw SknException(rc, lastError(MemorySegment.NULL))
            handle = out.get(ADDRESS, 0)
        }
    }

    private fun lastError(ctx: MemorySegment): String {
        val p = SknLib.lastError.invokeExact(ctx) as MemorySegment
        return if (p == MemorySegment.NULL) "libskainet_hip error" else p.reinterpret(4096).getString(0)
    }

    /** Maps a status code to the exception the reference throws for the same mistake. */
    internal fun check(rc: Int) {
        if (rc == SknLib.OK) return
        val msg = lastError(handle)
        when (rc) {
            // DoublesTensor.kt:256,268 ("Shapes do not align.") and Quants.kt:13-15 (block-multiple message): the
            // library words its SKN_ERR_SHAPE messages the same way
            SknLib.ERR_SHAPE, SknLib.ERR_ARG, SknLib.ERR_RANGE -> throw IllegalArgumentException(msg)
            SknLib.ERR_TYPE -> throw IllegalArgumentException("Invalid quantization type: $msg")  // GGUFReader.kt:358
            SknLib.ERR_OOM -> throw OutOfMemoryError(msg)
            else -> throw SknException(rc, msg)
        }
    }

    fun malloc(bytes: Long): MemorySegment = Arena.ofConfined().use { arena ->
        val out = arena.allocate(ADDRESS)
        check(SknLib.malloc.invokeExact(handle, maxOf(bytes, 16L), out) as Int)
        out.get(ADDRESS, 0)
    }

    fun free(dev: MemorySegment) = check(SknLib.free.invokeExact(handle, dev) as Int)

    fun upload(dev: MemorySegment, host: MemorySegment, bytes: Long) =
        check(SknLib.upload.invokeExact(handle, dev, host, bytes) as Int)

    fun download(host: MemorySegment, dev: MemorySegment, bytes: Long) =
        check(SknLib.download.invokeExact(handle, host, dev, bytes) as Int)

    fun sync() = check(SknLib.sync.invokeExact(handle) as Int)

    /** fp32 values -> a new device buffer. */
    fun uploadFloats(values: FloatArray): MemorySegment = Arena.ofConfined().use { arena ->
        val host = arena.allocateFrom(JAVA_FLOAT, *values)
        val dev = malloc(4L * values.size)
        upload(dev, host, 4L * values.size)
        dev
    }

    /** Raw GGUF block bytes (ReaderTensor.data, GGUFReader.kt:35-44) -> a new device buffer. */
    fun uploadBytes(bytes: ByteArray): MemorySegment = Arena.ofConfined().use { arena ->
        val host = arena.allocateFrom(JAVA_BYTE, *bytes)
        val dev = malloc(bytes.size.toLong())
        upload(dev, host, bytes.size.toLong())
        dev
    }

    fun downloadFloats(dev: MemorySegment, count: Int): FloatArray = Arena.ofConfined().use { arena ->
        val host = arena.allocate(JAVA_FLOAT, count.toLong())
        download(host, dev, 4L * count)
        host.toArray(JAVA_FLOAT)
    }

    /** Size of the expanded copy of an [n, k] weight matrix (skn_gemm_expanded_bytes; size_t is 64 bits here). */
    fun gemmExpandedBytes(type: Int, n: Int, k: Int): Long = Arena.ofConfined().use { arena ->
        val out = arena.allocate(JAVA_LONG)
        check(SknLib.gemmExpandedBytes.invokeExact(handle, type, n, k, out) as Int)
        out.get(JAVA_LONG, 0)
    }

    fun newTensor(shape: Shape): DeviceTensor = DeviceTensor(this, shape, malloc(4L * shape.volume))

    override fun close() {
        SknLib.shutdown.invokeExact(handle)
    }
}
