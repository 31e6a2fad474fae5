package sk.ainet.exec.hip

import java.lang.foreign.Arena
import java.lang.foreign.MemorySegment
import java.lang.foreign.ValueLayout
import java.util.IdentityHashMap
import sk.ainet.backend.api.kernel.KernelDispatch
import sk.ainet.backend.api.kernel.KernelKey
import sk.ainet.backend.api.kernel.LayoutClass
import sk.ainet.backend.api.kernel.MappedCapableKernel
import sk.ainet.backend.api.kernel.OperandKey
import sk.ainet.backend.api.kernel.ReferenceMatmulKernel
import sk.ainet.backend.api.kernel.ViewKernel
import sk.ainet.backend.api.kernel.ViewKernelPack
import sk.ainet.lang.memory.BlockOrder
import sk.ainet.lang.memory.DirectBufferStorage
import sk.ainet.lang.memory.Format
import sk.ainet.lang.memory.MappedBufferStorage
import sk.ainet.lang.memory.Storage
import sk.ainet.lang.memory.TensorView
import sk.ainet.lang.memory.trace.NoopTraceSink
import sk.ainet.lang.memory.trace.TraceEvent
import sk.ainet.lang.memory.trace.TraceSink
import sk.ainet.lang.tensor.storage.TensorEncoding
import sk.ainet.lang.types.FP32

/**
 * matmul(F32 dense contiguous x F32/<encoding> BLOCKED_ROW_MAJOR) on the device: all activation rows in one call
 * against a GGUF-ordered weight that is uploaded the first time its storage is seen and stays resident after that.
 * The device twin of the CPU library's view kernel, registered under the same kernel key and serving the same operand
 * classes (skainet-backends/skainet-backend-native-cpu/src/jvmMain/kotlin/sk/ainet/exec/kernel/FfmRowMajorKernels.kt:42-137,
 * its pack :140-169).
 *
 * A resident activation ([HipDeviceStorage]) with a resident output runs `skainet_hip_matmul_dev` in place. A heap
 * activation, per call: one copy of the rows into a native segment, `skainet_hip_matmul_host` (upload, product, download and one
 * wait on buffers the library keeps per thread), one copy back. Up to 8 rows run the weight-streaming GEMV kernels
 * (fp32 class, within 1e-3 of the exact product), more rows the matrix-core GEMM (bf16 operands, within 2e-2).
 */
public class HipRowMajorMatmulKernel internal constructor(
    private val encoding: TensorEncoding,
    private val encodingId: Int,
    private val blockElems: Int,
    private val blockBytes: Int,
    override val key: KernelKey,
) : ViewKernel, MappedCapableKernel {
    override val name: String = "hip-rowmajor-${encoding.name}"

    internal fun encodingOf(): TensorEncoding = encoding

    /** Weight handles by the identity of the storage that holds the packed bytes (a model's weights never move). */
    private val resident = IdentityHashMap<Storage, MemorySegment>()

    override fun run(inputs: List<TensorView>, out: TensorView): Unit = run(inputs, out, NoopTraceSink)

    override fun run(inputs: List<TensorView>, out: TensorView, sink: TraceSink) {
        require(inputs.size == 2) { "matmul takes two operands" }
        val a = inputs[0]
        val w = inputs[1]
        val rows = a.shape[0]
        val k = a.shape[1]
        val n = w.shape[0]
        require(w.shape[1] == k) { "inner dimensions disagree: [$rows, $k] x [$n, ${w.shape[1]}]" }
        require(out.shape[0] == rows && out.shape[1] == n) { "out must be [$rows, $n], was ${out.shape}" }
        check(w.layout.blockOrder == BlockOrder.ROW_MAJOR) { "$name reads canonical row-major weights; this one is ${w.layout.blockOrder}" }
        val fn = HipLibrary.matmulHost ?: return fallback(inputs, out, sink, "libskainet_hip unavailable")
        val aDev = a.storage as? HipDeviceStorage
        val oDev = out.storage as? HipDeviceStorage
        if (aDev != null && oDev != null) {
            // a resident activation into a resident output: the product runs where both already are, nothing is copied
            if (!a.isContiguous || !out.isContiguous) return fallback(inputs, out, sink, "strided activation or output")
            if (k % blockElems != 0) return fallback(inputs, out, sink, "inner dimension $k is not a multiple of $blockElems")
            if (rows == 0 || n == 0) return
            val dev = HipLibrary.matmulDev ?: return fallback(inputs, out, sink, "libskainet_hip unavailable")
            val handle = handleFor(w) ?: return fallback(inputs, out, sink, "upload failed: ${HipLibrary.error()}")
            val aPtr = MemorySegment.ofAddress(aDev.pointer().address() + a.layout.offsetElements * Float.SIZE_BYTES)
            val oPtr = MemorySegment.ofAddress(oDev.pointer().address() + out.layout.offsetElements * Float.SIZE_BYTES)
            val rc = dev.invoke(handle, aPtr, rows, oPtr) as Int
            check(rc == 0) { "$name: ${HipLibrary.error()}" }
            if (sink.isEnabled) sink.emit(TraceEvent.KernelRun(op = key.op, kernel = "$name (resident)", inputs = inputs.map { it.id }, output = out.id))
            return
        }
        val aHeap = a.storage as? Storage.Heap ?: return fallback(inputs, out, sink, "activation storage ${a.storage::class.simpleName}")
        val oHeap = out.storage as? Storage.Heap ?: return fallback(inputs, out, sink, "output storage ${out.storage::class.simpleName}")
        val activation = aHeap.floats ?: return fallback(inputs, out, sink, "activation is not a FloatArray")
        val output = oHeap.floats ?: return fallback(inputs, out, sink, "output is not a FloatArray")
        if (!a.isContiguous || !out.isContiguous) return fallback(inputs, out, sink, "strided activation or output")
        if (k % blockElems != 0) return fallback(inputs, out, sink, "inner dimension $k is not a multiple of $blockElems")
        if (rows == 0 || n == 0) return
        val handle = handleFor(w) ?: return fallback(inputs, out, sink, "upload failed: ${HipLibrary.error()}")
        Arena.ofConfined().use { arena ->
            val inSeg = arena.allocate(rows.toLong() * k * Float.SIZE_BYTES, 16)
            MemorySegment.copy(activation, aHeap.arrayOffset + a.layout.offsetElements.toInt(), inSeg, ValueLayout.JAVA_FLOAT, 0L, rows * k)
            val outSeg = arena.allocate(rows.toLong() * n * Float.SIZE_BYTES, 16)
            val rc = fn.invoke(handle, inSeg, rows, outSeg) as Int
            check(rc == 0) { "$name: ${HipLibrary.error()}" }
            MemorySegment.copy(outSeg, ValueLayout.JAVA_FLOAT, 0L, output, oHeap.arrayOffset + out.layout.offsetElements.toInt(), rows * n)
        }
        if (sink.isEnabled) sink.emit(TraceEvent.KernelRun(op = key.op, kernel = name, inputs = inputs.map { it.id }, output = out.id))
    }

    /** The resident handle of the weight behind [w] ([n, k] packed rows), uploaded the first time its storage is seen; `null` when the upload fails. */
    internal fun handleFor(w: TensorView): MemorySegment? = synchronized(resident) {
        resident[w.storage] ?: upload(w, w.shape[0], w.shape[1])?.also { resident[w.storage] = it }
    }

    /**
     * The packed bytes of [w] to the device. A mapped or direct buffer is handed to the library as it lies (no host
     * copy: the library reads the mapping once); a heap array goes through one native segment of its size.
     */
    private fun upload(w: TensorView, n: Int, k: Int): MemorySegment? {
        val fn = HipLibrary.weightUpload ?: return null
        val nbytes = n.toLong() * (k / blockElems) * blockBytes
        val offset = w.layout.offsetElements * w.layout.elementBytes
        return when (val s = w.storage) {
            is MappedBufferStorage, is DirectBufferStorage -> {
                val buffer = if (s is MappedBufferStorage) s.buffer() else (s as DirectBufferStorage).buffer()
                val bytes = MemorySegment.ofBuffer(buffer).asSlice(offset, nbytes)
                (fn.invoke(bytes, nbytes, encodingId, ORDER_ROW_MAJOR, n, k) as MemorySegment).takeUnless { it == MemorySegment.NULL }
            }
            is Storage.Heap -> {
                val array = s.bytes ?: return null
                Arena.ofConfined().use { arena ->
                    val bytes = arena.allocate(nbytes, 16)
                    MemorySegment.copy(array, s.arrayOffset + offset.toInt(), bytes, ValueLayout.JAVA_BYTE, 0L, nbytes.toInt())
                    (fn.invoke(bytes, nbytes, encodingId, ORDER_ROW_MAJOR, n, k) as MemorySegment).takeUnless { it == MemorySegment.NULL }
                }
            }
            else -> null
        }
    }

    /** Frees every resident weight of this kernel (a ModelScope close hook calls it when the model goes away). */
    public fun releaseWeights() {
        synchronized(resident) {
            resident.values.forEach { HipLibrary.weightFree?.invoke(it) }
            resident.clear()
        }
    }

    /** Never wrong numbers and never silent: the decoding reference runs, and the trace says why. */
    private fun fallback(inputs: List<TensorView>, out: TensorView, sink: TraceSink, reason: String) {
        if (sink.isEnabled) {
            sink.emit(TraceEvent.KernelRun(op = key.op, kernel = "reference-fallback from $name: $reason", inputs = inputs.map { it.id }, output = out.id))
        }
        ReferenceMatmulKernel(key).run(inputs, out)
    }

    public companion object {
        private const val ORDER_ROW_MAJOR = 0

        public fun keyFor(encoding: TensorEncoding): KernelKey = KernelKey(
            op = "matmul",
            operands = listOf(OperandKey.contiguous(Format.dense(FP32)), OperandKey(Format(FP32, encoding), LayoutClass.BLOCKED_ROW_MAJOR)),
        )
    }
}

/** Registers one [HipRowMajorMatmulKernel] per packed encoding; later registrations win, so these outrank the CPU pack. */
public object HipRowMajorKernelPack : ViewKernelPack {
    override val name: String = "hip-rowmajor"

    /** (encoding, GGML type id, elements per block, bytes per block) */
    private val FORMATS = listOf(
        Quad(TensorEncoding.Q4_K, 12, 256, 144), Quad(TensorEncoding.Q6_K, 14, 256, 210), Quad(TensorEncoding.Q5_K, 13, 256, 176),
        Quad(TensorEncoding.Q8_0, 8, 32, 34), Quad(TensorEncoding.Q4_0, 2, 32, 18), Quad(TensorEncoding.Q5_0, 6, 32, 22),
        Quad(TensorEncoding.Q5_1, 7, 32, 24),
    )
    private data class Quad(val encoding: TensorEncoding, val id: Int, val elems: Int, val bytes: Int)

    private val installed = mutableListOf<HipRowMajorMatmulKernel>()

    /** Idempotent, never throws; without a usable device nothing is registered. */
    @Synchronized
    override fun install() {
        if (installed.isNotEmpty() || !HipLibrary.usable || HipLibrary.matmulHost == null) return
        for (f in FORMATS) {
            val kernel = HipRowMajorMatmulKernel(f.encoding, f.id, f.elems, f.bytes, HipRowMajorMatmulKernel.keyFor(f.encoding))
            KernelDispatch.register(kernel)
            installed += kernel
        }
    }

    /**
     * The resident handle for a packed weight view (uploading it on first sight), for callers that run the device
     * entries themselves ([HipOps]); `null` for an encoding, block order or inner dimension this pack does not serve.
     */
    @Synchronized
    internal fun handleFor(w: TensorView): MemorySegment? {
        install()
        if (w.shape.rank != 2 || w.layout.blockOrder != BlockOrder.ROW_MAJOR) return null
        val format = FORMATS.firstOrNull { it.encoding == w.format.encoding } ?: return null
        if (w.shape[1] % format.elems != 0) return null
        return installed.firstOrNull { it.encodingOf() == format.encoding }?.handleFor(w)
    }

    /** Device memory of every weight uploaded through this pack goes back to the device. */
    @Synchronized
    public fun releaseWeights(): Unit = installed.forEach { it.releaseWeights() }
}

/** Public no-argument class for `ServiceLoader` (META-INF/services/sk.ainet.backend.api.kernel.ViewKernelPack). */
public class HipRowMajorKernelPackFactory : ViewKernelPack by HipRowMajorKernelPack
