package sk.ainet.exec.hip

import java.lang.foreign.Arena
import java.lang.foreign.MemorySegment
import java.lang.foreign.ValueLayout
import java.lang.invoke.MethodHandle
import kotlin.reflect.KClass
import sk.ainet.context.schedule.Schedule
import sk.ainet.exec.tensor.ops.DefaultCpuOpsBase
import sk.ainet.lang.memory.BlockOrder
import sk.ainet.lang.memory.Scope
import sk.ainet.lang.tensor.Shape
import sk.ainet.lang.tensor.Tensor
import sk.ainet.lang.tensor.data.TensorData
import sk.ainet.lang.tensor.data.TensorDataFactory
import sk.ainet.lang.tensor.ops.FusedNormOps
import sk.ainet.lang.tensor.ops.TensorOps
import sk.ainet.lang.tensor.storage.MemoryDomain
import sk.ainet.lang.types.DType
import sk.ainet.lang.types.FP32

/**
 * `TensorOps` with activations resident in the GPU's memory: the common CPU implementation with the dense matmuls, the
 * packed-weight product, the elementwise arithmetic, the activations, the reductions, softmax, the fused normalisations
 * and attention routed to libskainet_hip's device entries, their outputs kept on the device as [HipTensorData]. A model
 * built with the NN DSL on this ops instance runs its forward pass without an activation crossing PCIe; the first op
 * that does not know the device (anything not overridden here) reads the heap mirror, one download.
 *
 * The method set and the rules of the browser tier's resident ops
 * (skainet-backends/skainet-backend-wasm-simd/src/wasmJsMain/kotlin/sk/ainet/exec/wasm/WasmCpuOps.kt:180-428), with one
 * addition that tier does not need: a packed weight (Q4_K, Q6_K, Q5_K, Q8_0, Q4_0, Q5_0, Q5_1 in canonical row-major
 * block order) under a resident activation runs `skainet_hip_matmul_dev` on the weight handle the view kernel pack
 * keeps, instead of leaving the device for the kernel registry's heap route.
 *
 * What runs on the device, and when:
 *  - `matmul`, `matmulWeightTransposed` on dense FP32, `matmulWeightTransposed` on a packed weight,
 *    `scaledDotProductAttention`: always. A heap operand is uploaded for the call, the output is resident.
 *  - `add` / `subtract` / `multiply` / `divide`, the activations, `sum` / `mean`, `softmax` / `logSoftmax` over the last
 *    dimension and the normalisations of [FusedNormOps]: when an operand is already resident. A chain becomes resident
 *    at its first matmul (or at [toResident]); two heap operands stay on the CPU, where a copy each way over PCIe would
 *    cost more than the loop.
 *  - broadcasts the kernel takes: equal shapes, a single value, a bias along the last dimension.
 * Every other case, and every case while no device is usable, is the common implementation on the mirror.
 *
 * Outputs come from [slab] when one is given (reset by the caller once per forward pass, beside its forward scope),
 * from the active scope when it hands out device memory, else from ambient device allocations freed by `close()` of
 * their storage. Launches are asynchronous on the calling thread's stream; reading a value waits.
 */
public class HipOps(
    dataFactory: TensorDataFactory,
    schedule: Schedule,
    private val slab: HipActivationSlab? = null,
) : DefaultCpuOpsBase(dataFactory, schedule), FusedNormOps {

    public constructor(dataFactory: TensorDataFactory) : this(dataFactory, Schedule.Sequential, null)

    override fun withSchedule(schedule: Schedule): TensorOps =
        if (schedule === this.schedule) this else HipOps(dataFactory, schedule, slab)

    /** `x . W^T` reads the weight's rows as they lie; no transposed copy on the way. */
    override fun preferDirectWeightTransposed(): Boolean = false

    // ---- operands -------------------------------------------------------------------------------------------------------

    private fun deviceData(t: Tensor<*, *>): HipTensorData<*>? = (t.data as? HipTensorData<*>)?.takeIf { it.isResident }

    private fun onDevice(t: Tensor<*, *>): Boolean = deviceData(t) != null

    private fun denseFp32(t: Tensor<*, *>): Boolean = t.dtype == FP32::class && (t.data is HipTensorData<*> || t.data.heapFloats != null)

    /**
     * The device addresses of one call's operands. A resident operand is used where it is; a heap operand is uploaded
     * into a temporary that [close] frees (the free waits for the device, so the kernel has read it by then).
     */
    private class Call : AutoCloseable {
        private val temporaries = ArrayList<MemorySegment>()

        fun floats(src: FloatArray, offset: Int, count: Int): MemorySegment {
            val bytes = maxOf(count, 1).toLong() * Float.SIZE_BYTES
            val dev = HipLibrary.malloc!!.invoke(bytes) as MemorySegment
            check(dev != MemorySegment.NULL) { "HipOps: ${HipLibrary.error()}" }
            temporaries += dev
            if (count > 0) Arena.ofConfined().use { arena ->
                val host = arena.allocate(bytes, 16)
                MemorySegment.copy(src, offset, host, ValueLayout.JAVA_FLOAT, 0L, count)
                check((HipLibrary.h2d!!.invoke(dev, host, bytes) as Int) == 0) { "HipOps: ${HipLibrary.error()}" }
            }
            return dev
        }

        fun ints(src: IntArray): MemorySegment {
            val bytes = maxOf(src.size, 1).toLong() * Int.SIZE_BYTES
            val dev = HipLibrary.malloc!!.invoke(bytes) as MemorySegment
            check(dev != MemorySegment.NULL) { "HipOps: ${HipLibrary.error()}" }
            temporaries += dev
            if (src.isNotEmpty()) Arena.ofConfined().use { arena ->
                check((HipLibrary.h2d!!.invoke(dev, HipStaging.ints(arena, src), bytes) as Int) == 0) { "HipOps: ${HipLibrary.error()}" }
            }
            return dev
        }

        override fun close() {
            temporaries.forEach { HipLibrary.free?.invoke(it) }
            temporaries.clear()
        }
    }

    private fun Call.operand(t: Tensor<*, *>): MemorySegment? {
        deviceData(t)?.let { return it.pointer() }
        if (t.data is HipTensorData<*>) return null                 // its scope is gone: the common path reports it
        val heap = t.data.heapFloats ?: return null
        return floats(heap, t.data.heapFloatsOffset, t.shape.volume)
    }

    /** A norm gain or bias of [cols] values: in place, uploaded, or (not FP32) copied out first. */
    private fun Call.parameter(t: Tensor<*, *>, cols: Int): MemorySegment? {
        if (t.shape.volume != cols) return null
        if (t.dtype == FP32::class) operand(t)?.let { return it }
        return floats(t.data.copyToFloatArray(), 0, cols)
    }

    // ---- outputs --------------------------------------------------------------------------------------------------------

    private fun deviceBytes(bytes: Long): HipDeviceStorage {
        slab?.allocate(bytes)?.let { return it }
        val scope = dispatchScope()
        if (scope !== Scope.Ambient) {
            (runCatching { scope.allocate(bytes, MemoryDomain.DEVICE_LOCAL) }.getOrNull() as? HipDeviceStorage)?.let { return it }
        }
        return HipDeviceStorage.allocate(bytes)
    }

    @Suppress("UNCHECKED_CAST")
    private inline fun <T : DType, V> resident(
        shape: Shape, dtype: KClass<T>, inputs: Array<out Tensor<T, V>>, who: String, launch: (MemorySegment) -> Int,
    ): Tensor<T, V> {
        val storage = deviceBytes(maxOf(shape.volume, 1).toLong() * Float.SIZE_BYTES)
        val rc = launch(storage.pointer())
        check(rc == 0) { "HipOps.$who: ${HipLibrary.error()}" }
        return newTensor(HipTensorData<T>(shape, storage) as TensorData<T, V>, dtype, *inputs)
    }

    private fun ready(vararg handles: MethodHandle?): Boolean = HipLibrary.usable && handles.all { it != null }

    /**
     * A resident copy of a dense FP32 [tensor]: the explicit "upload once" for an input that many device ops will read
     * (a prompt's embeddings, a bench's operands). The tensor itself when it is resident already or cannot be.
     */
    public fun <T : DType, V> toResident(tensor: Tensor<T, V>): Tensor<T, V> {
        if (!ready(HipLibrary.d2d) || !denseFp32(tensor) || onDevice(tensor)) return tensor
        Call().use { call ->
            val src = call.operand(tensor) ?: return tensor
            val bytes = tensor.shape.volume.toLong() * Float.SIZE_BYTES
            return resident(tensor.shape, tensor.dtype, arrayOf(tensor), "toResident") { out ->
                if (bytes == 0L) 0 else HipLibrary.d2d!!.invoke(out, src, bytes) as Int
            }
        }
    }

    // ---- matmuls --------------------------------------------------------------------------------------------------------

    /** Dense `A[m, k] . B[k, n]` on FP32 operands: `skainet_hip_fp32_matmul_dev`, row strides k, n, n. */
    override fun <T : DType, V> matmul(a: Tensor<T, V>, b: Tensor<T, V>): Tensor<T, V> {
        if (!ready(HipLibrary.sgemmDev) || a.rank != 2 || b.rank != 2 || !denseFp32(a) || !denseFp32(b) || untransposedWeight(b) != null) {
            return super.matmul(a, b)
        }
        val m = a.shape[0]
        val k = a.shape[1]
        val n = b.shape[1]
        require(k == b.shape[0]) { "Matrix multiplication shape mismatch: ${a.shape} vs ${b.shape}" }
        if (m == 0 || n == 0) return super.matmul(a, b)
        Call().use { call ->
            val ap = call.operand(a) ?: return super.matmul(a, b)
            val bp = call.operand(b) ?: return super.matmul(a, b)
            return resident(Shape(m, n), a.dtype, arrayOf(a, b), "matmul") { out ->
                HipLibrary.sgemmDev!!.invoke(ap, 0, k, bp, 0, n, out, 0, n, m, n, k) as Int
            }
        }
    }

    /**
     * `x[..., k] . W[n, k]^T`: a dense FP32 weight through `skainet_hip_fp32_matmul_wt_dev`, a packed weight through
     * `skainet_hip_matmul_dev` on its resident handle (GEMV kernels up to 8 rows, the matrix-core GEMM above).
     */
    override fun <T : DType, V> matmulWeightTransposed(x: Tensor<T, V>, weight: Tensor<T, V>): Tensor<T, V> {
        if (!HipLibrary.usable || weight.rank != 2 || x.rank < 1 || !denseFp32(x)) return super.matmulWeightTransposed(x, weight)
        val n = weight.shape[0]
        val k = weight.shape[1]
        if (k == 0 || n == 0 || x.shape.dimensions.last() != k) return super.matmulWeightTransposed(x, weight)
        val m = x.shape.volume / k
        if (m == 0) return super.matmulWeightTransposed(x, weight)
        val outShape = if (x.rank == 1) Shape(n) else Shape(*(x.shape.dimensions.copyOf(x.rank - 1) + n))
        Call().use { call ->
            if (denseFp32(weight)) {
                val fn = HipLibrary.sgemmWtDev ?: return super.matmulWeightTransposed(x, weight)
                val xp = call.operand(x) ?: return super.matmulWeightTransposed(x, weight)
                val wp = call.operand(weight) ?: return super.matmulWeightTransposed(x, weight)
                return resident(outShape, x.dtype, arrayOf(x, weight), "matmulWeightTransposed") { out ->
                    fn.invoke(xp, 0, wp, 0, out, 0, m, n, k) as Int
                }
            }
            val fn = HipLibrary.matmulDev ?: return super.matmulWeightTransposed(x, weight)
            val view = weight.data.view ?: return super.matmulWeightTransposed(x, weight)
            if (view.format.isDense || view.layout.blockOrder != BlockOrder.ROW_MAJOR) return super.matmulWeightTransposed(x, weight)
            val handle = HipRowMajorKernelPack.handleFor(view) ?: return super.matmulWeightTransposed(x, weight)
            val xp = call.operand(x) ?: return super.matmulWeightTransposed(x, weight)
            return resident(outShape, x.dtype, arrayOf(x), "matmulWeightTransposed") { out -> fn.invoke(handle, xp, m, out) as Int }
        }
    }

    // ---- elementwise ----------------------------------------------------------------------------------------------------

    /** How the kernel indexes an operand of shape [s] against the output [out]; `null` for a broadcast it does not take. */
    private fun indexMode(s: Shape, out: Shape): Int? = when {
        s == out -> MODE_FULL
        s.volume == 1 -> MODE_SCALAR
        s.rank >= 1 && out.rank >= 1 && s[s.rank - 1] == out[out.rank - 1] && s.volume == s[s.rank - 1] -> MODE_BIAS
        else -> null
    }

    private fun <T : DType, V> binary(op: Int, a: Tensor<T, V>, b: Tensor<T, V>): Tensor<T, V>? {
        val fn = HipLibrary.binaryDev
        if (!ready(fn) || a.dtype != b.dtype || !denseFp32(a) || !denseFp32(b) || !(onDevice(a) || onDevice(b))) return null
        val outShape = runCatching { broadcastShapes(a.shape, b.shape) }.getOrNull() ?: return null
        val count = outShape.volume
        if (count == 0 || outShape.rank == 0) return null
        val am = indexMode(a.shape, outShape) ?: return null
        val bm = indexMode(b.shape, outShape) ?: return null
        Call().use { call ->
            val ap = call.operand(a) ?: return null
            val bp = call.operand(b) ?: return null
            return resident(outShape, a.dtype, arrayOf(a, b), "binary") { out ->
                fn!!.invoke(op, ap, am, bp, bm, out, count.toLong(), outShape[outShape.rank - 1]) as Int
            }
        }
    }

    override fun <T : DType, V> add(a: Tensor<T, V>, b: Tensor<T, V>): Tensor<T, V> = binary(0, a, b) ?: super.add(a, b)
    override fun <T : DType, V> subtract(a: Tensor<T, V>, b: Tensor<T, V>): Tensor<T, V> = binary(1, a, b) ?: super.subtract(a, b)
    override fun <T : DType, V> multiply(a: Tensor<T, V>, b: Tensor<T, V>): Tensor<T, V> = binary(2, a, b) ?: super.multiply(a, b)
    override fun <T : DType, V> divide(a: Tensor<T, V>, b: Tensor<T, V>): Tensor<T, V> = binary(3, a, b) ?: super.divide(a, b)

    // ---- activations ----------------------------------------------------------------------------------------------------

    private fun <T : DType, V> unary(op: Int, t: Tensor<T, V>): Tensor<T, V>? {
        val fn = HipLibrary.unaryDev
        if (!ready(fn) || !denseFp32(t) || !onDevice(t) || t.shape.volume == 0) return null
        val count = t.shape.volume.toLong()
        val src = deviceData(t)!!.pointer()
        return resident(t.shape, t.dtype, arrayOf(t), "unary") { out -> fn!!.invoke(op, src, out, count) as Int }
    }

    override fun <T : DType, V> relu(tensor: Tensor<T, V>): Tensor<T, V> = unary(0, tensor) ?: super.relu(tensor)
    override fun <T : DType, V> sigmoid(tensor: Tensor<T, V>): Tensor<T, V> = unary(1, tensor) ?: super.sigmoid(tensor)
    override fun <T : DType, V> silu(tensor: Tensor<T, V>): Tensor<T, V> = unary(2, tensor) ?: super.silu(tensor)
    override fun <T : DType, V> gelu(tensor: Tensor<T, V>, approximate: Boolean): Tensor<T, V> =
        unary(if (approximate) 3 else 4, tensor) ?: super.gelu(tensor, approximate)
    override fun <T : DType, V> erf(tensor: Tensor<T, V>): Tensor<T, V> = unary(5, tensor) ?: super.erf(tensor)
    override fun <T : DType, V> tanh(tensor: Tensor<T, V>): Tensor<T, V> = unary(6, tensor) ?: super.tanh(tensor)

    // ---- reductions -----------------------------------------------------------------------------------------------------

    private fun <T : DType, V> reduce(t: Tensor<T, V>, dim: Int?, mean: Boolean): Tensor<T, V>? {
        if (!ready(HipLibrary.reduceAllDev, HipLibrary.reduceAxisDev) || !denseFp32(t) || !onDevice(t) || t.shape.volume == 0) return null
        val src = deviceData(t)!!.pointer()
        val flag = if (mean) 1 else 0
        if (dim == null) {
            val count = t.shape.volume.toLong()
            return resident(Shape(), t.dtype, arrayOf(t), "reduce") { out -> HipLibrary.reduceAllDev!!.invoke(src, count, flag, out) as Int }
        }
        val axis = if (dim < 0) dim + t.rank else dim
        if (axis !in 0 until t.rank) return null
        val dims = t.shape.dimensions
        val outer = dims.take(axis).fold(1) { acc, d -> acc * d }
        val inner = dims.drop(axis + 1).fold(1) { acc, d -> acc * d }
        val kept = dims.filterIndexed { i, _ -> i != axis }.toIntArray()
        return resident(Shape(kept), t.dtype, arrayOf(t), "reduce") { out ->
            HipLibrary.reduceAxisDev!!.invoke(src, outer, dims[axis], inner, flag, out) as Int
        }
    }

    override fun <T : DType, V> sum(tensor: Tensor<T, V>, dim: Int?): Tensor<T, V> = reduce(tensor, dim, mean = false) ?: super.sum(tensor, dim)
    override fun <T : DType, V> mean(tensor: Tensor<T, V>, dim: Int?): Tensor<T, V> = reduce(tensor, dim, mean = true) ?: super.mean(tensor, dim)

    // ---- row kernels: softmax, the normalisations, attention ------------------------------------------------------------

    private fun <T : DType, V> softmaxRows(t: Tensor<T, V>, dim: Int, log: Boolean): Tensor<T, V>? {
        val fn = HipLibrary.softmaxDev
        if (!ready(fn) || !denseFp32(t) || !onDevice(t) || t.rank == 0) return null
        if ((if (dim < 0) dim + t.rank else dim) != t.rank - 1) return null
        val cols = t.shape[t.rank - 1]
        if (cols <= 0 || t.shape.volume == 0) return null
        val rows = t.shape.volume / cols
        val src = deviceData(t)!!.pointer()
        return resident(t.shape, t.dtype, arrayOf(t), "softmax") { out -> fn!!.invoke(src, out, rows, cols, if (log) 1 else 0) as Int }
    }

    override fun <T : DType, V> softmax(tensor: Tensor<T, V>, dim: Int): Tensor<T, V> = softmaxRows(tensor, dim, log = false) ?: super.softmax(tensor, dim)
    override fun <T : DType, V> logSoftmax(tensor: Tensor<T, V>, dim: Int): Tensor<T, V> = softmaxRows(tensor, dim, log = true) ?: super.logSoftmax(tensor, dim)

    private fun <T : DType, V> normalise(
        input: Tensor<T, V>, gamma: Tensor<T, V>?, beta: Tensor<T, V>?, eps: Float, normalizedRank: Int, rms: Boolean,
    ): Tensor<T, V>? {
        if (!ready(HipLibrary.rmsNormDev, HipLibrary.layerNormDev) || !denseFp32(input) || !onDevice(input)) return null
        if (normalizedRank !in 1..input.rank) return null
        val cols = input.shape.dimensions.drop(input.rank - normalizedRank).fold(1) { acc, d -> acc * d }
        if (cols == 0 || input.shape.volume == 0) return null
        val rows = input.shape.volume / cols
        Call().use { call ->
            val src = deviceData(input)!!.pointer()
            val g = if (gamma == null) MemorySegment.NULL else call.parameter(gamma, cols) ?: return null
            val b = if (beta == null) MemorySegment.NULL else call.parameter(beta, cols) ?: return null
            val inputs = listOfNotNull(input, gamma, beta).toTypedArray()
            return resident(input.shape, input.dtype, inputs, if (rms) "rmsNorm" else "layerNorm") { out ->
                if (rms) HipLibrary.rmsNormDev!!.invoke(src, g, out, rows, cols, eps) as Int
                else HipLibrary.layerNormDev!!.invoke(src, g, b, out, rows, cols, eps) as Int
            }
        }
    }

    /** `null` means "not this path": the caller (`LayerNormalization`) then composes the norm from plain ops. */
    override fun <T : DType, V> layerNorm(input: Tensor<T, V>, gamma: Tensor<T, V>?, beta: Tensor<T, V>?, eps: Float, normalizedRank: Int): Tensor<T, V>? =
        normalise(input, gamma, beta, eps, normalizedRank, rms = false)

    override fun <T : DType, V> rmsNorm(input: Tensor<T, V>, gamma: Tensor<T, V>?, eps: Float, normalizedRank: Int): Tensor<T, V>? =
        normalise(input, gamma, null, eps, normalizedRank, rms = true)

    /**
     * Attention in one device pass (`skainet_hip_f32_sdpa_dev`): the operand contract and the mask rules of the common
     * implementation (its validation runs first, so a bad call fails with the same message), scores never materialised.
     */
    override fun <T : DType, V> scaledDotProductAttention(
        query: Tensor<T, V>,
        key: Tensor<T, V>,
        value: Tensor<T, V>,
        mask: Tensor<T, V>?,
        scale: Float,
        causal: Boolean,
        keyLengths: Tensor<DType, *>?,
        window: Int,
        rightContext: Int,
    ): Tensor<T, V> {
        val fn = HipLibrary.sdpaDev
        val dense = denseFp32(query) && denseFp32(key) && denseFp32(value) && (mask == null || denseFp32(mask))
        if (!ready(fn) || !dense) return super.scaledDotProductAttention(query, key, value, mask, scale, causal, keyLengths, window, rightContext)
        requireSdpaOperands(query, key, value, window, rightContext)
        val (batch, heads, seqQ, headDim) = query.shape.dimensions
        val kvHeads = key.shape[1]
        val seqKv = key.shape[2]
        val lengths = sdpaKeyLengths(keyLengths, batch, seqKv)
        val md = sdpaMaskDims(mask, batch, heads, kvHeads, seqQ, seqKv) ?: intArrayOf(1, 1, 1, 1)
        val factor = if (scale == 0f) (1.0 / kotlin.math.sqrt(headDim.toDouble())).toFloat() else scale
        Call().use { call ->
            val qp = call.operand(query)
            val kp = call.operand(key)
            val vp = call.operand(value)
            val mp = if (mask == null) MemorySegment.NULL else call.operand(mask)
            if (qp == null || kp == null || vp == null || mp == null) {
                return super.scaledDotProductAttention(query, key, value, mask, scale, causal, keyLengths, window, rightContext)
            }
            val lp = if (lengths == null || batch == 0) MemorySegment.NULL else call.ints(lengths)
            return resident(Shape(batch, heads, seqQ, headDim), query.dtype, arrayOf(query, key, value), "scaledDotProductAttention") { out ->
                fn!!.invoke(
                    qp, kp, vp, out, batch, heads, kvHeads, seqQ, seqKv, headDim, factor, if (causal) 1 else 0, window, rightContext,
                    lp, mp, md[0], md[1], md[2], md[3],
                ) as Int
            }
        }
    }

    private companion object {
        const val MODE_FULL = 0
        const val MODE_SCALAR = 1
        const val MODE_BIAS = 2
    }
}
