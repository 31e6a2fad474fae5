package sk.ainet.exec.hip

import java.lang.foreign.Arena
import java.lang.foreign.MemorySegment
import sk.ainet.backend.api.kernel.Fp32AttentionKernel
import sk.ainet.backend.api.kernel.Fp32NormKernel
import sk.ainet.backend.api.kernel.Fp32SoftmaxKernel

/** softmax / log-softmax over the last axis of [rows, cols]. */
internal object HipFp32SoftmaxKernel : Fp32SoftmaxKernel {
    fun isAvailable(): Boolean = HipLibrary.softmax != null
    override fun softmaxRows(input: FloatArray, inputOffset: Int, out: FloatArray, outOffset: Int, rows: Int, cols: Int, log: Boolean) {
        require(rows >= 0 && cols >= 0) { "HipFp32SoftmaxKernel: rows and cols must be non-negative; got rows=$rows cols=$cols" }
        if (rows == 0 || cols == 0) return
        val fn = HipLibrary.softmax ?: error("HipFp32SoftmaxKernel invoked while libskainet_hip is unavailable")
        val n = rows.toLong() * cols
        Arena.ofConfined().use { arena ->
            val inSeg = HipStaging.floats(arena, input, inputOffset, n, "HipFp32SoftmaxKernel: input")
            val outSeg = HipStaging.output(arena, n)
            fn.invoke(inSeg, outSeg, rows, cols, if (log) 1 else 0)
            HipLibrary.checkHostCall("HipFp32SoftmaxKernel")
            HipStaging.read(outSeg, out, outOffset, n, "HipFp32SoftmaxKernel: output")
        }
    }
}

/** LayerNorm and RMSNorm over the last axis; gamma / beta optional. */
internal object HipFp32NormKernel : Fp32NormKernel {
    fun isAvailable(): Boolean = HipLibrary.layerNorm != null && HipLibrary.rmsNorm != null

    override fun layerNorm(input: FloatArray, inputOffset: Int, gamma: FloatArray?, beta: FloatArray?, out: FloatArray, outOffset: Int,
                           rows: Int, cols: Int, eps: Float) {
        require(rows >= 0 && cols >= 0) { "HipFp32NormKernel: rows and cols must be non-negative; got rows=$rows cols=$cols" }
        if (rows == 0 || cols == 0) return
        val fn = HipLibrary.layerNorm ?: error("HipFp32NormKernel invoked while libskainet_hip is unavailable")
        val n = rows.toLong() * cols
        Arena.ofConfined().use { arena ->
            val inSeg = HipStaging.floats(arena, input, inputOffset, n, "HipFp32NormKernel: input")
            val gSeg = gamma?.let { HipStaging.floats(arena, it, 0, cols.toLong(), "HipFp32NormKernel: gamma") } ?: MemorySegment.NULL
            val bSeg = beta?.let { HipStaging.floats(arena, it, 0, cols.toLong(), "HipFp32NormKernel: beta") } ?: MemorySegment.NULL
            val outSeg = HipStaging.output(arena, n)
            fn.invoke(inSeg, gSeg, bSeg, outSeg, rows, cols, eps)
            HipLibrary.checkHostCall("HipFp32NormKernel.layerNorm")
            HipStaging.read(outSeg, out, outOffset, n, "HipFp32NormKernel: output")
        }
    }

    override fun rmsNorm(input: FloatArray, inputOffset: Int, gamma: FloatArray?, out: FloatArray, outOffset: Int, rows: Int, cols: Int,
                         eps: Float) {
        require(rows >= 0 && cols >= 0) { "HipFp32NormKernel: rows and cols must be non-negative; got rows=$rows cols=$cols" }
        if (rows == 0 || cols == 0) return
        val fn = HipLibrary.rmsNorm ?: error("HipFp32NormKernel invoked while libskainet_hip is unavailable")
        val n = rows.toLong() * cols
        Arena.ofConfined().use { arena ->
            val inSeg = HipStaging.floats(arena, input, inputOffset, n, "HipFp32NormKernel: input")
            val gSeg = gamma?.let { HipStaging.floats(arena, it, 0, cols.toLong(), "HipFp32NormKernel: gamma") } ?: MemorySegment.NULL
            val outSeg = HipStaging.output(arena, n)
            fn.invoke(inSeg, gSeg, outSeg, rows, cols, eps)
            HipLibrary.checkHostCall("HipFp32NormKernel.rmsNorm")
            HipStaging.read(outSeg, out, outOffset, n, "HipFp32NormKernel: output")
        }
    }
}

/** Fused scaled-dot-product attention over whole contiguous arrays; `scale` applied as given, `out` fully overwritten. */
internal object HipFp32AttentionKernel : Fp32AttentionKernel {
    fun isAvailable(): Boolean = HipLibrary.sdpa != null

    override fun sdpa(
        query: FloatArray, key: FloatArray, value: FloatArray, out: FloatArray,
        batch: Int, heads: Int, kvHeads: Int,
        seqQ: Int, seqKV: Int, headDim: Int,
        scale: Float, causal: Boolean, window: Int, rightContext: Int,
        keyLengths: IntArray?,
        mask: FloatArray?, maskDims: IntArray?,
    ) {
        val who = "HipFp32AttentionKernel"
        require(batch >= 0 && heads >= 0 && kvHeads >= 0 && seqQ >= 0 && seqKV >= 0 && headDim >= 0) { "$who: dimensions must be non-negative" }
        require(kvHeads > 0 && heads % kvHeads == 0) { "$who: heads ($heads) must be a multiple of kvHeads ($kvHeads)" }
        require(window >= 0 && rightContext >= 0) { "$who: window and rightContext must be >= 0" }
        require(rightContext == 0 || window > 0) { "$who: rightContext ($rightContext) is only meaningful with window > 0" }
        require(keyLengths == null || keyLengths.size == batch) { "$who: keyLengths has ${keyLengths?.size} rows, batch is $batch" }
        require((mask == null) == (maskDims == null) && (maskDims == null || maskDims.size == 4)) { "$who: mask and maskDims (4 dims) go together" }
        val qCount = batch.toLong() * heads * seqQ * headDim
        val kvCount = batch.toLong() * kvHeads * seqKV * headDim
        if (qCount == 0L) return
        val fn = HipLibrary.sdpa ?: error("$who invoked while libskainet_hip is unavailable")
        Arena.ofConfined().use { arena ->
            val qSeg = HipStaging.floats(arena, query, 0, qCount, "$who: query")
            val kSeg = HipStaging.floats(arena, key, 0, kvCount, "$who: key")
            val vSeg = HipStaging.floats(arena, value, 0, kvCount, "$who: value")
            val lenSeg = keyLengths?.let { HipStaging.ints(arena, it) } ?: MemorySegment.NULL
            val md = maskDims ?: intArrayOf(0, 0, 0, 0)
            val maskSeg = mask?.let { HipStaging.floats(arena, it, 0, md[0].toLong() * md[1] * md[2] * md[3], "$who: mask") } ?: MemorySegment.NULL
            val outSeg = HipStaging.output(arena, qCount)
            fn.invoke(qSeg, kSeg, vSeg, outSeg, batch, heads, kvHeads, seqQ, seqKV, headDim, scale, if (causal) 1 else 0, window,
                      rightContext, lenSeg, maskSeg, md[0], md[1], md[2], md[3])
            HipLibrary.checkHostCall(who)
            HipStaging.read(outSeg, out, 0, qCount, "$who: out")
        }
    }
}
