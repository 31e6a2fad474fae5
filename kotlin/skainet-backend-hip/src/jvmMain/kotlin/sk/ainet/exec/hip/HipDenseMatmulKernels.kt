package sk.ainet.exec.hip

import java.lang.foreign.Arena
import java.lang.foreign.MemorySegment
import java.lang.invoke.MethodHandle
import sk.ainet.backend.api.kernel.Bf16MatmulKernel
import sk.ainet.backend.api.kernel.Fp16MatmulKernel
import sk.ainet.backend.api.kernel.Fp32MatmulKernel
import sk.ainet.backend.api.kernel.Fp32MatmulWtKernel

/** Floats an [m, cols] operand with row stride [stride] spans from its first element. */
private fun span(rows: Int, cols: Int, stride: Int): Long = if (rows == 0 || cols == 0) 0L else (rows - 1).toLong() * stride + cols

/** C(m, n) = A(m, k) . B(k, n), strides in floats, C overwritten (k == 0 zeroes it). */
internal object HipFp32MatmulKernel : Fp32MatmulKernel {
    fun isAvailable(): Boolean = HipLibrary.sgemm != null
    override fun matmul(
        a: FloatArray, aOffset: Int, aStride: Int,
        b: FloatArray, bOffset: Int, bStride: Int,
        out: FloatArray, outOffset: Int, outStride: Int,
        m: Int, n: Int, k: Int,
    ) {
        require(m >= 0 && n >= 0 && k >= 0) { "HipFp32MatmulKernel: m, n, k must be non-negative; got $m, $n, $k" }
        if (m == 0 || n == 0) return
        val fn = HipLibrary.sgemm ?: error("HipFp32MatmulKernel invoked while libskainet_hip is unavailable")
        Arena.ofConfined().use { arena ->
            val aSeg = HipStaging.floats(arena, a, aOffset, span(m, k, aStride), "HipFp32MatmulKernel: a")
            val bSeg = HipStaging.floats(arena, b, bOffset, span(k, n, bStride), "HipFp32MatmulKernel: b")
            val cSpan = span(m, n, outStride)
            // rows of C may be strided inside a larger array: stage what lies between so the copy back restores it
            val cSeg = HipStaging.floats(arena, out, outOffset, cSpan, "HipFp32MatmulKernel: out")
            fn.invoke(aSeg, 0, aStride, bSeg, 0, bStride, cSeg, 0, outStride, m, n, k)
            HipLibrary.checkHostCall("HipFp32MatmulKernel")
            HipStaging.read(cSeg, out, outOffset, cSpan, "HipFp32MatmulKernel: out")
        }
    }
}

/** out[i, o] = sum_p x[i, p] * w[o, p]: the Linear.forward shape, all three operands contiguous. */
internal object HipFp32MatmulWtKernel : Fp32MatmulWtKernel {
    fun isAvailable(): Boolean = HipLibrary.sgemmWt != null
    override fun matmulWt(x: FloatArray, xOffset: Int, w: FloatArray, wOffset: Int, out: FloatArray, outOffset: Int,
                          m: Int, n: Int, k: Int) {
        require(m >= 0 && n >= 0 && k >= 0) { "HipFp32MatmulWtKernel: m, n, k must be non-negative; got $m, $n, $k" }
        if (m == 0 || n == 0) return
        val fn = HipLibrary.sgemmWt ?: error("HipFp32MatmulWtKernel invoked while libskainet_hip is unavailable")
        Arena.ofConfined().use { arena ->
            val xSeg = HipStaging.floats(arena, x, xOffset, m.toLong() * k, "HipFp32MatmulWtKernel: x")
            val wSeg = HipStaging.floats(arena, w, wOffset, n.toLong() * k, "HipFp32MatmulWtKernel: w")
            val oSeg = HipStaging.output(arena, m.toLong() * n)
            fn.invoke(xSeg, 0, wSeg, 0, oSeg, 0, m, n, k)
            HipLibrary.checkHostCall("HipFp32MatmulWtKernel")
            HipStaging.read(oSeg, out, outOffset, m.toLong() * n, "HipFp32MatmulWtKernel: out")
        }
    }
}

/** A fp32, B two bytes per element (bf16 / fp16, little endian) with a byte offset and a byte row stride. */
private fun narrowMatmul(
    who: String, fn: MethodHandle?,
    a: FloatArray, aOffset: Int, aStride: Int,
    b: ByteArray, bByteOffset: Int, bByteStride: Int,
    out: FloatArray, outOffset: Int, outStride: Int,
    m: Int, n: Int, k: Int,
) {
    require(m >= 0 && n >= 0 && k >= 0) { "$who: m, n, k must be non-negative; got $m, $n, $k" }
    if (m == 0 || n == 0) return
    val handle = fn ?: error("$who invoked while libskainet_hip is unavailable")
    Arena.ofConfined().use { arena ->
        val aSeg = HipStaging.floats(arena, a, aOffset, span(m, k, aStride), "$who: a")
        val bBytes = if (k == 0) 0L else (k - 1).toLong() * bByteStride + 2L * n
        val bSeg: MemorySegment = HipStaging.bytes(arena, b, bByteOffset, bBytes, "$who: b")
        val cSpan = span(m, n, outStride)
        val cSeg = HipStaging.floats(arena, out, outOffset, cSpan, "$who: out")
        handle.invoke(aSeg, 0, aStride, bSeg, 0, bByteStride, cSeg, 0, outStride, m, n, k)
        HipLibrary.checkHostCall(who)
        HipStaging.read(cSeg, out, outOffset, cSpan, "$who: out")
    }
}

internal object HipBf16MatmulKernel : Bf16MatmulKernel {
    fun isAvailable(): Boolean = HipLibrary.bf16Gemm != null
    override fun matmul(a: FloatArray, aOffset: Int, aStride: Int, b: ByteArray, bByteOffset: Int, bByteStride: Int,
                        out: FloatArray, outOffset: Int, outStride: Int, m: Int, n: Int, k: Int): Unit =
        narrowMatmul("HipBf16MatmulKernel", HipLibrary.bf16Gemm, a, aOffset, aStride, b, bByteOffset, bByteStride, out, outOffset, outStride, m, n, k)
}

internal object HipFp16MatmulKernel : Fp16MatmulKernel {
    fun isAvailable(): Boolean = HipLibrary.fp16Gemm != null
    override fun matmul(a: FloatArray, aOffset: Int, aStride: Int, b: ByteArray, bByteOffset: Int, bByteStride: Int,
                        out: FloatArray, outOffset: Int, outStride: Int, m: Int, n: Int, k: Int): Unit =
        narrowMatmul("HipFp16MatmulKernel", HipLibrary.fp16Gemm, a, aOffset, aStride, b, bByteOffset, bByteStride, out, outOffset, outStride, m, n, k)
}

