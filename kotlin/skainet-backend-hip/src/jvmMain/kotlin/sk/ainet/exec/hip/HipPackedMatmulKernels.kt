package sk.ainet.exec.hip

import java.lang.foreign.Arena
import java.lang.invoke.MethodHandle
import sk.ainet.backend.api.kernel.Q4KMatmulKernel
import sk.ainet.backend.api.kernel.Q4_0MatmulKernel
import sk.ainet.backend.api.kernel.Q5KMatmulKernel
import sk.ainet.backend.api.kernel.Q5_0MatmulKernel
import sk.ainet.backend.api.kernel.Q5_1MatmulKernel
import sk.ainet.backend.api.kernel.Q6KMatmulKernel
import sk.ainet.backend.api.kernel.Q8_0MatmulKernel

/**
 * The packed GEMV accessors of the provider: one activation row against an input-block-major weight held in a heap
 * ByteArray. The weight is staged per call (this interface hands over an array, not a storage with an identity), so the
 * route is correct and slow by construction; the fast route is [HipRowMajorMatmulKernel], which keeps weights resident.
 */
internal class HipPackedGemv(
    private val who: String,
    private val blockElems: Int,
    private val blockBytes: Int,
    private val handle: () -> MethodHandle?,
) {
    fun isAvailable(): Boolean = handle() != null

    fun matmul(
        input: FloatArray, inputOffset: Int,
        weight: ByteArray, weightByteOffset: Int,
        inputDim: Int, outputDim: Int,
        output: FloatArray, outputOffset: Int,
    ) {
        require(inputDim >= 0 && outputDim >= 0) { "$who: dimensions must be non-negative; got inputDim=$inputDim outputDim=$outputDim" }
        require(inputDim % blockElems == 0) { "$who: inputDim must be a multiple of $blockElems; got $inputDim" }
        if (outputDim == 0) return
        if (inputDim == 0) {
            // an empty dot product: the 32-element formats of the CPU library write zeros, its K-quants return untouched
            if (blockElems == 32) output.fill(0f, outputOffset, outputOffset + outputDim)
            return
        }
        val fn = handle() ?: error("$who invoked while libskainet_hip is unavailable")
        val weightBytes = outputDim.toLong() * (inputDim / blockElems) * blockBytes
        Arena.ofConfined().use { arena ->
            val inSeg = HipStaging.floats(arena, input, inputOffset, inputDim.toLong(), "$who: input")
            val wSeg = HipStaging.bytes(arena, weight, weightByteOffset, weightBytes, "$who: weight")
            val outSeg = HipStaging.output(arena, outputDim.toLong())
            fn.invoke(inSeg, 0, wSeg, 0, inputDim, outputDim, outSeg, 0)
            HipLibrary.checkHostCall(who)
            HipStaging.read(outSeg, output, outputOffset, outputDim.toLong(), "$who: output")
        }
    }
}

internal object HipQ4KMatmulKernel : Q4KMatmulKernel {
    private val gemv = HipPackedGemv("HipQ4KMatmulKernel", 256, 144) { HipLibrary.q4k }
    fun isAvailable(): Boolean = gemv.isAvailable()
    override fun matmul(input: FloatArray, inputOffset: Int, weight: ByteArray, weightByteOffset: Int, inputDim: Int,
                        outputDim: Int, output: FloatArray, outputOffset: Int): Unit =
        gemv.matmul(input, inputOffset, weight, weightByteOffset, inputDim, outputDim, output, outputOffset)
}

internal object HipQ6KMatmulKernel : Q6KMatmulKernel {
    private val gemv = HipPackedGemv("HipQ6KMatmulKernel", 256, 210) { HipLibrary.q6k }
    fun isAvailable(): Boolean = gemv.isAvailable()
    override fun matmul(input: FloatArray, inputOffset: Int, weight: ByteArray, weightByteOffset: Int, inputDim: Int,
                        outputDim: Int, output: FloatArray, outputOffset: Int): Unit =
        gemv.matmul(input, inputOffset, weight, weightByteOffset, inputDim, outputDim, output, outputOffset)
}

internal object HipQ5KMatmulKernel : Q5KMatmulKernel {
    private val gemv = HipPackedGemv("HipQ5KMatmulKernel", 256, 176) { HipLibrary.q5k }
    fun isAvailable(): Boolean = gemv.isAvailable()
    override fun matmul(input: FloatArray, inputOffset: Int, weight: ByteArray, weightByteOffset: Int, inputDim: Int,
                        outputDim: Int, output: FloatArray, outputOffset: Int): Unit =
        gemv.matmul(input, inputOffset, weight, weightByteOffset, inputDim, outputDim, output, outputOffset)
}

internal object HipQ8_0MatmulKernel : Q8_0MatmulKernel {
    private val gemv = HipPackedGemv("HipQ8_0MatmulKernel", 32, 34) { HipLibrary.q80 }
    fun isAvailable(): Boolean = gemv.isAvailable()
    override fun matmul(input: FloatArray, inputOffset: Int, weight: ByteArray, weightByteOffset: Int, inputDim: Int,
                        outputDim: Int, output: FloatArray, outputOffset: Int): Unit =
        gemv.matmul(input, inputOffset, weight, weightByteOffset, inputDim, outputDim, output, outputOffset)
}

internal object HipQ4_0MatmulKernel : Q4_0MatmulKernel {
    private val gemv = HipPackedGemv("HipQ4_0MatmulKernel", 32, 18) { HipLibrary.q40 }
    fun isAvailable(): Boolean = gemv.isAvailable()
    override fun matmul(input: FloatArray, inputOffset: Int, weight: ByteArray, weightByteOffset: Int, inputDim: Int,
                        outputDim: Int, output: FloatArray, outputOffset: Int): Unit =
        gemv.matmul(input, inputOffset, weight, weightByteOffset, inputDim, outputDim, output, outputOffset)
}

internal object HipQ5_0MatmulKernel : Q5_0MatmulKernel {
    private val gemv = HipPackedGemv("HipQ5_0MatmulKernel", 32, 22) { HipLibrary.q50 }
    fun isAvailable(): Boolean = gemv.isAvailable()
    override fun matmul(input: FloatArray, inputOffset: Int, weight: ByteArray, weightByteOffset: Int, inputDim: Int,
                        outputDim: Int, output: FloatArray, outputOffset: Int): Unit =
        gemv.matmul(input, inputOffset, weight, weightByteOffset, inputDim, outputDim, output, outputOffset)
}

internal object HipQ5_1MatmulKernel : Q5_1MatmulKernel {
    private val gemv = HipPackedGemv("HipQ5_1MatmulKernel", 32, 24) { HipLibrary.q51 }
    fun isAvailable(): Boolean = gemv.isAvailable()
    override fun matmul(input: FloatArray, inputOffset: Int, weight: ByteArray, weightByteOffset: Int, inputDim: Int,
                        outputDim: Int, output: FloatArray, outputOffset: Int): Unit =
        gemv.matmul(input, inputOffset, weight, weightByteOffset, inputDim, outputDim, output, outputOffset)
}
