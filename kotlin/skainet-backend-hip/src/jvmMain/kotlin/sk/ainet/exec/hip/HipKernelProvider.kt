package sk.ainet.exec.hip

import sk.ainet.backend.api.kernel.Bf16MatmulKernel
import sk.ainet.backend.api.kernel.Fp16MatmulKernel
import sk.ainet.backend.api.kernel.Fp32AttentionKernel
import sk.ainet.backend.api.kernel.Fp32MatmulKernel
import sk.ainet.backend.api.kernel.Fp32MatmulWtKernel
import sk.ainet.backend.api.kernel.Fp32NormKernel
import sk.ainet.backend.api.kernel.Fp32SoftmaxKernel
import sk.ainet.backend.api.kernel.KernelProvider
import sk.ainet.backend.api.kernel.Q4KMatmulKernel
import sk.ainet.backend.api.kernel.Q4_0MatmulKernel
import sk.ainet.backend.api.kernel.Q5KMatmulKernel
import sk.ainet.backend.api.kernel.Q5_0MatmulKernel
import sk.ainet.backend.api.kernel.Q5_1MatmulKernel
import sk.ainet.backend.api.kernel.Q6KMatmulKernel
import sk.ainet.backend.api.kernel.Q8_0MatmulKernel

/**
 * The kernel provider of the HIP backend. Priority 200 puts it above the native CPU tiers (100), Panama (50) and the
 * scalar kernels (0); without the library or a gfx950 device `isAvailable()` is false and every accessor returns null,
 * so the registry falls through to those tiers.
 */
public object HipKernelProvider : KernelProvider {
    public const val PRIORITY: Int = 200

    override val name: String = "hip"
    override val priority: Int = PRIORITY
    override fun isAvailable(): Boolean = HipLibrary.usable

    override fun matmulFp32(): Fp32MatmulKernel? = HipFp32MatmulKernel.takeIf { isAvailable() && it.isAvailable() }
    override fun matmulFp32Wt(): Fp32MatmulWtKernel? = HipFp32MatmulWtKernel.takeIf { isAvailable() && it.isAvailable() }
    override fun matmulBf16(): Bf16MatmulKernel? = HipBf16MatmulKernel.takeIf { isAvailable() && it.isAvailable() }
    override fun matmulFp16(): Fp16MatmulKernel? = HipFp16MatmulKernel.takeIf { isAvailable() && it.isAvailable() }
    override fun matmulQ4K(): Q4KMatmulKernel? = HipQ4KMatmulKernel.takeIf { isAvailable() && it.isAvailable() }
    override fun matmulQ6K(): Q6KMatmulKernel? = HipQ6KMatmulKernel.takeIf { isAvailable() && it.isAvailable() }
    override fun matmulQ5K(): Q5KMatmulKernel? = HipQ5KMatmulKernel.takeIf { isAvailable() && it.isAvailable() }
    override fun matmulQ8_0(): Q8_0MatmulKernel? = HipQ8_0MatmulKernel.takeIf { isAvailable() && it.isAvailable() }
    override fun matmulQ4_0(): Q4_0MatmulKernel? = HipQ4_0MatmulKernel.takeIf { isAvailable() && it.isAvailable() }
    override fun matmulQ5_0(): Q5_0MatmulKernel? = HipQ5_0MatmulKernel.takeIf { isAvailable() && it.isAvailable() }
    override fun matmulQ5_1(): Q5_1MatmulKernel? = HipQ5_1MatmulKernel.takeIf { isAvailable() && it.isAvailable() }
    override fun softmaxFp32(): Fp32SoftmaxKernel? = HipFp32SoftmaxKernel.takeIf { isAvailable() && it.isAvailable() }
    override fun normFp32(): Fp32NormKernel? = HipFp32NormKernel.takeIf { isAvailable() && it.isAvailable() }
    override fun attentionFp32(): Fp32AttentionKernel? = HipFp32AttentionKernel.takeIf { isAvailable() && it.isAvailable() }
}

/** Public no-argument class for `ServiceLoader` (META-INF/services/sk.ainet.backend.api.kernel.KernelProvider). */
public class HipKernelProviderFactory : KernelProvider by HipKernelProvider
