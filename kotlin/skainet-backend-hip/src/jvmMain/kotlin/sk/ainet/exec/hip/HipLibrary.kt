package sk.ainet.exec.hip

import java.lang.foreign.Arena
import java.lang.foreign.FunctionDescriptor
import java.lang.foreign.Linker
import java.lang.foreign.MemorySegment
import java.lang.foreign.SymbolLookup
import java.lang.foreign.ValueLayout
import java.lang.invoke.MethodHandle

/**
 * libskainet_hip.so, loaded once. Every failure on the way (property switch, missing library, missing symbol, no
 * gfx950 device) ends in "unavailable", never in an exception: the registry then keeps the CPU tiers.
 *
 * Properties: `skainet.hip.enabled` (default true), `skainet.hip.device` (default 0).
 */
internal object HipLibrary {
    private val linker: Linker = Linker.nativeLinker()

    val lookup: SymbolLookup? = runCatching {
        if (System.getProperty("skainet.hip.enabled", "true") != "true") null
        else SymbolLookup.libraryLookup(System.mapLibraryName("skainet_hip"), Arena.global())
    }.getOrNull()

    private val I = ValueLayout.JAVA_INT
    private val L = ValueLayout.JAVA_LONG
    private val F = ValueLayout.JAVA_FLOAT
    private val P = ValueLayout.ADDRESS

    private fun bind(name: String, descriptor: FunctionDescriptor): MethodHandle? =
        lookup?.find(name)?.orElse(null)?.let { runCatching { linker.downcallHandle(it, descriptor) }.getOrNull() }

    // ---- runtime
    val available: MethodHandle? = bind("skainet_hip_available", FunctionDescriptor.of(I))
    val init: MethodHandle? = bind("skainet_hip_init", FunctionDescriptor.of(I, I))
    val lastError: MethodHandle? = bind("skainet_hip_last_error", FunctionDescriptor.of(P))
    val sync: MethodHandle? = bind("skainet_hip_sync", FunctionDescriptor.of(I))
    val threadRelease: MethodHandle? = bind("skainet_hip_thread_release", FunctionDescriptor.of(I))

    // ---- device memory (size_t == long on LP64)
    val malloc: MethodHandle? = bind("skainet_hip_malloc", FunctionDescriptor.of(P, L))
    val free: MethodHandle? = bind("skainet_hip_free", FunctionDescriptor.of(I, P))
    val h2d: MethodHandle? = bind("skainet_hip_memcpy_h2d", FunctionDescriptor.of(I, P, P, L))
    val d2h: MethodHandle? = bind("skainet_hip_memcpy_d2h", FunctionDescriptor.of(I, P, P, L))
    val d2d: MethodHandle? = bind("skainet_hip_memcpy_d2d", FunctionDescriptor.of(I, P, P, L))
    /** Page-locked host memory for a loader to read packed weights into: `weightUpload` from it is one DMA transfer. */
    val hostAlloc: MethodHandle? = bind("skainet_hip_host_alloc", FunctionDescriptor.of(P, L))
    val hostFree: MethodHandle? = bind("skainet_hip_host_free", FunctionDescriptor.of(I, P))

    // ---- resident weights
    val weightUpload: MethodHandle? = bind("skainet_hip_weight_upload", FunctionDescriptor.of(P, P, L, I, I, I, I))
    val weightFree: MethodHandle? = bind("skainet_hip_weight_free", FunctionDescriptor.ofVoid(P))
    val matmulHost: MethodHandle? = bind("skainet_hip_matmul_host", FunctionDescriptor.of(I, P, P, I, P))
    val matmulDev: MethodHandle? = bind("skainet_hip_matmul_dev", FunctionDescriptor.of(I, P, P, I, P))

    // ---- host entries with the CPU library's signatures
    /** (input, input_offset, weight, weight_byte_offset, input_dim, output_dim, output, output_offset) */
    private val GEMV: FunctionDescriptor = FunctionDescriptor.ofVoid(P, I, P, I, I, I, P, I)
    val q4k: MethodHandle? = bind("skainet_hip_q4k_matmul", GEMV)
    val q6k: MethodHandle? = bind("skainet_hip_q6k_matmul", GEMV)
    val q5k: MethodHandle? = bind("skainet_hip_q5k_matmul", GEMV)
    val q80: MethodHandle? = bind("skainet_hip_q8_0_matmul", GEMV)
    val q40: MethodHandle? = bind("skainet_hip_q4_0_matmul", GEMV)
    val q50: MethodHandle? = bind("skainet_hip_q5_0_matmul", GEMV)
    val q51: MethodHandle? = bind("skainet_hip_q5_1_matmul", GEMV)

    /** (a, a_offset, a_stride, b, b_offset, b_stride, c, c_offset, c_stride, m, n, k); b is bytes for the narrow floats */
    private val GEMM: FunctionDescriptor = FunctionDescriptor.ofVoid(P, I, I, P, I, I, P, I, I, I, I, I)
    val sgemm: MethodHandle? = bind("skainet_hip_fp32_matmul", GEMM)
    val bf16Gemm: MethodHandle? = bind("skainet_hip_bf16_matmul", GEMM)
    val fp16Gemm: MethodHandle? = bind("skainet_hip_fp16_matmul", GEMM)
    val sgemmWt: MethodHandle? = bind("skainet_hip_fp32_matmul_wt", FunctionDescriptor.ofVoid(P, I, P, I, P, I, I, I, I))

    val rmsNorm: MethodHandle? = bind("skainet_hip_f32_rms_norm", FunctionDescriptor.ofVoid(P, P, P, I, I, F))
    val layerNorm: MethodHandle? = bind("skainet_hip_f32_layer_norm", FunctionDescriptor.ofVoid(P, P, P, P, I, I, F))
    val softmax: MethodHandle? = bind("skainet_hip_f32_softmax_rows", FunctionDescriptor.ofVoid(P, P, I, I, I))
    val sdpa: MethodHandle? = bind(
        "skainet_hip_f32_sdpa",
        FunctionDescriptor.ofVoid(P, P, P, P, I, I, I, I, I, I, F, I, I, I, P, P, I, I, I, I),
    )

    // ---- device entries: every pointer in the GPU's memory, asynchronous on the calling thread's stream, 0 / -1
    val sgemmDev: MethodHandle? = bind("skainet_hip_fp32_matmul_dev", FunctionDescriptor.of(I, P, I, I, P, I, I, P, I, I, I, I, I))
    val sgemmWtDev: MethodHandle? = bind("skainet_hip_fp32_matmul_wt_dev", FunctionDescriptor.of(I, P, I, P, I, P, I, I, I, I))
    val rmsNormDev: MethodHandle? = bind("skainet_hip_f32_rms_norm_dev", FunctionDescriptor.of(I, P, P, P, I, I, F))
    val layerNormDev: MethodHandle? = bind("skainet_hip_f32_layer_norm_dev", FunctionDescriptor.of(I, P, P, P, P, I, I, F))
    val softmaxDev: MethodHandle? = bind("skainet_hip_f32_softmax_rows_dev", FunctionDescriptor.of(I, P, P, I, I, I))
    val sdpaDev: MethodHandle? = bind(
        "skainet_hip_f32_sdpa_dev",
        FunctionDescriptor.of(I, P, P, P, P, I, I, I, I, I, I, F, I, I, I, P, P, I, I, I, I),
    )
    /** (op, a, a_mode, b, b_mode, out, n, inner): op 0 add, 1 sub, 2 mul, 3 div; mode 0 full, 1 scalar, 2 bias */
    val binaryDev: MethodHandle? = bind("skainet_hip_f32_binary_dev", FunctionDescriptor.of(I, I, P, I, P, I, P, L, I))
    /** (op, in, out, n): op 0 relu, 1 sigmoid, 2 silu, 3 gelu (tanh form), 4 gelu (erf form), 5 erf, 6 tanh */
    val unaryDev: MethodHandle? = bind("skainet_hip_f32_unary_dev", FunctionDescriptor.of(I, I, P, P, L))
    val reduceAllDev: MethodHandle? = bind("skainet_hip_f32_reduce_all_dev", FunctionDescriptor.of(I, P, L, I, P))
    val reduceAxisDev: MethodHandle? = bind("skainet_hip_f32_reduce_axis_dev", FunctionDescriptor.of(I, P, I, I, I, I, P))

    // ---- fused device entries a decoder runtime on resident activations calls (no counterpart in the CPU library)
    /** (w, x, m, out, gain, eps, residual, epilogue): epilogue 0 none, 1 += residual, 2 SwiGLU over interleaved (gate, up) rows */
    val matmulFusedDev: MethodHandle? = bind("skainet_hip_matmul_fused_dev", FunctionDescriptor.of(I, P, P, I, P, P, F, P, I))
    /** (w_gate_up, w_down, x, m, gain, eps, residual, out): out = residual + Wdown . swiglu(Wgate_up . rmsnorm(x)) */
    val mlpSwigluDev: MethodHandle? = bind("skainet_hip_mlp_swiglu_dev", FunctionDescriptor.of(I, P, P, P, I, P, F, P, P))
    /** attention over a [kvHeads, capacity, headDim] cache, output head-major / as token rows */
    val sdpaCacheDev: MethodHandle? = bind(
        "skainet_hip_f32_sdpa_cache_dev",
        FunctionDescriptor.of(I, P, P, P, P, I, I, I, I, I, I, I, F, I, I, I, P),
    )
    val sdpaCacheRowsDev: MethodHandle? = bind(
        "skainet_hip_f32_sdpa_cache_rows_dev",
        FunctionDescriptor.of(I, P, P, P, P, I, I, I, I, I, I, I, F, I, I, I, P),
    )
    /** one decode token's attention + output projection (+ residual) */
    val attnOutProjDev: MethodHandle? = bind(
        "skainet_hip_attn_out_proj_dev",
        FunctionDescriptor.of(I, P, P, P, P, I, I, I, I, I, F, I, P, P, P, P),
    )
    val argmaxRowsDev: MethodHandle? = bind("skainet_hip_f32_argmax_rows_dev", FunctionDescriptor.of(I, P, I, I, P))

    /** Cheap, cached, false (not throwing) when the library or a gfx950 device is missing. */
    val usable: Boolean by lazy {
        runCatching {
            (available?.invoke() as? Int) == 1 &&
                (init?.invoke(Integer.getInteger("skainet.hip.device", 0)) as? Int) == 0
        }.getOrDefault(false)
    }

    /** The calling thread's last failure ("" when its last call succeeded). */
    fun error(): String = runCatching {
        (lastError!!.invoke() as MemorySegment).reinterpret(1024).getString(0)
    }.getOrDefault("")

    /** After a `void` host entry: those clear the thread's error text on entry and set it on failure. */
    fun checkHostCall(who: String) {
        val message = error()
        check(message.isEmpty()) { "$who: $message" }
    }
}
