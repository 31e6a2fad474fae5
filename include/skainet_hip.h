/*
 * skainet_hip.h -- C ABI of libskainet_hip.so, the MI355X (gfx950) kernel library behind SKaiNET's
 * kernel SPI (skainet-backend-api). Plain pointers and sizes only; a JVM binds it through Panama FFM
 * or JNI exactly as it binds the reference's libskainet_kernels.
 *
 * Two families of entry points:
 *
 *  1. Host-pointer entries with the reference's own signatures (names `skainet_hip_<ref name>`): every
 *     pointer is host memory, the call stages operands to the device, runs, copies the result back
 *     and returns when `output` is complete. They return void like the functions they replace: each
 *     clears the thread's error text on entry, and on a failure nothing is written and
 *     skainet_hip_last_error() tells why. Non-positive dimensions
 *     are no-ops, as in the reference.
 *
 *  2. Device entries (`*_dev`, weight handles): operands are device pointers owned by the caller (or by
 *     this library's allocator), launches are asynchronous on the calling thread's stream
 *     (skainet_hip_set_stream, default: the null stream) and return 0 / -1.
 *
 * Reference paths below are relative to
 *   REF = /root/reference/skainet-backends
 *   NAT = REF/skainet-backend-native-cpu/native/include/skainet_kernels.h
 *   API = REF/skainet-backend-api/src/commonMain/kotlin/sk/ainet/backend/api/kernel
 *
 * Threading: every entry point may be called from any thread. Error text, the current stream and
 * staging buffers are per thread; a weight handle may be shared by threads once uploaded.
 */
#ifndef SKAINET_HIP_H
#define SKAINET_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define SKAINET_HIP_API __attribute__((visibility("default")))

/* Weight encodings: the GGML tensor-type ids StreamingGGUFReader maps to TensorEncoding
 * (REF/../skainet-io/skainet-io-gguf/src/commonMain/kotlin/sk/ainet/io/gguf/StreamingGGUFReader.kt:190-211). */
#define SKAINET_HIP_ENC_Q4_0 2
#define SKAINET_HIP_ENC_Q5_0 6
#define SKAINET_HIP_ENC_Q5_1 7
#define SKAINET_HIP_ENC_Q8_0 8
#define SKAINET_HIP_ENC_Q4_K 12
#define SKAINET_HIP_ENC_Q5_K 13
#define SKAINET_HIP_ENC_Q6_K 14

/* Block orders of a packed weight (REF/../skainet-lang/skainet-lang-core/src/commonMain/kotlin/sk/ainet/lang/memory/Layout.kt:21-27). */
#define SKAINET_HIP_ORDER_ROW_MAJOR 0         /* canonical GGUF order: block (o, b) at (o * blocksPerRow + b) */
#define SKAINET_HIP_ORDER_INPUT_BLOCK_MAJOR 1 /* kernel feed order: block (b, o) at (b * rows + o) */

/* ------------------------------------------------------------------------------------------------
 * Runtime. Replaces what NativeLibraryLoader / KernelProvider.isAvailable() probe on the CPU side
 * (REF/skainet-backend-native-cpu/src/jvmMain/kotlin/sk/ainet/exec/kernel/NativeKernelProvider.kt:98-150):
 * "unavailable" is an answer, never a crash.
 * ---------------------------------------------------------------------------------------------- */

/* 1 when a gfx950 device is present and usable, else 0. Cheap after the first call; never aborts. */
SKAINET_HIP_API int32_t skainet_hip_available(void);
/* Select the device (default 0) for this process. 0 on success. */
SKAINET_HIP_API int32_t skainet_hip_init(int32_t device);
/* Message of the calling thread's last failed call ("" when none). Valid until that thread's next failure. */
SKAINET_HIP_API const char* skainet_hip_last_error(void);
/* Device name ("" when unavailable) and compute-unit count. */
SKAINET_HIP_API const char* skainet_hip_device_name(void);
SKAINET_HIP_API int32_t skainet_hip_compute_units(void);
/* Name of the kernel family the calling thread's last matmul / attention entry launched as its main kernel ("" before
 * the first): lets a measurement say which kernel a number belongs to. No reference counterpart. */
SKAINET_HIP_API const char* skainet_hip_last_kernel(void);
/* Stream (a hipStream_t, NULL = the null stream) used by this thread's later device entries. */
SKAINET_HIP_API int32_t skainet_hip_set_stream(void* stream);
/* Give the calling thread a non-blocking stream of its own (made on first use, destroyed by
 * skainet_hip_thread_release) and use it for this thread's later device entries. The null stream, the default, orders
 * every thread's work behind every other's: a host that calls in from several threads (the reference's schedule
 * workers) calls this once per thread. The caller then orders its own work on other streams against this thread's with
 * skainet_hip_sync. No reference counterpart. 0 on success. */
SKAINET_HIP_API int32_t skainet_hip_thread_stream(void);
/* Wait for this thread's stream. */
SKAINET_HIP_API int32_t skainet_hip_sync(void);
/* Frees the calling thread's scratch (workspace, staging buffers of the host-pointer entries, counters, timer events)
 * after waiting for its stream. For worker threads that end before the process does (the reference's schedule workers,
 * skainet-backend-api/.../kernel/KernelDispatch.kt:28-32, may call in from any thread); no reference counterpart: the CPU
 * library's per-call malloc / free needs none. Free this thread's recorded graphs first. 0 on success. */
SKAINET_HIP_API int32_t skainet_hip_thread_release(void);

/* Device buffers: the backing store of a Storage.Device
 * (REF/../skainet-lang/skainet-lang-core/src/commonMain/kotlin/sk/ainet/lang/memory/Storage.kt:230). */
SKAINET_HIP_API void* skainet_hip_malloc(size_t bytes);
SKAINET_HIP_API int32_t skainet_hip_free(void* device_ptr);
SKAINET_HIP_API int32_t skainet_hip_memcpy_h2d(void* dst_device, const void* src_host, size_t bytes);
SKAINET_HIP_API int32_t skainet_hip_memcpy_d2h(void* dst_host, const void* src_device, size_t bytes);
SKAINET_HIP_API int32_t skainet_hip_memcpy_d2d(void* dst_device, const void* src_device, size_t bytes);
/* Page-locked host memory for a loader to read packed weights into (wrap it as an off-heap MemorySegment, the kind of
 * weight operand REF/skainet-backend-native-cpu/src/jvmMain/kotlin/sk/ainet/exec/kernel/NativeQ4KMemSegMatmulKernel.kt:39-44
 * takes): skainet_hip_weight_upload from it is one DMA transfer with no staging copy on the host. NULL / -1 on failure. */
SKAINET_HIP_API void* skainet_hip_host_alloc(size_t bytes);
SKAINET_HIP_API int32_t skainet_hip_host_free(void* host_ptr);

/* Elapsed-time measurement on the calling thread's stream (HIP events): begin, launch, end -> milliseconds. */
SKAINET_HIP_API int32_t skainet_hip_timer_begin(void);
SKAINET_HIP_API float skainet_hip_timer_end_ms(void);

/* ------------------------------------------------------------------------------------------------
 * Packed weights resident on the device. The device-side analogue of the weight caches keyed by array
 * identity (WASM sidecar handles, REF/skainet-backend-wasm-simd/src/wasmJsMain/kotlin/sk/ainet/exec/wasm/WasmKernels.kt:206-223):
 * upload once, multiply many times.
 * ---------------------------------------------------------------------------------------------- */
typedef struct skainet_hip_weight skainet_hip_weight;

/* Copy `nbytes` packed bytes of a [rows, cols] weight to the device. `order` says how the host bytes are
 * laid out; the device copy is always canonical row-major (an input-block-major source is permuted on
 * the device, the inverse of API/PackedWeights.kt:63-93 toKernelOrder). Returns once the bytes are on the device: page-locked
 * sources (skainet_hip_host_alloc) go as one transfer; pageable ones through page-locked chunks that a few host threads
 * fill while earlier chunks are on the bus (the chunks, 64 MiB by default, are kept until the process ends; staged
 * uploads from several threads take turns). NULL on failure. */
SKAINET_HIP_API skainet_hip_weight* skainet_hip_weight_upload(
    const uint8_t* bytes, int64_t nbytes, int32_t encoding, int32_t order, int32_t rows, int32_t cols);
/* Describe packed row-major bytes that already live on the device (not owned, not freed). */
SKAINET_HIP_API skainet_hip_weight* skainet_hip_weight_wrap(
    const void* device_bytes, int32_t encoding, int32_t rows, int32_t cols);
SKAINET_HIP_API void skainet_hip_weight_free(skainet_hip_weight* w);
SKAINET_HIP_API const void* skainet_hip_weight_data(const skainet_hip_weight* w);
SKAINET_HIP_API int64_t skainet_hip_weight_nbytes(const skainet_hip_weight* w);

/* out[m, rows] = x[m, cols] . W^T, fp32 in and out, device pointers. What a ViewKernel registered for
 * matmul(F32 dense x packed BLOCKED_ROW_MAJOR) runs (API/MatmulKernels.kt:11-40; CPU twin
 * REF/skainet-backend-native-cpu/src/jvmMain/kotlin/sk/ainet/exec/kernel/FfmRowMajorKernels.kt:52-106).
 * m <= 8 streams the weight once per 4 (Q4_K: 8) rows, within 1e-3 of the exact fp32 product; the arithmetic class
 * depends on format and m:
 *   - Q4_K, m = 1, K a multiple of 1024 up to 16384, and Q8_0, m = 1, K a multiple of 1024 up to 4096: codes stay
 *     integers, the activations are rounded to 22-bit fixed point against the largest magnitude of their 64-element
 *     group and contracted on the int8 matrix instruction; scales and minima are applied in fp32 (measured 4e-5 / 2e-5
 *     in the GEMV parity metric). A NaN or an infinity among the activations makes every output NaN.
 *   - Q4_K, m = 3 .. 8: codes exact, an activation enters as bf16 hi + bf16 lo (16 to 17 significant bits) on the bf16
 *     matrix instructions, fp32 sums (2e-4 in the metric).
 *   - everything else (Q4_K m = 2 or other K, Q6_K, Q5_K, Q4_0, Q5_0, Q5_1, Q8_0 at other K): fp32 multiply-adds on
 *     decoded codes, the reference's exact-fp32 products in another summation order.
 *   skainet_hip_set_tuning("q4k_mfma_enable", 0) / ("q8_0_mfma_enable", 0) force the fp32 kernels at m = 1,
 *   ("q4k_wide_enable", 0) + ("q4k_quads_stream_enable", 0) + ("q4k_rows_enable", 0) the fp32 slot kernel at every m.
 * Larger m uses the MFMA dequant-GEMM, which rounds activations and decoded weights to bf16 and accumulates in fp32
 * (within 2e-2 of the largest output): the switch at m = 9 is a switch of precision class as well as of kernel, and
 * skainet_hip_matmul_kind_dev pins either one. */
SKAINET_HIP_API int32_t skainet_hip_matmul_dev(const skainet_hip_weight* w, const float* x, int32_t m, float* out);
/* The same product for the SPI's own calling convention: `x_host` [m, cols] and `out_host` [m, rows] are ordinary
 * host arrays (what MatmulKernels.kt:11-40 hands a ViewKernel), the weight is the resident handle. One upload, the
 * product, one download and one wait per call; the page-locked staging and the device buffers belong to the calling
 * thread and are reused, so a call allocates nothing after the thread's largest shape has been seen. This is the entry
 * HipRowMajorMatmulKernel.run binds. */
SKAINET_HIP_API int32_t skainet_hip_matmul_host(const skainet_hip_weight* w, const float* x_host, int32_t m, float* out_host);
/* Same product, forcing one of the two kernels (kind 0 = GEMV path, 1 = MFMA GEMM path). */
SKAINET_HIP_API int32_t skainet_hip_matmul_kind_dev(const skainet_hip_weight* w, const float* x, int32_t m, float* out, int32_t kind);
/* out = epilogue(W . prologue(x)): a product with the row ops a decoder block puts around it folded in (no reference
 * counterpart as one call; the parts are f32_fused.c:255-286 RMSNorm, f32_ops.c:222-244 SiLU, binary add / mul).
 *   gain != NULL: every activation row is RMS-normalised first, x / sqrt(mean(x^2) + eps) * gain;
 *   epilogue 0: out [m, rows] = product; 1: out = residual + product (residual [m, rows], may alias out);
 *   2: out [m, rows/2], out[j] = silu(p[2j]) * p[2j+1] -- for a weight whose rows alternate gate row, up row.
 * Q4_K weights with m <= 2 run as one kernel; other shapes run the same arithmetic as separate launches. */
SKAINET_HIP_API int32_t skainet_hip_matmul_fused_dev(const skainet_hip_weight* w, const float* x, int32_t m, float* out,
    const float* gain, float eps, const float* residual, int32_t epilogue);
/* One decode token's q/k/v projection with its neighbours folded in (no reference counterpart as one call: RMSNorm
 * f32_fused.c:255-286, the product, RoPE and KvCacheStore.appendToken
 * skainet-lang/skainet-lang-core/src/commonMain/kotlin/sk/ainet/lang/tensor/storage/KvCacheStore.kt:125):
 * row = W . rmsnorm(x) (gain == NULL: no norm), W's rows being [q | k | v] heads of head_dim; adjacent pairs of the q
 * and k heads are rotated by pos * theta^(-2i/head_dim) with pos = *pos_dev; q -> q_out [heads, head_dim], k and v ->
 * row pos of caches [kv_heads, kv_capacity, head_dim]. Q4_K weights run as one kernel. rope_table (may be NULL) is
 * the (cos, sin) table of that position from skainet_hip_f32_rope_table_dev: every layer of a token shares it. */
SKAINET_HIP_API int32_t skainet_hip_matmul_qkv_rope_dev(const skainet_hip_weight* w, const float* x, const float* gain,
    float eps, float* q_out, float* k_cache, float* v_cache, int32_t heads, int32_t kv_heads, int32_t head_dim,
    int32_t kv_capacity, const int32_t* pos_dev, float theta, const float* rope_table);
/* table[2i], table[2i+1] = cos, sin of (*pos_dev) * theta^(-2i/head_dim), i < head_dim/2 (head_dim floats). */
SKAINET_HIP_API int32_t skainet_hip_f32_rope_table_dev(const int32_t* pos_dev, float theta, int32_t head_dim, float* table);
/* Measurement aid: `iters` such products back to back on this thread's stream, weight number i % nweights at
 * step i, timed with HIP events; returns the elapsed milliseconds of one pass of `iters` steps (< 0 on failure): the pass
 * is timed `replays` times (1 .. 64) and the median is returned. use_graph != 0 captures the launches into a HIP graph
 * first and times replays of it, so host launch cost stays off the GPU timeline; about 400 untimed launches come first
 * whatever `iters` is, so a short pass reads the same time per step as a long one.
 * (The reference times its kernels the same way, in a loop around the call: NativeKernel microbench,
 * REF/skainet-backend-native-cpu/src/jvmTest/kotlin/sk/ainet/exec/kernel/Q4KMatmulMicrobenchTest.kt:53-70.) */
SKAINET_HIP_API float skainet_hip_matmul_repeat_dev(const skainet_hip_weight* const* weights, int32_t nweights,
    const float* x, int32_t m, float* out, int32_t iters, int32_t kind, int32_t use_graph, int32_t replays);
/* Calibration aid with no reference counterpart: `iters` launches of a pure streaming-read kernel (16-byte loads,
 * no arithmetic) over buffers[i % nbuffers], each `bytes` long, timed with HIP events; returns milliseconds.
 * The rate it reaches on rotating copies of a weight is the device's ceiling for a read-once pass of that size. */
SKAINET_HIP_API float skainet_hip_read_probe_dev(const void* const* buffers, int32_t nbuffers, int64_t bytes,
    int32_t iters, int32_t grid);
/* Bit-exact decode of the whole weight to fp32 [rows, cols] (the TensorData.dequantizeBlock semantics,
 * REF/../skainet-lang/skainet-lang-core/src/commonMain/kotlin/sk/ainet/lang/tensor/data/Q4_KTensorData.kt:120,
 * Q6_KTensorData.kt:112, Q8_0TensorData.kt:80, Q4_0TensorData.kt:93, Q5_0TensorData.kt:68, Q5_1TensorData.kt:73,
 * Q5_KTensorData.kt:126). */
SKAINET_HIP_API int32_t skainet_hip_dequantize_dev(const skainet_hip_weight* w, float* out);
/* Decode `count` rows picked by `row_ids` (device int32) into out[count, cols]: the packed embedding
 * lookup (RowDequantSource.dequantRow, .../tensor/data/Q8_0TensorData.kt:91-100). */
SKAINET_HIP_API int32_t skainet_hip_dequantize_rows_dev(const skainet_hip_weight* w, const int32_t* row_ids, int32_t count, float* out);

/* ------------------------------------------------------------------------------------------------
 * Host-pointer entries with the reference's signatures.
 * ---------------------------------------------------------------------------------------------- */

/* NAT:57 skainet_q4k_matmul / NAT:80 skainet_q4k_matmul_rm (Q4KMatmulKernel.matmul, API/Q4KMatmulKernel.kt:54-59).
 * The plain name takes the SPI's input-block-major weight, `_rm` the canonical GGUF order. */
SKAINET_HIP_API void skainet_hip_q4k_matmul(const float* input, int32_t input_offset, const uint8_t* weight,
    int32_t weight_byte_offset, int32_t input_dim, int32_t output_dim, float* output, int32_t output_offset);
SKAINET_HIP_API void skainet_hip_q4k_matmul_rm(const float* input, int32_t input_offset, const uint8_t* weight,
    int32_t weight_byte_offset, int32_t input_dim, int32_t output_dim, float* output, int32_t output_offset);
/* NAT:135 / NAT:157 (Q6KMatmulKernel.matmul, API/Q6KMatmulKernel.kt:34). */
SKAINET_HIP_API void skainet_hip_q6k_matmul(const float* input, int32_t input_offset, const uint8_t* weight,
    int32_t weight_byte_offset, int32_t input_dim, int32_t output_dim, float* output, int32_t output_offset);
SKAINET_HIP_API void skainet_hip_q6k_matmul_rm(const float* input, int32_t input_offset, const uint8_t* weight,
    int32_t weight_byte_offset, int32_t input_dim, int32_t output_dim, float* output, int32_t output_offset);
/* NAT:327 / NAT:179 (Q8_0MatmulKernel.matmul, API/Q8_0MatmulKernel.kt:42). */
SKAINET_HIP_API void skainet_hip_q8_0_matmul(const float* input, int32_t input_offset, const uint8_t* weight,
    int32_t weight_byte_offset, int32_t input_dim, int32_t output_dim, float* output, int32_t output_offset);
SKAINET_HIP_API void skainet_hip_q8_0_matmul_rm(const float* input, int32_t input_offset, const uint8_t* weight,
    int32_t weight_byte_offset, int32_t input_dim, int32_t output_dim, float* output, int32_t output_offset);
/* The remaining packed formats of the provider SPI (API/KernelProvider.kt:74-104): NAT:353 skainet_q4_0_matmul / NAT:197
 * skainet_q4_0_matmul_rm (Q4_0MatmulKernel.matmul, API/Q4_0MatmulKernel.kt:40), NAT:381 / NAT:215 (Q5_0MatmulKernel.matmul,
 * API/Q5_0MatmulKernel.kt:37), NAT:409 / NAT:233 (Q5_1MatmulKernel.matmul, API/Q5_1MatmulKernel.kt:47), NAT:105 / NAT:251
 * (Q5KMatmulKernel.matmul, API/Q5KMatmulKernel.kt:53). Plain name: input-block-major weight, `_rm`: canonical order. */
SKAINET_HIP_API void skainet_hip_q4_0_matmul(const float* input, int32_t input_offset, const uint8_t* weight,
    int32_t weight_byte_offset, int32_t input_dim, int32_t output_dim, float* output, int32_t output_offset);
SKAINET_HIP_API void skainet_hip_q4_0_matmul_rm(const float* input, int32_t input_offset, const uint8_t* weight,
    int32_t weight_byte_offset, int32_t input_dim, int32_t output_dim, float* output, int32_t output_offset);
SKAINET_HIP_API void skainet_hip_q5_0_matmul(const float* input, int32_t input_offset, const uint8_t* weight,
    int32_t weight_byte_offset, int32_t input_dim, int32_t output_dim, float* output, int32_t output_offset);
SKAINET_HIP_API void skainet_hip_q5_0_matmul_rm(const float* input, int32_t input_offset, const uint8_t* weight,
    int32_t weight_byte_offset, int32_t input_dim, int32_t output_dim, float* output, int32_t output_offset);
SKAINET_HIP_API void skainet_hip_q5_1_matmul(const float* input, int32_t input_offset, const uint8_t* weight,
    int32_t weight_byte_offset, int32_t input_dim, int32_t output_dim, float* output, int32_t output_offset);
SKAINET_HIP_API void skainet_hip_q5_1_matmul_rm(const float* input, int32_t input_offset, const uint8_t* weight,
    int32_t weight_byte_offset, int32_t input_dim, int32_t output_dim, float* output, int32_t output_offset);
SKAINET_HIP_API void skainet_hip_q5k_matmul(const float* input, int32_t input_offset, const uint8_t* weight,
    int32_t weight_byte_offset, int32_t input_dim, int32_t output_dim, float* output, int32_t output_offset);
SKAINET_HIP_API void skainet_hip_q5k_matmul_rm(const float* input, int32_t input_offset, const uint8_t* weight,
    int32_t weight_byte_offset, int32_t input_dim, int32_t output_dim, float* output, int32_t output_offset);

/* NAT:290 skainet_bf16_matmul / NAT:307 skainet_fp16_matmul (Bf16MatmulKernel.matmul / Fp16MatmulKernel.matmul,
 * API/NarrowFloatMatmulKernel.kt:44-49): C(m,n) = A(m,k) B(k,n), A and C fp32 with float strides, B two bytes per element
 * (bf16 = the high half of an fp32; fp16 = IEEE binary16, little-endian) with BYTE offset and row stride; full overwrite,
 * k == 0 zeroes C. */
SKAINET_HIP_API void skainet_hip_bf16_matmul(const float* a, int32_t a_offset, int32_t a_stride, const uint8_t* b,
    int32_t b_byte_offset, int32_t b_byte_stride, float* c, int32_t c_offset, int32_t c_stride, int32_t m, int32_t n, int32_t k);
SKAINET_HIP_API void skainet_hip_fp16_matmul(const float* a, int32_t a_offset, int32_t a_stride, const uint8_t* b,
    int32_t b_byte_offset, int32_t b_byte_stride, float* c, int32_t c_offset, int32_t c_stride, int32_t m, int32_t n, int32_t k);

/* NAT:271 skainet_fp32_matmul (Fp32MatmulKernel.matmul, API/Fp32MatmulKernel.kt:25-50): C(m,n) = A(m,k) B(k,n),
 * strides in floats, full overwrite; k == 0 zeroes C. */
SKAINET_HIP_API void skainet_hip_fp32_matmul(const float* a, int32_t a_offset, int32_t a_stride,
    const float* b, int32_t b_offset, int32_t b_stride, float* c, int32_t c_offset, int32_t c_stride,
    int32_t m, int32_t n, int32_t k);
/* NAT:510 skainet_fp32_matmul_wt (Fp32MatmulWtKernel, API/Fp32MatmulWtKernel.kt:21-28): out[i,o] = sum_p in[i,p] w[o,p]. */
SKAINET_HIP_API void skainet_hip_fp32_matmul_wt(const float* in, int32_t in_offset, const float* w, int32_t w_offset,
    float* out, int32_t out_offset, int32_t m, int32_t n, int32_t k);

/* NAT:573 skainet_f32_rms_norm (Fp32NormKernel.rmsNorm, API/Fp32FusedKernels.kt:37-53); gamma may be NULL. */
SKAINET_HIP_API void skainet_hip_f32_rms_norm(const float* in, const float* gamma, float* out,
    int32_t rows, int32_t cols, float eps);
/* NAT:568 skainet_f32_layer_norm (Fp32NormKernel.layerNorm, API/Fp32FusedKernels.kt:37-53); gamma / beta may be NULL. */
SKAINET_HIP_API void skainet_hip_f32_layer_norm(const float* in, const float* gamma, const float* beta, float* out,
    int32_t rows, int32_t cols, float eps);
/* NAT:566 skainet_f32_softmax_rows (Fp32SoftmaxKernel, API/Fp32FusedKernels.kt:15-35). */
SKAINET_HIP_API void skainet_hip_f32_softmax_rows(const float* in, float* out, int32_t rows, int32_t cols, int32_t log_form);
/* NAT:577-584 skainet_f32_sdpa (Fp32AttentionKernel.sdpa, API/Fp32FusedKernels.kt:54-85). */
SKAINET_HIP_API void skainet_hip_f32_sdpa(const float* q, const float* k, const float* v, float* out,
    int32_t batch, int32_t heads, int32_t kv_heads, int32_t seq_q, int32_t seq_kv, int32_t head_dim,
    float scale, int32_t causal, int32_t window, int32_t right_context, const int32_t* lengths,
    const float* mask, int32_t mask_b, int32_t mask_h, int32_t mask_q, int32_t mask_k);

/* ------------------------------------------------------------------------------------------------
 * Device entries of the same kernels (all pointers on the device, asynchronous, 0 / -1).
 * ---------------------------------------------------------------------------------------------- */
SKAINET_HIP_API int32_t skainet_hip_fp32_matmul_dev(const float* a, int32_t a_offset, int32_t a_stride,
    const float* b, int32_t b_offset, int32_t b_stride, float* c, int32_t c_offset, int32_t c_stride,
    int32_t m, int32_t n, int32_t k);
SKAINET_HIP_API int32_t skainet_hip_fp32_matmul_wt_dev(const float* in, int32_t in_offset, const float* w, int32_t w_offset,
    float* out, int32_t out_offset, int32_t m, int32_t n, int32_t k);
SKAINET_HIP_API int32_t skainet_hip_f32_rms_norm_dev(const float* in, const float* gamma, float* out,
    int32_t rows, int32_t cols, float eps);
SKAINET_HIP_API int32_t skainet_hip_f32_layer_norm_dev(const float* in, const float* gamma, const float* beta, float* out,
    int32_t rows, int32_t cols, float eps);
SKAINET_HIP_API int32_t skainet_hip_f32_softmax_rows_dev(const float* in, float* out, int32_t rows, int32_t cols, int32_t log_form);
SKAINET_HIP_API int32_t skainet_hip_f32_sdpa_dev(const float* q, const float* k, const float* v, float* out,
    int32_t batch, int32_t heads, int32_t kv_heads, int32_t seq_q, int32_t seq_kv, int32_t head_dim,
    float scale, int32_t causal, int32_t window, int32_t right_context, const int32_t* lengths,
    const float* mask, int32_t mask_b, int32_t mask_h, int32_t mask_q, int32_t mask_k);
/* The same attention reading K / V in place from a cache laid out [batch, kv_heads, kv_capacity, head_dim] (the
 * per-layer layout KvCacheStore.readKeys / readValues return,
 * skainet-lang/skainet-lang-core/src/commonMain/kotlin/sk/ainet/lang/tensor/storage/KvCacheStore.kt:125-149): only the
 * first seq_kv rows of every head are keys, kv_capacity >= seq_kv is the row count of the storage. No additive mask. */
SKAINET_HIP_API int32_t skainet_hip_f32_sdpa_cache_dev(const float* q, const float* k_cache, const float* v_cache, float* out,
    int32_t batch, int32_t heads, int32_t kv_heads, int32_t seq_q, int32_t seq_kv, int32_t kv_capacity, int32_t head_dim,
    float scale, int32_t causal, int32_t window, int32_t right_context, const int32_t* lengths);
/* The same with the output laid out [batch, seq_q, heads, head_dim] -- token rows, which is what the output projection
 * multiplies -- so a prompt pass needs no transposing launch between attention and projection. No reference counterpart
 * (the reference's attention output is head-major, f32_fused.c:290-396; its callers transpose). */
SKAINET_HIP_API int32_t skainet_hip_f32_sdpa_cache_rows_dev(const float* q, const float* k_cache, const float* v_cache, float* out,
    int32_t batch, int32_t heads, int32_t kv_heads, int32_t seq_q, int32_t seq_kv, int32_t kv_capacity, int32_t head_dim,
    float scale, int32_t causal, int32_t window, int32_t right_context, const int32_t* lengths);
/* One decode token's attention over the KV cache and the output projection behind it:
 *   out[rows of wo] = (residual ? residual : 0) + Wo . sdpa(q [heads, head_dim], cache [kv_heads, kv_capacity, head_dim]),
 * causal over seq_kv keys (or lengths[0] of them when `lengths` is given: a device-side key count, so a recorded graph
 * follows the cache as it grows), `window` as in skainet_hip_f32_sdpa_dev. No reference counterpart as one call: the
 * parts are f32_fused.c:290-396 (attention), the packed product and a binary add. For a Q4_K projection of at most 4096
 * inputs and up to "attn_merge_splits" x "attn_merge_max_keys" keys (6 x 176) the attention kernel leaves its key splits unmerged and the projection
 * merges them while it loads its activations (two launches instead of four); other shapes run attention into
 * `attn_tmp` [heads * head_dim] and the fused product. `residual` may alias `out`. */
SKAINET_HIP_API int32_t skainet_hip_attn_out_proj_dev(const skainet_hip_weight* wo, const float* q, const float* k_cache,
                                                      const float* v_cache, int32_t heads, int32_t kv_heads, int32_t head_dim,
                                                      int32_t seq_kv, int32_t kv_capacity, float scale, int32_t window,
                                                      const int32_t* lengths, const float* residual, float* out, float* attn_tmp);

/* A gated MLP block in one call:
 *   out[m, rows of w_down] = (residual ? residual : 0) + Wdown . swiglu(Wgate_up . rmsnorm(x)),
 * x [m, cols of w_gate_up]; w_gate_up's rows are interleaved (gate_0, up_0, gate_1, up_1, ...), swiglu(g, u) =
 * g / (1 + exp(-g)) * u; gain == NULL: no norm; `residual` may alias `out`. No reference counterpart as one call: the
 * parts are the fused norm (f32_fused.c), two packed products and NAT:532-539's unary silu / binary mul / binary add.
 * Prompt shapes (m > 8, packed weights): the (gate, up) product is parked once as fp32 pairs in the library's scratch and
 * the pass that rounds the down projection's activations to bf16 takes the SwiGLU on the way (the activation is never
 * stored as fp32), the residual is added where the down projection stores its tiles. Other shapes: the two
 * skainet_hip_matmul_fused_dev calls in a row. Arithmetic class per row count as for skainet_hip_matmul_dev. */
SKAINET_HIP_API int32_t skainet_hip_mlp_swiglu_dev(const skainet_hip_weight* w_gate_up, const skainet_hip_weight* w_down,
                                                   const float* x, int32_t m, const float* gain, float eps,
                                                   const float* residual, float* out);

/* Decoder glue with the reference ops' semantics (device pointers):
 *   silu_mul: out[i] = gate[i] * (1 / (1 + exp(-gate[i]))) * up[i]   (NAT:532-539 unary op 2 then binary mul,
 *             REF/skainet-backend-native-cpu/native/src/f32_ops.c:222-244)
 *   add:      out[i] = a[i] + b[i]                                  (NAT:532 binary op 0)
 *   argmax:   index of the first maximum of each row, int32          (TensorOps.argMax ties -> lowest index,
 *             REF/../skainet-lang/skainet-lang-core/src/commonMain/kotlin/sk/ainet/lang/tensor/ops/TensorOps.kt:263-277) */
SKAINET_HIP_API int32_t skainet_hip_f32_silu_mul_dev(const float* gate, const float* up, float* out, int64_t n);
SKAINET_HIP_API int32_t skainet_hip_f32_add_dev(const float* a, const float* b, float* out, int64_t n);
/* Dense elementwise, activation and reduction kernels on device operands: the resident-activation set of
 * REF/skainet-backend-wasm-simd/src/wasmJsMain/kotlin/sk/ainet/exec/wasm/WasmCpuOps.kt:30-40 with the contracts of the CPU
 * library (NAT:515-546, REF/skainet-backend-native-cpu/native/src/f32_ops.c:130-330):
 *   binary: out[i] = a[ia] op b[ib]; op 0 add, 1 sub, 2 mul, 3 div; a_mode / b_mode 0 full (ia = i), 1 scalar (ia = 0),
 *           2 bias (ia = i % inner); inner <= 0 counts as 1;
 *   unary:  op 0 relu, 1 sigmoid, 2 silu, 3 gelu (tanh form), 4 gelu (erf form, evaluated in double), 5 erf, 6 tanh;
 *   reduce_all: *out = sum of in[0..n) (divided by n when mean != 0; n <= 0 gives 0);
 *   reduce_axis: out[o * inner + x] = sum over k < red of in[(o * red + k) * inner + x] (divided by red when mean != 0).
 * n <= 0 (outer or inner <= 0) is a no-op; unknown ops or modes return -1. */
SKAINET_HIP_API int32_t skainet_hip_f32_binary_dev(int32_t op, const float* a, int32_t a_mode, const float* b, int32_t b_mode,
    float* out, int64_t n, int32_t inner);
SKAINET_HIP_API int32_t skainet_hip_f32_unary_dev(int32_t op, const float* in, float* out, int64_t n);
SKAINET_HIP_API int32_t skainet_hip_f32_reduce_all_dev(const float* in, int64_t n, int32_t mean, float* out);
SKAINET_HIP_API int32_t skainet_hip_f32_reduce_axis_dev(const float* in, int32_t outer, int32_t red, int32_t inner, int32_t mean,
    float* out);
SKAINET_HIP_API int32_t skainet_hip_f32_argmax_rows_dev(const float* in, int32_t rows, int32_t cols, int32_t* out);
/* skainet_hip_f32_argmax_rows_dev for callers that cannot allocate device memory (code under HIP graph capture, tight
 * serving loops, harnesses that forbid it). No counterpart in the reference. Same result (first maximum of each row);
 * the partial pairs and arrival counters live in a fixed array inside the library's code object (8 slots of 33 KiB, 264
 * KiB per GPU) instead of scratch the library allocates, so the call makes no allocation of any kind. At most 64 rows
 * per call (more is refused with -1 and a message; cols is unbounded). A host thread is handed one slot on its first
 * call and keeps it until the process ends (the library's streams are per host thread, so threads do not share
 * counters); the ninth thread is refused with -1 and a message. Calls of ONE thread share its slot: issued on one stream
 * they are safe, overlapping on two streams they race. */
SKAINET_HIP_API int32_t skainet_hip_f32_argmax_rows_noalloc_dev(const float* in, int32_t rows, int32_t cols, int32_t* out);
/* The calling thread's slot of that array (handed out on first use), -1 when all are taken. Makes no device call. */
SKAINET_HIP_API int32_t skainet_hip_f32_argmax_rows_noalloc_slot(void);

/* Decoder glue the reference keeps in its external transformer repository (no counterpart in /root/reference; the
 * semantics are the standard Llama ones and are checked against closed forms):
 *   rope_scatter: token t, head h read at in + t*in_row_pitch + h*head_dim (a column slice of a token-major projection
 *                 output) -> out element (h, row0 + t, d) at h*out_head_stride + (row0+t)*head_dim + d,
 *                 row0 = *pos_dev when pos_dev != NULL else pos_start if out_row_is_pos, else 0; rotate != 0 rotates the
 *                 adjacent pairs (x[2i], x[2i+1]) by (pos + t) * theta^(-2i/head_dim), rotate == 0 copies (cache values).
 *                 Writes straight into the [kv_heads, positions, head_dim] layout KvCacheStore.readKeys/readValues expose
 *                 (REF/../skainet-lang/skainet-lang-core/src/commonMain/kotlin/sk/ainet/lang/tensor/storage/KvCacheStore.kt:125-149).
 *   heads_to_rows: [heads, tokens, head_dim] -> [tokens, heads*head_dim].
 *   swiglu_pairs:  interleaved (gate, up) pairs -> out[i] = silu(gu[2i]) * gu[2i+1] for i < n, silu as in silu_mul
 *                  (the output of one product against a weight whose rows alternate gate row, up row).
 *   rope_qkv:      the three rope_scatter calls of a decoder block in one launch: token rows [q | k | v] -> rotated
 *                  q [heads, tokens, head_dim], rotated k and raw v into rows pos + t of [kv_heads, kv_capacity, head_dim].
 *   i32_increment: *value += delta on the device (the position counter of a recorded decode step). */
SKAINET_HIP_API int32_t skainet_hip_f32_rope_scatter_dev(const float* in, int64_t in_row_pitch, float* out, int32_t tokens,
    int32_t heads, int32_t head_dim, int32_t pos_start, const int32_t* pos_dev, float theta, int32_t rotate,
    int64_t out_head_stride, int32_t out_row_is_pos);
SKAINET_HIP_API int32_t skainet_hip_f32_swiglu_pairs_dev(const float* gate_up, float* out, int64_t n);
SKAINET_HIP_API int32_t skainet_hip_f32_rope_qkv_dev(const float* qkv, float* q_out, float* k_cache, float* v_cache,
    int32_t tokens, int32_t heads, int32_t kv_heads, int32_t head_dim, int32_t kv_capacity, int32_t pos_start,
    const int32_t* pos_dev, float theta);
SKAINET_HIP_API int32_t skainet_hip_f32_heads_to_rows_dev(const float* in, float* out, int32_t heads, int32_t tokens, int32_t head_dim);
SKAINET_HIP_API int32_t skainet_hip_i32_increment_dev(int32_t* value, int32_t delta);
/* dst[index_dev[0] + offset] = src[0], all on the device: appends a sampled token to a log at the device-side position. */
/* End of a greedy decode step: *pos += 1, *kv_len += 1, log[*pos] = *token (all device memory, one launch). `capacity` is
 * the cache's row count (the log holds capacity + 1 entries): at *pos == capacity the call changes nothing, so a recorded
 * step replayed past the end of the cache writes nowhere (the K / V append of that step is skipped the same way) and the
 * host reads the saturated position. */
SKAINET_HIP_API int32_t skainet_hip_decode_advance_dev(int32_t* pos, int32_t* kv_len, const int32_t* token, int32_t* log,
    int32_t capacity);
SKAINET_HIP_API int32_t skainet_hip_i32_store_at_dev(int32_t* dst, const int32_t* index_dev, int32_t offset, const int32_t* src);

/* HIP graphs (no reference counterpart; for launch-bound loops such as a decode step): graph_begin redirects this
 * thread's device entries into a stream capture, graph_end closes it and returns an executable graph (NULL on
 * failure), graph_launch replays it on the calling thread's stream (in order with that thread's eager device
 * entries), graph_sync waits for that stream. Nothing that
 * allocates (a first call that grows the library's scratch) may run between begin and end: such a call fails with a
 * message instead of freeing memory under the capture, so run the sequence once eagerly first. A graph is tied to the
 * scratch addresses of its recording: when a later call on the thread makes the library reallocate scratch, the graph
 * is refused from then on (graph_valid / graph_launch). It is also tied to the thread that recorded it (scratch is per
 * thread): graph_valid is 0 and graph_launch fails on any other thread. Only kernel launches are recorded. */
typedef struct skainet_hip_graph skainet_hip_graph;
SKAINET_HIP_API int32_t skainet_hip_graph_begin(void);
SKAINET_HIP_API skainet_hip_graph* skainet_hip_graph_end(void);
SKAINET_HIP_API int32_t skainet_hip_graph_launch(skainet_hip_graph* graph);
/* 1 while the graph may still be launched from this thread, 0 once the thread's scratch has been reallocated since the
 * recording (a later call needed more, or skainet_hip_thread_release ran): graph_launch then returns -1 without
 * launching anything, and the sequence has to be recorded again. */
SKAINET_HIP_API int32_t skainet_hip_graph_valid(const skainet_hip_graph* graph);
SKAINET_HIP_API int32_t skainet_hip_graph_sync(skainet_hip_graph* graph);
SKAINET_HIP_API void skainet_hip_graph_free(skainet_hip_graph* graph);

/* Launch-shape knobs for experiments (defaults are the measured best). Keys: "upload_chunk_mib" (size of the
 * page-locked chunks skainet_hip_weight_upload stages pageable sources through, two per lane: 1 to 256 MiB, default 8;
 * 0 = one blocking copy straight from the caller's memory), "upload_lanes" (host threads that fill those chunks, each
 * with a stream of its own: 1 to 8, default 4), "gemv_waves_per_cu",
 * "q4k_rows_waves_per_cu" (resident waves per compute unit used to size the row shares, 0 = chosen from the shape),
 * "dense_mfma" (0: dense fp32 products stay on the vector-ALU tile kernel instead of the fp32 matrix instruction),
 * "gemv_stream_enable" (0: one-row Q8_0 / Q4_0 / Q5_0 / Q5_1 products stay on the row kernel instead of the one that
 * streams each wave's rows through LDS),
 * "q4k_rows_enable" (0: Q4_K decode shapes take the generic slot kernel), "q6k_slot64" (0: Q6_K at batch 1 keeps the
 * 32-weight slot of the batched kernel), "q4k_ksplit_enable" (0: long Q4_K rows are not
 * split over the waves of a workgroup), "q4k_mfma_enable" (0: one-row Q4_K products stay off the integer matrix-core
 * kernel and run the fp32 row-streaming one), "q4k_quads_stream_enable" (0: Q4_K products of 3 to 8 rows at K = 4096 stay on the
 * kernel that loads a lane's codes into registers instead of the one that streams the weight through an LDS ring),
 * "q4k_mfma_teams" (teams of four waves per workgroup of the one-row integer matrix-core kernel at K = 4096: 1, 2 = the
 * teams split the row quads and each wave prepares half of its slice's activations, 0 = two where a workgroup owns five
 * quads or more), "q4k_mfma_waves8" (0: the one-row integer matrix-core kernel keeps four waves per workgroup on rows of 8192 elements
 * and more instead of eight),
 * "q4k_mfma_window" (row quads the one-row integer matrix-core kernel keeps in flight per wave: 2 or 3,
 * 0 = chosen from K), "gemm_ksplit" (K splits of the MFMA GEMM,
 * 0 = automatic), "gemm_wide" (1 / 0: force the 256-column / 128-column tile, -1 = chosen from the shape), "gemm_rows" (2 / 4: 128 / 256
 * activation rows per tile, 0 = 128 up to 128 rows and 256 above), "gemm_ksw" (the Q4_K kernel that splits K over the
 * waves of a workgroup: 0 never, 1 where the launcher's estimate favours it, 2 wherever it fits), "gemm_ksw_teams" (teams
 * of four waves per workgroup of that kernel, each with its own share of K: 1 or 2, default 2; rows with an odd number
 * of 256-element super-blocks always run one team), "gemm_ksw_stages" (activation tiles the one-team form keeps in LDS: 3 to 7,
 * default 5), "gemm_frag" (the Q4_K kernel that reads its activations in matrix-fragment order: 0 never, 1 where the
 * launcher's estimate favours it, 2 wherever it fits), "gemm_frag_waves" (waves per workgroup of that kernel: 8 = one
 * workgroup per CU, 4 = two, 0 = eight for one round of tiles and four for more), "gemm_frag_gm" (row tiles per group of
 * its tile order, 0 = by the launcher's traffic estimate), "gemm_frag_touch" (0: the pass in front of it does not touch the
 * weight's lines), "gemm_frag_pieces" (64-element groups a workgroup of that pass takes: 1, 2 or 4),
 * "q4k_wide_enable" (0: Q4_K products of 5 to 8 rows at K = 4096 stay on the 4 x 4 x 4 matrix-instruction kernel instead of
 * the 16 x 16 x 32 one), "q4k_wide_min_batch" (fewest rows that kernel takes: 3 to 8, default 5), "q8_0_mfma_enable" (0:
 * one-row Q8_0 products stay off the integer matrix cores), "q8_0_mfma_per_cu" (workgroups per CU of that kernel: 1, 2
 * or 4, default 2),
 * "sdpa_prefill_mfma" (0: prompt-shape attention on the fp32 kernel), "sdpa_prefill_teams" (query groups per workgroup of
 * the matrix-core prompt kernel: 1, 2 = a late and an early group paired, 0 = paired where that still fills the chip), "sdpa_decode_split_keys" (least keys per split of
 * decode-shape attention, default 64), "sdpa_decode_gs" (query heads per workgroup of decode-shape attention: 1, 2 or 4, 0 = chosen from
 * the shape), "attn_merge_enable" (0: skainet_hip_attn_out_proj_dev always merges the key
 * splits in a launch of its own), "attn_merge_max_keys" (most keys per split for which that entry leaves the merge to
 * the projection, default 176), "attn_merge_splits" (most key splits it then uses, 1 to 8, default 6).
 * 0 when the key is known. No reference counterpart. */
SKAINET_HIP_API int32_t skainet_hip_set_tuning(const char* key, int32_t value);

#ifdef __cplusplus
}
#endif

#endif /* SKAINET_HIP_H */
