// Decode-time dequant-GEMV for GGUF Q4_K / Q6_K / Q8_0 weights in canonical row-major block order:
//   y[b, o] = sum_j x[b, j] * dequant(W[o, j])     b < batch <= 4 per launch, fp32 activations and sums.
//
// Semantics follow the reference's exact-fp32 kernels (same products, different summation order):
//   /root/reference/skainet-backends/skainet-backend-cpu/src/commonMain/kotlin/sk/ainet/exec/kernel/
//   ScalarQ4_KMatmulKernel.kt:40-78, ScalarQ6_KMatmulKernel.kt:33-44, ScalarQ8_0MatmulKernel.kt:41-62
// and the row-major weight addressing of the native entries
//   /root/reference/skainet-backends/skainet-backend-native-cpu/native/src/q4k_matmul.c:294-309.
//
// Mapping (HBM-bound, one pass over the weight, nothing staged in LDS):
//   * A weight row is cut into "slots" of SLOT_ELEMS consecutive-in-memory quants (Q4_K: one 16-byte
//     nibble chunk = 16 + 16 elements of two sub-blocks; Q6_K: 4 x 4 elements sharing 12 code bytes;
//     Q8_0: one 34-byte block). Lane l of wave s in a workgroup owns slot s * 64 + l of EVERY row the
//     workgroup processes, so the activation slice that slot needs lives in registers for the whole
//     kernel and each wave-wide load instruction covers one contiguous span of the row.
//   * Rows are streamed R at a time with all loads issued before the arithmetic; the R * B per-lane
//     partial sums are folded across the wave with a multi-value butterfly (log2(R*B) halving steps,
//     then plain xor-shuffles), written to LDS per (wave, row) and summed over the waves in a fixed
//     order, so results are deterministic.
//   * Grid: contiguous row ranges, sized so the whole chip gets an even share (rows_per_wg from the host).
#include "gemv_slots.h"
#include <type_traits>

#include <cstring>

namespace skh {

constexpr int GEMV_MAX_WAVES = 8;    // waves per workgroup = K segments processed concurrently (2 per SIMD: 256 VGPRs each)
constexpr int GEMV_MAX_ROWS = 64;    // rows per workgroup (bounds the LDS partial-sum buffer)

// F: slot policy, B: activation rows per launch (1, 2 or 4; unused ones are zero), R: weight rows in flight.
template <class F, int B, int R>
__global__ __launch_bounds__(64 * GEMV_MAX_WAVES) void gemv_kernel(
    const uint8_t* __restrict__ w, const float* __restrict__ x, float* __restrict__ y,
    int k, int n, int batch, int64_t row_bytes, int rows_per_wg) {
    constexpr int NX = F::NX, NS = XSumCount<F>::N;
    constexpr int NV = (R * B <= 2) ? 2 : (R * B <= 4) ? 4 : (R * B <= 8) ? 8 : 16;   // fold width: the next power of two, zero padded
    static_assert(R * B <= 16, "at most 16 values per fold");
    __shared__ float partial[GEMV_MAX_WAVES][GEMV_MAX_ROWS][B];

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nwaves = blockDim.x >> 6;
    const int nslots = k / F::SLOT_ELEMS;
    const int nseg = (nslots + 63) >> 6;
    const int r0 = blockIdx.x * rows_per_wg;
    const int r1 = min(n, r0 + rows_per_wg);
    const int nrows = r1 - r0;
    if (nrows <= 0) return;
    const uint8_t* wbase = w + (int64_t)r0 * row_bytes;
    const int my_value = wave_fold_index<NV>(lane);

    for (int seg = wave, pass = 0; seg < nseg; seg += nwaves, ++pass) {
        const int slot = seg * 64 + lane;
        const bool active = slot < nslots;
        typename F::Lane ln;
        F::init(ln, active ? slot : 0);

        // The activation slice is requested first and unconditionally (clamped address, zeroed afterwards), the first
        // R rows of weights right behind it: loads return in issue order, so the L2-resident activations must not
        // queue behind the weight stream, and a branch around a load would make the wave wait for every load in flight.
        float xs[B][NX], xsum[B][NS];
        const int xslot = active ? slot : 0;
#pragma unroll
        for (int b = 0; b < B; ++b) {
            const float* xb = x + (int64_t)(b < batch ? b : 0) * k;
#pragma unroll
            for (int i = 0; i < NX; i += 4) {
                const float4 v = *reinterpret_cast<const float4*>(xb + F::x_index(xslot, i));
                xs[b][i] = v.x; xs[b][i + 1] = v.y; xs[b][i + 2] = v.z; xs[b][i + 3] = v.w;
            }
        }
        __builtin_amdgcn_sched_barrier(0);
        typename F::Raw raw[R];
#pragma unroll
        for (int i = 0; i < R; ++i) F::load(raw[i], wbase + (int64_t)min(i, nrows - 1) * row_bytes, ln);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int b = 0; b < B; ++b) {
            const float keep = (active && b < batch) ? 1.0f : 0.0f;
#pragma unroll
            for (int i = 0; i < NX; ++i) xs[b][i] *= keep;
            F::prep(xs[b], xsum[b]);
        }

        for (int r = 0; r < nrows; r += R) {
            float acc[NV];
#pragma unroll
            for (int i = R * B; i < NV; ++i) acc[i] = 0.f;
#pragma unroll
            for (int i = 0; i < R; ++i) {
                float a[B];
#pragma unroll
                for (int b = 0; b < B; ++b) a[b] = 0.f;
                if (r + i < nrows) F::template dot<B>(raw[i], ln, xs, xsum, a);   // wave-uniform: no arithmetic on padding rows
#pragma unroll
                for (int b = 0; b < B; ++b) acc[i * B + b] = active ? a[b] : 0.f;
                // refill this register set with the row R ahead (clamped: a repeated last row is discarded)
                F::load(raw[i], wbase + (int64_t)min(r + R + i, nrows - 1) * row_bytes, ln);
            }
            wave_fold<NV>(acc, lane);
            if (lane < NV) {
                const int i = my_value / B, b = my_value % B;
                if (i < R && r + i < nrows) {
                    float* dst = &partial[wave][r + i][b];
                    *dst = pass == 0 ? acc[0] : *dst + acc[0];
                }
            }
        }
    }
    __syncthreads();
    const int used_waves = min(nwaves, nseg);
    for (int t = threadIdx.x; t < nrows * B; t += blockDim.x) {
        const int rr = t / B, b = t % B;
        if (b >= batch) continue;
        float s = 0.f;
        for (int wv = 0; wv < used_waves; ++wv) s += partial[wv][rr][b];
        y[(int64_t)b * n + r0 + rr] = s;
    }
}

template <class F, int B, int R>
static int launch_one(const uint8_t* w, const float* x, float* y, int k, int n, int batch, int waves_per_cu) {
    const int nslots = k / F::SLOT_ELEMS;
    const int nseg = (nslots + 63) / 64;
    const int nwaves = nseg < GEMV_MAX_WAVES ? nseg : GEMV_MAX_WAVES;
    const int64_t row_bytes = (int64_t)(k / (F::SLOT_ELEMS * F::SLOTS_PER_BLOCK)) * F::BLOCK_BYTES;
    // Even contiguous row shares: about waves_per_cu resident waves on every CU.
    int target_wgs = (num_cus() * waves_per_cu) / nwaves;
    if (target_wgs < 1) target_wgs = 1;
    int rows_per_wg = (n + target_wgs - 1) / target_wgs;
    if (rows_per_wg < 1) rows_per_wg = 1;
    if (rows_per_wg > GEMV_MAX_ROWS) rows_per_wg = GEMV_MAX_ROWS;
    const int grid = (n + rows_per_wg - 1) / rows_per_wg;
    note_kernel("gemv_kernel");
    gemv_kernel<F, B, R><<<dim3(grid), dim3(64 * nwaves), 0, current_stream()>>>(w, x, y, k, n, batch, row_bytes, rows_per_wg);
    SKH_CHECK(hipGetLastError());
    return 0;
}

// Weight rows a wave keeps in flight at batch 1, per format (measured over 2 .. 8 on the 11008 x 4096, 32000 x 4096 and
// 4096 x 4096 shapes: the formats with many loads per row are faster with fewer rows requested at once).
template <class F> struct RowsInFlight { static constexpr int B1 = 8; };
template <> struct RowsInFlight<Q80Slot> { static constexpr int B1 = 3; };
template <> struct RowsInFlight<Q6KSlot> { static constexpr int B1 = 2; };
template <> struct RowsInFlight<Q5KSlot> { static constexpr int B1 = 3; };

static std::atomic<int> g_gemv_waves_per_cu{0};   // 0: per encoding (measured best: Q8_0 4, Q6_K at batch 1 6, the others 8)
static std::atomic<int> g_q6k_slot64{1};   // 0: Q6_K at batch 1 stays on the 32-weight slot

template <class F>
static int launch_format(const uint8_t* w, const float* x, float* y, int k, int n, int batch, int waves_per_cu) {
    if (batch == 1) {
        // Q6_K: the 64-weight slot, 2 rows in flight, 6 waves per CU unless the caller set a count (measured on 32000 x 4096
        // over 1 .. 4 rows and 5 .. 16 waves: 23.1 us against 25.5 us for the 32-weight slot at its best, 2 rows and 8 waves)
        if (std::is_same<F, Q6KSlot>::value && g_q6k_slot64)
            return launch_one<Q6KSlot64, 1, 2>(w, x, y, k, n, batch, g_gemv_waves_per_cu.load() > 0 ? g_gemv_waves_per_cu.load() : 6);
        return launch_one<F, 1, RowsInFlight<F>::B1>(w, x, y, k, n, batch, waves_per_cu);
    }
    if (batch == 2) return launch_one<F, 2, 4>(w, x, y, k, n, batch, waves_per_cu);
    return launch_one<F, 4, 2>(w, x, y, k, n, batch, waves_per_cu);
}

static std::atomic<int> g_q4k_rows_enable{1};
void set_q4k_rows_waves_per_cu(int v);
void set_gemm_wide(int v);
void set_gemm_ksplit(int v);
void set_gemm_rows(int v);
void set_gemm_ksw(int v);
void set_gemm_ksw_teams(int v);
void set_gemm_ksw_stages(int v);
void set_gemm_frag(int v);
void set_gemm_frag_touch(int v);
void set_gemm_frag_pieces(int v);
void set_gemm_frag_waves(int v);
void set_gemm_frag_gm(int v);
void set_sdpa_prefill_mfma(int v);
void set_sdpa_prefill_teams(int v);
void set_sdpa_decode_split_keys(int v);
void set_q4k_ksplit_enable(int v);
void set_q4k_mfma_enable(int v);
void set_q4k_mfma_window(int v);
void set_q4k_mfma_teams(int v);
void set_q4k_mfma_waves8(int v);
void set_q4k_quads_stream_enable(int v);
void set_q4k_wide_enable(int v);
void set_q4k_wide_min_batch(int v);
void set_attn_merge_enable(int v);
void set_sdpa_decode_gs(int v);
void set_attn_merge_max_keys(int v);
void set_attn_merge_splits(int v);
int launch_q4k_gemv_rows(const uint8_t* w, const float* x, float* y, int k, int n, int batch);   // gemv_q4k.hip
int launch_q4k_gemv_quads(const uint8_t* w, const float* x, float* y, int k, int n, int batch);  // gemv_q4k_quads.hip
int launch_gemv_stream(int enc, const uint8_t* w, const float* x, float* y, int k, int n);        // gemv_stream.hip
void set_gemv_stream_enable(int v);
int launch_q8_0_gemv_mfma(const uint8_t* w, const float* x, float* y, int k, int n);                  // gemv_q8_0_mfma.hip
void set_q8_0_mfma_enable(int v);
void set_q8_0_mfma_per_cu(int v);
void set_dense_mfma(int v);

// Experiment knobs (defaults are the measured best): returns 0 when the key is known.
int set_tuning(const char* key, int value) {
    if (!strcmp(key, "gemv_waves_per_cu")) { if (value >= 0) g_gemv_waves_per_cu = value; return 0; }
    if (!strcmp(key, "q4k_rows_waves_per_cu")) { set_q4k_rows_waves_per_cu(value); return 0; }
    if (!strcmp(key, "q6k_slot64")) { g_q6k_slot64 = value != 0; return 0; }
    if (!strcmp(key, "gemv_stream_enable")) { set_gemv_stream_enable(value); return 0; }
    if (!strcmp(key, "q8_0_mfma_enable")) { set_q8_0_mfma_enable(value); return 0; }
    if (!strcmp(key, "q8_0_mfma_per_cu")) { set_q8_0_mfma_per_cu(value); return 0; }
    if (!strcmp(key, "dense_mfma")) { set_dense_mfma(value); return 0; }
    if (!strcmp(key, "gemm_wide")) { set_gemm_wide(value); return 0; }
    if (!strcmp(key, "q4k_rows_enable")) { g_q4k_rows_enable = value; return 0; }
    if (!strcmp(key, "gemm_ksplit")) { set_gemm_ksplit(value); return 0; }
    if (!strcmp(key, "gemm_rows")) { set_gemm_rows(value); return 0; }
    if (!strcmp(key, "gemm_ksw")) { set_gemm_ksw(value); return 0; }
    if (!strcmp(key, "gemm_ksw_teams")) { set_gemm_ksw_teams(value); return 0; }
    if (!strcmp(key, "gemm_ksw_stages")) { set_gemm_ksw_stages(value); return 0; }
    if (!strcmp(key, "gemm_frag")) { set_gemm_frag(value); return 0; }
    if (!strcmp(key, "gemm_frag_touch")) { set_gemm_frag_touch(value); return 0; }
    if (!strcmp(key, "gemm_frag_pieces")) { set_gemm_frag_pieces(value); return 0; }
    if (!strcmp(key, "gemm_frag_waves")) { set_gemm_frag_waves(value); return 0; }
    if (!strcmp(key, "gemm_frag_gm")) { set_gemm_frag_gm(value); return 0; }
    if (!strcmp(key, "sdpa_prefill_mfma")) { set_sdpa_prefill_mfma(value); return 0; }
    if (!strcmp(key, "sdpa_prefill_teams")) { set_sdpa_prefill_teams(value); return 0; }
    if (!strcmp(key, "q4k_ksplit_enable")) { set_q4k_ksplit_enable(value); return 0; }
    if (!strcmp(key, "q4k_mfma_enable")) { set_q4k_mfma_enable(value); return 0; }
    if (!strcmp(key, "q4k_quads_stream_enable")) { set_q4k_quads_stream_enable(value); return 0; }
    if (!strcmp(key, "q4k_wide_enable")) { set_q4k_wide_enable(value); return 0; }
    if (!strcmp(key, "q4k_wide_min_batch")) { set_q4k_wide_min_batch(value); return 0; }
    if (!strcmp(key, "q4k_mfma_waves8")) { set_q4k_mfma_waves8(value); return 0; }
    if (!strcmp(key, "q4k_mfma_teams")) { set_q4k_mfma_teams(value); return 0; }
    if (!strcmp(key, "q4k_mfma_window")) { set_q4k_mfma_window(value); return 0; }
    if (!strcmp(key, "sdpa_decode_split_keys")) { set_sdpa_decode_split_keys(value); return 0; }
    if (!strcmp(key, "attn_merge_enable")) { set_attn_merge_enable(value); return 0; }
    if (!strcmp(key, "sdpa_decode_gs")) { set_sdpa_decode_gs(value); return 0; }
    if (!strcmp(key, "attn_merge_max_keys")) { set_attn_merge_max_keys(value); return 0; }
    if (!strcmp(key, "attn_merge_splits")) { set_attn_merge_splits(value); return 0; }
    return -1;
}

// y[m, n] = x[m, k] . W^T for m activation rows, at most 4 per pass over the weight.
int launch_gemv(int enc, const uint8_t* w, const float* x, int m, int k, int n, float* y) {
    if (m <= 0 || n <= 0) return 0;
    if (!is_packed(enc)) return set_error("gemv: unsupported encoding %d", enc);
    if (k <= 0 || k % block_elems(enc) != 0)
        return set_error("gemv: inputDim must be a positive multiple of %d; got %d", block_elems(enc), k);
    const int waves_per_cu = g_gemv_waves_per_cu.load() > 0 ? g_gemv_waves_per_cu.load() : (block_elems(enc) == 32 ? 4 : 8);
    for (int b0 = 0; b0 < m;) {
        const int left = m - b0;
        const float* xb = x + (int64_t)b0 * k;
        float* yb = y + (int64_t)b0 * n;
        int rc;
        if (enc == ENC_Q4_K && g_q4k_rows_enable) {
            // 3 to 8 rows: the fp32 matrix-instruction kernel; 1 or 2: the row-streaming kernel
            const int nq = left < 8 ? left : 8;
            rc = left >= 3 ? launch_q4k_gemv_quads(w, xb, yb, k, n, nq) : launch_q4k_gemv_rows(w, xb, yb, k, n, left);
            if (rc < 0) return rc;
            if (rc == 1) { b0 += left >= 3 ? nq : left; continue; }
        }
        if (left == 1 && enc == ENC_Q8_0) {
            // one row of Q8_0, K a multiple of 1024 up to 4096: the codes straight onto the integer matrix cores
            rc = launch_q8_0_gemv_mfma(w, xb, yb, k, n);
            if (rc < 0) return rc;
            if (rc == 1) { b0 += 1; continue; }
        }
        if (left == 1 && enc != ENC_Q4_K) {
            // one row: the weight streamed through LDS in consecutive kilobytes, where the row shape allows it
            rc = launch_gemv_stream(enc, w, xb, yb, k, n);
            if (rc < 0) return rc;
            if (rc == 1) { b0 += 1; continue; }
        }
        const int nb = left < 4 ? left : 4;
        if (enc == ENC_Q4_K) rc = launch_format<Q4KSlot>(w, xb, yb, k, n, nb, waves_per_cu);
        else if (enc == ENC_Q6_K) rc = launch_format<Q6KSlot>(w, xb, yb, k, n, nb, waves_per_cu);
        else if (enc == ENC_Q5_K) rc = launch_format<Q5KSlot>(w, xb, yb, k, n, nb, waves_per_cu);
        else if (enc == ENC_Q4_0) rc = launch_format<Q45Slot<0>>(w, xb, yb, k, n, nb, waves_per_cu);
        else if (enc == ENC_Q5_0) rc = launch_format<Q45Slot<1>>(w, xb, yb, k, n, nb, waves_per_cu);
        else if (enc == ENC_Q5_1) rc = launch_format<Q45Slot<2>>(w, xb, yb, k, n, nb, waves_per_cu);
        else rc = launch_format<Q80Slot>(w, xb, yb, k, n, nb, waves_per_cu);
        if (rc != 0) return rc;
        b0 += nb;
    }
    return 0;
}

}  // namespace skh
