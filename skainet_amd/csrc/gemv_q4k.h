// Pieces of the Q4_K row-streaming GEMV kernel (gemv_q4k.hip) that its launcher and callers share: the raw bytes a
// lane holds per row, the 6-bit scale / min unpack, the epilogue selector.
#pragma once
#include "common.h"

namespace skh {

constexpr int Q4K_RMAX = 12;   // rows a wave can own per chunk (bounds the per-row accumulators)

struct Q4KRow { uint4 hdr, q0, q1; };

enum { EPI_NONE = 0, EPI_RESIDUAL = 1, EPI_SWIGLU = 2, EPI_ROPE_QKV = 3 };

// Destination of the RoPE epilogue: output rows are one token's [q | k | v] (heads, kv_heads, kv_heads heads of
// head_dim); q goes rotated to q_out [heads, head_dim] (the kernel's y), k rotated and v raw to row *pos_dev of caches
// laid out [kv_heads, capacity, head_dim].
struct RopeQkvEpilogue {
    float *k_cache, *v_cache;
    const int32_t* pos_dev;
    const float2* table;   // (cos, sin) of pos * theta^(-2i / head_dim), i < head_dim / 2, for the position in *pos_dev; or null
    float theta;
    int heads, kv_heads, head_dim, capacity;
};

// Activations handed over as the unmerged per-split results of a one-query attention: the consumer forms
//   x[h * head_dim + d] = sum_s c[h][s] * part[(h * splits + s) * head_dim + d],
//   c[h][s] = 2^(m[h][s] - max_s m) / sum_s 2^(m[h][s] - max_s m) * l[h][s]   (0 where that sum is 0),
// (m, l) = ml[(h * splits + s) * 2 ..]: the running maximum in units of ln 2 and the sum of a split's softmax weights.
constexpr int ATTN_MERGE_MAX_SPLITS = 8;
struct AttnMergePrologue { const float* part; const float* ml; int splits; int head_dim; };

// d * sc and dmin * m of the two sub-blocks (2g, 2g + 1) a lane owns. ggml get_scale_min_k4: both packings are
// evaluated and picked with a lane-constant mask (g < 2: bytes j and j + 4; g >= 2: the split 4 + 2 bit form).
__device__ __forceinline__ void q4k_lane_scales(const uint4& hdr, int sh, uint32_t hi_mask, float& dlo, float& dhi,
                                                float& mlo, float& mhi) {
    const float d = half_bits_to_float_fast(hdr.x & 0xFFFFu), dmin = half_bits_to_float_fast(hdr.x >> 16);
    const uint32_t u = hdr.y >> sh, v = hdr.z >> sh, t = hdr.w >> sh;
    const uint32_t sc = ((u & 0x3F3Fu) & ~hi_mask) | (((t & 0x0F0Fu) | ((u >> 2) & 0x3030u)) & hi_mask);
    const uint32_t mn = ((v & 0x3F3Fu) & ~hi_mask) | ((((t >> 4) & 0x0F0Fu) | ((v >> 2) & 0x3030u)) & hi_mask);
    dlo = d * ubyte0_to_float(sc); dhi = d * ubyte1_to_float(sc);
    mlo = dmin * ubyte0_to_float(mn); mhi = dmin * ubyte1_to_float(mn);
}

int q4k_rows_waves_per_cu();

}  // namespace skh
