// Heads of queries, keys and values on their way into attention, for mixers that norm them:
//
//   query / key head:  y = x / sqrt(mean(x^2) + eps) * w   (w: one weight [dk] for all heads; null: no norm),
//                      then the rotation by position (PtaRotation; null: none), queries out, keys into their page
//   value head:        y = x / sqrt(mean(x^2) + eps)        (no weight; or as it is), into its page
//
// Queries and keys have dk elements, values dv; the queries' frame and the pages hold heads of D >= max(dk, dv)
// elements, and the elements past a head's own are written as zeros, so that the attention kernels, which take one
// head size for keys and values, see scores and sums that the padding does not change.  One wave per (token, head);
// norms, angles, cosines and sines in 32-bit.
#include "common.h"
#include "pta_kernels.h"
#include "qkv_tail.h"

template <typename T>
__global__ __launch_bounds__(64) void head_norm_rope_cache_kernel(
    T* __restrict__ q_out, const T* __restrict__ q_in, const T* __restrict__ k_in, const T* __restrict__ v_in, long in_ld,
    const float* __restrict__ q_w, const float* __restrict__ k_w, float eps, int v_norm, PtaRotation rot,
    const int* __restrict__ token_pos, const int* __restrict__ token_seq, const int* __restrict__ block_table,
    int bt_stride, T* __restrict__ k_pool, T* __restrict__ v_pool, int nh, int nkv, int dk, int dv, int D, int write_cache) {
    __shared__ float y_s[256];
    const int m = blockIdx.x, unit = blockIdx.y, lane = threadIdx.x;
    const int kind = unit < nh ? 0 : unit < nh + nkv ? 1 : 2;
    const int head = kind == 0 ? unit : kind == 1 ? unit - nh : unit - nh - nkv;
    const int d = kind == 2 ? dv : dk;
    const T* src = (kind == 0 ? q_in : kind == 1 ? k_in : v_in) + (long)m * in_ld + (long)head * d;
    const float* w = kind == 0 ? q_w : kind == 1 ? k_w : nullptr;
    const bool normed = kind == 2 ? v_norm != 0 : w != nullptr;
    const int pos = token_pos[m];
    float x[4], ss = 0.f;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        const int i = lane + r * PTA_WAVE;
        x[r] = i < d ? Io<T>::ld(src + i) : 0.f;
        ss += x[r] * x[r];
    }
    const float inv = normed ? rsqrtf(wave_sum(ss) / (float)d + eps) : 1.f;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        const int i = lane + r * PTA_WAVE;
        if (i < d) x[r] = x[r] * inv * (w ? w[i] : 1.f);
        y_s[i] = i < d ? x[r] : 0.f;
    }
    __syncthreads();
    const int R = (kind != 2 && rot.inv_freq) ? rot.rotary_dim : 0, half = R >> 1;
    const float* freq = R ? rot.inv_freq + (rot.inv_freq_ld ? (long)token_seq[m] * rot.inv_freq_ld : 0L) : nullptr;
    long page = 0;
    if (kind != 0) page = block_table[(long)token_seq[m] * bt_stride + pos / PTA_PAGE];
    const int in_page = pos % PTA_PAGE;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        const int i = lane + r * PTA_WAVE;
        if (i >= D) continue;
        float y = i < d ? x[r] : 0.f;
        if (i < R) {
            int p, other;  // the pair's index, and the element this one is rotated with
            float sign;    // -1 for the pair's first element, +1 for its second
            if (rot.pairing == PTA_PAIR_INTERLEAVED) { p = i >> 1; other = i ^ 1; sign = (i & 1) ? 1.f : -1.f; }
            else { p = i < half ? i : i - half; other = i < half ? i + half : i - half; sign = i < half ? -1.f : 1.f; }
            const float ang = (float)pos * freq[p];
            y = y * (cosf(ang) * rot.cs_scale) + sign * y_s[other] * (sinf(ang) * rot.cs_scale);
        }
        if (kind == 0) Io<T>::st(q_out + ((long)m * nh + head) * D + i, y);
        else if (kind == 1) Io<T>::st(k_pool + ((page * nkv + head) * PTA_PAGE + in_page) * (long)D + i, y);
        else Io<T>::st(v_pool + ((page * nkv + head) * (long)D + i) * PTA_PAGE + in_page, y);
    }
}

// q_out [M, nh, D]; q_in, k_in, v_in: rows in_ld apart holding nh * dk, nkv * dk and nkv * dv elements; pools of head
// size D.  With write_cache = 0 only the queries are made.
extern "C" int pta_head_norm_rope_cache(void* q_out, const void* q_in, const void* k_in, const void* v_in, long in_ld,
                                        const float* q_w, const float* k_w, float eps, int v_norm,
                                        const PtaRotation* rotation, const int* token_pos, const int* token_seq,
                                        const int* block_table, int bt_stride, void* k_pool, void* v_pool, int M, int nh,
                                        int nkv, int dk, int dv, int D, int write_cache, int dtype, void* stream) {
    PTA_REQUIRE(M > 0 && nh > 0 && nkv > 0 && dk > 0 && dv > 0, "head_norm_rope_cache: sizes must be positive");
    PTA_REQUIRE(nh % nkv == 0, "head_norm_rope_cache: heads (%d) must be a multiple of kv heads (%d)", nh, nkv);
    PTA_REQUIRE(D >= dk && D >= dv && D <= 256, "head_norm_rope_cache: a frame of %d elements must hold heads of %d and %d and be at most 256", D, dk, dv);
    PTA_REQUIRE(nh + 2 * nkv <= 65535, "head_norm_rope_cache: too many heads for one launch");
    PTA_REQUIRE(q_out && q_in && token_pos && token_seq, "head_norm_rope_cache: null pointer");
    PTA_REQUIRE(!write_cache || (k_in && v_in && k_pool && v_pool && block_table), "head_norm_rope_cache: null cache pointer");
    const PtaRotation rot = pta_rotation_of(rotation);
    if (pta_check_rotation("head_norm_rope_cache", rot, dk, token_seq)) return 1;
    PTA_REQUIRE(dtype == PTA_F32 || dtype == PTA_BF16, "head_norm_rope_cache: unknown dtype %d", dtype);
    hipStream_t s = (hipStream_t)stream;
    const dim3 grid(M, write_cache ? nh + 2 * nkv : nh);
    if (dtype == PTA_F32)
        hipLaunchKernelGGL(head_norm_rope_cache_kernel<float>, grid, dim3(64), 0, s, (float*)q_out, (const float*)q_in,
                           (const float*)k_in, (const float*)v_in, in_ld, q_w, k_w, eps, v_norm, rot, token_pos, token_seq,
                           block_table, bt_stride, (float*)k_pool, (float*)v_pool, nh, nkv, dk, dv, D, write_cache);
    else
        hipLaunchKernelGGL(head_norm_rope_cache_kernel<bf16_t>, grid, dim3(64), 0, s, (bf16_t*)q_out, (const bf16_t*)q_in,
                           (const bf16_t*)k_in, (const bf16_t*)v_in, in_ld, q_w, k_w, eps, v_norm, rot, token_pos,
                           token_seq, block_table, bt_stride, (bf16_t*)k_pool, (bf16_t*)v_pool, nh, nkv, dk, dv, D, write_cache);
    return pta_check_launch("head_norm_rope_cache");
}
