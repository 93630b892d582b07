// Attention over a cache of latents on the matrix cores (bfloat16 cache rows, 32-bit softmax and accumulation);
// prompts and decode steps are the same kernel.  What is computed is said in attn_latent.hip.
//
// All heads read the same cache rows, so the (new token, head) pairs of a sequence, token-major, are the columns
// of one wide problem.  A workgroup of four waves owns 64 columns (16 a wave) and walks the keys 32 at a time; a
// block of 32 cache rows is staged once in LDS for the four waves, row-major for the scores and, its value part,
// transposed for the second product (a matrix operand wants eight consecutive keys of one value element):
//
//   S^T[32 keys x 16 cols] = K[32 x D] . Q^T[D x 16]            (A = cache rows, B = query columns, D in steps of 32)
//   online softmax over keys per column (32-bit; four lanes hold a column)
//   O^T[R x 16 cols]      += V^T[R x 32 keys] . P^T[32 x 16]     (A = transposed value part out of LDS)
//
// Key rows are assigned to the two 16-row score tiles so that a lane ends up with the eight consecutive keys
// 8 * (lane / 16) .. + 7, which is what the B operand of the second product wants (as in attn_mfma_impl.h).
//
// A decode step splits a long context over several workgroups (`split_size` keys each); each leaves an
// unnormalised partial result with its maximum and sum, and latent_combine_kernel merges them in split order.
#pragma once

#include "common.h"
#include "pta_kernels.h"

typedef __bf16 lat_bf16x8_t __attribute__((ext_vector_type(8)));
typedef float lat_f32x4_t __attribute__((ext_vector_type(4)));
typedef __bf16 lat_bf16x2_t __attribute__((ext_vector_type(2)));
typedef float lat_f32x2_t __attribute__((ext_vector_type(2)));

union LatFrag {
    uint4 u;
    lat_bf16x8_t v;
};

__device__ __forceinline__ uint32_t lat_pack(float lo, float hi) {
    union { lat_bf16x2_t b; uint32_t u; } c;
    c.b = __builtin_convertvector(lat_f32x2_t{lo, hi}, lat_bf16x2_t);
    return c.u;
}

#define LAT_KB 32            // keys per block
#define LAT_VP (LAT_KB + 8)  // row distance of the transposed value part in LDS (a multiple of 8 elements)

struct LatentArgs {
    float* out;         // [M, H, R], written when n_splits == 1
    float* po;          // [M, H, n_splits, R] partial results, else
    float* pm;          // [M, H, n_splits]
    float* pl;          // [M, H, n_splits]
    const float* q;     // [M, H, D]
    const bf16_t* k_pool;
    const int* block_table;
    int bt_stride;
    const int* cu_tokens;
    const int* seq_start;
    int H, R, D;
    float scale;
    int split_size, n_splits;
};

// DKC: 32-element pieces of a (padded) cache row; RT: 16-element tiles of the (padded) value part
template <int DKC, int RT>
__global__ __launch_bounds__(256) void attn_latent_mfma_kernel(const LatentArgs a) {
    extern __shared__ __attribute__((aligned(16))) bf16_t lat_lds[];
    constexpr int DP = DKC * 32 + 8;  // row distance of the staged block, in elements
    bf16_t* Ks = lat_lds;             // [LAT_KB][DP]
    bf16_t* Vt = lat_lds + LAT_KB * DP;  // [RT * 16][LAT_VP]
    const int s = blockIdx.z, split = blockIdx.y;
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, j = lane & 15, g = lane >> 4;
    const int t0 = a.cu_tokens[s], n_new = a.cu_tokens[s + 1] - t0, start = a.seq_start[s];
    const int H = a.H, R = a.R, D = a.D;
    const long rows_total = (long)n_new * H;
    const long row0 = (long)blockIdx.x * 64;
    if (row0 >= rows_total) return;
    // this wave's column of the lane
    const long rr = row0 + wave * 16 + j;
    const bool valid = rr < rows_total;
    const int tq = valid ? (int)(rr / H) : 0, head = valid ? (int)(rr % H) : 0;
    const int pos_q = start + tq;
    const long row_global = (long)(t0 + tq) * H + head;
    // keys this workgroup walks: its split's range, up to the position of its last column
    const int last_tq = (int)min((long)n_new - 1, (row0 + 63) / H);
    const int k_begin = split * a.split_size;
    const int k_end = min(start + last_tq + 1, a.n_splits > 1 ? k_begin + a.split_size : 0x7fffffff);
    const int wave_last = start + (int)min((long)n_new - 1, (row0 + wave * 16 + 15) / H);  // last position this wave sees

    // the wave's queries as B operands, scaled: column j, elements c * 32 + g * 8 .. + 7
    LatFrag qf[DKC];
#pragma unroll
    for (int c = 0; c < DKC; ++c) {
        float v[8];
        const int el0 = c * 32 + g * 8;
        if (valid && (D & 3) == 0 && el0 + 8 <= D) {  // sixteen-byte loads where a query's elements line up
            const float4 lo = *reinterpret_cast<const float4*>(a.q + row_global * D + el0);
            const float4 hi = *reinterpret_cast<const float4*>(a.q + row_global * D + el0 + 4);
            v[0] = lo.x * a.scale, v[1] = lo.y * a.scale, v[2] = lo.z * a.scale, v[3] = lo.w * a.scale;
            v[4] = hi.x * a.scale, v[5] = hi.y * a.scale, v[6] = hi.z * a.scale, v[7] = hi.w * a.scale;
        } else {
#pragma unroll
            for (int e = 0; e < 8; ++e) v[e] = (valid && el0 + e < D) ? a.q[row_global * D + el0 + e] * a.scale : 0.f;
        }
        qf[c].u = make_uint4(lat_pack(v[0], v[1]), lat_pack(v[2], v[3]), lat_pack(v[4], v[5]), lat_pack(v[6], v[7]));
    }
    lat_f32x4_t oacc[RT];
#pragma unroll
    for (int dt = 0; dt < RT; ++dt) oacc[dt] = lat_f32x4_t{0.f, 0.f, 0.f, 0.f};
    float m_run = -INFINITY, l_run = 0.f;
    const int* bt = a.block_table + (long)s * a.bt_stride;
    const bool wide_rows = (D % 8) == 0;

    // Staging: a thread owns one of the block's 32 rows (eight threads a row) and every eighth 16-byte piece of it,
    // so the page is looked up once and all of a block's loads are in flight together; the next block's loads are
    // issued before this block's arithmetic and land in LDS at the top of the next pass of the loop.
    constexpr int PIECES = (DKC * 4 + 7) / 8;  // pieces of a row per thread
    constexpr bool AHEAD = DKC <= 12;          // (the largest rows leave no registers for a block in flight)
    const int st_key = tid >> 3, st_ch = tid & 7;
    uint4 pre[PIECES];
    auto fetch = [&](int kb) {
        const int pos = kb + st_key;
        const bool live = pos < k_end;
        const bf16_t* src = nullptr;
        if (live) {
            const long page = bt[pos / PTA_PAGE];
            src = a.k_pool + (page * PTA_PAGE + pos % PTA_PAGE) * (long)D;
        }
#pragma unroll
        for (int i = 0; i < PIECES; ++i) {
            const int ch = st_ch + 8 * i;
            uint4 val = make_uint4(0u, 0u, 0u, 0u);
            if (live && ch * 8 < D) {
                if (wide_rows) {
                    val = *reinterpret_cast<const uint4*>(src + ch * 8);
                } else {
                    uint32_t w[4] = {0u, 0u, 0u, 0u};
#pragma unroll
                    for (int e = 0; e < 8; ++e)
                        if (ch * 8 + e < D) w[e >> 1] |= (uint32_t)src[ch * 8 + e] << ((e & 1) * 16);
                    val = make_uint4(w[0], w[1], w[2], w[3]);
                }
            }
            pre[i] = val;
        }
    };
    if (AHEAD && k_begin < k_end) fetch(k_begin);

    for (int kb = k_begin; kb < k_end; kb += LAT_KB) {
        __syncthreads();  // the last block's reads are done
        if (!AHEAD) fetch(kb);
        // 32 cache rows, padded with zeros to DKC * 32 elements (and past the range's end)
#pragma unroll
        for (int i = 0; i < PIECES; ++i) {
            const int ch = st_ch + 8 * i;
            if (ch < DKC * 4) *reinterpret_cast<uint4*>(Ks + st_key * DP + ch * 8) = pre[i];
        }
        if (AHEAD && kb + LAT_KB < k_end) fetch(kb + LAT_KB);
        __syncthreads();
        // the value part transposed: Vt[element][key]; elements past R are never read out of the result
        for (int idx = tid; idx < LAT_KB * RT * 2; idx += 256) {
            const int key = idx & (LAT_KB - 1), ch = idx / LAT_KB;
            const uint4 val = *reinterpret_cast<const uint4*>(Ks + key * DP + ch * 8);
            const uint32_t w[4] = {val.x, val.y, val.z, val.w};
#pragma unroll
            for (int e = 0; e < 8; ++e)
                Vt[(ch * 8 + e) * LAT_VP + key] = (bf16_t)((w[e >> 1] >> ((e & 1) * 16)) & 0xffffu);
        }
        __syncthreads();
        if (kb > wave_last || row0 + wave * 16 >= rows_total) continue;  // nothing here for this wave's columns (or it has none)

        // scores of 32 keys x 16 columns: tile tt's row i is key 8 * (i / 4) + 4 * tt + i % 4 of the block
        // (operands come out of LDS in batches ahead of the products that use them: a read that is waited for
        // in front of every product costs its whole latency each time)
        lat_f32x4_t sc[2];
        sc[0] = lat_f32x4_t{0.f, 0.f, 0.f, 0.f};
        sc[1] = lat_f32x4_t{0.f, 0.f, 0.f, 0.f};
        const bf16_t* krow0 = Ks + (8 * (j >> 2) + (j & 3)) * DP + g * 8;
        const bf16_t* krow1 = krow0 + 4 * DP;
#pragma unroll
        for (int c0 = 0; c0 < DKC; c0 += 4) {
            LatFrag kf[2][4];
#pragma unroll
            for (int i = 0; i < 4; ++i)
                if (c0 + i < DKC) {
                    kf[0][i].u = *reinterpret_cast<const uint4*>(krow0 + (c0 + i) * 32);
                    kf[1][i].u = *reinterpret_cast<const uint4*>(krow1 + (c0 + i) * 32);
                }
#pragma unroll
            for (int i = 0; i < 4; ++i)
                if (c0 + i < DKC) {
                    sc[0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[0][i].v, qf[c0 + i].v, sc[0], 0, 0, 0);
                    sc[1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[1][i].v, qf[c0 + i].v, sc[1], 0, 0, 0);
                }
        }
        // the lane holds column j, keys kb + 8 g + 4 tt + r
        float p[8];
        float m_blk = -INFINITY;
#pragma unroll
        for (int tt = 0; tt < 2; ++tt)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int key_pos = kb + 8 * g + 4 * tt + r;
                const bool see = valid && key_pos <= pos_q && key_pos < k_end;
                p[tt * 4 + r] = see ? sc[tt][r] : -INFINITY;
                m_blk = fmaxf(m_blk, p[tt * 4 + r]);
            }
        m_blk = fmaxf(m_blk, __shfl_xor(m_blk, 16, 64));
        m_blk = fmaxf(m_blk, __shfl_xor(m_blk, 32, 64));
        const float m_new = fmaxf(m_run, m_blk);
        const bool none = m_new == -INFINITY;  // the column has seen no key yet
        const float corr = none ? 1.f : expf(m_run - m_new);
        float l_blk = 0.f;
#pragma unroll
        for (int e = 0; e < 8; ++e) p[e] = none ? 0.f : expf(p[e] - m_new);
        LatFrag pf;
        pf.u = make_uint4(lat_pack(p[0], p[1]), lat_pack(p[2], p[3]), lat_pack(p[4], p[5]), lat_pack(p[6], p[7]));
        {   // the sum of the weights as they were rounded
            const uint32_t w[4] = {pf.u.x, pf.u.y, pf.u.z, pf.u.w};
#pragma unroll
            for (int e = 0; e < 4; ++e)
                l_blk += bf16_bits_to_f32((bf16_t)(w[e] & 0xffffu)) + bf16_bits_to_f32((bf16_t)(w[e] >> 16));
        }
        l_run = l_run * corr + l_blk;
        m_run = m_new;
        const bool rescale = __any(corr != 1.f);
        const bf16_t* vrow = Vt + j * LAT_VP + g * 8;
#pragma unroll
        for (int d0 = 0; d0 < RT; d0 += 8) {
            LatFrag vf[8];
#pragma unroll
            for (int i = 0; i < 8; ++i)
                if (d0 + i < RT) vf[i].u = *reinterpret_cast<const uint4*>(vrow + (d0 + i) * 16 * LAT_VP);
#pragma unroll
            for (int i = 0; i < 8; ++i)
                if (d0 + i < RT) {
                    if (rescale) {
#pragma unroll
                        for (int r = 0; r < 4; ++r) oacc[d0 + i][r] *= corr;
                    }
                    oacc[d0 + i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf[i].v, pf.v, oacc[d0 + i], 0, 0, 0);
                }
        }
    }
    float l_tot = l_run + __shfl_xor(l_run, 16, 64);
    l_tot += __shfl_xor(l_tot, 32, 64);
    if (!valid) return;
    // oacc[dt][r] is element dt * 16 + g * 4 + r of column j
    if (a.n_splits == 1) {
        const float inv = 1.0f / l_tot;
        float* orow = a.out + row_global * R;
#pragma unroll
        for (int dt = 0; dt < RT; ++dt)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int el = dt * 16 + g * 4 + r;
                if (el < R) orow[el] = oacc[dt][r] * inv;
            }
    } else {
        const long pr = row_global * a.n_splits + split;
        float* orow = a.po + pr * R;
#pragma unroll
        for (int dt = 0; dt < RT; ++dt)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int el = dt * 16 + g * 4 + r;
                if (el < R) orow[el] = oacc[dt][r];
            }
        if (g == 0) {
            a.pm[pr] = m_run;
            a.pl[pr] = l_tot;
        }
    }
}

template <int DKC, int RT>
static int launch_latent_mfma(const LatentArgs& a, int n_seqs, int max_rows, hipStream_t s) {
    constexpr int DP = DKC * 32 + 8;
    const size_t lds = (size_t)(LAT_KB * DP + RT * 16 * LAT_VP) * sizeof(bf16_t);
    auto kern = attn_latent_mfma_kernel<DKC, RT>;
    if (lds > 48 * 1024) {
        static bool raised = false;
        if (!raised) {
            if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)
                return pta_fail("attn_latent_mfma: %zu bytes of LDS were refused", lds);
            raised = true;
        }
    }
    const dim3 grid((max_rows + 63) / 64, a.n_splits, n_seqs), block(256);
    hipLaunchKernelGGL(kern, grid, block, lds, s, a);
    return pta_check_launch("attn_latent_mfma");
}

// the size classes, each group compiled in a translation unit of its own so that they build side by side
int latent_mfma_small(int dkc, int rt, const LatentArgs& a, int n_seqs, int max_rows, hipStream_t s);
int latent_mfma_mid(int dkc, int rt, const LatentArgs& a, int n_seqs, int max_rows, hipStream_t s);
int latent_mfma_large(int dkc, int rt, const LatentArgs& a, int n_seqs, int max_rows, hipStream_t s);
