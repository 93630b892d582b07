// Layers that carry a state of fixed size from token to token instead of keys and values.  A sequence's state is
// a row of a 32-bit table, found through the step's `seq_slot`; a step's tokens of sequence s are rows
// cu_tokens[s] .. cu_tokens[s + 1] - 1 of its activations.  A launch reads the state, walks the sequence's
// tokens in order and leaves the state of the last one, so cutting a sequence into steps changes nothing
// but the places of roundings.  Gates, decays, step sizes and states are 32-bit whatever the compute type.
#include "common.h"
#include "pta_kernels.h"

__device__ __forceinline__ float sigmoid_f(float x) { return 1.0f / (1.0f + expf(-x)); }
__device__ __forceinline__ float softplus_f(float x) { return x > 20.f ? x : log1pf(expf(x)); }

// ---- a gated recurrence whose gate and candidate read the current token only ------------------------------
// zxg[t] = [gate pre-activation | candidate pre-activation | output gate], W each.
// z = sigmoid(zxg_z + bz); u = zxg_x + bx; c = u + 1/2 where u >= 0, sigmoid(u) below; S = (1 - z) S + z c;
// y = S * silu(zxg_g).  One thread per (sequence, channel); the loads of UNROLL tokens are in flight together.
template <typename T, int UNROLL>
__global__ void gated_scan_kernel(T* __restrict__ y, const T* __restrict__ zxg, long ld, const float* __restrict__ bz,
                                  const float* __restrict__ bx, float* __restrict__ state, long state_ld,
                                  const int* __restrict__ cu_tokens, const int* __restrict__ seq_slot, int W) {
    const int c = blockIdx.x * blockDim.x + threadIdx.x, s = blockIdx.y;
    if (c >= W) return;
    const int t0 = cu_tokens[s], t1 = cu_tokens[s + 1];
    float* sp = state + (long)seq_slot[s] * state_ld + c;
    float S = *sp;
    const float b_z = bz ? bz[c] : 0.f, b_x = bx ? bx[c] : 0.f;
    for (int t = t0; t < t1; t += UNROLL) {
        float zr[UNROLL], ur[UNROLL], gr[UNROLL];
#pragma unroll
        for (int i = 0; i < UNROLL; ++i) {
            const long row = (long)min(t + i, t1 - 1) * ld + c;
            zr[i] = Io<T>::ld(zxg + row);
            ur[i] = Io<T>::ld(zxg + row + W);
            gr[i] = Io<T>::ld(zxg + row + 2 * W);
        }
#pragma unroll
        for (int i = 0; i < UNROLL; ++i) {
            if (t + i < t1) {
                const float z = sigmoid_f(zr[i] + b_z);
                const float u = ur[i] + b_x;
                const float cand = u >= 0.f ? u + 0.5f : sigmoid_f(u);
                S = (1.0f - z) * S + z * cand;
                const float g = gr[i];
                Io<T>::st(y + (long)(t + i) * W + c, S * (g / (1.0f + expf(-g))));
            }
        }
    }
    *sp = S;
}

extern "C" int pta_gated_scan(void* y, const void* zxg, long ld, const float* bz, const float* bx, float* state,
                              long state_ld, const int* cu_tokens, const int* seq_slot, int n_seqs, int W, int dtype,
                              void* stream) {
    PTA_REQUIRE(n_seqs > 0 && W > 0, "gated_scan: sequences=%d width=%d must be positive", n_seqs, W);
    PTA_REQUIRE(y && zxg && state && cu_tokens && seq_slot, "gated_scan: null pointer");
    PTA_REQUIRE(ld >= 3L * W && state_ld >= W, "gated_scan: rows lie closer together than they are long");
    PTA_REQUIRE(n_seqs <= 65535, "gated_scan: at most 65535 sequences in a step, got %d", n_seqs);
    hipStream_t s = (hipStream_t)stream;
    const dim3 grid((W + 63) / 64, n_seqs), block(64);
    if (dtype == PTA_F32)
        hipLaunchKernelGGL((gated_scan_kernel<float, 8>), grid, block, 0, s, (float*)y, (const float*)zxg, ld, bz, bx,
                           state, state_ld, cu_tokens, seq_slot, W);
    else if (dtype == PTA_BF16)
        hipLaunchKernelGGL((gated_scan_kernel<bf16_t, 8>), grid, block, 0, s, (bf16_t*)y, (const bf16_t*)zxg, ld, bz,
                           bx, state, state_ld, cu_tokens, seq_slot, W);
    else
        return pta_fail("gated_scan: unknown dtype %d", dtype);
    return pta_check_launch("gated_scan");
}

// ---- a short causal convolution per channel, with its activation ------------------------------------------
// out[t, c] = silu(b[c] + sum_k w[c, k] * in[t - (K - 1 - k), c]): the last tap is the token's own.  Inputs from
// before the step come out of the sequence's tail (the last K - 1 inputs, oldest first, [K - 1, C], zeros at a
// sequence's start), which conv_tail_kernel moves on once every token of the step has been formed.
#define PTA_CONV_MAX_TAPS 16

template <typename T>
__global__ void conv_silu_kernel(float* __restrict__ out, const T* __restrict__ in, long ld, const float* __restrict__ w,
                                 const float* __restrict__ b, const float* __restrict__ tail, long tail_ld,
                                 const int* __restrict__ cu_tokens, const int* __restrict__ token_seq,
                                 const int* __restrict__ seq_slot, int C, int K) {
    const int c = blockIdx.y * blockDim.x + threadIdx.x, m = blockIdx.x;
    if (c >= C) return;
    const int s = token_seq[m];
    const int first = cu_tokens[s], j = m - first;
    const float* tl = tail + (long)seq_slot[s] * tail_ld;
    float acc = b ? b[c] : 0.f;
    for (int k = 0; k < K; ++k) {
        const int jj = j - (K - 1 - k);
        const float v = jj >= 0 ? Io<T>::ld(in + (long)(first + jj) * ld + c) : tl[(long)(K - 1 + jj) * C + c];
        acc += w[(long)c * K + k] * v;
    }
    out[(long)m * C + c] = acc / (1.0f + expf(-acc));
}

template <typename T>
__global__ void conv_tail_kernel(const T* __restrict__ in, long ld, float* __restrict__ tail, long tail_ld,
                                 const int* __restrict__ cu_tokens, const int* __restrict__ seq_slot, int C, int K) {
    const int c = blockIdx.x * blockDim.x + threadIdx.x, s = blockIdx.y;
    if (c >= C) return;
    const int first = cu_tokens[s], n = cu_tokens[s + 1] - first;
    float* tl = tail + (long)seq_slot[s] * tail_ld;
    float keep[PTA_CONV_MAX_TAPS];
#pragma unroll
    for (int r = 0; r < PTA_CONV_MAX_TAPS; ++r) {
        if (r < K - 1) {
            const int jj = n - (K - 1) + r;  // the step's own row, or (negative) a row of the old tail
            keep[r] = jj >= 0 ? Io<T>::ld(in + (long)(first + jj) * ld + c) : tl[(long)(K - 1 + jj) * C + c];
        }
    }
#pragma unroll
    for (int r = 0; r < PTA_CONV_MAX_TAPS; ++r)
        if (r < K - 1) tl[(long)r * C + c] = keep[r];
}

extern "C" int pta_conv_silu(float* out, const void* in, long ld, const float* w, const float* b, float* tail,
                             long tail_ld, const int* cu_tokens, const int* token_seq, const int* seq_slot, int n_seqs,
                             int M, int C, int K, int dtype, void* stream) {
    PTA_REQUIRE(M > 0 && n_seqs > 0 && C > 0, "conv_silu: tokens=%d sequences=%d channels=%d must be positive", M, n_seqs, C);
    PTA_REQUIRE(K >= 1 && K <= PTA_CONV_MAX_TAPS, "conv_silu: %d taps are outside 1..%d", K, PTA_CONV_MAX_TAPS);
    PTA_REQUIRE(out && in && w && (tail || K == 1) && cu_tokens && token_seq && seq_slot, "conv_silu: null pointer");
    PTA_REQUIRE(ld >= C && tail_ld >= (long)(K - 1) * C, "conv_silu: rows lie closer together than they are long");
    PTA_REQUIRE(n_seqs <= 65535 && C <= 65535 * 64, "conv_silu: too many sequences or channels for one launch");
    PTA_REQUIRE(dtype == PTA_F32 || dtype == PTA_BF16, "conv_silu: unknown dtype %d", dtype);
    hipStream_t s = (hipStream_t)stream;
    const dim3 block(C >= 256 ? 256 : 64);
    const dim3 grid(M, (C + block.x - 1) / block.x), grid_tail((C + block.x - 1) / block.x, n_seqs);
    if (dtype == PTA_F32) {
        hipLaunchKernelGGL(conv_silu_kernel<float>, grid, block, 0, s, out, (const float*)in, ld, w, b, tail, tail_ld,
                           cu_tokens, token_seq, seq_slot, C, K);
        if (K > 1)
            hipLaunchKernelGGL(conv_tail_kernel<float>, grid_tail, block, 0, s, (const float*)in, ld, tail, tail_ld,
                               cu_tokens, seq_slot, C, K);
    } else {
        hipLaunchKernelGGL(conv_silu_kernel<bf16_t>, grid, block, 0, s, out, (const bf16_t*)in, ld, w, b, tail, tail_ld,
                           cu_tokens, token_seq, seq_slot, C, K);
        if (K > 1)
            hipLaunchKernelGGL(conv_tail_kernel<bf16_t>, grid_tail, block, 0, s, (const bf16_t*)in, ld, tail, tail_ld,
                               cu_tokens, seq_slot, C, K);
    }
    return pta_check_launch("conv_silu");
}

// ---- a state-space recurrence with a scalar decay per head --------------------------------------------------
// Per head h (of group g = h / (heads / groups)), with state S [N, P]:
//   dt = softplus(dt_raw + dt_bias[h]);  S = exp(-exp(A_log[h]) dt) S + dt B_t x_t^T;  y_t = S^T C_t + D[h] x_t
// xbc[t] = [x: heads * P | B: groups * N | C: groups * N] in 32-bit (the convolution's output).
// A workgroup of four waves owns (sequence, head, 64 columns p of the state); a wave owns sixteen columns, and its
// four groups of sixteen lanes take the rows n = q, q + 4, q + 8, ... each (NPT of them in registers).  A chunk
// of tokens' x, B, C and dt is staged in LDS by the whole workgroup, then walked in order.
#define SSM_CHUNK 16

template <typename T, int NPT>
__global__ __launch_bounds__(256) void ssm_scan_kernel(float* __restrict__ y, const float* __restrict__ xbc,
                                                       const T* __restrict__ dt_in, long dt_ld,
                                                       const float* __restrict__ dt_bias, const float* __restrict__ A_log,
                                                       const float* __restrict__ Dp, float* __restrict__ state,
                                                       long state_ld, const int* __restrict__ cu_tokens,
                                                       const int* __restrict__ seq_slot, int heads, int P, int N, int G) {
    extern __shared__ float lds[];
    const int h = blockIdx.y, s = blockIdx.z;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int pl = lane & 15, q = lane >> 4;
    const int p0 = blockIdx.x * 64;
    const int p = p0 + wave * 16 + pl;
    const int g = h / (heads / G);
    const int inner = heads * P, C = inner + 2 * G * N;
    const int t0 = cu_tokens[s], t1 = cu_tokens[s + 1];
    float* sb = state + (long)seq_slot[s] * state_ld + (long)h * N * P;
    float* B_s = lds;                        // [SSM_CHUNK][N]
    float* C_s = B_s + SSM_CHUNK * N;        // [SSM_CHUNK][N]
    float* x_s = C_s + SSM_CHUNK * N;        // [SSM_CHUNK][64]
    float* d_s = x_s + SSM_CHUNK * 64;       // [SSM_CHUNK] dt, then [SSM_CHUNK] decay
    float S[NPT];
#pragma unroll
    for (int i = 0; i < NPT; ++i) {
        const int n = q + 4 * i;
        S[i] = (n < N && p < P) ? sb[(long)n * P + p] : 0.f;
    }
    const float a = -expf(A_log[h]), bias = dt_bias[h], Dh = Dp[h];
    for (int c0 = t0; c0 < t1; c0 += SSM_CHUNK) {
        const int cnt = min(SSM_CHUNK, t1 - c0);
        __syncthreads();
        for (int i = threadIdx.x; i < cnt * N; i += 256) {
            const int tt = i / N, n = i - tt * N;
            const float* row = xbc + (long)(c0 + tt) * C + inner + g * N + n;
            B_s[tt * N + n] = row[0];
            C_s[tt * N + n] = row[(long)G * N];
        }
        for (int i = threadIdx.x; i < cnt * 64; i += 256) {
            const int tt = i >> 6, pp = i & 63;
            x_s[i] = p0 + pp < P ? xbc[(long)(c0 + tt) * C + (long)h * P + p0 + pp] : 0.f;
        }
        if (threadIdx.x < cnt) {
            const float dt = softplus_f(Io<T>::ld(dt_in + (long)(c0 + threadIdx.x) * dt_ld + h) + bias);
            d_s[threadIdx.x] = dt;
            d_s[SSM_CHUNK + threadIdx.x] = expf(a * dt);
        }
        __syncthreads();
        for (int tt = 0; tt < cnt; ++tt) {
            const float dt = d_s[tt], dA = d_s[SSM_CHUNK + tt];
            const float xv = x_s[tt * 64 + wave * 16 + pl];
            const float dx = dt * xv;
            float acc = 0.f;
#pragma unroll
            for (int i = 0; i < NPT; ++i) {
                const int n = q + 4 * i;
                if (n < N) {
                    S[i] = dA * S[i] + dx * B_s[tt * N + n];
                    acc += S[i] * C_s[tt * N + n];
                }
            }
            acc += __shfl_xor(acc, 16, 64);
            acc += __shfl_xor(acc, 32, 64);
            if (q == 0 && p < P) y[(long)(c0 + tt) * inner + (long)h * P + p] = acc + Dh * xv;
        }
    }
#pragma unroll
    for (int i = 0; i < NPT; ++i) {
        const int n = q + 4 * i;
        if (n < N && p < P) sb[(long)n * P + p] = S[i];
    }
}

template <typename T>
static int launch_ssm(float* y, const float* xbc, const T* dt_in, long dt_ld, const float* dt_bias, const float* A_log,
                      const float* Dp, float* state, long state_ld, const int* cu_tokens, const int* seq_slot,
                      int n_seqs, int heads, int P, int N, int G, hipStream_t s) {
    const dim3 grid((P + 63) / 64, heads, n_seqs), block(256);
    const size_t lds = (size_t)(2 * SSM_CHUNK * N + SSM_CHUNK * 64 + 2 * SSM_CHUNK) * sizeof(float);
#define SSM_LAUNCH(NPT_) hipLaunchKernelGGL((ssm_scan_kernel<T, NPT_>), grid, block, lds, s, y, xbc, dt_in, dt_ld, dt_bias, \
                                            A_log, Dp, state, state_ld, cu_tokens, seq_slot, heads, P, N, G)
    const int npt = (N + 3) / 4;
    if (npt <= 4) SSM_LAUNCH(4);
    else if (npt <= 8) SSM_LAUNCH(8);
    else if (npt <= 16) SSM_LAUNCH(16);
    else if (npt <= 32) SSM_LAUNCH(32);
    else SSM_LAUNCH(64);
#undef SSM_LAUNCH
    return pta_check_launch("ssm_scan");
}

extern "C" int pta_ssm_scan(float* y, const float* xbc, const void* dt_in, long dt_ld, const float* dt_bias,
                            const float* A_log, const float* Dp, float* state, long state_ld, const int* cu_tokens,
                            const int* seq_slot, int n_seqs, int heads, int P, int N, int G, int dtype, void* stream) {
    PTA_REQUIRE(n_seqs > 0 && heads > 0 && P > 0 && N > 0 && G > 0, "ssm_scan: sizes must be positive");
    PTA_REQUIRE(heads % G == 0, "ssm_scan: %d heads do not split into %d groups", heads, G);
    PTA_REQUIRE(N <= 256, "ssm_scan: a state of %d rows per head is more than the 256 the kernel holds", N);
    PTA_REQUIRE(heads <= 65535 && n_seqs <= 65535, "ssm_scan: too many heads or sequences for one launch");
    PTA_REQUIRE(y && xbc && dt_in && dt_bias && A_log && Dp && state && cu_tokens && seq_slot, "ssm_scan: null pointer");
    PTA_REQUIRE(dt_ld >= heads && state_ld >= (long)heads * N * P, "ssm_scan: rows lie closer together than they are long");
    hipStream_t s = (hipStream_t)stream;
    if (dtype == PTA_F32)
        return launch_ssm<float>(y, xbc, (const float*)dt_in, dt_ld, dt_bias, A_log, Dp, state, state_ld, cu_tokens,
                                 seq_slot, n_seqs, heads, P, N, G, s);
    if (dtype == PTA_BF16)
        return launch_ssm<bf16_t>(y, xbc, (const bf16_t*)dt_in, dt_ld, dt_bias, A_log, Dp, state, state_ld, cu_tokens,
                                  seq_slot, n_seqs, heads, P, N, G, s);
    return pta_fail("ssm_scan: unknown dtype %d", dtype);
}
