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
// y = S * silu(zxg_g).  One thread per (run of tokens, channel); the loads of UNROLL tokens are in flight together.
// Short steps are one launch from state to state (SCAN_WHOLE); a long prompt is cut into chunks that run side by
// side, as the state-space recurrence below is: SCAN_LOCAL (each chunk from zero: what it adds, and the product of
// its 1 - z), gated_carry_kernel (chunk after chunk), SCAN_OUTPUT (each chunk from its start, with the outputs).
enum { SCAN_WHOLE = 0, SCAN_LOCAL = 1, SCAN_OUTPUT = 2 };

template <typename T, int UNROLL, int MODE>
__global__ void gated_scan_kernel(T* __restrict__ y, const T* __restrict__ zxg, long ld, const float* __restrict__ bz,
                                  const float* __restrict__ bx, float* __restrict__ state, long state_ld,
                                  float* __restrict__ chunk_state, float* __restrict__ chunk_decay,
                                  const int* __restrict__ cu_tokens, const int* __restrict__ seq_slot, int W, int chunk,
                                  int max_chunks) {
    const int c = blockIdx.x * blockDim.x + threadIdx.x;
    const int s = MODE == SCAN_WHOLE ? blockIdx.y : blockIdx.y / max_chunks;
    if (c >= W) return;
    int t0 = cu_tokens[s], t1 = cu_tokens[s + 1];
    if (MODE != SCAN_WHOLE) {
        t0 += (blockIdx.y - s * max_chunks) * chunk;
        if (t0 >= t1) return;
        t1 = min(t1, t0 + chunk);
    }
    float* sp = MODE == SCAN_WHOLE ? state + (long)seq_slot[s] * state_ld + c : chunk_state + (long)blockIdx.y * W + c;
    float S = MODE == SCAN_LOCAL ? 0.f : *sp;
    float decay = 1.f;
    const float b_z = bz ? bz[c] : 0.f, b_x = bx ? bx[c] : 0.f;
    for (int t = t0; t < t1; t += UNROLL) {
        float zr[UNROLL], ur[UNROLL], gr[UNROLL];
#pragma unroll
        for (int i = 0; i < UNROLL; ++i) {
            const long row = (long)min(t + i, t1 - 1) * ld + c;
            zr[i] = Io<T>::ld(zxg + row);
            ur[i] = Io<T>::ld(zxg + row + W);
            if (MODE != SCAN_LOCAL) gr[i] = Io<T>::ld(zxg + row + 2 * W);
        }
#pragma unroll
        for (int i = 0; i < UNROLL; ++i) {
            if (t + i < t1) {
                const float z = sigmoid_f(zr[i] + b_z);
                const float u = ur[i] + b_x;
                const float cand = u >= 0.f ? u + 0.5f : sigmoid_f(u);
                S = (1.0f - z) * S + z * cand;
                decay *= 1.0f - z;
                if (MODE != SCAN_LOCAL) {
                    const float g = gr[i];
                    Io<T>::st(y + (long)(t + i) * W + c, S * (g / (1.0f + expf(-g))));
                }
            }
        }
    }
    if (MODE != SCAN_OUTPUT) *sp = S;
    if (MODE == SCAN_LOCAL) chunk_decay[(long)blockIdx.y * W + c] = decay;
}

__global__ void gated_carry_kernel(float* __restrict__ state, long state_ld, float* __restrict__ chunk_state,
                                   const float* __restrict__ chunk_decay, const int* __restrict__ cu_tokens,
                                   const int* __restrict__ seq_slot, int W, int chunk, int max_chunks) {
    const int c = blockIdx.x * blockDim.x + threadIdx.x, s = blockIdx.y;
    if (c >= W) return;
    const int n_chunks = (cu_tokens[s + 1] - cu_tokens[s] + chunk - 1) / chunk;
    float* sp = state + (long)seq_slot[s] * state_ld + c;
    float S = *sp;
    for (int k = 0; k < n_chunks; ++k) {
        const long at = ((long)s * max_chunks + k) * W + c;
        const float add = chunk_state[at];
        chunk_state[at] = S;
        S = chunk_decay[at] * S + add;
    }
    *sp = S;
}

template <typename T>
static int launch_gated(T* y, const T* zxg, long ld, const float* bz, const float* bx, float* state, long state_ld,
                        float* chunk_state, float* chunk_decay, const int* cu_tokens, const int* seq_slot, int n_seqs, int W,
                        int chunk, int max_chunks, hipStream_t s) {
    const dim3 block(64);
    const unsigned cb = (W + 63) / 64;
#define SCAN_ARGS y, zxg, ld, bz, bx, state, state_ld, chunk_state, chunk_decay, cu_tokens, seq_slot, W, chunk, max_chunks
    if (max_chunks <= 1) {
        hipLaunchKernelGGL((gated_scan_kernel<T, 8, SCAN_WHOLE>), dim3(cb, n_seqs), block, 0, s, SCAN_ARGS);
        return pta_check_launch("gated_scan");
    }
    hipLaunchKernelGGL((gated_scan_kernel<T, 8, SCAN_LOCAL>), dim3(cb, n_seqs * max_chunks), block, 0, s, SCAN_ARGS);
    hipLaunchKernelGGL(gated_carry_kernel, dim3(cb, n_seqs), block, 0, s, state, state_ld, chunk_state, chunk_decay, cu_tokens,
                       seq_slot, W, chunk, max_chunks);
    hipLaunchKernelGGL((gated_scan_kernel<T, 8, SCAN_OUTPUT>), dim3(cb, n_seqs * max_chunks), block, 0, s, SCAN_ARGS);
#undef SCAN_ARGS
    return pta_check_launch("gated_scan");
}

// chunk_state and chunk_decay [n_seqs * max_chunks, W] are scratch for steps whose longest sequence is cut into
// max_chunks > 1 chunks of `chunk` tokens; else unused
extern "C" int pta_gated_scan(void* y, const void* zxg, long ld, const float* bz, const float* bx, float* state,
                              long state_ld, float* chunk_state, float* chunk_decay, const int* cu_tokens,
                              const int* seq_slot, int n_seqs, int W, int chunk, int max_chunks, int dtype, void* stream) {
    PTA_REQUIRE(n_seqs > 0 && W > 0, "gated_scan: sequences=%d width=%d must be positive", n_seqs, W);
    PTA_REQUIRE(y && zxg && state && cu_tokens && seq_slot, "gated_scan: null pointer");
    PTA_REQUIRE(ld >= 3L * W && state_ld >= W, "gated_scan: rows lie closer together than they are long");
    PTA_REQUIRE(max_chunks >= 1 && (max_chunks == 1 || (chunk > 0 && chunk_state && chunk_decay)),
                "gated_scan: chunks need their size and scratch memory");
    PTA_REQUIRE((long)n_seqs * max_chunks <= 65535, "gated_scan: %ld runs are more than one launch takes", (long)n_seqs * max_chunks);
    hipStream_t s = (hipStream_t)stream;
    if (dtype == PTA_F32)
        return launch_gated<float>((float*)y, (const float*)zxg, ld, bz, bx, state, state_ld, chunk_state, chunk_decay,
                                   cu_tokens, seq_slot, n_seqs, W, chunk, max_chunks, s);
    if (dtype == PTA_BF16)
        return launch_gated<bf16_t>((bf16_t*)y, (const bf16_t*)zxg, ld, bz, bx, state, state_ld, chunk_state, chunk_decay,
                                    cu_tokens, seq_slot, n_seqs, W, chunk, max_chunks, s);
    return pta_fail("gated_scan: unknown dtype %d", dtype);
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
// A workgroup of four waves owns (sequence, head, 64 columns p of the state) and a run of tokens; a wave owns sixteen
// columns, and its four groups of sixteen lanes take NPT consecutive rows n each (in registers).  A piece of the
// run's x, B, C and dt is staged in LDS by the whole workgroup, then walked in order.
//
// Short steps (decoding, short prompts) are one launch that walks each sequence's tokens from its state to its
// state (SSM_WHOLE).  A long prompt is cut into chunks of `chunk` tokens that run side by side:
//   SSM_LOCAL  every chunk from a zero state: what it adds to the state, S_loc, and the product of its decays;
//   ssm_carry  chunk after chunk, S_in(c + 1) = decay(c) S_in(c) + S_loc(c), from the sequence's state to its state;
//   SSM_OUTPUT every chunk again from its S_in, now with the outputs.
// The recurrence is linear in the state, so this is the same sum in another order.
#define SSM_PIECE 16
enum { SSM_WHOLE = 0, SSM_LOCAL = 1, SSM_OUTPUT = 2 };

template <typename T, int NPT, int MODE>
__global__ __launch_bounds__(256) void ssm_scan_kernel(float* __restrict__ y, const float* __restrict__ xbc,
                                                       const T* __restrict__ dt_in, long dt_ld,
                                                       const float* __restrict__ dt_bias, const float* __restrict__ A_log,
                                                       const float* __restrict__ Dp, float* __restrict__ state,
                                                       long state_ld, float* __restrict__ chunk_state,
                                                       float* __restrict__ chunk_decay, const int* __restrict__ cu_tokens,
                                                       const int* __restrict__ seq_slot, int heads, int P, int N, int G,
                                                       int chunk, int max_chunks) {
    extern __shared__ __attribute__((aligned(16))) float lds[];
    constexpr int NP = 4 * NPT;  // rows of the state as the lanes hold them: N padded
    const int h = blockIdx.y;
    const int s = MODE == SSM_WHOLE ? blockIdx.z : blockIdx.z / max_chunks;
    const int c = MODE == SSM_WHOLE ? 0 : blockIdx.z - s * max_chunks;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int pl = lane & 15, q = lane >> 4;
    const int p0 = blockIdx.x * 64;
    const int p = p0 + wave * 16 + pl;
    const int g = h / (heads / G);
    const int inner = heads * P, C = inner + 2 * G * N;
    int t0 = cu_tokens[s];
    int t1 = cu_tokens[s + 1];
    if (MODE != SSM_WHOLE) {
        t0 += c * chunk;
        if (t0 >= t1) return;  // the sequence has fewer chunks
        t1 = min(t1, t0 + chunk);
    }
    const long hs = (long)N * P;  // a head's state
    float* sb = MODE == SSM_WHOLE ? state + (long)seq_slot[s] * state_ld + h * hs
                                  : chunk_state + ((long)blockIdx.z * heads + h) * hs;
    float* B_s = lds;                     // [SSM_PIECE][NP]
    float* C_s = B_s + SSM_PIECE * NP;    // [SSM_PIECE][NP]
    float* x_s = C_s + SSM_PIECE * NP;    // [SSM_PIECE][64]
    float* d_s = x_s + SSM_PIECE * 64;    // [SSM_PIECE] dt, then [SSM_PIECE] decay
    float S[NPT];
#pragma unroll
    for (int i = 0; i < NPT; ++i) {
        const int n = q * NPT + i;
        S[i] = (MODE != SSM_LOCAL && n < N && p < P) ? sb[(long)n * P + p] : 0.f;
    }
    const float a = -expf(A_log[h]), bias = dt_bias[h], Dh = Dp[h];
    float decay = 1.f;
    for (int c0 = t0; c0 < t1; c0 += SSM_PIECE) {
        const int cnt = min(SSM_PIECE, t1 - c0);
        __syncthreads();
        for (int i = threadIdx.x; i < cnt * NP; i += 256) {
            const int tt = i / NP, n = i - tt * NP;
            const float* row = xbc + (long)(c0 + tt) * C + inner + g * N + n;
            B_s[i] = n < N ? row[0] : 0.f;
            if (MODE != SSM_LOCAL) C_s[i] = n < N ? row[(long)G * N] : 0.f;
        }
        for (int i = threadIdx.x; i < cnt * 64; i += 256) {
            const int tt = i >> 6, pp = i & 63;
            x_s[i] = p0 + pp < P ? xbc[(long)(c0 + tt) * C + (long)h * P + p0 + pp] : 0.f;
        }
        if (threadIdx.x < cnt) {
            const float dt = softplus_f(Io<T>::ld(dt_in + (long)(c0 + threadIdx.x) * dt_ld + h) + bias);
            d_s[threadIdx.x] = dt;
            d_s[SSM_PIECE + threadIdx.x] = expf(a * dt);
        }
        __syncthreads();
        for (int tt = 0; tt < cnt; ++tt) {
            const float dt = d_s[tt], dA = d_s[SSM_PIECE + tt];
            const float xv = x_s[tt * 64 + wave * 16 + pl];
            const float dx = dt * xv;
            const float4* Bv = reinterpret_cast<const float4*>(B_s + tt * NP + q * NPT);
            const float4* Cv = reinterpret_cast<const float4*>(C_s + tt * NP + q * NPT);
            float acc = 0.f;
            decay *= dA;
#pragma unroll
            for (int i = 0; i < NPT; i += 4) {
                const float4 b = Bv[i >> 2];
                S[i] = dA * S[i] + dx * b.x;
                S[i + 1] = dA * S[i + 1] + dx * b.y;
                S[i + 2] = dA * S[i + 2] + dx * b.z;
                S[i + 3] = dA * S[i + 3] + dx * b.w;
                if (MODE != SSM_LOCAL) {
                    const float4 cc = Cv[i >> 2];
                    acc += S[i] * cc.x;
                    acc += S[i + 1] * cc.y;
                    acc += S[i + 2] * cc.z;
                    acc += S[i + 3] * cc.w;
                }
            }
            if (MODE != SSM_LOCAL) {
                acc += __shfl_xor(acc, 16, 64);
                acc += __shfl_xor(acc, 32, 64);
                if (q == 0 && p < P) y[(long)(c0 + tt) * inner + (long)h * P + p] = acc + Dh * xv;
            }
        }
    }
    if (MODE != SSM_OUTPUT) {
#pragma unroll
        for (int i = 0; i < NPT; ++i) {
            const int n = q * NPT + i;
            if (n < N && p < P) sb[(long)n * P + p] = S[i];
        }
    }
    if (MODE == SSM_LOCAL && threadIdx.x == 0 && blockIdx.x == 0) chunk_decay[(long)blockIdx.z * heads + h] = decay;
}

// chunk after chunk: what a chunk starts from takes the place of what it adds; the sequence's state moves to its end
__global__ void ssm_carry_kernel(float* __restrict__ state, long state_ld, float* __restrict__ chunk_state,
                                 const float* __restrict__ chunk_decay, const int* __restrict__ cu_tokens,
                                 const int* __restrict__ seq_slot, int heads, long hs, int chunk, int max_chunks) {
    const long e = (long)blockIdx.x * blockDim.x + threadIdx.x;  // element of the sequence's state
    const int s = blockIdx.y;
    if (e >= heads * hs) return;
    const int h = (int)(e / hs);
    const int n_chunks = (cu_tokens[s + 1] - cu_tokens[s] + chunk - 1) / chunk;
    float* sp = state + (long)seq_slot[s] * state_ld + e;
    float S = *sp;
    for (int c = 0; c < n_chunks; ++c) {
        const long seg = (long)s * max_chunks + c;
        float* cs = chunk_state + seg * heads * hs + e;
        const float add = *cs;
        *cs = S;
        S = chunk_decay[seg * heads + h] * S + add;
    }
    *sp = S;
}

template <typename T, int NPT>
static int launch_ssm_n(float* y, const float* xbc, const T* dt_in, long dt_ld, const float* dt_bias, const float* A_log,
                        const float* Dp, float* state, long state_ld, float* chunk_state, float* chunk_decay,
                        const int* cu_tokens, const int* seq_slot, int n_seqs, int heads, int P, int N, int G, int chunk,
                        int max_chunks, hipStream_t s) {
    const dim3 block(256);
    const size_t lds = (size_t)(2 * SSM_PIECE * 4 * NPT + SSM_PIECE * 64 + 2 * SSM_PIECE) * sizeof(float);
#define SSM_ARGS y, xbc, dt_in, dt_ld, dt_bias, A_log, Dp, state, state_ld, chunk_state, chunk_decay, cu_tokens, seq_slot, \
                 heads, P, N, G, chunk, max_chunks
    if (max_chunks <= 1) {
        hipLaunchKernelGGL((ssm_scan_kernel<T, NPT, SSM_WHOLE>), dim3((P + 63) / 64, heads, n_seqs), block, lds, s, SSM_ARGS);
        return pta_check_launch("ssm_scan");
    }
    const dim3 grid((P + 63) / 64, heads, n_seqs * max_chunks);
    const long hs = (long)N * P;
    hipLaunchKernelGGL((ssm_scan_kernel<T, NPT, SSM_LOCAL>), grid, block, lds, s, SSM_ARGS);
    hipLaunchKernelGGL(ssm_carry_kernel, dim3((unsigned)((heads * hs + 255) / 256), n_seqs), block, 0, s, state, state_ld,
                       chunk_state, chunk_decay, cu_tokens, seq_slot, heads, hs, chunk, max_chunks);
    hipLaunchKernelGGL((ssm_scan_kernel<T, NPT, SSM_OUTPUT>), grid, block, lds, s, SSM_ARGS);
#undef SSM_ARGS
    return pta_check_launch("ssm_scan");
}

template <typename T>
static int launch_ssm(float* y, const float* xbc, const T* dt_in, long dt_ld, const float* dt_bias, const float* A_log,
                      const float* Dp, float* state, long state_ld, float* chunk_state, float* chunk_decay,
                      const int* cu_tokens, const int* seq_slot, int n_seqs, int heads, int P, int N, int G, int chunk,
                      int max_chunks, hipStream_t s) {
#define SSM_LAUNCH(NPT_) return launch_ssm_n<T, NPT_>(y, xbc, dt_in, dt_ld, dt_bias, A_log, Dp, state, state_ld, chunk_state, \
                                                       chunk_decay, cu_tokens, seq_slot, n_seqs, heads, P, N, G, chunk, max_chunks, s)
    const int npt = (N + 3) / 4;
    if (npt <= 4) SSM_LAUNCH(4);
    if (npt <= 8) SSM_LAUNCH(8);
    if (npt <= 16) SSM_LAUNCH(16);
    if (npt <= 32) SSM_LAUNCH(32);
    SSM_LAUNCH(64);
#undef SSM_LAUNCH
}

// chunk_state [n_seqs * max_chunks, heads, N, P] and chunk_decay [n_seqs * max_chunks, heads] are scratch for steps
// whose longest sequence brings more than `chunk` tokens (max_chunks > 1: chunks per sequence, at most); else unused
extern "C" int pta_ssm_scan(float* y, const float* xbc, const void* dt_in, long dt_ld, const float* dt_bias,
                            const float* A_log, const float* Dp, float* state, long state_ld, float* chunk_state,
                            float* chunk_decay, const int* cu_tokens, const int* seq_slot, int n_seqs, int heads, int P,
                            int N, int G, int chunk, int max_chunks, int dtype, void* stream) {
    PTA_REQUIRE(n_seqs > 0 && heads > 0 && P > 0 && N > 0 && G > 0, "ssm_scan: sizes must be positive");
    PTA_REQUIRE(heads % G == 0, "ssm_scan: %d heads do not split into %d groups", heads, G);
    PTA_REQUIRE(N <= 256, "ssm_scan: a state of %d rows per head is more than the 256 the kernel holds", N);
    PTA_REQUIRE(heads <= 65535 && n_seqs <= 65535, "ssm_scan: too many heads or sequences for one launch");
    PTA_REQUIRE(y && xbc && dt_in && dt_bias && A_log && Dp && state && cu_tokens && seq_slot, "ssm_scan: null pointer");
    PTA_REQUIRE(dt_ld >= heads && state_ld >= (long)heads * N * P, "ssm_scan: rows lie closer together than they are long");
    PTA_REQUIRE(max_chunks >= 1 && (max_chunks == 1 || (chunk > 0 && chunk_state && chunk_decay)),
                "ssm_scan: chunks need their size and scratch memory");
    PTA_REQUIRE((long)n_seqs * max_chunks <= 65535, "ssm_scan: %ld chunks are more than one launch takes", (long)n_seqs * max_chunks);
    hipStream_t s = (hipStream_t)stream;
    if (dtype == PTA_F32)
        return launch_ssm<float>(y, xbc, (const float*)dt_in, dt_ld, dt_bias, A_log, Dp, state, state_ld, chunk_state,
                                 chunk_decay, cu_tokens, seq_slot, n_seqs, heads, P, N, G, chunk, max_chunks, s);
    if (dtype == PTA_BF16)
        return launch_ssm<bf16_t>(y, xbc, (const bf16_t*)dt_in, dt_ld, dt_bias, A_log, Dp, state, state_ld, chunk_state,
                                  chunk_decay, cu_tokens, seq_slot, n_seqs, heads, P, N, G, chunk, max_chunks, s);
    return pta_fail("ssm_scan: unknown dtype %d", dtype);
}
