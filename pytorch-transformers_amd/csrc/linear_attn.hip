// Linear attention with a constant decay per head, as a recurrence over a state per head:
//
//   q = act(q_raw), k = act(k_raw), v = act(v_raw)        act: silu, or the identity
//   S_t = decay[h] * S_(t-1) + k_t v_t^T                  S: [N, P] per head, N the key size, P the value size
//   o_t = S_t^T q_t
//
// The state is 32-bit, a row of a state table per slot, and so is all arithmetic; q, k and v come in the compute
// type (rows of one product, ld apart).  A workgroup of four waves owns (sequence, head, 64 columns p of the state)
// and a run of tokens; a wave owns sixteen columns, and its four groups of sixteen lanes hold NPT consecutive rows n
// each in registers; the sum over rows ends with two exchanges between the groups.  A piece of the run's q, k, v is
// staged in LDS by the whole workgroup, activated on the way, then walked in order.
//
// Short steps are one launch from each sequence's state to its state (LA_WHOLE).  A long prompt is cut into chunks
// that run side by side: LA_LOCAL (every chunk from a zero state: what it adds), la_carry (chunk after chunk,
// S_in(c + 1) = decay^len(c) S_in(c) + S_loc(c), from the sequence's state to its state), LA_OUTPUT (every chunk
// again from its S_in, with the outputs).  The recurrence is linear in the state: the same sum in another order.
#include "common.h"
#include "pta_kernels.h"

#define LA_PIECE 16
enum { LA_WHOLE = 0, LA_LOCAL = 1, LA_OUTPUT = 2 };

template <typename T, int NPT, int MODE>
__global__ __launch_bounds__(256) void decay_scan_kernel(
    float* __restrict__ y, const T* __restrict__ q_in, const T* __restrict__ k_in, const T* __restrict__ v_in, long ld,
    const float* __restrict__ decay, float* __restrict__ state, long state_ld, float* __restrict__ chunk_state,
    const int* __restrict__ cu_tokens, const int* __restrict__ seq_slot, int heads, int P, int N, int act, int chunk,
    int max_chunks) {
    extern __shared__ __attribute__((aligned(16))) float lds[];
    constexpr int NP = 4 * NPT;  // rows of the state as the lanes hold them: N padded
    const int h = blockIdx.y;
    const int s = MODE == LA_WHOLE ? blockIdx.z : blockIdx.z / max_chunks;
    const int c = MODE == LA_WHOLE ? 0 : blockIdx.z - s * max_chunks;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int pl = lane & 15, g4 = lane >> 4;
    const int p0 = blockIdx.x * 64;
    const int p = p0 + wave * 16 + pl;
    int t0 = cu_tokens[s];
    int t1 = cu_tokens[s + 1];
    if (MODE != LA_WHOLE) {
        t0 += c * chunk;
        if (t0 >= t1) return;  // the sequence has fewer chunks
        t1 = min(t1, t0 + chunk);
    }
    const long hs = (long)N * P;  // a head's state
    float* sb = MODE == LA_WHOLE ? state + (long)seq_slot[s] * state_ld + h * hs
                                 : chunk_state + ((long)blockIdx.z * heads + h) * hs;
    float* k_s = lds;                    // [LA_PIECE][NP]
    float* q_s = k_s + LA_PIECE * NP;    // [LA_PIECE][NP]
    float* v_s = q_s + LA_PIECE * NP;    // [LA_PIECE][64]
    float S[NPT];
#pragma unroll
    for (int i = 0; i < NPT; ++i) {
        const int n = g4 * NPT + i;
        S[i] = (MODE != LA_LOCAL && n < N && p < P) ? sb[(long)n * P + p] : 0.f;
    }
    const float a = decay[h];
    for (int c0 = t0; c0 < t1; c0 += LA_PIECE) {
        const int cnt = min(LA_PIECE, t1 - c0);
        __syncthreads();
        for (int i = threadIdx.x; i < cnt * NP; i += 256) {
            const int tt = i / NP, n = i - tt * NP;
            const long at = (long)(c0 + tt) * ld + (long)h * N + n;
            k_s[i] = n < N ? apply_act(Io<T>::ld(k_in + at), act) : 0.f;
            if (MODE != LA_LOCAL) q_s[i] = n < N ? apply_act(Io<T>::ld(q_in + at), act) : 0.f;
        }
        for (int i = threadIdx.x; i < cnt * 64; i += 256) {
            const int tt = i >> 6, pp = i & 63;
            v_s[i] = p0 + pp < P ? apply_act(Io<T>::ld(v_in + (long)(c0 + tt) * ld + (long)h * P + p0 + pp), act) : 0.f;
        }
        __syncthreads();
        for (int tt = 0; tt < cnt; ++tt) {
            const float xv = v_s[tt * 64 + wave * 16 + pl];
            const float4* kv = reinterpret_cast<const float4*>(k_s + tt * NP + g4 * NPT);
            const float4* qv = reinterpret_cast<const float4*>(q_s + tt * NP + g4 * NPT);
            float acc = 0.f;
#pragma unroll
            for (int i = 0; i < NPT; i += 4) {
                const float4 b = kv[i >> 2];
                S[i] = a * S[i] + xv * b.x;
                S[i + 1] = a * S[i + 1] + xv * b.y;
                S[i + 2] = a * S[i + 2] + xv * b.z;
                S[i + 3] = a * S[i + 3] + xv * b.w;
                if (MODE != LA_LOCAL) {
                    const float4 cc = qv[i >> 2];
                    acc += S[i] * cc.x;
                    acc += S[i + 1] * cc.y;
                    acc += S[i + 2] * cc.z;
                    acc += S[i + 3] * cc.w;
                }
            }
            if (MODE != LA_LOCAL) {
                acc += __shfl_xor(acc, 16, 64);
                acc += __shfl_xor(acc, 32, 64);
                if (g4 == 0 && p < P) y[(long)(c0 + tt) * heads * P + (long)h * P + p] = acc;
            }
        }
    }
    if (MODE != LA_OUTPUT) {
#pragma unroll
        for (int i = 0; i < NPT; ++i) {
            const int n = g4 * NPT + i;
            if (n < N && p < P) sb[(long)n * P + p] = S[i];
        }
    }
}

// chunk after chunk: what a chunk starts from takes the place of what it adds; the sequence's state moves to its end
__global__ void la_carry_kernel(float* __restrict__ state, long state_ld, float* __restrict__ chunk_state,
                                const float* __restrict__ decay, const int* __restrict__ cu_tokens,
                                const int* __restrict__ seq_slot, int heads, long hs, int chunk, int max_chunks) {
    const long e = (long)blockIdx.x * blockDim.x + threadIdx.x;  // element of the sequence's state
    const int s = blockIdx.y;
    if (e >= heads * hs) return;
    const int h = (int)(e / hs);
    const int n_new = cu_tokens[s + 1] - cu_tokens[s];
    const int n_chunks = (n_new + chunk - 1) / chunk;
    const float a = decay[h];
    float* sp = state + (long)seq_slot[s] * state_ld + e;
    float S = *sp;
    const long step = (long)heads * hs;  // from a chunk's element to the next chunk's
    float* cs = chunk_state + (long)s * max_chunks * step + e;
    float pw_full = 1.f;  // decay^chunk as the chunks' own walks multiply it up
    for (int i = 0; i < chunk; ++i) pw_full *= a;
    // eight chunks' additions are asked for at once: the walk itself is a chain, its loads need not be
    for (int c0 = 0; c0 < n_chunks; c0 += 8) {
        float add[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) add[j] = c0 + j < n_chunks ? cs[(long)(c0 + j) * step] : 0.f;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const int c = c0 + j;
            if (c < n_chunks) {
                cs[(long)c * step] = S;
                float pw = pw_full;
                const int len = n_new - c * chunk;
                if (len < chunk) {
                    pw = 1.f;
                    for (int i = 0; i < len; ++i) pw *= a;
                }
                S = pw * S + add[j];
            }
        }
    }
    *sp = S;
}

template <typename T, int NPT>
static int launch_la_n(float* y, const T* q, const T* k, const T* v, long ld, const float* decay, float* state,
                       long state_ld, float* chunk_state, const int* cu_tokens, const int* seq_slot, int n_seqs, int heads,
                       int P, int N, int act, int chunk, int max_chunks, hipStream_t s) {
    const dim3 block(256);
    const size_t lds = (size_t)(2 * LA_PIECE * 4 * NPT + LA_PIECE * 64) * sizeof(float);
#define LA_ARGS y, q, k, v, ld, decay, state, state_ld, chunk_state, cu_tokens, seq_slot, heads, P, N, act, chunk, max_chunks
    if (max_chunks <= 1) {
        hipLaunchKernelGGL((decay_scan_kernel<T, NPT, LA_WHOLE>), dim3((P + 63) / 64, heads, n_seqs), block, lds, s, LA_ARGS);
        return pta_check_launch("decay_scan");
    }
    const dim3 grid((P + 63) / 64, heads, n_seqs * max_chunks);
    const long hs = (long)N * P;
    hipLaunchKernelGGL((decay_scan_kernel<T, NPT, LA_LOCAL>), grid, block, lds, s, LA_ARGS);
    hipLaunchKernelGGL(la_carry_kernel, dim3((unsigned)((heads * hs + 255) / 256), n_seqs), block, 0, s, state, state_ld,
                       chunk_state, decay, cu_tokens, seq_slot, heads, hs, chunk, max_chunks);
    hipLaunchKernelGGL((decay_scan_kernel<T, NPT, LA_OUTPUT>), grid, block, lds, s, LA_ARGS);
#undef LA_ARGS
    return pta_check_launch("decay_scan");
}

template <typename T>
static int launch_la(float* y, const T* q, const T* k, const T* v, long ld, const float* decay, float* state, long state_ld,
                     float* chunk_state, const int* cu_tokens, const int* seq_slot, int n_seqs, int heads, int P, int N,
                     int act, int chunk, int max_chunks, hipStream_t s) {
#define LA_LAUNCH(NPT_) return launch_la_n<T, NPT_>(y, q, k, v, ld, decay, state, state_ld, chunk_state, cu_tokens, seq_slot, \
                                                     n_seqs, heads, P, N, act, chunk, max_chunks, s)
    const int npt = (N + 3) / 4;
    if (npt <= 4) LA_LAUNCH(4);
    if (npt <= 8) LA_LAUNCH(8);
    if (npt <= 16) LA_LAUNCH(16);
    if (npt <= 32) LA_LAUNCH(32);
    LA_LAUNCH(64);
#undef LA_LAUNCH
}

// y [M, heads * P] 32-bit; q, k [M, heads * N] and v [M, heads * P] in the compute type, rows ld apart; decay [heads];
// state [slots, >= heads * N * P] rows state_ld apart.  chunk_state [n_seqs * max_chunks, heads, N, P] is scratch for
// steps whose longest sequence brings more than `chunk` tokens (max_chunks > 1: chunks per sequence, at most).
extern "C" int pta_decay_scan(float* y, const void* q, const void* k, const void* v, long ld, const float* decay,
                              float* state, long state_ld, float* chunk_state, const int* cu_tokens, const int* seq_slot,
                              int n_seqs, int heads, int P, int N, int act, int chunk, int max_chunks, int dtype, void* stream) {
    PTA_REQUIRE(n_seqs > 0 && heads > 0 && P > 0 && N > 0, "decay_scan: sizes must be positive");
    PTA_REQUIRE(N <= 256, "decay_scan: keys of %d elements are more than the 256 rows of state the kernel holds", N);
    PTA_REQUIRE(heads <= 65535 && n_seqs <= 65535, "decay_scan: too many heads or sequences for one launch");
    PTA_REQUIRE(y && q && k && v && decay && state && cu_tokens && seq_slot, "decay_scan: null pointer");
    PTA_REQUIRE(ld >= (long)heads * N && ld >= (long)heads * P && state_ld >= (long)heads * N * P,
                "decay_scan: rows lie closer together than they are long");
    PTA_REQUIRE(pta_act_known(act), "decay_scan: unknown activation %d", act);
    PTA_REQUIRE(max_chunks >= 1 && (max_chunks == 1 || (chunk > 0 && chunk_state)), "decay_scan: chunks need their size and scratch memory");
    PTA_REQUIRE((long)n_seqs * max_chunks <= 65535, "decay_scan: %ld chunks are more than one launch takes", (long)n_seqs * max_chunks);
    hipStream_t s = (hipStream_t)stream;
    if (dtype == PTA_F32)
        return launch_la<float>(y, (const float*)q, (const float*)k, (const float*)v, ld, decay, state, state_ld, chunk_state,
                                cu_tokens, seq_slot, n_seqs, heads, P, N, act, chunk, max_chunks, s);
    if (dtype == PTA_BF16)
        return launch_la<bf16_t>(y, (const bf16_t*)q, (const bf16_t*)k, (const bf16_t*)v, ld, decay, state, state_ld,
                                 chunk_state, cu_tokens, seq_slot, n_seqs, heads, P, N, act, chunk, max_chunks, s);
    return pta_fail("decay_scan: unknown dtype %d", dtype);
}
