// The head of a block whose residual stream is 32-bit and whose mixer reads a token-shifted norm:
//
//   x     = base + (t1 + t2)                      (the terms a block left; none, one or two)
//   n1    = x / sqrt(mean(x^2) + eps) * w1
//   a     = n1 + (n1' - n1) * mu                  n1' : n1 of the token before (zeros at position 0)
//   m     = x / sqrt(mean(x^2) + eps) * w2        (optional second norm of the same x)
//
// One workgroup per token holds the token's row and the row before it in LDS.  The row before the first token of a
// step's piece of a sequence is the sequence's state, a row of a state table per slot, which holds the n1 of the
// sequence's last token so far.  A sequence that brings one token has its state read and then written by the same
// workgroup; a sequence that brings more has it written by a second small launch (PTA_SHIFT_STATE) once every
// token has read what it needs.  All arithmetic is 32-bit; a and m are stored in the compute type.
#include "common.h"
#include "pta_kernels.h"

#include <algorithm>

enum { PTA_SHIFT_TOKENS = 0, PTA_SHIFT_STATE = 1 };

template <typename T>
__device__ __forceinline__ float row_value(const float* base, const T* t1, const T* t2, long at) {
    float v = base[at];
    if (t1) {
        float add = Io<T>::ld(t1 + at);
        if (t2) add += Io<T>::ld(t2 + at);
        v += add;
    }
    return v;
}

template <typename T>
__global__ __launch_bounds__(1024) void shift_norm_kernel(
    T* __restrict__ a_out, T* __restrict__ m_out, float* __restrict__ x_out, const float* __restrict__ base,
    const T* __restrict__ t1, const T* __restrict__ t2, const float* __restrict__ w1, const float* __restrict__ w2,
    const float* __restrict__ mu, float* __restrict__ state, long state_ld, const int* __restrict__ token_seq,
    const int* __restrict__ token_pos, const int* __restrict__ cu_tokens, const int* __restrict__ seq_slot, int H,
    float eps, int mode) {
    extern __shared__ __attribute__((aligned(16))) float rows_s[];  // this token's row, then the row before it
    __shared__ float red[16];
    float* cur = rows_s;
    float* prv = rows_s + H;
    int m, s;
    if (mode == PTA_SHIFT_STATE) {
        s = blockIdx.x;
        const int n_new = cu_tokens[s + 1] - cu_tokens[s];
        if (n_new <= 1) return;  // written by the token's own workgroup
        m = cu_tokens[s + 1] - 1;
    } else {
        m = blockIdx.x;
        s = token_seq[m];
    }
    const int first = cu_tokens[s], last = cu_tokens[s + 1] - 1;
    const bool in_step = mode == PTA_SHIFT_TOKENS && m > first;  // the token before is a row of this step
    float ss = 0.f, sp = 0.f;
    for (int i = threadIdx.x; i < H; i += blockDim.x) {
        const float v = mode == PTA_SHIFT_STATE ? x_out[(long)m * H + i] : row_value<T>(base, t1, t2, (long)m * H + i);
        cur[i] = v;
        ss += v * v;
        if (in_step) {
            const float u = row_value<T>(base, t1, t2, (long)(m - 1) * H + i);
            prv[i] = u;
            sp += u * u;
        }
    }
    const float r = rsqrtf(block_sum(ss, red) / (float)H + eps);
    float rp = 0.f;
    if (in_step) rp = rsqrtf(block_sum(sp, red) / (float)H + eps);
    float* st = state + (long)seq_slot[s] * state_ld;
    if (mode == PTA_SHIFT_STATE) {
        for (int i = threadIdx.x; i < H; i += blockDim.x) st[i] = cur[i] * r * w1[i];
        return;
    }
    const bool at_zero = token_pos[m] == 0;
    const bool keep = m == last && first == last;
    for (int i = threadIdx.x; i < H; i += blockDim.x) {
        const float v = cur[i];
        const float n1 = v * r * w1[i];
        const float before = in_step ? prv[i] * rp * w1[i] : (at_zero ? 0.f : st[i]);
        Io<T>::st(a_out + (long)m * H + i, n1 + (before - n1) * mu[i]);
        if (m_out) Io<T>::st(m_out + (long)m * H + i, v * r * w2[i]);
        if (x_out) x_out[(long)m * H + i] = v;
        if (keep) st[i] = n1;
    }
}

// a_out, m_out (null: no second norm) [M, H] in the compute type; x_out (null only if there are no terms: the
// stream is then `base` itself) and base [M, H] 32-bit, two different buffers; t1, t2 (null: none) [M, H] in the
// compute type; state [slots, >= H] 32-bit rows state_ld apart.  several: some sequence brings more than one token.
extern "C" int pta_shift_norm(void* a_out, void* m_out, float* x_out, const float* base, const void* t1, const void* t2,
                              const float* w1, const float* w2, const float* mu, float* state, long state_ld,
                              const int* token_seq, const int* token_pos, const int* cu_tokens, const int* seq_slot,
                              int n_seqs, int M, int H, float eps, int several, int dtype, void* stream) {
    PTA_REQUIRE(M > 0 && n_seqs > 0 && H > 0, "shift_norm: tokens=%d sequences=%d features=%d must be positive", M, n_seqs, H);
    PTA_REQUIRE(a_out && base && w1 && mu && state && token_seq && token_pos && cu_tokens && seq_slot, "shift_norm: null pointer");
    PTA_REQUIRE((m_out == nullptr) == (w2 == nullptr), "shift_norm: a second norm needs its weight and its output");
    PTA_REQUIRE(t1 || !t2, "shift_norm: a second term without a first");
    PTA_REQUIRE(x_out != base, "shift_norm: the stream is written to a buffer of its own");
    PTA_REQUIRE(x_out || !t1, "shift_norm: a sum of terms needs a buffer for the stream");
    PTA_REQUIRE(state_ld >= H, "shift_norm: state rows of %d features cannot lie %ld apart", H, state_ld);
    PTA_REQUIRE(H <= 16384, "shift_norm: rows of %d features are more than the 16384 that fit the kernel's LDS", H);
    PTA_REQUIRE(dtype == PTA_F32 || dtype == PTA_BF16, "shift_norm: unknown dtype %d", dtype);
    hipStream_t s = (hipStream_t)stream;
    // a thread takes four features or so: a row's loads are then few rounds of many, not many rounds of few
    const dim3 block(std::min(1024, std::max(64, (H / 4 + 63) / 64 * 64)));
    const size_t lds = (size_t)2 * H * sizeof(float);
    if (lds > 64 * 1024) {
        if (dtype == PTA_F32)
            (void)hipFuncSetAttribute(reinterpret_cast<const void*>(shift_norm_kernel<float>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        else
            (void)hipFuncSetAttribute(reinterpret_cast<const void*>(shift_norm_kernel<bf16_t>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    }
    const float* stream_rows = x_out ? x_out : base;
    for (int mode = PTA_SHIFT_TOKENS; mode <= (several ? PTA_SHIFT_STATE : PTA_SHIFT_TOKENS); ++mode) {
        const dim3 grid(mode == PTA_SHIFT_TOKENS ? M : n_seqs);
        // the second launch reads the stream as the first one left it
        float* xo = mode == PTA_SHIFT_TOKENS ? x_out : const_cast<float*>(stream_rows);
        if (dtype == PTA_F32)
            hipLaunchKernelGGL(shift_norm_kernel<float>, grid, block, lds, s, (float*)a_out, (float*)m_out, xo, base,
                               (const float*)t1, (const float*)t2, w1, w2, mu, state, state_ld, token_seq, token_pos,
                               cu_tokens, seq_slot, H, eps, mode);
        else
            hipLaunchKernelGGL(shift_norm_kernel<bf16_t>, grid, block, lds, s, (bf16_t*)a_out, (bf16_t*)m_out, xo, base,
                               (const bf16_t*)t1, (const bf16_t*)t2, w1, w2, mu, state, state_ld, token_seq, token_pos,
                               cu_tokens, seq_slot, H, eps, mode);
    }
    return pta_check_launch("shift_norm");
}

// out = base + (t1 + t2), 32-bit: a stream and the terms a block left, for whoever wants the sum itself
template <typename T>
__global__ void wide_sum_kernel(float* __restrict__ out, const float* __restrict__ base, const T* __restrict__ t1,
                                const T* __restrict__ t2, long n) {
    const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) out[i] = row_value<T>(base, t1, t2, i);
}

extern "C" int pta_wide_sum(float* out, const float* base, const void* t1, const void* t2, long n, int dtype, void* stream) {
    PTA_REQUIRE(n > 0 && out && base && t1, "wide_sum: null pointer or nothing to add");
    PTA_REQUIRE(dtype == PTA_F32 || dtype == PTA_BF16, "wide_sum: unknown dtype %d", dtype);
    hipStream_t s = (hipStream_t)stream;
    const dim3 grid((unsigned)((n + 255) / 256));
    if (dtype == PTA_F32)
        hipLaunchKernelGGL(wide_sum_kernel<float>, grid, dim3(256), 0, s, out, base, (const float*)t1, (const float*)t2, n);
    else
        hipLaunchKernelGGL(wide_sum_kernel<bf16_t>, grid, dim3(256), 0, s, out, base, (const bf16_t*)t1, (const bf16_t*)t2, n);
    return pta_check_launch("wide_sum");
}
