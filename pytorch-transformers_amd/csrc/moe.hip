// A feed-forward of routed experts.
//
//   z = W_r h (32-bit); s = score(z) (sigmoid, or softmax over the experts); the `top` largest s are taken;
//   weights = s / (sum of the taken s + 1e-20) * scale   (or the taken s times scale, unnormalised);
//   out = sum over the taken experts e of weight_e * D_e (act(G_e h) * (U_e h))
//
// Expert matrices are held stacked: gate_up [E, 2F, H] (an expert's gate rows, then its up rows) and down [E, H, F].
//
// pta_moe_route     one workgroup per token: scores, the taken experts and their weights
// pta_moe_up        per (token, taken expert): act(G h) * (U h), a wave per few rows of the expert, H walked by lanes
// pta_moe_down      per token: the weighted sum of the taken experts' down products, in the order they were taken
// These three read an expert's matrices once per (token, expert): right for steps of few tokens, whose time is the
// bytes of the experts they touch.  Steps of many tokens sort the (token, expert) pairs by expert and run tiles of
// rows of one expert on the matrix cores (pta_moe_sort, pta_moe_grouped_*), so that an expert's matrices are read
// once per tile of tokens.
#include "common.h"
#include "pta_kernels.h"

// sum over K of w[k] * x_s[k] for one row of W, the lanes of a wave striding over K; every lane gets the sum
template <typename T>
__device__ __forceinline__ float wave_dot(const T* __restrict__ w, const float* __restrict__ x_s, int K, int lane) {
    float acc = 0.f;
    if (sizeof(T) == 2 && (K & 7) == 0 && ((uintptr_t)w & 15) == 0) {
        for (int k = lane * 8; k < K; k += PTA_WAVE * 8) {
            float f[8];
            unpack8(*reinterpret_cast<const uint4*>((const bf16_t*)w + k), f);
#pragma unroll
            for (int e = 0; e < 8; ++e) acc += f[e] * x_s[k + e];
        }
    } else {
        for (int k = lane; k < K; k += PTA_WAVE) acc += Io<T>::ld(w + k) * x_s[k];
    }
    return wave_sum(acc);
}

template <typename T>
__global__ __launch_bounds__(256) void moe_route_kernel(int* __restrict__ ids, float* __restrict__ wts,
                                                        const T* __restrict__ h, long h_ld, const float* __restrict__ Wr,
                                                        int H, int E, int top, int score_kind, int normalise, float scale) {
    extern __shared__ __attribute__((aligned(16))) float sm[];
    float* x_s = sm;       // [H]
    float* s_s = sm + H;   // [E]
    const int m = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
    for (int i = threadIdx.x; i < H; i += blockDim.x) x_s[i] = Io<T>::ld(h + (long)m * h_ld + i);
    __syncthreads();
    for (int e = wave; e < E; e += nw) {
        const float z = wave_dot<float>(Wr + (long)e * H, x_s, H, lane);
        if (lane == 0) s_s[e] = z;
    }
    __syncthreads();
    if (wave != 0) return;
    if (score_kind == PTA_ROUTE_SOFTMAX) {
        float mx = -INFINITY;
        for (int e = lane; e < E; e += PTA_WAVE) mx = fmaxf(mx, s_s[e]);
        mx = wave_max(mx);
        float sum = 0.f;
        for (int e = lane; e < E; e += PTA_WAVE) sum += expf(s_s[e] - mx);
        sum = wave_sum(sum);
        for (int e = lane; e < E; e += PTA_WAVE) s_s[e] = expf(s_s[e] - mx) / sum;
    } else {
        for (int e = lane; e < E; e += PTA_WAVE) s_s[e] = 1.0f / (1.0f + expf(-s_s[e]));
    }
    // the largest score `top` times over; of equal scores the expert with the lower index first
    float total = 0.f, mine = 0.f;
    int mine_id = 0;
    unsigned taken = 0;  // bit j: this lane's expert lane + 64 j has been taken
    for (int k = 0; k < top; ++k) {
        float best = -INFINITY;
        int at = E;
        for (int e = lane, j = 0; e < E; e += PTA_WAVE, ++j) {
            const float v = s_s[e];
            if (!((taken >> j) & 1u) && (v > best || at == E)) { best = v; at = e; }
        }
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) {
            const float ob = __shfl_xor(best, o, 64);
            const int oa = __shfl_xor(at, o, 64);
            if (oa < E && (at == E || ob > best || (ob == best && oa < at))) { best = ob; at = oa; }
        }
        if (lane == k) { mine = best; mine_id = at; }
        total += best;
        if ((at & 63) == lane) taken |= 1u << (at >> 6);
    }
    if (lane < top) {
        ids[(long)m * top + lane] = mine_id;
        wts[(long)m * top + lane] = (normalise ? mine / (total + 1e-20f) : mine) * scale;
    }
}

extern "C" int pta_moe_route(int* ids, float* wts, const void* h, long h_ld, const float* Wr, int M, int H, int E, int top,
                             int score_kind, int normalise, float scale, int dtype, void* stream) {
    PTA_REQUIRE(M > 0 && H > 0 && E > 0 && top > 0, "moe_route: sizes must be positive");
    PTA_REQUIRE(top <= E && top <= 64 && E <= 2048, "moe_route: %d experts per token of %d (at most 64 of at most 2048)", top, E);
    PTA_REQUIRE(ids && wts && h && Wr && h_ld >= H, "moe_route: null pointer or rows too close");
    PTA_REQUIRE(score_kind == PTA_ROUTE_SIGMOID || score_kind == PTA_ROUTE_SOFTMAX, "moe_route: score kind %d is not built", score_kind);
    PTA_REQUIRE((size_t)(H + E) * 4 <= 64 * 1024, "moe_route: %d features and %d experts do not fit the kernel's LDS", H, E);
    PTA_REQUIRE(dtype == PTA_F32 || dtype == PTA_BF16, "moe_route: unknown dtype %d", dtype);
    hipStream_t s = (hipStream_t)stream;
    const size_t lds = (size_t)(H + E) * sizeof(float);
    if (dtype == PTA_F32)
        hipLaunchKernelGGL(moe_route_kernel<float>, dim3(M), dim3(256), lds, s, ids, wts, (const float*)h, h_ld, Wr, H, E, top, score_kind, normalise, scale);
    else
        hipLaunchKernelGGL(moe_route_kernel<bf16_t>, dim3(M), dim3(256), lds, s, ids, wts, (const bf16_t*)h, h_ld, Wr, H, E, top, score_kind, normalise, scale);
    return pta_check_launch("moe_route");
}

#define MOE_ROWS 16  // rows of an expert's matrix per workgroup of four waves

template <typename T>
__global__ __launch_bounds__(256) void moe_up_kernel(T* __restrict__ act_out, const T* __restrict__ h, long h_ld,
                                                     const T* __restrict__ gate_up, const int* __restrict__ ids, int H,
                                                     int F, int top, int act) {
    extern __shared__ __attribute__((aligned(16))) float x_s[];  // [H]
    const int pair = blockIdx.x, m = pair / top, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int e = ids[pair];
    for (int i = threadIdx.x; i < H; i += blockDim.x) x_s[i] = Io<T>::ld(h + (long)m * h_ld + i);
    __syncthreads();
    const T* G = gate_up + (long)e * 2 * F * H;
    const T* U = G + (long)F * H;
    for (int f = blockIdx.y * MOE_ROWS + wave; f < min(F, (int)(blockIdx.y + 1) * MOE_ROWS); f += 4) {
        const float g = wave_dot<T>(G + (long)f * H, x_s, H, lane);
        const float u = wave_dot<T>(U + (long)f * H, x_s, H, lane);
        // (each product rounded to the compute type first, as a product on its own would leave it)
        if (lane == 0) Io<T>::st(act_out + (long)pair * F + f, apply_act(Io<T>::round(g), act) * Io<T>::round(u));
    }
}

template <typename T>
__global__ __launch_bounds__(256) void moe_down_kernel(T* __restrict__ out, const T* __restrict__ act_in,
                                                       const T* __restrict__ down, const int* __restrict__ ids,
                                                       const float* __restrict__ wts, int H, int F, int top) {
    extern __shared__ __attribute__((aligned(16))) float a_s[];  // [top][F]
    const int m = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    for (int i = threadIdx.x; i < top * F; i += blockDim.x) a_s[i] = Io<T>::ld(act_in + (long)m * top * F + i);
    __syncthreads();
    for (int n = blockIdx.y * MOE_ROWS + wave; n < min(H, (int)(blockIdx.y + 1) * MOE_ROWS); n += 4) {
        float acc = 0.f;
        for (int k = 0; k < top; ++k) {
            const T* D = down + ((long)ids[(long)m * top + k] * H + n) * F;
            acc += wts[(long)m * top + k] * Io<T>::round(wave_dot<T>(D, a_s + k * F, F, lane));
        }
        if (lane == 0) Io<T>::st(out + (long)m * H + n, acc);
    }
}

// act_out [M * top, F]; h [M, H] rows h_ld apart; gate_up [E, 2F, H]; ids [M, top]
extern "C" int pta_moe_up(void* act_out, const void* h, long h_ld, const void* gate_up, const int* ids, int M, int H, int F,
                          int top, int act, int dtype, void* stream) {
    PTA_REQUIRE(M > 0 && H > 0 && F > 0 && top > 0 && act_out && h && gate_up && ids && h_ld >= H, "moe_up: sizes must be positive and pointers given");
    PTA_REQUIRE(pta_act_known(act), "moe_up: unknown activation %d", act);
    PTA_REQUIRE((size_t)H * 4 <= 64 * 1024 && (F + MOE_ROWS - 1) / MOE_ROWS <= 65535, "moe_up: sizes beyond one launch");
    PTA_REQUIRE(dtype == PTA_F32 || dtype == PTA_BF16, "moe_up: unknown dtype %d", dtype);
    hipStream_t s = (hipStream_t)stream;
    const dim3 grid((unsigned)((long)M * top), (F + MOE_ROWS - 1) / MOE_ROWS);
    if (dtype == PTA_F32)
        hipLaunchKernelGGL(moe_up_kernel<float>, grid, dim3(256), (size_t)H * 4, s, (float*)act_out, (const float*)h, h_ld, (const float*)gate_up, ids, H, F, top, act);
    else
        hipLaunchKernelGGL(moe_up_kernel<bf16_t>, grid, dim3(256), (size_t)H * 4, s, (bf16_t*)act_out, (const bf16_t*)h, h_ld, (const bf16_t*)gate_up, ids, H, F, top, act);
    return pta_check_launch("moe_up");
}

// out [M, H]; act_in [M * top, F]; down [E, H, F]
extern "C" int pta_moe_down(void* out, const void* act_in, const void* down, const int* ids, const float* wts, int M, int H,
                            int F, int top, int dtype, void* stream) {
    PTA_REQUIRE(M > 0 && H > 0 && F > 0 && top > 0 && out && act_in && down && ids && wts, "moe_down: sizes must be positive and pointers given");
    PTA_REQUIRE((size_t)top * F * 4 <= 64 * 1024 && (H + MOE_ROWS - 1) / MOE_ROWS <= 65535, "moe_down: sizes beyond one launch");
    PTA_REQUIRE(dtype == PTA_F32 || dtype == PTA_BF16, "moe_down: unknown dtype %d", dtype);
    hipStream_t s = (hipStream_t)stream;
    const dim3 grid(M, (H + MOE_ROWS - 1) / MOE_ROWS);
    if (dtype == PTA_F32)
        hipLaunchKernelGGL(moe_down_kernel<float>, grid, dim3(256), (size_t)top * F * 4, s, (float*)out, (const float*)act_in, (const float*)down, ids, wts, H, F, top);
    else
        hipLaunchKernelGGL(moe_down_kernel<bf16_t>, grid, dim3(256), (size_t)top * F * 4, s, (bf16_t*)out, (const bf16_t*)act_in, (const bf16_t*)down, ids, wts, H, F, top);
    return pta_check_launch("moe_down");
}
