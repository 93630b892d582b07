// A residual stream that is held in 32-bit whatever the model's compute type: RMS norm with the pieces that
// stand around it (a gate in front, a gain stored around zero or around one, groups of a row normalised apart,
// a residual that the scaled result is added to), the weighted sum of the streams that earlier layers left,
// and the small conversions between the 32-bit stream and the compute type.
//
// Every sum over a row is taken in 32-bit in an order that depends on the row's length alone, so a token's
// values do not depend on what else is in the step.
#include "common.h"
#include "pta_kernels.h"

// v = x (* silu(gate)); n = v / sqrt(mean_group(v^2) + eps) * (offset + w); out = residual + mult * n (or n).
// With `planes` the result (in out_wide) is the last of `count` streams that lie `plane` floats apart, and the launch
// goes on to their weighted sum (mix_wide, and out_narrow in the compute type), as depth_mix_kernel forms it.
// One workgroup per (row, group).  TI: type of x (float or the compute type), T: compute type (gate, narrow output).
template <typename TI, typename T>
__global__ void rmsnorm_kernel(T* __restrict__ out_narrow, float* __restrict__ out_wide, const TI* __restrict__ x,
                               long x_ld, const T* __restrict__ gate, long gate_ld, const int* __restrict__ rows,
                               const float* __restrict__ w, float offset, int group_len, float eps,
                               const float* __restrict__ residual, float mult, int H,
                               const float* __restrict__ planes, long plane, const float* __restrict__ coef, int count,
                               float* __restrict__ mix_wide) {
    __shared__ float red[16];
    const int m = blockIdx.x, g = blockIdx.y;
    const long src = rows ? rows[m] : m;
    const TI* xr = x + src * x_ld + (long)g * group_len;
    const T* gr = gate ? gate + src * gate_ld + (long)g * group_len : nullptr;
    float ss = 0.f;
    for (int i = threadIdx.x; i < group_len; i += blockDim.x) {
        float v = Io<TI>::ld(xr + i);
        if (gr) { const float z = Io<T>::ld(gr + i); v *= z / (1.0f + expf(-z)); }
        ss += v * v;
    }
    ss = block_sum(ss, red);
    const float inv = 1.0f / sqrtf(ss / (float)group_len + eps);
    const long o = (long)m * H + (long)g * group_len;
    for (int i = threadIdx.x; i < group_len; i += blockDim.x) {
        float v = Io<TI>::ld(xr + i);
        if (gr) { const float z = Io<T>::ld(gr + i); v *= z / (1.0f + expf(-z)); }
        float n = v * inv * (offset + w[g * group_len + i]);
        if (residual) n = residual[src * H + (long)g * group_len + i] + mult * n;
        if (out_wide) out_wide[o + i] = n;
        if (planes) {  // the result is the last of `count` streams: what goes on is their weighted sum, added in order
            float acc = 0.f;
#pragma unroll 8
            for (int j = 0; j + 1 < count; ++j) acc += coef[j] * planes[(long)j * plane + o + i];
            n = acc + coef[count - 1] * n;
            mix_wide[o + i] = n;
        }
        if (out_narrow) Io<T>::st(out_narrow + o + i, n);
    }
}

// The same for groups of at most VPT * blockDim elements: a thread keeps its VPT elements in registers between the
// two passes, and every pass asks for all of its loads before it uses one (a row of a few thousand elements in a
// step of a few rows is a chain of memory round trips and nothing else).
template <typename TI, typename T, int VPT>
__global__ void rmsnorm_reg_kernel(T* __restrict__ out_narrow, float* __restrict__ out_wide, const TI* __restrict__ x,
                                   long x_ld, const T* __restrict__ gate, long gate_ld, const int* __restrict__ rows,
                                   const float* __restrict__ w, float offset, int group_len, float eps,
                                   const float* __restrict__ residual, float mult, int H,
                                   const float* __restrict__ planes, long plane, const float* __restrict__ coef, int count,
                                   float* __restrict__ mix_wide) {
    __shared__ float red[16];
    const int m = blockIdx.x, g = blockIdx.y;
    const long src = rows ? rows[m] : m;
    const TI* xr = x + src * x_ld + (long)g * group_len;
    const T* gr = gate ? gate + src * gate_ld + (long)g * group_len : nullptr;
    float v[VPT], z[VPT];
#pragma unroll
    for (int k = 0; k < VPT; ++k) {
        const int i = threadIdx.x + k * blockDim.x;
        v[k] = i < group_len ? Io<TI>::ld(xr + i) : 0.f;
        z[k] = (gr && i < group_len) ? Io<T>::ld(gr + i) : 0.f;
    }
    const long o = (long)m * H + (long)g * group_len;
    float wv[VPT], rv[VPT];
#pragma unroll
    for (int k = 0; k < VPT; ++k) {  // asked for now, used after the sum
        const int i = threadIdx.x + k * blockDim.x;
        wv[k] = i < group_len ? w[g * group_len + i] : 0.f;
        rv[k] = (residual && i < group_len) ? residual[src * H + (long)g * group_len + i] : 0.f;
    }
    float ss = 0.f;
#pragma unroll
    for (int k = 0; k < VPT; ++k) {
        if (gr) v[k] *= z[k] / (1.0f + expf(-z[k]));
        ss += v[k] * v[k];
    }
    ss = block_sum(ss, red);
    const float inv = 1.0f / sqrtf(ss / (float)group_len + eps);
    float n[VPT];
#pragma unroll
    for (int k = 0; k < VPT; ++k) {
        n[k] = v[k] * inv * (offset + wv[k]);
        if (residual) n[k] = rv[k] + mult * n[k];
    }
    if (out_wide) {
#pragma unroll
        for (int k = 0; k < VPT; ++k) {
            const int i = threadIdx.x + k * blockDim.x;
            if (i < group_len) out_wide[o + i] = n[k];
        }
    }
    if (planes) {
        float acc[VPT];
#pragma unroll
        for (int k = 0; k < VPT; ++k) acc[k] = 0.f;
        for (int j = 0; j + 1 < count; ++j) {
            const float c = coef[j];
            const float* pj = planes + (long)j * plane + o;
            float pv[VPT];
#pragma unroll
            for (int k = 0; k < VPT; ++k) {
                const int i = threadIdx.x + k * blockDim.x;
                pv[k] = i < group_len ? pj[i] : 0.f;
            }
#pragma unroll
            for (int k = 0; k < VPT; ++k) acc[k] += c * pv[k];
        }
        const float c = coef[count - 1];
#pragma unroll
        for (int k = 0; k < VPT; ++k) {
            const int i = threadIdx.x + k * blockDim.x;
            n[k] = acc[k] + c * n[k];
            if (i < group_len) mix_wide[o + i] = n[k];
        }
    }
    if (out_narrow) {
#pragma unroll
        for (int k = 0; k < VPT; ++k) {
            const int i = threadIdx.x + k * blockDim.x;
            if (i < group_len) Io<T>::st(out_narrow + o + i, n[k]);
        }
    }
}

extern "C" int pta_rmsnorm(void* out_narrow, float* out_wide, const void* x, int x_wide, long x_ld, const void* gate,
                           long gate_ld, const int* rows, const float* w, float offset, int groups, float eps,
                           const float* residual, float mult, const float* planes, long plane, const float* coef,
                           int count, float* mix_wide, int M, int H, int dtype, void* stream) {
    PTA_REQUIRE(M > 0 && H > 0, "rmsnorm: M=%d H=%d must be positive", M, H);
    PTA_REQUIRE(x && w && (out_narrow || out_wide), "rmsnorm: null pointer");
    PTA_REQUIRE(groups > 0 && H % groups == 0, "rmsnorm: %d features do not split into %d equal groups", H, groups);
    PTA_REQUIRE(groups <= 65535, "rmsnorm: at most 65535 groups, got %d", groups);
    PTA_REQUIRE(x_ld >= H && (!gate || gate_ld >= H), "rmsnorm: rows lie closer together than they are long");
    PTA_REQUIRE(dtype == PTA_F32 || dtype == PTA_BF16, "rmsnorm: unknown dtype %d", dtype);
    PTA_REQUIRE(!planes || (coef && count >= 1 && mix_wide && out_wide && !rows && plane >= (long)M * H),
                "rmsnorm: a sum of streams needs their weights, the planes' distance and both 32-bit results");
    hipStream_t s = (hipStream_t)stream;
    const int L = H / groups;
    const dim3 grid(M, groups), block(L >= 2048 ? 512 : L > 64 ? 256 : 64);
#define RMS_ARGS(TN, TX, TG) (TN*)out_narrow, out_wide, (const TX*)x, x_ld, (const TG*)gate, gate_ld, rows, w, offset, L, eps, \
                             residual, mult, H, planes, plane, coef, count, mix_wide
    if (L <= 8 * (int)block.x) {  // the group fits the threads' registers
        if (dtype == PTA_F32) hipLaunchKernelGGL((rmsnorm_reg_kernel<float, float, 8>), grid, block, 0, s, RMS_ARGS(float, float, float));
        else if (x_wide) hipLaunchKernelGGL((rmsnorm_reg_kernel<float, bf16_t, 8>), grid, block, 0, s, RMS_ARGS(bf16_t, float, bf16_t));
        else hipLaunchKernelGGL((rmsnorm_reg_kernel<bf16_t, bf16_t, 8>), grid, block, 0, s, RMS_ARGS(bf16_t, bf16_t, bf16_t));
        return pta_check_launch("rmsnorm");
    }
#undef RMS_ARGS
    if (dtype == PTA_F32)
        hipLaunchKernelGGL((rmsnorm_kernel<float, float>), grid, block, 0, s, (float*)out_narrow, out_wide,
                           (const float*)x, x_ld, (const float*)gate, gate_ld, rows, w, offset, L, eps, residual, mult, H, planes, plane, coef, count, mix_wide);
    else if (x_wide)
        hipLaunchKernelGGL((rmsnorm_kernel<float, bf16_t>), grid, block, 0, s, (bf16_t*)out_narrow, out_wide,
                           (const float*)x, x_ld, (const bf16_t*)gate, gate_ld, rows, w, offset, L, eps, residual, mult, H, planes, plane, coef, count, mix_wide);
    else
        hipLaunchKernelGGL((rmsnorm_kernel<bf16_t, bf16_t>), grid, block, 0, s, (bf16_t*)out_narrow, out_wide,
                           (const bf16_t*)x, x_ld, (const bf16_t*)gate, gate_ld, rows, w, offset, L, eps, residual, mult, H, planes, plane, coef, count, mix_wide);
    return pta_check_launch("rmsnorm");
}

// out[i] = sum_j coef[j] * planes[j][i], j = 0 .. count - 1 in that order; the planes lie `plane` floats apart.
template <typename T, int V>
__global__ void depth_mix_kernel(float* __restrict__ out_wide, T* __restrict__ out_narrow,
                                 const float* __restrict__ planes, long plane, const float* __restrict__ coef,
                                 int count, long n) {
    const long i0 = ((long)blockIdx.x * blockDim.x + threadIdx.x) * V;
    if (i0 >= n) return;
    float acc[V];
#pragma unroll
    for (int v = 0; v < V; ++v) acc[v] = 0.f;
    for (int j = 0; j < count; ++j) {
        const float c = coef[j];
        const float* p = planes + (long)j * plane + i0;
        if (V == 4) {
            const float4 q = *reinterpret_cast<const float4*>(p);
            acc[0] += c * q.x; acc[1 % V] += c * q.y; acc[2 % V] += c * q.z; acc[3 % V] += c * q.w;
        } else {
            acc[0] += c * p[0];
        }
    }
#pragma unroll
    for (int v = 0; v < V; ++v) {
        if (out_wide) out_wide[i0 + v] = acc[v];
        if (out_narrow) Io<T>::st(out_narrow + i0 + v, acc[v]);
    }
}

extern "C" int pta_depth_mix(float* out_wide, void* out_narrow, const float* planes, long plane, const float* coef,
                             int count, long n, int dtype, void* stream) {
    PTA_REQUIRE(n > 0 && count > 0, "depth_mix: n=%ld count=%d must be positive", n, count);
    PTA_REQUIRE(planes && coef && (out_wide || out_narrow), "depth_mix: null pointer");
    PTA_REQUIRE(plane >= n, "depth_mix: the planes overlap");
    PTA_REQUIRE(dtype == PTA_F32 || dtype == PTA_BF16, "depth_mix: unknown dtype %d", dtype);
    hipStream_t s = (hipStream_t)stream;
    const bool wide4 = n % 4 == 0 && plane % 4 == 0 && ((uintptr_t)planes % 16) == 0;
    const long threads = wide4 ? n / 4 : n;
    const dim3 grid((unsigned)((threads + 255) / 256)), block(256);
    if (dtype == PTA_F32) {
        if (wide4) hipLaunchKernelGGL((depth_mix_kernel<float, 4>), grid, block, 0, s, out_wide, (float*)out_narrow, planes, plane, coef, count, n);
        else hipLaunchKernelGGL((depth_mix_kernel<float, 1>), grid, block, 0, s, out_wide, (float*)out_narrow, planes, plane, coef, count, n);
    } else {
        if (wide4) hipLaunchKernelGGL((depth_mix_kernel<bf16_t, 4>), grid, block, 0, s, out_wide, (bf16_t*)out_narrow, planes, plane, coef, count, n);
        else hipLaunchKernelGGL((depth_mix_kernel<bf16_t, 1>), grid, block, 0, s, out_wide, (bf16_t*)out_narrow, planes, plane, coef, count, n);
    }
    return pta_check_launch("depth_mix");
}

// out (32-bit) = in (compute type), element by element
template <typename T>
__global__ void widen_kernel(float* __restrict__ out, const T* __restrict__ in, long n) {
    const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) out[i] = Io<T>::ld(in + i);
}

extern "C" int pta_widen(float* out, const void* in, long n, int dtype, void* stream) {
    PTA_REQUIRE(n > 0 && out && in, "widen: nothing to convert");
    hipStream_t s = (hipStream_t)stream;
    const dim3 grid((unsigned)((n + 255) / 256)), block(256);
    if (dtype == PTA_F32) hipLaunchKernelGGL(widen_kernel<float>, grid, block, 0, s, out, (const float*)in, n);
    else if (dtype == PTA_BF16) hipLaunchKernelGGL(widen_kernel<bf16_t>, grid, block, 0, s, out, (const bf16_t*)in, n);
    else return pta_fail("widen: unknown dtype %d", dtype);
    return pta_check_launch("widen");
}

__global__ void scale_kernel(float* __restrict__ x, float f, long n) {
    const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) x[i] *= f;
}

// in place: x *= f (32-bit)
extern "C" int pta_scale_f32(float* x, float f, long n, void* stream) {
    PTA_REQUIRE(n > 0 && x, "scale: nothing to scale");
    hipLaunchKernelGGL(scale_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, (hipStream_t)stream, x, f, n);
    return pta_check_launch("scale");
}
