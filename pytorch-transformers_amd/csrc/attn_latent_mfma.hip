// Entry points of the latent attention on the matrix cores: the choice of a size class, and the merge of the
// partial results that a decode step's key ranges leave.
#include "attn_latent_mfma.h"

// (pieces of 32 elements of a cache row, tiles of 16 elements of its value part) that are built, smallest first
static const int LAT_CLASSES[][2] = {{2, 2}, {2, 4}, {3, 4}, {4, 4}, {4, 8}, {6, 8}, {8, 8}, {8, 16}, {12, 16}, {20, 32}};

static bool latent_class(int D, int R, int* dkc, int* rt) {
    for (const auto& c : LAT_CLASSES)
        if (c[0] * 32 >= D && c[1] * 16 >= R) {
            *dkc = c[0], *rt = c[1];
            return true;
        }
    return false;
}

// 1 if a kernel is built for cache rows of D elements whose first R are the value
extern "C" int pta_attn_latent_mfma_ok(int R, int D) {
    int dkc, rt;
    return R > 0 && D >= R && latent_class(D, R, &dkc, &rt) ? 1 : 0;
}

// out[row, :] = sum_s po[row, s, :] e^(pm[row, s] - m) / sum_s pl[row, s] e^(pm[row, s] - m), m = max_s pm[row, s];
// splits in order.  One workgroup per row (a token's head); the splits' weights are formed once, in LDS.
#define LAT_MAX_SPLITS 1024

__global__ void latent_combine_kernel(float* __restrict__ out, const float* __restrict__ po, const float* __restrict__ pm,
                                      const float* __restrict__ pl, int n_splits, int R) {
    __shared__ float w_s[LAT_MAX_SPLITS];
    __shared__ float red[16];
    const long row = blockIdx.x;
    const float* m_row = pm + row * n_splits;
    float m = -INFINITY;
    for (int s = threadIdx.x; s < n_splits; s += blockDim.x) m = fmaxf(m, m_row[s]);
    m = block_max(m, red);
    float denom = 0.f;
    for (int s = threadIdx.x; s < n_splits; s += blockDim.x) {
        const float w = m_row[s] == -INFINITY ? 0.f : expf(m_row[s] - m);
        w_s[s] = w;
        denom += pl[row * n_splits + s] * w;
    }
    denom = block_sum(denom, red);  // (its barriers also publish w_s)
    const float inv = 1.0f / denom;
    const float* prow = po + row * n_splits * R;
    for (int el = threadIdx.x; el < R; el += blockDim.x) {
        float acc = 0.f;
        int s = 0;
        for (; s + 4 <= n_splits; s += 4) {
            const float a0 = prow[(long)s * R + el], a1 = prow[(long)(s + 1) * R + el], a2 = prow[(long)(s + 2) * R + el],
                        a3 = prow[(long)(s + 3) * R + el];
            acc += a0 * w_s[s];
            acc += a1 * w_s[s + 1];
            acc += a2 * w_s[s + 2];
            acc += a3 * w_s[s + 3];
        }
        for (; s < n_splits; ++s) acc += prow[(long)s * R + el] * w_s[s];
        out[row * R + el] = acc * inv;
    }
}

extern "C" int pta_attn_latent_mfma(float* out, float* po, float* pm, float* pl, const float* q, const void* k_pool,
                                    const int* block_table, int bt_stride, const int* cu_tokens, const int* seq_start,
                                    int n_seqs, int max_new, int M, int H, int R, int dr, float scale, int split_size,
                                    int n_splits, void* stream) {
    PTA_REQUIRE(M > 0 && n_seqs > 0 && max_new > 0 && H > 0 && R > 0 && dr >= 0, "attn_latent_mfma: sizes must be positive");
    PTA_REQUIRE(out && q && k_pool && block_table && cu_tokens && seq_start, "attn_latent_mfma: null pointer");
    PTA_REQUIRE(n_splits >= 1 && n_splits <= LAT_MAX_SPLITS && n_seqs <= 65535, "attn_latent_mfma: too many key ranges or sequences");
    PTA_REQUIRE(n_splits == 1 || (po && pm && pl && split_size > 0 && split_size % LAT_KB == 0),
                "attn_latent_mfma: key ranges need room for partial results and a size that is a multiple of %d", LAT_KB);
    PTA_REQUIRE(n_splits == 1 || max_new == 1, "attn_latent_mfma: key ranges are for steps of one token per sequence");
    int dkc = 0, rt = 0;
    PTA_REQUIRE(latent_class(R + dr, R, &dkc, &rt), "attn_latent_mfma: no kernel for rows of %d elements with %d of value", R + dr, R);
    hipStream_t s = (hipStream_t)stream;
    LatentArgs a;
    a.out = out, a.po = po, a.pm = pm, a.pl = pl, a.q = q, a.k_pool = (const bf16_t*)k_pool;
    a.block_table = block_table, a.bt_stride = bt_stride, a.cu_tokens = cu_tokens, a.seq_start = seq_start;
    a.H = H, a.R = R, a.D = R + dr, a.scale = scale, a.split_size = split_size, a.n_splits = n_splits;
    const long max_rows = (long)max_new * H;
    PTA_REQUIRE(max_rows < (1L << 31), "attn_latent_mfma: too many columns in a sequence");
    int rc;
    if (dkc <= 4) rc = latent_mfma_small(dkc, rt, a, n_seqs, (int)max_rows, s);
    else if (dkc <= 8) rc = latent_mfma_mid(dkc, rt, a, n_seqs, (int)max_rows, s);
    else rc = latent_mfma_large(dkc, rt, a, n_seqs, (int)max_rows, s);
    if (rc) return rc;
    if (n_splits > 1) {
        hipLaunchKernelGGL(latent_combine_kernel, dim3((unsigned)((long)M * H)), dim3(R > 64 ? 256 : 64), 0, s, out, po, pm, pl,
                           n_splits, R);
        return pta_check_launch("latent_combine");
    }
    return 0;
}
