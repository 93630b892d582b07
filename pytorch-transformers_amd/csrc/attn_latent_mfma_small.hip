#include "attn_latent_mfma.h"

int latent_mfma_small(int dkc, int rt, const LatentArgs& a, int n_seqs, int max_rows, hipStream_t s) {
    if (dkc == 2 && rt == 2) return launch_latent_mfma<2, 2>(a, n_seqs, max_rows, s);
    if (dkc == 2 && rt == 4) return launch_latent_mfma<2, 4>(a, n_seqs, max_rows, s);
    if (dkc == 3 && rt == 4) return launch_latent_mfma<3, 4>(a, n_seqs, max_rows, s);
    if (dkc == 4 && rt == 4) return launch_latent_mfma<4, 4>(a, n_seqs, max_rows, s);
    if (dkc == 4 && rt == 8) return launch_latent_mfma<4, 8>(a, n_seqs, max_rows, s);
    return pta_fail("attn_latent_mfma: no kernel for %d pieces of a row and %d value tiles", dkc, rt);
}
