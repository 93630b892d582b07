#include "attn_latent_mfma.h"

int latent_mfma_large(int dkc, int rt, const LatentArgs& a, int n_seqs, int max_rows, hipStream_t s) {
    if (dkc == 12 && rt == 16) return launch_latent_mfma<12, 16>(a, n_seqs, max_rows, s);
    if (dkc == 20 && rt == 32) return launch_latent_mfma<20, 32>(a, n_seqs, max_rows, s);
    return pta_fail("attn_latent_mfma: no kernel for %d pieces of a row and %d value tiles", dkc, rt);
}
