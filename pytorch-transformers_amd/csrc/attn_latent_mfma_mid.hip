#include "attn_latent_mfma.h"

int latent_mfma_mid(int dkc, int rt, const LatentArgs& a, int n_seqs, int max_rows, hipStream_t s) {
    if (dkc == 6 && rt == 8) return launch_latent_mfma<6, 8>(a, n_seqs, max_rows, s);
    if (dkc == 8 && rt == 8) return launch_latent_mfma<8, 8>(a, n_seqs, max_rows, s);
    if (dkc == 8 && rt == 16) return launch_latent_mfma<8, 16>(a, n_seqs, max_rows, s);
    return pta_fail("attn_latent_mfma: no kernel for %d pieces of a row and %d value tiles", dkc, rt);
}
