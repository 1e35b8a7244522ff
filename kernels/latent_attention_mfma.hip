// MFMA prompt-portion kernel for latent attention (bf16).  Placeholder until
// the tiled kernel lands: reports "not usable", so the general kernel runs.

#include "common.h"

bool latent_prefill_mfma_usable(int rank, int rot, int block_size) {
  (void)rank; (void)rot; (void)block_size;
  return false;
}

void launch_latent_prefill_mfma(__hip_bfloat16*, long, long,
                                const __hip_bfloat16*, long, long,
                                const __hip_bfloat16*, long, long,
                                const __hip_bfloat16*, const int*, int,
                                const int*, const int*, int, const float*,
                                float, int, int, int, int, int, int,
                                hipStream_t) {}
