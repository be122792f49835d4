// Library-internal definition of the policy object (opaque in include/cfp.h).
#pragma once

#include "cfp_common.h"

struct cfp_policy {
    int n = 0;
    int layers = 0;
    int variant = 0;   // 0 full game, 1 classic
    size_t param_count = 0;
    float* params = nullptr;
    float* we_pk = nullptr;
    uint16_t* we_s3 = nullptr;    // map rows of W_enc split in three bf16 terms
    float* wg_pk = nullptr;
    float* wav_pk = nullptr;
    uint16_t* we_bf = nullptr;    // bf16 mirrors (MFMA 32x32x16 order)
    uint16_t* wg_bf = nullptr;
    uint16_t* wav_bf = nullptr;
    int gemm_bf16 = 0;            // forward entry points run the bf16-input kernel
    void* t16 = nullptr;          // mirrors of the 16-env-tile kernel (full game only)
    int small_tiles = 0;          // batches of at most 4096 envs run on 16-env tiles
    float* h_state = nullptr;
    uint8_t* rec = nullptr;
    float* h_enc = nullptr;
    float* h3 = nullptr;
    float* logits = nullptr;
    hipStream_t stream = nullptr;
};

namespace cfp {
// weight pointers, variant and action count of a policy into launch arguments
void fill_forward_weights(const cfp_policy* p, FwdArgs& a);
}  // namespace cfp
