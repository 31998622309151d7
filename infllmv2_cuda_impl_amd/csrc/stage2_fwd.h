// Parameters of the Stage-2 forward kernels.
#pragma once
#include "common.h"

namespace IV2_NS {

struct FwdParams {
    const elem_bits* q;
    elem_bits* out;
    float* lse;
    const elem_bits* kimg;
    const elem_bits* vimg;
    const int* cu_seqlens_q;
    const int* cu_seqlens_k;
    const uint64_t* mask;           // (Hk, total_q, n64) or null for dense
    int64_t q_tok_stride, q_grp_stride, q_kvh_stride;
    int64_t o_tok_stride, o_grp_stride, o_kvh_stride;
    int64_t lse_tok_stride, lse_grp_stride, lse_kvh_stride;
    int64_t n_slots;
    int64_t total_q;
    int n64;
    int group;                      // query heads per KV head, 1..16: MFMA rows >= group repeat head group - 1 and are never stored
    float scale_log2;               // softmax_scale * log2(e)
};

// Workgroup-hybrid forward (stage2_fwd_hybrid.hip): 8 consecutive tokens per workgroup stage the blocks they all
// select once in LDS and walk the rest of their rows one wavefront each.
int launch_stage2_fwd_hybrid(hipStream_t st, const FwdParams& p, int batch, int num_heads_k, int max_seqlen_q,
                             int max_seqlen_k, bool causal);

}  // namespace IV2_NS
