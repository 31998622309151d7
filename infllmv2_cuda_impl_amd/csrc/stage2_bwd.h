// Parameters shared by the Stage-2 backward kernels.
#pragma once
#include "common.h"

namespace IV2_NS {

constexpr float kLog2e = 1.44269504088896340736f;

struct BwdParams {
    const elem_bits* q;
    const elem_bits* dout;
    const elem_bits* out;
    elem_bits* dq;
    const float* lse;
    float* dsum;                    // (Hk, total_q * 16): D of head 16h+g of token t at [h][16 t + g]
    float* rowstat;                 // (Hk, total_q, 32): LSE * log2(e) of the 16 heads, then D of the 16 heads
    const elem_bits* kimg;          // K, K-image order
    const elem_bits* vimg_r;        // V, K-image order
    float* dk_acc;                  // (total_k, Hk, 128) fp32
    float* dv_acc;
    elem_bits* dk;
    elem_bits* dv;
    const uint64_t* fwd_mask;       // (Hk, total_q, n64_fwd) or null
    const uint64_t* bwd_mask;       // (Hk, k_blocks, n64_bwd) or null
    const int* cu_seqlens_q;
    const int* cu_seqlens_k;
    int64_t q_tok, q_grp, q_kvh;    // element strides {token, head-in-group, kv-head}
    int64_t do_tok, do_grp, do_kvh;
    int64_t o_tok, o_grp, o_kvh;
    int64_t dq_tok, dq_grp, dq_kvh;
    int64_t lse_tok, lse_grp, lse_kvh;
    int64_t dk_row, dk_head, dv_row, dv_head;
    int64_t n_slots, total_q, total_k;
    int n64_fwd, n64_bwd, k_blocks, num_heads_k;
    int group;                      // query heads per KV head, 1..16: rows >= group repeat head group - 1 with LSE = +inf (P = dS = 0)
    float scale_log2, scale;
    // deterministic dK/dV: every (block, 512-token slice) work item stores its two tiles in a slot of its own and a
    // second kernel adds the slots of a block in slice order (no atomics); null: fp32 atomics into dk_acc / dv_acc
    float* det_slots;               // (Hk, n_slots, det_slices, 2, 64, 128) fp32
    uint32_t* det_flags;            // (Hk, n_slots, det_slices): 1 where a slot was written
    int det_slices;
    int dkdv_spread;                // dK/dV work items: 1 = all XCDs share every slice (few slices), 0 = an XCD owns whole slice groups
};

// dQ, 8 consecutive tokens per workgroup sharing their common blocks through LDS: stage2_bwd_dq.hip
int launch_bwd_dq_hybrid(hipStream_t st, const BwdParams& p, int batch, int max_seqlen_q, bool causal);
// dK/dV, two wavefronts (32 keys each) per (64-key block, 512-token slice): stage2_bwd_dkdv.hip
int launch_bwd_dkdv_wave(hipStream_t st, const BwdParams& p, int batch, int max_seqlen_q, bool causal);

// deterministic mode only: adds the slots of every key block in slice order into dk_acc / dv_acc
int launch_bwd_dkdv_reduce(hipStream_t st, const BwdParams& p, int batch);
// Query tokens per dK/dV work item (slices are cut on the packed token axis).  Long inputs use 512-token slices (one
// flush of the accumulators per 512 tokens); short ones 128, so that a few thousand tokens still make enough work
// items to fill the device; the deterministic mode, whose workspace grows with the slice count, keeps 512.
constexpr int kDkdvSlice = 512;
constexpr int kDkdvSliceSmall = 128;
inline int dkdv_slice_tokens(int64_t total_q, bool deterministic) {
    return (total_q <= 8192 && !deterministic) ? kDkdvSliceSmall : kDkdvSlice;   // deterministic mode: one slot per slice, so few slices
}

}  // namespace IV2_NS
