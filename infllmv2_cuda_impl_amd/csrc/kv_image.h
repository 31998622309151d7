// Fragment-major K/V block images.
//
// Stage-2 kernels never read K or V in the caller's (token, head, d) layout.  A pre-pass
// rewrites every 64-key block of one KV head into two 16 KiB "images" whose 16-byte units are
// already the per-lane operands of v_mfma_f32_16x16x32_bf16, so a wavefront fetches one MFMA
// operand with a single fully-coalesced 1 KiB load (global) or a conflict-free ds_read_b128
// (LDS copy of the image).  With lane = 16*g + r (r = lane % 16, g = lane / 16):
//
//   K image  unit (kt, c, lane), kt,c in [0,4):   8 x bf16  K[key = 16*kt + r][d = 32*c + 8*g + j]
//            = A operand of  S^T(16 keys x 16 heads) += K(16 x 32) * Q^T(32 x 16)
//   V image  unit (dt, cc, lane), dt in [0,8), cc in [0,2):
//            8 x bf16  V[key = 32*cc + (j < 4 ? 4*g + j : 16 + 4*g + j - 4)][d = 16*dt + r]
//            = A operand of  O^T(16 d x 16 heads) += V^T(16 x 32) * P^T(32 x 16)
//            where the key order inside a 32-key chunk is exactly the order in which one lane
//            holds two S^T accumulator tiles, so P needs no data movement between the GEMMs.
//
// Keys past the end of a sequence are stored as zeros.  Block `j` of packed sequence `b` lives in
// slot  cu_seqlens_k[b] / 64 + b + j  (a bound that never overlaps and needs no host sync).
#pragma once
#include "common.h"

namespace IV2_NS {

constexpr int kImageElems = kBlockN * kHeadDim;            // 8192 bf16 = 16 KiB per image

__host__ __device__ inline int64_t image_slots(int64_t total_k, int batch) {
    return total_k / kBlockN + batch + 1;
}

__device__ __forceinline__ int64_t image_slot0(const int* cu_seqlens_k, int b) {
    return cu_seqlens_k[b] / kBlockN + b;
}

// Launches the packing pre-pass.  workspace receives [K image | V image] for the forward or, with
// backward_images, [K image | V in K-image order] (the backward contracts V over d, and reads K^T out of the
// K image by transposed LDS loads).
int launch_pack(hipStream_t st, const void* k, const void* v, const int32_t* cu_seqlens_k, void* workspace,
                size_t workspace_bytes, int batch, int64_t total_k, int num_heads_k, int max_seqlen_k,
                const int64_t* k_strides, const int64_t* v_strides, bool backward_images);

}  // namespace IV2_NS
