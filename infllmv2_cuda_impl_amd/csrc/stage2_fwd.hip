// Stage-2 block-sparse flash-attention forward for gfx950 (head_dim 128, up to 16 query heads per KV head): the
// K/V image pre-pass and the C entry point; the attention kernel itself is in stage2_fwd_hybrid.hip.
//
// Semantics follow compute_attn_1rowblock (csrc/flash_attn/src/flash_fwd_kernel.h:137-602) with
// the bitmask walk of flash_blockmask.h:5-100: token i of a sequence attends key t iff
// t <= i + Sk - Sq (causal, bottom-right aligned), t < Sk, and bit t/64 of its mask row is set;
// O = softmax(scale * q.K^T) V with fp32 softmax and P rounded to bf16 before P.V; rows with no
// allowed key give O = 0 and LSE = +inf (softmax.h:240-256).
//
// Design (not the reference's): the 16 grouped heads of one token form the 16-column N side of
// v_mfma_f32_16x16x32_bf16.  S^T = K.Q^T puts keys on the M side, so one lane owns one head's
// scores for 16 keys and the same registers, converted to bf16, are the B operand of
// O^T = V^T.P^T.  K and V come from fragment-major block images (kv_image.h) built by
// pack_kv_kernel, so every operand fetch is one contiguous 1 KiB wavefront load.  Q, O and the
// LSE are addressed through strides: the caller's (T, Hq, d) tensors are used in place.
#include "common.h"
#include "kv_image.h"
#include "block_walker.h"
#include "stage2_fwd.h"
#include "infllmv2_hip.h"
#include <math.h>

namespace IV2_NS {

// ---------------------------------------------------------------------------------------------
// K/V -> block images
// ---------------------------------------------------------------------------------------------
struct PackParams {
    const elem_bits* k;
    const elem_bits* v;
    elem_bits* kimg;                // K in K-image order (operand of a GEMM contracting over d)
    elem_bits* vimg;                // forward: V in V-image order (A operand of a GEMM contracting over keys), else null
    elem_bits* vimg_r;              // backward: V in K-image order (dP = dO V^T contracts over d), else null
    const int* cu_seqlens_k;
    int64_t k_row_stride, k_head_stride;
    int64_t v_row_stride, v_head_stride;
    int64_t n_slots;
};

constexpr int kVPad = 8;            // LDS row padding (elements) for the V transposition

__global__ __launch_bounds__(256)
void pack_kv_kernel(const PackParams p) {
    __shared__ __attribute__((aligned(16))) elem_bits vt[kBlockN][kHeadDim + kVPad];
    const int j = blockIdx.x, b = blockIdx.y, h = blockIdx.z;
    const int k0 = p.cu_seqlens_k[b];
    const int Sk = p.cu_seqlens_k[b + 1] - k0;
    if (static_cast<int64_t>(j) * kBlockN >= Sk) return;
    const int64_t slot = image_slot0(p.cu_seqlens_k, b) + j;
    const int tid = threadIdx.x;
    const elem_bits* kb = p.k + (k0 + static_cast<int64_t>(j) * kBlockN) * p.k_row_stride + h * p.k_head_stride;
    const elem_bits* vb = p.v + (k0 + static_cast<int64_t>(j) * kBlockN) * p.v_row_stride + h * p.v_head_stride;
    const int64_t img_off = (static_cast<int64_t>(h) * p.n_slots + slot) * kImageElems;
    const int valid = Sk - j * kBlockN;                       // keys of this block inside the sequence
    const uint4 zero = make_uint4(0, 0, 0, 0);

    for (int u = tid; u < 1024; u += 256) {
        const int kt = u >> 8, c = (u >> 6) & 3, lane = u & 63;
        const int r = lane & 15, g = lane >> 4;
        const int key = 16 * kt + r;
        uint4 val = zero;
        if (key < valid) val = *reinterpret_cast<const uint4*>(kb + key * p.k_row_stride + 32 * c + 8 * g);
        *reinterpret_cast<uint4*>(p.kimg + img_off + u * 8) = val;
        if (p.vimg_r != nullptr) {
            uint4 vv = zero;
            if (key < valid) vv = *reinterpret_cast<const uint4*>(vb + key * p.v_row_stride + 32 * c + 8 * g);
            *reinterpret_cast<uint4*>(p.vimg_r + img_off + u * 8) = vv;
        }
    }
    // the image that contracts over the keys: V for the forward
    if (p.vimg == nullptr) return;                            // uniform per workgroup
    __syncthreads();
    for (int u = tid; u < 1024; u += 256) {
        const int key = u >> 4, d0 = (u & 15) * 8;
        uint4 val = zero;
        if (key < valid) val = *reinterpret_cast<const uint4*>(vb + key * p.v_row_stride + d0);
        *reinterpret_cast<uint4*>(&vt[key][d0]) = val;
    }
    __syncthreads();
    for (int u = tid; u < 1024; u += 256) {
        const int dt = u >> 7, cc = (u >> 6) & 1, lane = u & 63;
        const int r = lane & 15, g = lane >> 4;
        const int d = 16 * dt + r;
        uint32_t w[4];
#pragma unroll
        for (int jj = 0; jj < 8; jj += 2) {
            const int key_a = 32 * cc + (jj < 4 ? 4 * g + jj : 16 + 4 * g + jj - 4);
            w[jj >> 1] = static_cast<uint32_t>(vt[key_a][d]) | (static_cast<uint32_t>(vt[key_a + 1][d]) << 16);
        }
        *reinterpret_cast<uint4*>(p.vimg + img_off + u * 8) = make_uint4(w[0], w[1], w[2], w[3]);
    }
}

}  // namespace IV2_NS

using namespace IV2_NS;

#ifndef IV2_F16        // both element types are 2 bytes wide: defined once
extern "C" size_t infllmv2_kv_image_bytes(int64_t total_k, int batch, int num_heads_k) {
    return static_cast<size_t>(image_slots(total_k, batch)) * num_heads_k * kImageElems * sizeof(elem_bits) * 2;
}
#endif

namespace IV2_NS {
int launch_pack(hipStream_t st, const void* k, const void* v, const int32_t* cu_seqlens_k, void* workspace,
                size_t workspace_bytes, int batch, int64_t total_k, int num_heads_k, int max_seqlen_k,
                const int64_t* k_strides, const int64_t* v_strides, bool backward_images) {
    IV2_CHECK(k && v && cu_seqlens_k && workspace, "pack_kv: null pointer");
    IV2_CHECK(batch > 0 && num_heads_k > 0 && total_k >= 0 && max_seqlen_k >= 0, "pack_kv: bad sizes");
    IV2_CHECK(num_heads_k <= 65535 && batch <= 65535, "pack_kv: batch and num_heads_k must not exceed 65535");
    IV2_CHECK(workspace_bytes >= infllmv2_kv_image_bytes(total_k, batch, num_heads_k), "pack_kv: workspace too small");
    IV2_CHECK(reinterpret_cast<uintptr_t>(k) % 16 == 0 && reinterpret_cast<uintptr_t>(v) % 16 == 0 &&
              reinterpret_cast<uintptr_t>(workspace) % 16 == 0, "pack_kv: k, v and workspace must be 16-byte aligned");
    IV2_CHECK(k_strides[0] % 8 == 0 && k_strides[1] % 8 == 0 && v_strides[0] % 8 == 0 && v_strides[1] % 8 == 0,
              "pack_kv: k/v row and head strides must be multiples of 8 elements");
    const int64_t n_slots = image_slots(total_k, batch);
    const int max_blocks = (max_seqlen_k + kBlockN - 1) / kBlockN;
    if (max_blocks == 0 || total_k == 0) return 0;
    PackParams pp{};
    pp.k = static_cast<const elem_bits*>(k);
    pp.v = static_cast<const elem_bits*>(v);
    pp.kimg = static_cast<elem_bits*>(workspace);
    elem_bits* second = pp.kimg + n_slots * num_heads_k * kImageElems;
    if (backward_images) pp.vimg_r = second; else pp.vimg = second;
    pp.cu_seqlens_k = cu_seqlens_k;
    pp.k_row_stride = k_strides[0]; pp.k_head_stride = k_strides[1];
    pp.v_row_stride = v_strides[0]; pp.v_head_stride = v_strides[1];
    pp.n_slots = n_slots;
    hipLaunchKernelGGL(pack_kv_kernel, dim3(max_blocks, batch, num_heads_k), dim3(256), 0, st, pp);
    IV2_LAUNCH_CHECK();
    return 0;
}
}  // namespace IV2_NS

#ifndef IV2_F16        // the images are a permutation of 2-byte elements: one entry point serves both element types
extern "C" int infllmv2_pack_kv(void* stream, const void* k, const void* v, const int32_t* cu_seqlens_k,
                                void* workspace, size_t workspace_bytes, int batch, int64_t total_k,
                                int num_heads_k, int head_dim, int max_seqlen_k, const int64_t* k_strides,
                                const int64_t* v_strides) {
    IV2_CHECK(head_dim == kHeadDim, "pack_kv: this build only supports head_dim 128 (got %d)", head_dim);
    return launch_pack(static_cast<hipStream_t>(stream), k, v, cu_seqlens_k, workspace, workspace_bytes, batch,
                       total_k, num_heads_k, max_seqlen_k, k_strides, v_strides, false);
}
#endif

extern "C" int IV2_ENTRY(infllmv2_varlen_fwd)(void* stream, const void* q, const void* k, const void* v, void* out,
                                   float* softmax_lse, const int32_t* cu_seqlens_q, const int32_t* cu_seqlens_k,
                                   const uint64_t* blockmask, void* workspace, size_t workspace_bytes,
                                   int kv_prepacked, int batch, int64_t total_q, int64_t total_k, int num_heads,
                                   int num_heads_k, int head_dim, int max_seqlen_q, int max_seqlen_k,
                                   const int64_t* q_strides, const int64_t* k_strides, const int64_t* v_strides,
                                   const int64_t* o_strides, const int64_t* lse_strides,
                                   int n_uint64_per_row, float softmax_scale, int is_causal) {
    IV2_CHECK(head_dim == kHeadDim, "varlen_fwd: this build only supports head_dim 128 (got %d)", head_dim);
    IV2_CHECK(valid_group(num_heads, num_heads_k),
              "varlen_fwd: requires num_heads == g * num_heads_k with g in {1, 2, 4, 8, 16} (got %d and %d)", num_heads, num_heads_k);
    IV2_CHECK(batch > 0 && total_q >= 0 && total_k >= 0 && max_seqlen_q >= 0 && max_seqlen_k >= 0, "varlen_fwd: bad sizes");
    IV2_CHECK(q && out && softmax_lse && cu_seqlens_q && cu_seqlens_k && workspace, "varlen_fwd: null pointer");
    IV2_CHECK(num_heads_k <= 65535 && batch <= 65535, "varlen_fwd: batch and num_heads_k must not exceed 65535");
    IV2_CHECK(workspace_bytes >= infllmv2_kv_image_bytes(total_k, batch, num_heads_k), "varlen_fwd: workspace too small");
    IV2_CHECK(reinterpret_cast<uintptr_t>(q) % 16 == 0 && reinterpret_cast<uintptr_t>(out) % 8 == 0 &&
              reinterpret_cast<uintptr_t>(workspace) % 16 == 0, "varlen_fwd: q and workspace must be 16-byte aligned, out 8-byte");
    for (int s = 0; s < 3; ++s) {
        IV2_CHECK(q_strides[s] % 8 == 0 && o_strides[s] % 4 == 0, "varlen_fwd: q strides must be multiples of 8 and out strides of 4 elements");
    }
    IV2_CHECK(blockmask == nullptr || n_uint64_per_row > 0, "varlen_fwd: mask given without words per row");
    IV2_CHECK(softmax_scale > 0.f, "varlen_fwd: softmax_scale must be positive");
    if (total_q == 0 || max_seqlen_q == 0) return 0;
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (!kv_prepacked) {
        int rc = launch_pack(st, k, v, cu_seqlens_k, workspace, workspace_bytes, batch, total_k, num_heads_k,
                             max_seqlen_k, k_strides, v_strides, false);
        if (rc != 0) return rc;
    }
    const int64_t n_slots = image_slots(total_k, batch);
    FwdParams fp{};
    fp.q = static_cast<const elem_bits*>(q);
    fp.out = static_cast<elem_bits*>(out);
    fp.lse = softmax_lse;
    fp.kimg = static_cast<const elem_bits*>(workspace);
    fp.vimg = fp.kimg + n_slots * num_heads_k * kImageElems;
    fp.cu_seqlens_q = cu_seqlens_q; fp.cu_seqlens_k = cu_seqlens_k;
    fp.mask = blockmask;
    fp.q_tok_stride = q_strides[0]; fp.q_grp_stride = q_strides[1]; fp.q_kvh_stride = q_strides[2];
    fp.o_tok_stride = o_strides[0]; fp.o_grp_stride = o_strides[1]; fp.o_kvh_stride = o_strides[2];
    fp.lse_tok_stride = lse_strides[0]; fp.lse_grp_stride = lse_strides[1]; fp.lse_kvh_stride = lse_strides[2];
    fp.n_slots = n_slots;
    fp.total_q = total_q;
    fp.group = num_heads / num_heads_k;
    fp.n64 = n_uint64_per_row;
    fp.scale_log2 = softmax_scale * 1.44269504088896340736f;
    return launch_stage2_fwd_hybrid(st, fp, batch, num_heads_k, max_seqlen_q, max_seqlen_k, is_causal != 0);
}
