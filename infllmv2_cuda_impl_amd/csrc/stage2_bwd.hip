// Stage-2 block-sparse attention backward for gfx950 (bf16, head_dim 128, 16 heads per KV head).
//
// Mathematics as in compute_dq_dk_dv_1colblock (csrc/flash_attn/src/flash_bwd_kernel.h:498-794)
// and compute_dot_do_o (flash_bwd_preprocess_kernel.h:56-137):
//   D = rowsum(dO * O);  P = exp(scale * S - LSE) on allowed entries;  dV = P^T dO;  dP = dO V^T;
//   dS = P * (dP - D);  dQ = scale * dS K;  dK = scale * dS^T Q;  P and dS are rounded to bf16
//   before the second GEMMs; the 16 grouped heads accumulate into their KV head's dK / dV.
//
// Accumulation strategy (differs from the reference, which runs one column-parallel kernel and
// sends every 16x128 dQ tile through fp32 atomics, 8 KiB per (token, block)):
//   * dQ: its own row-parallel kernel with the forward's schedule (stage2_bwd_dq.hip); S and dP
//     are recomputed, dQ stays in registers and is written once as bf16.  No dq scratch, no zero
//     fill, no conversion pass, bit-reproducible.
//   * dK/dV: column-parallel (stage2_bwd_dkdv.hip).  Two wavefronts own a 64-key block (32 keys each) and a
//     slice of 512 query tokens, walk the transposed mask, keep their 32x128 dK^T and dV^T tiles
//     in accumulation registers and flush once per slice with fp32 atomics.
// This file holds the preprocessing kernel, the fp32 -> bf16 conversion of dK/dV and the C entry
// point.
#include "common.h"
#include "kv_image.h"
#include "block_walker.h"
#include "stage2_bwd.h"
#include "infllmv2_hip.h"
#include <math.h>
#include <stdlib.h>

namespace IV2_NS {

// ---------------------------------------------------------------------------------------------
// preprocessing: D = rowsum(dO * O) (compute_dot_do_o, flash_bwd_preprocess_kernel.h:56-137) and, per token,
// the 32 row scalars the dK/dV kernel fetches with one 128-byte transfer
// ---------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256)
void bwd_prep_kernel(const BwdParams p) {
    // one 16-lane group per (token, head-in-group): 16 lanes x 8 elements = 128
    const int64_t tok = static_cast<int64_t>(blockIdx.x);
    const int h = blockIdx.y;
    const int tid = threadIdx.x;
    const int row = tid >> 4, part = tid & 15;
    const bool spare = row >= p.group;                         // a row that only fills the 16-row tiles of the other kernels
    const int rowc = spare ? p.group - 1 : row;
    const uint4 dv = *reinterpret_cast<const uint4*>(p.dout + tok * p.do_tok + h * p.do_kvh + rowc * p.do_grp + part * 8);
    const uint4 ov = *reinterpret_cast<const uint4*>(p.out + tok * p.o_tok + h * p.o_kvh + rowc * p.o_grp + part * 8);
    const uint32_t dw[4] = {dv.x, dv.y, dv.z, dv.w};
    const uint32_t ow[4] = {ov.x, ov.y, ov.z, ov.w};
    float acc = 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        acc += elem_to_f32(static_cast<elem_bits>(dw[i] & 0xffff)) * elem_to_f32(static_cast<elem_bits>(ow[i] & 0xffff));
        acc += elem_to_f32(static_cast<elem_bits>(dw[i] >> 16)) * elem_to_f32(static_cast<elem_bits>(ow[i] >> 16));
    }
#pragma unroll
    for (int off = 1; off < 16; off <<= 1) acc += __shfl_xor(acc, off);
    if (part == 0) {
        // spare rows get LSE = +inf and D = 0: their P = exp2(x - inf) and dS = P (dP - D) vanish in every kernel
        p.dsum[static_cast<int64_t>(h) * p.total_q * 16 + tok * 16 + row] = spare ? 0.f : acc;
        float* rs = p.rowstat + (static_cast<int64_t>(h) * p.total_q + tok) * 32;
        rs[row] = spare ? INFINITY : p.lse[h * p.lse_kvh + tok * p.lse_tok + row * p.lse_grp] * kLog2e;
        rs[16 + row] = spare ? 0.f : acc;
    }
}

__global__ __launch_bounds__(256)
void zero_f32_kernel(float4* __restrict__ ptr, int64_t n4) {
    const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < n4; i += stride)
        ptr[i] = make_float4(0.f, 0.f, 0.f, 0.f);
}

__global__ __launch_bounds__(256)
void bwd_convert_dkdv_kernel(const BwdParams p) {
    // one thread converts 4 consecutive d of one (row, head)
    const int64_t idx = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    const int64_t total = p.total_k * p.num_heads_k * (kHeadDim / 4);
    if (idx >= total) return;
    const int d4 = static_cast<int>(idx % (kHeadDim / 4));
    const int64_t rh = idx / (kHeadDim / 4);
    const int h = static_cast<int>(rh % p.num_heads_k);
    const int64_t row = rh / p.num_heads_k;
    const float4 a = *reinterpret_cast<const float4*>(p.dk_acc + rh * kHeadDim + d4 * 4);
    const float4 c = *reinterpret_cast<const float4*>(p.dv_acc + rh * kHeadDim + d4 * 4);
    uint2 ka, va;
    ka.x = pack_elem2(a.x, a.y); ka.y = pack_elem2(a.z, a.w);
    va.x = pack_elem2(c.x, c.y); va.y = pack_elem2(c.z, c.w);
    *reinterpret_cast<uint2*>(p.dk + row * p.dk_row + h * p.dk_head + d4 * 4) = ka;
    *reinterpret_cast<uint2*>(p.dv + row * p.dv_row + h * p.dv_head + d4 * 4) = va;
}

static size_t align256(size_t x) { return (x + 255) & ~static_cast<size_t>(255); }

struct BwdLayout {
    size_t images, mask, dsum, rowstat, dk_acc, dv_acc, total;
    size_t det_flags, det_slots, det_total;                    // deterministic mode only, after everything else
    int det_slices;
};

static BwdLayout bwd_layout(int batch, int64_t total_q, int64_t total_k, int num_heads_k, int max_seqlen_k) {
    BwdLayout L;
    size_t off = 0;
    L.images = off; off += align256(infllmv2_kv_image_bytes(total_k, batch, num_heads_k));   // K image | V in K-image order
    const int64_t k_blocks = (max_seqlen_k + kBlockN - 1) / kBlockN;
    L.mask = off; off += align256(static_cast<size_t>(num_heads_k) * k_blocks * ((total_q + 63) / 64) * 8);
    L.dsum = off; off += align256(static_cast<size_t>(num_heads_k) * total_q * 16 * 4);
    L.rowstat = off; off += align256(static_cast<size_t>(num_heads_k) * total_q * 32 * 4);
    L.dk_acc = off; off += align256(static_cast<size_t>(total_k) * num_heads_k * kHeadDim * 4);
    L.dv_acc = off; off += align256(static_cast<size_t>(total_k) * num_heads_k * kHeadDim * 4);
    L.total = off;
    L.det_slices = static_cast<int>((total_q + kDkdvSlice - 1) / kDkdvSlice) + 1;
    const size_t items = static_cast<size_t>(num_heads_k) * image_slots(total_k, batch) * L.det_slices;
    L.det_flags = off; off += align256(items * 4);
    L.det_slots = off; off += align256(items * 2 * kBlockN * kHeadDim * 4);
    L.det_total = off;
    return L;
}

}  // namespace IV2_NS

using namespace IV2_NS;

#ifndef IV2_F16        // both element types are 2 bytes wide: defined once
extern "C" size_t infllmv2_varlen_bwd_workspace_bytes(int batch, int64_t total_q, int64_t total_k, int num_heads_k,
                                                      int max_seqlen_k) {
    return bwd_layout(batch, total_q, total_k, num_heads_k, max_seqlen_k).total;
}

extern "C" size_t infllmv2_varlen_bwd_deterministic_workspace_bytes(int batch, int64_t total_q, int64_t total_k,
                                                                    int num_heads_k, int max_seqlen_k) {
    return bwd_layout(batch, total_q, total_k, num_heads_k, max_seqlen_k).det_total;
}

#endif

extern "C" int IV2_ENTRY(infllmv2_varlen_bwd)(void* stream, const void* dout, const void* q, const void* k, const void* v,
                                   const void* out, const float* softmax_lse, void* dq, void* dk, void* dv,
                                   const int32_t* cu_seqlens_q, const int32_t* cu_seqlens_k,
                                   const uint64_t* fwd_blockmask, void* workspace, size_t workspace_bytes, int batch,
                                   int64_t total_q, int64_t total_k, int num_heads, int num_heads_k, int head_dim,
                                   int max_seqlen_q, int max_seqlen_k, const int64_t* q_strides,
                                   const int64_t* k_strides, const int64_t* v_strides, const int64_t* o_strides,
                                   const int64_t* do_strides, const int64_t* dq_strides, const int64_t* dk_strides,
                                   const int64_t* dv_strides, const int64_t* lse_strides, int n_uint64_per_row,
                                   float softmax_scale, int is_causal, int deterministic) {
    IV2_CHECK(head_dim == kHeadDim, "varlen_bwd: this build only supports head_dim 128 (got %d)", head_dim);
    IV2_CHECK(valid_group(num_heads, num_heads_k),
              "varlen_bwd: requires num_heads == g * num_heads_k with g in {1, 2, 4, 8, 16} (got %d and %d)", num_heads, num_heads_k);
    IV2_CHECK(batch > 0 && total_q >= 0 && total_k >= 0 && max_seqlen_q >= 0 && max_seqlen_k >= 0, "varlen_bwd: bad sizes");
    IV2_CHECK(dout && q && k && v && out && softmax_lse && dq && dk && dv && cu_seqlens_q && cu_seqlens_k && workspace,
              "varlen_bwd: null pointer");
    IV2_CHECK(num_heads_k <= 65535 && batch <= 65535, "varlen_bwd: batch and num_heads_k must not exceed 65535");
    const BwdLayout L = bwd_layout(batch, total_q, total_k, num_heads_k, max_seqlen_k);
    const size_t ws_needed = deterministic ? L.det_total : L.total;
    IV2_CHECK(workspace_bytes >= ws_needed, "varlen_bwd: workspace too small (%zu < %zu)", workspace_bytes, ws_needed);
    IV2_CHECK(reinterpret_cast<uintptr_t>(workspace) % 256 == 0, "varlen_bwd: workspace must be 256-byte aligned");
    const void* ptrs16[] = {dout, q, k, v, out};
    for (const void* ptr16 : ptrs16) IV2_CHECK(reinterpret_cast<uintptr_t>(ptr16) % 16 == 0, "varlen_bwd: inputs must be 16-byte aligned");
    IV2_CHECK(reinterpret_cast<uintptr_t>(dq) % 8 == 0 && reinterpret_cast<uintptr_t>(dk) % 8 == 0 &&
              reinterpret_cast<uintptr_t>(dv) % 8 == 0, "varlen_bwd: gradients must be 8-byte aligned");
    for (int s = 0; s < 3; ++s)
        IV2_CHECK(q_strides[s] % 8 == 0 && o_strides[s] % 8 == 0 && do_strides[s] % 8 == 0 && dq_strides[s] % 4 == 0,
                  "varlen_bwd: q/out/dout strides must be multiples of 8 and dq strides of 4 elements");
    for (int s = 0; s < 2; ++s)
        IV2_CHECK(dk_strides[s] % 4 == 0 && dv_strides[s] % 4 == 0, "varlen_bwd: dk/dv strides must be multiples of 4 elements");
    IV2_CHECK(fwd_blockmask == nullptr || n_uint64_per_row > 0, "varlen_bwd: mask given without words per row");
    IV2_CHECK(softmax_scale > 0.f, "varlen_bwd: softmax_scale must be positive");
    hipStream_t st = static_cast<hipStream_t>(stream);
    unsigned char* ws = static_cast<unsigned char*>(workspace);

    BwdParams p{};
    p.q = static_cast<const elem_bits*>(q);
    p.dout = static_cast<const elem_bits*>(dout);
    p.out = static_cast<const elem_bits*>(out);
    p.dq = static_cast<elem_bits*>(dq);
    p.lse = softmax_lse;
    p.dsum = reinterpret_cast<float*>(ws + L.dsum);
    p.rowstat = reinterpret_cast<float*>(ws + L.rowstat);
    const int64_t n_slots = image_slots(total_k, batch);
    const int64_t img_elems = n_slots * num_heads_k * kImageElems;
    p.kimg = reinterpret_cast<const elem_bits*>(ws + L.images);
    p.vimg_r = p.kimg + img_elems;
    p.dk_acc = reinterpret_cast<float*>(ws + L.dk_acc);
    p.dv_acc = reinterpret_cast<float*>(ws + L.dv_acc);
    p.dk = static_cast<elem_bits*>(dk);
    p.dv = static_cast<elem_bits*>(dv);
    p.fwd_mask = fwd_blockmask;
    p.cu_seqlens_q = cu_seqlens_q; p.cu_seqlens_k = cu_seqlens_k;
    p.group = num_heads / num_heads_k;
    p.q_tok = q_strides[0]; p.q_grp = q_strides[1]; p.q_kvh = q_strides[2];
    p.do_tok = do_strides[0]; p.do_grp = do_strides[1]; p.do_kvh = do_strides[2];
    p.o_tok = o_strides[0]; p.o_grp = o_strides[1]; p.o_kvh = o_strides[2];
    p.dq_tok = dq_strides[0]; p.dq_grp = dq_strides[1]; p.dq_kvh = dq_strides[2];
    p.lse_tok = lse_strides[0]; p.lse_grp = lse_strides[1]; p.lse_kvh = lse_strides[2];
    p.dk_row = dk_strides[0]; p.dk_head = dk_strides[1]; p.dv_row = dv_strides[0]; p.dv_head = dv_strides[1];
    p.n_slots = n_slots; p.total_q = total_q; p.total_k = total_k;
    p.n64_fwd = n_uint64_per_row;
    p.n64_bwd = static_cast<int>((total_q + 63) / 64);
    p.k_blocks = (max_seqlen_k + kBlockN - 1) / kBlockN;
    p.num_heads_k = num_heads_k;
    p.scale = softmax_scale;
    p.scale_log2 = softmax_scale * kLog2e;

    if (deterministic) {
        p.det_flags = reinterpret_cast<uint32_t*>(ws + L.det_flags);
        p.det_slots = reinterpret_cast<float*>(ws + L.det_slots);
        p.det_slices = L.det_slices;
        hipLaunchKernelGGL(zero_f32_kernel, dim3(256), dim3(256), 0, st, reinterpret_cast<float4*>(p.det_flags),
                           static_cast<int64_t>((L.det_slots - L.det_flags) / 16));
        IV2_LAUNCH_CHECK();
    }
    // dK/dV accumulators start at zero (fill kernel, no memset node)
    if (total_k > 0) {
        const int64_t n4 = static_cast<int64_t>((L.dv_acc - L.dk_acc) / 16) * 2;
        IV2_CHECK((L.dv_acc - L.dk_acc) == align256(static_cast<size_t>(total_k) * num_heads_k * kHeadDim * 4), "varlen_bwd: layout");
        hipLaunchKernelGGL(zero_f32_kernel, dim3(2048), dim3(256), 0, st, reinterpret_cast<float4*>(p.dk_acc), n4);
        IV2_LAUNCH_CHECK();
    }
    if (total_q > 0 && max_seqlen_q > 0 && total_k > 0 && max_seqlen_k > 0) {
        int rc = launch_pack(st, k, v, cu_seqlens_k, ws + L.images, L.mask - L.images, batch, total_k, num_heads_k,
                             max_seqlen_k, k_strides, v_strides, true);   // K image | V in K-image order
        if (rc != 0) return rc;
        if (fwd_blockmask != nullptr) {
            uint64_t* bwd_mask = reinterpret_cast<uint64_t*>(ws + L.mask);
            rc = infllmv2_transpose_blockmask(stream, fwd_blockmask, bwd_mask, num_heads_k, total_q, n_uint64_per_row,
                                              p.k_blocks, p.n64_bwd);
            if (rc != 0) return rc;
            p.bwd_mask = bwd_mask;
        }
        IV2_CHECK(total_q <= 0x7fffffffll, "varlen_bwd: too many query tokens");
        hipLaunchKernelGGL(bwd_prep_kernel, dim3(static_cast<unsigned>(total_q), num_heads_k), dim3(256), 0, st, p);
        IV2_LAUNCH_CHECK();
        rc = launch_bwd_dq_hybrid(st, p, batch, max_seqlen_q, is_causal != 0);
        if (rc != 0) return rc;
        rc = launch_bwd_dkdv_wave(st, p, batch, max_seqlen_q, is_causal != 0);
        if (rc != 0) return rc;
        if (deterministic) {
            rc = launch_bwd_dkdv_reduce(st, p, batch);
            if (rc != 0) return rc;
        }
    } else if (total_q > 0) {
        // no keys at all: dq = 0
        IV2_CHECK(false, "varlen_bwd: empty key set is not supported");
    }
    if (total_k > 0) {
        const int64_t total = total_k * num_heads_k * (kHeadDim / 4);
        hipLaunchKernelGGL(bwd_convert_dkdv_kernel, dim3(static_cast<unsigned>((total + 255) / 256)), dim3(256), 0, st, p);
        IV2_LAUNCH_CHECK();
    }
    return 0;
}
