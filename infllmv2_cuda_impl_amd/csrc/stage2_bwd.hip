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
//   * dQ: its own row-parallel kernel with the forward's schedule (one wavefront per token walks
//     the token's mask row); S and dP are recomputed, dQ stays in registers and is written once
//     as bf16.  No dq scratch, no zero fill, no conversion pass, bit-reproducible.
//   * dK/dV: column-parallel.  A workgroup owns one 64-key block and a slice of 2048 query
//     tokens; it walks the transposed mask and keeps the 64x128 dK^T and dV^T tiles in accumulator
//     registers (8 wavefronts = 4 disjoint token streams x 2 key halves), reduces the streams
//     through LDS and flushes once per slice with fp32 atomics, so atomic traffic is one
//     64 KiB tile per >= 100 tokens instead of 8 KiB per (token, block).  Slicing bounds the work
//     of a workgroup: block 0 and the local window are selected by every token.
//   * S = Q K^T is formed with the 16 heads of a token as MFMA rows; two tokens fill the 32-deep
//     contraction of the transposed GEMMs, and their accumulator registers are, unchanged, the B
//     operand (no movement of P or dS).  The matching A operands dO^T and Q^T come from per-token
//     transposed images written by the preprocessing kernel.
#include "common.h"
#include "kv_image.h"
#include "block_walker.h"
#include "stage2_bwd.h"
#include "../../include/infllmv2_hip.h"
#include <math.h>
#include <stdlib.h>

namespace infllmv2 {

// ---------------------------------------------------------------------------------------------
// preprocessing: D = rowsum(dO * O) and the transposed per-token images of Q and dO
// ---------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256)
void bwd_prep_kernel(const BwdParams p) {
    __shared__ bf16_bits tq[16][kHeadDim + 8];
    __shared__ bf16_bits tdo[16][kHeadDim + 8];
    const int64_t tok = blockIdx.x;
    const int h = blockIdx.y;
    const int tid = threadIdx.x;
    const int row = tid >> 4, part = tid & 15;                 // head-in-group, 8-element column chunk
    const uint4 qv = *reinterpret_cast<const uint4*>(p.q + tok * p.q_tok + h * p.q_kvh + row * p.q_grp + part * 8);
    const uint4 dv = *reinterpret_cast<const uint4*>(p.dout + tok * p.do_tok + h * p.do_kvh + row * p.do_grp + part * 8);
    const uint4 ov = *reinterpret_cast<const uint4*>(p.out + tok * p.o_tok + h * p.o_kvh + row * p.o_grp + part * 8);
    *reinterpret_cast<uint4*>(&tq[row][part * 8]) = qv;
    *reinterpret_cast<uint4*>(&tdo[row][part * 8]) = dv;
    {
        const int unit = (part >> 2) * 64 + (part & 3) * 16 + row;            // chunk c = part / 4, k-group g = part % 4
        const int64_t base = (static_cast<int64_t>(h) * p.total_q + tok) * kTImageElems + unit * 8;
        *reinterpret_cast<uint4*>(p.qF + base) = qv;
        *reinterpret_cast<uint4*>(p.doF + base) = dv;
    }
    const uint32_t dw[4] = {dv.x, dv.y, dv.z, dv.w};
    const uint32_t ow[4] = {ov.x, ov.y, ov.z, ov.w};
    float acc = 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        acc += bf16_to_f32(static_cast<bf16_bits>(dw[i] & 0xffff)) * bf16_to_f32(static_cast<bf16_bits>(ow[i] & 0xffff));
        acc += bf16_to_f32(static_cast<bf16_bits>(dw[i] >> 16)) * bf16_to_f32(static_cast<bf16_bits>(ow[i] >> 16));
    }
#pragma unroll
    for (int off = 1; off < 16; off <<= 1) acc += __shfl_xor(acc, off);
    if (part == 0) {
        p.dsum[static_cast<int64_t>(h) * p.total_q * 16 + tok * 16 + row] = acc;
        float* rs = p.rowstat + (static_cast<int64_t>(h) * p.total_q + tok) * 32;
        rs[row] = p.lse[h * p.lse_kvh + tok * p.lse_tok + row * p.lse_grp] * kLog2e;
        rs[16 + row] = acc;
    }
    __syncthreads();
    bf16_bits* qdst = p.qT + (static_cast<int64_t>(h) * p.total_q + tok) * kTImageElems;
    bf16_bits* ddst = p.doT + (static_cast<int64_t>(h) * p.total_q + tok) * kTImageElems;
    for (int u = tid; u < 512; u += 256) {
        const int dt = u >> 6, lane = u & 63;
        const int r = lane & 15, g = lane >> 4;
        const int d = 16 * dt + r;
        uint2 a, b;
        a.x = static_cast<uint32_t>(tq[4 * g][d]) | (static_cast<uint32_t>(tq[4 * g + 1][d]) << 16);
        a.y = static_cast<uint32_t>(tq[4 * g + 2][d]) | (static_cast<uint32_t>(tq[4 * g + 3][d]) << 16);
        b.x = static_cast<uint32_t>(tdo[4 * g][d]) | (static_cast<uint32_t>(tdo[4 * g + 1][d]) << 16);
        b.y = static_cast<uint32_t>(tdo[4 * g + 2][d]) | (static_cast<uint32_t>(tdo[4 * g + 3][d]) << 16);
        *reinterpret_cast<uint2*>(qdst + u * 4) = a;
        *reinterpret_cast<uint2*>(ddst + u * 4) = b;
    }
}

// ---------------------------------------------------------------------------------------------
// dQ: one wavefront per token, same walk as the forward
// ---------------------------------------------------------------------------------------------
template <bool kCausal>
__global__ __launch_bounds__(256)
void bwd_dq_kernel(const BwdParams p) {
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int b = blockIdx.y, h = blockIdx.z;
    const int i = blockIdx.x * 4 + wave;
    const int q0 = p.cu_seqlens_q[b];
    const int Sq = p.cu_seqlens_q[b + 1] - q0;
    if (i >= Sq) return;                                        // uniform per wavefront; no barriers below
    const int Sk = p.cu_seqlens_k[b + 1] - p.cu_seqlens_k[b];
    const int64_t tok = static_cast<int64_t>(q0) + i;
    const int n = lane & 15, g = lane >> 4;

    bf16x8 qf[4], dof[4];
    {
        const bf16_bits* qp = p.q + tok * p.q_tok + h * p.q_kvh + n * p.q_grp + 8 * g;
        const bf16_bits* dp = p.dout + tok * p.do_tok + h * p.do_kvh + n * p.do_grp + 8 * g;
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            qf[c] = *reinterpret_cast<const bf16x8*>(qp + 32 * c);
            dof[c] = *reinterpret_cast<const bf16x8*>(dp + 32 * c);
        }
    }
    const float lse2 = p.lse[h * p.lse_kvh + tok * p.lse_tok + n * p.lse_grp] * kLog2e;
    const float dsum = p.dsum[static_cast<int64_t>(h) * p.total_q * 16 + tok * 16 + n];

    int last_key = kCausal ? (i + Sk - Sq) : (Sk - 1);
    if (last_key > Sk - 1) last_key = Sk - 1;
    const int last_blk = last_key < 0 ? -1 : (last_key >> 6);
    BlockWalker walk;
    walk.init(p.fwd_mask ? p.fwd_mask + (static_cast<int64_t>(h) * p.total_q + tok) * p.n64_fwd : nullptr, p.n64_fwd, last_blk);

    const int64_t img0 = (static_cast<int64_t>(h) * p.n_slots + image_slot0(p.cu_seqlens_k, b)) * kImageElems + lane * 8;
    floatx4 dq[8];
#pragma unroll
    for (int dt = 0; dt < 8; ++dt) dq[dt] = floatx4{0.f, 0.f, 0.f, 0.f};

    for (int j = walk.next(); j >= 0; j = walk.next()) {
        const bf16_bits* ksrc = p.kimg + img0 + static_cast<int64_t>(j) * kImageElems;
        const bf16_bits* vsrc = p.vimg_r + img0 + static_cast<int64_t>(j) * kImageElems;
        const bf16_bits* ktsrc = p.kimg_t + img0 + static_cast<int64_t>(j) * kImageElems;
        floatx4 s[4], dp[4];
#pragma unroll
        for (int kt = 0; kt < 4; ++kt) {
            s[kt] = floatx4{0.f, 0.f, 0.f, 0.f};
            dp[kt] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                const bf16x8 kf = *reinterpret_cast<const bf16x8*>(ksrc + (kt * 4 + c) * 512);
                const bf16x8 vf = *reinterpret_cast<const bf16x8*>(vsrc + (kt * 4 + c) * 512);
                s[kt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf, qf[c], s[kt], 0, 0, 0);
                dp[kt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, dof[c], dp[kt], 0, 0, 0);
            }
        }
        const int lim = (j == last_blk) ? last_key - j * kBlockN : kBlockN;
        bf16x8 dsf[2];
#pragma unroll
        for (int kt = 0; kt < 4; ++kt)
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                float pv = __builtin_amdgcn_exp2f(s[kt][e] * p.scale_log2 - lse2);
                if (16 * kt + 4 * g + e > lim) pv = 0.f;
                const float ds = pv * (dp[kt][e] - dsum);
                dsf[kt >> 1][(kt & 1) * 4 + e] = static_cast<__bf16>(ds);
            }
#pragma unroll
        for (int dt = 0; dt < 8; ++dt)
#pragma unroll
            for (int cc = 0; cc < 2; ++cc) {
                const bf16x8 kt_f = *reinterpret_cast<const bf16x8*>(ktsrc + (dt * 2 + cc) * 512);
                dq[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kt_f, dsf[cc], dq[dt], 0, 0, 0);
            }
    }
    bf16_bits* op = p.dq + tok * p.dq_tok + h * p.dq_kvh + n * p.dq_grp + 4 * g;
#pragma unroll
    for (int dt = 0; dt < 8; ++dt) {
        uint2 w;
        w.x = pack_bf16x2(dq[dt][0] * p.scale, dq[dt][1] * p.scale);
        w.y = pack_bf16x2(dq[dt][2] * p.scale, dq[dt][3] * p.scale);
        *reinterpret_cast<uint2*>(op + 16 * dt) = w;
    }
}

// ---------------------------------------------------------------------------------------------
// dK / dV: one workgroup per (64-key block, 2048-token slice)
// ---------------------------------------------------------------------------------------------
constexpr int kRedPitch = 65;                                  // floats per d row of the LDS reduction tile

template <bool kCausal>
__global__ __launch_bounds__(512)
void bwd_dkdv_kernel(const BwdParams p) {
    extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
    uint4* ldsK = reinterpret_cast<uint4*>(smem_raw);          // 1024 units: K image
    uint4* ldsV = ldsK + 1024;                                 // 1024 units: V in K-image order
    float* red = reinterpret_cast<float*>(smem_raw);           // reused after the main loop: [128][65]

    // 8 wavefronts = 4 token streams x 2 key halves: a wavefront owns 32 of the block's 64 keys, so
    // its dK^T / dV^T accumulators are 128 registers and two wavefronts fit on a SIMD.
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int kh = wave & 1, ts = wave >> 1;
    const int n = lane & 15, g = lane >> 4;
    const int j = blockIdx.x / p.n_slices;                     // key block inside the sequence
    const int slice = blockIdx.x - j * p.n_slices;
    const int b = blockIdx.y, h = blockIdx.z;
    const int q0 = p.cu_seqlens_q[b];
    const int Sq = p.cu_seqlens_q[b + 1] - q0;
    const int k0 = p.cu_seqlens_k[b];
    const int Sk = p.cu_seqlens_k[b + 1] - k0;
    if (j * kBlockN >= Sk) return;                             // uniform per workgroup
    int i_lo = slice * kSliceTokens;
    if (kCausal) {
        const int first = j * kBlockN - (Sk - Sq);             // first token that can see key 64 j
        if (first > i_lo) i_lo = first;
    }
    int i_hi = (slice + 1) * kSliceTokens;
    if (i_hi > Sq) i_hi = Sq;
    if (i_lo >= i_hi) return;                                  // uniform per workgroup

    {
        const int64_t img = (static_cast<int64_t>(h) * p.n_slots + image_slot0(p.cu_seqlens_k, b) + j) * kImageElems;
        const uint4* ks = reinterpret_cast<const uint4*>(p.kimg + img);
        const uint4* vs = reinterpret_cast<const uint4*>(p.vimg_r + img);
#pragma unroll
        for (int u = tid; u < 1024; u += 512) { ldsK[u] = ks[u]; ldsV[u] = vs[u]; }
    }
    __syncthreads();

    floatx4 dKt[8][2], dVt[8][2];                              // [d tile][local key tile]: lane (n, g) holds [16dt+4g+e][16(2kh+kt)+n]
#pragma unroll
    for (int dt = 0; dt < 8; ++dt)
#pragma unroll
        for (int kt = 0; kt < 2; ++kt) {
            dKt[dt][kt] = floatx4{0.f, 0.f, 0.f, 0.f};
            dVt[dt][kt] = floatx4{0.f, 0.f, 0.f, 0.f};
        }

    const int64_t t_lo = static_cast<int64_t>(q0) + i_lo, t_hi = static_cast<int64_t>(q0) + i_hi;   // packed token range
    const int w_lo = static_cast<int>(t_lo >> 6), w_hi = static_cast<int>((t_hi - 1) >> 6);
    const uint64_t* mrow = p.bwd_mask ? p.bwd_mask + (static_cast<int64_t>(h) * p.k_blocks + j) * p.n64_bwd : nullptr;
    const int64_t head_tok0 = static_cast<int64_t>(h) * p.total_q;
    const uint4* myK = ldsK + (2 * kh) * 4 * 64 + lane;
    const uint4* myV = ldsV + (2 * kh) * 4 * 64 + lane;

    for (int w = w_lo + ts; w <= w_hi; w += 4) {
        uint64_t bits = mrow ? mrow[w] : ~0ull;
        const int64_t base = static_cast<int64_t>(w) << 6;
        if (base < t_lo) bits &= ~0ull << (t_lo - base);
        if (base + 64 > t_hi) bits &= ~0ull >> (base + 64 - t_hi);
        {
            const uint32_t lo = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(bits));
            const uint32_t hi = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(bits >> 32));
            bits = (static_cast<uint64_t>(hi) << 32) | lo;
        }
        while (bits != 0ull) {
            const int64_t ta = base + __builtin_ctzll(bits);
            bits &= bits - 1ull;
            const bool has_b = bits != 0ull;
            const int64_t tb = has_b ? base + __builtin_ctzll(bits) : ta;
            bits &= bits - 1ull;                                // no-op on zero

            float lse_a[4], lse_b[4], D_a[4], D_b[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int hd = 4 * g + e;
                lse_a[e] = p.lse[h * p.lse_kvh + ta * p.lse_tok + hd * p.lse_grp] * kLog2e;
                lse_b[e] = p.lse[h * p.lse_kvh + tb * p.lse_tok + hd * p.lse_grp] * kLog2e;
                D_a[e] = p.dsum[head_tok0 * 16 + ta * 16 + hd];
                D_b[e] = p.dsum[head_tok0 * 16 + tb * 16 + hd];
            }
            int lim_a, lim_b;                                   // in-block key index limit (inclusive)
            {
                const int valid = Sk - j * kBlockN - 1;
                lim_a = valid; lim_b = valid;
                if (kCausal) {
                    const int ca = static_cast<int>(ta - q0) + Sk - Sq - j * kBlockN;
                    const int cb = static_cast<int>(tb - q0) + Sk - Sq - j * kBlockN;
                    lim_a = ca < lim_a ? ca : lim_a;
                    lim_b = cb < lim_b ? cb : lim_b;
                }
                if (!has_b) lim_b = -1;
            }
            // phase 1: P = exp2(scale*S - lse) for both tokens on this wavefront's 32 keys (fp32, kept for dS)
            float pa[2][4], pb[2][4];
            {
                bf16x8 qa[4], qb[4];
                const bf16_bits* ptr_a = p.q + ta * p.q_tok + h * p.q_kvh + n * p.q_grp + 8 * g;
                const bf16_bits* ptr_b = p.q + tb * p.q_tok + h * p.q_kvh + n * p.q_grp + 8 * g;
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    qa[c] = *reinterpret_cast<const bf16x8*>(ptr_a + 32 * c);
                    qb[c] = *reinterpret_cast<const bf16x8*>(ptr_b + 32 * c);
                }
#pragma unroll
                for (int kt = 0; kt < 2; ++kt) {
                    floatx4 sa = floatx4{0.f, 0.f, 0.f, 0.f}, sb = sa;
#pragma unroll
                    for (int c = 0; c < 4; ++c) {
                        const uint4 kraw = myK[(kt * 4 + c) * 64];
                        bf16x8 kf;
                        __builtin_memcpy(&kf, &kraw, 16);
                        sa = __builtin_amdgcn_mfma_f32_16x16x32_bf16(qa[c], kf, sa, 0, 0, 0);
                        sb = __builtin_amdgcn_mfma_f32_16x16x32_bf16(qb[c], kf, sb, 0, 0, 0);
                    }
                    const int key = 16 * (2 * kh + kt) + n;
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const float xa = __builtin_amdgcn_exp2f(sa[e] * p.scale_log2 - lse_a[e]);
                        const float xb = __builtin_amdgcn_exp2f(sb[e] * p.scale_log2 - lse_b[e]);
                        pa[kt][e] = key > lim_a ? 0.f : xa;
                        pb[kt][e] = key > lim_b ? 0.f : xb;
                    }
                }
            }
            // phase 2: dP = dO V^T, dS = P * (dP - D); both packed to bf16 as B operands
            bf16x8 pfr[2], dsfr[2];
            {
                bf16x8 doa[4], dob[4];
                const bf16_bits* ptr_a = p.dout + ta * p.do_tok + h * p.do_kvh + n * p.do_grp + 8 * g;
                const bf16_bits* ptr_b = p.dout + tb * p.do_tok + h * p.do_kvh + n * p.do_grp + 8 * g;
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    doa[c] = *reinterpret_cast<const bf16x8*>(ptr_a + 32 * c);
                    dob[c] = *reinterpret_cast<const bf16x8*>(ptr_b + 32 * c);
                }
#pragma unroll
                for (int kt = 0; kt < 2; ++kt) {
                    floatx4 dpa = floatx4{0.f, 0.f, 0.f, 0.f}, dpb = dpa;
#pragma unroll
                    for (int c = 0; c < 4; ++c) {
                        const uint4 vraw = myV[(kt * 4 + c) * 64];
                        bf16x8 vf;
                        __builtin_memcpy(&vf, &vraw, 16);
                        dpa = __builtin_amdgcn_mfma_f32_16x16x32_bf16(doa[c], vf, dpa, 0, 0, 0);
                        dpb = __builtin_amdgcn_mfma_f32_16x16x32_bf16(dob[c], vf, dpb, 0, 0, 0);
                    }
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        pfr[kt][e] = static_cast<__bf16>(pa[kt][e]);
                        pfr[kt][4 + e] = static_cast<__bf16>(pb[kt][e]);
                        dsfr[kt][e] = static_cast<__bf16>(pa[kt][e] * (dpa[e] - D_a[e]));
                        dsfr[kt][4 + e] = static_cast<__bf16>(pb[kt][e] * (dpb[e] - D_b[e]));
                    }
                }
            }
            __builtin_amdgcn_sched_barrier(0);
            const bf16_bits* qTa = p.qT + (head_tok0 + ta) * kTImageElems + lane * 4;
            const bf16_bits* qTb = p.qT + (head_tok0 + tb) * kTImageElems + lane * 4;
            const bf16_bits* dTa = p.doT + (head_tok0 + ta) * kTImageElems + lane * 4;
            const bf16_bits* dTb = p.doT + (head_tok0 + tb) * kTImageElems + lane * 4;
#pragma unroll
            for (int dt = 0; dt < 8; ++dt) {
                const uint2 a0 = *reinterpret_cast<const uint2*>(qTa + dt * 256);
                const uint2 a1 = *reinterpret_cast<const uint2*>(qTb + dt * 256);
                const uint2 d0 = *reinterpret_cast<const uint2*>(dTa + dt * 256);
                const uint2 d1 = *reinterpret_cast<const uint2*>(dTb + dt * 256);
                const uint4 aq_raw = make_uint4(a0.x, a0.y, a1.x, a1.y);
                const uint4 ad_raw = make_uint4(d0.x, d0.y, d1.x, d1.y);
                bf16x8 aq, ad;
                __builtin_memcpy(&aq, &aq_raw, 16);
                __builtin_memcpy(&ad, &ad_raw, 16);
#pragma unroll
                for (int kt = 0; kt < 2; ++kt) {
                    dVt[dt][kt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ad, pfr[kt], dVt[dt][kt], 0, 0, 0);
                    dKt[dt][kt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(aq, dsfr[kt], dKt[dt][kt], 0, 0, 0);
                }
            }
        }
    }

    // reduce the four token streams through LDS (dK then dV), one atomic flush per workgroup and tensor
    const int valid_keys = (Sk - j * kBlockN) < kBlockN ? (Sk - j * kBlockN) : kBlockN;
    const int64_t row0 = static_cast<int64_t>(k0) + static_cast<int64_t>(j) * kBlockN;
#pragma unroll
    for (int which = 0; which < 2; ++which) {
        __syncthreads();                                       // LDS free: images consumed / previous flush done
        for (int r = 0; r < 4; ++r) {
            if (ts == r) {
#pragma unroll
                for (int dt = 0; dt < 8; ++dt)
#pragma unroll
                    for (int kt = 0; kt < 2; ++kt)
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            const int idx = (16 * dt + 4 * g + e) * kRedPitch + 16 * (2 * kh + kt) + n;
                            const float val = which == 0 ? dKt[dt][kt][e] : dVt[dt][kt][e];
                            if (r == 0) red[idx] = val; else red[idx] += val;
                        }
            }
            __syncthreads();
        }
        float* acc = which == 0 ? p.dk_acc : p.dv_acc;
        const float mul = which == 0 ? p.scale : 1.f;
        for (int idx = tid; idx < kBlockN * kHeadDim; idx += 512) {
            const int key = idx >> 7, d = idx & 127;
            if (key < valid_keys)
                unsafeAtomicAdd(acc + ((row0 + key) * p.num_heads_k + h) * kHeadDim + d, red[d * kRedPitch + key] * mul);
        }
    }
}

// ---------------------------------------------------------------------------------------------
// dK / dV, streamed variant: same work split (64-key block x 2048-token slice per workgroup) but the
// workgroup is ONE token stream.  Four wavefronts each own 16 of the block's keys (their K and V
// operands stay in registers for the whole kernel, their dK^T / dV^T tiles are 64 accumulator
// registers), and every token pair's operands (q, dout, their transposed images, LSE and D) are
// copied (flat 1 KiB transfers from fragment-major images the preprocessing kernel wrote) into a
// 4-stage LDS ring by LDS-DMA loads issued three pairs ahead, so no wavefront
// ever waits on global-memory latency and no operand passes through registers on its way in.
// ---------------------------------------------------------------------------------------------
constexpr int kStages = 4;
constexpr int kStageBytes = 32768 + 1024;                      // 8 operand tiles of 4 KiB + 4 copies of the pair's 64 scalars
constexpr int kMaxSliceWords = kSliceTokens / 64 + 1;

__device__ __forceinline__ uint32_t lds_address(const void* ptr) {
    return static_cast<uint32_t>(reinterpret_cast<uintptr_t>((__attribute__((address_space(3))) const void*)ptr));
}
// LDS-DMA: lane l's 16 (or 4) bytes at its own global address land at lds_base + 16 l (4 l).  Invisible to
// the compiler's wait-count tracking; ordered by hand with s_waitcnt vmcnt(n) + barrier.
__device__ __forceinline__ void dma16(const void* src_lane, uint32_t lds_base) {
    lds_base = __builtin_amdgcn_readfirstlane(lds_base);
    asm volatile("s_mov_b32 m0, %1\n\tglobal_load_lds_dwordx4 %0, off" : : "v"(src_lane), "s"(lds_base) : "memory", "m0");
}
__device__ __forceinline__ void dma4(const void* src_lane, uint32_t lds_base) {
    lds_base = __builtin_amdgcn_readfirstlane(lds_base);
    asm volatile("s_mov_b32 m0, %1\n\tglobal_load_lds_dword %0, off" : : "v"(src_lane), "s"(lds_base) : "memory", "m0");
}

struct PairCursor {                                            // walks the slice's mask words (in LDS) two tokens at a time
    const unsigned long long* words;
    int n_words, w;
    uint64_t bits;
    int64_t base0;                                             // packed token index of bit 0 of word 0
    __device__ __forceinline__ void init(const unsigned long long* wd, int n, int64_t b0) {
        words = wd; n_words = n; w = -1; bits = 0ull; base0 = b0;
    }
    __device__ __forceinline__ bool next(int64_t& ta, int64_t& tb, bool& has_b) {
        while (bits == 0ull) {
            if (++w >= n_words) return false;
            const uint64_t v = words[w];
            const uint32_t lo = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(v));
            const uint32_t hi = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(v >> 32));
            bits = (static_cast<uint64_t>(hi) << 32) | lo;
        }
        const int64_t base = base0 + (static_cast<int64_t>(w) << 6);
        ta = base + __builtin_ctzll(bits);
        bits &= bits - 1ull;
        has_b = bits != 0ull;
        tb = has_b ? base + __builtin_ctzll(bits) : ta;
        bits &= bits - 1ull;
        return true;
    }
};

template <bool kCausal>
__global__ __launch_bounds__(256)
void bwd_dkdv_stream_kernel(const BwdParams p) {
    extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
    unsigned char* ring = smem_raw;                                              // kStages * kStageBytes
    unsigned long long* words = reinterpret_cast<unsigned long long*>(smem_raw + kStages * kStageBytes);
    float* red = reinterpret_cast<float*>(smem_raw);                             // reused after the main loop: [128][65]

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);                   // = key tile (16 keys); scalar, so branches on it are uniform
    const int n = lane & 15, g = lane >> 4;
    const int j = blockIdx.x / p.n_slices;
    const int slice = blockIdx.x - j * p.n_slices;
    const int b = blockIdx.y, h = blockIdx.z;
    const int q0 = p.cu_seqlens_q[b];
    const int Sq = p.cu_seqlens_q[b + 1] - q0;
    const int k0 = p.cu_seqlens_k[b];
    const int Sk = p.cu_seqlens_k[b + 1] - k0;
    if (j * kBlockN >= Sk) return;                                               // uniform per workgroup
    int i_lo = slice * kSliceTokens;
    if (kCausal) {
        const int first = j * kBlockN - (Sk - Sq);
        if (first > i_lo) i_lo = first;
    }
    int i_hi = (slice + 1) * kSliceTokens;
    if (i_hi > Sq) i_hi = Sq;
    if (i_lo >= i_hi) return;                                                    // uniform per workgroup

    // this wavefront's K and V operands (B side of S = Q K^T and dP = dO V^T), resident in registers
    bf16x8 kreg[4], vreg[4];
    {
        const int64_t img = (static_cast<int64_t>(h) * p.n_slots + image_slot0(p.cu_seqlens_k, b) + j) * kImageElems;
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            kreg[c] = *reinterpret_cast<const bf16x8*>(p.kimg + img + ((wave * 4 + c) * 64 + lane) * 8);
            vreg[c] = *reinterpret_cast<const bf16x8*>(p.vimg_r + img + ((wave * 4 + c) * 64 + lane) * 8);
        }
    }
    // the slice's mask words, clipped to [t_lo, t_hi), into LDS
    const int64_t t_lo = static_cast<int64_t>(q0) + i_lo, t_hi = static_cast<int64_t>(q0) + i_hi;
    const int w_lo = static_cast<int>(t_lo >> 6), w_hi = static_cast<int>((t_hi - 1) >> 6);
    const int n_words = w_hi - w_lo + 1;                                         // <= kMaxSliceWords
    const uint64_t* mrow = p.bwd_mask ? p.bwd_mask + (static_cast<int64_t>(h) * p.k_blocks + j) * p.n64_bwd : nullptr;
    for (int w = tid; w < n_words; w += 256) {
        uint64_t v = mrow ? mrow[w_lo + w] : ~0ull;
        const int64_t base = static_cast<int64_t>(w_lo + w) << 6;
        if (base < t_lo) v &= ~0ull << (t_lo - base);
        if (base + 64 > t_hi) v &= ~0ull >> (base + 64 - t_hi);
        words[w] = v;
    }
    __syncthreads();

    const int64_t head_tok0 = static_cast<int64_t>(h) * p.total_q;
    const uint32_t ring_lds = __builtin_amdgcn_readfirstlane(lds_address(ring));
    // what this wavefront fetches for a pair: wave 0 q, wave 1 dout (both as gathered A-operand fragments),
    // wave 2 the transposed q image, wave 3 the transposed dout image (flat copies); plus its own scalar copy
    auto issue = [&](int64_t ta, int64_t tb, int stage) {
        const uint32_t st = ring_lds + stage * kStageBytes;
        const bf16_bits* src = wave == 0 ? p.qF : (wave == 1 ? p.doF : (wave == 2 ? p.qT : p.doT));
        const bf16_bits* pa = src + (head_tok0 + ta) * kTImageElems + lane * 8;
        const bf16_bits* pb = src + (head_tok0 + tb) * kTImageElems + lane * 8;
        const uint32_t dst = st + wave * 8192;
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            dma16(pa + 512 * c, dst + c * 1024);
            dma16(pb + 512 * c, dst + 4096 + c * 1024);
        }
        // the pair's row statistics: [lse_a (16) | D_a (16) | lse_b (16) | D_b (16)], one private copy per wavefront
        dma4(p.rowstat + (head_tok0 + (lane < 32 ? ta : tb)) * 32 + (lane & 31), st + 32768 + wave * 256);
    };

    floatx4 dKt[8], dVt[8];                                                       // lane (n, g): [16 dt + 4 g + e][16 wave + n]
#pragma unroll
    for (int dt = 0; dt < 8; ++dt) {
        dKt[dt] = floatx4{0.f, 0.f, 0.f, 0.f};
        dVt[dt] = floatx4{0.f, 0.f, 0.f, 0.f};
    }

    PairCursor fetch_cur, use_cur;
    fetch_cur.init(words, n_words, static_cast<int64_t>(w_lo) << 6);
    use_cur.init(words, n_words, static_cast<int64_t>(w_lo) << 6);
    // Every ordinary load issued so far must have landed before the first LDS-DMA goes out: the compiler
    // would otherwise place its own "wait for kreg/vreg" inside the loop, and such a wait also drains the
    // DMA loads that are meant to stay in flight.
    __builtin_amdgcn_s_waitcnt(0x0F70);
#pragma unroll
    for (int c = 0; c < 4; ++c) asm volatile("" : "+v"(kreg[c]), "+v"(vreg[c]));
    int ahead = 0;                                                                // pairs issued and not yet consumed
    int fetch_stage = 0;
    {
        int64_t ta, tb; bool hb;
        while (ahead < kStages - 1 && fetch_cur.next(ta, tb, hb)) {
            issue(ta, tb, fetch_stage);
            fetch_stage = fetch_stage == kStages - 1 ? 0 : fetch_stage + 1;
            ++ahead;
        }
    }
    int use_stage = 0;
    int64_t ta, tb;
    bool has_b;
    while (use_cur.next(ta, tb, has_b)) {
        // every wavefront issued 9 loads per pair, in order: allow the younger pairs' loads to stay in flight
        if (ahead >= 3) __builtin_amdgcn_s_waitcnt(0x4F72);                       // vmcnt(18)
        else if (ahead == 2) __builtin_amdgcn_s_waitcnt(0x0F79);                  // vmcnt(9)
        else __builtin_amdgcn_s_waitcnt(0x0F70);                                  // vmcnt(0)
        __syncthreads();                                                          // pair is in LDS for all; the stage consumed last turn is free
        {
            int64_t na, nb; bool hb;
            if (fetch_cur.next(na, nb, hb)) {
                issue(na, nb, fetch_stage);
                fetch_stage = fetch_stage == kStages - 1 ? 0 : fetch_stage + 1;
            } else {
                --ahead;
            }
        }
        const unsigned char* st = ring + use_stage * kStageBytes;
        use_stage = use_stage == kStages - 1 ? 0 : use_stage + 1;

        const float* scal = reinterpret_cast<const float*>(st + 32768 + wave * 256);
        const float4 la = *reinterpret_cast<const float4*>(scal + 4 * g);
        const float4 Da = *reinterpret_cast<const float4*>(scal + 16 + 4 * g);
        const float4 lb = *reinterpret_cast<const float4*>(scal + 32 + 4 * g);
        const float4 Db = *reinterpret_cast<const float4*>(scal + 48 + 4 * g);
        const float lse_a[4] = {la.x, la.y, la.z, la.w};
        const float lse_b[4] = {lb.x, lb.y, lb.z, lb.w};
        const float D_a[4] = {Da.x, Da.y, Da.z, Da.w};
        const float D_b[4] = {Db.x, Db.y, Db.z, Db.w};
        int lim_a, lim_b;
        {
            const int valid = Sk - j * kBlockN - 1;
            lim_a = valid; lim_b = valid;
            if (kCausal) {
                const int ca = static_cast<int>(ta - q0) + Sk - Sq - j * kBlockN;
                const int cb = static_cast<int>(tb - q0) + Sk - Sq - j * kBlockN;
                lim_a = ca < lim_a ? ca : lim_a;
                lim_b = cb < lim_b ? cb : lim_b;
            }
            if (!has_b) lim_b = -1;
        }
        const uint4* frag = reinterpret_cast<const uint4*>(st) + lane;            // fragment c of tile t at frag[t*256 + c*64]
        floatx4 sa = floatx4{0.f, 0.f, 0.f, 0.f}, sb = sa, dpa = sa, dpb = sa;
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            const uint4 ra = frag[0 * 256 + c * 64], rb = frag[1 * 256 + c * 64];
            const uint4 rc = frag[2 * 256 + c * 64], rd = frag[3 * 256 + c * 64];
            bf16x8 qa, qb, doa, dob;
            __builtin_memcpy(&qa, &ra, 16);
            __builtin_memcpy(&qb, &rb, 16);
            __builtin_memcpy(&doa, &rc, 16);
            __builtin_memcpy(&dob, &rd, 16);
            sa = __builtin_amdgcn_mfma_f32_16x16x32_bf16(qa, kreg[c], sa, 0, 0, 0);
            sb = __builtin_amdgcn_mfma_f32_16x16x32_bf16(qb, kreg[c], sb, 0, 0, 0);
            dpa = __builtin_amdgcn_mfma_f32_16x16x32_bf16(doa, vreg[c], dpa, 0, 0, 0);
            dpb = __builtin_amdgcn_mfma_f32_16x16x32_bf16(dob, vreg[c], dpb, 0, 0, 0);
        }
        bf16x8 pfr, dsfr;
        {
            const int key = 16 * wave + n;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                float xa = __builtin_amdgcn_exp2f(sa[e] * p.scale_log2 - lse_a[e]);
                float xb = __builtin_amdgcn_exp2f(sb[e] * p.scale_log2 - lse_b[e]);
                xa = key > lim_a ? 0.f : xa;
                xb = key > lim_b ? 0.f : xb;
                pfr[e] = static_cast<__bf16>(xa);
                pfr[4 + e] = static_cast<__bf16>(xb);
                dsfr[e] = static_cast<__bf16>(xa * (dpa[e] - D_a[e]));
                dsfr[4 + e] = static_cast<__bf16>(xb * (dpb[e] - D_b[e]));
            }
        }
        const uint2* timg = reinterpret_cast<const uint2*>(st + 16384) + lane;    // tile t, d-tile dt at timg[t*512 + dt*64]
#pragma unroll
        for (int dt = 0; dt < 8; ++dt) {
            const uint2 a0 = timg[0 * 512 + dt * 64], a1 = timg[1 * 512 + dt * 64];
            const uint2 d0 = timg[2 * 512 + dt * 64], d1 = timg[3 * 512 + dt * 64];
            const uint4 aq_raw = make_uint4(a0.x, a0.y, a1.x, a1.y);
            const uint4 ad_raw = make_uint4(d0.x, d0.y, d1.x, d1.y);
            bf16x8 aq, ad;
            __builtin_memcpy(&aq, &aq_raw, 16);
            __builtin_memcpy(&ad, &ad_raw, 16);
            dVt[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ad, pfr, dVt[dt], 0, 0, 0);
            dKt[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(aq, dsfr, dKt[dt], 0, 0, 0);
        }
    }

    // each wavefront owns its 16 key columns: transpose through LDS for coalesced atomics
    const int valid_keys = (Sk - j * kBlockN) < kBlockN ? (Sk - j * kBlockN) : kBlockN;
    const int64_t row0 = static_cast<int64_t>(k0) + static_cast<int64_t>(j) * kBlockN;
#pragma unroll
    for (int which = 0; which < 2; ++which) {
        __syncthreads();
#pragma unroll
        for (int dt = 0; dt < 8; ++dt)
#pragma unroll
            for (int e = 0; e < 4; ++e)
                red[(16 * dt + 4 * g + e) * kRedPitch + 16 * wave + n] = which == 0 ? dKt[dt][e] : dVt[dt][e];
        __syncthreads();
        float* acc = which == 0 ? p.dk_acc : p.dv_acc;
        const float mul = which == 0 ? p.scale : 1.f;
        for (int idx = tid; idx < kBlockN * kHeadDim; idx += 256) {
            const int key = idx >> 7, d = idx & 127;
            if (key < valid_keys)
                unsafeAtomicAdd(acc + ((row0 + key) * p.num_heads_k + h) * kHeadDim + d, red[d * kRedPitch + key] * mul);
        }
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
    ka.x = pack_bf16x2(a.x, a.y); ka.y = pack_bf16x2(a.z, a.w);
    va.x = pack_bf16x2(c.x, c.y); va.y = pack_bf16x2(c.z, c.w);
    *reinterpret_cast<uint2*>(p.dk + row * p.dk_row + h * p.dk_head + d4 * 4) = ka;
    *reinterpret_cast<uint2*>(p.dv + row * p.dv_row + h * p.dv_head + d4 * 4) = va;
}

static size_t align256(size_t x) { return (x + 255) & ~static_cast<size_t>(255); }

struct BwdLayout {
    size_t images, mask, dsum, qT, doT, qF, doF, rowstat, dk_acc, dv_acc, total;
};

static BwdLayout bwd_layout(int batch, int64_t total_q, int64_t total_k, int num_heads_k, int max_seqlen_k) {
    BwdLayout L;
    size_t off = 0;
    L.images = off; off += align256(infllmv2_kv_image_bytes(total_k, batch, num_heads_k) * 2);
    const int64_t k_blocks = (max_seqlen_k + kBlockN - 1) / kBlockN;
    L.mask = off; off += align256(static_cast<size_t>(num_heads_k) * k_blocks * ((total_q + 63) / 64) * 8);
    L.dsum = off; off += align256(static_cast<size_t>(num_heads_k) * total_q * 16 * 4);
    L.qT = off; off += align256(static_cast<size_t>(num_heads_k) * total_q * kTImageElems * 2);
    L.doT = off; off += align256(static_cast<size_t>(num_heads_k) * total_q * kTImageElems * 2);
    L.qF = off; off += align256(static_cast<size_t>(num_heads_k) * total_q * kTImageElems * 2);
    L.doF = off; off += align256(static_cast<size_t>(num_heads_k) * total_q * kTImageElems * 2);
    L.rowstat = off; off += align256(static_cast<size_t>(num_heads_k) * total_q * 32 * 4);
    L.dk_acc = off; off += align256(static_cast<size_t>(total_k) * num_heads_k * kHeadDim * 4);
    L.dv_acc = off; off += align256(static_cast<size_t>(total_k) * num_heads_k * kHeadDim * 4);
    L.total = off;
    return L;
}

}  // namespace infllmv2

using namespace infllmv2;

extern "C" size_t infllmv2_varlen_bwd_workspace_bytes(int batch, int64_t total_q, int64_t total_k, int num_heads_k,
                                                      int max_seqlen_k) {
    return bwd_layout(batch, total_q, total_k, num_heads_k, max_seqlen_k).total;
}

extern "C" int infllmv2_varlen_bwd(void* stream, const void* dout, const void* q, const void* k, const void* v,
                                   const void* out, const float* softmax_lse, void* dq, void* dk, void* dv,
                                   const int32_t* cu_seqlens_q, const int32_t* cu_seqlens_k,
                                   const uint64_t* fwd_blockmask, void* workspace, size_t workspace_bytes, int batch,
                                   int64_t total_q, int64_t total_k, int num_heads, int num_heads_k, int head_dim,
                                   int max_seqlen_q, int max_seqlen_k, const int64_t* q_strides,
                                   const int64_t* k_strides, const int64_t* v_strides, const int64_t* o_strides,
                                   const int64_t* do_strides, const int64_t* dq_strides, const int64_t* dk_strides,
                                   const int64_t* dv_strides, const int64_t* lse_strides, int n_uint64_per_row,
                                   float softmax_scale, int is_causal) {
    IV2_CHECK(head_dim == kHeadDim, "varlen_bwd: this build only supports head_dim 128 (got %d)", head_dim);
    IV2_CHECK(num_heads_k > 0 && num_heads == num_heads_k * kGroup,
              "varlen_bwd: requires num_heads == 16 * num_heads_k (got %d and %d)", num_heads, num_heads_k);
    IV2_CHECK(batch > 0 && total_q >= 0 && total_k >= 0 && max_seqlen_q >= 0 && max_seqlen_k >= 0, "varlen_bwd: bad sizes");
    IV2_CHECK(dout && q && k && v && out && softmax_lse && dq && dk && dv && cu_seqlens_q && cu_seqlens_k && workspace,
              "varlen_bwd: null pointer");
    IV2_CHECK(num_heads_k <= 65535 && batch <= 65535, "varlen_bwd: batch and num_heads_k must not exceed 65535");
    const BwdLayout L = bwd_layout(batch, total_q, total_k, num_heads_k, max_seqlen_k);
    IV2_CHECK(workspace_bytes >= L.total, "varlen_bwd: workspace too small (%zu < %zu)", workspace_bytes, L.total);
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
    p.q = static_cast<const bf16_bits*>(q);
    p.dout = static_cast<const bf16_bits*>(dout);
    p.out = static_cast<const bf16_bits*>(out);
    p.dq = static_cast<bf16_bits*>(dq);
    p.lse = softmax_lse;
    p.dsum = reinterpret_cast<float*>(ws + L.dsum);
    p.qT = reinterpret_cast<bf16_bits*>(ws + L.qT);
    p.doT = reinterpret_cast<bf16_bits*>(ws + L.doT);
    p.qF = reinterpret_cast<bf16_bits*>(ws + L.qF);
    p.doF = reinterpret_cast<bf16_bits*>(ws + L.doF);
    p.rowstat = reinterpret_cast<float*>(ws + L.rowstat);
    const int64_t n_slots = image_slots(total_k, batch);
    const int64_t img_elems = n_slots * num_heads_k * kImageElems;
    p.kimg = reinterpret_cast<const bf16_bits*>(ws + L.images);
    p.kimg_t = p.kimg + 2 * img_elems;
    p.vimg_r = p.kimg + 3 * img_elems;
    p.dk_acc = reinterpret_cast<float*>(ws + L.dk_acc);
    p.dv_acc = reinterpret_cast<float*>(ws + L.dv_acc);
    p.dk = static_cast<bf16_bits*>(dk);
    p.dv = static_cast<bf16_bits*>(dv);
    p.fwd_mask = fwd_blockmask;
    p.cu_seqlens_q = cu_seqlens_q; p.cu_seqlens_k = cu_seqlens_k;
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
    p.n_slices = (max_seqlen_q + kSliceTokens - 1) / kSliceTokens;
    p.scale = softmax_scale;
    p.scale_log2 = softmax_scale * kLog2e;

    // dK/dV accumulators start at zero (fill kernel, no memset node)
    if (total_k > 0) {
        const int64_t n4 = static_cast<int64_t>((L.dv_acc - L.dk_acc) / 16) * 2;
        IV2_CHECK((L.dv_acc - L.dk_acc) == align256(static_cast<size_t>(total_k) * num_heads_k * kHeadDim * 4), "varlen_bwd: layout");
        hipLaunchKernelGGL(zero_f32_kernel, dim3(2048), dim3(256), 0, st, reinterpret_cast<float4*>(p.dk_acc), n4);
        IV2_LAUNCH_CHECK();
    }
    if (total_q > 0 && max_seqlen_q > 0 && total_k > 0 && max_seqlen_k > 0) {
        int rc = launch_pack(st, k, v, cu_seqlens_k, ws + L.images, L.mask - L.images, batch, total_k, num_heads_k,
                             max_seqlen_k, k_strides, v_strides, true);
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
        static const bool dq_per_token = [] {                  // diagnostic switch: one wavefront per token, no sharing
            const char* e = getenv("INFLLMV2_BWD_DQ_PER_TOKEN");
            return e != nullptr && e[0] == '1';
        }();
        if (dq_per_token) {
            const dim3 gq((max_seqlen_q + 3) / 4, batch, num_heads_k);
            if (is_causal) hipLaunchKernelGGL(bwd_dq_kernel<true>, gq, dim3(256), 0, st, p);
            else hipLaunchKernelGGL(bwd_dq_kernel<false>, gq, dim3(256), 0, st, p);
            IV2_LAUNCH_CHECK();
        } else {
            rc = launch_bwd_dq_hybrid(st, p, batch, max_seqlen_q, is_causal != 0);
            if (rc != 0) return rc;
        }
        const dim3 gk(static_cast<unsigned>(p.k_blocks) * p.n_slices, batch, num_heads_k);
        static const int variant = [] {                         // experiment switch: 1 = workgroup-streamed, 2 = 4 streams x 2 key halves
            const char* e = getenv("INFLLMV2_BWD_DKDV");
            return e == nullptr ? 0 : atoi(e);
        }();
        if (variant == 0) {
            rc = launch_bwd_dkdv_wave(st, p, batch, max_seqlen_q, is_causal != 0);
            if (rc != 0) return rc;
        } else if (variant == 2) {
            const size_t lds = kHeadDim * kRedPitch * sizeof(float);      // 33280 B >= the 32 KiB of staged images
            if (is_causal) hipLaunchKernelGGL(bwd_dkdv_kernel<true>, gk, dim3(512), lds, st, p);
            else hipLaunchKernelGGL(bwd_dkdv_kernel<false>, gk, dim3(512), lds, st, p);
        } else {
            const size_t lds = kStages * kStageBytes + kMaxSliceWords * 8;
            const void* fn = is_causal ? reinterpret_cast<const void*>(&bwd_dkdv_stream_kernel<true>)
                                       : reinterpret_cast<const void*>(&bwd_dkdv_stream_kernel<false>);
            hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds));
            IV2_CHECK(e == hipSuccess, "varlen_bwd: cannot reserve %zu bytes of LDS: %s", lds, hipGetErrorString(e));
            if (is_causal) hipLaunchKernelGGL(bwd_dkdv_stream_kernel<true>, gk, dim3(256), lds, st, p);
            else hipLaunchKernelGGL(bwd_dkdv_stream_kernel<false>, gk, dim3(256), lds, st, p);
        }
        IV2_LAUNCH_CHECK();
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
