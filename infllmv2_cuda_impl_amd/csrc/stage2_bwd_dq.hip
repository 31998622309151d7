// Stage-2 backward, dQ (gfx950): row-parallel, workgroup-hybrid like the forward.
//
// Mathematics as in compute_dq_dk_dv_1colblock (csrc/flash_attn/src/flash_bwd_kernel.h:498-794)
// restricted to dQ:  P = exp(scale S - LSE),  dP = dO V^T,  dS = P (dP - D),  dQ = scale dS K.
// S and dP are recomputed here (the column-parallel dK/dV kernel forms them again on its side), so
// dQ stays in registers for a token's whole row and is written once as bf16: no fp32 dQ scratch,
// no atomics, no conversion pass, bit-reproducible.
//
// Schedule as in stage2_fwd_hybrid.hip: 8 wavefronts = 8 consecutive tokens; the blocks all 8
// mask rows select go once through a 2-tile LDS ring ([K image | V in K-image order], 32 KiB),
// and there the K^T operand of dQ^T = K^T dS^T is a transposed read (ds_read_b64_tr_b16) of
// the same K tile; the remaining blocks of each row are walked by its wavefront alone, K and V
// fragments straight from global memory into registers, the K fragments parked in a private LDS
// tile for the same transposed read.  The two walks are interleaved, one block of each per turn.
#include "common.h"
#include "kv_image.h"
#include "block_walker.h"
#include "stage2_bwd.h"
#include <math.h>

namespace IV2_NS {

constexpr int kDqTokens = 8;
constexpr int kDqChunk = 16;                                   // token groups per XCD chunk
constexpr int kDqTileBytes = 32768;
constexpr int kDqMaskWords = 256;                              // LDS copies of the mask rows hold at most this many words each: 16384 key blocks
constexpr int kDqLdsTiles = 2 * kDqTileBytes + 8 * 8192;       // 2-tile ring + 8 private half K tiles

typedef short short4q __attribute__((ext_vector_type(4)));

struct DqExtra {
    int groups_per_seq;
    int batch;
    int total_groups;
    int mask_words;                                            // words per LDS mask row: what the longest key sequence needs
};

__device__ __forceinline__ uint32_t lds_address_dq(const void* ptr) {
    return static_cast<uint32_t>(reinterpret_cast<uintptr_t>((__attribute__((address_space(3))) const void*)ptr));
}
// 4 KiB flat copy global -> LDS by one wavefront (see stage2_fwd_hybrid.hip)
__device__ __forceinline__ void dq_dma_copy_4k(const void* src_lane, uint32_t lds_dst) {
    asm volatile("s_mov_b32 m0, %1\n\t"
                 "global_load_lds_dwordx4 %0, off\n\t"
                 "global_load_lds_dwordx4 %0, off offset:1024\n\t"
                 "global_load_lds_dwordx4 %0, off offset:2048\n\t"
                 "global_load_lds_dwordx4 %0, off offset:3072\n\t"
                 :
                 : "v"(src_lane), "s"(lds_dst)
                 : "memory", "m0");
}
__device__ __forceinline__ uint64_t dq_uniform_u64(uint64_t v) {
    const uint32_t lo = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(v));
    const uint32_t hi = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(v >> 32));
    return (static_cast<uint64_t>(hi) << 32) | lo;
}
__device__ __forceinline__ short4q dq_read_tr(const unsigned char* ptr) {
    return __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) short4q*)(ptr));
}

// dS^T of one block as the B operand of dQ^T = K^T dS^T, from the S^T and dP^T accumulators
// dS^T of one block as the B operand of dQ^T += K^T dS^T.  The dP accumulators were started at -D, so dp holds dP - D.
// lim: last in-block key index the token may see (>= 63 for a whole block, which is the common case).
__device__ __forceinline__ void ds_tile(const floatx4 (&s)[4], const floatx4 (&dp)[4], elem8 (&dsf)[2], int lim, int g,
                                        float scale_log2, float lse2) {
    if (lim >= kBlockN - 1) {                                  // uniform per wavefront
#pragma unroll
        for (int kt = 0; kt < 4; ++kt)
#pragma unroll
            for (int e = 0; e < 4; ++e)
                dsf[kt >> 1][(kt & 1) * 4 + e] = static_cast<elem_t>(__builtin_amdgcn_exp2f(s[kt][e] * scale_log2 - lse2) * dp[kt][e]);
    } else {
#pragma unroll
        for (int kt = 0; kt < 4; ++kt)
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                float pv = __builtin_amdgcn_exp2f(s[kt][e] * scale_log2 - lse2);
                if (16 * kt + 4 * g + e > lim) pv = 0.f;
                dsf[kt >> 1][(kt & 1) * 4 + e] = static_cast<elem_t>(pv * dp[kt][e]);
            }
    }
}

template <bool kCausal>
__global__ __launch_bounds__(512)
void bwd_dq_hybrid_kernel(const BwdParams p, const DqExtra x) {
    extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
    uint4* ring = reinterpret_cast<uint4*>(smem_raw);                               // [2][2048]: K units 0..1023, V (K-image order) 1024..2047
    unsigned long long* com = reinterpret_cast<unsigned long long*>(smem_raw + kDqLdsTiles);       // [mask_words]
    unsigned long long* rows = com + x.mask_words;                                                  // [kDqTokens][mask_words]

    const int bid = blockIdx.x;
    const int xcd = bid & 7, sidx = bid >> 3;
    int G = ((sidx / kDqChunk) * 8 + xcd) * kDqChunk + (sidx % kDqChunk);
    if (G >= x.total_groups) return;                                                // uniform per workgroup
    G = x.total_groups - 1 - G;
    const int grp = G % x.groups_per_seq;
    const int hb = G / x.groups_per_seq;
    const int b = hb % x.batch, h = hb / x.batch;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int n = lane & 15, g = lane >> 4;
    const int q0 = p.cu_seqlens_q[b];
    const int Sq = p.cu_seqlens_q[b + 1] - q0;
    const int i0 = grp * kDqTokens;
    if (i0 >= Sq) return;                                                           // uniform per workgroup
    const int Sk = p.cu_seqlens_k[b + 1] - p.cu_seqlens_k[b];

    const int i = i0 + wave;
    const bool live = i < Sq;
    int last_key = kCausal ? (i + Sk - Sq) : (Sk - 1);
    if (last_key > Sk - 1) last_key = Sk - 1;
    if (!live) last_key = -1;
    const int last_blk = last_key < 0 ? -1 : (last_key >> 6);
    const int64_t tok = static_cast<int64_t>(q0) + (live ? i : i0);
    const uint64_t* mrow = p.fwd_mask ? p.fwd_mask + (static_cast<int64_t>(h) * p.total_q + tok) * p.n64_fwd : nullptr;

    // ---- the row words every live token of the group has in common, and what is left of each row ----
    int nw;
    {
        const int i_last = (i0 + kDqTokens - 1 < Sq) ? i0 + kDqTokens - 1 : Sq - 1;
        int lk = kCausal ? (i_last + Sk - Sq) : (Sk - 1);
        if (lk > Sk - 1) lk = Sk - 1;
        nw = lk < 0 ? 0 : (lk >> 12) + 1;
        if (mrow && nw > p.n64_fwd) nw = p.n64_fwd;
        if (nw > x.mask_words) nw = x.mask_words;                                    // a sequence longer than the announced max_seqlen_k
    }
    unsigned long long* own = rows + wave * x.mask_words;
    for (int w = tid; w < nw; w += 512) com[w] = ~0ull;
    __syncthreads();
    for (int w = lane; w < nw; w += 64) {
        uint64_t v = 0ull;
        if (last_blk >= 0 && w <= (last_blk >> 6)) {
            v = mrow ? mrow[w] : ~0ull;
            if (w == (last_blk >> 6)) {
                const int tb = last_blk & 63;
                v &= (tb == 63) ? ~0ull : ((1ull << (tb + 1)) - 1ull);
            }
        }
        own[w] = v;
        if (live && v != ~0ull) atomicAnd(&com[w], static_cast<unsigned long long>(v));
    }
    __syncthreads();
    for (int w = lane; w < nw; w += 64) own[w] &= ~com[w];

    // ---- this token's operands ----
    elem8 qf[4], dof[4];
    {
        const int nq = n < p.group ? n : p.group - 1;          // rows beyond the group repeat its last head; their LSE is +inf
        const elem_bits* qp = p.q + tok * p.q_tok + h * p.q_kvh + nq * p.q_grp + 8 * g;
        const elem_bits* dp = p.dout + tok * p.do_tok + h * p.do_kvh + nq * p.do_grp + 8 * g;
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            qf[c] = *reinterpret_cast<const elem8*>(qp + 32 * c);
            dof[c] = *reinterpret_cast<const elem8*>(dp + 32 * c);
        }
    }
    const float* rs = p.rowstat + (static_cast<int64_t>(h) * p.total_q + tok) * 32;    // [LSE * log2(e) x 16 | D x 16]
    float lse2 = rs[n];
    float dsum = rs[16 + n];
    const floatx4 neg_dsum = {-dsum, -dsum, -dsum, -dsum};     // the dP accumulators start here: dS = P (dP - D) is then one product
    floatx4 dq[8];
#pragma unroll
    for (int dt = 0; dt < 8; ++dt) dq[dt] = floatx4{0.f, 0.f, 0.f, 0.f};

    const int64_t slot0 = static_cast<int64_t>(h) * p.n_slots + image_slot0(p.cu_seqlens_k, b);
    // byte offset, inside a K tile, of this lane's row of the 16 x 4 transposed read: row rho = lane % 16 of d tile
    // dt and key chunk kt2 is K[16 kt2 + 4 g + rho / 4][16 dt + 4 (rho % 4) ..]
    const int tr_lane = (((n & 3) >> 1) * 16 + 4 * g + (n >> 2)) * 16 + (n & 1) * 8;

    // ---- the walk: one turn = one common block (lock step, operands from the 2-tile LDS ring) + one own block
    //      (K and V fragments from global memory into registers, prefetched a turn ahead).  The K fragments of an own
    //      block feed S from registers and are parked, 32 keys at a time, in this wavefront's 8 KiB LDS tile, from
    //      which dQ's K^T operand is a transposed read: an own block costs 32 KiB of global loads, not 48. ----
    const uint4* src_lane = (wave < 4 ? reinterpret_cast<const uint4*>(p.kimg) + slot0 * 1024 + wave * 256
                                      : reinterpret_cast<const uint4*>(p.vimg_r) + slot0 * 1024 + (wave - 4) * 256) + lane;
    const uint32_t ring_base = __builtin_amdgcn_readfirstlane(lds_address_dq(ring) + wave * 4096);
    auto issue = [&](int jj, int tile) { dq_dma_copy_4k(src_lane + static_cast<int64_t>(jj) * 1024, ring_base + tile * kDqTileBytes); };
    int cw = -1, ow = -1;
    uint64_t cbits = 0ull, obits = 0ull;
    auto next_common = [&]() -> int {
        while (cbits == 0ull) {
            if (++cw >= nw) return -1;
            cbits = dq_uniform_u64(com[cw]);
        }
        const int bit = __builtin_ctzll(cbits);
        cbits &= cbits - 1ull;
        return cw * 64 + bit;
    };
    auto next_own = [&]() -> int {
        while (obits == 0ull) {
            if (++ow >= nw) return -1;
            obits = dq_uniform_u64(own[ow]);
        }
        const int bit = __builtin_ctzll(obits);
        obits &= obits - 1ull;
        return ow * 64 + bit;
    };
    const int64_t img0 = slot0 * kImageElems + lane * 8;
    uint4* mine = reinterpret_cast<uint4*>(smem_raw + 2 * kDqTileBytes + wave * 8192) + lane;     // 32 keys of K: 8 fragments
    const unsigned char* mine_tr = smem_raw + 2 * kDqTileBytes + wave * 8192 + tr_lane;
    elem8 kreg[16], vreg[16];
    int jp = live ? next_own() : -1;
    if (jp >= 0) {
        const elem_bits* ksrc = p.kimg + img0 + static_cast<int64_t>(jp) * kImageElems;
#pragma unroll
        for (int f = 0; f < 16; ++f) kreg[f] = *reinterpret_cast<const elem8*>(ksrc + f * 512);
    }
    // All ordinary loads so far land before the first LDS-DMA.  From here on the compiler's wait counts know nothing
    // of the DMA loads; they stay correct because loads complete in order, and the waits written by hand below
    // count the ordinary loads that may be younger than the DMA they wait for.
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#pragma unroll
    for (int c = 0; c < 4; ++c) asm volatile("" : "+v"(qf[c]), "+v"(dof[c]));
#pragma unroll
    for (int f = 0; f < 16; ++f) asm volatile("" : "+v"(kreg[f]));
    asm volatile("" : "+v"(lse2), "+v"(dsum));
    int j0 = next_common();
    if (j0 >= 0) issue(j0, 0);
    int tile = 0;
    bool k_ahead = false;                                      // the coming own block's 16 K-fragment loads were issued last turn
    while (j0 >= 0 || jp >= 0) {
        if (j0 >= 0) {                                         // uniform over the workgroup
            // younger than this wavefront's 4 DMA loads of block j0: last turn's 16 K loads
            if (k_ahead) asm volatile("s_waitcnt vmcnt(16)" ::: "memory"); else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            __syncthreads();                                   // block j0 is in LDS for everyone; the other tile is free
            const int j1 = next_common();
            if (j1 >= 0) issue(j1, tile ^ 1);
            if (live) {
                const uint4* kb = ring + tile * 2048 + lane;
                const uint4* vb = kb + 1024;
                floatx4 s[4], dp[4];
#pragma unroll
                for (int kt = 0; kt < 4; ++kt) {
                    s[kt] = floatx4{0.f, 0.f, 0.f, 0.f};
                    dp[kt] = neg_dsum;
                }
                // vreg is free between own blocks: it stages 16 fragments at a time
#pragma unroll
                for (int f = 0; f < 16; ++f) {
                    const uint4 raw = kb[f * 64];
                    __builtin_memcpy(&vreg[f], &raw, 16);
                }
#pragma unroll
                for (int c = 0; c < 4; ++c)
#pragma unroll
                    for (int kt = 0; kt < 4; ++kt)
                        s[kt] = IV2_MFMA(vreg[kt * 4 + c], qf[c], s[kt], 0, 0, 0);
#pragma unroll
                for (int f = 0; f < 16; ++f) {
                    const uint4 raw = vb[f * 64];
                    __builtin_memcpy(&vreg[f], &raw, 16);
                }
#pragma unroll
                for (int c = 0; c < 4; ++c)
#pragma unroll
                    for (int kt = 0; kt < 4; ++kt)
                        dp[kt] = IV2_MFMA(vreg[kt * 4 + c], dof[c], dp[kt], 0, 0, 0);
                elem8 dsf[2];
                ds_tile(s, dp, dsf, (j0 == last_blk) ? last_key - j0 * kBlockN : kBlockN - 1, g, p.scale_log2, lse2);
                const unsigned char* ktile = reinterpret_cast<const unsigned char*>(ring + tile * 2048) + tr_lane;
#pragma unroll
                for (int cc = 0; cc < 2; ++cc)
#pragma unroll
                    for (int dt = 0; dt < 8; ++dt) {
                        // K image unit (kt2, c, g', r') sits at ((kt2 * 4 + c) * 64 + g' * 16 + r') * 16 bytes
                        const unsigned char* at = ktile + ((2 * cc) * 4 + (dt >> 1)) * 1024 + (dt & 1) * 512;
                        const short4q lo = dq_read_tr(at), hi = dq_read_tr(at + 4096);
                        elem8 kt_f;
                        __builtin_memcpy(&kt_f, &lo, 8);
                        __builtin_memcpy(reinterpret_cast<unsigned char*>(&kt_f) + 8, &hi, 8);
                        dq[dt] = IV2_MFMA(kt_f, dsf[cc], dq[dt], 0, 0, 0);
                    }
            }
            j0 = j1;
            tile ^= 1;
        }
        k_ahead = false;
        if (jp >= 0) {                                         // per wavefront
            {
                const elem_bits* vsrc = p.vimg_r + img0 + static_cast<int64_t>(jp) * kImageElems;
#pragma unroll
                for (int f = 0; f < 16; ++f) vreg[f] = *reinterpret_cast<const elem8*>(vsrc + f * 512);
            }
            floatx4 s[4], dp[4];
#pragma unroll
            for (int kt = 0; kt < 4; ++kt) {
                s[kt] = floatx4{0.f, 0.f, 0.f, 0.f};
                dp[kt] = neg_dsum;
            }
#pragma unroll
            for (int c = 0; c < 4; ++c)
#pragma unroll
                for (int kt = 0; kt < 4; ++kt)
                    s[kt] = IV2_MFMA(kreg[kt * 4 + c], qf[c], s[kt], 0, 0, 0);
#pragma unroll
            for (int f = 0; f < 8; ++f) {                      // keys 0..31 of K -> private tile
                uint4 raw;
                __builtin_memcpy(&raw, &kreg[f], 16);
                mine[f * 64] = raw;
            }
#pragma unroll
            for (int c = 0; c < 4; ++c)
#pragma unroll
                for (int kt = 0; kt < 4; ++kt)
                    dp[kt] = IV2_MFMA(vreg[kt * 4 + c], dof[c], dp[kt], 0, 0, 0);
            elem8 dsf[2];
            ds_tile(s, dp, dsf, (jp == last_blk) ? last_key - jp * kBlockN : kBlockN - 1, g, p.scale_log2, lse2);
#pragma unroll
            for (int cc = 0; cc < 2; ++cc) {
                if (cc == 1) {
#pragma unroll
                    for (int f = 0; f < 8; ++f) {              // keys 32..63 (LDS executes a wavefront's accesses in order)
                        uint4 raw;
                        __builtin_memcpy(&raw, &kreg[8 + f], 16);
                        mine[f * 64] = raw;
                    }
                }
#pragma unroll
                for (int dt = 0; dt < 8; ++dt) {
                    const unsigned char* at = mine_tr + (dt >> 1) * 1024 + (dt & 1) * 512;
                    const short4q lo = dq_read_tr(at), hi = dq_read_tr(at + 4096);
                    elem8 kt_f;
                    __builtin_memcpy(&kt_f, &lo, 8);
                    __builtin_memcpy(reinterpret_cast<unsigned char*>(&kt_f) + 8, &hi, 8);
                    dq[dt] = IV2_MFMA(kt_f, dsf[cc], dq[dt], 0, 0, 0);
                }
            }
            // the K fragments of the next own block go out last: they are the only ordinary loads in flight when the
            // next turn waits for its DMA
            const int jn = next_own();
            if (jn >= 0) {
                const elem_bits* ksrc = p.kimg + img0 + static_cast<int64_t>(jn) * kImageElems;
#pragma unroll
                for (int f = 0; f < 16; ++f) kreg[f] = *reinterpret_cast<const elem8*>(ksrc + f * 512);
                k_ahead = true;
            }
            jp = jn;
        }
    }
    if (!live || n >= p.group) return;

    elem_bits* op = p.dq + tok * p.dq_tok + h * p.dq_kvh + n * p.dq_grp + 4 * g;
#pragma unroll
    for (int dt = 0; dt < 8; ++dt) {
        uint2 wv;
        wv.x = pack_elem2(dq[dt][0] * p.scale, dq[dt][1] * p.scale);
        wv.y = pack_elem2(dq[dt][2] * p.scale, dq[dt][3] * p.scale);
        *reinterpret_cast<uint2*>(op + 16 * dt) = wv;
    }
}

int launch_bwd_dq_hybrid(hipStream_t st, const BwdParams& p, int batch, int max_seqlen_q, bool causal) {
    DqExtra x{};
    x.batch = batch;
    x.groups_per_seq = (max_seqlen_q + kDqTokens - 1) / kDqTokens;
    const int64_t total = static_cast<int64_t>(p.num_heads_k) * batch * x.groups_per_seq;
    IV2_CHECK(total <= 0x3fffffff, "varlen_bwd: too many token groups");
    IV2_CHECK(p.k_blocks <= kDqMaskWords * 64, "varlen_bwd: more than %d key blocks per sequence", kDqMaskWords * 64);
    x.total_groups = static_cast<int>(total);
    x.mask_words = (p.k_blocks + 63) / 64 > 0 ? (p.k_blocks + 63) / 64 : 1;
    const int64_t per_round = 8 * kDqChunk;
    const int64_t grid = (total + per_round - 1) / per_round * per_round;
    const size_t lds = kDqLdsTiles + static_cast<size_t>(1 + kDqTokens) * x.mask_words * 8;
    const void* fn = causal ? reinterpret_cast<const void*>(&bwd_dq_hybrid_kernel<true>)
                            : reinterpret_cast<const void*>(&bwd_dq_hybrid_kernel<false>);
    hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds));
    IV2_CHECK(e == hipSuccess, "varlen_bwd: cannot reserve %zu bytes of LDS: %s", lds, hipGetErrorString(e));
    if (causal) hipLaunchKernelGGL(bwd_dq_hybrid_kernel<true>, dim3(static_cast<unsigned>(grid)), dim3(512), lds, st, p, x);
    else hipLaunchKernelGGL(bwd_dq_hybrid_kernel<false>, dim3(static_cast<unsigned>(grid)), dim3(512), lds, st, p, x);
    IV2_LAUNCH_CHECK();
    return 0;
}

}  // namespace IV2_NS
