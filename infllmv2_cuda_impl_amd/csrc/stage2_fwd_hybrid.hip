// Stage-2 forward, workgroup-hybrid kernel (gfx950).
//
// Same mathematics and register layout as stage2_fwd_kernel (stage2_fwd.hip: one wavefront owns
// one token, S^T = K Q^T, O^T = V^T P^T, online softmax); what changes is who fetches K/V.
// A workgroup of 8 wavefronts owns 8 consecutive tokens of one sequence and KV head and splits
// each token's mask row in two:
//
//   * the blocks that ALL 8 rows select (for InfLLM-V2 masks: the initial block and the local
//     window, which neighbouring tokens share) are walked in lock step: every such block is
//     copied once, by LDS-DMA, from its fragment-major image into a 4-tile LDS ring (two blocks in
//     use, the next two in flight: one workgroup barrier per two blocks), and each wavefront
//     reads its MFMA operands with conflict-free ds_read_b128;
//   * the remaining blocks of a row are walked by its wavefront alone, operands straight from
//     global memory into registers, as in stage2_fwd_kernel;
//   * the two walks are interleaved, common, own, common, own per turn: the first is bound by
//     the matrix pipeline and the VALU, the second by the vector memory path.
//
// A per-token kernel is bound by what the vector memory path can deliver (32 KiB of operands per
// 512 MFMA cycles); the shared walk takes the common half of the work off that path.  Online
// softmax is order-independent, so the split changes nothing in the result.
//
// Workgroups are numbered so that each of the 8 XCDs takes whole chunks of consecutive token
// groups of one KV head (their L2 sees one head's images and neighbouring local windows), and
// the longest causal prefixes are scheduled first.
#include "common.h"
#include "kv_image.h"
#include "block_walker.h"
#include "stage2_fwd.h"
#include <math.h>

namespace IV2_NS {

constexpr int kHybTokens = 8;                                  // tokens (= wavefronts) per workgroup
constexpr int kHybChunk = 16;                                  // token groups per XCD chunk
constexpr int kRingTiles = 4;
constexpr int kTileBytes = 32768;                              // K image | V image of one block
constexpr int kMaxMaskWords = 256;                             // LDS copies of the mask rows hold at most this many words each: 16384 key blocks

struct HybridExtra {
    int groups_per_seq;                                        // ceil(max_seqlen_q / kHybTokens)
    int batch;
    int total_groups;                                          // num_heads_k * batch * groups_per_seq
    int mask_words;                                            // words per LDS mask row: what max_seqlen_k needs, not the maximum
};

__device__ __forceinline__ uint32_t lds_address_of(const void* ptr) {
    return static_cast<uint32_t>(reinterpret_cast<uintptr_t>((__attribute__((address_space(3))) const void*)ptr));
}
// One wavefront copies 4 KiB from global memory straight into LDS (no registers): lane l moves bytes
// [16 l, 16 l + 16) of each 1 KiB quarter (the instruction offset advances source and destination alike).
// The compiler does not see these loads; callers order them by hand with s_waitcnt vmcnt(n) + barrier.
__device__ __forceinline__ void dma_copy_4k(const void* src_lane, uint32_t lds_dst) {
    asm volatile("s_mov_b32 m0, %1\n\t"
                 "global_load_lds_dwordx4 %0, off\n\t"
                 "global_load_lds_dwordx4 %0, off offset:1024\n\t"
                 "global_load_lds_dwordx4 %0, off offset:2048\n\t"
                 "global_load_lds_dwordx4 %0, off offset:3072\n\t"
                 :
                 : "v"(src_lane), "s"(lds_dst)
                 : "memory", "m0");
}
__device__ __forceinline__ uint64_t uniform_u64(uint64_t v) {
    const uint32_t lo = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(v));
    const uint32_t hi = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(v >> 32));
    return (static_cast<uint64_t>(hi) << 32) | lo;
}

// Online-softmax update with one 16 x 64 score tile (s: S^T accumulators); returns P as the B operand of P.V.
//
// m is the REFERENCE exponent of the lane's head (log2 units, the same in the four lanes that share a head), not
// necessarily its running maximum: P = exp2(scale s - m), l and O are all kept relative to m, and out = O / l and
// LSE = m ln2 + log l hold for any finite m.  So the common path takes m as it is - no row maximum, no cross-lane
// exchange, no rescale of O - and only checks afterwards that its sixteen P values stayed small (their sum is needed
// anyway): a lane whose sum exceeds 2^kLazyBits, or whose head has no reference yet, sends the wavefront through the
// exact path, which moves m to the true running maximum and rescales.  P is rounded to the element type relative to
// m: its relative rounding error does not depend on the offset, and fp32 l and O have room for 2^kLazyBits many times over.
constexpr float kLazyLimit = 64.f;                             // 2^6

__device__ __forceinline__ void softmax_step(floatx4 (&s)[4], float& m, float& l, floatx4 (&o)[8], elem8 (&pf)[2],
                                             int lim, int g, float scale_log2) {
    if (lim < kBlockN - 1) {
#pragma unroll
        for (int kt = 0; kt < 4; ++kt)
#pragma unroll
            for (int e = 0; e < 4; ++e)
                if (16 * kt + 4 * g + e > lim) s[kt][e] = -INFINITY;
    }
    floatx4 pv[4];
    float rs = 0.f;
#pragma unroll
    for (int kt = 0; kt < 4; ++kt)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            pv[kt][e] = __builtin_amdgcn_exp2f(__builtin_fmaf(s[kt][e], scale_log2, -m));   // m = -inf (no reference yet): +inf or NaN, caught below
            rs += pv[kt][e];
        }
    if (__ballot(!(rs <= kLazyLimit)) != 0ull) {               // rare after a row's first blocks; also catches NaN
        float mx = -INFINITY;
#pragma unroll
        for (int kt = 0; kt < 4; ++kt)
#pragma unroll
            for (int e = 0; e < 4; ++e) mx = fmaxf(mx, s[kt][e]);
        mx = wave_max_over_g(mx);
        const float m_new = fmaxf(m, mx * scale_log2);
        const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
        const float alpha = __builtin_amdgcn_exp2f(m - m_use);  // 0 when there was no reference
        rs = 0.f;
#pragma unroll
        for (int kt = 0; kt < 4; ++kt)
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                pv[kt][e] = __builtin_amdgcn_exp2f(__builtin_fmaf(s[kt][e], scale_log2, -m_use));
                rs += pv[kt][e];
            }
        l *= alpha;
        m = m_new;
#pragma unroll
        for (int dt = 0; dt < 8; ++dt) o[dt] *= alpha;
    }
    l += rs;
#pragma unroll
    for (int cc = 0; cc < 2; ++cc)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            pf[cc][e] = static_cast<elem_t>(pv[2 * cc][e]);
            pf[cc][4 + e] = static_cast<elem_t>(pv[2 * cc + 1][e]);
        }
}

template <bool kCausal>
__global__ __launch_bounds__(512)
void stage2_fwd_hybrid_kernel(const FwdParams p, const HybridExtra x) {
    extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
    uint4* ring = reinterpret_cast<uint4*>(smem_raw);                               // [kRingTiles][2048]: K units 0..1023, V units 1024..2047
    unsigned long long* com = reinterpret_cast<unsigned long long*>(smem_raw + kRingTiles * kTileBytes);   // [mask_words]
    unsigned long long* rows = com + x.mask_words;                                  // [kHybTokens][mask_words]

    // ---- which tokens: XCD-chunked, heaviest first ----
    const int bid = blockIdx.x;
    const int xcd = bid & 7, sidx = bid >> 3;
    int G = ((sidx / kHybChunk) * 8 + xcd) * kHybChunk + (sidx % kHybChunk);
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
    const int i0 = grp * kHybTokens;
    if (i0 >= Sq) return;                                                           // uniform per workgroup
    const int Sk = p.cu_seqlens_k[b + 1] - p.cu_seqlens_k[b];

    const int i = i0 + wave;                                                        // this wavefront's token
    const bool live = i < Sq;
    int last_key = kCausal ? (i + Sk - Sq) : (Sk - 1);                              // largest allowed key index
    if (last_key > Sk - 1) last_key = Sk - 1;
    if (!live) last_key = -1;
    const int last_blk = last_key < 0 ? -1 : (last_key >> 6);
    const int64_t tok = static_cast<int64_t>(q0) + (live ? i : i0);
    const uint64_t* mrow = p.mask ? p.mask + (static_cast<int64_t>(h) * p.total_q + tok) * p.n64 : nullptr;

    // ---- the row words every live token of the group has in common, and what is left of each row ----
    int nw;                                                                          // words that can hold an allowed block of any token
    {
        const int i_last = (i0 + kHybTokens - 1 < Sq) ? i0 + kHybTokens - 1 : Sq - 1;
        int lk = kCausal ? (i_last + Sk - Sq) : (Sk - 1);
        if (lk > Sk - 1) lk = Sk - 1;
        nw = lk < 0 ? 0 : (lk >> 12) + 1;
        if (mrow && nw > p.n64) nw = p.n64;
        if (nw > x.mask_words) nw = x.mask_words;                                    // a sequence longer than the announced max_seqlen_k
    }
    unsigned long long* own = rows + wave * x.mask_words;                           // this token's row, later minus the common part
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

    // ---- Q operand ----
    elem8 qf[4];
    {
        const int nq = n < p.group ? n : p.group - 1;
        const elem_bits* qp = p.q + tok * p.q_tok_stride + h * p.q_kvh_stride + nq * p.q_grp_stride + 8 * g;
#pragma unroll
        for (int c = 0; c < 4; ++c) qf[c] = *reinterpret_cast<const elem8*>(qp + 32 * c);
    }
    float m = -INFINITY, l = 0.f;
    floatx4 o[8];
#pragma unroll
    for (int dt = 0; dt < 8; ++dt) o[dt] = floatx4{0.f, 0.f, 0.f, 0.f};

    const int64_t slot0 = static_cast<int64_t>(h) * p.n_slots + image_slot0(p.cu_seqlens_k, b);

    // ---- the walk: one turn = two common blocks (lock step, operands from the LDS ring) alternating with two own
    //      blocks (operands from global memory into registers).  The own blocks' loads keep the vector memory path
    //      busy while the matrix pipeline works on a common block, and the other way round. ----
    const uint4* src_lane = (wave < 4 ? reinterpret_cast<const uint4*>(p.kimg) + slot0 * 1024 + wave * 256
                                      : reinterpret_cast<const uint4*>(p.vimg) + slot0 * 1024 + (wave - 4) * 256) + lane;
    const uint32_t ring_base = __builtin_amdgcn_readfirstlane(lds_address_of(ring) + wave * 4096);
    auto issue = [&](int jj, int tile) { dma_copy_4k(src_lane + static_cast<int64_t>(jj) * 1024, ring_base + tile * kTileBytes); };
    int cw = -1, ow = -1;
    uint64_t cbits = 0ull, obits = 0ull;
    auto next_common = [&]() -> int {
        while (cbits == 0ull) {
            if (++cw >= nw) return -1;
            cbits = uniform_u64(com[cw]);
        }
        const int bit = __builtin_ctzll(cbits);
        cbits &= cbits - 1ull;
        return cw * 64 + bit;
    };
    auto next_own = [&]() -> int {
        while (obits == 0ull) {
            if (++ow >= nw) return -1;
            obits = uniform_u64(own[ow]);
        }
        const int bit = __builtin_ctzll(obits);
        obits &= obits - 1ull;
        return ow * 64 + bit;
    };
    const elem_bits* kimg = p.kimg + slot0 * kImageElems + lane * 8;
    const elem_bits* vimg = p.vimg + slot0 * kImageElems + lane * 8;
    elem8 kreg[16], vreg[16];
    int jp = live ? next_own() : -1;                           // own block of this turn; its K fragments are loaded a turn ahead
    if (jp >= 0) {
        const elem_bits* src = kimg + static_cast<int64_t>(jp) * kImageElems;
#pragma unroll
        for (int f = 0; f < 16; ++f) kreg[f] = *reinterpret_cast<const elem8*>(src + f * 512);
    }
    // All ordinary loads so far (Q, mask words, first K fragments) land before the first LDS-DMA.  From here on the
    // compiler's wait counts know nothing of the DMA loads; they stay correct because loads complete in order (an
    // unknown younger load only makes a wait stricter), and the waits written by hand below count the ordinary
    // loads that may be younger than the DMA they wait for.
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#pragma unroll
    for (int c = 0; c < 4; ++c) asm volatile("" : "+v"(qf[c]));
#pragma unroll
    for (int f = 0; f < 16; ++f) asm volatile("" : "+v"(kreg[f]));
    // The common blocks go through the ring in pairs: tiles {0, 1} and {2, 3} alternate, the pair after the current
    // one is in flight, and one workgroup barrier serves two blocks.
    int c0 = next_common();
    int c1 = c0 >= 0 ? next_common() : -1;
    if (c0 >= 0) issue(c0, 0);
    if (c1 >= 0) issue(c1, 1);
    int half = 0;
    bool k_ahead = false;                                      // the coming own block's 16 K-fragment loads were issued already
    auto common_part = [&](int j0, int tile) {
        // all 16 fragments of a tile are fetched before the MFMAs that use them (vreg is free between own
        // blocks), and the MFMAs run over independent accumulators first
        const uint4* kb = ring + tile * 2048 + lane;
        const uint4* vb = kb + 1024;
#pragma unroll
        for (int f = 0; f < 16; ++f) {
            const uint4 raw = kb[f * 64];
            __builtin_memcpy(&vreg[f], &raw, 16);
        }
        floatx4 s[4];
#pragma unroll
        for (int kt = 0; kt < 4; ++kt) s[kt] = floatx4{0.f, 0.f, 0.f, 0.f};
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
        elem8 pf[2];
        softmax_step(s, m, l, o, pf, (j0 == last_blk) ? last_key - j0 * kBlockN : kBlockN, g, p.scale_log2);
#pragma unroll
        for (int cc = 0; cc < 2; ++cc)
#pragma unroll
            for (int dt = 0; dt < 8; ++dt)
                o[dt] = IV2_MFMA(vreg[dt * 2 + cc], pf[cc], o[dt], 0, 0, 0);
    };
    auto own_part = [&]() {
        {
            const elem_bits* src = vimg + static_cast<int64_t>(jp) * kImageElems;
#pragma unroll
            for (int f = 0; f < 16; ++f) vreg[f] = *reinterpret_cast<const elem8*>(src + f * 512);
        }
        floatx4 s[4];
#pragma unroll
        for (int kt = 0; kt < 4; ++kt) s[kt] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int c = 0; c < 4; ++c)
#pragma unroll
            for (int kt = 0; kt < 4; ++kt)
                s[kt] = IV2_MFMA(kreg[kt * 4 + c], qf[c], s[kt], 0, 0, 0);
        elem8 pf[2];
        softmax_step(s, m, l, o, pf, (jp == last_blk) ? last_key - jp * kBlockN : kBlockN, g, p.scale_log2);
#pragma unroll
        for (int cc = 0; cc < 2; ++cc)
#pragma unroll
            for (int dt = 0; dt < 8; ++dt)
                o[dt] = IV2_MFMA(vreg[dt * 2 + cc], pf[cc], o[dt], 0, 0, 0);
        const int jn = next_own();
        k_ahead = false;
        if (jn >= 0) {                                         // K fragments of the next own block
            const elem_bits* src = kimg + static_cast<int64_t>(jn) * kImageElems;
#pragma unroll
            for (int f = 0; f < 16; ++f) kreg[f] = *reinterpret_cast<const elem8*>(src + f * 512);
            k_ahead = true;
        }
        jp = jn;
    };
    while (c0 >= 0 || jp >= 0) {
        int n0 = -1, n1 = -1;
        if (c0 >= 0) {                                         // uniform over the workgroup
            // younger than this wavefront's DMA loads of the pair: the 16 K loads of the coming own block
            if (k_ahead) asm volatile("s_waitcnt vmcnt(16)" ::: "memory");
            else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            __syncthreads();                                   // the pair is in LDS for everyone; the other two tiles are free
            n0 = c1 >= 0 ? next_common() : -1;
            n1 = n0 >= 0 ? next_common() : -1;
            if (n0 >= 0) issue(n0, 2 - 2 * half);
            if (n1 >= 0) issue(n1, 3 - 2 * half);
            if (live) common_part(c0, 2 * half);
        }
        if (jp >= 0) own_part();                               // per wavefront
        if (c1 >= 0 && live) common_part(c1, 2 * half + 1);
        if (jp >= 0 && c1 >= 0) own_part();
        if (c0 >= 0) {
            c0 = n0;
            c1 = n1;
            half ^= 1;
        }
    }
    if (!live) return;

    // ---- epilogue ----
    const float l_tot = wave_sum_over_g(l);
    const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
    if (n >= p.group) return;                                  // rows that only fill the MFMA tile
    elem_bits* op = p.out + tok * p.o_tok_stride + h * p.o_kvh_stride + n * p.o_grp_stride + 4 * g;
#pragma unroll
    for (int dt = 0; dt < 8; ++dt) {
        uint2 wv;
        wv.x = pack_elem2(o[dt][0] * inv, o[dt][1] * inv);
        wv.y = pack_elem2(o[dt][2] * inv, o[dt][3] * inv);
        *reinterpret_cast<uint2*>(op + 16 * dt) = wv;
    }
    if (g == 0) {
        const float lse = l_tot > 0.f ? m * 0.69314718055994530942f + logf(l_tot) : INFINITY;
        p.lse[h * p.lse_kvh_stride + tok * p.lse_tok_stride + n * p.lse_grp_stride] = lse;
    }
}

int launch_stage2_fwd_hybrid(hipStream_t st, const FwdParams& p, int batch, int num_heads_k, int max_seqlen_q,
                             int max_seqlen_k, bool causal) {
    HybridExtra x{};
    x.batch = batch;
    x.groups_per_seq = (max_seqlen_q + kHybTokens - 1) / kHybTokens;
    const int64_t total = static_cast<int64_t>(num_heads_k) * batch * x.groups_per_seq;
    IV2_CHECK(total <= 0x3fffffff, "varlen_fwd: too many token groups");
    IV2_CHECK((max_seqlen_k + kBlockN - 1) / kBlockN <= kMaxMaskWords * 64, "varlen_fwd: more than %d key blocks per sequence", kMaxMaskWords * 64);
    x.total_groups = static_cast<int>(total);
    x.mask_words = ((max_seqlen_k + kBlockN - 1) / kBlockN + 63) / 64;
    if (x.mask_words < 1) x.mask_words = 1;
    const int64_t per_round = 8 * kHybChunk;
    const int64_t grid = (total + per_round - 1) / per_round * per_round;
    const size_t lds = kRingTiles * kTileBytes + static_cast<size_t>(1 + kHybTokens) * x.mask_words * 8;
    const void* fn = causal ? reinterpret_cast<const void*>(&stage2_fwd_hybrid_kernel<true>)
                            : reinterpret_cast<const void*>(&stage2_fwd_hybrid_kernel<false>);
    hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds));
    IV2_CHECK(e == hipSuccess, "varlen_fwd: cannot reserve %zu bytes of LDS: %s", lds, hipGetErrorString(e));
    if (causal) hipLaunchKernelGGL(stage2_fwd_hybrid_kernel<true>, dim3(static_cast<unsigned>(grid)), dim3(512), lds, st, p, x);
    else hipLaunchKernelGGL(stage2_fwd_hybrid_kernel<false>, dim3(static_cast<unsigned>(grid)), dim3(512), lds, st, p, x);
    IV2_LAUNCH_CHECK();
    return 0;
}

}  // namespace IV2_NS
