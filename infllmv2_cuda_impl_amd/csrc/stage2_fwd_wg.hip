// Stage-2 forward, workgroup-shared variant (gfx950).
//
// Same mathematics and register layout as stage2_fwd_kernel (stage2_fwd.hip); what changes is who
// fetches K/V.  A workgroup of 8 wavefronts owns 16 consecutive tokens of one sequence and KV
// head (2 tokens per wavefront).  It ORs the 16 mask rows into a union row and walks the union in
// ascending block order: every block of the union is copied once, cooperatively, from its
// fragment-major image into a double-buffered LDS tile (a flat 32 KiB copy, conflict-free
// ds_read_b128 afterwards), and each wavefront runs the MFMAs only for those of its tokens whose
// own row has the bit.  The forced blocks (initial block + local window), which all 16 tokens
// share, are therefore read from L2 once per 16 tokens instead of 16 times, and inside a
// wavefront one K/V operand read feeds both tokens' MFMAs.
//
// Workgroups are numbered so that the 8 XCDs each take whole chunks of 32 consecutive token
// groups of one KV head (their L2s see one head's images and neighbouring local windows), and
// the longest causal prefixes are scheduled first.
#include "common.h"
#include "kv_image.h"
#include "block_walker.h"
#include "stage2_fwd.h"
#include <math.h>
#include <stdlib.h>

namespace infllmv2 {

constexpr int kChunkGroups = 32;                               // token groups per XCD chunk
constexpr int kImgUnits = 2048;                                // 16-byte units of one K + V image pair

struct SharedFwdExtra {
    int groups_per_seq;                                        // ceil(max_seqlen_q / tokens per workgroup)
    int batch;
    int num_heads_k;
    int nw_alloc;                                              // mask words reserved per row in LDS
    int total_groups;                                          // num_heads_k * batch * groups_per_seq
};

// online-softmax update of one token's 16 x 64 score tile; returns P as the B operand of P.V
__device__ __forceinline__ void softmax_tile(floatx4 (&s)[4], float& m, float& l, floatx4 (&o)[8], bf16x8 (&pf)[2],
                                             int lim, int g, float scale_log2) {
    if (lim < kBlockN - 1) {
#pragma unroll
        for (int kt = 0; kt < 4; ++kt)
#pragma unroll
            for (int e = 0; e < 4; ++e)
                if (16 * kt + 4 * g + e > lim) s[kt][e] = -INFINITY;
    }
    float mx = -INFINITY;
#pragma unroll
    for (int kt = 0; kt < 4; ++kt)
#pragma unroll
        for (int e = 0; e < 4; ++e) mx = fmaxf(mx, s[kt][e]);
    mx = wave_max_over_g(mx);
    const float m_new = fmaxf(m, mx * scale_log2);
    const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
    const float alpha = __builtin_amdgcn_exp2f(m - m_use);
    float rs = 0.f;
#pragma unroll
    for (int kt = 0; kt < 4; ++kt)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const float pv = __builtin_amdgcn_exp2f(s[kt][e] * scale_log2 - m_use);
            s[kt][e] = pv;
            rs += pv;
        }
    l = l * alpha + rs;
    m = m_new;
#pragma unroll
    for (int dt = 0; dt < 8; ++dt) o[dt] *= alpha;
#pragma unroll
    for (int cc = 0; cc < 2; ++cc)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            pf[cc][e] = static_cast<__bf16>(s[2 * cc][e]);
            pf[cc][4 + e] = static_cast<__bf16>(s[2 * cc + 1][e]);
        }
}

template <bool kDoA, bool kDoB>
__device__ __forceinline__ void process_block(const uint4* kb, const uint4* vb, int lane, int g,
                                              const bf16x8 (&qA)[4], const bf16x8 (&qB)[4], floatx4 (&oA)[8],
                                              floatx4 (&oB)[8], float& mA, float& mB, float& lA, float& lB,
                                              int limA, int limB, float scale_log2) {
    floatx4 sA[4], sB[4];
#pragma unroll
    for (int kt = 0; kt < 4; ++kt) {
        sA[kt] = floatx4{0.f, 0.f, 0.f, 0.f};
        sB[kt] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            const uint4 raw = kb[(kt * 4 + c) * 64 + lane];
            bf16x8 kf;
            __builtin_memcpy(&kf, &raw, 16);
            if (kDoA) sA[kt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf, qA[c], sA[kt], 0, 0, 0);
            if (kDoB) sB[kt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf, qB[c], sB[kt], 0, 0, 0);
        }
    }
    bf16x8 pA[2], pB[2];
    if (kDoA) softmax_tile(sA, mA, lA, oA, pA, limA, g, scale_log2);
    if (kDoB) softmax_tile(sB, mB, lB, oB, pB, limB, g, scale_log2);
#pragma unroll
    for (int dt = 0; dt < 8; ++dt)
#pragma unroll
        for (int cc = 0; cc < 2; ++cc) {
            const uint4 raw = vb[(dt * 2 + cc) * 64 + lane];
            bf16x8 vf;
            __builtin_memcpy(&vf, &raw, 16);
            if (kDoA) oA[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, pA[cc], oA[dt], 0, 0, 0);
            if (kDoB) oB[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, pB[cc], oB[dt], 0, 0, 0);
        }
}

__device__ __forceinline__ uint64_t uniform64(uint64_t v) {
    const uint32_t lo = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(v));
    const uint32_t hi = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(v >> 32));
    return (static_cast<uint64_t>(hi) << 32) | lo;
}

__device__ __forceinline__ uint32_t lds_address(const void* ptr) {
    return static_cast<uint32_t>(reinterpret_cast<uintptr_t>((__attribute__((address_space(3))) const void*)ptr));
}

// One wavefront copies 4 KiB from global memory straight into LDS (no registers): lane l moves bytes
// [16 l, 16 l + 16) of each 1 KiB quarter; the destination base travels in M0.  The compiler does not
// see these loads, so the callers order them by hand with s_waitcnt vmcnt(n) + barrier.
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

constexpr int kWaitVm4 = 0x0F74;                               // s_waitcnt vmcnt(4), other counters untouched
constexpr int kWaitVm0 = 0x0F70;                               // s_waitcnt vmcnt(0)

template <bool kCausal, int kTW>
__global__ __launch_bounds__(512)
void stage2_fwd_shared_kernel(const FwdParams p, const SharedFwdExtra x) {
    constexpr int kTokWG = 8 * kTW;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
    uint4* img = reinterpret_cast<uint4*>(smem_raw);                               // [3][2048]: K units 0..1023, V units 1024..2047
    unsigned long long* uni = reinterpret_cast<unsigned long long*>(smem_raw + 3 * kImgUnits * 16);
    unsigned long long* rows = uni + x.nw_alloc;                                   // [kTokWG][nw_alloc]

    // ---- which tokens: XCD-chunked, heaviest first ----
    const int bid = blockIdx.x;
    const int xcd = bid & 7, s = bid >> 3;
    int G = ((s / kChunkGroups) * 8 + xcd) * kChunkGroups + (s % kChunkGroups);
    if (G >= x.total_groups) return;                                               // uniform per workgroup
    G = x.total_groups - 1 - G;
    const int grp = G % x.groups_per_seq;
    const int hb = G / x.groups_per_seq;
    const int b = hb % x.batch, h = hb / x.batch;

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int n = lane & 15, g = lane >> 4;
    const int q0 = p.cu_seqlens_q[b];
    const int Sq = p.cu_seqlens_q[b + 1] - q0;
    const int i0 = grp * kTokWG;
    if (i0 >= Sq) return;                                                          // uniform per workgroup
    const int Sk = p.cu_seqlens_k[b + 1] - p.cu_seqlens_k[b];

    int tok_i[kTW], last_key[kTW], last_blk[kTW];
    bool live[kTW];
#pragma unroll
    for (int t = 0; t < kTW; ++t) {
        tok_i[t] = i0 + kTW * wave + t;
        live[t] = tok_i[t] < Sq;
        int lk = kCausal ? (tok_i[t] + Sk - Sq) : (Sk - 1);
        if (lk > Sk - 1) lk = Sk - 1;
        if (!live[t]) lk = -1;
        last_key[t] = lk;
        last_blk[t] = lk < 0 ? -1 : (lk >> 6);
    }
    int wg_last;                                                                   // largest last_blk in the workgroup
    {
        const int i_last = (i0 + kTokWG - 1 < Sq) ? i0 + kTokWG - 1 : Sq - 1;
        int lk = kCausal ? (i_last + Sk - Sq) : (Sk - 1);
        if (lk > Sk - 1) lk = Sk - 1;
        wg_last = lk < 0 ? -1 : (lk >> 6);
    }
    int nw = wg_last < 0 ? 0 : (wg_last >> 6) + 1;
    if (nw > x.nw_alloc) nw = x.nw_alloc;

    for (int w = tid; w < nw; w += 512) uni[w] = 0ull;
    __syncthreads();
#pragma unroll
    for (int t = 0; t < kTW; ++t) {
        const int64_t tok = static_cast<int64_t>(q0) + (live[t] ? tok_i[t] : 0);
        const uint64_t* mrow = p.mask ? p.mask + (static_cast<int64_t>(h) * p.total_q + tok) * p.n64 : nullptr;
        for (int w = lane; w < nw; w += 64) {
            uint64_t v = 0ull;
            if (last_blk[t] >= 0 && w <= (last_blk[t] >> 6)) {
                v = mrow ? mrow[w] : ~0ull;
                if (w == (last_blk[t] >> 6)) {
                    const int tb = last_blk[t] & 63;
                    v &= (tb == 63) ? ~0ull : ((1ull << (tb + 1)) - 1ull);
                }
            }
            rows[(kTW * wave + t) * x.nw_alloc + w] = v;
            if (v != 0ull) atomicOr(&uni[w], static_cast<unsigned long long>(v));
        }
    }
    __syncthreads();

    // ---- Q operands (dead tokens read a live row and never compute) ----
    bf16x8 qf[kTW][4];
#pragma unroll
    for (int t = 0; t < kTW; ++t) {
        const int64_t tok = static_cast<int64_t>(q0) + (live[t] ? tok_i[t] : i0);
        const bf16_bits* qp = p.q + tok * p.q_tok_stride + h * p.q_kvh_stride + n * p.q_grp_stride + 8 * g;
#pragma unroll
        for (int c = 0; c < 4; ++c) qf[t][c] = *reinterpret_cast<const bf16x8*>(qp + 32 * c);
    }
    float m[kTW], l[kTW];
    floatx4 o[kTW][8];
#pragma unroll
    for (int t = 0; t < kTW; ++t) {
        m[t] = -INFINITY;
        l[t] = 0.f;
#pragma unroll
        for (int dt = 0; dt < 8; ++dt) o[t][dt] = floatx4{0.f, 0.f, 0.f, 0.f};
    }

    // ---- walk the union; tiles are filled two blocks ahead by LDS DMA ----
    const int64_t slot0 = static_cast<int64_t>(h) * p.n_slots + image_slot0(p.cu_seqlens_k, b);
    const uint4* src_lane = (wave < 4 ? reinterpret_cast<const uint4*>(p.kimg) + slot0 * 1024 + wave * 256
                                      : reinterpret_cast<const uint4*>(p.vimg) + slot0 * 1024 + (wave - 4) * 256) + lane;
    const uint32_t ring_base = __builtin_amdgcn_readfirstlane(lds_address(img) + wave * 4096);
    auto issue = [&](int jj, int tile) { dma_copy_4k(src_lane + static_cast<int64_t>(jj) * 1024, ring_base + tile * (kImgUnits * 16)); };

    int cw = -1, row_w = -1;
    uint64_t ubits = 0ull;
    uint64_t word[kTW];
#pragma unroll
    for (int t = 0; t < kTW; ++t) word[t] = 0ull;
    auto next_block = [&]() -> int {
        while (ubits == 0ull) {
            if (++cw >= nw) return -1;
            ubits = uniform64(uni[cw]);
        }
        const int bit = __builtin_ctzll(ubits);
        ubits &= ubits - 1ull;
        return cw * 64 + bit;
    };

    // all ordinary loads (Q operands) land before the first LDS-DMA: otherwise the compiler's own wait for
    // them sits inside the loop and drains the DMA loads that are meant to stay in flight
    __builtin_amdgcn_s_waitcnt(kWaitVm0);
#pragma unroll
    for (int t = 0; t < kTW; ++t)
#pragma unroll
        for (int c = 0; c < 4; ++c) asm volatile("" : "+v"(qf[t][c]));
    int j0 = next_block();
    int j1 = j0 >= 0 ? next_block() : -1;
    if (j0 >= 0) issue(j0, 0);
    if (j1 >= 0) issue(j1, 1);
    int tile = 0;
    while (j0 >= 0) {
        if (j1 >= 0) __builtin_amdgcn_s_waitcnt(kWaitVm4); else __builtin_amdgcn_s_waitcnt(kWaitVm0);
        __syncthreads();                                       // block j0 is in LDS for everyone; tile (tile+2)%3 is free
        const int j2 = j1 >= 0 ? next_block() : -1;
        if (j2 >= 0) issue(j2, tile >= 1 ? tile - 1 : 2);
        if ((j0 >> 6) != row_w) {
            row_w = j0 >> 6;
#pragma unroll
            for (int t = 0; t < kTW; ++t) word[t] = uniform64(rows[(kTW * wave + t) * x.nw_alloc + row_w]);
        }
        const uint4* kb = img + tile * kImgUnits;
        const uint4* vb = kb + 1024;
#pragma unroll
        for (int pr = 0; pr < kTW / 2; ++pr) {
            const int tA = 2 * pr, tB = 2 * pr + 1;
            const bool doA = (word[tA] >> (j0 & 63)) & 1ull;
            const bool doB = (word[tB] >> (j0 & 63)) & 1ull;
            const int limA = (j0 == last_blk[tA]) ? last_key[tA] - j0 * kBlockN : kBlockN;
            const int limB = (j0 == last_blk[tB]) ? last_key[tB] - j0 * kBlockN : kBlockN;
            if (doA && doB)
                process_block<true, true>(kb, vb, lane, g, qf[tA], qf[tB], o[tA], o[tB], m[tA], m[tB], l[tA], l[tB], limA, limB, p.scale_log2);
            else if (doA)
                process_block<true, false>(kb, vb, lane, g, qf[tA], qf[tB], o[tA], o[tB], m[tA], m[tB], l[tA], l[tB], limA, limB, p.scale_log2);
            else if (doB)
                process_block<false, true>(kb, vb, lane, g, qf[tA], qf[tB], o[tA], o[tB], m[tA], m[tB], l[tA], l[tB], limA, limB, p.scale_log2);
        }
        j0 = j1;
        j1 = j2;
        tile = tile == 2 ? 0 : tile + 1;
    }

    // ---- epilogue ----
#pragma unroll
    for (int t = 0; t < kTW; ++t) {
        if (!live[t]) continue;
        const int64_t tok = static_cast<int64_t>(q0) + tok_i[t];
        const float l_tot = wave_sum_over_g(l[t]);
        const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
        bf16_bits* op = p.out + tok * p.o_tok_stride + h * p.o_kvh_stride + n * p.o_grp_stride + 4 * g;
#pragma unroll
        for (int dt = 0; dt < 8; ++dt) {
            uint2 w;
            w.x = pack_bf16x2(o[t][dt][0] * inv, o[t][dt][1] * inv);
            w.y = pack_bf16x2(o[t][dt][2] * inv, o[t][dt][3] * inv);
            *reinterpret_cast<uint2*>(op + 16 * dt) = w;
        }
        if (g == 0) {
            const float lse = l_tot > 0.f ? m[t] * 0.69314718055994530942f + logf(l_tot) : INFINITY;
            p.lse[h * p.lse_kvh_stride + tok * p.lse_tok_stride + n * p.lse_grp_stride] = lse;
        }
    }
}

template <bool kCausal, int kTW>
static int launch_variant(hipStream_t st, const FwdParams& p, SharedFwdExtra x, int max_seqlen_q) {
    constexpr int kTokWG = 8 * kTW;
    x.groups_per_seq = (max_seqlen_q + kTokWG - 1) / kTokWG;
    const int64_t total = static_cast<int64_t>(x.num_heads_k) * x.batch * x.groups_per_seq;
    IV2_CHECK(total <= 0x3fffffff, "varlen_fwd: too many token groups");
    x.total_groups = static_cast<int>(total);
    const int64_t per_round = 8 * kChunkGroups;
    const int64_t grid = (total + per_round - 1) / per_round * per_round;
    const size_t lds = 3 * kImgUnits * 16 + static_cast<size_t>(1 + kTokWG) * x.nw_alloc * 8;
    IV2_CHECK(lds <= 160 * 1024, "varlen_fwd: mask rows too wide for LDS (%d words)", x.nw_alloc);
    const void* fn = reinterpret_cast<const void*>(&stage2_fwd_shared_kernel<kCausal, kTW>);
    hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds));
    IV2_CHECK(e == hipSuccess, "varlen_fwd: cannot reserve %zu bytes of LDS: %s", lds, hipGetErrorString(e));
    hipLaunchKernelGGL((stage2_fwd_shared_kernel<kCausal, kTW>), dim3(static_cast<unsigned>(grid)), dim3(512), lds, st, p, x);
    IV2_LAUNCH_CHECK();
    return 0;
}

int launch_stage2_fwd_shared(hipStream_t st, const FwdParams& p, int batch, int num_heads_k, int max_seqlen_q,
                             int max_seqlen_k, bool causal) {
    SharedFwdExtra x{};
    x.batch = batch;
    x.num_heads_k = num_heads_k;
    const int k_blocks = (max_seqlen_k + kBlockN - 1) / kBlockN;
    x.nw_alloc = p.mask ? p.n64 : (k_blocks + 63) / 64;
    if (x.nw_alloc < 1) x.nw_alloc = 1;
    static const int tokens_per_wave = [] {                    // diagnostic switch: 2 or 4 tokens per wavefront
        const char* e = getenv("INFLLMV2_FWD_TOKENS_PER_WAVE");
        return (e != nullptr && e[0] == '4') ? 4 : 2;
    }();
    if (tokens_per_wave == 4)
        return causal ? launch_variant<true, 4>(st, p, x, max_seqlen_q) : launch_variant<false, 4>(st, p, x, max_seqlen_q);
    return causal ? launch_variant<true, 2>(st, p, x, max_seqlen_q) : launch_variant<false, 2>(st, p, x, max_seqlen_q);
}

}  // namespace infllmv2
