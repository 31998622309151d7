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

namespace infllmv2 {

constexpr int kTokWG = 16;
constexpr int kWavesWG = 8;
constexpr int kChunkGroups = 32;                               // token groups per XCD chunk
constexpr int kImgUnits = 2048;                                // 16-byte units of one K + V image pair

struct SharedFwdExtra {
    int groups_per_seq;                                        // ceil(max_seqlen_q / 16)
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
                                              const bf16x8 (&qf)[2][4], floatx4 (&o)[2][8], float (&m)[2],
                                              float (&l)[2], int limA, int limB, float scale_log2) {
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
            if (kDoA) sA[kt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf, qf[0][c], sA[kt], 0, 0, 0);
            if (kDoB) sB[kt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf, qf[1][c], sB[kt], 0, 0, 0);
        }
    }
    bf16x8 pA[2], pB[2];
    if (kDoA) softmax_tile(sA, m[0], l[0], o[0], pA, limA, g, scale_log2);
    if (kDoB) softmax_tile(sB, m[1], l[1], o[1], pB, limB, g, scale_log2);
#pragma unroll
    for (int dt = 0; dt < 8; ++dt)
#pragma unroll
        for (int cc = 0; cc < 2; ++cc) {
            const uint4 raw = vb[(dt * 2 + cc) * 64 + lane];
            bf16x8 vf;
            __builtin_memcpy(&vf, &raw, 16);
            if (kDoA) o[0][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, pA[cc], o[0][dt], 0, 0, 0);
            if (kDoB) o[1][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, pB[cc], o[1][dt], 0, 0, 0);
        }
}

__device__ __forceinline__ uint64_t uniform64(uint64_t v) {
    const uint32_t lo = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(v));
    const uint32_t hi = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(v >> 32));
    return (static_cast<uint64_t>(hi) << 32) | lo;
}

template <bool kCausal>
__global__ __launch_bounds__(512)
void stage2_fwd_shared_kernel(const FwdParams p, const SharedFwdExtra x) {
    extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
    uint4* img = reinterpret_cast<uint4*>(smem_raw);                               // [2][2048]
    unsigned long long* uni = reinterpret_cast<unsigned long long*>(smem_raw + 2 * kImgUnits * 16);
    unsigned long long* rows = uni + x.nw_alloc;                                   // [16][nw_alloc]

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

    int tok_i[2], last_key[2], last_blk[2];
    bool live[2];
#pragma unroll
    for (int t = 0; t < 2; ++t) {
        tok_i[t] = i0 + 2 * wave + t;
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
    for (int t = 0; t < 2; ++t) {
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
            rows[(2 * wave + t) * x.nw_alloc + w] = v;
            if (v != 0ull) atomicOr(&uni[w], static_cast<unsigned long long>(v));
        }
    }
    __syncthreads();

    // ---- Q operands (dead tokens read a live row and never compute) ----
    bf16x8 qf[2][4];
#pragma unroll
    for (int t = 0; t < 2; ++t) {
        const int64_t tok = static_cast<int64_t>(q0) + (live[t] ? tok_i[t] : i0);
        const bf16_bits* qp = p.q + tok * p.q_tok_stride + h * p.q_kvh_stride + n * p.q_grp_stride + 8 * g;
#pragma unroll
        for (int c = 0; c < 4; ++c) qf[t][c] = *reinterpret_cast<const bf16x8*>(qp + 32 * c);
    }
    float m[2] = {-INFINITY, -INFINITY}, l[2] = {0.f, 0.f};
    floatx4 o[2][8];
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int dt = 0; dt < 8; ++dt) o[t][dt] = floatx4{0.f, 0.f, 0.f, 0.f};

    // ---- walk the union ----
    const int64_t slot0 = static_cast<int64_t>(h) * p.n_slots + image_slot0(p.cu_seqlens_k, b);
    const uint4* kimg = reinterpret_cast<const uint4*>(p.kimg) + slot0 * 1024;
    const uint4* vimg = reinterpret_cast<const uint4*>(p.vimg) + slot0 * 1024;
    int cw = -1;                                                                   // word index being walked
    uint64_t ubits = 0ull, wordA = 0ull, wordB = 0ull;
    auto next_block = [&]() -> int {
        while (ubits == 0ull) {
            if (++cw >= nw) return -1;
            ubits = uniform64(uni[cw]);
        }
        const int bit = __builtin_ctzll(ubits);
        ubits &= ubits - 1ull;
        return cw * 64 + bit;
    };
    uint4 stage[4];
    auto fetch = [&](int j) {
#pragma unroll
        for (int it = 0; it < 4; ++it) {
            const int u = tid + it * 512;
            stage[it] = (u < 1024) ? kimg[static_cast<int64_t>(j) * 1024 + u] : vimg[static_cast<int64_t>(j) * 1024 + (u - 1024)];
        }
    };
    auto deposit = [&](int buf) {
#pragma unroll
        for (int it = 0; it < 4; ++it) img[buf * kImgUnits + tid + it * 512] = stage[it];
    };

    int j = next_block();
    int row_w = -1;
    if (j >= 0) {
        fetch(j);
        deposit(0);
    }
    __syncthreads();
    int cur = 0;
    while (j >= 0) {
        if ((j >> 6) != row_w) {
            row_w = j >> 6;
            wordA = uniform64(rows[(2 * wave) * x.nw_alloc + row_w]);
            wordB = uniform64(rows[(2 * wave + 1) * x.nw_alloc + row_w]);
        }
        const bool doA = (wordA >> (j & 63)) & 1ull;
        const bool doB = (wordB >> (j & 63)) & 1ull;
        // the union walker may already have advanced cw past row_w; remember j before asking for the next
        const int jn = next_block();
        if (jn >= 0) fetch(jn);
        const uint4* kb = img + cur * kImgUnits;
        const uint4* vb = kb + 1024;
        const int limA = (j == last_blk[0]) ? last_key[0] - j * kBlockN : kBlockN;
        const int limB = (j == last_blk[1]) ? last_key[1] - j * kBlockN : kBlockN;
        if (doA && doB) process_block<true, true>(kb, vb, lane, g, qf, o, m, l, limA, limB, p.scale_log2);
        else if (doA) process_block<true, false>(kb, vb, lane, g, qf, o, m, l, limA, limB, p.scale_log2);
        else if (doB) process_block<false, true>(kb, vb, lane, g, qf, o, m, l, limA, limB, p.scale_log2);
        if (jn >= 0) deposit(cur ^ 1);
        __syncthreads();
        j = jn;
        cur ^= 1;
    }

    // ---- epilogue ----
#pragma unroll
    for (int t = 0; t < 2; ++t) {
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

int launch_stage2_fwd_shared(hipStream_t st, const FwdParams& p, int batch, int num_heads_k, int max_seqlen_q,
                             int max_seqlen_k, bool causal) {
    SharedFwdExtra x{};
    x.groups_per_seq = (max_seqlen_q + kTokWG - 1) / kTokWG;
    x.batch = batch;
    x.num_heads_k = num_heads_k;
    const int k_blocks = (max_seqlen_k + kBlockN - 1) / kBlockN;
    x.nw_alloc = p.mask ? p.n64 : (k_blocks + 63) / 64;
    if (x.nw_alloc < 1) x.nw_alloc = 1;
    const int64_t total = static_cast<int64_t>(num_heads_k) * batch * x.groups_per_seq;
    IV2_CHECK(total <= 0x3fffffff, "varlen_fwd: too many token groups");
    x.total_groups = static_cast<int>(total);
    const int64_t per_round = 8 * kChunkGroups;
    const int64_t grid = (total + per_round - 1) / per_round * per_round;
    const size_t lds = 2 * kImgUnits * 16 + static_cast<size_t>(1 + kTokWG) * x.nw_alloc * 8;
    IV2_CHECK(lds <= 160 * 1024, "varlen_fwd: mask rows too wide for LDS (%d words)", x.nw_alloc);
    hipError_t e;
    if (causal) {
        e = hipFuncSetAttribute(reinterpret_cast<const void*>(&stage2_fwd_shared_kernel<true>),
                                hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds));
        IV2_CHECK(e == hipSuccess, "varlen_fwd: cannot reserve %zu bytes of LDS: %s", lds, hipGetErrorString(e));
        hipLaunchKernelGGL(stage2_fwd_shared_kernel<true>, dim3(static_cast<unsigned>(grid)), dim3(512), lds, st, p, x);
    } else {
        e = hipFuncSetAttribute(reinterpret_cast<const void*>(&stage2_fwd_shared_kernel<false>),
                                hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds));
        IV2_CHECK(e == hipSuccess, "varlen_fwd: cannot reserve %zu bytes of LDS: %s", lds, hipGetErrorString(e));
        hipLaunchKernelGGL(stage2_fwd_shared_kernel<false>, dim3(static_cast<unsigned>(grid)), dim3(512), lds, st, p, x);
    }
    IV2_LAUNCH_CHECK();
    return 0;
}

}  // namespace infllmv2
