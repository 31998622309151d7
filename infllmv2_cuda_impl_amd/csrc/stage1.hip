// Stage-1 scoring for gfx950: softmax-like scores of the 16 grouped query heads against the
// compressed keys, normalised by a log-sum-exp taken over a (usually coarser) second key set,
// summed over the 16 heads.
//
// Semantics follow compute_attn_1rowblock_splitkv_stage1
// (csrc/flash_attn/src/flash_fwd_kernel.h:1203-1744), Mask::apply_mask_stage1
// (csrc/flash_attn/src/mask.h:225-319), softmax_rescale_simple / softmax_rescale_gt
// (csrc/flash_attn/src/softmax.h:94-121,198-237) and hdim16_reduce (flash_fwd_kernel.h:53-112):
//   vis_s(i) = min(L, max(0, (i+1)/s - 1 + L - (Sq - s + 1)/s))     (C++ truncating divisions)
//   lse_g(i) = log sum_{c < vis_c(i)} exp(scale * q_g . kc_c),  s = 64, or 16 when Lc == Lk
//   score[h, i, j] = bf16( sum_g exp(scale * q_g . kf_j - lse_g(i)) )   for j < vis_16(i), else 0
//   rows with vis_c(i) == 0 are all zero (the reference's early exit leaves its zero fill).
//
// Design: S = Q.K^T with the 16 heads of one token as the 16 MFMA rows and 16 compressed keys as
// the columns, so a lane owns four heads of one key column; the per-head running max/sum of
// pass 1 stay lane-local until one 16-lane butterfly at the end, and the sum over the 16 heads
// in pass 2 is an in-lane add of four values plus two cross-lane adds.  A workgroup is 8
// wavefronts x 2 consecutive tokens; each 64-key tile of compressed keys is staged once in LDS
// (LDS-DMA, straight into MFMA-operand order, read back with conflict-free ds_read_b128) and reused
// by all 16 tokens, and inside a wavefront one operand read feeds two MFMAs.
#include "common.h"
#include "block_walker.h"
#include "infllmv2_hip.h"
#include <math.h>

namespace IV2_NS {

struct Stage1Params {
    const elem_bits* q;
    const elem_bits* k;              // fine compressed keys   (sum Lk, Hk, d)
    const elem_bits* c;              // coarse compressed keys (sum Lc, Hk, d)
    elem_bits* score;                // (Hk, total_q, row_stride); pooled output: (Hk, total_q, pool_len), dense
    const int* cu_seqlens_q;
    const int* cu_seqlens_k;
    const int* cu_seqlens_c;
    int64_t q_tok_stride, q_grp_stride, q_kvh_stride;
    int64_t k_row_stride, k_head_stride, c_row_stride, c_head_stride;
    int64_t score_head_stride, score_row_stride;
    int score_cols;                  // columns to define in every row (max_seqlen_k)
    float scale_log2;
    int causal;
    int group;                       // query heads per KV head, 1..16: MFMA rows >= group repeat head group - 1 and add nothing
    // pooled output only
    const int* cache_lens;           // per sequence, or null: cache_len for all
    int cache_len;
    int pool_len;                    // key blocks per output row
    int local_blocks, init_blocks;
};

// 8 wavefronts x 2 tokens: 112 registers, so four wavefronts share a SIMD and the exp-heavy VALU work of one hides
// behind the MFMAs of another (4 x 4 at two wavefronts per SIMD measures 6 % slower, 8 x 1 15 % slower)
constexpr int kTokPerWave = 2;
constexpr int kWavesS1 = 8;
constexpr int kWavesPerSimdS1 = 4;
constexpr int kTokPerBlock = kTokPerWave * kWavesS1;   // 16
constexpr int kKeysPerBlock = 4;                       // compressed keys (stride 16) per 64-token key block

__device__ __forceinline__ int trunc_div(int a, int b) { return a / b; }   // C++ semantics on purpose

__device__ __forceinline__ int stage1_visible(int i, int s, int L, int Sq, bool causal) {
    if (!causal) return L;
    const int cq = trunc_div(Sq - s + 1, s);
    int v = (i + 1) / s - 1 + L - cq;
    v = v < 0 ? 0 : v;
    return v < L ? v : L;
}

// A (64 keys x 128 d) tile goes from global memory to LDS by LDS-DMA, in MFMA-operand order: 16-byte unit
// u = (kt*4 + c)*64 + 16*g + n holds K[16*kt + n][32*c + 8*g ..].  Wavefront w of the workgroup moves the 64-unit groups
// grp = w, w + 8 (key tile grp / 4, chunk grp % 4 of its 16 keys): lane l's unit lands at lds_base + 16 l, which is exactly operand order, so the operand reads are linear and free of bank conflicts.
// Keys beyond the last one are read from the last row (finite values that every consumer masks).
// The compiler's wait counts do not see these loads: the code waits for them by hand before the barrier that
// publishes the tile.
__device__ __forceinline__ uint32_t s1_lds_addr(const void* ptr) {
    return static_cast<uint32_t>(reinterpret_cast<uintptr_t>((__attribute__((address_space(3))) const void*)ptr));
}
__device__ __forceinline__ void s1_dma16(const void* base, uint32_t lane_off, uint32_t lds_base) {
    asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dwordx4 %0, %1"
                 : : "v"(lane_off), "s"(base), "s"(lds_base) : "memory", "m0");
}
__device__ __forceinline__ void issue_tile(const elem_bits* base, int row_stride, int key0, int L, uint32_t lds_tile,
                                           int wave, int n, int g) {
#pragma unroll
    for (int it = 0; it < 16 / kWavesS1; ++it) {
        const int grp = it * kWavesS1 + wave;                  // (kt, c) = (grp / 4, grp % 4)
        int row = key0 + 16 * (grp >> 2) + n;
        row = row < L ? row : L - 1;
        const uint32_t off = static_cast<uint32_t>(row * row_stride + 32 * (grp & 3) + 8 * g) * 2u;
        s1_dma16(base, off, lds_tile + grp * 1024);
    }
}

// x, y -> (x's even 16-lane rows interleaved with y's even rows, x's odd rows interleaved with y's odd rows), summed:
// row 2r of the result is x.row(2r) + x.row(2r+1), row 2r+1 is y.row(2r) + y.row(2r+1).
__device__ __forceinline__ float fold_rows16(float x, float y) {
    typedef unsigned u2 __attribute__((ext_vector_type(2)));
    const u2 r = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(y), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}
// rows 0,1 of the result are x.row(r) + x.row(r+2), rows 2,3 are y.row(r-2) + y.row(r)
__device__ __forceinline__ float fold_rows32(float x, float y) {
    typedef unsigned u2 __attribute__((ext_vector_type(2)));
    const u2 r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(y), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}
// value of lane (n + k) % 16 of the same 16-lane row (DPP row_ror:k)
template <int kRot>
__device__ __forceinline__ float dpp_row_ror(float x) {
    return __uint_as_float(__builtin_amdgcn_mov_dpp(__float_as_uint(x), 0x120 + kRot, 0xF, 0xF, false));
}
// maximum / sum over the 16 lanes of a row, left in every lane: rotations by 8, 4, 2, 1 each double the covered set
__device__ __forceinline__ float row16_max(float x) {
    x = fmaxf(x, dpp_row_ror<8>(x));
    x = fmaxf(x, dpp_row_ror<4>(x));
    x = fmaxf(x, dpp_row_ror<2>(x));
    return fmaxf(x, dpp_row_ror<1>(x));
}
__device__ __forceinline__ float row16_sum(float x) {
    x += dpp_row_ror<8>(x);
    x += dpp_row_ror<4>(x);
    x += dpp_row_ror<2>(x);
    return x + dpp_row_ror<1>(x);
}
__device__ __forceinline__ float dpp_quad_xor1(float x) {
    return __uint_as_float(__builtin_amdgcn_mov_dpp(__float_as_uint(x), 0xB1, 0xF, 0xF, false));    // quad_perm:[1,0,3,2]
}
__device__ __forceinline__ float dpp_quad_xor2(float x) {
    return __uint_as_float(__builtin_amdgcn_mov_dpp(__float_as_uint(x), 0x4E, 0xF, 0xF, false));    // quad_perm:[2,3,0,1]
}

// kPool: instead of the score rows, write their 1-D max-pooling onto 64-token key blocks (window of 5 compressed
// keys, stride 4, padding 1, forced blocks +inf, empty windows -inf: the rule of csrc/max_pooling_1d.cuh:12-160
// applied to the scores this kernel would have written, which never reach memory).
template <bool kCausal, bool kPool>
__global__ __launch_bounds__(64 * kWavesS1) __attribute__((amdgpu_waves_per_eu(kWavesPerSimdS1, kWavesPerSimdS1)))
void stage1_kernel(const Stage1Params p) {
    __shared__ uint4 tile[2][1024];                            // two 16 KiB operand-ordered key tiles
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);     // wavefront-uniform: what depends on it alone stays in scalar registers
    const int n = lane & 15, g = lane >> 4;
    const int b = blockIdx.y, h = blockIdx.z;
    const int q0 = p.cu_seqlens_q[b];
    const int Sq = p.cu_seqlens_q[b + 1] - q0;
    // late tokens see the most keys: they go first, so the long workgroups do not form the tail of the launch
    const int tok_block0 = (static_cast<int>(gridDim.x) - 1 - static_cast<int>(blockIdx.x)) * kTokPerBlock;
    if (tok_block0 >= Sq) return;                              // uniform per workgroup
    const int k0 = p.cu_seqlens_k[b], Lk = p.cu_seqlens_k[b + 1] - k0;
    const int c0 = p.cu_seqlens_c[b], Lc = p.cu_seqlens_c[b + 1] - c0;
    const int s1 = (Lk == Lc) ? 16 : 64;                       // flash_fwd_kernel.h:1236-1240

    const int tok0 = tok_block0 + wave * kTokPerWave;          // first token of this wavefront
    int vis_f[kTokPerWave], vis_c[kTokPerWave];
    bool live[kTokPerWave];
    int min_vis_c = 0x7fffffff;
#pragma unroll
    for (int t = 0; t < kTokPerWave; ++t) {
        const int i = tok0 + t;
        live[t] = i < Sq;
        vis_f[t] = live[t] ? stage1_visible(i, 16, Lk, Sq, kCausal) : 0;
        vis_c[t] = live[t] ? stage1_visible(i, s1, Lc, Sq, kCausal) : 0;
        if (vis_c[t] == 0) vis_f[t] = 0;                       // early exit of flash_fwd_kernel.h:1271-1276
        if (kPool && vis_f[t] > p.score_cols) vis_f[t] = p.score_cols;               // the score row the pooling would have read ends there
        min_vis_c = vis_c[t] < min_vis_c ? vis_c[t] : min_vis_c;
    }
    // tile counts are taken over the whole workgroup (its last live token sees the most keys)
    const int i_last = (tok_block0 + kTokPerBlock - 1 < Sq ? tok_block0 + kTokPerBlock - 1 : Sq - 1);
    const int wg_vis_c = stage1_visible(i_last, s1, Lc, Sq, kCausal);
    const int wg_vis_f = wg_vis_c == 0 ? 0 : stage1_visible(i_last, 16, Lk, Sq, kCausal);
    const int tiles_c = (wg_vis_c + 63) >> 6;
    const int tiles_f = (wg_vis_f + 63) >> 6;

    // Q as the A operand: r = lane % 16 is the head, g the k-group
    elem8 qf[kTokPerWave][4];
#pragma unroll
    for (int t = 0; t < kTokPerWave; ++t) {
        const int i = live[t] ? tok0 + t : Sq - 1;
        const elem_bits* qp = p.q + (static_cast<int64_t>(q0) + i) * p.q_tok_stride + h * p.q_kvh_stride + (n < p.group ? n : p.group - 1) * p.q_grp_stride + 8 * g;
#pragma unroll
        for (int c = 0; c < 4; ++c) qf[t][c] = *reinterpret_cast<const elem8*>(qp + 32 * c);
    }

    // ---------------- pass 1: per-head log-sum-exp over the coarse keys ----------------
    float m[kTokPerWave][4], l[kTokPerWave][4];                // lane-local over keys == n (mod 16); head 4g+e
#pragma unroll
    for (int t = 0; t < kTokPerWave; ++t)
#pragma unroll
        for (int e = 0; e < 4; ++e) { m[t][e] = -INFINITY; l[t][e] = 0.f; }

    const elem_bits* cbase = p.c + static_cast<int64_t>(c0) * p.c_row_stride + h * p.c_head_stride;
    const elem_bits* kbase = p.k + static_cast<int64_t>(k0) * p.k_row_stride + h * p.k_head_stride;
    const uint32_t lds_tiles = __builtin_amdgcn_readfirstlane(s1_lds_addr(tile));
    const int wave_u = wave;
    const int c_stride = static_cast<int>(p.c_row_stride), k_stride = static_cast<int>(p.k_row_stride);
    // every ordinary load so far (q) lands before the first LDS-DMA goes out
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#pragma unroll
    for (int t = 0; t < kTokPerWave; ++t)
#pragma unroll
        for (int c = 0; c < 4; ++c) asm volatile("" : "+v"(qf[t][c]));
    if (tiles_c > 0) issue_tile(cbase, c_stride, 0, Lc, lds_tiles, wave_u, n, g);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    for (int ti = 0; ti < tiles_c; ++ti) {
        if (ti + 1 < tiles_c) issue_tile(cbase, c_stride, (ti + 1) * 64, Lc, lds_tiles + ((ti + 1) & 1) * 16384, wave_u, n, g);
        const uint4* cur = tile[ti & 1];
        floatx4 s[kTokPerWave][4];
#pragma unroll
        for (int kt = 0; kt < 4; ++kt) {
#pragma unroll
            for (int t = 0; t < kTokPerWave; ++t) s[t][kt] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                const uint4 raw = cur[(kt * 4 + c) * 64 + lane];
                elem8 kf;
                __builtin_memcpy(&kf, &raw, 16);
#pragma unroll
                for (int t = 0; t < kTokPerWave; ++t)
                    s[t][kt] = IV2_MFMA(qf[t][c], kf, s[t][kt], 0, 0, 0);
            }
        }
        // only the tile that holds a token's last visible key needs the per-key test
        const bool cut = (ti + 1) * 64 > min_vis_c;            // uniform per wavefront
        if (!cut) {
            // every key of the tile is visible to both tokens: the maximum is finite, no key test, and the scale
            // rides in the multiply-add that feeds exp2
#pragma unroll
            for (int t = 0; t < kTokPerWave; ++t) {
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const float mx = fmaxf(fmaxf(s[t][0][e], s[t][1][e]), fmaxf(s[t][2][e], s[t][3][e]));
                    const float m_new = fmaxf(m[t][e], mx * p.scale_log2);
                    float acc = l[t][e] * __builtin_amdgcn_exp2f(m[t][e] - m_new);
#pragma unroll
                    for (int kt = 0; kt < 4; ++kt) acc += __builtin_amdgcn_exp2f(s[t][kt][e] * p.scale_log2 - m_new);
                    l[t][e] = acc;
                    m[t][e] = m_new;
                }
            }
        } else {
#pragma unroll
            for (int t = 0; t < kTokPerWave; ++t) {
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    float v[4];
#pragma unroll
                    for (int kt = 0; kt < 4; ++kt)
                        v[kt] = (ti * 64 + kt * 16 + n < vis_c[t]) ? s[t][kt][e] * p.scale_log2 : -INFINITY;
                    const float mx = fmaxf(fmaxf(v[0], v[1]), fmaxf(v[2], v[3]));
                    const float m_new = fmaxf(m[t][e], mx);
                    const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
                    float acc = l[t][e] * __builtin_amdgcn_exp2f(m[t][e] - m_use);
#pragma unroll
                    for (int kt = 0; kt < 4; ++kt) acc += __builtin_amdgcn_exp2f(v[kt] - m_use);
                    l[t][e] = acc;
                    m[t][e] = m_new;
                }
            }
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");         // this wavefront's share of the next tile has landed
        __syncthreads();
    }
    // merge the 16 key-column lanes of each head: lse2 = m + log2(l) in log2 units
    float lse2[kTokPerWave][4];
#pragma unroll
    for (int t = 0; t < kTokPerWave; ++t)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            // the row's maximum first, then every lane's sum rescaled to it once, then the sum of those
            const float mm = row16_max(m[t][e]);
            const float mu = (mm == -INFINITY) ? 0.f : mm;
            const float ll = row16_sum(l[t][e] * __builtin_amdgcn_exp2f(m[t][e] - mu));
            lse2[t][e] = mm + __builtin_amdgcn_logf(ll);        // v_log_f32 is log2
            if (4 * g + e >= p.group) lse2[t][e] = INFINITY;    // a row that only fills the tile: exp2(x - inf) = 0 in the head sum
        }

    // ---------------- pass 2: scores over the fine keys ----------------
    if (tiles_f > 0) issue_tile(kbase, k_stride, 0, Lk, lds_tiles, wave_u, n, g);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    elem_bits* out_rows[kTokPerWave];
    int bq[kTokPerWave];                                       // pooled output: the key block the token itself sits in
    float carry[kTokPerWave];                                  // pooled output: score of the last key of the previous tile
    {
        const int cache_len = kPool ? (p.cache_lens ? p.cache_lens[b] : p.cache_len) : 0;
#pragma unroll
        for (int t = 0; t < kTokPerWave; ++t) {
            const int64_t row = static_cast<int64_t>(q0) + tok0 + t;
            out_rows[t] = kPool ? p.score + (static_cast<int64_t>(h) * p.score_head_stride + row * p.pool_len)
                                : p.score + h * p.score_head_stride + row * p.score_row_stride;
            bq[t] = (tok0 + t + cache_len) / kBlockN;
            carry[t] = 0.f;
        }
    }
    // value of a pooled entry that no visible key reaches
    auto pool_rest = [&](int kb, int bq_t, float reached) -> elem_bits {
        const bool forced = (kb < p.init_blocks) || (bq_t >= kb && bq_t <= kb + p.local_blocks);
        const int first = kb * kKeysPerBlock - 1;              // first key of the window (before clipping at 0)
        const bool empty = (first < 0 ? 0 : first) >= (Lk < p.score_cols ? Lk : p.score_cols);
        return forced ? kElemPosInf : (empty ? kElemNegInf : f32_to_elem_hw(reached));
    };

    for (int ti = 0; ti < tiles_f; ++ti) {
        if (ti + 1 < tiles_f) issue_tile(kbase, k_stride, (ti + 1) * 64, Lk, lds_tiles + ((ti + 1) & 1) * 16384, wave_u, n, g);
        const uint4* cur = tile[ti & 1];
        float part[kTokPerWave][4];                            // [t][kt]: this lane's four heads summed, key 16 kt + n
#pragma unroll
        for (int kt = 0; kt < 4; ++kt) {
            floatx4 s[kTokPerWave];
#pragma unroll
            for (int t = 0; t < kTokPerWave; ++t) s[t] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                const uint4 raw = cur[(kt * 4 + c) * 64 + lane];
                elem8 kf;
                __builtin_memcpy(&kf, &raw, 16);
#pragma unroll
                for (int t = 0; t < kTokPerWave; ++t)
                    s[t] = IV2_MFMA(qf[t][c], kf, s[t], 0, 0, 0);
            }
#pragma unroll
            for (int t = 0; t < kTokPerWave; ++t) {
                float sum = 0.f;
#pragma unroll
                for (int e = 0; e < 4; ++e) sum += __builtin_amdgcn_exp2f(s[t][e] * p.scale_log2 - lse2[t][e]);
                part[t][kt] = sum;
            }
        }
        const int col = ti * 64 + lane;                        // lane = 16*g + n  <->  key 16*g + n of this tile
#pragma unroll
        for (int t = 0; t < kTokPerWave; ++t) {
            // sum over the four 16-lane rows (the head groups) and hand row kt the total of key tile kt, in three
            // exchanges: (row0 + row1 | row2 + row3) of tiles 0/1 and of tiles 2/3, then the two halves
            float mine = fold_rows32(fold_rows16(part[t][0], part[t][1]), fold_rows16(part[t][2], part[t][3]));
            if ((ti + 1) * 64 > vis_f[t]) mine = (col < vis_f[t]) ? mine : 0.f;   // keys the token may not see score 0 (last tiles only)
            if (!kPool) {
                if (live[t] && col < p.score_cols) out_rows[t][col] = f32_to_elem_hw(mine);
            } else {
                // block kb = col / 4 pools keys 4 kb - 1 .. 4 kb + 3: its quad and the last key of the quad before
                // the score of the key before: the lane below (one DPP shift over the whole wavefront; lane 0 takes the
                // last key of the tile before), no trip through the LDS crossbar
                float left = __uint_as_float(__builtin_amdgcn_update_dpp(__float_as_uint(carry[t]), __float_as_uint(mine),
                                                                         0x138 /* wave_shr:1 */, 0xF, 0xF, false));
                carry[t] = __uint_as_float(__builtin_amdgcn_readlane(__float_as_uint(mine), 63));
                float best = fmaxf(mine, dpp_quad_xor1(mine));
                best = fmaxf(best, dpp_quad_xor2(best));
                best = fmaxf(best, left);
                const int kb = col >> 2;
                // most tiles lie wholly before the token's local window and after the initial blocks, inside the visible
                // keys and the pooled row: no block of theirs is forced or empty (wavefront-uniform test)
                const int kb0 = ti * 16;
                const bool plain = live[t] && (ti + 1) * 64 <= vis_f[t] && kb0 >= p.init_blocks && kb0 + 15 < bq[t] - p.local_blocks &&
                                   kb0 + 15 < p.pool_len;
                if (plain) {
                    if ((lane & 3) == 0) out_rows[t][kb] = f32_to_elem_hw(best);
                } else if (live[t] && (lane & 3) == 0 && kb < p.pool_len) {
                    out_rows[t][kb] = pool_rest(kb, bq[t], best);
                }
            }
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
    }
    // columns no tile covered
#pragma unroll
    for (int t = 0; t < kTokPerWave; ++t) {
        if (!live[t]) continue;
        if (!kPool) {
            for (int col = tiles_f * 64 + lane; col < p.score_cols; col += 64) out_rows[t][col] = 0;
        } else {
            // the first of them still sees the last key of the last tile
            for (int kb = tiles_f * 16 + lane; kb < p.pool_len; kb += 64)
                out_rows[t][kb] = pool_rest(kb, bq[t], kb == tiles_f * 16 ? carry[t] : 0.f);
        }
    }
}

}  // namespace IV2_NS

using namespace IV2_NS;

namespace {

struct Stage1Pool {                  // pooled-output mode of the launch below
    const int32_t* cache_lens;
    int cache_len, pool_len, local_blocks, init_blocks;
};

int launch_stage1(const char* who, void* stream, const void* q, const void* k, const void* v, void* out,
                  const int32_t* cu_seqlens_q, const int32_t* cu_seqlens_k, const int32_t* cu_seqlens_v, int batch,
                  int64_t total_q, int num_heads, int num_heads_k, int head_dim, int max_seqlen_q, int max_seqlen_k,
                  const int64_t* q_strides, const int64_t* k_strides, const int64_t* v_strides,
                  int64_t out_head_stride, int64_t out_row_stride, float softmax_scale, int is_causal,
                  const Stage1Pool* pool) {
    IV2_CHECK(head_dim == kHeadDim, "%s: this build only supports head_dim 128 (got %d)", who, head_dim);
    IV2_CHECK(valid_group(num_heads, num_heads_k),
              "%s: requires num_heads == g * num_heads_k with g in {1, 2, 4, 8, 16} (got %d and %d)", who, num_heads, num_heads_k);
    IV2_CHECK(batch > 0 && total_q >= 0 && max_seqlen_q >= 0 && max_seqlen_k >= 0, "%s: bad sizes", who);
    IV2_CHECK(q && k && v && out && cu_seqlens_q && cu_seqlens_k && cu_seqlens_v, "%s: null pointer", who);
    IV2_CHECK(num_heads_k <= 65535 && batch <= 65535, "%s: batch and num_heads_k must not exceed 65535", who);
    IV2_CHECK(reinterpret_cast<uintptr_t>(q) % 16 == 0 && reinterpret_cast<uintptr_t>(k) % 16 == 0 &&
              reinterpret_cast<uintptr_t>(v) % 16 == 0, "%s: q, k, v must be 16-byte aligned", who);
    for (int s = 0; s < 3; ++s) IV2_CHECK(q_strides[s] % 8 == 0, "%s: q strides must be multiples of 8 elements", who);
    IV2_CHECK(k_strides[0] % 8 == 0 && k_strides[1] % 8 == 0 && v_strides[0] % 8 == 0 && v_strides[1] % 8 == 0,
              "%s: k/v strides must be multiples of 8 elements", who);
    // a lane's byte offset from its sequence's first compressed key is a 32-bit LDS-DMA operand
    IV2_CHECK(k_strides[0] > 0 && v_strides[0] > 0 &&
              (static_cast<int64_t>(max_seqlen_k) + 64) * k_strides[0] < (1ll << 30) &&
              (static_cast<int64_t>(max_seqlen_k) + 64) * v_strides[0] < (1ll << 30),
              "%s: compressed-key rows too far apart (row stride x max_seqlen_k must stay below 2^30 elements)", who);
    if (total_q == 0 || max_seqlen_q == 0) return 0;
    Stage1Params p{};
    p.q = static_cast<const elem_bits*>(q);
    p.k = static_cast<const elem_bits*>(k);
    p.c = static_cast<const elem_bits*>(v);
    p.score = static_cast<elem_bits*>(out);
    p.cu_seqlens_q = cu_seqlens_q; p.cu_seqlens_k = cu_seqlens_k; p.cu_seqlens_c = cu_seqlens_v;
    p.q_tok_stride = q_strides[0]; p.q_grp_stride = q_strides[1]; p.q_kvh_stride = q_strides[2];
    p.k_row_stride = k_strides[0]; p.k_head_stride = k_strides[1];
    p.c_row_stride = v_strides[0]; p.c_head_stride = v_strides[1];
    p.score_head_stride = out_head_stride; p.score_row_stride = out_row_stride;
    p.score_cols = max_seqlen_k;
    p.group = num_heads / num_heads_k;
    p.scale_log2 = softmax_scale * 1.44269504088896340736f;
    p.causal = is_causal;
    if (pool) {
        p.cache_lens = pool->cache_lens; p.cache_len = pool->cache_len; p.pool_len = pool->pool_len;
        p.local_blocks = pool->local_blocks; p.init_blocks = pool->init_blocks;
    }
    const dim3 grid((max_seqlen_q + kTokPerBlock - 1) / kTokPerBlock, batch, num_heads_k);
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (pool) {
        if (is_causal) hipLaunchKernelGGL((stage1_kernel<true, true>), grid, dim3(64 * kWavesS1), 0, st, p);
        else hipLaunchKernelGGL((stage1_kernel<false, true>), grid, dim3(64 * kWavesS1), 0, st, p);
    } else {
        if (is_causal) hipLaunchKernelGGL((stage1_kernel<true, false>), grid, dim3(64 * kWavesS1), 0, st, p);
        else hipLaunchKernelGGL((stage1_kernel<false, false>), grid, dim3(64 * kWavesS1), 0, st, p);
    }
    IV2_LAUNCH_CHECK();
    return 0;
}

}  // namespace

extern "C" int IV2_ENTRY(infllmv2_varlen_fwd_stage1)(void* stream, const void* q, const void* k, const void* v, void* score,
                                          const int32_t* cu_seqlens_q, const int32_t* cu_seqlens_k,
                                          const int32_t* cu_seqlens_v, int batch, int64_t total_q, int num_heads,
                                          int num_heads_k, int head_dim, int max_seqlen_q, int max_seqlen_k,
                                          const int64_t* q_strides, const int64_t* k_strides,
                                          const int64_t* v_strides, int64_t score_head_stride,
                                          int64_t score_row_stride, float softmax_scale, int is_causal) {
    IV2_CHECK(score_row_stride >= max_seqlen_k, "varlen_fwd_stage1: score row stride shorter than max_seqlen_k");
    return launch_stage1("varlen_fwd_stage1", stream, q, k, v, score, cu_seqlens_q, cu_seqlens_k, cu_seqlens_v, batch,
                         total_q, num_heads, num_heads_k, head_dim, max_seqlen_q, max_seqlen_k, q_strides, k_strides,
                         v_strides, score_head_stride, score_row_stride, softmax_scale, is_causal, nullptr);
}

extern "C" int IV2_ENTRY(infllmv2_varlen_fwd_stage1_pooled)(void* stream, const void* q, const void* k, const void* v,
                                                 void* pooled, const int32_t* cu_seqlens_q,
                                                 const int32_t* cu_seqlens_k, const int32_t* cu_seqlens_v,
                                                 const int32_t* cache_lens, int cache_len, int batch,
                                                 int64_t total_q, int num_heads, int num_heads_k, int head_dim,
                                                 int max_seqlen_q, int max_seqlen_k, const int64_t* q_strides,
                                                 const int64_t* k_strides, const int64_t* v_strides, int out_len,
                                                 float softmax_scale, int is_causal, int kernel_size, int stride,
                                                 int padding, int block_size, int local_blocks, int init_blocks) {
    IV2_CHECK(kernel_size == 5 && stride == 4 && padding == 1 && block_size == kBlockN,
              "varlen_fwd_stage1_pooled: only the 5/4/1 window on 64-token blocks is fused (got %d/%d/%d on %d); "
              "use varlen_fwd_stage1 and max_pooling_1d", kernel_size, stride, padding, block_size);
    IV2_CHECK(out_len >= 0 && cache_len >= 0, "varlen_fwd_stage1_pooled: negative out_len or cache_len");
    if (out_len == 0) return 0;
    const Stage1Pool pool{cache_lens, cache_len, out_len, local_blocks, init_blocks};
    return launch_stage1("varlen_fwd_stage1_pooled", stream, q, k, v, pooled, cu_seqlens_q, cu_seqlens_k, cu_seqlens_v,
                         batch, total_q, num_heads, num_heads_k, head_dim, max_seqlen_q, max_seqlen_k, q_strides,
                         k_strides, v_strides, total_q * static_cast<int64_t>(out_len), out_len, softmax_scale,
                         is_causal, &pool);
}
