// Stage-1 scoring for decode on gfx950: ONE query token per sequence, a batch of sequences, each scored against
// its own compressed keys.
//
// Same arithmetic and rules as stage1.hip (compute_attn_1rowblock_splitkv_stage1,
// csrc/flash_attn/src/flash_fwd_kernel.h:1203-1744; Mask::apply_mask_stage1, mask.h:225-319; hdim16_reduce,
// flash_fwd_kernel.h:53-112) for a sequence with q_len == 1:
//   vis_s = L for a non-causal launch, clamp(L - 1, 0, L) for a causal one (mask.h:273-281 with i = 0, q_len = 1)
//   lse_g = log sum_{c < vis_c} exp(scale * q_g . kc_c)
//   score[h, b, j] = bf16( sum_g exp(scale * q_g . kf_j - lse_g) )  for j < vis_f, else 0; all 0 when vis_c == 0
// and, with pooling, the max-pooling rule of csrc/max_pooling_1d.cuh:12-160 applied to that row.
//
// Shape of the work: per sequence and KV head the whole compressed-key set is read once (256 bytes per key) for 16
// query rows, so the launch is bound by memory bandwidth and the stage1.hip kernel (one workgroup per 16 tokens,
// keys staged for reuse by 16 tokens) is the wrong shape: it would stream every sequence through one workgroup.
// Here the keys of one (sequence, KV head) are cut into runs of 64-key tiles, the same run length (two tiles unless
// the longest sequence would then need more than 64 runs) for every sequence of the batch, and every run goes to a
// single-wavefront workgroup that loads its tiles straight into MFMA operand registers: long sequences get many
// workgroups, short ones few, and every workgroup carries the same load.
// The log-sum-exp needs all coarse keys before any score can be normalised, so there are two launches:
//   1. stage1_decode_lse_kernel: per run of coarse tiles the running (max, sum) of the 16 heads -> workspace;
//   2. stage1_decode_score_kernel: merges the partials of its (sequence, head) (16 lanes in parallel), then scores its run of
//      fine tiles and writes either the score row or its pooling onto key blocks.  A pooled block needs the last
//      key of the tile before the run: that one 16-key group is scored again by the run that needs it (same MFMA,
//      same operands, same bits).
// Keys can be packed (cu_seqlens) or lie in per-sequence caches (batch stride + lengths).
#include "common.h"
#include "infllmv2_hip.h"
#include <math.h>

namespace IV2_NS {

struct S1DecodeParams {
    const elem_bits* q;
    const elem_bits* k;              // fine compressed keys
    const elem_bits* c;              // coarse compressed keys (the key set of the log-sum-exp)
    elem_bits* out;
    float* partial;                  // (batch, Hk, splits_c, 32): log2-domain max of the 16 heads, then their sums
    const int* cu_seqlens_q;         // null: sequence b's query is row b
    const int* cu_seqlens_k;         // packed keys: rows [cu[b], cu[b+1]); null: cache layout, k_lens[b] rows at b * k_batch
    const int* k_lens;
    const int* cu_seqlens_c;
    const int* c_lens;
    int64_t q_tok_stride, q_grp_stride, q_kvh_stride;
    int64_t k_batch_stride, k_row_stride, k_head_stride;
    int64_t c_batch_stride, c_row_stride, c_head_stride;
    int64_t out_head_stride, out_row_stride;
    int cols;                        // score columns to define per row (max_seqlen_k)
    float scale_log2;
    int causal;
    int group;                       // query heads per KV head, 1..16: MFMA rows >= group repeat head group - 1 and add nothing
    int splits_c, splits_f;          // runs the longest sequence is cut into (grid size; record slots per pair)
    int run_c, run_f;                // tiles per run
    // pooled output
    const int* cache_lens;           // per sequence, or null: cache_len for all
    int cache_len;
    int pool_len, local_blocks, init_blocks;
};

__device__ __forceinline__ int s1d_visible(int s, int L, bool causal) {
    if (!causal) return L;
    // mask.h:273-281 for token 0 of a 1-token query: (0+1)/s - 1 + L - (1 - s + 1)/s, C++ truncating divisions
    int v = 1 / s - 1 + L - (2 - s) / s;
    v = v < 0 ? 0 : v;
    return v < L ? v : L;
}

struct S1DecodeSeq {
    int q_row, Sq, Lk, Lc;
    const elem_bits* kbase;
    const elem_bits* cbase;
};

__device__ __forceinline__ S1DecodeSeq s1d_sequence(const S1DecodeParams& p, int b, int h) {
    S1DecodeSeq s;
    if (p.cu_seqlens_q) { s.q_row = p.cu_seqlens_q[b]; s.Sq = p.cu_seqlens_q[b + 1] - s.q_row; }
    else { s.q_row = b; s.Sq = 1; }
    int64_t koff, coff;
    if (p.cu_seqlens_k) { const int k0 = p.cu_seqlens_k[b]; s.Lk = p.cu_seqlens_k[b + 1] - k0; koff = k0 * p.k_row_stride; }
    else { s.Lk = p.k_lens[b]; koff = b * p.k_batch_stride; }
    if (p.cu_seqlens_c) { const int c0 = p.cu_seqlens_c[b]; s.Lc = p.cu_seqlens_c[b + 1] - c0; coff = c0 * p.c_row_stride; }
    else { s.Lc = p.c_lens[b]; coff = b * p.c_batch_stride; }
    s.kbase = p.k + koff + h * p.k_head_stride;
    s.cbase = p.c + coff + h * p.c_head_stride;
    return s;
}

// 64 keys x 128 d as MFMA B operands: register kt*4 + c of lane (n, g) = K[key0 + 16 kt + n][32 c + 8 g ..].
// Rows past the last key read the last key (finite values that every consumer masks).
__device__ __forceinline__ void s1d_load_tile(elem8 (&t)[16], const elem_bits* base, int64_t row_stride, int key0,
                                              int L, int n, int g) {
#pragma unroll
    for (int kt = 0; kt < 4; ++kt) {
        int row = key0 + 16 * kt + n;
        row = row < L ? row : L - 1;
        const elem_bits* src = base + row * row_stride + 8 * g;
#pragma unroll
        for (int c = 0; c < 4; ++c) t[kt * 4 + c] = *reinterpret_cast<const elem8*>(src + 32 * c);
    }
}

__device__ __forceinline__ void s1d_load_q(elem8 (&qf)[4], const S1DecodeParams& p, const S1DecodeSeq& s, int h, int n, int g) {
    const elem_bits* qp = p.q + static_cast<int64_t>(s.q_row) * p.q_tok_stride + h * p.q_kvh_stride + (n < p.group ? n : p.group - 1) * p.q_grp_stride + 8 * g;
#pragma unroll
    for (int c = 0; c < 4; ++c) qf[c] = *reinterpret_cast<const elem8*>(qp + 32 * c);
}

// run [t0, t1) of `tiles` tiles that split `split` works on: runs of `per` tiles, the same length for every sequence
// of the batch (a long sequence has many runs, a short one few: every wavefront gets the same amount of work)
__device__ __forceinline__ void s1d_run_fixed(int tiles, int per, int split, int& t0, int& t1) {
    t0 = split * per;
    t0 = t0 < tiles ? t0 : tiles;
    t1 = t0 + per;
    t1 = t1 < tiles ? t1 : tiles;
}
// (max, sum) in log2 units of head 4g + e over the coarse tiles [t0, t1) of one sequence and KV head, merged over the
// 16 key-column lanes: every lane of row g returns the values of its four heads.
__device__ __forceinline__ void s1d_lse_run(const S1DecodeParams& p, const S1DecodeSeq& sq, const elem8 (&qf)[4], int vis_c,
                                            int t0, int t1, int n, int g, float (&m_out)[4], float (&l_out)[4]) {
    float m[4], l[4];                                          // head 4g + e over the keys == n (mod 16) of the run
#pragma unroll
    for (int e = 0; e < 4; ++e) { m[e] = -INFINITY; l[e] = 0.f; }

    auto consume = [&](const elem8 (&t)[16], int ti) {
        floatx4 s[4];
#pragma unroll
        for (int kt = 0; kt < 4; ++kt) {
            s[kt] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int c = 0; c < 4; ++c) s[kt] = IV2_MFMA(qf[c], t[kt * 4 + c], s[kt], 0, 0, 0);
        }
        const bool cut = (ti + 1) * 64 > vis_c;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            float v[4];
#pragma unroll
            for (int kt = 0; kt < 4; ++kt) v[kt] = s[kt][e] * p.scale_log2;
            if (cut) {
#pragma unroll
                for (int kt = 0; kt < 4; ++kt) v[kt] = (ti * 64 + kt * 16 + n < vis_c) ? v[kt] : -INFINITY;
            }
            const float mx = fmaxf(fmaxf(v[0], v[1]), fmaxf(v[2], v[3]));
            const float m_new = fmaxf(m[e], mx);
            const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
            float acc = l[e] * __builtin_amdgcn_exp2f(m[e] - m_use);
#pragma unroll
            for (int kt = 0; kt < 4; ++kt) acc += __builtin_amdgcn_exp2f(v[kt] - m_use);
            l[e] = acc;
            m[e] = m_new;
        }
    };

    elem8 ta[16], tb[16];
    if (t0 < t1) s1d_load_tile(ta, sq.cbase, p.c_row_stride, t0 * 64, sq.Lc, n, g);
    if (t0 + 1 < t1) s1d_load_tile(tb, sq.cbase, p.c_row_stride, (t0 + 1) * 64, sq.Lc, n, g);
    for (int ti = t0; ti < t1; ti += 2) {
        consume(ta, ti);
        if (ti + 2 < t1) s1d_load_tile(ta, sq.cbase, p.c_row_stride, (ti + 2) * 64, sq.Lc, n, g);
        if (ti + 1 < t1) {
            consume(tb, ti + 1);
            if (ti + 3 < t1) s1d_load_tile(tb, sq.cbase, p.c_row_stride, (ti + 3) * 64, sq.Lc, n, g);
        }
    }
    // merge the 16 key-column lanes of each head
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        float mm = m[e], ll = l[e];
#pragma unroll
        for (int off = 1; off < 16; off <<= 1) {
            const float mo = __shfl_xor(mm, off);
            const float lo = __shfl_xor(ll, off);
            const float mn = fmaxf(mm, mo);
            const float mu = (mn == -INFINITY) ? 0.f : mn;
            ll = ll * __builtin_amdgcn_exp2f(mm - mu) + lo * __builtin_amdgcn_exp2f(mo - mu);
            mm = mn;
        }
        m_out[e] = mm;
        l_out[e] = ll;
    }
}

// The partial records {max x 16, sum x 16} of one (sequence, head) as a lane needs them: lane (n, g) takes the records
// n, n + 16, n + 32, n + 48 (at most 64 runs) for its four heads, two 16-byte loads per record.  The number of loads
// does not depend on the data (an index beyond the last record reads the last one again and is ignored later), so that
// the loads requested after these can stay in flight while these are waited for.
struct S1DRecords {
    floatx4 m[4], l[4];
};
__device__ __forceinline__ void s1d_load_records(S1DRecords& r, const float* part, int count, int n, int g) {
    auto fetch = [&](int k) {
        int s = n + 16 * k;
        s = s < count ? s : count - 1;
        r.m[k] = *reinterpret_cast<const floatx4*>(part + s * 32 + 4 * g);
        r.l[k] = *reinterpret_cast<const floatx4*>(part + s * 32 + 16 + 4 * g);
    };
    fetch(0);
    if (count > 16) {                                          // uniform
#pragma unroll
        for (int k = 1; k < 4; ++k) fetch(k);
    }
}
// log-sum-exp (log2 units) of head 4g + e from those records: each lane folds its own in run order, then the 16 lanes
// of a row merge among themselves (the merge of (max, sum) pairs is associative and commutative up to rounding, and
// every lane of a row ends with the same bits because the butterfly combines the same pairs in the same order on both
// sides).
__device__ __forceinline__ void s1d_merge_records(const S1DRecords& r, int count, int n, int g, int group, float (&lse2)[4]) {
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        float mm = -INFINITY, ll = 0.f;
        auto fold = [&](int k) {
            const bool have = n + 16 * k < count;              // a record that is not there is the neutral element
            const float mo = have ? r.m[k][e] : -INFINITY, lo = have ? r.l[k][e] : 0.f;
            const float mn = fmaxf(mm, mo);
            const float mu = (mn == -INFINITY) ? 0.f : mn;
            ll = ll * __builtin_amdgcn_exp2f(mm - mu) + lo * __builtin_amdgcn_exp2f(mo - mu);
            mm = mn;
        };
        fold(0);
        if (count > 16) {                                      // uniform
#pragma unroll
            for (int k = 1; k < 4; ++k) fold(k);
        }
#pragma unroll
        for (int off = 1; off < 16; off <<= 1) {
            const float mo = __shfl_xor(mm, off);
            const float lo = __shfl_xor(ll, off);
            const float mn = fmaxf(mm, mo);
            const float mu = (mn == -INFINITY) ? 0.f : mn;
            // the same sum on both partners: add the term of the lane with the lower number first
            const float mine = ll * __builtin_amdgcn_exp2f(mm - mu), theirs = lo * __builtin_amdgcn_exp2f(mo - mu);
            ll = (n & off) ? theirs + mine : mine + theirs;
            mm = mn;
        }
        lse2[e] = mm + __builtin_amdgcn_logf(ll);                // v_log_f32 is log2
        if (4 * g + e >= group) lse2[e] = INFINITY;              // a row that only fills the tile adds exp2(x - inf) = 0
    }
}

__global__ __launch_bounds__(64)
void stage1_decode_lse_kernel(const S1DecodeParams p) {
    const int lane = threadIdx.x, n = lane & 15, g = lane >> 4;
    const int split = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
    const S1DecodeSeq sq = s1d_sequence(p, b, h);
    if (sq.Sq <= 0) return;
    const int s1 = (sq.Lk == sq.Lc) ? 16 : 64;                 // flash_fwd_kernel.h:1236-1240
    const int vis_c = s1d_visible(s1, sq.Lc, p.causal != 0);
    int t0, t1;
    s1d_run_fixed((vis_c + 63) >> 6, p.run_c, split, t0, t1);
    if (t0 >= t1 && split > 0) return;                         // beyond this sequence's runs; run 0 always leaves a record
    elem8 qf[4];
    s1d_load_q(qf, p, sq, h, n, g);
    float mm[4], ll[4];
    s1d_lse_run(p, sq, qf, vis_c, t0, t1, n, g, mm, ll);
    float* slot = p.partial + ((static_cast<int64_t>(b) * gridDim.y + h) * p.splits_c + split) * 32;
    if (n == 0) {
#pragma unroll
        for (int e = 0; e < 4; ++e) { slot[4 * g + e] = mm[e]; slot[16 + 4 * g + e] = ll[e]; }
    }
}

__device__ __forceinline__ float s1d_fold_rows16(float x, float y) {
    typedef unsigned u2 __attribute__((ext_vector_type(2)));
    const u2 r = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(y), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}
__device__ __forceinline__ float s1d_fold_rows32(float x, float y) {
    typedef unsigned u2 __attribute__((ext_vector_type(2)));
    const u2 r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(y), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}
__device__ __forceinline__ float s1d_quad_xor1(float x) {
    return __uint_as_float(__builtin_amdgcn_mov_dpp(__float_as_uint(x), 0xB1, 0xF, 0xF, false));
}
__device__ __forceinline__ float s1d_quad_xor2(float x) {
    return __uint_as_float(__builtin_amdgcn_mov_dpp(__float_as_uint(x), 0x4E, 0xF, 0xF, false));
}

// The 16 keys before tile t0 (the last group of tile t0 - 1), whose last key opens the first pooling window of a run
// that does not start the row; with t0 == 0 the request goes to the row's first keys and is ignored.
__device__ __forceinline__ void s1d_load_group_before(elem8 (&t4)[4], const S1DecodeSeq& sq, int64_t row_stride, int t0, int n, int g) {
    int row = (t0 > 0 ? t0 * 64 - 16 : 0) + n;
    row = row < sq.Lk ? row : sq.Lk - 1;
    const elem_bits* src = sq.kbase + row * row_stride + 8 * g;
#pragma unroll
    for (int c = 0; c < 4; ++c) t4[c] = *reinterpret_cast<const elem8*>(src + 32 * c);
}

// Scores (or pooled block scores) of the fine tiles [t0, t1) of one sequence and KV head, by one wavefront; ta / tb
// hold tiles t0 and t0 + 1 already and before4 the 16 keys before tile t0 (all requested by the caller before it
// waited for the log-sum-exp).
template <bool kPool>
__device__ __forceinline__ void s1d_score_run(const S1DecodeParams& p, const S1DecodeSeq& sq, const elem8 (&qf)[4],
                                              const float (&lse2)[4], const elem8 (&before4)[4], elem8 (&ta)[16], elem8 (&tb)[16], int vis_f,
                                              int tiles, int t0, int t1, bool owns_tail, int b, int h, int lane) {
    const int n = lane & 15, g = lane >> 4;
    const int64_t out_row = static_cast<int64_t>(h) * p.out_head_stride + static_cast<int64_t>(sq.q_row) * p.out_row_stride;
    elem_bits* out = p.out + out_row;
    const int bq = kPool ? ((p.cache_lens ? p.cache_lens[b] : p.cache_len) / kBlockN) : 0;   // the query's own key block
    const int Lk_cols = sq.Lk < p.cols ? sq.Lk : p.cols;
    auto pool_rest = [&](int kb, float reached) -> elem_bits {
        const bool forced = (kb < p.init_blocks) || (bq >= kb && bq <= kb + p.local_blocks);
        const int first = kb * 4 - 1;
        const bool empty = (first < 0 ? 0 : first) >= Lk_cols;
        return forced ? kElemPosInf : (empty ? kElemNegInf : f32_to_elem_hw(reached));
    };
    // one 16-key group: this lane's four heads summed for key 16 kt + n of the tile
    auto group_part = [&](const elem8* t4) -> float {
        floatx4 s = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int c = 0; c < 4; ++c) s = IV2_MFMA(qf[c], t4[c], s, 0, 0, 0);
        float sum = 0.f;
#pragma unroll
        for (int e = 0; e < 4; ++e) sum += __builtin_amdgcn_exp2f(s[e] * p.scale_log2 - lse2[e]);
        return sum;
    };

    float carry = 0.f;                                         // score of the last key before the current tile
    if (kPool && t0 > 0 && t0 < t1) {
        const float part3 = group_part(before4);               // keys of the last group of tile t0 - 1: all exist
        float prev = s1d_fold_rows32(s1d_fold_rows16(0.f, 0.f), s1d_fold_rows16(0.f, part3));
        prev = (t0 * 64 - 64 + lane < vis_f) ? prev : 0.f;
        carry = __shfl(prev, 63);
    }

    auto consume = [&](const elem8 (&t)[16], int ti) {
        float part[4];
#pragma unroll
        for (int kt = 0; kt < 4; ++kt) part[kt] = group_part(&t[kt * 4]);
        const int col = ti * 64 + lane;                        // lane 16 g + n <-> key 16 g + n of the tile
        float mine = s1d_fold_rows32(s1d_fold_rows16(part[0], part[1]), s1d_fold_rows16(part[2], part[3]));
        mine = (col < vis_f) ? mine : 0.f;
        if (!kPool) {
            if (col < p.cols) out[col] = f32_to_elem_hw(mine);
        } else {
            float left = __shfl_up(mine, 1);
            if (lane == 0) left = carry;
            carry = __shfl(mine, 63);
            float best = fmaxf(mine, s1d_quad_xor1(mine));
            best = fmaxf(best, s1d_quad_xor2(best));
            best = fmaxf(best, left);
            const int kb = col >> 2;
            if ((lane & 3) == 0 && kb < p.pool_len) out[kb] = pool_rest(kb, best);
        }
    };

    for (int ti = t0; ti < t1; ti += 2) {
        consume(ta, ti);
        if (ti + 2 < t1) s1d_load_tile(ta, sq.kbase, p.k_row_stride, (ti + 2) * 64, sq.Lk, n, g);
        if (ti + 1 < t1) {
            consume(tb, ti + 1);
            if (ti + 3 < t1) s1d_load_tile(tb, sq.kbase, p.k_row_stride, (ti + 3) * 64, sq.Lk, n, g);
        }
    }
    if (owns_tail) {                                           // columns no tile covers
        if (!kPool) {
            for (int col = tiles * 64 + lane; col < p.cols; col += 64) out[col] = 0;
        } else {
            // the first of them still sees the last key of the last tile
            for (int kb = tiles * 16 + lane; kb < p.pool_len; kb += 64) out[kb] = pool_rest(kb, kb == tiles * 16 ? carry : 0.f);
        }
    }
}

// visible fine keys and tiles of a sequence (0 when no coarse key is visible: early exit of flash_fwd_kernel.h:1271-1276)
template <bool kPool>
__device__ __forceinline__ void s1d_fine_extent(const S1DecodeParams& p, const S1DecodeSeq& sq, int& vis_c, int& vis_f, int& tiles) {
    const int s1 = (sq.Lk == sq.Lc) ? 16 : 64;                 // flash_fwd_kernel.h:1236-1240
    vis_c = s1d_visible(s1, sq.Lc, p.causal != 0);
    vis_f = vis_c == 0 ? 0 : s1d_visible(16, sq.Lk, p.causal != 0);
    if (kPool && vis_f > p.cols) vis_f = p.cols;               // the score row the pooling would have read ends there
    tiles = (vis_f + 63) >> 6;
}

template <bool kPool>
__global__ __launch_bounds__(64)
void stage1_decode_score_kernel(const S1DecodeParams p) {
    const int lane = threadIdx.x, n = lane & 15, g = lane >> 4;
    const int split = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
    const S1DecodeSeq sq = s1d_sequence(p, b, h);
    if (sq.Sq <= 0) return;
    int vis_c, vis_f, tiles;
    s1d_fine_extent<kPool>(p, sq, vis_c, vis_f, tiles);
    int t0, t1;
    s1d_run_fixed(tiles, p.run_f, split, t0, t1);
    const bool owns_tail = tiles == 0 ? split == 0 : (t0 < t1 && t1 == tiles);
    if (t0 >= t1 && !owns_tail) return;

    // Everything this run reads is requested before anything waits on memory, in the order in which it is needed:
    // the partial records of the log-sum-exp (merged while the keys are still on their way), the query, two tiles.
    // A run has one or two tiles (more only when a sequence has over 128 of them); with one, the second request
    // repeats the first, so that the number of requests in flight is the same on every path.
    int records = (((vis_c + 63) >> 6) + p.run_c - 1) / p.run_c;                    // the coarse runs of this sequence
    records = records < 1 ? 1 : records;
    S1DRecords rec;
    elem8 qf[4], before4[4], ta[16], tb[16];
    float lse2[4] = {0.f, 0.f, 0.f, 0.f};
    if (t0 < t1) {                                             // uniform; otherwise this run only fills the row's tail
        s1d_load_records(rec, p.partial + (static_cast<int64_t>(b) * gridDim.y + h) * p.splits_c * 32, records, n, g);
        s1d_load_q(qf, p, sq, h, n, g);
        if (kPool) s1d_load_group_before(before4, sq, p.k_row_stride, t0, n, g);
        s1d_load_tile(ta, sq.kbase, p.k_row_stride, t0 * 64, sq.Lk, n, g);
        s1d_load_tile(tb, sq.kbase, p.k_row_stride, (t0 + 1 < t1 ? t0 + 1 : t0) * 64, sq.Lk, n, g);
        s1d_merge_records(rec, records, n, g, p.group, lse2);
    }
    s1d_score_run<kPool>(p, sq, qf, lse2, before4, ta, tb, vis_f, tiles, t0, t1, owns_tail, b, h, lane);
}

}  // namespace IV2_NS

using namespace IV2_NS;

namespace {

// Runs of the two-launch form: every run is `run` tiles long whatever its sequence's length, so the single-wavefront
// workgroups all carry the same load; the longest sequence is cut into at most 64 runs.
void s1d_splits(int batch, int num_heads_k, int max_keys, int max_coarse, int& splits_f, int& splits_c, int& run_f, int& run_c) {
    (void)batch; (void)num_heads_k;
    auto plan = [&](int tiles, int want_run, int& splits, int& run) {
        run = want_run;
        if ((tiles + run - 1) / run > 64) run = (tiles + 63) / 64;
        splits = (tiles + run - 1) / run;
        if (splits < 1) splits = 1;
    };
    plan((max_keys + 63) / 64, 2, splits_f, run_f);
    plan((max_coarse + 63) / 64, 2, splits_c, run_c);
}

}  // namespace

#ifndef IV2_F16        // element-type independent: defined once
extern "C" size_t infllmv2_stage1_decode_workspace_bytes(int batch, int num_heads_k, int max_seqlen_k, int max_seqlen_v) {
    int sf, sc, rf, rc;
    s1d_splits(batch, num_heads_k, max_seqlen_k, max_seqlen_v, sf, sc, rf, rc);
    return static_cast<size_t>(batch > 0 ? batch : 0) * (num_heads_k > 0 ? num_heads_k : 0) * sc * 32 * sizeof(float);
}
#endif

extern "C" int IV2_ENTRY(infllmv2_stage1_decode)(void* stream, const void* q, const void* k, const void* v, void* out,
                                      const int32_t* cu_seqlens_q, const int32_t* cu_seqlens_k, const int32_t* k_lens,
                                      const int32_t* cu_seqlens_v, const int32_t* v_lens, void* workspace,
                                      size_t workspace_bytes, int batch, int num_heads, int num_heads_k, int head_dim,
                                      int max_seqlen_k, int max_seqlen_v, const int64_t* q_strides,
                                      const int64_t* k_strides, const int64_t* v_strides, int64_t out_head_stride,
                                      int64_t out_row_stride, float softmax_scale, int is_causal, int pooled,
                                      const int32_t* cache_lens, int cache_len, int out_len, int kernel_size, int stride,
                                      int padding, int block_size, int local_blocks, int init_blocks) {
    const char* who = "stage1_decode";
    IV2_CHECK(head_dim == kHeadDim, "%s: this build only supports head_dim 128 (got %d)", who, head_dim);
    IV2_CHECK(valid_group(num_heads, num_heads_k),
              "%s: requires num_heads == g * num_heads_k with g in {1, 2, 4, 8, 16} (got %d and %d)", who, num_heads, num_heads_k);
    IV2_CHECK(batch > 0 && max_seqlen_k >= 0 && max_seqlen_v >= 0, "%s: bad sizes", who);
    IV2_CHECK(num_heads_k <= 65535 && batch <= 65535, "%s: batch and num_heads_k must not exceed 65535", who);
    IV2_CHECK(q && k && v && out, "%s: null pointer", who);
    IV2_CHECK((cu_seqlens_k != nullptr) != (k_lens != nullptr) && (cu_seqlens_v != nullptr) != (v_lens != nullptr),
              "%s: give either cumulative lengths (packed keys) or per-sequence lengths (key caches), for k and for v", who);
    IV2_CHECK(reinterpret_cast<uintptr_t>(q) % 16 == 0 && reinterpret_cast<uintptr_t>(k) % 16 == 0 &&
              reinterpret_cast<uintptr_t>(v) % 16 == 0, "%s: q, k, v must be 16-byte aligned", who);
    for (int s = 0; s < 3; ++s)
        IV2_CHECK(q_strides[s] % 8 == 0 && k_strides[s] % 8 == 0 && v_strides[s] % 8 == 0,
                  "%s: strides must be multiples of 8 elements", who);
    if (pooled) {
        IV2_CHECK(kernel_size == 5 && stride == 4 && padding == 1 && block_size == kBlockN,
                  "%s: only the 5/4/1 pooling window on 64-token blocks is fused (got %d/%d/%d on %d)", who, kernel_size,
                  stride, padding, block_size);
        IV2_CHECK(out_len >= 0 && cache_len >= 0 && out_row_stride >= out_len, "%s: bad out_len, cache_len or output row stride", who);
        if (out_len == 0) return 0;
    } else {
        IV2_CHECK(out_row_stride >= max_seqlen_k, "%s: score row stride shorter than max_seqlen_k", who);
    }
    S1DecodeParams p{};
    s1d_splits(batch, num_heads_k, max_seqlen_k, max_seqlen_v, p.splits_f, p.splits_c, p.run_f, p.run_c);
    IV2_CHECK(workspace != nullptr && reinterpret_cast<uintptr_t>(workspace) % 16 == 0 &&
              workspace_bytes >= infllmv2_stage1_decode_workspace_bytes(batch, num_heads_k, max_seqlen_k, max_seqlen_v),
              "%s: workspace missing, misaligned or too small", who);
    p.q = static_cast<const elem_bits*>(q);
    p.k = static_cast<const elem_bits*>(k);
    p.c = static_cast<const elem_bits*>(v);
    p.out = static_cast<elem_bits*>(out);
    p.partial = static_cast<float*>(workspace);
    p.cu_seqlens_q = cu_seqlens_q;
    p.cu_seqlens_k = cu_seqlens_k; p.k_lens = k_lens;
    p.cu_seqlens_c = cu_seqlens_v; p.c_lens = v_lens;
    p.q_tok_stride = q_strides[0]; p.q_grp_stride = q_strides[1]; p.q_kvh_stride = q_strides[2];
    p.k_batch_stride = k_strides[0]; p.k_row_stride = k_strides[1]; p.k_head_stride = k_strides[2];
    p.c_batch_stride = v_strides[0]; p.c_row_stride = v_strides[1]; p.c_head_stride = v_strides[2];
    p.out_head_stride = out_head_stride; p.out_row_stride = out_row_stride;
    p.cols = max_seqlen_k;
    p.group = num_heads / num_heads_k;
    p.scale_log2 = softmax_scale * 1.44269504088896340736f;
    p.causal = is_causal;
    p.cache_lens = cache_lens; p.cache_len = cache_len; p.pool_len = out_len;
    p.local_blocks = local_blocks; p.init_blocks = init_blocks;
    hipStream_t st = static_cast<hipStream_t>(stream);
    hipLaunchKernelGGL(stage1_decode_lse_kernel, dim3(p.splits_c, num_heads_k, batch), dim3(64), 0, st, p);
    IV2_LAUNCH_CHECK();
    const dim3 grid(p.splits_f, num_heads_k, batch);
    if (pooled) hipLaunchKernelGGL(stage1_decode_score_kernel<true>, grid, dim3(64), 0, st, p);
    else hipLaunchKernelGGL(stage1_decode_score_kernel<false>, grid, dim3(64), 0, st, p);
    IV2_LAUNCH_CHECK();
    return 0;
}
