// Deterministic top-k over rows of 16-bit scores (gfx950), one wavefront per row, with the uint64 block mask of
// the selection emitted by the same wavefront.
//
// Order contract: the first k entries of a stable descending sort of the row — larger value
// first, equal values by ascending column — the comparator the reference states in
// csrc/topk.cuh:17,26,37.  Rows shorter than k are padded with -1.  The reference's own
// kernel (kernel_bitonic_topk_multiblock, csrc/topk.cuh:99-117) is limited to rows of at most
// 1024 columns and k <= 32; this kernel has no such limit within (n <= 8192, k <= 2048).
// The mask words are what csrc/topk_to_uint64.cuh:10-52 computes from the index list: bit (c % 64) of word
// c / 64 for every selected column c.
//
// The kernel is bound by instruction issue (vector and scalar units alike), not by memory: a row of 512 scores is
// 1 KiB.  So the method counts instructions:
//  * every lane keeps its strided share of the row (column 64 e + lane) in registers as order-preserving 16-bit
//    keys; a wavefront-wide count of "key >= candidate" is one compare per register plus scalar popcounts;
//  * the k-th largest key is found by bisection on that count.  A wavefront works through consecutive rows
//    (neighbouring query tokens) and starts each search at the previous row's threshold, galloping outward (first
//    step: twice the last move) until the count brackets k: about 8 counts instead of 16 on rows that resemble
//    their neighbour, exact whatever the data;
//  * with the strided layout the ballot of "column selected" over register e IS mask word e;
//  * survivors are compacted through a ballot prefix (ties taken by ascending column) into LDS as unique 32-bit
//    keys (key << 16 | inverted column); lanes that take nothing write a dummy slot, so there is no divergent
//    branch.  In score order up to 64 survivors are then ordered by a bitonic network across the lanes whose
//    exchanges are DPP operands of the min / max instructions themselves (no LDS traffic), more than 64 by rank
//    counting in LDS.  Index order (ascending column) needs no ordering step at all;
//  * the next row's scores are requested before the current row's search starts.
#include "common.h"
#include "infllmv2_hip.h"

namespace infllmv2 {

// order-preserving map of IEEE half / bfloat16 bits onto 1..0xffff: larger float <=> larger key; -0 and +0 share
// 0x8000; key 0 is free and marks "no element" (it loses every comparison and, lying in columns >= n, every tie)
__device__ __forceinline__ uint32_t sortable16(uint32_t b) {
    return b < 0x8000u ? b + 0x8000u : 0x10000u - b;
}
constexpr uint32_t kKeyNegInfBf16 = 0x10000u - 0xff80u;
constexpr uint32_t kKeyNegInfFp16 = 0x10000u - 0xfc00u;

struct TopkParams {
    const uint16_t* x;
    int64_t row_stride;
    int32_t* out_idx;
    uint16_t* out_val;               // optional: the selected values, in output order
    uint64_t* out_mask;              // optional: (rows, n64) mask words of the selection
    int out_stride, n64;
    int64_t rows;
    int n, k;
    int by_index;                    // 1: indices in ascending column order; 0: value order (the reference's comparator)
    int drop_neg_inf;                // 1: columns whose score is -inf are never selected (-1 instead)
    int rows_per_wave;
    uint32_t neg_inf_key;
};

constexpr int kTopkWaves = 4;

__device__ __forceinline__ int lanes_below(uint64_t mask, int base) {          // base + set bits of mask below this lane
    return __builtin_amdgcn_mbcnt_hi(static_cast<uint32_t>(mask >> 32),
                                     __builtin_amdgcn_mbcnt_lo(static_cast<uint32_t>(mask), static_cast<uint32_t>(base)));
}
// lane `which` (a constant) of the pair (lo, hi) replaced by the two halves of a wavefront-uniform 64-bit value.
// The value usually comes straight out of a vector compare: a vector instruction must not read a scalar register
// in the two slots after a vector instruction wrote it, and the compiler does not look inside asm (s_nop 1).
__device__ __forceinline__ void write_lane64(uint32_t& lo, uint32_t& hi, uint64_t uniform_value, int which) {
    asm volatile("s_nop 1\n\tv_writelane_b32 %0, %2, %4\n\tv_writelane_b32 %1, %3, %4"
                 : "+v"(lo), "+v"(hi)
                 : "s"(static_cast<uint32_t>(uniform_value)), "s"(static_cast<uint32_t>(uniform_value >> 32)), "n"(which));
}
// b where the lane's bit of the lane mask (a compile-time constant, so no vector instruction wrote it) is set, else a
__device__ __forceinline__ uint32_t select_by_lane_mask(uint32_t a, uint32_t b, uint64_t lane_mask) {
    uint32_t r;
    asm("v_cndmask_b32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "s"(lane_mask));
    return r;
}
// lanes that keep the larger key in the step (size, dist) of a bitonic network that sorts descending
constexpr uint64_t bitonic_keep_max_mask(int size, int dist) {
    uint64_t m = 0;
    for (int lane = 0; lane < 64; ++lane)
        if (((lane & dist) == 0) == ((lane & size) == 0)) m |= 1ull << lane;
    return m;
}
// One compare-exchange step with the lane at distance kDist.  Inside a 16-lane row the partner's key is a DPP operand
// of the min / max themselves; a DPP operand must not have been written by the two preceding instructions (s_nop 1).
// Across rows the row swaps hand every lane {its own key, the partner's} in some order, which min / max do not mind.
template <int kSize, int kDist>
__device__ __forceinline__ uint32_t bitonic_step(uint32_t x) {
    uint32_t mx, mn;
    if constexpr (kDist == 1) {
        asm("s_nop 1\n\tv_max_u32_dpp %0, %2, %2 quad_perm:[1,0,3,2] row_mask:0xf bank_mask:0xf\n\t"
            "v_min_u32_dpp %1, %2, %2 quad_perm:[1,0,3,2] row_mask:0xf bank_mask:0xf" : "=&v"(mx), "=&v"(mn) : "v"(x));
    } else if constexpr (kDist == 2) {
        asm("s_nop 1\n\tv_max_u32_dpp %0, %2, %2 quad_perm:[2,3,0,1] row_mask:0xf bank_mask:0xf\n\t"
            "v_min_u32_dpp %1, %2, %2 quad_perm:[2,3,0,1] row_mask:0xf bank_mask:0xf" : "=&v"(mx), "=&v"(mn) : "v"(x));
    } else if constexpr (kDist == 4) {
        // lanes 0-3 and 8-11 of a row (banks 0, 2) read four lanes up, the others four lanes down
        asm("s_nop 1\n\tv_max_u32_dpp %0, %2, %2 row_shl:4 row_mask:0xf bank_mask:0x5\n\t"
            "v_max_u32_dpp %0, %2, %2 row_shr:4 row_mask:0xf bank_mask:0xa\n\t"
            "v_min_u32_dpp %1, %2, %2 row_shl:4 row_mask:0xf bank_mask:0x5\n\t"
            "v_min_u32_dpp %1, %2, %2 row_shr:4 row_mask:0xf bank_mask:0xa" : "=&v"(mx), "=&v"(mn) : "v"(x));
    } else if constexpr (kDist == 8) {
        asm("s_nop 1\n\tv_max_u32_dpp %0, %2, %2 row_ror:8 row_mask:0xf bank_mask:0xf\n\t"
            "v_min_u32_dpp %1, %2, %2 row_ror:8 row_mask:0xf bank_mask:0xf" : "=&v"(mx), "=&v"(mn) : "v"(x));
    } else {
        typedef unsigned u2 __attribute__((ext_vector_type(2)));
        u2 r;
        if constexpr (kDist == 16) r = __builtin_amdgcn_permlane16_swap(x, x, false, false);
        else r = __builtin_amdgcn_permlane32_swap(x, x, false, false);
        mx = r[0] > r[1] ? r[0] : r[1];
        mn = r[0] > r[1] ? r[1] : r[0];
    }
    return select_by_lane_mask(mn, mx, bitonic_keep_max_mask(kSize, kDist));
}
template <int kSize, int kDist>
__device__ __forceinline__ uint32_t bitonic_merge(uint32_t x) {
    x = bitonic_step<kSize, kDist>(x);
    if constexpr (kDist > 1) x = bitonic_merge<kSize, kDist / 2>(x);
    return x;
}
template <int kSize>
__device__ __forceinline__ uint32_t bitonic_sort_desc(uint32_t x) {      // 64 keys, one per lane; lane 0 ends with the largest
    if constexpr (kSize > 2) x = bitonic_sort_desc<kSize / 2>(x);
    return bitonic_merge<kSize, kSize / 2>(x);
}

// kFull: the row has exactly 64 * kItems columns (no lane ever holds "no element")
template <int kItems, bool kByIndex, bool kMask, bool kFull>
__global__ __launch_bounds__(kTopkWaves * 64)
void topk_rows_kernel(const TopkParams p) {
    extern __shared__ uint32_t lds_keys[];                    // kTopkWaves * (k + 64): survivors, then one dummy slot per lane
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int64_t row_begin = (static_cast<int64_t>(blockIdx.x) * kTopkWaves + wave) * p.rows_per_wave;
    if (row_begin >= p.rows) return;                           // uniform per wavefront; no workgroup barrier below
    const int64_t row_end = row_begin + p.rows_per_wave < p.rows ? row_begin + p.rows_per_wave : p.rows;
    const int n = p.n, k = p.k;
    const int k_sel = k < n ? k : n;
    uint32_t* sel = lds_keys + wave * (k + 64);
    const int dummy = k + lane;                                // where a lane that takes nothing writes
    constexpr bool kPrefetch = kItems <= 32;

    // columns beyond the row read column 0 and get key 0 ("no element"); n == 0 reads nothing
    auto load_row = [&](uint32_t (&dst)[kItems], int64_t row) {
        if (n <= 0) return;
        const uint16_t* src = p.x + row * p.row_stride;
#pragma unroll
        for (int e = 0; e < kItems; ++e) {
            const int col = e * 64 + lane;
            dst[e] = src[kFull || col < n ? col : 0];
        }
    };
    auto to_keys = [&](uint32_t (&key)[kItems], const uint32_t (&raw)[kItems]) {
#pragma unroll
        for (int e = 0; e < kItems; ++e) key[e] = (kFull || e * 64 + lane < n) ? sortable16(raw[e]) : 0u;
    };

    uint32_t raw[kItems];                                      // short rows: the next row's scores
    if constexpr (kPrefetch) load_row(raw, row_begin);
    uint32_t thr_prev = 0, step_prev = 8;
    bool have_prev = false;

    for (int64_t row = row_begin; row < row_end; ++row) {
        uint32_t key[kItems];
        if constexpr (kPrefetch) {
            to_keys(key, raw);
            if (row + 1 < row_end) load_row(raw, row + 1);
        } else {
            load_row(raw, row);
            to_keys(key, raw);
        }

        auto count_ge = [&](uint32_t cand) -> int {
            int cnt = 0;
#pragma unroll
            for (int e = 0; e < kItems; ++e) cnt += __builtin_popcountll(__builtin_amdgcn_ballot_w64(key[e] >= cand));
            return cnt;
        };

        // thr = largest candidate with count(key >= thr) >= k_sel.  lo always satisfies it, hi never does.
        uint32_t lo = 0, hi = 0x10000u;
        int cnt_lo = kItems * 64;
        if (k_sel > 0) {
            if (have_prev) {
                // gallop away from the previous row's threshold until the count brackets k_sel
                const int c0 = count_ge(thr_prev);
                const bool up = c0 >= k_sel;
                uint32_t w = step_prev;
                if (up) { lo = thr_prev; cnt_lo = c0; } else hi = thr_prev;
                for (;;) {
                    uint32_t probe;
                    if (up) {
                        probe = lo + w;
                        if (probe >= 0x10000u) break;
                    } else {
                        if (hi <= w) break;                    // lo = 0 holds by construction
                        probe = hi - w;
                    }
                    const int c = count_ge(probe);
                    if (c >= k_sel) { lo = probe; cnt_lo = c; if (!up) break; }
                    else { hi = probe; if (up) break; }
                    w <<= 2;
                }
            }
            while (hi - lo > 1) {
                const uint32_t mid = (lo + hi) >> 1;
                const int c = count_ge(mid);
                if (c >= k_sel) { lo = mid; cnt_lo = c; } else hi = mid;
            }
        }
        uint32_t thr = lo;
        {
            const uint32_t moved = thr > thr_prev ? thr - thr_prev : thr_prev - thr;
            step_prev = have_prev ? (moved < 4 ? 8 : (moved > 2048 ? 4096 : 2 * moved)) : 8;
        }
        thr_prev = thr;
        have_prev = true;

        // which elements are taken: everything above thr, and of the elements equal to thr the first by column
        bool all_ge = (cnt_lo == k_sel);                       // no tie to break: take key >= thr
        if (p.drop_neg_inf && thr <= p.neg_inf_key) {          // fewer than k_sel scores lie above -inf: take exactly those
            thr = p.neg_inf_key + 1;
            all_ge = true;
        }
        if (k_sel == 0) { thr = 0x10000u; all_ge = true; }     // nothing to take

        int base = 0;
        uint32_t words0_lo = 0, words0_hi = 0, words1_lo = 0, words1_hi = 0;   // lane e holds mask word e (e + 64)
        const uint32_t inv_lane = 0xffffu - static_cast<uint32_t>(lane);
        auto emit = [&](int e, bool take, uint64_t take_mask) {
            const int slot = lanes_below(take_mask, base);
            uint32_t val;
            if constexpr (kByIndex) val = static_cast<uint32_t>(e * 64 + lane);
            else val = (key[e] << 16) | (inv_lane - static_cast<uint32_t>(e * 64));
            sel[take ? slot : dummy] = val;
            base += __builtin_popcountll(take_mask);
            if constexpr (kMask) {                             // the ballot is the mask word
                if (e < 64) write_lane64(words0_lo, words0_hi, take_mask, e & 63);
                else write_lane64(words1_lo, words1_hi, take_mask, e & 63);
            }
        };
        if (all_ge) {
#pragma unroll
            for (int e = 0; e < kItems; ++e) {
                const bool take = key[e] >= thr;
                emit(e, take, __builtin_amdgcn_ballot_w64(take));
            }
        } else {
            int ties_left = k_sel - count_ge(thr + 1);
#pragma unroll
            for (int e = 0; e < kItems; ++e) {
                const bool eq = key[e] == thr;
                const uint64_t eq_mask = __builtin_amdgcn_ballot_w64(eq);
                const bool take = key[e] > thr || (eq && lanes_below(eq_mask, 0) < ties_left);
                emit(e, take, __builtin_amdgcn_ballot_w64(take));
                const int eq_total = __builtin_popcountll(eq_mask);
                ties_left -= eq_total < ties_left ? eq_total : ties_left;
            }
        }
        if constexpr (kMask) {
            uint64_t* mask_row = p.out_mask + row * p.n64;
            const uint64_t words0 = (static_cast<uint64_t>(words0_hi) << 32) | words0_lo;
            const uint64_t words1 = (static_cast<uint64_t>(words1_hi) << 32) | words1_lo;
            for (int w = lane; w < p.n64; w += 64) mask_row[w] = w < 64 ? words0 : (w < 128 ? words1 : 0ull);
        }
        const int taken = base;                                // <= k_sel
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");

        int32_t* dst = p.out_idx + row * p.out_stride;
        uint16_t* dst_val = p.out_val ? p.out_val + row * p.out_stride : nullptr;
        const uint16_t* src = p.x + row * p.row_stride;
        if constexpr (kByIndex) {
            for (int i = lane; i < taken; i += 64) {
                const uint32_t col = sel[i];
                dst[i] = static_cast<int32_t>(col);
                if (dst_val) dst_val[i] = src[col];
            }
        } else if (taken <= 64) {
            // one survivor per lane, ordered by a bitonic network over the lanes (descending; empty lanes hold 0)
            const uint32_t mine = bitonic_sort_desc<64>(lane < taken ? sel[lane] : 0u);
            if (lane < taken) {
                const uint32_t col = 0xffffu - (mine & 0xffffu);
                dst[lane] = static_cast<int32_t>(col);
                if (dst_val) dst_val[lane] = src[col];
            }
        } else {
            // rank of each survivor among the survivors = its output slot
            for (int i = lane; i < taken; i += 64) {
                const uint32_t mine = sel[i];
                int rank = 0;
                for (int j = 0; j < taken; ++j) rank += sel[j] > mine;
                const uint32_t col = 0xffffu - (mine & 0xffffu);
                dst[rank] = static_cast<int32_t>(col);
                if (dst_val) dst_val[rank] = src[col];
            }
        }
        for (int i = taken + lane; i < p.out_stride; i += 64) {
            dst[i] = -1;
            if (dst_val) dst_val[i] = 0;
        }
        // the next row reuses sel: every lane has read what it needs
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
    }
}

template <int kItems>
static int launch_topk(void* stream, const TopkParams& p) {
    const int64_t waves = (p.rows + p.rows_per_wave - 1) / p.rows_per_wave;
    const int64_t blocks = (waves + kTopkWaves - 1) / kTopkWaves;
    IV2_CHECK(blocks <= 0x7fffffffll, "topk: too many rows");
    const size_t lds = sizeof(uint32_t) * kTopkWaves * (p.k + 64);
    const dim3 grid(static_cast<unsigned>(blocks)), block(kTopkWaves * 64);
    hipStream_t st = static_cast<hipStream_t>(stream);
    const int variant = (p.by_index ? 4 : 0) | (p.out_mask ? 2 : 0) | (p.n == kItems * 64 ? 1 : 0);
    switch (variant) {
        case 0: hipLaunchKernelGGL((topk_rows_kernel<kItems, false, false, false>), grid, block, lds, st, p); break;
        case 1: hipLaunchKernelGGL((topk_rows_kernel<kItems, false, false, true>), grid, block, lds, st, p); break;
        case 2: hipLaunchKernelGGL((topk_rows_kernel<kItems, false, true, false>), grid, block, lds, st, p); break;
        case 3: hipLaunchKernelGGL((topk_rows_kernel<kItems, false, true, true>), grid, block, lds, st, p); break;
        case 4: hipLaunchKernelGGL((topk_rows_kernel<kItems, true, false, false>), grid, block, lds, st, p); break;
        case 5: hipLaunchKernelGGL((topk_rows_kernel<kItems, true, false, true>), grid, block, lds, st, p); break;
        case 6: hipLaunchKernelGGL((topk_rows_kernel<kItems, true, true, false>), grid, block, lds, st, p); break;
        default: hipLaunchKernelGGL((topk_rows_kernel<kItems, true, true, true>), grid, block, lds, st, p); break;
    }
    IV2_LAUNCH_CHECK();
    return 0;
}

static int topk_dispatch(void* stream, const uint16_t* x, int64_t row_stride, int32_t* idx, uint16_t* val,
                         uint64_t* mask, int n64, int out_stride, int64_t rows, int n, int k, int by_index,
                         int drop_neg_inf, int dtype) {
    IV2_CHECK(rows >= 0 && n >= 0 && k >= 0, "topk: negative size");
    IV2_CHECK(n <= 8192, "topk: row length %d exceeds 8192", n);
    IV2_CHECK(k <= 2048, "topk: k %d exceeds 2048", k);
    IV2_CHECK(out_stride >= k, "topk: output row stride %d shorter than k %d", out_stride, k);
    IV2_CHECK(mask == nullptr || (n64 > 0 && static_cast<int64_t>(n64) * 64 >= n),
              "topk: %d mask words per row cannot hold %d columns", n64, n);
    if (rows == 0 || (out_stride == 0 && mask == nullptr)) return 0;
    TopkParams p{};
    p.x = x; p.row_stride = row_stride; p.out_idx = idx; p.out_val = val; p.out_mask = mask;
    p.out_stride = out_stride; p.n64 = n64; p.rows = rows; p.n = n; p.k = k;
    p.by_index = by_index; p.drop_neg_inf = drop_neg_inf; p.neg_inf_key = dtype == 0 ? kKeyNegInfFp16 : kKeyNegInfBf16;
    // consecutive rows per wavefront (each search starts from the previous row's threshold), but never so many
    // that fewer than ~32 wavefronts per CU of a 256-CU device remain
    int rpw = 16;
    while (rpw > 1 && rows / rpw < 8192) rpw >>= 1;
    p.rows_per_wave = rpw;
    if (n <= 256) return launch_topk<4>(stream, p);
    if (n <= 512) return launch_topk<8>(stream, p);
    if (n <= 1024) return launch_topk<16>(stream, p);
    if (n <= 2048) return launch_topk<32>(stream, p);
    if (n <= 4096) return launch_topk<64>(stream, p);
    return launch_topk<128>(stream, p);
}

}  // namespace infllmv2

using namespace infllmv2;

extern "C" int infllmv2_topk_blocks(void* stream, const void* pooled, int64_t row_stride, int32_t* topk_idx,
                                    int64_t rows, int n, int k) {
    return topk_dispatch(stream, static_cast<const uint16_t*>(pooled), row_stride, topk_idx, nullptr, nullptr, 0, k,
                         rows, n, k, 0, 0, 1);
}

extern "C" int infllmv2_topk_select(void* stream, const void* pooled, int64_t row_stride, int dtype, int32_t* topk_idx,
                                    uint64_t* mask_words, int64_t rows, int n, int k, int n_uint64_per_row,
                                    int by_index, int drop_neg_inf) {
    IV2_CHECK(dtype == 0 || dtype == 1, "topk_select: dtype must be 0 (fp16) or 1 (bf16)");
    IV2_CHECK(topk_idx != nullptr, "topk_select: topk_idx must be given");
    return topk_dispatch(stream, static_cast<const uint16_t*>(pooled), row_stride, topk_idx, nullptr, mask_words,
                         n_uint64_per_row, k, rows, n, k, by_index ? 1 : 0, drop_neg_inf ? 1 : 0, dtype);
}

extern "C" int infllmv2_topk(void* stream, int num_tokens, int dim, int top, int dtype, const void* x,
                             void* topk_val, int32_t* topk_pos) {
    IV2_CHECK(dtype == 0 || dtype == 1, "topk: dtype must be 0 (fp16) or 1 (bf16)");
    IV2_CHECK(top >= 1, "topk: top must be at least 1");
    int top_size = 1;
    while (top_size < top) top_size <<= 1;                     // output row stride, csrc/topk.cuh:108,119-141
    return topk_dispatch(stream, static_cast<const uint16_t*>(x), dim, topk_pos,
                         static_cast<uint16_t*>(topk_val), nullptr, 0, top_size, num_tokens, dim, top, 0, 0, dtype);
}
