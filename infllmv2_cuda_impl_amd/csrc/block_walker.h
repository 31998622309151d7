// Mask-row iteration and small cross-lane helpers shared by the Stage-2 kernels.
#pragma once
#include "common.h"

namespace IV2_NS {

// Walks the set bits of one mask row in ascending block order, clipped to [0, last_blk].
struct BlockWalker {
    const uint64_t* row;
    int n_words;                    // words that can hold an allowed block
    int last_blk;
    int w;
    uint64_t bits;

    __device__ __forceinline__ uint64_t load_word(int word) const {
        uint64_t v = row ? row[word] : ~0ull;
        if (word == (last_blk >> 6)) {
            const int t = last_blk & 63;
            v &= (t == 63) ? ~0ull : ((1ull << (t + 1)) - 1ull);
        }
        // the row is shared by the whole wavefront: keep the loop control in scalar registers
        const uint32_t lo = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(v));
        const uint32_t hi = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(v >> 32));
        return (static_cast<uint64_t>(hi) << 32) | lo;
    }
    __device__ __forceinline__ void init(const uint64_t* r, int words_in_row, int last) {
        row = r;
        last_blk = last;
        n_words = last < 0 ? 0 : (last >> 6) + 1;
        if (row && n_words > words_in_row) n_words = words_in_row;
        w = 0;
        bits = n_words > 0 ? load_word(0) : 0ull;
    }
    __device__ __forceinline__ int next() {
        while (bits == 0ull) {
            if (++w >= n_words) return -1;
            bits = load_word(w);
        }
        const int bit = __builtin_ctzll(bits);
        bits &= bits - 1ull;
        return w * 64 + bit;
    }
};

// Cross-row exchanges with gfx950's v_permlane16_swap / v_permlane32_swap (VALU speed; a ds_bpermute takes a trip
// through the LDS crossbar): swapping a register with itself hands every lane its own row's value and the partner
// row's value.
__device__ __forceinline__ void row_pair_xor16(float x, float& mine, float& other) {
    typedef unsigned u2 __attribute__((ext_vector_type(2)));
    const u2 r = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    mine = __uint_as_float(r[0]);
    other = __uint_as_float(r[1]);
}
__device__ __forceinline__ void row_pair_xor32(float x, float& mine, float& other) {
    typedef unsigned u2 __attribute__((ext_vector_type(2)));
    const u2 r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    mine = __uint_as_float(r[0]);
    other = __uint_as_float(r[1]);
}
// reductions over the four 16-lane groups g of a wavefront (lanes l, l ^ 16, l ^ 32, l ^ 48)
__device__ __forceinline__ float wave_max_over_g(float x) {
    float a, b;
    row_pair_xor16(x, a, b);
    x = fmaxf(a, b);
    row_pair_xor32(x, a, b);
    return fmaxf(a, b);
}
__device__ __forceinline__ float wave_sum_over_g(float x) {
    float a, b;
    row_pair_xor16(x, a, b);
    x = a + b;
    row_pair_xor32(x, a, b);
    return a + b;
}

}  // namespace IV2_NS
