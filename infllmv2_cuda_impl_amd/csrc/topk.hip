// Deterministic top-k over rows of 16-bit scores (gfx950), one wavefront per row.
//
// Order contract: the first k entries of a stable descending sort of the row — larger value
// first, equal values by ascending column — the comparator the reference states in
// csrc/topk.cuh:17,26,37.  Rows shorter than k are padded with -1.  The reference's own
// kernel (kernel_bitonic_topk_multiblock, csrc/topk.cuh:99-117) is limited to rows of at most
// 1024 columns and k <= 32; this kernel has no such limit within (n <= 8192, k <= 2048).
//
// Method: every lane keeps its strided share of the row in registers as order-preserving
// 16-bit keys.  A 16-step bitwise search with ballot/popcount finds the k-th largest value V;
// entries greater than V plus the lowest-column ties are compacted into LDS through a ballot
// prefix, then each survivor's output slot is its rank among the survivors (keys are made
// unique by appending the inverted column).  No sort of the whole row, no global scratch.
#include "common.h"
#include "../../include/infllmv2_hip.h"

namespace infllmv2 {

// order-preserving map of IEEE half / bfloat16 bits: larger float <=> larger key; -0 == +0.
__device__ __forceinline__ uint32_t sortable16(uint16_t b) {
    if (b == 0x8000) b = 0;
    return (b & 0x8000) ? static_cast<uint16_t>(~b) : static_cast<uint16_t>(b | 0x8000);
}

template <int kItems, int kWavesPerBlock>
__global__ __launch_bounds__(kWavesPerBlock * 64)
void topk_rows_kernel(const uint16_t* __restrict__ x, int64_t row_stride, int32_t* __restrict__ out_idx,
                      uint16_t* __restrict__ out_val, int out_stride, int64_t rows, int n, int k) {
    extern __shared__ uint32_t lds_keys[];                    // kWavesPerBlock * k_sel_cap
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int64_t row = static_cast<int64_t>(blockIdx.x) * kWavesPerBlock + wave;
    if (row >= rows) return;                                   // uniform per wavefront; no block barriers below
    const int k_sel = k < n ? k : n;
    uint32_t* sel = lds_keys + wave * k;
    const uint16_t* src = x + row * row_stride;

    uint32_t key[kItems];
#pragma unroll
    for (int e = 0; e < kItems; ++e) {
        const int col = e * 64 + lane;
        key[e] = col < n ? (sortable16(src[col]) + 1u) : 0u;   // 0 marks "no element"; real keys are 1..65536
    }

    // largest V (in key units) with count(key >= V) >= k_sel
    uint32_t thr = 0;
    if (k_sel > 0) {
        for (int bit = 16; bit >= 0; --bit) {
            const uint32_t cand = thr | (1u << bit);
            int cnt = 0;
#pragma unroll
            for (int e = 0; e < kItems; ++e) cnt += __builtin_popcountll(__builtin_amdgcn_ballot_w64(key[e] >= cand));
            if (cnt >= k_sel) thr = cand;
        }
    }
    int n_gt = 0;
#pragma unroll
    for (int e = 0; e < kItems; ++e) n_gt += __builtin_popcountll(__builtin_amdgcn_ballot_w64(key[e] > thr));
    int ties_left = k_sel - n_gt;                              // ties taken in ascending column order

    // compact survivors into LDS as unique 32-bit keys (value key << 16 | inverted column)
    int base = 0;
    const uint64_t lane_lt = (lane == 0) ? 0ull : (~0ull >> (64 - lane));
#pragma unroll
    for (int e = 0; e < kItems; ++e) {
        const bool gt = key[e] > thr;
        const bool eq = (key[e] == thr) && thr != 0;
        const uint64_t eq_mask = __builtin_amdgcn_ballot_w64(eq);
        const int eq_before = __builtin_popcountll(eq_mask & lane_lt);
        const bool take = gt || (eq && eq_before < ties_left);
        const uint64_t take_mask = __builtin_amdgcn_ballot_w64(take);
        if (take) {
            const int slot = base + __builtin_popcountll(take_mask & lane_lt);
            const uint32_t col = static_cast<uint32_t>(e * 64 + lane);
            sel[slot] = ((key[e] - 1u) << 16) | (0xffffu - col);
        }
        base += __builtin_popcountll(take_mask);
        const int eq_total = __builtin_popcountll(eq_mask);
        ties_left -= eq_total < ties_left ? eq_total : ties_left;
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");

    // rank of each survivor among the survivors = its output slot
    int32_t* dst = out_idx + row * out_stride;
    uint16_t* dst_val = out_val ? out_val + row * out_stride : nullptr;
    for (int i = lane; i < k_sel; i += 64) {
        const uint32_t mine = sel[i];
        int rank = 0;
        for (int j = 0; j < k_sel; ++j) rank += sel[j] > mine;
        const uint32_t col = 0xffffu - (mine & 0xffffu);
        dst[rank] = static_cast<int32_t>(col);
        if (dst_val) dst_val[rank] = src[col];
    }
    for (int i = k_sel + lane; i < out_stride; i += 64) {
        dst[i] = -1;
        if (dst_val) dst_val[i] = (i < k) ? 0 : 0;
    }
}

template <int kItems>
static int launch_topk(void* stream, const uint16_t* x, int64_t row_stride, int32_t* idx, uint16_t* val,
                       int out_stride, int64_t rows, int n, int k) {
    constexpr int kWaves = 4;
    const int64_t blocks = (rows + kWaves - 1) / kWaves;
    IV2_CHECK(blocks <= 0x7fffffffll, "topk: too many rows");
    const size_t lds = sizeof(uint32_t) * kWaves * (k > 0 ? k : 1);
    hipLaunchKernelGGL((topk_rows_kernel<kItems, kWaves>), dim3(static_cast<unsigned>(blocks)), dim3(kWaves * 64), lds,
                       static_cast<hipStream_t>(stream), x, row_stride, idx, val, out_stride, rows, n, k);
    IV2_LAUNCH_CHECK();
    return 0;
}

static int topk_dispatch(void* stream, const uint16_t* x, int64_t row_stride, int32_t* idx, uint16_t* val,
                         int out_stride, int64_t rows, int n, int k) {
    IV2_CHECK(rows >= 0 && n >= 0 && k >= 0, "topk: negative size");
    IV2_CHECK(n <= 8192, "topk: row length %d exceeds 8192", n);
    IV2_CHECK(k <= 2048, "topk: k %d exceeds 2048", k);
    IV2_CHECK(out_stride >= k, "topk: output row stride %d shorter than k %d", out_stride, k);
    if (rows == 0 || out_stride == 0) return 0;
    if (n <= 256) return launch_topk<4>(stream, x, row_stride, idx, val, out_stride, rows, n, k);
    if (n <= 512) return launch_topk<8>(stream, x, row_stride, idx, val, out_stride, rows, n, k);
    if (n <= 1024) return launch_topk<16>(stream, x, row_stride, idx, val, out_stride, rows, n, k);
    if (n <= 2048) return launch_topk<32>(stream, x, row_stride, idx, val, out_stride, rows, n, k);
    if (n <= 4096) return launch_topk<64>(stream, x, row_stride, idx, val, out_stride, rows, n, k);
    return launch_topk<128>(stream, x, row_stride, idx, val, out_stride, rows, n, k);
}

}  // namespace infllmv2

using namespace infllmv2;

extern "C" int infllmv2_topk_blocks(void* stream, const void* pooled, int64_t row_stride, int32_t* topk_idx,
                                    int64_t rows, int n, int k) {
    return topk_dispatch(stream, static_cast<const uint16_t*>(pooled), row_stride, topk_idx, nullptr, k, rows, n, k);
}

extern "C" int infllmv2_topk(void* stream, int num_tokens, int dim, int top, int dtype, const void* x,
                             void* topk_val, int32_t* topk_pos) {
    IV2_CHECK(dtype == 0 || dtype == 1, "topk: dtype must be 0 (fp16) or 1 (bf16)");
    IV2_CHECK(top >= 1, "topk: top must be at least 1");
    int top_size = 1;
    while (top_size < top) top_size <<= 1;                     // output row stride, csrc/topk.cuh:108,119-141
    return topk_dispatch(stream, static_cast<const uint16_t*>(x), dim, topk_pos,
                         static_cast<uint16_t*>(topk_val), top_size, num_tokens, dim, top);
}
