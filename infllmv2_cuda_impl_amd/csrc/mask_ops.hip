// Block-mask bit kernels for gfx950: index list -> uint64 words, words <-> bool bytes, and the
// 64x64 bit-matrix transposition that turns the forward (row-major) mask into the mask the
// backward walks.  One wavefront is 64 lanes, so one ballot is exactly one mask word.
//
// Behaviour follows csrc/topk_to_uint64.cuh:10-52, csrc/uint64_to_bool.cuh:10-43,
// csrc/blockmask_to_uint64.cuh:10-51 and infllm_v2/infllmv2_sparse_attention.py:344-350 of the
// reference; the kernels themselves are new.
#include "common.h"
#include "infllmv2_hip.h"

namespace infllmv2 {

// ---------------------------------------------------------------------------------------------
// topk_idx (rows, k) int32  ->  words (rows, n64) uint64.
// One wavefront per row.  Each lane ORs its indices into an LDS copy of the row's words
// (ds_or_b64), then the first n64 lanes store the row: every input index is read exactly once
// and every output word is written exactly once.
// ---------------------------------------------------------------------------------------------
template <int kWavesPerBlock>
__global__ __launch_bounds__(kWavesPerBlock * 64)
void topk_to_uint64_kernel(const int32_t* __restrict__ idx, uint64_t* __restrict__ out,
                           int64_t rows, int k, int n64) {
    extern __shared__ unsigned long long lds_words[];          // kWavesPerBlock * n64
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int64_t row = static_cast<int64_t>(blockIdx.x) * kWavesPerBlock + wave;
    unsigned long long* words = lds_words + wave * n64;
    for (int w = lane; w < n64; w += 64) words[w] = 0ull;
    __syncthreads();
    if (row < rows) {
        const int32_t* src = idx + row * k;
        const int limit = n64 * 64;
        for (int i = lane; i < k; i += 64) {
            const int v = src[i];
            if (v >= 0 && v < limit) atomicOr(&words[v >> 6], 1ull << (v & 63));
        }
    }
    __syncthreads();
    if (row < rows) {
        for (int w = lane; w < n64; w += 64) out[row * n64 + w] = words[w];
    }
}

// ---------------------------------------------------------------------------------------------
// words (rows, n64) -> bool bytes (rows, last_dim).  One thread expands one byte of a word
// into eight 0/1 bytes and stores them as a single 8-byte write when the row is 8-aligned.
// ---------------------------------------------------------------------------------------------
__device__ __forceinline__ uint64_t spread_bits_to_bytes(uint32_t b) {
    uint64_t x = (static_cast<uint64_t>(b) * 0x0101010101010101ull) & 0x8040201008040201ull;
    return ((x + 0x7f7f7f7f7f7f7f7full) >> 7) & 0x0101010101010101ull;
}

__global__ __launch_bounds__(256)
void uint64_to_bool_kernel(const uint64_t* __restrict__ in, uint8_t* __restrict__ out,
                           int64_t rows, int last_dim, int n64, int groups_per_row, bool aligned) {
    const int64_t gid = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (gid >= rows * groups_per_row) return;
    const int64_t row = gid / groups_per_row;
    const int grp = static_cast<int>(gid - row * groups_per_row);     // 8 columns per group
    const int col0 = grp * 8;
    const uint64_t word = in[row * n64 + (col0 >> 6)];
    const uint32_t byte = static_cast<uint32_t>(word >> (col0 & 63)) & 0xffu;
    const uint64_t bytes = spread_bits_to_bytes(byte);
    uint8_t* dst = out + row * last_dim + col0;
    if (aligned && col0 + 8 <= last_dim) {
        *reinterpret_cast<uint64_t*>(dst) = bytes;
    } else {
        for (int j = 0; j < 8 && col0 + j < last_dim; ++j) dst[j] = static_cast<uint8_t>((bytes >> (8 * j)) & 1u);
    }
}

// ---------------------------------------------------------------------------------------------
// bool bytes (rows, last_dim) -> words (rows, n64).  One wavefront per output word: lane j
// reads byte 64w + j (a 64-byte coalesced read) and the ballot is the word.
// ---------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256)
void blockmask_to_uint64_kernel(const uint8_t* __restrict__ in, uint64_t* __restrict__ out,
                                int64_t rows, int last_dim, int n64) {
    const int lane = threadIdx.x & 63;
    const int64_t word_id = static_cast<int64_t>(blockIdx.x) * (blockDim.x >> 6) + (threadIdx.x >> 6);
    if (word_id >= rows * n64) return;                       // uniform per wavefront
    const int64_t row = word_id / n64;
    const int w = static_cast<int>(word_id - row * n64);
    const int col = w * 64 + lane;
    const bool bit = col < last_dim && in[row * last_dim + col] != 0;
    const uint64_t word = __builtin_amdgcn_ballot_w64(bit);
    if (lane == 0) out[word_id] = word;
}

// ---------------------------------------------------------------------------------------------
// Forward mask (heads, total_q, n64_fwd) -> backward mask (heads, k_blocks, n64_bwd):
//   bwd[h, kb, w] bit u  =  fwd[h, 64w + u, kb / 64] bit (kb % 64).
// One wavefront transposes one 64x64 bit tile: lane u holds the forward word of token 64w+u,
// 64 ballots produce the 64 backward words of the tile, lane b stores word b.
// ---------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256)
void transpose_blockmask_kernel(const uint64_t* __restrict__ fwd, uint64_t* __restrict__ bwd,
                                int heads, int64_t total_q, int n64_fwd, int k_blocks, int n64_bwd) {
    const int lane = threadIdx.x & 63;
    const int64_t tile = static_cast<int64_t>(blockIdx.x) * (blockDim.x >> 6) + (threadIdx.x >> 6);
    const int64_t tiles_per_head = static_cast<int64_t>(n64_bwd) * n64_fwd;
    if (tile >= tiles_per_head * heads) return;              // uniform per wavefront
    const int h = static_cast<int>(tile / tiles_per_head);
    const int64_t rem = tile - h * tiles_per_head;
    const int w = static_cast<int>(rem / n64_fwd);           // 64-token group
    const int c = static_cast<int>(rem - static_cast<int64_t>(w) * n64_fwd);   // forward word column
    const int64_t tok = static_cast<int64_t>(w) * 64 + lane;
    uint64_t mine = 0;
    if (tok < total_q) mine = fwd[(static_cast<int64_t>(h) * total_q + tok) * n64_fwd + c];
    uint64_t result = 0;
#pragma unroll
    for (int b = 0; b < 64; ++b) {
        const uint64_t col = __builtin_amdgcn_ballot_w64(((mine >> b) & 1ull) != 0);
        if (lane == b) result = col;
    }
    const int kb = c * 64 + lane;
    if (kb < k_blocks) bwd[(static_cast<int64_t>(h) * k_blocks + kb) * n64_bwd + w] = result;
}

}  // namespace infllmv2

using namespace infllmv2;

extern "C" int infllmv2_topk_to_uint64(void* stream, const int32_t* topk_idx, uint64_t* result,
                                       int64_t rows, int k, int k_blocks, int n_uint64_per_row) {
    IV2_CHECK(rows >= 0 && k >= 0 && n_uint64_per_row >= 0, "topk_to_uint64: negative size");
    IV2_CHECK(n_uint64_per_row <= 1024, "topk_to_uint64: n_uint64_per_row %d exceeds 1024", n_uint64_per_row);
    (void)k_blocks;
    if (rows == 0 || n_uint64_per_row == 0) return 0;
    constexpr int kWaves = 4;
    const int64_t blocks = (rows + kWaves - 1) / kWaves;
    IV2_CHECK(blocks <= 0x7fffffffll, "topk_to_uint64: too many rows");
    const size_t lds = sizeof(uint64_t) * kWaves * n_uint64_per_row;
    hipLaunchKernelGGL(topk_to_uint64_kernel<kWaves>, dim3(static_cast<unsigned>(blocks)), dim3(kWaves * 64), lds,
                       static_cast<hipStream_t>(stream), topk_idx, result, rows, k, n_uint64_per_row);
    IV2_LAUNCH_CHECK();
    return 0;
}

extern "C" int infllmv2_uint64_to_bool(void* stream, const uint64_t* input, uint8_t* result,
                                       int64_t rows, int last_dim_size, int n_uint64_per_row) {
    IV2_CHECK(rows >= 0 && last_dim_size >= 0, "uint64_to_bool: negative size");
    IV2_CHECK(static_cast<int64_t>(n_uint64_per_row) * 64 >= last_dim_size,
              "uint64_to_bool: %d words cannot hold %d bits", n_uint64_per_row, last_dim_size);
    if (rows == 0 || last_dim_size == 0) return 0;
    const int groups = (last_dim_size + 7) / 8;
    const int64_t total = rows * groups;
    const int64_t blocks = (total + 255) / 256;
    IV2_CHECK(blocks <= 0x7fffffffll, "uint64_to_bool: too many elements");
    const bool aligned = (last_dim_size % 8 == 0) && (reinterpret_cast<uintptr_t>(result) % 8 == 0);
    hipLaunchKernelGGL(uint64_to_bool_kernel, dim3(static_cast<unsigned>(blocks)), dim3(256), 0,
                       static_cast<hipStream_t>(stream), input, result, rows, last_dim_size,
                       n_uint64_per_row, groups, aligned);
    IV2_LAUNCH_CHECK();
    return 0;
}

extern "C" int infllmv2_blockmask_to_uint64(void* stream, const uint8_t* blockmask, uint64_t* result,
                                            int64_t rows, int last_dim_size, int n_uint64_per_row) {
    IV2_CHECK(rows >= 0 && last_dim_size >= 0, "blockmask_to_uint64: negative size");
    IV2_CHECK(n_uint64_per_row == (last_dim_size + 63) / 64,
              "blockmask_to_uint64: n_uint64_per_row %d does not match last dim %d", n_uint64_per_row, last_dim_size);
    const int64_t words = rows * n_uint64_per_row;
    if (words == 0) return 0;
    const int64_t blocks = (words + 3) / 4;
    IV2_CHECK(blocks <= 0x7fffffffll, "blockmask_to_uint64: too many elements");
    hipLaunchKernelGGL(blockmask_to_uint64_kernel, dim3(static_cast<unsigned>(blocks)), dim3(256), 0,
                       static_cast<hipStream_t>(stream), blockmask, result, rows, last_dim_size, n_uint64_per_row);
    IV2_LAUNCH_CHECK();
    return 0;
}

extern "C" int infllmv2_transpose_blockmask(void* stream, const uint64_t* fwd_mask, uint64_t* bwd_mask,
                                            int heads, int64_t total_q, int n64_fwd, int k_blocks, int n64_bwd) {
    IV2_CHECK(heads >= 0 && total_q >= 0 && k_blocks >= 0, "transpose_blockmask: negative size");
    IV2_CHECK(n64_bwd == static_cast<int>((total_q + 63) / 64), "transpose_blockmask: n64_bwd %d != ceil(total_q/64)", n64_bwd);
    IV2_CHECK(static_cast<int64_t>(n64_fwd) * 64 >= k_blocks, "transpose_blockmask: forward words too few for %d blocks", k_blocks);
    const int64_t tiles = static_cast<int64_t>(heads) * n64_bwd * n64_fwd;
    if (tiles == 0 || k_blocks == 0) return 0;
    const int64_t blocks = (tiles + 3) / 4;
    IV2_CHECK(blocks <= 0x7fffffffll, "transpose_blockmask: too many tiles");
    hipLaunchKernelGGL(transpose_blockmask_kernel, dim3(static_cast<unsigned>(blocks)), dim3(256), 0,
                       static_cast<hipStream_t>(stream), fwd_mask, bwd_mask, heads, total_q, n64_fwd, k_blocks, n64_bwd);
    IV2_LAUNCH_CHECK();
    return 0;
}
