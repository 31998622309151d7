// 1-D max-pooling of Stage-1 scores onto 64-token key blocks (gfx950).
//
// Rule (csrc/max_pooling_1d.cuh:107-160 fixed length, :12-103 packed):
//   bq = (q + cache_len) / block_size
//   out[h, q, kb] = +inf                     if kb < init_blocks or kb <= bq <= kb + local_blocks
//                 = max(in[h, q, max(0, kb*stride - padding) : min(k_len, kb*stride - padding + kernel_size)])
//                 = -inf                     if that window is empty
// The maximum is taken with the reference's sequential ">" scan so NaN and signed-zero inputs
// pick the same element.  Values are copied, never re-rounded, so the result is bit-exact.
//
// The kernel is HBM-bound.  Score rows are rarely aligned (2047 columns at 32768 tokens), so a
// wavefront copies a whole row into its own LDS slice with 16-byte loads from the aligned address
// below the row (a 16-byte unit that holds one valid byte lies in the same page, so the few bytes
// read before and after the row cannot fault), and every window is then read from LDS.  Rows too
// long for LDS take the direct kernel, one workgroup per (query row, head).
#include "common.h"
#include "infllmv2_hip.h"

namespace infllmv2 {

struct PoolParams {
    const uint16_t* in;
    uint16_t* out;
    const int* cu_seqlens_q;     // null for fixed length
    const int* cu_seqlens_k;
    const int* cache_lens;
    int64_t in_head_stride, in_row_stride;     // elements
    int batch, num_heads;
    int total_q, k_len, out_len;
    int cache_len;
    int kernel_size, stride, padding, block_size, local_blocks, init_blocks;
    bool is_bf16;
    bool vec4;                   // 5/4/1 window and 8-byte aligned rows
};

__device__ __forceinline__ float elem_to_f32(uint16_t v, bool is_bf16) {
    return is_bf16 ? bf16_to_f32(v) : f16_to_f32(v);
}

__global__ __launch_bounds__(256)
void max_pooling_1d_kernel(const PoolParams p) {
    const int q_global = blockIdx.x;
    const int h = blockIdx.y;
    int q_local = q_global, seqlen_k = p.k_len, cache_len = p.cache_len;
    if (p.cu_seqlens_q != nullptr) {
        // binary search for the sequence that owns this packed row (uniform per workgroup)
        int lo = 0, hi = p.batch;                       // invariant: cu[lo] <= q_global < cu[hi]
        while (hi - lo > 1) {
            const int mid = (lo + hi) >> 1;
            if (p.cu_seqlens_q[mid] <= q_global) lo = mid; else hi = mid;
        }
        q_local = q_global - p.cu_seqlens_q[lo];
        seqlen_k = p.cu_seqlens_k[lo + 1] - p.cu_seqlens_k[lo];
        seqlen_k = seqlen_k < p.k_len ? seqlen_k : p.k_len;
        cache_len = p.cache_lens[lo];
    }
    const uint16_t* in = p.in + static_cast<int64_t>(h) * p.in_head_stride + static_cast<int64_t>(q_global) * p.in_row_stride;
    uint16_t* out = p.out + (static_cast<int64_t>(h) * p.total_q + q_global) * p.out_len;
    const int bq = (q_local + cache_len) / p.block_size;
    const uint16_t pos_inf = p.is_bf16 ? 0x7f80 : 0x7c00;
    const uint16_t neg_inf = p.is_bf16 ? 0xff80 : 0xfc00;

    for (int kb = threadIdx.x; kb < p.out_len; kb += blockDim.x) {
        const bool forced = (kb < p.init_blocks) || (bq >= kb && bq <= kb + p.local_blocks);
        uint16_t best = neg_inf;
        if (forced) {
            best = pos_inf;
        } else {
            int start = kb * p.stride - p.padding;
            int end = start + p.kernel_size;
            start = start < 0 ? 0 : start;
            end = end < seqlen_k ? end : seqlen_k;
            if (end > start) {
                if (p.vec4 && kb > 0 && kb * 4 + 4 <= seqlen_k) {
                    const uint16_t first = in[kb * 4 - 1];
                    const uint64_t four = *reinterpret_cast<const uint64_t*>(in + kb * 4);
                    best = first;
                    float best_f = elem_to_f32(first, p.is_bf16);
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        const uint16_t v = static_cast<uint16_t>(four >> (16 * j));
                        const float f = elem_to_f32(v, p.is_bf16);
                        if (f > best_f) { best_f = f; best = v; }
                    }
                } else {
                    best = in[start];
                    float best_f = elem_to_f32(best, p.is_bf16);
                    for (int i = start + 1; i < end; ++i) {
                        const uint16_t v = in[i];
                        const float f = elem_to_f32(v, p.is_bf16);
                        if (f > best_f) { best_f = f; best = v; }
                    }
                }
            }
        }
        out[kb] = best;
    }
}

// One wavefront per row at a time, kWaves wavefronts per workgroup, each with an LDS slice of `units` 16-byte units.
template <int kWaves>
__global__ __launch_bounds__(kWaves * 64)
void max_pooling_1d_rows_kernel(const PoolParams p, int units, int rows_per_wave) {
    extern __shared__ uint4 pool_lds[];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    uint4* slice = pool_lds + wave * units;
    const uint16_t* elems = reinterpret_cast<const uint16_t*>(slice);
    const int64_t total_rows = static_cast<int64_t>(p.num_heads) * p.total_q;
    const uint16_t pos_inf = p.is_bf16 ? 0x7f80 : 0x7c00;
    const uint16_t neg_inf = p.is_bf16 ? 0xff80 : 0xfc00;
    const int64_t first_row = (static_cast<int64_t>(blockIdx.x) * kWaves + wave) * rows_per_wave;
    for (int r = 0; r < rows_per_wave; ++r) {
        const int64_t row = first_row + r;
        if (row >= total_rows) break;                           // uniform per wavefront; no workgroup barriers in this kernel
        const int h = static_cast<int>(row / p.total_q);
        const int q_global = static_cast<int>(row - static_cast<int64_t>(h) * p.total_q);
        int q_local = q_global, seqlen_k = p.k_len, cache_len = p.cache_len;
        if (p.cu_seqlens_q != nullptr) {
            int lo = 0, hi = p.batch;                           // invariant: cu[lo] <= q_global < cu[hi]
            while (hi - lo > 1) {
                const int mid = (lo + hi) >> 1;
                if (p.cu_seqlens_q[mid] <= q_global) lo = mid; else hi = mid;
            }
            q_local = q_global - p.cu_seqlens_q[lo];
            seqlen_k = p.cu_seqlens_k[lo + 1] - p.cu_seqlens_k[lo];
            seqlen_k = seqlen_k < p.k_len ? seqlen_k : p.k_len;
            cache_len = p.cache_lens[lo];
        }
        const uint16_t* in = p.in + static_cast<int64_t>(h) * p.in_head_stride + static_cast<int64_t>(q_global) * p.in_row_stride;
        const uintptr_t addr = reinterpret_cast<uintptr_t>(in);
        const uint4* aligned = reinterpret_cast<const uint4*>(addr & ~static_cast<uintptr_t>(15));
        const int shift = static_cast<int>(addr & 15) >> 1;     // the row starts at element `shift` of the slice
        const int n_units = seqlen_k > 0 ? ((shift + seqlen_k) * 2 + 15) >> 4 : 0;
        for (int u = lane; u < n_units; u += 64) slice[u] = aligned[u];
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
        uint16_t* out = p.out + (static_cast<int64_t>(h) * p.total_q + q_global) * p.out_len;
        const int bq = (q_local + cache_len) / p.block_size;
        for (int kb = lane; kb < p.out_len; kb += 64) {
            const bool forced = (kb < p.init_blocks) || (bq >= kb && bq <= kb + p.local_blocks);
            uint16_t best = neg_inf;
            if (forced) {
                best = pos_inf;
            } else {
                int start = kb * p.stride - p.padding;
                int end = start + p.kernel_size;
                start = start < 0 ? 0 : start;
                end = end < seqlen_k ? end : seqlen_k;
                if (end > start) {
                    best = elems[shift + start];
                    float best_f = elem_to_f32(best, p.is_bf16);
                    for (int i = start + 1; i < end; ++i) {
                        const uint16_t v = elems[shift + i];
                        const float f = elem_to_f32(v, p.is_bf16);
                        if (f > best_f) { best_f = f; best = v; }
                    }
                }
            }
            out[kb] = best;
        }
        // the slice is overwritten by the next row only after every lane has read this one
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
    }
}

static int launch_pool(void* stream, PoolParams& p) {
    IV2_CHECK(p.num_heads >= 0 && p.total_q >= 0 && p.k_len >= 0 && p.out_len >= 0, "max_pooling_1d: negative size");
    IV2_CHECK(p.block_size > 0 && p.stride > 0 && p.kernel_size > 0, "max_pooling_1d: block_size, stride and kernel_size must be positive");
    IV2_CHECK(p.num_heads <= 65535, "max_pooling_1d: num_heads %d exceeds 65535", p.num_heads);
    if (p.num_heads == 0 || p.total_q == 0 || p.out_len == 0) return 0;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const int units = (p.k_len * 2 + 14) / 16 + 2;              // a row plus the bytes before its first element
    const size_t slice_bytes = static_cast<size_t>(units) * 16;
    const int64_t total_rows = static_cast<int64_t>(p.num_heads) * p.total_q;
    if (slice_bytes <= 36 * 1024) {
        constexpr int kWaves = 4;
        const int rows_per_wave = total_rows >= 64 * 1024 ? 4 : 1;
        const int64_t blocks = (total_rows + kWaves * rows_per_wave - 1) / (kWaves * rows_per_wave);
        IV2_CHECK(blocks <= 0x7fffffffll, "max_pooling_1d: too many rows");
        hipLaunchKernelGGL(max_pooling_1d_rows_kernel<kWaves>, dim3(static_cast<unsigned>(blocks)), dim3(kWaves * 64),
                           kWaves * slice_bytes, st, p, units, rows_per_wave);
        IV2_LAUNCH_CHECK();
        return 0;
    }
    p.vec4 = p.kernel_size == 5 && p.stride == 4 && p.padding == 1 &&
             (p.in_row_stride % 4 == 0) && (p.in_head_stride % 4 == 0) &&
             (reinterpret_cast<uintptr_t>(p.in) % 8 == 0);
    const int threads = p.out_len >= 256 ? 256 : (p.out_len > 64 ? 128 : 64);
    hipLaunchKernelGGL(max_pooling_1d_kernel, dim3(p.total_q, p.num_heads), dim3(threads), 0, st, p);
    IV2_LAUNCH_CHECK();
    return 0;
}

}  // namespace infllmv2

using namespace infllmv2;

extern "C" int infllmv2_max_pooling_1d_strided(void* stream, const void* input, void* output, int dtype,
                                               int num_heads, int q_len, int k_len, int64_t in_head_stride,
                                               int64_t in_row_stride, int out_len, int cache_len, int kernel_size,
                                               int stride, int padding, int block_size, int local_blocks,
                                               int init_blocks) {
    IV2_CHECK(dtype == 0 || dtype == 1, "max_pooling_1d: dtype must be 0 (fp16) or 1 (bf16)");
    IV2_CHECK(in_row_stride >= k_len, "max_pooling_1d: row stride %lld shorter than k_len %d", (long long)in_row_stride, k_len);
    PoolParams p{};
    p.in = static_cast<const uint16_t*>(input);
    p.out = static_cast<uint16_t*>(output);
    p.in_head_stride = in_head_stride;
    p.in_row_stride = in_row_stride;
    p.batch = 1; p.num_heads = num_heads; p.total_q = q_len; p.k_len = k_len; p.out_len = out_len;
    p.cache_len = cache_len; p.kernel_size = kernel_size; p.stride = stride; p.padding = padding;
    p.block_size = block_size; p.local_blocks = local_blocks; p.init_blocks = init_blocks;
    p.is_bf16 = dtype == 1;
    return launch_pool(stream, p);
}

extern "C" int infllmv2_max_pooling_1d(void* stream, const void* input, void* output, int dtype, int num_heads,
                                       int q_len, int k_len, int out_len, int cache_len, int kernel_size,
                                       int stride, int padding, int block_size, int local_blocks, int init_blocks) {
    return infllmv2_max_pooling_1d_strided(stream, input, output, dtype, num_heads, q_len, k_len,
                                           static_cast<int64_t>(q_len) * k_len, k_len, out_len, cache_len,
                                           kernel_size, stride, padding, block_size, local_blocks, init_blocks);
}

extern "C" int infllmv2_max_pooling_1d_varlen_strided(void* stream, const void* input, void* output,
                                                      const int* cu_seqlens_q, const int* cu_seqlens_k,
                                                      const int* cache_lens, int dtype, int batch_size,
                                                      int num_heads, int total_q, int max_seqlen_q, int max_seqlen_k,
                                                      int64_t in_head_stride, int64_t in_row_stride, int out_len,
                                                      int kernel_size, int stride, int padding, int block_size,
                                                      int local_blocks, int init_blocks) {
    IV2_CHECK(dtype == 0 || dtype == 1, "max_pooling_1d_varlen: dtype must be 0 (fp16) or 1 (bf16)");
    IV2_CHECK(batch_size >= 1, "max_pooling_1d_varlen: batch_size must be at least 1");
    IV2_CHECK(cu_seqlens_q && cu_seqlens_k && cache_lens, "max_pooling_1d_varlen: null sequence-length pointer");
    IV2_CHECK(in_row_stride >= max_seqlen_k, "max_pooling_1d_varlen: row stride shorter than max_seqlen_k");
    (void)max_seqlen_q;
    PoolParams p{};
    p.in = static_cast<const uint16_t*>(input);
    p.out = static_cast<uint16_t*>(output);
    p.cu_seqlens_q = cu_seqlens_q; p.cu_seqlens_k = cu_seqlens_k; p.cache_lens = cache_lens;
    p.in_head_stride = in_head_stride;
    p.in_row_stride = in_row_stride;
    p.batch = batch_size; p.num_heads = num_heads; p.total_q = total_q; p.k_len = max_seqlen_k; p.out_len = out_len;
    p.cache_len = 0; p.kernel_size = kernel_size; p.stride = stride; p.padding = padding;
    p.block_size = block_size; p.local_blocks = local_blocks; p.init_blocks = init_blocks;
    p.is_bf16 = dtype == 1;
    return launch_pool(stream, p);
}

extern "C" int infllmv2_max_pooling_1d_varlen(void* stream, const void* input, void* output,
                                              const int* cu_seqlens_q, const int* cu_seqlens_k,
                                              const int* cache_lens, int dtype, int batch_size, int num_heads,
                                              int max_seqlen_q, int max_seqlen_k, int out_len, int kernel_size,
                                              int stride, int padding, int block_size, int local_blocks,
                                              int init_blocks) {
    IV2_CHECK(batch_size >= 1 && cu_seqlens_q, "max_pooling_1d_varlen: bad batch or null cu_seqlens_q");
    int total_q = 0;                    // same host read-back as csrc/max_pooling_1d.cuh:187-190
    hipStream_t st = static_cast<hipStream_t>(stream);
    hipError_t e = hipMemcpyAsync(&total_q, cu_seqlens_q + batch_size, sizeof(int), hipMemcpyDeviceToHost, st);
    if (e == hipSuccess) e = hipStreamSynchronize(st);
    IV2_CHECK(e == hipSuccess, "max_pooling_1d_varlen: reading total_q failed: %s", hipGetErrorString(e));
    return infllmv2_max_pooling_1d_varlen_strided(stream, input, output, cu_seqlens_q, cu_seqlens_k, cache_lens,
                                                  dtype, batch_size, num_heads, total_q, max_seqlen_q, max_seqlen_k,
                                                  static_cast<int64_t>(total_q) * max_seqlen_k, max_seqlen_k, out_len,
                                                  kernel_size, stride, padding, block_size, local_blocks, init_blocks);
}
