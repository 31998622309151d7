// Compressed keys for Stage 1 (gfx950): row j of a sequence is the mean of its K rows
// [stride*j, stride*j + kernel_size), full windows only.
//
// The reference leaves this step to its callers; the rule is the one its tests use to build the
// Stage-1 inputs (compress_tensor / calc_chunks_with_stride, tests/test_stage1_compressed_lse.py:16-99:
// windows that fit entirely inside a sequence, mean over the window, result in the input dtype).
// The mean is an fp32 sum taken in window order divided by kernel_size, rounded once to bf16.
//
// HBM-bound and small: K is read once from memory (the overlapping windows hit in cache) and
// the output is 1/stride of its size.  A thread owns 8 contiguous d values (16 bytes) of one output row.
#include "common.h"
#include "infllmv2_hip.h"

namespace IV2_NS {

__device__ __forceinline__ int compressed_rows(int len, int kernel_size, int stride) {
    return len >= kernel_size ? (len - kernel_size) / stride + 1 : 0;
}

// cu_out[b] = rows of the sequences before b; one thread (batch is small)
__global__ void compressed_cu_seqlens_kernel(const int* __restrict__ cu_k, int* __restrict__ cu_out, int batch,
                                             int kernel_size, int stride) {
    if (blockIdx.x != 0 || threadIdx.x != 0) return;
    int acc = 0;
    cu_out[0] = 0;
    for (int b = 0; b < batch; ++b) {
        acc += compressed_rows(cu_k[b + 1] - cu_k[b], kernel_size, stride);
        cu_out[b + 1] = acc;
    }
}

struct CompressParams {
    const elem_bits* k;
    elem_bits* out;
    const int* cu_k;
    const int* cu_out;
    int64_t k_row_stride, k_head_stride;
    int units_per_row;               // num_heads * head_dim / 8
    int units_per_head;              // head_dim / 8
    int kernel_size, stride;
    int first_row;                   // rows before this one are left alone (appending to a cache of compressed keys)
};

constexpr int kCompressRowsPerWg = 8;

__global__ __launch_bounds__(256)
void compress_keys_kernel(const CompressParams p) {
    const int b = blockIdx.y;
    const int k0 = p.cu_k[b];
    const int rows = compressed_rows(p.cu_k[b + 1] - k0, p.kernel_size, p.stride);
    const int j0 = p.first_row + blockIdx.x * kCompressRowsPerWg;
    for (int item = threadIdx.x; item < kCompressRowsPerWg * p.units_per_row; item += 256) {
        const int j = j0 + item / p.units_per_row;
        if (j >= rows) break;                                  // items are ordered by row
        const int u = item % p.units_per_row;
        const int head = u / p.units_per_head, piece = u % p.units_per_head;
        const elem_bits* src = p.k + (static_cast<int64_t>(k0) + static_cast<int64_t>(j) * p.stride) * p.k_row_stride +
                               head * p.k_head_stride + piece * 8;
        float acc[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[e] = 0.f;
        for (int i = 0; i < p.kernel_size; ++i) {
            const uint4 raw = *reinterpret_cast<const uint4*>(src + i * p.k_row_stride);
            const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                acc[2 * e] += elem_lo_to_f32(w[e]);
                acc[2 * e + 1] += elem_hi_to_f32(w[e]);
            }
        }
        const float n = static_cast<float>(p.kernel_size);
        uint4 o;
        o.x = pack_elem2(acc[0] / n, acc[1] / n);
        o.y = pack_elem2(acc[2] / n, acc[3] / n);
        o.z = pack_elem2(acc[4] / n, acc[5] / n);
        o.w = pack_elem2(acc[6] / n, acc[7] / n);
        *reinterpret_cast<uint4*>(p.out + (static_cast<int64_t>(p.cu_out[b]) + j) * p.units_per_row * 8 + u * 8) = o;
    }
}

// The same means for per-sequence key caches (decode): sequence b's keys are rows [0, new_lens[b]) of kcache[b]; the
// rows of its compressed-key cache that windows completed since old_lens[b] tokens are written, the others are left
// alone.  A decode step (one more token) completes at most one window per set.
struct CompressCacheParams {
    const elem_bits* k;
    elem_bits* out;
    const int* old_lens;             // null: 0 for every sequence (build everything)
    const int* new_lens;
    int* out_lens;                   // null, or (batch): rows the compressed cache holds afterwards
    int64_t k_batch, k_row, k_head, o_batch, o_row, o_head;
    int units_per_row, units_per_head;
    int kernel_size, stride;
    int k_capacity;                  // rows of one sequence's key cache: a length beyond it is read as the capacity
    int out_capacity;                // rows of one sequence's compressed cache: nothing is written beyond it
    int max_new_rows;                // rows this call may add per sequence (what the launch covers)
};

// Rows sequence b's compressed cache holds after the call, and the first of them this call writes: the windows
// completed by new_lens[b] tokens, never more than the output has rows, the key cache has windows, or the launch
// covers (so that the reported length never includes a row that was not written).
__device__ __forceinline__ void cache_row_range(const CompressCacheParams& p, int b, int& first, int& rows) {
    int new_len = p.new_lens[b];
    if (new_len > p.k_capacity) new_len = p.k_capacity;
    rows = compressed_rows(new_len, p.kernel_size, p.stride);
    first = p.old_lens ? compressed_rows(p.old_lens[b], p.kernel_size, p.stride) : 0;
    if (first < 0) first = 0;
    if (rows > p.out_capacity) rows = p.out_capacity;
    if (rows > first + p.max_new_rows) rows = first + p.max_new_rows;
}

__global__ __launch_bounds__(256)
void compress_keys_cache_kernel(const CompressCacheParams p) {
    const int b = blockIdx.y;
    int first, rows;
    cache_row_range(p, b, first, rows);
    if (blockIdx.x == 0 && threadIdx.x == 0 && p.out_lens) p.out_lens[b] = rows;
    const int j0 = first + blockIdx.x * kCompressRowsPerWg;
    for (int item = threadIdx.x; item < kCompressRowsPerWg * p.units_per_row; item += 256) {
        const int j = j0 + item / p.units_per_row;
        if (j >= rows) break;
        const int u = item % p.units_per_row;
        const int head = u / p.units_per_head, piece = u % p.units_per_head;
        const elem_bits* src = p.k + b * p.k_batch + static_cast<int64_t>(j) * p.stride * p.k_row + head * p.k_head + piece * 8;
        float acc[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[e] = 0.f;
        for (int i = 0; i < p.kernel_size; ++i) {
            const uint4 raw = *reinterpret_cast<const uint4*>(src + i * p.k_row);
            const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                acc[2 * e] += elem_lo_to_f32(w[e]);
                acc[2 * e + 1] += elem_hi_to_f32(w[e]);
            }
        }
        const float n = static_cast<float>(p.kernel_size);
        uint4 o;
        o.x = pack_elem2(acc[0] / n, acc[1] / n);
        o.y = pack_elem2(acc[2] / n, acc[3] / n);
        o.z = pack_elem2(acc[4] / n, acc[5] / n);
        o.w = pack_elem2(acc[6] / n, acc[7] / n);
        *reinterpret_cast<uint4*>(p.out + b * p.o_batch + static_cast<int64_t>(j) * p.o_row + head * p.o_head + piece * 8) = o;
    }
}

// The append of a decode step: few new rows per sequence, so one workgroup takes ONE output row (32 of its 16-byte
// units).  Walking the window row by row in one thread, as the kernel above does, is a chain of kernel_size dependent
// round trips to memory when only a handful of threads are busy; here the whole window goes into LDS with every
// load in flight at once, and then one thread per output element adds its column in window order (the same fp32
// additions in the same order as above: the results are the same bits).
constexpr int kAppendUnits = 32;
constexpr int kAppendMaxLds = 65536;

// new_row: which of the sequence's new rows this workgroup takes
__device__ __forceinline__ void append_one_row(const CompressCacheParams& p, int new_row, uint4* window) {
    const int b = blockIdx.y;
    int first, rows;
    cache_row_range(p, b, first, rows);
    if (new_row == 0 && blockIdx.z == 0 && threadIdx.x == 0 && p.out_lens) p.out_lens[b] = rows;
    const int j = first + new_row;
    if (j >= rows) return;                                     // uniform per workgroup
    const int u0 = blockIdx.z * kAppendUnits;
    const int nu = p.units_per_row - u0 < kAppendUnits ? p.units_per_row - u0 : kAppendUnits;
    const elem_bits* src = p.k + b * p.k_batch + static_cast<int64_t>(j) * p.stride * p.k_row;
    const int items = p.kernel_size * kAppendUnits;
#pragma unroll 8
    for (int it = threadIdx.x; it < items; it += 256) {
        const int i = it / kAppendUnits, uu = it % kAppendUnits;
        if (uu < nu) {
            const int u = u0 + uu;
            window[it] = *reinterpret_cast<const uint4*>(src + i * p.k_row + (u / p.units_per_head) * p.k_head + (u % p.units_per_head) * 8);
        }
    }
    __syncthreads();
    const int uu = threadIdx.x >> 3, e = threadIdx.x & 7;      // one thread per (unit, element)
    if (uu >= nu) return;
    const elem_bits* col = reinterpret_cast<const elem_bits*>(window) + uu * 8 + e;
    float acc = 0.f;
    for (int i = 0; i < p.kernel_size; ++i) acc += elem_to_f32(col[i * kAppendUnits * 8]);
    const float n = static_cast<float>(p.kernel_size);
    const int u = u0 + uu;
    p.out[b * p.o_batch + static_cast<int64_t>(j) * p.o_row + (u / p.units_per_head) * p.o_head + (u % p.units_per_head) * 8 + e] =
        f32_to_elem(acc / n);
}

__global__ __launch_bounds__(256)
void compress_keys_cache_append_kernel(const CompressCacheParams p) {
    extern __shared__ uint4 window[];                          // [kernel_size][kAppendUnits]
    append_one_row(p, blockIdx.x, window);
}
// the appends to two compressed caches of the same key cache (the fine and the coarse keys of a decode step) in one
// launch: the first rows_a workgroups of a sequence belong to cache a
__global__ __launch_bounds__(256)
void compress_keys_cache_append_pair_kernel(const CompressCacheParams pa, const CompressCacheParams pb, int rows_a) {
    extern __shared__ uint4 window[];                          // [the larger kernel_size][kAppendUnits]
    if (static_cast<int>(blockIdx.x) < rows_a) append_one_row(pa, blockIdx.x, window);
    else append_one_row(pb, blockIdx.x - rows_a, window);
}

}  // namespace IV2_NS

using namespace IV2_NS;

extern "C" int IV2_ENTRY(infllmv2_compress_keys)(void* stream, const void* k, void* out, const int32_t* cu_seqlens_k,
                                      int32_t* cu_seqlens_out, int batch, int max_seqlen_k, int num_heads_k,
                                      int head_dim, int64_t k_row_stride, int64_t k_head_stride, int kernel_size,
                                      int stride, int first_row) {
    IV2_CHECK(batch > 0 && batch <= 65535 && max_seqlen_k >= 0, "compress_keys: bad batch or max_seqlen_k");
    IV2_CHECK(kernel_size > 0 && stride > 0 && first_row >= 0, "compress_keys: kernel_size and stride must be positive");
    IV2_CHECK(k && out && cu_seqlens_k && cu_seqlens_out, "compress_keys: null pointer");
    IV2_CHECK(head_dim > 0 && head_dim % 8 == 0 && num_heads_k > 0, "compress_keys: head_dim must be a multiple of 8");
    const int units = num_heads_k * head_dim / 8;
    IV2_CHECK(reinterpret_cast<uintptr_t>(k) % 16 == 0 && reinterpret_cast<uintptr_t>(out) % 16 == 0 &&
              k_row_stride % 8 == 0 && k_head_stride % 8 == 0, "compress_keys: k and out must be 16-byte aligned, strides multiples of 8");
    hipStream_t st = static_cast<hipStream_t>(stream);
    hipLaunchKernelGGL(compressed_cu_seqlens_kernel, dim3(1), dim3(64), 0, st, cu_seqlens_k, cu_seqlens_out, batch,
                       kernel_size, stride);
    IV2_LAUNCH_CHECK();
    const int max_rows = max_seqlen_k >= kernel_size ? (max_seqlen_k - kernel_size) / stride + 1 : 0;
    if (max_rows <= first_row) return 0;
    CompressParams p{};
    p.k = static_cast<const elem_bits*>(k);
    p.out = static_cast<elem_bits*>(out);
    p.cu_k = cu_seqlens_k; p.cu_out = cu_seqlens_out;
    p.k_row_stride = k_row_stride; p.k_head_stride = k_head_stride;
    p.units_per_row = units; p.units_per_head = head_dim / 8;
    p.kernel_size = kernel_size; p.stride = stride; p.first_row = first_row;
    const dim3 grid((max_rows - first_row + kCompressRowsPerWg - 1) / kCompressRowsPerWg, batch);
    hipLaunchKernelGGL(compress_keys_kernel, grid, dim3(256), 0, st, p);
    IV2_LAUNCH_CHECK();
    return 0;
}

namespace {

// checks and parameters of one compressed cache; 0 or an error code
int cache_params(const char* who, CompressCacheParams& p, const void* kcache, void* out_cache, const int32_t* old_lens,
                 const int32_t* new_lens, int32_t* out_lens, int batch, int max_new_rows, int num_heads_k, int head_dim,
                 const int64_t* kcache_strides, const int64_t* out_strides, int kernel_size, int stride, int kcache_rows,
                 int out_rows) {
    IV2_CHECK(batch > 0 && batch <= 65535 && max_new_rows >= 0, "%s: bad batch or max_new_rows", who);
    IV2_CHECK(kcache_rows >= 0 && out_rows >= 0, "%s: negative cache capacity", who);
    IV2_CHECK(kernel_size > 0 && stride > 0, "%s: kernel_size and stride must be positive", who);
    IV2_CHECK(kcache && out_cache && new_lens, "%s: null pointer", who);
    IV2_CHECK(head_dim > 0 && head_dim % 8 == 0 && num_heads_k > 0, "%s: head_dim must be a multiple of 8", who);
    IV2_CHECK(reinterpret_cast<uintptr_t>(kcache) % 16 == 0 && reinterpret_cast<uintptr_t>(out_cache) % 16 == 0,
              "%s: caches must be 16-byte aligned", who);
    for (int s = 0; s < 3; ++s)
        IV2_CHECK(kcache_strides[s] % 8 == 0 && out_strides[s] % 8 == 0, "%s: strides must be multiples of 8 elements", who);
    p = CompressCacheParams{};
    p.k = static_cast<const elem_bits*>(kcache);
    p.out = static_cast<elem_bits*>(out_cache);
    p.old_lens = old_lens; p.new_lens = new_lens; p.out_lens = out_lens;
    p.k_batch = kcache_strides[0]; p.k_row = kcache_strides[1]; p.k_head = kcache_strides[2];
    p.o_batch = out_strides[0]; p.o_row = out_strides[1]; p.o_head = out_strides[2];
    p.units_per_row = num_heads_k * head_dim / 8; p.units_per_head = head_dim / 8;
    p.kernel_size = kernel_size; p.stride = stride;
    p.k_capacity = kcache_rows; p.out_capacity = out_rows; p.max_new_rows = max_new_rows;
    return 0;
}
size_t append_window_bytes(const CompressCacheParams& p) { return static_cast<size_t>(p.kernel_size) * kAppendUnits * 16; }
// a decode step's append: one workgroup per new row and 32 units
bool append_shaped(const CompressCacheParams& p) {
    return p.max_new_rows >= 1 && p.max_new_rows <= 8 && append_window_bytes(p) <= kAppendMaxLds;
}
int launch_cache(hipStream_t st, const CompressCacheParams& p, int batch) {
    if (append_shaped(p)) {
        const dim3 grid(p.max_new_rows, batch, (p.units_per_row + kAppendUnits - 1) / kAppendUnits);
        hipLaunchKernelGGL(compress_keys_cache_append_kernel, grid, dim3(256), append_window_bytes(p), st, p);
        IV2_LAUNCH_CHECK();
        return 0;
    }
    // at least one workgroup per sequence so that out_lens is always written
    const int groups = p.max_new_rows > 0 ? (p.max_new_rows + kCompressRowsPerWg - 1) / kCompressRowsPerWg : 1;
    hipLaunchKernelGGL(compress_keys_cache_kernel, dim3(groups, batch), dim3(256), 0, st, p);
    IV2_LAUNCH_CHECK();
    return 0;
}

}  // namespace

extern "C" int IV2_ENTRY(infllmv2_compress_keys_cache)(void* stream, const void* kcache, void* out_cache, const int32_t* old_lens,
                                            const int32_t* new_lens, int32_t* out_lens, int batch, int max_new_rows,
                                            int num_heads_k, int head_dim, const int64_t* kcache_strides,
                                            const int64_t* out_strides, int kernel_size, int stride,
                                            int kcache_rows, int out_rows) {
    CompressCacheParams p;
    if (int rc = cache_params("compress_keys_cache", p, kcache, out_cache, old_lens, new_lens, out_lens, batch, max_new_rows,
                              num_heads_k, head_dim, kcache_strides, out_strides, kernel_size, stride, kcache_rows, out_rows))
        return rc;
    return launch_cache(static_cast<hipStream_t>(stream), p, batch);
}

extern "C" int IV2_ENTRY(infllmv2_compress_keys_cache_pair)(void* stream, const void* kcache, void* out_cache_a, void* out_cache_b,
                                                 const int32_t* old_lens, const int32_t* new_lens, int32_t* out_lens_a,
                                                 int32_t* out_lens_b, int batch, int max_new_rows_a, int max_new_rows_b,
                                                 int num_heads_k, int head_dim, const int64_t* kcache_strides,
                                                 const int64_t* out_strides_a, const int64_t* out_strides_b,
                                                 int kernel_size_a, int stride_a, int kernel_size_b, int stride_b,
                                                 int kcache_rows, int out_rows_a, int out_rows_b) {
    CompressCacheParams pa, pb;
    if (int rc = cache_params("compress_keys_cache_pair", pa, kcache, out_cache_a, old_lens, new_lens, out_lens_a, batch,
                              max_new_rows_a, num_heads_k, head_dim, kcache_strides, out_strides_a, kernel_size_a, stride_a,
                              kcache_rows, out_rows_a))
        return rc;
    if (int rc = cache_params("compress_keys_cache_pair", pb, kcache, out_cache_b, old_lens, new_lens, out_lens_b, batch,
                              max_new_rows_b, num_heads_k, head_dim, kcache_strides, out_strides_b, kernel_size_b, stride_b,
                              kcache_rows, out_rows_b))
        return rc;
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (append_shaped(pa) && append_shaped(pb)) {
        const size_t lds = append_window_bytes(pa) > append_window_bytes(pb) ? append_window_bytes(pa) : append_window_bytes(pb);
        const dim3 grid(pa.max_new_rows + pb.max_new_rows, batch, (pa.units_per_row + kAppendUnits - 1) / kAppendUnits);
        hipLaunchKernelGGL(compress_keys_cache_append_pair_kernel, grid, dim3(256), lds, st, pa, pb, pa.max_new_rows);
        IV2_LAUNCH_CHECK();
        return 0;
    }
    if (int rc = launch_cache(st, pa, batch)) return rc;
    return launch_cache(st, pb, batch);
}
