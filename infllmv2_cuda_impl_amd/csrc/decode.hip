// Stage-2 decode against a KV cache for gfx950: one query token per sequence, attention restricted
// to the 64-key blocks set in the sequence's mask row, optional in-place append of new keys/values.
//
// Semantics follow mha_fwd_kvcache (csrc/flash_attn/flash_api.cpp:1549-1843) on the path the
// Python wrapper takes (infllm_v2/infllmv2_sparse_attention.py:730-757): seqlen_q == 1, so the
// causal flag is dropped (flash_api.cpp:1628); the 16 grouped heads of a KV head form the row tile
// (flash_api.cpp:1633-1639); keys [0, cache_seqlens[b] + seqlen_new) are visible; new k/v are
// written at cache_seqlens[b] first (flash_fwd_kernel.h:792-891); the result must not depend on
// the number of KV splits (combine by LSE, flash_fwd_kernel.h:1866-1946).
//
// Design: decode is HBM-bound (each selected block is 32 KiB of K+V read exactly once, ~2 MiB per
// sequence and KV head), so the kernel reads the cache in the caller's layout, with no repacking
// pass.  One single-wavefront workgroup handles one (sequence, KV head, split); a split is a
// contiguous run of the row's selected blocks (by ordinal, so splits are balanced whatever the
// mask looks like).  K rows are the MFMA A operand as they lie in memory (contraction over d);
// V is contracted over keys, so its tile takes one trip through a wavefront-private LDS buffer and
// is read back transposed.  Partial results are merged by a small combine kernel.
#include "common.h"
#include "block_walker.h"
#include "infllmv2_hip.h"
#include <math.h>
#include <mutex>

namespace IV2_NS {

struct DecodeParams {
    const elem_bits* q;
    elem_bits* kcache;
    elem_bits* vcache;
    const elem_bits* knew;
    const elem_bits* vnew;
    elem_bits* out;
    float* lse;                     // (batch, Hq)
    float* o_part;                  // (batch, Hk, splits, 16, 128) fp32, normalised per split
    float* lse_part;                // (batch, Hk, splits, 16)
    const int* cache_seqlens;       // null: every sequence fills the whole cache
    const uint64_t* mask;           // (batch, Hk, n64) or null
    int64_t q_batch, q_head;        // element strides of q (batch, head); head dim dense
    int64_t o_batch, o_head;
    int64_t kc_batch, kc_row, kc_head, vc_batch, vc_row, vc_head;
    int64_t kn_batch, kn_row, kn_head, vn_batch, vn_row, vn_head;
    int batch, num_heads_k, capacity, seqlen_new, n64, splits;
    int group;                      // query heads per KV head, 1..16
    float scale_log2;
    // where a sequence's rows lie (flash_api.cpp:1593-1611, 1762-1771, 1800-1808)
    const int* cache_batch_idx;     // sequence b uses cache row cache_batch_idx[b]; null: b
    const int* leftpad;             // the sequence's keys start at cache row leftpad[b]; null: 0
    const int* block_table;         // (batch, pages per sequence): the caches are (pages, page_size, Hk, d)
    int64_t bt_batch;
    int page_size;
    // rotary embedding of the appended keys and of the query (flash_fwd_kernel.h:787-929, rotary.h)
    const elem_bits* rot_cos;       // (seqlen_ro, rotary_dim / 2)
    const elem_bits* rot_sin;
    int rotary_dim, rotary_interleaved;
    elem_bits* q_rot;               // (batch, Hq, 128): the turned query, in the workspace
};

// element offset of cache row `row` of sequence b (head 0)
__device__ __forceinline__ int64_t cache_row_offset(const DecodeParams& p, int b, int row, int64_t batch_stride,
                                                    int64_t row_stride) {
    if (p.block_table) {
        const int page = p.block_table[b * p.bt_batch + row / p.page_size];
        return page * batch_stride + static_cast<int64_t>(row % p.page_size) * row_stride;
    }
    const int cb = p.cache_batch_idx ? p.cache_batch_idx[b] : b;
    return cb * batch_stride + static_cast<int64_t>(row) * row_stride;
}

// One 16-byte chunk (8 values, d = 8 chunk ...) of a head vector turned at position pos.  Interleaved: pairs
// (2i, 2i+1) lie inside the chunk; contiguous: the partner of d is d +- rotary_dim / 2, in another chunk of the
// same head vector.  (a, b) -> (a cos - b sin, a sin + b cos) in fp32, one rounding (rotary.h:57-62, 131-133).
__device__ __forceinline__ uint4 rotary_chunk(const DecodeParams& p, const elem_bits* head_vec, int chunk, int pos) {
    const uint4 raw = *reinterpret_cast<const uint4*>(head_vec + chunk * 8);
    const int d0 = chunk * 8, half = p.rotary_dim >> 1;
    if (d0 >= p.rotary_dim) return raw;
    const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
    float x[8], y[8];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        x[2 * e] = elem_lo_to_f32(w[e]);
        x[2 * e + 1] = elem_hi_to_f32(w[e]);
    }
    const elem_bits* cs = p.rot_cos + static_cast<int64_t>(pos) * half;
    const elem_bits* sn = p.rot_sin + static_cast<int64_t>(pos) * half;
    if (p.rotary_interleaved) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const float c = elem_to_f32(cs[(d0 >> 1) + i]), s = elem_to_f32(sn[(d0 >> 1) + i]);
            y[2 * i] = x[2 * i] * c - x[2 * i + 1] * s;
            y[2 * i + 1] = x[2 * i] * s + x[2 * i + 1] * c;
        }
    } else {
        const bool left = d0 < half;
        const uint4 oraw = *reinterpret_cast<const uint4*>(head_vec + (left ? d0 + half : d0 - half));
        const uint32_t ow[4] = {oraw.x, oraw.y, oraw.z, oraw.w};
        const int i0 = left ? d0 : d0 - half;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const float o = (e & 1) ? elem_hi_to_f32(ow[e >> 1]) : elem_lo_to_f32(ow[e >> 1]);
            const float c = elem_to_f32(cs[i0 + e]), s = elem_to_f32(sn[i0 + e]);
            y[e] = left ? x[e] * c - o * s : x[e] * c + o * s;
        }
    }
    return make_uint4(pack_elem2(y[0], y[1]), pack_elem2(y[2], y[3]), pack_elem2(y[4], y[5]), pack_elem2(y[6], y[7]));
}

constexpr int kVtPitch = kHeadDim + 16;                        // LDS row pitch (elements) of the V tile: rows 8 banks apart, so the
                                                               // transposing reads of four rows at a time do not collide

__global__ __launch_bounds__(256)
void decode_append_kernel(const DecodeParams p) {
    // one thread moves 16 bytes of one new row of K and of V
    const int64_t idx = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    const int64_t total = static_cast<int64_t>(p.batch) * p.seqlen_new * p.num_heads_k * 16;
    if (idx >= total) return;
    const int chunk = static_cast<int>(idx & 15);
    int64_t r = idx >> 4;
    const int h = static_cast<int>(r % p.num_heads_k); r /= p.num_heads_k;
    const int t = static_cast<int>(r % p.seqlen_new);
    const int b = static_cast<int>(r / p.seqlen_new);
    const int pos = (p.cache_seqlens ? p.cache_seqlens[b] : 0) + t;             // cache row, left padding included
    if (pos >= p.capacity) return;
    const elem_bits* kvec = p.knew + b * p.kn_batch + t * p.kn_row + h * p.kn_head;
    const uint4 kv = p.rotary_dim > 0 ? rotary_chunk(p, kvec, chunk, pos) : *reinterpret_cast<const uint4*>(kvec + chunk * 8);
    const uint4 vv = *reinterpret_cast<const uint4*>(p.vnew + b * p.vn_batch + t * p.vn_row + h * p.vn_head + chunk * 8);
    *reinterpret_cast<uint4*>(p.kcache + cache_row_offset(p, b, pos, p.kc_batch, p.kc_row) + h * p.kc_head + chunk * 8) = kv;
    *reinterpret_cast<uint4*>(p.vcache + cache_row_offset(p, b, pos, p.vc_batch, p.vc_row) + h * p.vc_head + chunk * 8) = vv;
}

// the query turned at the position of the first appended key (all 16 grouped heads of the single query token take
// the same position: the non-causal rule of flash_fwd_kernel.h:899-901)
__global__ __launch_bounds__(256)
void decode_rotate_q_kernel(const DecodeParams p) {
    const int64_t idx = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    const int heads = p.num_heads_k * p.group;
    if (idx >= static_cast<int64_t>(p.batch) * heads * 16) return;
    const int chunk = static_cast<int>(idx & 15);
    const int head = static_cast<int>((idx >> 4) % heads), b = static_cast<int>((idx >> 4) / heads);
    const int pos = p.cache_seqlens ? p.cache_seqlens[b] : 0;
    *reinterpret_cast<uint4*>(p.q_rot + (static_cast<int64_t>(b) * heads + head) * kHeadDim + chunk * 8) =
        rotary_chunk(p, p.q + b * p.q_batch + head * p.q_head, chunk, pos);
}

typedef short short4d __attribute__((ext_vector_type(4)));
// 16 lanes x 4 halfwords, transposed (ds_read_b64_tr_b16): lane 16 g + r receives element r % 4 of the four-halfword
// rows offered by lanes 16 g + r / 4 + {0, 4, 8, 12}
__device__ __forceinline__ short4d lds_read_tr(const elem_bits* ptr) {
    return __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) short4d*)(ptr));
}

template <bool kDirect>
__global__ __launch_bounds__(64)
void decode_split_kernel(const DecodeParams p) {
    __shared__ __attribute__((aligned(16))) elem_bits vt[kBlockN * kVtPitch];
    const int lane = threadIdx.x;
    const int n = lane & 15, g = lane >> 4;
    const int split = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
    const int lp = p.leftpad ? p.leftpad[b] : 0;              // the sequence's key 0 is cache row lp
    int L = (p.cache_seqlens ? p.cache_seqlens[b] : p.capacity - p.seqlen_new) + p.seqlen_new;
    if (L > p.capacity) L = p.capacity;
    L -= lp;                                                   // keys of the sequence; mask block j = keys 64 j ..
    const int last_blk = L <= 0 ? -1 : ((L - 1) >> 6);
    const uint64_t* row = p.mask ? p.mask + (static_cast<int64_t>(b) * p.num_heads_k + h) * p.n64 : nullptr;
    BlockWalker walk;
    walk.init(row, p.n64, last_blk);

    // how many blocks does the row select, and which run of them is this split's
    int total = 0;
    for (int w = lane; w < walk.n_words; w += 64) {
        uint64_t v = row ? row[w] : ~0ull;
        if (w == (last_blk >> 6)) {
            const int t = last_blk & 63;
            v &= (t == 63) ? ~0ull : ((1ull << (t + 1)) - 1ull);
        }
        total += __builtin_popcountll(v);
    }
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) total += __shfl_xor(total, off);
    total = __builtin_amdgcn_readfirstlane(total);
    const int per = (total + p.splits - 1) / p.splits;
    const int begin = split * per;
    int count = total - begin;
    if (count > per) count = per;

    elem8 qf[4];
    {
        const int qh = p.group * h + (n < p.group ? n : p.group - 1);      // rows beyond the group repeat its last head
        const elem_bits* qp = p.rotary_dim > 0
            ? p.q_rot + (static_cast<int64_t>(b) * p.num_heads_k * p.group + qh) * kHeadDim + 8 * g
            : p.q + b * p.q_batch + qh * p.q_head + 8 * g;
#pragma unroll
        for (int c = 0; c < 4; ++c) qf[c] = *reinterpret_cast<const elem8*>(qp + 32 * c);
    }
    float m = -INFINITY, l = 0.f;
    floatx4 o[8];
#pragma unroll
    for (int dt = 0; dt < 8; ++dt) o[dt] = floatx4{0.f, 0.f, 0.f, 0.f};

    int j = -1;
    for (int skip = 0; skip <= begin && count > 0; ++skip) j = walk.next();   // ordinal `begin` of the row
    // K rows as A operands and the V rows of block jb, requested together; rows past the end are clamped to a valid row
    // (K is masked below, P is zero there).  A block never straddles two pages (page_size is a multiple of 64 and
    // paged caches have no left padding).
    elem8 kreg[16], vreg[16];
    auto request = [&](int jb) {
        const int key0 = jb * kBlockN;
        const elem_bits* kbase = p.kcache + cache_row_offset(p, b, lp + key0, p.kc_batch, p.kc_row) + h * p.kc_head;
        const elem_bits* vbase = p.vcache + cache_row_offset(p, b, lp + key0, p.vc_batch, p.vc_row) + h * p.vc_head;
#pragma unroll
        for (int kt = 0; kt < 4; ++kt) {
            int key = key0 + 16 * kt + n;
            key = key < L ? key : L - 1;
            const elem_bits* src = kbase + static_cast<int64_t>(key - key0) * p.kc_row + 8 * g;
#pragma unroll
            for (int c = 0; c < 4; ++c) kreg[kt * 4 + c] = *reinterpret_cast<const elem8*>(src + 32 * c);
        }
#pragma unroll
        for (int u = 0; u < 16; ++u) {
            const int unit = lane + 64 * u;
            int key = key0 + (unit >> 4);
            key = key < L ? key : L - 1;
            vreg[u] = *reinterpret_cast<const elem8*>(vbase + static_cast<int64_t>(key - key0) * p.vc_row + (unit & 15) * 8);
        }
    };
    // One loop turn: S and the V tile of the block whose rows are in the registers (j), then - both register sets
    // being free again - the request for the next block (j_req), then the softmax and P V of block j while those
    // rows travel.  The first turn only requests.
    int j_req = count > 0 ? j : -1, issued = 0;
    j = -1;
    for (;;) {
        const int key0 = j * kBlockN;
        floatx4 s[4];
        if (j >= 0) {
#pragma unroll
            for (int kt = 0; kt < 4; ++kt) {
                s[kt] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int c = 0; c < 4; ++c)
                    s[kt] = IV2_MFMA(kreg[kt * 4 + c], qf[c], s[kt], 0, 0, 0);
            }
#pragma unroll
            for (int u = 0; u < 16; ++u) {
                const int unit = lane + 64 * u;
                *reinterpret_cast<elem8*>(&vt[(unit >> 4) * kVtPitch + (unit & 15) * 8]) = vreg[u];
            }
        }
        if (j_req >= 0) { request(j_req); ++issued; }
        if (j < 0) {                                           // first turn: nothing to work on yet
            if (j_req < 0) break;
            j = j_req;
            j_req = issued < count ? walk.next() : -1;
            continue;
        }
        const int lim = L - 1 - key0;                           // in-block index of the last valid key
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
        const float m_new = fmaxf(m, mx * p.scale_log2);
        const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
        const float alpha = __builtin_amdgcn_exp2f(m - m_use);
        float rs = 0.f;
#pragma unroll
        for (int kt = 0; kt < 4; ++kt)
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const float pv = __builtin_amdgcn_exp2f(s[kt][e] * p.scale_log2 - m_use);
                s[kt][e] = pv;
                rs += pv;
            }
        l = l * alpha + rs;
        m = m_new;
#pragma unroll
        for (int dt = 0; dt < 8; ++dt) o[dt] *= alpha;
        elem8 pf[2];
#pragma unroll
        for (int cc = 0; cc < 2; ++cc)
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                pf[cc][e] = static_cast<elem_t>(s[2 * cc][e]);
                pf[cc][4 + e] = static_cast<elem_t>(s[2 * cc + 1][e]);
            }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
        __builtin_amdgcn_s_barrier();                          // single-wavefront workgroup: orders the LDS tile
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
        // A operand of O^T += V^T P^T: lane (n, g) needs V[32 cc + 4 g + {0..3}, 32 cc + 16 + 4 g + {0..3}][16 dt + n], the
        // keys in the order in which the lane holds P.  One transposing read hands a lane four rows' worth of one
        // column: within 16 lanes, lane i offers the four columns 16 dt + 4 (i % 4) .. of key 4 g + i / 4 (+ 32 cc),
        // and lane n receives column 16 dt + n of the keys 4 g + {0, 1, 2, 3}.
        const elem_bits* tr_base = vt + (4 * g + (n >> 2)) * kVtPitch + 4 * (n & 3);
#pragma unroll
        for (int dt = 0; dt < 8; ++dt)
#pragma unroll
            for (int cc = 0; cc < 2; ++cc) {
                const short4d lo = lds_read_tr(tr_base + (32 * cc) * kVtPitch + 16 * dt);
                const short4d hi = lds_read_tr(tr_base + (32 * cc + 16) * kVtPitch + 16 * dt);
                elem8 vf;
                __builtin_memcpy(&vf, &lo, 8);
                __builtin_memcpy(reinterpret_cast<unsigned char*>(&vf) + 8, &hi, 8);
                o[dt] = IV2_MFMA(vf, pf[cc], o[dt], 0, 0, 0);
            }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
        __builtin_amdgcn_s_barrier();                          // tile consumed before the next block overwrites it
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
        if (j_req < 0) break;
        j = j_req;
        j_req = issued < count ? walk.next() : -1;
    }

    const float l_tot = wave_sum_over_g(l);
    const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
    const float lse = l_tot > 0.f ? m * 0.69314718055994530942f + logf(l_tot) : (kDirect ? INFINITY : -INFINITY);
    if (kDirect) {
        if (n >= p.group) return;
        elem_bits* op = p.out + b * p.o_batch + (p.group * h + n) * p.o_head + 4 * g;
#pragma unroll
        for (int dt = 0; dt < 8; ++dt) {
            uint2 w;
            w.x = pack_elem2(o[dt][0] * inv, o[dt][1] * inv);
            w.y = pack_elem2(o[dt][2] * inv, o[dt][3] * inv);
            *reinterpret_cast<uint2*>(op + 16 * dt) = w;
        }
        if (g == 0) p.lse[static_cast<int64_t>(b) * p.num_heads_k * p.group + p.group * h + n] = lse;
    } else {
        const int64_t slot = (static_cast<int64_t>(b) * p.num_heads_k + h) * p.splits + split;
        float* op = p.o_part + (slot * 16 + n) * kHeadDim + 4 * g;
#pragma unroll
        for (int dt = 0; dt < 8; ++dt)
            *reinterpret_cast<float4*>(op + 16 * dt) = make_float4(o[dt][0] * inv, o[dt][1] * inv, o[dt][2] * inv, o[dt][3] * inv);
        if (g == 0) p.lse_part[slot * 16 + n] = lse;
    }
}

// merge the per-split partials: one workgroup per (sequence, KV head); thread t -> head t / 16, 8 columns.
// kSplits > 0: the split count is known at compile time, so every partial is requested before the first is used
// (one round trip to memory instead of one per split); 0: any count.
template <int kSplits>
__global__ __launch_bounds__(256)
void decode_combine_kernel(const DecodeParams p) {
    const int h = blockIdx.x, b = blockIdx.y;
    const int tid = threadIdx.x;
    const int head = tid >> 4, d0 = (tid & 15) * 8;
    if (head >= p.group) return;                               // partial rows that only filled the MFMA tile
    const int64_t slot0 = (static_cast<int64_t>(b) * p.num_heads_k + h) * p.splits;
    float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    float wsum = 0.f, mx = -INFINITY;
    if constexpr (kSplits > 0) {
        float ls[kSplits];
        float4 a[kSplits], c[kSplits];
#pragma unroll
        for (int s = 0; s < kSplits; ++s) ls[s] = p.lse_part[(slot0 + s) * 16 + head];
#pragma unroll
        for (int s = 0; s < kSplits; ++s) {
            const float* src = p.o_part + ((slot0 + s) * 16 + head) * kHeadDim + d0;
            a[s] = *reinterpret_cast<const float4*>(src);
            c[s] = *reinterpret_cast<const float4*>(src + 4);
        }
#pragma unroll
        for (int s = 0; s < kSplits; ++s) mx = fmaxf(mx, ls[s]);
        if (mx != -INFINITY) {
#pragma unroll
            for (int s = 0; s < kSplits; ++s) {
                const float w = ls[s] == -INFINITY ? 0.f : expf(ls[s] - mx);       // a split without blocks: zeros and -inf
                wsum += w;
                acc[0] += w * a[s].x; acc[1] += w * a[s].y; acc[2] += w * a[s].z; acc[3] += w * a[s].w;
                acc[4] += w * c[s].x; acc[5] += w * c[s].y; acc[6] += w * c[s].z; acc[7] += w * c[s].w;
            }
        }
    } else {
        for (int s = 0; s < p.splits; ++s) mx = fmaxf(mx, p.lse_part[(slot0 + s) * 16 + head]);
        if (mx != -INFINITY) {
            for (int s = 0; s < p.splits; ++s) {
                const float ls = p.lse_part[(slot0 + s) * 16 + head];
                if (ls == -INFINITY) continue;
                const float w = expf(ls - mx);
                wsum += w;
                const float* src = p.o_part + ((slot0 + s) * 16 + head) * kHeadDim + d0;
                const float4 a = *reinterpret_cast<const float4*>(src);
                const float4 c = *reinterpret_cast<const float4*>(src + 4);
                acc[0] += w * a.x; acc[1] += w * a.y; acc[2] += w * a.z; acc[3] += w * a.w;
                acc[4] += w * c.x; acc[5] += w * c.y; acc[6] += w * c.z; acc[7] += w * c.w;
            }
        }
    }
    const float inv = wsum > 0.f ? 1.f / wsum : 0.f;
    uint4 outv;
    outv.x = pack_elem2(acc[0] * inv, acc[1] * inv);
    outv.y = pack_elem2(acc[2] * inv, acc[3] * inv);
    outv.z = pack_elem2(acc[4] * inv, acc[5] * inv);
    outv.w = pack_elem2(acc[6] * inv, acc[7] * inv);
    *reinterpret_cast<uint4*>(p.out + b * p.o_batch + (p.group * h + head) * p.o_head + d0) = outv;
    if ((tid & 15) == 0)
        p.lse[static_cast<int64_t>(b) * p.num_heads_k * p.group + p.group * h + head] = wsum > 0.f ? mx + logf(wsum) : INFINITY;
}

}  // namespace IV2_NS

using namespace IV2_NS;

#ifndef IV2_F16        // element-type independent: defined once
extern "C" int infllmv2_fwd_kvcache_num_splits(int batch, int num_heads_k, int requested) {
    if (requested > 0) return requested > 64 ? 64 : requested;
    // aim at two single-wavefront workgroups per CU of a 256-CU device (each keeps the next block's rows in flight, so
    // longer runs beat more workgroups: 53 us with 4 splits against 55 with 8 at 128 pairs), rounded up to a power of
    // two, for which the combine kernel is compiled
    const int pairs = batch * num_heads_k;
    const int want = (512 + pairs - 1) / (pairs > 0 ? pairs : 1);
    int s = 1;
    while (s < want && s < 16) s <<= 1;
    return s;
}
#endif

static size_t decode_partials_bytes(int batch, int num_heads_k, int num_splits) {
    if (num_splits <= 1) return 0;
    return static_cast<size_t>(batch) * num_heads_k * num_splits * 16 * (kHeadDim + 1) * sizeof(float);
}

#ifndef IV2_F16        // both element types are 2 bytes wide: defined once
extern "C" size_t infllmv2_fwd_kvcache_workspace_bytes(int batch, int num_heads_k, int num_splits) {
    // per-split partial results, then room for the query turned by the rotary embedding
    return decode_partials_bytes(batch, num_heads_k, num_splits) +
           static_cast<size_t>(batch) * num_heads_k * 16 * kHeadDim * sizeof(elem_bits);
}
#endif

static int fwd_kvcache_impl(void* stream, const void* q, void* kcache, void* vcache, const void* k_new,
                                    const void* v_new, const int32_t* cache_seqlens, void* out, float* softmax_lse,
                                    const uint64_t* blockmask, void* workspace, size_t workspace_bytes, int batch,
                                    int seqlen_q, int num_heads, int num_heads_k, int head_dim, int cache_capacity,
                                    int seqlen_new, const int64_t* q_strides, const int64_t* kcache_strides,
                                    const int64_t* vcache_strides, const int64_t* knew_strides,
                                    const int64_t* vnew_strides, const int64_t* o_strides, int n_uint64_per_row,
                                    int num_splits, float softmax_scale, const int32_t* cache_batch_idx,
                                    const int32_t* cache_leftpad, const int32_t* block_table,
                                    int64_t block_table_batch_stride, int page_block_size, const void* rotary_cos,
                                    const void* rotary_sin, int rotary_dim, int rotary_interleaved) {
    IV2_CHECK(head_dim == kHeadDim, "fwd_kvcache: this build only supports head_dim 128 (got %d)", head_dim);
    IV2_CHECK(seqlen_q == 1, "fwd_kvcache: this build only supports one query token per sequence (got %d)", seqlen_q);
    IV2_CHECK(valid_group(num_heads, num_heads_k),
              "fwd_kvcache: requires num_heads == g * num_heads_k with g in {1, 2, 4, 8, 16} (got %d and %d)", num_heads, num_heads_k);
    IV2_CHECK(batch > 0 && cache_capacity > 0, "fwd_kvcache: batch size and cache capacity must be positive");
    IV2_CHECK(batch <= 65535 && num_heads_k <= 65535, "fwd_kvcache: batch and num_heads_k must not exceed 65535");
    IV2_CHECK(q && kcache && vcache && out && softmax_lse, "fwd_kvcache: null pointer");
    IV2_CHECK((k_new == nullptr) == (v_new == nullptr), "fwd_kvcache: k and v must be given together");
    IV2_CHECK(k_new == nullptr || seqlen_new > 0, "fwd_kvcache: new keys given with seqlen_new == 0");
    IV2_CHECK(blockmask == nullptr || n_uint64_per_row > 0, "fwd_kvcache: mask given without words per row");
    IV2_CHECK(softmax_scale > 0.f, "fwd_kvcache: softmax_scale must be positive");
    IV2_CHECK(num_splits >= 1 && num_splits <= 64, "fwd_kvcache: num_splits must be in [1, 64]");
    IV2_CHECK(workspace_bytes >= infllmv2_fwd_kvcache_workspace_bytes(batch, num_heads_k, num_splits),
              "fwd_kvcache: workspace too small");
    IV2_CHECK(workspace != nullptr || (num_splits == 1 && rotary_cos == nullptr), "fwd_kvcache: split decode and rotary need a workspace");
    IV2_CHECK(block_table == nullptr || cache_batch_idx == nullptr, "Paged KVcache does not support cache_batch_idx");
    IV2_CHECK(block_table == nullptr || cache_leftpad == nullptr,
              "We don't support Paged KV and leftpad_k running at the same time yet");
    IV2_CHECK(block_table == nullptr || (page_block_size > 0 && page_block_size % kBlockN == 0 && block_table_batch_stride > 0),
              "fwd_kvcache: the page size of a paged KV cache must be a positive multiple of 64 (got %d)", page_block_size);
    IV2_CHECK((rotary_cos == nullptr) == (rotary_sin == nullptr), "If rotary cos is provided, rotary sin must also be provided");
    IV2_CHECK(rotary_cos == nullptr || k_new != nullptr,
              "If rotary cos/sin are provided, new key / value to be appended to KV cache must also be provided");
    IV2_CHECK(rotary_cos == nullptr || (rotary_dim > 0 && rotary_dim <= head_dim), "rotary_dim must be <= headdim");
    IV2_CHECK(rotary_cos == nullptr || rotary_dim % 16 == 0, "Only rotary dimensions divisible by 16 are currently supported");
    IV2_CHECK(rotary_cos == nullptr || (reinterpret_cast<uintptr_t>(rotary_cos) % 2 == 0 && reinterpret_cast<uintptr_t>(rotary_sin) % 2 == 0),
              "fwd_kvcache: rotary tables must be 2-byte aligned");
    const void* aligned16[] = {q, kcache, vcache, out};
    for (const void* a : aligned16) IV2_CHECK(reinterpret_cast<uintptr_t>(a) % 16 == 0, "fwd_kvcache: tensors must be 16-byte aligned");
    IV2_CHECK(q_strides[0] % 8 == 0 && q_strides[1] % 8 == 0 && o_strides[0] % 8 == 0 && o_strides[1] % 8 == 0,
              "fwd_kvcache: q/out strides must be multiples of 8 elements");
    for (int s = 0; s < 3; ++s)
        IV2_CHECK(kcache_strides[s] % 8 == 0 && vcache_strides[s] % 8 == 0, "fwd_kvcache: cache strides must be multiples of 8 elements");

    DecodeParams p{};
    p.q = static_cast<const elem_bits*>(q);
    p.kcache = static_cast<elem_bits*>(kcache);
    p.vcache = static_cast<elem_bits*>(vcache);
    p.knew = static_cast<const elem_bits*>(k_new);
    p.vnew = static_cast<const elem_bits*>(v_new);
    p.out = static_cast<elem_bits*>(out);
    p.lse = softmax_lse;
    p.cache_seqlens = cache_seqlens;
    p.mask = blockmask;
    p.q_batch = q_strides[0]; p.q_head = q_strides[1];
    p.o_batch = o_strides[0]; p.o_head = o_strides[1];
    p.kc_batch = kcache_strides[0]; p.kc_row = kcache_strides[1]; p.kc_head = kcache_strides[2];
    p.vc_batch = vcache_strides[0]; p.vc_row = vcache_strides[1]; p.vc_head = vcache_strides[2];
    p.batch = batch; p.num_heads_k = num_heads_k; p.capacity = cache_capacity;
    p.group = num_heads / num_heads_k;
    p.seqlen_new = k_new ? seqlen_new : 0;
    p.n64 = n_uint64_per_row; p.splits = num_splits;
    p.scale_log2 = softmax_scale * 1.44269504088896340736f;
    p.cache_batch_idx = cache_batch_idx; p.leftpad = cache_leftpad;
    p.block_table = block_table; p.bt_batch = block_table_batch_stride; p.page_size = block_table ? page_block_size : 1;
    p.rot_cos = static_cast<const elem_bits*>(rotary_cos); p.rot_sin = static_cast<const elem_bits*>(rotary_sin);
    p.rotary_dim = rotary_cos ? rotary_dim : 0; p.rotary_interleaved = rotary_interleaved;
    p.q_rot = reinterpret_cast<elem_bits*>(static_cast<unsigned char*>(workspace) + decode_partials_bytes(batch, num_heads_k, num_splits));
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (k_new != nullptr) {
        IV2_CHECK(reinterpret_cast<uintptr_t>(k_new) % 16 == 0 && reinterpret_cast<uintptr_t>(v_new) % 16 == 0,
                  "fwd_kvcache: new k/v must be 16-byte aligned");
        for (int s = 0; s < 3; ++s)
            IV2_CHECK(knew_strides[s] % 8 == 0 && vnew_strides[s] % 8 == 0, "fwd_kvcache: new k/v strides must be multiples of 8 elements");
        p.kn_batch = knew_strides[0]; p.kn_row = knew_strides[1]; p.kn_head = knew_strides[2];
        p.vn_batch = vnew_strides[0]; p.vn_row = vnew_strides[1]; p.vn_head = vnew_strides[2];
        const int64_t total = static_cast<int64_t>(batch) * seqlen_new * num_heads_k * 16;
        hipLaunchKernelGGL(decode_append_kernel, dim3(static_cast<unsigned>((total + 255) / 256)), dim3(256), 0, st, p);
        IV2_LAUNCH_CHECK();
        if (p.rotary_dim > 0) {
            const int64_t units = static_cast<int64_t>(batch) * num_heads * 16;
            hipLaunchKernelGGL(decode_rotate_q_kernel, dim3(static_cast<unsigned>((units + 255) / 256)), dim3(256), 0, st, p);
            IV2_LAUNCH_CHECK();
        }
    }
    const dim3 grid(num_splits, num_heads_k, batch);
    if (num_splits == 1) {
        hipLaunchKernelGGL(decode_split_kernel<true>, grid, dim3(64), 0, st, p);
        IV2_LAUNCH_CHECK();
    } else {
        float* ws = static_cast<float*>(workspace);
        p.o_part = ws;
        p.lse_part = ws + static_cast<size_t>(batch) * num_heads_k * num_splits * 16 * kHeadDim;
        hipLaunchKernelGGL(decode_split_kernel<false>, grid, dim3(64), 0, st, p);
        IV2_LAUNCH_CHECK();
        const dim3 cgrid(num_heads_k, batch);
        switch (num_splits) {
            case 2: hipLaunchKernelGGL(decode_combine_kernel<2>, cgrid, dim3(256), 0, st, p); break;
            case 4: hipLaunchKernelGGL(decode_combine_kernel<4>, cgrid, dim3(256), 0, st, p); break;
            case 8: hipLaunchKernelGGL(decode_combine_kernel<8>, cgrid, dim3(256), 0, st, p); break;
            case 16: hipLaunchKernelGGL(decode_combine_kernel<16>, cgrid, dim3(256), 0, st, p); break;
            default: hipLaunchKernelGGL(decode_combine_kernel<0>, cgrid, dim3(256), 0, st, p); break;
        }
        IV2_LAUNCH_CHECK();
    }
    return 0;
}

extern "C" int IV2_ENTRY(infllmv2_fwd_kvcache)(void* stream, const void* q, void* kcache, void* vcache, const void* k_new,
                                    const void* v_new, const int32_t* cache_seqlens, void* out, float* softmax_lse,
                                    const uint64_t* blockmask, void* workspace, size_t workspace_bytes, int batch,
                                    int seqlen_q, int num_heads, int num_heads_k, int head_dim, int cache_capacity,
                                    int seqlen_new, const int64_t* q_strides, const int64_t* kcache_strides,
                                    const int64_t* vcache_strides, const int64_t* knew_strides,
                                    const int64_t* vnew_strides, const int64_t* o_strides, int n_uint64_per_row,
                                    int num_splits, float softmax_scale, const int32_t* cache_batch_idx,
                                    const int32_t* cache_leftpad, const int32_t* block_table,
                                    int64_t block_table_batch_stride, int page_block_size, const void* rotary_cos,
                                    const void* rotary_sin, int rotary_dim, int rotary_interleaved) {
    return fwd_kvcache_impl(stream, q, kcache, vcache, k_new, v_new, cache_seqlens, out, softmax_lse, blockmask, workspace,
                            workspace_bytes, batch, seqlen_q, num_heads, num_heads_k, head_dim, cache_capacity, seqlen_new,
                            q_strides, kcache_strides, vcache_strides, knew_strides, vnew_strides, o_strides,
                            n_uint64_per_row, num_splits, softmax_scale, cache_batch_idx, cache_leftpad, block_table,
                            block_table_batch_stride, page_block_size, rotary_cos, rotary_sin, rotary_dim,
                            rotary_interleaved);
}

#ifndef IV2_F16        // one such entry point in the library: bfloat16 only
// ---- decode for callers that cannot allocate ---------------------------------------------------------------------
//
// The split partials and the turned query live in a device array that belongs to the library's code object: every GPU
// the library runs on holds one copy of it, at its own address, from module load to process end.  `scratch` below is
// only the host-side handle of that array; the device address is looked up once per device with
// hipGetSymbolAddress and is what the kernels get.  Nothing in the array has to start at zero: every (sequence, KV
// head, split) workgroup writes its whole partial slot before the combine kernel reads it, and the turned query is
// written before it is read.  All calls on one GPU share the array, so calls that overlap on one GPU (two streams, two
// threads) race; calls on one stream are ordered by the stream.
static __device__ __align__(256) unsigned char scratch[INFLLMV2_STATIC_SCRATCH_BYTES];

namespace {
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
void* g_scratch_ptr[kMaxDevices] = {};
}  // namespace

extern "C" int infllmv2_fwd_kvcache_static(void* stream, const void* q, void* kcache, void* vcache, const void* k_new,
                                           const void* v_new, const int32_t* cache_seqlens, void* out,
                                           float* softmax_lse, const uint64_t* blockmask, int batch, int seqlen_q,
                                           int num_heads, int num_heads_k, int head_dim, int cache_capacity,
                                           int seqlen_new, const int64_t* q_strides, const int64_t* kcache_strides,
                                           const int64_t* vcache_strides, const int64_t* knew_strides,
                                           const int64_t* vnew_strides, const int64_t* o_strides, int n_uint64_per_row,
                                           int num_splits, float softmax_scale, const int32_t* cache_batch_idx,
                                           const int32_t* cache_leftpad, const int32_t* block_table,
                                           int64_t block_table_batch_stride, int page_block_size,
                                           const void* rotary_cos, const void* rotary_sin, int rotary_dim,
                                           int rotary_interleaved) {
    IV2_CHECK(batch > 0 && num_heads_k > 0 && num_splits >= 1 && num_splits <= 64,
              "fwd_kvcache_static: batch, num_heads_k must be positive and num_splits in [1, 64]");
    const size_t need = infllmv2_fwd_kvcache_workspace_bytes(batch, num_heads_k, num_splits);
    IV2_CHECK(need <= static_cast<size_t>(INFLLMV2_STATIC_SCRATCH_BYTES),
              "fwd_kvcache_static: batch %d x %d KV heads x %d splits needs %zu bytes of scratch, the built-in buffer holds %zu; "
              "use fewer splits or infllmv2_fwd_kvcache with a workspace", batch, num_heads_k, num_splits, need,
              static_cast<size_t>(INFLLMV2_STATIC_SCRATCH_BYTES));
    // the copy of the array that belongs to the GPU the stream runs on (the null stream: the current device); the
    // symbol lookup below answers for the current device, so the two must be the same
    int dev = -1, stream_dev = -1;
    hipError_t e = hipGetDevice(&dev);
    IV2_CHECK(e == hipSuccess && dev >= 0 && dev < kMaxDevices, "fwd_kvcache_static: hipGetDevice failed or device index %d out of range", dev);
    if (stream != nullptr) {
        e = hipStreamGetDevice(static_cast<hipStream_t>(stream), &stream_dev);
        IV2_CHECK(e == hipSuccess, "fwd_kvcache_static: hipStreamGetDevice failed: %s", hipGetErrorString(e));
        IV2_CHECK(stream_dev == dev, "fwd_kvcache_static: the stream belongs to device %d but the current device is %d; "
                  "make the stream's device current before the call", stream_dev, dev);
    }
    void* ws = nullptr;
    {
        std::lock_guard<std::mutex> lock(g_scratch_mutex);
        if (g_scratch_ptr[dev] == nullptr) {
            void* sym = nullptr;
            e = hipGetSymbolAddress(&sym, HIP_SYMBOL(scratch));           // this device's copy of the array
            IV2_CHECK(e == hipSuccess && sym != nullptr, "fwd_kvcache_static: hipGetSymbolAddress failed: %s", hipGetErrorString(e));
            g_scratch_ptr[dev] = sym;
        }
        ws = g_scratch_ptr[dev];
    }
    return fwd_kvcache_impl(stream, q, kcache, vcache, k_new, v_new, cache_seqlens, out, softmax_lse, blockmask, ws,
                            static_cast<size_t>(INFLLMV2_STATIC_SCRATCH_BYTES), batch, seqlen_q, num_heads, num_heads_k,
                            head_dim, cache_capacity, seqlen_new, q_strides, kcache_strides, vcache_strides, knew_strides,
                            vnew_strides, o_strides, n_uint64_per_row, num_splits, softmax_scale, cache_batch_idx,
                            cache_leftpad, block_table, block_table_batch_stride, page_block_size, rotary_cos, rotary_sin,
                            rotary_dim, rotary_interleaved);
}
#endif
