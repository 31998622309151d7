// Stage-2 backward, dQ from handed-over dS tiles (gfx950).
//
// dQ = scale dS K (compute_dq_dk_dv_1colblock, csrc/flash_attn/src/flash_bwd_kernel.h:700-760).  The
// column-parallel dK/dV kernel forms dS = P (dP - D) for every (token, block) pair anyway; when the
// caller announces an upper bound of selected blocks per mask row it stores each 64 x 16 dS^T tile
// (bf16, 2 KiB) at slot (kv head, token, rank of the block in the token's mask row), and this kernel
// computes dQ from those tiles and K alone: per pair 2 KiB + 16 KiB (K) come through the CU's
// vector-memory path instead of the 32 KiB (K and V) that recomputing S and dP needs, and 16
// MFMAs are left of 48.  The row-parallel kernels are bound by that path, so this is what makes
// dQ faster; dQ still stays in registers for the whole row and is written once.
//
// Schedule as in stage2_bwd_dq.hip: 8 wavefronts = 8 consecutive tokens; one turn = one block
// common to the 8 mask rows + one own block per wavefront.  K comes as the "K in V-image order"
// image the packing pre-pass writes for this kernel (keys contracted: the A operand of
// dQ^T = K^T dS^T as it lies in memory): the common block's image goes once through a 2-tile LDS
// ring and is read with plain ds_read_b128, the own block's 16 fragments are ordinary loads into
// registers one turn ahead.  dS^T arrives as [key][head] rows and becomes the B operand
// (contraction over keys) by transposed LDS reads (ds_read_b64_tr_b16).  The dS tiles are read
// once from HBM, so they are requested two turns ahead (two staging tiles per wavefront and
// kind); K is requested one turn ahead.
#include "common.h"
#include "kv_image.h"
#include "stage2_bwd.h"
#include <math.h>

namespace IV2_NS {

constexpr int kHoTokens = 8;
constexpr int kHoChunk = 16;                                   // token groups per XCD chunk
constexpr int kHoMaskWords = 256;                              // LDS copies of the mask rows: up to 16384 key blocks
constexpr int kHoRingBytes = 2 * 16384;                        // two K images (V-image order)
constexpr int kHoDsBytes = kHoTokens * 4 * 2048;               // per wavefront: {common, own} x {even, odd turn} dS^T tiles
constexpr int kHoTileLds = kHoRingBytes + kHoDsBytes;
constexpr int kHoLds = kHoTileLds + (1 + kHoTokens) * kHoMaskWords * 8 + kHoTokens * kHoMaskWords * 2;

typedef short short4h __attribute__((ext_vector_type(4)));

struct HoExtra {
    int groups_per_seq;
    int batch;
    int total_groups;
};

__device__ __forceinline__ uint32_t ho_lds_address(const void* ptr) {
    return static_cast<uint32_t>(reinterpret_cast<uintptr_t>((__attribute__((address_space(3))) const void*)ptr));
}
// 2 KiB flat copy global -> LDS by one wavefront: lane l moves bytes [16 l, 16 l + 16) of each KiB.  The compiler's
// wait counts do not see these loads; the kernel counts them itself (two per call) in its s_waitcnt vmcnt.
__device__ __forceinline__ void ho_dma_copy_2k(const void* src_lane, uint32_t lds_dst) {
    asm volatile("s_mov_b32 m0, %1\n\t"
                 "global_load_lds_dwordx4 %0, off\n\t"
                 "global_load_lds_dwordx4 %0, off offset:1024\n\t"
                 :
                 : "v"(src_lane), "s"(lds_dst)
                 : "memory", "m0");
}
__device__ __forceinline__ uint64_t ho_uniform_u64(uint64_t v) {
    const uint32_t lo = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(v));
    const uint32_t hi = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(v >> 32));
    return (static_cast<uint64_t>(hi) << 32) | lo;
}
__device__ __forceinline__ short4h ho_read_tr(const unsigned char* ptr) {
    return __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) short4h*)(ptr));
}

template <bool kCausal>
__global__ __launch_bounds__(512)
void bwd_dq_handoff_kernel(const BwdParams p, const HoExtra x) {
    extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
    unsigned long long* com = reinterpret_cast<unsigned long long*>(smem_raw + kHoTileLds);        // [kHoMaskWords]
    unsigned long long* rows = com + kHoMaskWords;                                                  // [kHoTokens][kHoMaskWords]
    unsigned short* before_all = reinterpret_cast<unsigned short*>(rows + kHoTokens * kHoMaskWords); // [kHoTokens][kHoMaskWords]

    const int bid = blockIdx.x;
    const int xcd = bid & 7, sidx = bid >> 3;
    int G = ((sidx / kHoChunk) * 8 + xcd) * kHoChunk + (sidx % kHoChunk);
    if (G >= x.total_groups) return;                                                // uniform per workgroup
    G = x.total_groups - 1 - G;
    const int grp = G % x.groups_per_seq;
    const int hb = G / x.groups_per_seq;
    const int b = hb % x.batch, h = hb / x.batch;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int n = lane & 15, g = lane >> 4;
    const int q0 = p.cu_seqlens_q[b];
    const int Sq = p.cu_seqlens_q[b + 1] - q0;
    const int i0 = grp * kHoTokens;
    if (i0 >= Sq) return;                                                           // uniform per workgroup
    const int Sk = p.cu_seqlens_k[b + 1] - p.cu_seqlens_k[b];

    const int i = i0 + wave;
    const bool live = i < Sq;
    int last_key = kCausal ? (i + Sk - Sq) : (Sk - 1);
    if (last_key > Sk - 1) last_key = Sk - 1;
    if (!live) last_key = -1;
    const int last_blk = last_key < 0 ? -1 : (last_key >> 6);
    const int64_t tok = static_cast<int64_t>(q0) + (live ? i : i0);
    const uint64_t* mrow = p.fwd_mask + (static_cast<int64_t>(h) * p.total_q + tok) * p.n64_fwd;   // the hand-off needs a mask

    // ---- the row words every live token of the group has in common, and what is left of each row ----
    int nw;
    {
        const int i_last = (i0 + kHoTokens - 1 < Sq) ? i0 + kHoTokens - 1 : Sq - 1;
        int lk = kCausal ? (i_last + Sk - Sq) : (Sk - 1);
        if (lk > Sk - 1) lk = Sk - 1;
        nw = lk < 0 ? 0 : (lk >> 12) + 1;
        if (nw > p.n64_fwd) nw = p.n64_fwd;                                          // nw <= kHoMaskWords: checked by the launcher
    }
    unsigned long long* own = rows + wave * kHoMaskWords;
    unsigned short* before = before_all + wave * kHoMaskWords;
    for (int w = tid; w < nw; w += 512) com[w] = ~0ull;
    __syncthreads();
    for (int w = lane; w < nw; w += 64) {
        uint64_t v = 0ull;
        if (last_blk >= 0 && w <= (last_blk >> 6)) {
            v = mrow[w];
            if (w == (last_blk >> 6)) {
                const int tb = last_blk & 63;
                v &= (tb == 63) ? ~0ull : ((1ull << (tb + 1)) - 1ull);
            }
        }
        own[w] = v;
        if (live && v != ~0ull) atomicAnd(&com[w], static_cast<unsigned long long>(v));
    }
    __syncthreads();
    // set bits of the (clipped) row in the words before w: with them the rank of a block in the row, which is the slot
    // of its dS^T tile, is one popcount away
    {
        int acc = 0;
        for (int w = 0; w < nw; ++w) {
            if (lane == 0) before[w] = static_cast<unsigned short>(acc);
            acc += __builtin_popcountll(ho_uniform_u64(own[w]));
        }
    }
    for (int w = lane; w < nw; w += 64) own[w] &= ~com[w];
    __syncthreads();

    floatx4 dq[8];
#pragma unroll
    for (int dt = 0; dt < 8; ++dt) dq[dt] = floatx4{0.f, 0.f, 0.f, 0.f};

    const int64_t slot0 = static_cast<int64_t>(h) * p.n_slots + image_slot0(p.cu_seqlens_k, b);
    // byte offset, inside a dS^T tile of [key][16 heads] rows (32 bytes), of this lane's row of the transposed reads
    // that yield the B operand of head n: its contraction slots are, as in the K image (V-image order), keys
    // 4 g .. 4 g + 3 of key tile 2 cc and then of key tile 2 cc + 1; row rho supplies key 4 g + rho / 4, heads 4 (rho % 4) ..
    const int ds_lane = (4 * g + (n >> 2)) * 32 + (n & 3) * 8;

    // ---- addresses ----
    const uint4* kt_units = reinterpret_cast<const uint4*>(p.ktimg) + slot0 * 1024;
    const uint4* ring_src = kt_units + wave * 128 + lane;                          // this wavefront's 2 KiB of an image
    const uint32_t ring_dst = __builtin_amdgcn_readfirstlane(ho_lds_address(smem_raw) + wave * 2048);
    auto issue_k = [&](int jj, int tile) { ho_dma_copy_2k(ring_src + static_cast<int64_t>(jj) * 1024, ring_dst + tile * 16384); };
    unsigned char* ds_tiles = smem_raw + kHoRingBytes + wave * 8192;               // [common | own][turn parity] x 2 KiB
    const uint32_t ds_lds = __builtin_amdgcn_readfirstlane(ho_lds_address(ds_tiles));
    const elem_bits* ds_row = p.ds_buf + (static_cast<int64_t>(h) * p.total_q + tok) * (p.max_sel + 1) * (kBlockN * 16) + lane * 8;
    // rank of block j in this token's row; blocks past the announced bound were stored in the row's spare slot
    auto rank_of = [&](int j) -> int {
        const int w = j >> 6;
        const uint64_t full = ho_uniform_u64(com[w] | own[w]);
        int r = __builtin_amdgcn_readfirstlane(static_cast<int>(before[w])) +
                __builtin_popcountll(full & ((1ull << (j & 63)) - 1ull));
        return r < p.max_sel ? r : p.max_sel;
    };
    auto issue_ds = [&](int j, int kind, int par) {
        ho_dma_copy_2k(ds_row + static_cast<int64_t>(rank_of(j)) * (kBlockN * 16), ds_lds + (kind * 2 + par) * 2048);
    };

    int cw = -1, ow = -1;
    uint64_t cbits = 0ull, obits = 0ull;
    auto next_common = [&]() -> int {
        while (cbits == 0ull) {
            if (++cw >= nw) return -1;
            cbits = ho_uniform_u64(com[cw]);
        }
        const int bit = __builtin_ctzll(cbits);
        cbits &= cbits - 1ull;
        return cw * 64 + bit;
    };
    auto next_own = [&]() -> int {
        while (obits == 0ull) {
            if (++ow >= nw) return -1;
            obits = ho_uniform_u64(own[ow]);
        }
        const int bit = __builtin_ctzll(obits);
        obits &= obits - 1ull;
        return ow * 64 + bit;
    };
    // The own block's 16 fragments (f = 2 dt + cc), 1 KiB apart.  Written as asm so that the compiler's wait counts do
    // not see them either: it would otherwise wait for everything in flight, the dS tiles of the next turn included,
    // before their first use.  Nothing may touch dst between here and the wait at the top of the next turn.
    const unsigned char* kt_bytes = reinterpret_cast<const unsigned char*>(p.ktimg) + slot0 * (kImageElems * 2);
    const uint32_t lane16 = lane * 16;
    auto load_k = [&](elem8 (&dst)[16], int j) {
        const unsigned char* blk = kt_bytes + static_cast<int64_t>(j) * (kImageElems * 2);         // uniform
#pragma unroll
        for (int qd = 0; qd < 4; ++qd) {
            const unsigned char* base = blk + qd * 4096;
            asm volatile("global_load_dwordx4 %0, %4, %5\n\t"
                         "global_load_dwordx4 %1, %4, %5 offset:1024\n\t"
                         "global_load_dwordx4 %2, %4, %5 offset:2048\n\t"
                         "global_load_dwordx4 %3, %4, %5 offset:3072\n\t"
                         : "=&v"(dst[4 * qd]), "=&v"(dst[4 * qd + 1]), "=&v"(dst[4 * qd + 2]), "=&v"(dst[4 * qd + 3])
                         : "v"(lane16), "s"(base)
                         : "memory");
        }
    };
    // B operands of the two 32-key chunks from a dS^T tile in LDS
    auto read_ds = [&](const unsigned char* tile, elem8 (&dsf)[2]) {
#pragma unroll
        for (int cc = 0; cc < 2; ++cc) {
            const short4h lo = ho_read_tr(tile + ds_lane + cc * 1024), hi = ho_read_tr(tile + ds_lane + cc * 1024 + 512);
            __builtin_memcpy(&dsf[cc], &lo, 8);
            __builtin_memcpy(reinterpret_cast<unsigned char*>(&dsf[cc]) + 8, &hi, 8);
        }
    };

    // ---- prologue: what the first two turns need, oldest request first ----
    // c0/c1/c2: the common blocks of this turn, the next and the one after; o0/o1/o2: the same for the own blocks
    elem8 ka[16], kb[16];
    int c0 = next_common();
    int c1 = c0 >= 0 ? next_common() : -1;
    int o0 = live ? next_own() : -1;
    int o1 = o0 >= 0 ? next_own() : -1;
    if (c0 >= 0 && live) issue_ds(c0, 0, 0);
    if (o0 >= 0) issue_ds(o0, 1, 0);
    if (c0 >= 0) issue_k(c0, 0);
    if (o0 >= 0) load_k(ka, o0);
    if (c1 >= 0 && live) issue_ds(c1, 0, 1);
    if (o1 >= 0) issue_ds(o1, 1, 1);
    int tile = 0, par = 0;
    // one turn; the K fragments of the next own block are loaded into the buffer the last turn used
    auto turn = [&](elem8 (&kcur)[16], elem8 (&knxt)[16]) {
        // This turn's K (requested during the last turn) and dS tiles (requested the turn before) have landed when
        // only the dS tiles of the next turn, the youngest requests, are still in flight (loads complete in order).
        const int young = ((c1 >= 0 && live) ? 2 : 0) + (o1 >= 0 ? 2 : 0);
        if (young == 4) asm volatile("s_waitcnt vmcnt(4)" ::: "memory");
        else if (young == 2) asm volatile("s_waitcnt vmcnt(2)" ::: "memory");
        else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#pragma unroll
        for (int f = 0; f < 16; ++f) asm volatile("" : "+v"(kcur[f]));
        // block c0 is in LDS for everyone and the other tile is free; once the common blocks are used up (uniform over
        // the workgroup) the wavefronts go on alone, each as long as its own row lasts
        if (c0 >= 0) __syncthreads();
        const int c2 = c1 >= 0 ? next_common() : -1;
        const int o2 = o1 >= 0 ? next_own() : -1;
        if (c1 >= 0) issue_k(c1, tile ^ 1);
        if (o1 >= 0) load_k(knxt, o1);
        if (c0 >= 0 && live) {                                 // the common block
            elem8 dsf[2];
            read_ds(ds_tiles + par * 2048, dsf);
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // the tile is in registers: its buffer takes the tile of
#pragma unroll                                                  // the turn after next
            for (int cc = 0; cc < 2; ++cc) asm volatile("" : "+v"(dsf[cc]));
            if (c2 >= 0) issue_ds(c2, 0, par);
            const uint4* kt = reinterpret_cast<const uint4*>(smem_raw + tile * 16384) + lane;
#pragma unroll
            for (int dt = 0; dt < 8; ++dt)
#pragma unroll
                for (int cc = 0; cc < 2; ++cc) {
                    const uint4 raw = kt[(dt * 2 + cc) * 64];
                    elem8 kf;
                    __builtin_memcpy(&kf, &raw, 16);
                    dq[dt] = IV2_MFMA(kf, dsf[cc], dq[dt], 0, 0, 0);
                }
        }
        if (o0 >= 0) {                                         // the own block
            elem8 dsf[2];
            read_ds(ds_tiles + (2 + par) * 2048, dsf);
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
            for (int cc = 0; cc < 2; ++cc) asm volatile("" : "+v"(dsf[cc]));
            if (o2 >= 0) issue_ds(o2, 1, par);
#pragma unroll
            for (int dt = 0; dt < 8; ++dt)
#pragma unroll
                for (int cc = 0; cc < 2; ++cc)
                    dq[dt] = IV2_MFMA(kcur[dt * 2 + cc], dsf[cc], dq[dt], 0, 0, 0);
        }
        if (c0 >= 0) tile ^= 1;
        par ^= 1;
        c0 = c1; c1 = c2;
        o0 = o1; o1 = o2;
    };
    while (c0 >= 0 || o0 >= 0) {
        turn(ka, kb);
        if (c0 < 0 && o0 < 0) break;
        turn(kb, ka);
    }
    if (!live || n >= p.group) return;

    elem_bits* op = p.dq + tok * p.dq_tok + h * p.dq_kvh + n * p.dq_grp + 4 * g;
#pragma unroll
    for (int dt = 0; dt < 8; ++dt) {
        uint2 wv;
        wv.x = pack_elem2(dq[dt][0] * p.scale, dq[dt][1] * p.scale);
        wv.y = pack_elem2(dq[dt][2] * p.scale, dq[dt][3] * p.scale);
        *reinterpret_cast<uint2*>(op + 16 * dt) = wv;
    }
}

int launch_bwd_dq_handoff(hipStream_t st, const BwdParams& p, int batch, int max_seqlen_q, bool causal) {
    HoExtra x{};
    x.batch = batch;
    x.groups_per_seq = (max_seqlen_q + kHoTokens - 1) / kHoTokens;
    const int64_t total = static_cast<int64_t>(p.num_heads_k) * batch * x.groups_per_seq;
    IV2_CHECK(total <= 0x3fffffff, "varlen_bwd: too many token groups");
    IV2_CHECK(p.k_blocks <= kHoMaskWords * 64, "varlen_bwd: more than %d key blocks per sequence", kHoMaskWords * 64);
    IV2_CHECK(p.fwd_mask != nullptr && p.ds_buf != nullptr && p.max_sel > 0, "varlen_bwd: the dS hand-off needs a mask");
    x.total_groups = static_cast<int>(total);
    const int64_t per_pass = 8 * kHoChunk;
    const int64_t grid = (total + per_pass - 1) / per_pass * per_pass;
    const void* fn = causal ? reinterpret_cast<const void*>(&bwd_dq_handoff_kernel<true>)
                            : reinterpret_cast<const void*>(&bwd_dq_handoff_kernel<false>);
    hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, kHoLds);
    IV2_CHECK(e == hipSuccess, "varlen_bwd: cannot reserve %d bytes of LDS: %s", kHoLds, hipGetErrorString(e));
    if (causal) hipLaunchKernelGGL(bwd_dq_handoff_kernel<true>, dim3(static_cast<unsigned>(grid)), dim3(512), kHoLds, st, p, x);
    else hipLaunchKernelGGL(bwd_dq_handoff_kernel<false>, dim3(static_cast<unsigned>(grid)), dim3(512), kHoLds, st, p, x);
    IV2_LAUNCH_CHECK();
    return 0;
}

}  // namespace IV2_NS
