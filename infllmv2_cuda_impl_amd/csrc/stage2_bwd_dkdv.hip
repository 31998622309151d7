// Stage-2 backward, dK / dV (gfx950): two wavefronts per (64-key block, slice of 512 or 128 query tokens), each owning
// 32 of the keys.
//
// Mathematics as in compute_dq_dk_dv_1colblock (csrc/flash_attn/src/flash_bwd_kernel.h:498-794):
// P = exp(scale S - LSE), dV += P^T dO, dS = P (dP - D), dK += scale dS^T Q, the 16 grouped heads
// of a token accumulating into their KV head.
//
// Why the key block stays put.  Per (token, block) pair the query side is only 16 rows (the grouped
// heads), so every MFMA needs a fresh 1 KiB query-side operand unless that operand is reused across
// key tiles.  Here a wavefront keeps its 32 keys of K and V (B operands of S = Q K^T and
// dP = dO V^T, 64 registers) in VGPRs for the whole slice, its 32 x 128 dK^T and dV^T tiles are
// 128 accumulation registers (AGPRs), and each query-side operand fetched from LDS feeds two MFMAs.
// With 256 registers per wavefront a SIMD holds two of them (one wavefront owning all 64 keys needs
// all 512 registers and then has nobody to fill its issue gaps: measured 6 % slower); the price is
// that the two wavefronts of a block read every query-side fragment once each, which makes the LDS
// pipe the busiest unit of the kernel.
//
// Query-side data path.  q and dout of a token pair are gathered straight from the caller's
// tensors into a two-stage LDS ring by LDS-DMA loads issued one pair ahead (no registers, no
// transposed copies in memory; wavefront 0 fetches q, wavefront 1 dout, one workgroup barrier per
// pair): the ring holds them as A-operand fragments of the first two GEMMs, and the transposed
// operands of dV^T = dO^T P and dK^T = Q^T dS are read from the same bytes with ds_read_b64_tr_b16.
// Two tokens fill the 32-deep contraction of those GEMMs, and the S / dS accumulator registers are,
// converted to bf16, their B operands.
//
// The slice ends with one fp32 atomic flush of the two tiles (transposed through the ring's LDS so
// that every atomic instruction covers 256 contiguous bytes).
#include "common.h"
#include "kv_image.h"
#include "stage2_bwd.h"
#include <math.h>

namespace IV2_NS {

constexpr int kGroupWords = 32;                                // one mask word per lane of the lower half-wavefront: a group is 2048 tokens
constexpr int kStage = 16384 + 512 + 512;                      // q a|b, dout a|b (4 KiB each), the pair's 64 row scalars; padded so that two stages are the flush tile
constexpr int kWaveLds = 2 * kStage;                           // = 64 rows x 132 floats: also the flush tile
constexpr int kFlushPitch = 132;                               // floats per key row of the flush tile
constexpr int kWaveTiles = 2;                                  // 16-key tiles per wavefront: a wavefront owns 32 of the block's 64 keys

typedef short short4v __attribute__((ext_vector_type(4)));
typedef int int4v __attribute__((ext_vector_type(4)));

__device__ __forceinline__ uint32_t lds_addr(const void* ptr) {
    return static_cast<uint32_t>(reinterpret_cast<uintptr_t>((__attribute__((address_space(3))) const void*)ptr));
}
// LDS-DMA: lane l's 16 (4) bytes at base (scalar) + its own byte offset land at lds_base + 16 l (4 l).  The
// compiler's wait-count tracking does not see these loads; they are ordered by hand with s_waitcnt vmcnt(n).
// The instruction's immediate offset moves the global source AND the LDS destination, hence the subtraction.
// kLds is added to the scalar LDS base inside the asm (one SALU instruction writes M0).
template <int kOffset, int kLds>
__device__ __forceinline__ void dma16(const void* base, uint32_t lane_off, uint32_t lds_base) {
    asm volatile("s_add_i32 m0, %2, %4\n\tglobal_load_lds_dwordx4 %0, %1 offset:%3"
                 : : "v"(lane_off), "s"(base), "s"(lds_base), "n"(kOffset), "n"(kLds - kOffset) : "memory", "m0", "scc");
}
template <int kLds>
__device__ __forceinline__ void dma4(const void* base, uint32_t lane_off, uint32_t lds_base) {
    asm volatile("s_add_i32 m0, %2, %3\n\tglobal_load_lds_dword %0, %1"
                 : : "v"(lane_off), "s"(base), "s"(lds_base), "n"(kLds) : "memory", "m0", "scc");
}
// One d tile of one of the second GEMMs: acc[kt] += a * b[kt] for the wavefront's two key tiles, accumulators in AGPRs.
// Written as one asm block because the compiler cannot see that these are MFMAs: an MFMA must not read a VGPR in
// the two issue slots after a VALU instruction wrote it, so the block opens with the wait states itself and
// contains nothing but MFMAs; only MFMAs touch these accumulators inside the main loop.
__device__ __forceinline__ void mfma_dtile(floatx4 (&acc)[kWaveTiles], const elem8& a, const elem8 (&b)[kWaveTiles]) {
    int4v ai, bi[kWaveTiles];
    __builtin_memcpy(&ai, &a, 16);
#pragma unroll
    for (int kt = 0; kt < kWaveTiles; ++kt) __builtin_memcpy(&bi[kt], &b[kt], 16);
    asm("s_nop 1\n\t"
        IV2_MFMA_ASM " %0, %2, %3, %0\n\t"
        IV2_MFMA_ASM " %1, %2, %4, %1"
        : "+a"(acc[0]), "+a"(acc[1])
        : "v"(ai), "v"(bi[0]), "v"(bi[1]));
}
// 16 lanes x 4 halfwords, transposed: lane (16 g + r) receives element r % 4 of the rows supplied by lanes
// 16 g + r / 4 + {0, 4, 8, 12}.
__device__ __forceinline__ short4v lds_read_tr(const unsigned char* ptr) {
    return __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) short4v*)(ptr));
}

// kColSlice: query tokens per work item (512, or 128 for short inputs)
template <bool kCausal, int kColSlice>
__global__ __launch_bounds__(128) __attribute__((amdgpu_waves_per_eu(2, 2)))
void bwd_dkdv_wave_kernel(const BwdParams p) {
    constexpr int kSliceWords = kColSlice / 64;                // mask words per slice (a power of two)
    constexpr int kGroupSlices = kGroupWords / kSliceWords;    // slices that pool their light members
    constexpr int kHeavyPairs = kColSlice / 4;                 // a slice with fewer selected tokens is "light"
    extern __shared__ __attribute__((aligned(16))) unsigned char ring[];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(static_cast<int>(threadIdx.x >> 6));   // which half of the block's keys
    const int n = lane & 15, g = lane >> 4;
    const int b = blockIdx.y, h = blockIdx.z;
    const int q0 = p.cu_seqlens_q[b];
    const int Sq = p.cu_seqlens_q[b + 1] - q0;
    const int k0 = p.cu_seqlens_k[b];
    const int Sk = p.cu_seqlens_k[b + 1] - k0;
    const int nb = (Sk + kBlockN - 1) / kBlockN;               // key blocks of this sequence

    // ---- which (slice, block) ----
    // Slices are cut on the packed token axis (so they are whole mask words) and clipped to the sequence; the slices
    // of 2048 consecutive tokens form a group.  Workgroup ids go round-robin over the 8 XCDs, and XCD x takes the groups
    // whose index on the packed axis is x modulo 8, latest first, one slice at a time: the wavefronts sharing an L2
    // stream the same tokens of q and dout, and because the assignment follows the packed axis (not each
    // sequence's own first group) the groups of a batch of sequences spread evenly over the XCDs.  Within a slice
    // the shared first block comes first, then the diagonal block and outwards, so the long items are dispatched early.
    // With fewer groups than XCDs (short inputs) that would leave XCDs idle: then all 8 XCDs share every slice, block
    // rel going to XCD rel % 8, slices latest first.
    const int xcd = blockIdx.x & 7, turn = blockIdx.x >> 3;
    if (Sq <= 0) return;                                       // uniform
    const int last_slice = (q0 + Sq - 1) / kColSlice;
    int rel, slice;
    if (p.dkdv_spread) {
        const int turns_per_slice = (p.k_blocks + 7) >> 3;
        rel = (turn % turns_per_slice) * 8 + xcd;
        slice = last_slice - turn / turns_per_slice;
    } else {
        rel = turn % p.k_blocks;
        const int top_group = last_slice / kGroupSlices;
        const int round = turn / p.k_blocks;                   // an XCD works through one group of slices in consecutive rounds
        const int grp_idx = top_group - ((top_group - xcd) & 7) - 8 * (round / kGroupSlices);
        slice = grp_idx < 0 ? -1 : grp_idx * kGroupSlices + (kGroupSlices - 1 - round % kGroupSlices);
    }
    if (rel >= nb || slice > last_slice || slice < q0 / kColSlice) return;      // uniform
    int j;
    if (rel == 0) {
        j = 0;
    } else {
        int i_last = (slice + 1) * kColSlice - 1 - q0;         // last token of the slice, inside the sequence
        if (i_last > Sq - 1) i_last = Sq - 1;
        int jd = kCausal ? (i_last + Sk - Sq) / kBlockN : nb - 1;                // last block any token of the slice may see
        if (jd > nb - 1) jd = nb - 1;
        if (jd < 0) jd = 0;
        j = jd - rel + 1;
        if (j < 1) j += nb - 1;
    }
    // tokens of the sequence that may see key 64 j at all
    int64_t t_lo = q0, t_hi = static_cast<int64_t>(q0) + Sq;
    if (kCausal) {
        const int first = j * kBlockN - (Sk - Sq);
        if (first > 0) t_lo += first;
    }
    if (t_lo >= t_hi) return;                                  // uniform

    // ---- light slices are merged ----
    // A flush costs 32768 fp32 atomics whatever the slice held, so a slice works on its own only if at least
    // kHeavyPairs of its tokens selected the block; the other slices of the same group hand their tokens
    // to the first non-empty one among them.  Every workgroup of the group takes the same decision from the
    // group's 32 mask words (lane l < 32 holds word l; a slice is kSliceWords consecutive lanes).
    unsigned long long* wbuf = reinterpret_cast<unsigned long long*>(ring + kWaveLds);      // [kGroupWords]
    const int group = slice / kGroupSlices, sub = slice % kGroupSlices;
    const int64_t w0 = static_cast<int64_t>(group) * kGroupWords;
    {
        const uint64_t* mrow = p.bwd_mask ? p.bwd_mask + (static_cast<int64_t>(h) * p.k_blocks + j) * p.n64_bwd : nullptr;
        uint64_t wv = 0ull;
        if (lane < kGroupWords) {
            const int64_t w = w0 + lane;
            const int64_t base = w << 6;
            if (base < t_hi && base + 64 > t_lo) {
                wv = mrow ? mrow[w] : ~0ull;
                if (base < t_lo) wv &= ~0ull << (t_lo - base);
                if (base + 64 > t_hi) wv &= ~0ull >> (base + 64 - t_hi);
            }
        }
        int cnt = __builtin_popcountll(wv);
#pragma unroll
        for (int off = 1; off < kSliceWords; off <<= 1) cnt += __shfl_xor(cnt, off);   // tokens of this lane's slice that selected the block
        const uint64_t heavy = __ballot(cnt >= kHeavyPairs);   // kSliceWords equal bits per slice
        const uint64_t filled = __ballot(cnt > 0);
        bool keep;
        if ((heavy >> (kSliceWords * sub)) & 1ull) {
            keep = (lane / kSliceWords) == sub;
        } else {
            const uint64_t light = filled & ~heavy;
            if (light == 0ull || (__builtin_ctzll(light) / kSliceWords) != sub) return;   // uniform: empty, or another slice collects
            keep = !((heavy >> lane) & 1ull);
        }
        if (lane < kGroupWords) wbuf[lane] = keep ? wv : 0ull;
    }
    __syncthreads();

    // ---- K and V of the block: B operands, resident in registers ----
    elem8 kreg[kWaveTiles][4], vreg[kWaveTiles][4];
    {
        const int64_t img = (static_cast<int64_t>(h) * p.n_slots + image_slot0(p.cu_seqlens_k, b) + j) * kImageElems +
                            wave * (kWaveTiles * 4 * 512) + lane * 8;
#pragma unroll
        for (int kt = 0; kt < kWaveTiles; ++kt)
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                kreg[kt][c] = *reinterpret_cast<const elem8*>(p.kimg + img + (kt * 4 + c) * 512);
                vreg[kt][c] = *reinterpret_cast<const elem8*>(p.vimg_r + img + (kt * 4 + c) * 512);
            }
    }
    floatx4 dKt[8][kWaveTiles], dVt[8][kWaveTiles];            // [d tile][key tile]: lane (n, g) holds [16 dt + 4 g + e][32 wave + 16 kt + n]
#pragma unroll
    for (int dt = 0; dt < 8; ++dt)
#pragma unroll
        for (int kt = 0; kt < kWaveTiles; ++kt) {
            dKt[dt][kt] = floatx4{0.f, 0.f, 0.f, 0.f};
            dVt[dt][kt] = floatx4{0.f, 0.f, 0.f, 0.f};
        }

    // ---- token-pair cursor over the kept mask words (scalar state) ----
    int cw = -1;
    uint64_t bits = 0ull;
    auto next_pair = [&](int64_t& ta, int64_t& tb, bool& has_b) -> bool {
        while (bits == 0ull) {
            if (++cw >= kGroupWords) return false;
            const uint64_t v = wbuf[cw];
            const uint32_t lo = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(v));
            const uint32_t hi = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(v >> 32));
            bits = (static_cast<uint64_t>(hi) << 32) | lo;
        }
        const int64_t base = (w0 + cw) << 6;
        ta = base + __builtin_ctzll(bits);
        bits &= bits - 1ull;
        has_b = bits != 0ull;
        tb = has_b ? base + __builtin_ctzll(bits) : ta;
        bits &= bits - 1ull;                                   // no-op on zero
        return true;
    };

    // ---- LDS-DMA of one pair: per 64-byte chunk c of the 16 head rows, one 1 KiB transfer ----
    const uint32_t ring_lds = __builtin_amdgcn_readfirstlane(lds_addr(ring));
    // Which 16 bytes a lane fetches: the four lanes of a quad take the four 16-byte pieces of one head's 64-byte
    // chunk, so a quad is one contiguous 64-byte request.  LDS unit l = 4 * head + j of a chunk then holds piece
    // (j + head / 4) % 4: the rotation makes the operand reads below bank-conflict free.
    const int dma_piece = ((lane & 3) + (lane >> 4)) & 3;
    const int dma_head = (lane >> 2) < p.group ? (lane >> 2) : p.group - 1;    // rows beyond the group repeat its last head: their LSE is +inf
    // byte offsets inside one token and KV head; wavefront 0 fetches q, wavefront 1 dout
    const uint32_t q_lane = static_cast<uint32_t>((dma_head * (wave == 0 ? p.q_grp : p.do_grp) + 8 * dma_piece) * 2);
    const uint32_t do_lane = q_lane;
    const uint32_t stat_lane = static_cast<uint32_t>((lane & 31) * 4);
    const elem_bits* q_head = p.q + static_cast<int64_t>(h) * p.q_kvh;
    const elem_bits* do_head = p.dout + static_cast<int64_t>(h) * p.do_kvh;
    const float* stat_head = p.rowstat + static_cast<int64_t>(h) * p.total_q * 32;
    // byte strides per token as 32-bit scalars (checked by the launcher): a token's address is one 32 x 32 -> 64 bit
    // multiplication away
    const uint32_t q_tok_bytes = static_cast<uint32_t>(p.q_tok * 2), do_tok_bytes = static_cast<uint32_t>(p.do_tok * 2);
    const unsigned char* q_bytes = reinterpret_cast<const unsigned char*>(q_head);
    const unsigned char* do_bytes = reinterpret_cast<const unsigned char*>(do_head);
    const unsigned char* stat_bytes = reinterpret_cast<const unsigned char*>(stat_head);
    auto issue = [&](int64_t ta, int64_t tb, int stage) {
        const uint32_t st = ring_lds + stage * kStage;
        const uint64_t ua = static_cast<uint32_t>(ta), ub = static_cast<uint32_t>(tb);     // packed token indices fit 31 bits
        const unsigned char* qa = q_bytes + ua * q_tok_bytes;
        const unsigned char* qb = q_bytes + ub * q_tok_bytes;
        const unsigned char* da = do_bytes + ua * do_tok_bytes;
        const unsigned char* db = do_bytes + ub * do_tok_bytes;
        // the two wavefronts share the pair's transfers: wavefront 0 fetches q, wavefront 1 dout
        if (wave == 0) {
            dma16<0, 0>(qa, q_lane, st);        dma16<64, 1024>(qa, q_lane, st);
            dma16<128, 2048>(qa, q_lane, st);   dma16<192, 3072>(qa, q_lane, st);
            dma16<0, 4096>(qb, q_lane, st);     dma16<64, 5120>(qb, q_lane, st);
            dma16<128, 6144>(qb, q_lane, st);   dma16<192, 7168>(qb, q_lane, st);
            // token a's [lse * log2e (16) | D (16)] (both half-wavefronts fetch the same 128 bytes)
            dma4<16384>(stat_bytes + (ua << 7), stat_lane, st);
        } else {
            dma16<0, 8192>(da, do_lane, st);    dma16<64, 9216>(da, do_lane, st);
            dma16<128, 10240>(da, do_lane, st); dma16<192, 11264>(da, do_lane, st);
            dma16<0, 12288>(db, do_lane, st);   dma16<64, 13312>(db, do_lane, st);
            dma16<128, 14336>(db, do_lane, st); dma16<192, 15360>(db, do_lane, st);
            dma4<16384 + 256>(stat_bytes + (ub << 7), stat_lane, st);
        }
    };

    // Every ordinary load issued so far must have landed before the first LDS-DMA goes out: the compiler would
    // otherwise place its own wait for K/V inside the loop, and such a wait also drains the DMA loads that are
    // meant to stay in flight.
    __builtin_amdgcn_s_waitcnt(0x0F70);                        // vmcnt(0)
#pragma unroll
    for (int kt = 0; kt < kWaveTiles; ++kt)
#pragma unroll
        for (int c = 0; c < 4; ++c) asm volatile("" : "+v"(kreg[kt][c]), "+v"(vreg[kt][c]));

    // lane's byte offset inside a token's 4 KiB fragment tile for the transposed reads: row rho = lane % 16 of
    // the 16 x 4 group is X[head 4 g + rho / 4][16 dt + 4 (rho % 4) ..]
    // piece g' = 2 (dt % 2) + (rho % 4) / 2 of head 4 g + rho / 4 sits in unit 4 * head + (g' - g) % 4
    const int tr_head = 4 * g + (n >> 2);
    const int tr_off_even = (4 * tr_head + ((((n & 3) >> 1) - g) & 3)) * 16 + (n & 1) * 8;
    const int tr_off_odd = (4 * tr_head + ((2 + ((n & 3) >> 1) - g) & 3)) * 16 + (n & 1) * 8;
    // operand fragment (head n, piece g) of a chunk: unit 4 n + (g - n / 4) % 4
    const int frag_unit = 4 * n + ((g - (n >> 2)) & 3);

    int64_t ta, tb;
    bool has_b;
    bool more = next_pair(ta, tb, has_b);
    if (more) issue(ta, tb, 0);
    int stage = 0;
    while (more) {
        // This wavefront's half of the pair's transfers has landed (nothing younger is in flight: the next pair goes out
        // below); the barrier adds the other wavefront's half and says that both are done with the other stage.
        __builtin_amdgcn_s_waitcnt(0x0F70);                    // vmcnt(0)
        __syncthreads();
        int64_t na, nb2;
        bool nhb;
        const bool have_next = next_pair(na, nb2, nhb);
        if (have_next) issue(na, nb2, stage ^ 1);
        const unsigned char* st = ring + stage * kStage;

        int lim_a, lim_b;                                      // in-block key index limit (inclusive)
        {
            const int valid = Sk - j * kBlockN - 1;
            lim_a = valid; lim_b = valid;
            if (kCausal) {
                const int ca = static_cast<int>(ta - q0) + Sk - Sq - j * kBlockN;
                const int cb = static_cast<int>(tb - q0) + Sk - Sq - j * kBlockN;
                lim_a = ca < lim_a ? ca : lim_a;
                lim_b = cb < lim_b ? cb : lim_b;
            }
            if (!has_b) lim_b = -1;
        }

        const float* scal = reinterpret_cast<const float*>(st + 16384);
        const bool edge = (lim_a < kBlockN - 1) || (lim_b < kBlockN - 1);
        // Per wavefront 64 MFMAs in four GEMM phases with the softmax backward between them; the other wavefront of the
        // SIMD fills the matrix pipeline while this one does vector work:
        //   A  S = Q K^T                       (both tokens, this wavefront's 32 keys; a fragment read from LDS feeds 2 MFMAs)
        //      P = exp2(scale S - LSE)         (fp32 in place of S, and bf16)
        //   B  dP = dO V^T                     (accumulators start at -D)
        //   C  dV^T += dO^T P                  while the VALU forms dS = P (dP - D) (bf16)
        //   D  dK^T += Q^T dS
        const uint4* frag = reinterpret_cast<const uint4*>(st) + frag_unit;      // tile t, chunk c at frag[t * 256 + c * 64]
        elem8 pfr[kWaveTiles], dsfr[kWaveTiles];              // per key tile: [token a heads 4g..4g+3 | token b heads 4g..4g+3]
        floatx4 sa[kWaveTiles], sb[kWaveTiles], dpa[kWaveTiles], dpb[kWaveTiles];
        // The S accumulators start at -LSE / scale, so that P = exp2(scale S') needs no subtraction (and the LSE no
        // registers) after the MFMAs; a row without visible keys has LSE = +inf: S' = -inf, P = 0.
        {
            const float4 la = *reinterpret_cast<const float4*>(scal + 4 * g);
            const float4 lb = *reinterpret_cast<const float4*>(scal + 64 + 4 * g);
            const float inv = -1.f / p.scale_log2;
            const floatx4 ia = {la.x * inv, la.y * inv, la.z * inv, la.w * inv}, ib = {lb.x * inv, lb.y * inv, lb.z * inv, lb.w * inv};
#pragma unroll
            for (int kt = 0; kt < kWaveTiles; ++kt) { sa[kt] = ia; sb[kt] = ib; }
        }
        {   // A
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                const uint4 fa = frag[c * 64], fb = frag[256 + c * 64];
                elem8 qa, qb;
                __builtin_memcpy(&qa, &fa, 16);
                __builtin_memcpy(&qb, &fb, 16);
#pragma unroll
                for (int kt = 0; kt < kWaveTiles; ++kt) {
                    sa[kt] = IV2_MFMA(qa, kreg[kt][c], sa[kt], 0, 0, 0);
                    sb[kt] = IV2_MFMA(qb, kreg[kt][c], sb[kt], 0, 0, 0);
                }
            }
        }
        __builtin_amdgcn_sched_barrier(0);
        {   // P, kept in fp32 in place of S
#pragma unroll
            for (int kt = 0; kt < kWaveTiles; ++kt)
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    float xa = __builtin_amdgcn_exp2f(sa[kt][e] * p.scale_log2);
                    float xb = __builtin_amdgcn_exp2f(sb[kt][e] * p.scale_log2);
                    sa[kt][e] = xa;
                    sb[kt][e] = xb;
                    pfr[kt][e] = static_cast<elem_t>(xa);
                    pfr[kt][4 + e] = static_cast<elem_t>(xb);
                }
        }
        __builtin_amdgcn_sched_barrier(0);
        {   // B
            const float4 Da = *reinterpret_cast<const float4*>(scal + 16 + 4 * g);
            const float4 Db = *reinterpret_cast<const float4*>(scal + 80 + 4 * g);
            // the dP accumulators start at -D, so that dS = P (dP - D) is one multiplication per element
            const floatx4 negD_a = {-Da.x, -Da.y, -Da.z, -Da.w}, negD_b = {-Db.x, -Db.y, -Db.z, -Db.w};
#pragma unroll
            for (int kt = 0; kt < kWaveTiles; ++kt) { dpa[kt] = negD_a; dpb[kt] = negD_b; }
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                const uint4 fa = frag[512 + c * 64], fb = frag[768 + c * 64];
                elem8 doa, dob;
                __builtin_memcpy(&doa, &fa, 16);
                __builtin_memcpy(&dob, &fb, 16);
#pragma unroll
                for (int kt = 0; kt < kWaveTiles; ++kt) {
                    dpa[kt] = IV2_MFMA(doa, vreg[kt][c], dpa[kt], 0, 0, 0);
                    dpb[kt] = IV2_MFMA(dob, vreg[kt][c], dpb[kt], 0, 0, 0);
                }
            }
        }
        __builtin_amdgcn_sched_barrier(0);
        if (edge) {
            // a block cut by the causal diagonal or by the sequence end (rare): keys beyond the limit get P = 0
#pragma unroll
            for (int kt = 0; kt < kWaveTiles; ++kt) {
                const int key0 = 16 * (kWaveTiles * wave + kt);
                const bool off_a = n > lim_a - key0, off_b = n > lim_b - key0;
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    sa[kt][e] = off_a ? 0.f : sa[kt][e];
                    sb[kt][e] = off_b ? 0.f : sb[kt][e];
                    pfr[kt][e] = static_cast<elem_t>(sa[kt][e]);
                    pfr[kt][4 + e] = static_cast<elem_t>(sb[kt][e]);
                }
            }
        }
        __builtin_amdgcn_sched_barrier(0);
        const unsigned char* tr_e = st + tr_off_even;
        const unsigned char* tr_o = st + tr_off_odd;
        auto tr_at = [&](int tile_bytes, int dt) { return ((dt & 1) ? tr_o : tr_e) + tile_bytes + (dt >> 1) * 1024; };
        {   // C: the A operands are transposed reads of the dout tiles, fetched one d tile ahead
            short4v t_a[2], t_b[2];
            t_a[0] = lds_read_tr(tr_at(8192, 0)); t_b[0] = lds_read_tr(tr_at(12288, 0));
#pragma unroll
            for (int dt = 0; dt < 8; ++dt) {
                if (dt < 7) { t_a[(dt + 1) & 1] = lds_read_tr(tr_at(8192, dt + 1)); t_b[(dt + 1) & 1] = lds_read_tr(tr_at(12288, dt + 1)); }
                elem8 ad;
                __builtin_memcpy(&ad, &t_a[dt & 1], 8);
                __builtin_memcpy(reinterpret_cast<unsigned char*>(&ad) + 8, &t_b[dt & 1], 8);
                mfma_dtile(dVt[dt], ad, pfr);
                {   // dS of a quarter key tile
                    const int kt = dt >> 2, e = dt & 3;
                    dsfr[kt][e] = static_cast<elem_t>(sa[kt][e] * dpa[kt][e]);
                    dsfr[kt][4 + e] = static_cast<elem_t>(sb[kt][e] * dpb[kt][e]);
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        {   // D: transposed reads of the q tiles
            short4v t_a[2], t_b[2];
            t_a[0] = lds_read_tr(tr_at(0, 0)); t_b[0] = lds_read_tr(tr_at(4096, 0));
#pragma unroll
            for (int dt = 0; dt < 8; ++dt) {
                if (dt < 7) { t_a[(dt + 1) & 1] = lds_read_tr(tr_at(0, dt + 1)); t_b[(dt + 1) & 1] = lds_read_tr(tr_at(4096, dt + 1)); }
                elem8 aq;
                __builtin_memcpy(&aq, &t_a[dt & 1], 8);
                __builtin_memcpy(reinterpret_cast<unsigned char*>(&aq) + 8, &t_b[dt & 1], 8);
                mfma_dtile(dKt[dt], aq, dsfr);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        more = have_next;
        ta = na; tb = nb2; has_b = nhb;
        stage ^= 1;
    }

    // the last MFMAs' results must be out of the matrix pipeline before ordinary instructions read them
    asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");

    // ---- flush: through LDS as [key][d] rows, then one 256-byte atomic row segment per instruction ----
    float* tile = reinterpret_cast<float*>(ring);
    const int valid_keys = (Sk - j * kBlockN) < kBlockN ? (Sk - j * kBlockN) : kBlockN;
    const int64_t row0 = static_cast<int64_t>(k0) + static_cast<int64_t>(j) * kBlockN;
    const int key_lo = 16 * kWaveTiles * wave;                 // this wavefront's rows of the tile
    const int key_hi = key_lo + 16 * kWaveTiles < valid_keys ? key_lo + 16 * kWaveTiles : valid_keys;
#pragma unroll
    for (int which = 0; which < 2; ++which) {
        __syncthreads();
#pragma unroll
        for (int dt = 0; dt < 8; ++dt)
#pragma unroll
            for (int kt = 0; kt < kWaveTiles; ++kt) {
                const floatx4 v = which == 0 ? dKt[dt][kt] : dVt[dt][kt];
                *reinterpret_cast<float4*>(tile + (key_lo + 16 * kt + n) * kFlushPitch + 16 * dt + 4 * g) = make_float4(v[0], v[1], v[2], v[3]);
            }
        __syncthreads();
        const float mul = which == 0 ? p.scale : 1.f;
        if (p.det_slots != nullptr) {
            // deterministic mode: the tile goes to this work item's own slot (all 64 rows: rows past the sequence
            // end hold zeros), to be added in slice order by bwd_dkdv_reduce_kernel
            const int64_t item = (static_cast<int64_t>(h) * p.n_slots + image_slot0(p.cu_seqlens_k, b) + j) * p.det_slices + slice;
            float* dst = p.det_slots + (item * 2 + which) * (kBlockN * kHeadDim) + lane;
            for (int key = key_lo; key < key_lo + 16 * kWaveTiles; ++key) {
                dst[key * kHeadDim] = tile[key * kFlushPitch + lane] * mul;
                dst[key * kHeadDim + 64] = tile[key * kFlushPitch + 64 + lane] * mul;
            }
            if (which == 1 && lane == 0 && wave == 0) p.det_flags[item] = 1u;
            continue;
        }
        float* acc = (which == 0 ? p.dk_acc : p.dv_acc) + (row0 * p.num_heads_k + h) * kHeadDim + lane;
        for (int key = key_lo; key < key_hi; ++key) {
            float* dst = acc + static_cast<int64_t>(key) * p.num_heads_k * kHeadDim;
            unsafeAtomicAdd(dst, tile[key * kFlushPitch + lane] * mul);
            unsafeAtomicAdd(dst + 64, tile[key * kFlushPitch + 64 + lane] * mul);
        }
    }
}

// Deterministic mode: one workgroup per (key block, sequence, KV head) adds the slots its work items wrote, in
// ascending slice order, and stores the sums where the atomic mode accumulates.
__global__ __launch_bounds__(256)
void bwd_dkdv_reduce_kernel(const BwdParams p) {
    const int j = blockIdx.x, b = blockIdx.y, h = blockIdx.z;
    const int k0 = p.cu_seqlens_k[b];
    const int Sk = p.cu_seqlens_k[b + 1] - k0;
    if (j * kBlockN >= Sk) return;
    const int64_t item0 = (static_cast<int64_t>(h) * p.n_slots + image_slot0(p.cu_seqlens_k, b) + j) * p.det_slices;
    const int valid_keys = (Sk - j * kBlockN) < kBlockN ? (Sk - j * kBlockN) : kBlockN;
    float4 acc[2][8];                                          // [dK | dV][8 x (256 threads x 4 floats)] = 64 x 128 each
#pragma unroll
    for (int w = 0; w < 2; ++w)
#pragma unroll
        for (int i = 0; i < 8; ++i) acc[w][i] = make_float4(0.f, 0.f, 0.f, 0.f);
    for (int s = 0; s < p.det_slices; ++s) {
        if (p.det_flags[item0 + s] == 0u) continue;            // uniform per workgroup
        const float4* src = reinterpret_cast<const float4*>(p.det_slots + (item0 + s) * 2 * (kBlockN * kHeadDim)) + threadIdx.x;
#pragma unroll
        for (int w = 0; w < 2; ++w)
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const float4 v = src[w * 2048 + i * 256];
                acc[w][i].x += v.x; acc[w][i].y += v.y; acc[w][i].z += v.z; acc[w][i].w += v.w;
            }
    }
    const int64_t row0 = static_cast<int64_t>(k0) + static_cast<int64_t>(j) * kBlockN;
#pragma unroll
    for (int w = 0; w < 2; ++w)
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int e = (i * 256 + threadIdx.x) * 4;         // element of the 64 x 128 tile
            const int key = e >> 7, d = e & 127;
            if (key < valid_keys)
                *reinterpret_cast<float4*>((w == 0 ? p.dk_acc : p.dv_acc) + ((row0 + key) * p.num_heads_k + h) * kHeadDim + d) = acc[w][i];
        }
}

int launch_bwd_dkdv_reduce(hipStream_t st, const BwdParams& p, int batch) {
    hipLaunchKernelGGL(bwd_dkdv_reduce_kernel, dim3(p.k_blocks, batch, p.num_heads_k), dim3(256), 0, st, p);
    IV2_LAUNCH_CHECK();
    return 0;
}

template <int kColSlice>
static int launch_bwd_dkdv_sliced(hipStream_t st, const BwdParams& p_in, int batch, int max_seqlen_q, bool causal) {
    BwdParams p = p_in;
    constexpr int kGroupSlices = kGroupWords * 64 / kColSlice;
    // a sequence of max_seqlen_q tokens touches at most `groups` consecutive slice groups wherever it starts
    const int group_tokens = kGroupWords * 64;
    const int groups = (max_seqlen_q + group_tokens - 1) / group_tokens + 1;
    int64_t items;
    // fewer groups than XCDs in the whole batch: every XCD takes a share of every slice
    p.dkdv_spread = static_cast<int64_t>(batch) * (groups - 1) < 8 ? 1 : 0;
    if (p.dkdv_spread) {
        const int n_slices = (max_seqlen_q + kColSlice - 1) / kColSlice + 1;               // a sequence need not start on a slice boundary
        items = static_cast<int64_t>(n_slices) * ((p.k_blocks + 7) / 8 * 8);
    } else {
        // an XCD takes every 8th group: ceil(groups / 8) rounds of kGroupSlices slices each
        const int n_slices8 = (groups + 7) / 8 * (8 * kGroupSlices);
        items = static_cast<int64_t>(n_slices8) * p.k_blocks;
    }
    IV2_CHECK(items <= 0x7fffffffll, "varlen_bwd: too many (slice, block) work items");
    IV2_CHECK(p.q_tok >= 0 && p.q_tok < (1ll << 31) && p.do_tok >= 0 && p.do_tok < (1ll << 31) && p.total_q < (1ll << 31),
              "varlen_bwd: token strides of q and dout must lie in [0, 2^31) elements");
    const dim3 grid(static_cast<unsigned>(items), batch, p.num_heads_k);
    const size_t lds = kWaveLds + kGroupWords * 8;
    if (causal) hipLaunchKernelGGL((bwd_dkdv_wave_kernel<true, kColSlice>), grid, dim3(128), lds, st, p);
    else hipLaunchKernelGGL((bwd_dkdv_wave_kernel<false, kColSlice>), grid, dim3(128), lds, st, p);
    IV2_LAUNCH_CHECK();
    return 0;
}

int launch_bwd_dkdv_wave(hipStream_t st, const BwdParams& p, int batch, int max_seqlen_q, bool causal) {
    if (dkdv_slice_tokens(p.total_q, p.det_slots != nullptr) == kDkdvSliceSmall) return launch_bwd_dkdv_sliced<kDkdvSliceSmall>(st, p, batch, max_seqlen_q, causal);
    return launch_bwd_dkdv_sliced<kDkdvSlice>(st, p, batch, max_seqlen_q, causal);
}

}  // namespace IV2_NS
