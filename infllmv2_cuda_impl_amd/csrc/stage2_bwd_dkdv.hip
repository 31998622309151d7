// Stage-2 backward, dK / dV (gfx950): one wavefront per (64-key block, 512-token slice).
//
// Mathematics as in compute_dq_dk_dv_1colblock (csrc/flash_attn/src/flash_bwd_kernel.h:498-794):
// P = exp(scale S - LSE), dV += P^T dO, dS = P (dP - D), dK += scale dS^T Q, the 16 grouped heads
// of a token accumulating into their KV head.
//
// Why one wavefront owns a whole key block.  Per (token, block) pair the query side is only 16
// rows (the grouped heads), so every MFMA needs a fresh 1 KiB query-side operand unless that
// operand is reused across key tiles.  Here the block's K and V (B operands of S = Q K^T and
// dP = dO V^T, 128 registers) stay in VGPRs for the whole slice, the 64 x 128 dK^T and dV^T
// tiles are the wavefront's 256 accumulation registers (AGPRs), and each query-side operand
// fetched from LDS feeds four MFMAs.  No workgroup barrier and no cross-wavefront reduction is
// left; the CU runs four such wavefronts, one per SIMD.
//
// Query-side data path.  q and dout of a token pair are gathered straight from the caller's
// tensors into a two-stage LDS ring by LDS-DMA loads issued one pair ahead (no registers, no
// transposed copies in memory): the ring holds them as A-operand fragments of the first two
// GEMMs, and the transposed operands of dV^T = dO^T P and dK^T = Q^T dS are read from the same
// bytes with ds_read_b64_tr_b16.  Two tokens fill the 32-deep contraction of those GEMMs, and
// the S / dS accumulator registers are, converted to bf16, their B operands.
//
// The slice ends with one fp32 atomic flush of the two 64 x 128 tiles (transposed through the
// ring's LDS so that every atomic instruction covers 256 contiguous bytes).
#include "common.h"
#include "kv_image.h"
#include "stage2_bwd.h"
#include <math.h>

namespace infllmv2 {

constexpr int kColSlice = 512;                                 // query tokens per work item
constexpr int kColWords = kColSlice / 64 + 1;                  // mask words a slice can touch
constexpr int kStage = 16384 + 512;                            // q a|b, dout a|b (4 KiB each) + the pair's 64 row scalars
constexpr int kWaveLds = 2 * kStage;                           // = 64 rows x 132 floats: also the flush tile
constexpr int kFlushPitch = 132;                               // floats per key row of the flush tile

typedef short short4v __attribute__((ext_vector_type(4)));
typedef int int4v __attribute__((ext_vector_type(4)));

__device__ __forceinline__ uint32_t lds_addr(const void* ptr) {
    return static_cast<uint32_t>(reinterpret_cast<uintptr_t>((__attribute__((address_space(3))) const void*)ptr));
}
// LDS-DMA: lane l's 16 (4) bytes at base (scalar) + its own byte offset land at lds_base + 16 l (4 l).  The
// compiler's wait-count tracking does not see these loads; they are ordered by hand with s_waitcnt vmcnt(n).
// The instruction's immediate offset moves the global source AND the LDS destination, hence the subtraction.
template <int kOffset>
__device__ __forceinline__ void dma16(const void* base, uint32_t lane_off, uint32_t lds_base) {
    asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dwordx4 %0, %1 offset:%3"
                 : : "v"(lane_off), "s"(base), "s"(lds_base - kOffset), "n"(kOffset) : "memory", "m0");
}
__device__ __forceinline__ void dma4(const void* base, uint32_t lane_off, uint32_t lds_base) {
    asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dword %0, %1" : : "v"(lane_off), "s"(base), "s"(lds_base) : "memory", "m0");
}
// One d tile of the second GEMMs: dV^T[dt][kt] += ad * p[kt] and dK^T[dt][kt] += aq * ds[kt] for the four key tiles,
// accumulators in AGPRs.  Written as one asm block because the compiler cannot see that these are MFMAs: an MFMA
// must not read a VGPR in the two issue slots after a VALU instruction wrote it, so the block opens with the wait
// states itself and contains nothing but MFMAs; only MFMAs touch these accumulators inside the main loop.
__device__ __forceinline__ void mfma_dtile(floatx4 (&dv)[4], floatx4 (&dk)[4], const bf16x8& ad, const bf16x8& aq,
                                           const bf16x8 (&p)[4], const bf16x8 (&ds)[4]) {
    int4v adi, aqi, pi[4], dsi[4];
    __builtin_memcpy(&adi, &ad, 16);
    __builtin_memcpy(&aqi, &aq, 16);
#pragma unroll
    for (int kt = 0; kt < 4; ++kt) {
        __builtin_memcpy(&pi[kt], &p[kt], 16);
        __builtin_memcpy(&dsi[kt], &ds[kt], 16);
    }
    asm("s_nop 1\n\t"
        "v_mfma_f32_16x16x32_bf16 %0, %8, %10, %0\n\t"
        "v_mfma_f32_16x16x32_bf16 %4, %9, %14, %4\n\t"
        "v_mfma_f32_16x16x32_bf16 %1, %8, %11, %1\n\t"
        "v_mfma_f32_16x16x32_bf16 %5, %9, %15, %5\n\t"
        "v_mfma_f32_16x16x32_bf16 %2, %8, %12, %2\n\t"
        "v_mfma_f32_16x16x32_bf16 %6, %9, %16, %6\n\t"
        "v_mfma_f32_16x16x32_bf16 %3, %8, %13, %3\n\t"
        "v_mfma_f32_16x16x32_bf16 %7, %9, %17, %7"
        : "+a"(dv[0]), "+a"(dv[1]), "+a"(dv[2]), "+a"(dv[3]), "+a"(dk[0]), "+a"(dk[1]), "+a"(dk[2]), "+a"(dk[3])
        : "v"(adi), "v"(aqi), "v"(pi[0]), "v"(pi[1]), "v"(pi[2]), "v"(pi[3]), "v"(dsi[0]), "v"(dsi[1]), "v"(dsi[2]), "v"(dsi[3]));
}
// 16 lanes x 4 halfwords, transposed: lane (16 g + r) receives element r % 4 of the rows supplied by lanes
// 16 g + r / 4 + {0, 4, 8, 12}.
__device__ __forceinline__ short4v lds_read_tr(const unsigned char* ptr) {
    return __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) short4v*)(ptr));
}

template <bool kCausal>
__global__ __launch_bounds__(64)
void bwd_dkdv_wave_kernel(const BwdParams p, const int n_items_slices) {
    extern __shared__ __attribute__((aligned(16))) unsigned char ring[];
    const int lane = threadIdx.x;
    const int n = lane & 15, g = lane >> 4;
    const int b = blockIdx.y, h = blockIdx.z;
    const int q0 = p.cu_seqlens_q[b];
    const int Sq = p.cu_seqlens_q[b + 1] - q0;
    const int k0 = p.cu_seqlens_k[b];
    const int Sk = p.cu_seqlens_k[b + 1] - k0;
    const int nb = (Sk + kBlockN - 1) / kBlockN;               // key blocks of this sequence

    // ---- which (slice, block): the slices' shared first block, then the diagonal block and outwards, so the
    //      long items (initial block, local window) are dispatched first ----
    const int rel = blockIdx.x / n_items_slices;
    const int slice = blockIdx.x - rel * n_items_slices;
    int i_lo = slice * kColSlice;
    int i_hi = i_lo + kColSlice;
    if (i_hi > Sq) i_hi = Sq;
    if (i_lo >= i_hi || rel >= nb) return;                     // uniform
    int j;
    if (rel == 0) {
        j = 0;
    } else {
        int jd = kCausal ? (i_hi - 1 + Sk - Sq) / kBlockN : nb - 1;   // last block any token of the slice may see
        if (jd > nb - 1) jd = nb - 1;
        if (jd < 0) jd = 0;
        j = jd - rel + 1;
        if (j < 1) j += nb - 1;
    }
    if (kCausal) {
        const int first = j * kBlockN - (Sk - Sq);             // first token that can see key 64 j
        if (first > i_lo) i_lo = first;
    }
    if (i_lo >= i_hi) return;                                  // uniform

    // ---- the slice's mask words, clipped to its tokens: word w lives in lane w ----
    const int64_t t_lo = static_cast<int64_t>(q0) + i_lo, t_hi = static_cast<int64_t>(q0) + i_hi;
    const int w_lo = static_cast<int>(t_lo >> 6), w_hi = static_cast<int>((t_hi - 1) >> 6);
    const int n_words = w_hi - w_lo + 1;                       // <= kColWords
    uint64_t my_word = 0ull;
    if (lane < n_words) {
        const uint64_t* mrow = p.bwd_mask ? p.bwd_mask + (static_cast<int64_t>(h) * p.k_blocks + j) * p.n64_bwd : nullptr;
        uint64_t v = mrow ? mrow[w_lo + lane] : ~0ull;
        const int64_t base = static_cast<int64_t>(w_lo + lane) << 6;
        if (base < t_lo) v &= ~0ull << (t_lo - base);
        if (base + 64 > t_hi) v &= ~0ull >> (base + 64 - t_hi);
        my_word = v;
    }
    if (__ballot(my_word != 0ull) == 0ull) return;             // nobody in the slice selected this block

    // ---- K and V of the block: B operands, resident in registers ----
    bf16x8 kreg[4][4], vreg[4][4];
    {
        const int64_t img = (static_cast<int64_t>(h) * p.n_slots + image_slot0(p.cu_seqlens_k, b) + j) * kImageElems + lane * 8;
#pragma unroll
        for (int kt = 0; kt < 4; ++kt)
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                kreg[kt][c] = *reinterpret_cast<const bf16x8*>(p.kimg + img + (kt * 4 + c) * 512);
                vreg[kt][c] = *reinterpret_cast<const bf16x8*>(p.vimg_r + img + (kt * 4 + c) * 512);
            }
    }
    floatx4 dKt[8][4], dVt[8][4];                              // [d tile][key tile]: lane (n, g) holds [16 dt + 4 g + e][16 kt + n]
#pragma unroll
    for (int dt = 0; dt < 8; ++dt)
#pragma unroll
        for (int kt = 0; kt < 4; ++kt) {
            dKt[dt][kt] = floatx4{0.f, 0.f, 0.f, 0.f};
            dVt[dt][kt] = floatx4{0.f, 0.f, 0.f, 0.f};
        }

    // ---- token-pair cursor over the mask words (scalar state) ----
    int cw = -1;
    uint64_t bits = 0ull;
    auto next_pair = [&](int64_t& ta, int64_t& tb, bool& has_b) -> bool {
        while (bits == 0ull) {
            if (++cw >= n_words) return false;
            const uint32_t lo = __builtin_amdgcn_readlane(static_cast<uint32_t>(my_word), cw);
            const uint32_t hi = __builtin_amdgcn_readlane(static_cast<uint32_t>(my_word >> 32), cw);
            bits = (static_cast<uint64_t>(hi) << 32) | lo;
        }
        const int64_t base = static_cast<int64_t>(w_lo + cw) << 6;
        ta = base + __builtin_ctzll(bits);
        bits &= bits - 1ull;
        has_b = bits != 0ull;
        tb = has_b ? base + __builtin_ctzll(bits) : ta;
        bits &= bits - 1ull;                                   // no-op on zero
        return true;
    };

    // ---- LDS-DMA of one pair: lane (r, g') of chunk c gathers X[token][head r][32 c + 8 g' ..] ----
    const uint32_t ring_lds = __builtin_amdgcn_readfirstlane(lds_addr(ring));
    const uint32_t q_lane = static_cast<uint32_t>((n * p.q_grp + 8 * g) * 2);       // byte offsets inside one token and KV head
    const uint32_t do_lane = static_cast<uint32_t>((n * p.do_grp + 8 * g) * 2);
    const uint32_t stat_lane = static_cast<uint32_t>((lane & 31) * 4);
    const bf16_bits* q_head = p.q + static_cast<int64_t>(h) * p.q_kvh;
    const bf16_bits* do_head = p.dout + static_cast<int64_t>(h) * p.do_kvh;
    const float* stat_head = p.rowstat + static_cast<int64_t>(h) * p.total_q * 32;
    auto issue = [&](int64_t ta, int64_t tb, int stage) {
        const uint32_t st = ring_lds + stage * kStage;
        const bf16_bits* qa = q_head + ta * p.q_tok;
        const bf16_bits* qb = q_head + tb * p.q_tok;
        const bf16_bits* da = do_head + ta * p.do_tok;
        const bf16_bits* db = do_head + tb * p.do_tok;
        dma16<0>(qa, q_lane, st);           dma16<64>(qa, q_lane, st + 1024);
        dma16<128>(qa, q_lane, st + 2048);  dma16<192>(qa, q_lane, st + 3072);
        dma16<0>(qb, q_lane, st + 4096);    dma16<64>(qb, q_lane, st + 5120);
        dma16<128>(qb, q_lane, st + 6144);  dma16<192>(qb, q_lane, st + 7168);
        dma16<0>(da, do_lane, st + 8192);   dma16<64>(da, do_lane, st + 9216);
        dma16<128>(da, do_lane, st + 10240); dma16<192>(da, do_lane, st + 11264);
        dma16<0>(db, do_lane, st + 12288);  dma16<64>(db, do_lane, st + 13312);
        dma16<128>(db, do_lane, st + 14336); dma16<192>(db, do_lane, st + 15360);
        // token a's [lse * log2e (16) | D (16)] (both half-wavefronts fetch the same 128 bytes), then token b's
        dma4(stat_head + ta * 32, stat_lane, st + 16384);
        dma4(stat_head + tb * 32, stat_lane, st + 16384 + 256);
    };

    // Every ordinary load issued so far must have landed before the first LDS-DMA goes out: the compiler would
    // otherwise place its own wait for K/V inside the loop, and such a wait also drains the DMA loads that are
    // meant to stay in flight.
    __builtin_amdgcn_s_waitcnt(0x0F70);                        // vmcnt(0)
#pragma unroll
    for (int kt = 0; kt < 4; ++kt)
#pragma unroll
        for (int c = 0; c < 4; ++c) asm volatile("" : "+v"(kreg[kt][c]), "+v"(vreg[kt][c]));

    // lane's byte offset inside a token's 4 KiB fragment tile for the transposed reads: row rho = lane % 16 of
    // the 16 x 4 group is X[head 4 g + rho / 4][16 dt + 4 (rho % 4) ..]
    const int tr_off = ((n & 3) >> 1) * 256 + (4 * g + (n >> 2)) * 16 + (n & 1) * 8;

    int64_t ta, tb;
    bool has_b;
    bool more = next_pair(ta, tb, has_b);
    if (more) issue(ta, tb, 0);
    int stage = 0;
    while (more) {
        int64_t na, nb2;
        bool nhb;
        const bool have_next = next_pair(na, nb2, nhb);
        if (have_next) {
            issue(na, nb2, stage ^ 1);                         // the other stage was consumed by the previous turn
            __builtin_amdgcn_s_waitcnt(0x4F72);                // vmcnt(18): this turn's 18 loads have landed
        } else {
            __builtin_amdgcn_s_waitcnt(0x0F70);
        }
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
        const float4 la = *reinterpret_cast<const float4*>(scal + 4 * g);
        const float4 Da = *reinterpret_cast<const float4*>(scal + 16 + 4 * g);
        const float4 lb = *reinterpret_cast<const float4*>(scal + 64 + 4 * g);
        const float4 Db = *reinterpret_cast<const float4*>(scal + 80 + 4 * g);
        const float lse_a[4] = {la.x, la.y, la.z, la.w};
        const float lse_b[4] = {lb.x, lb.y, lb.z, lb.w};
        const float D_a[4] = {Da.x, Da.y, Da.z, Da.w};
        const float D_b[4] = {Db.x, Db.y, Db.z, Db.w};
        const bool edge = (lim_a < kBlockN - 1) || (lim_b < kBlockN - 1);

        // S = Q K^T and dP = dO V^T for both tokens, 32 keys at a time (bounds the live accumulators), then
        // P = exp2(scale S - LSE) and dS = P (dP - D), packed to bf16 as the B operands of the second GEMMs
        const uint4* frag = reinterpret_cast<const uint4*>(st) + lane;           // tile t, chunk c at frag[t * 256 + c * 64]
        bf16x8 pfr[4], dsfr[4];                                // per key tile: [token a heads 4g..4g+3 | token b heads 4g..4g+3]
#pragma unroll
        for (int hf = 0; hf < 2; ++hf) {
            floatx4 sa[2], sb[2], dpa[2], dpb[2];
#pragma unroll
            for (int k2 = 0; k2 < 2; ++k2) {
                sa[k2] = floatx4{0.f, 0.f, 0.f, 0.f};
                sb[k2] = sa[k2]; dpa[k2] = sa[k2]; dpb[k2] = sa[k2];
            }
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                const uint4 r0 = frag[0 * 256 + c * 64], r1 = frag[1 * 256 + c * 64];
                const uint4 r2 = frag[2 * 256 + c * 64], r3 = frag[3 * 256 + c * 64];
                bf16x8 qa, qb, doa, dob;
                __builtin_memcpy(&qa, &r0, 16);
                __builtin_memcpy(&qb, &r1, 16);
                __builtin_memcpy(&doa, &r2, 16);
                __builtin_memcpy(&dob, &r3, 16);
#pragma unroll
                for (int k2 = 0; k2 < 2; ++k2) {
                    const int kt = 2 * hf + k2;
                    sa[k2] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(qa, kreg[kt][c], sa[k2], 0, 0, 0);
                    sb[k2] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(qb, kreg[kt][c], sb[k2], 0, 0, 0);
                    dpa[k2] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(doa, vreg[kt][c], dpa[k2], 0, 0, 0);
                    dpb[k2] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(dob, vreg[kt][c], dpb[k2], 0, 0, 0);
                }
            }
#pragma unroll
            for (int k2 = 0; k2 < 2; ++k2) {
                const int kt = 2 * hf + k2;
                const int nlim_a = lim_a - 16 * kt, nlim_b = lim_b - 16 * kt;
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    float xa = __builtin_amdgcn_exp2f(sa[k2][e] * p.scale_log2 - lse_a[e]);
                    float xb = __builtin_amdgcn_exp2f(sb[k2][e] * p.scale_log2 - lse_b[e]);
                    if (edge) {
                        xa = n > nlim_a ? 0.f : xa;
                        xb = n > nlim_b ? 0.f : xb;
                    }
                    pfr[kt][e] = static_cast<__bf16>(xa);
                    pfr[kt][4 + e] = static_cast<__bf16>(xb);
                    dsfr[kt][e] = static_cast<__bf16>(xa * (dpa[k2][e] - D_a[e]));
                    dsfr[kt][4 + e] = static_cast<__bf16>(xb * (dpb[k2][e] - D_b[e]));
                }
            }
            __builtin_amdgcn_sched_barrier(0);                 // keep the halves apart: interleaving them costs 32 more live registers
        }

        // dV^T += dO^T P and dK^T += Q^T dS: the A operands are transposed reads of the same LDS tiles
        const unsigned char* tr = st + tr_off;
#pragma unroll
        for (int dt = 0; dt < 8; ++dt) {
            const short4v q_a = lds_read_tr(tr + dt * 512), q_b = lds_read_tr(tr + 4096 + dt * 512);
            const short4v d_a = lds_read_tr(tr + 8192 + dt * 512), d_b = lds_read_tr(tr + 12288 + dt * 512);
            bf16x8 aq, ad;
            __builtin_memcpy(&aq, &q_a, 8);
            __builtin_memcpy(reinterpret_cast<unsigned char*>(&aq) + 8, &q_b, 8);
            __builtin_memcpy(&ad, &d_a, 8);
            __builtin_memcpy(reinterpret_cast<unsigned char*>(&ad) + 8, &d_b, 8);
            mfma_dtile(dVt[dt], dKt[dt], ad, aq, pfr, dsfr);
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
#pragma unroll
    for (int which = 0; which < 2; ++which) {
        __syncthreads();
#pragma unroll
        for (int dt = 0; dt < 8; ++dt)
#pragma unroll
            for (int kt = 0; kt < 4; ++kt) {
                const floatx4 v = which == 0 ? dKt[dt][kt] : dVt[dt][kt];
                *reinterpret_cast<float4*>(tile + (16 * kt + n) * kFlushPitch + 16 * dt + 4 * g) = make_float4(v[0], v[1], v[2], v[3]);
            }
        __syncthreads();
        float* acc = (which == 0 ? p.dk_acc : p.dv_acc) + (row0 * p.num_heads_k + h) * kHeadDim + lane;
        const float mul = which == 0 ? p.scale : 1.f;
        for (int key = 0; key < valid_keys; ++key) {
            float* dst = acc + static_cast<int64_t>(key) * p.num_heads_k * kHeadDim;
            unsafeAtomicAdd(dst, tile[key * kFlushPitch + lane] * mul);
            unsafeAtomicAdd(dst + 64, tile[key * kFlushPitch + 64 + lane] * mul);
        }
    }
}

int launch_bwd_dkdv_wave(hipStream_t st, const BwdParams& p, int batch, int max_seqlen_q, bool causal) {
    const int n_slices = (max_seqlen_q + kColSlice - 1) / kColSlice;
    const int64_t items = static_cast<int64_t>(n_slices) * p.k_blocks;
    IV2_CHECK(items <= 0x7fffffffll, "varlen_bwd: too many (slice, block) work items");
    const dim3 grid(static_cast<unsigned>(items), batch, p.num_heads_k);
    if (causal) hipLaunchKernelGGL(bwd_dkdv_wave_kernel<true>, grid, dim3(64), kWaveLds, st, p, n_slices);
    else hipLaunchKernelGGL(bwd_dkdv_wave_kernel<false>, grid, dim3(64), kWaveLds, st, p, n_slices);
    IV2_LAUNCH_CHECK();
    return 0;
}

}  // namespace infllmv2
