// Shared declarations for the gfx950 kernels of the InfLLM-V2 sparse-attention path.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>

// The attention kernels exist once per element type: a translation unit compiled with -DIV2_F16 holds the IEEE-half
// instantiation (namespace infllmv2_f16, C entry points with the suffix _f16), one compiled without it the bfloat16
// one (namespace infllmv2, the plain entry-point names).  The two differ in the MFMA instruction, the conversions
// between fp32 and the element type, and nothing else: operand layouts, images and LDS traffic are the same bytes.
#ifdef IV2_F16
#define IV2_NS infllmv2_f16
#define IV2_ENTRY(name) name##_f16
#define IV2_MFMA(a, b, c, x, y, z) __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, x, y, z)
#define IV2_MFMA_ASM "v_mfma_f32_16x16x32_f16"
#else
#define IV2_NS infllmv2
#define IV2_ENTRY(name) name
#define IV2_MFMA(a, b, c, x, y, z) __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, x, y, z)
#define IV2_MFMA_ASM "v_mfma_f32_16x16x32_bf16"
#endif

namespace infllmv2 {
// Thread-local text of the last failure; every C entry point returns 0 on success.
void set_error(const char* fmt, ...);
}  // namespace infllmv2

namespace IV2_NS {

constexpr int kWave = 64;          // CDNA wavefront width
constexpr int kHeadDim = 128;      // only head size the reference build instantiates (static_switch.h:79-89)
constexpr int kGroup = 16;         // query heads per KV head the MFMA tiles are laid out for (flash_api.cpp:941)
constexpr int kBlockN = 64;        // key-block size of the sparse mask (flash_api.cpp:706-710)

#ifdef IV2_F16
typedef _Float16 elem_t;
#else
typedef __bf16 elem_t;
#endif
typedef __attribute__((__vector_size__(8 * sizeof(elem_t)))) elem_t elem8;     // one lane's MFMA operand
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4;
typedef uint16_t bf16_bits;
typedef uint16_t elem_bits;                                  // an element as it lies in memory

// Group sizes served: the reference build is hard-wired to 16 heads per KV head; smaller powers of two run on the same
// 16-row tiles with the spare rows repeating the last head (their results are never stored and never accumulated).
inline bool valid_group(int num_heads, int num_heads_k) {
    if (num_heads_k <= 0 || num_heads <= 0 || num_heads % num_heads_k != 0) return false;
    const int grp = num_heads / num_heads_k;
    return grp == 1 || grp == 2 || grp == 4 || grp == 8 || grp == 16;
}

#define IV2_CHECK(cond, ...)                         \
    do {                                             \
        if (!(cond)) {                               \
            infllmv2::set_error(__VA_ARGS__);        \
            return 1;                                \
        }                                            \
    } while (0)

#define IV2_LAUNCH_CHECK()                                                        \
    do {                                                                          \
        hipError_t e__ = hipGetLastError();                                       \
        if (e__ != hipSuccess) {                                                  \
            infllmv2::set_error("kernel launch failed: %s", hipGetErrorString(e__)); \
            return 2;                                                             \
        }                                                                         \
    } while (0)

__device__ __forceinline__ float bf16_to_f32(bf16_bits b) {
    return __uint_as_float(static_cast<uint32_t>(b) << 16);
}

// round-to-nearest-even fp32 -> bf16 bits; NaN stays NaN
__device__ __forceinline__ bf16_bits f32_to_bf16(float f) {
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return static_cast<bf16_bits>((u >> 16) | 0x40);
    u += 0x7fffu + ((u >> 16) & 1u);
    return static_cast<bf16_bits>(u >> 16);
}

__device__ __forceinline__ float f16_to_f32(uint16_t h) {
    _Float16 x;
    __builtin_memcpy(&x, &h, 2);
    return static_cast<float>(x);
}

__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
    return static_cast<uint32_t>(f32_to_bf16(lo)) | (static_cast<uint32_t>(f32_to_bf16(hi)) << 16);
}

// ---- the element type of this translation unit ----
#ifdef IV2_F16
constexpr elem_bits kElemPosInf = 0x7c00, kElemNegInf = 0xfc00;
__device__ __forceinline__ float elem_to_f32(elem_bits b) { return f16_to_f32(b); }
// round-to-nearest-even (v_cvt_f16_f32 in the default rounding mode); NaN stays NaN, overflow gives inf
__device__ __forceinline__ elem_bits f32_to_elem(float f) {
    const _Float16 x = static_cast<_Float16>(f);
    elem_bits b;
    __builtin_memcpy(&b, &x, 2);
    return b;
}
#else
constexpr elem_bits kElemPosInf = 0x7f80, kElemNegInf = 0xff80;
__device__ __forceinline__ float elem_to_f32(elem_bits b) { return bf16_to_f32(b); }
__device__ __forceinline__ elem_bits f32_to_elem(float f) { return f32_to_bf16(f); }
#endif
// the same rounding by the conversion instruction (v_cvt_pk_bf16_f32 / v_cvt_f16_f32: round to nearest even): one
// instruction where f32_to_bf16 spells the rounding out in integer steps; for kernels bound by vector instructions
__device__ __forceinline__ elem_bits f32_to_elem_hw(float f) {
    const elem_t x = static_cast<elem_t>(f);
    elem_bits b;
    __builtin_memcpy(&b, &x, 2);
    return b;
}
__device__ __forceinline__ uint32_t pack_elem2(float lo, float hi) {
    return static_cast<uint32_t>(f32_to_elem(lo)) | (static_cast<uint32_t>(f32_to_elem(hi)) << 16);
}
// the two elements of a 32-bit word
__device__ __forceinline__ float elem_lo_to_f32(uint32_t w) { return elem_to_f32(static_cast<elem_bits>(w & 0xffffu)); }
__device__ __forceinline__ float elem_hi_to_f32(uint32_t w) { return elem_to_f32(static_cast<elem_bits>(w >> 16)); }

}  // namespace IV2_NS
