// Shared declarations for the gfx950 kernels of the InfLLM-V2 sparse-attention path.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>

namespace infllmv2 {

constexpr int kWave = 64;          // CDNA wavefront width
constexpr int kHeadDim = 128;      // only head size the reference build instantiates (static_switch.h:79-89)
constexpr int kGroup = 16;         // query heads per KV head (flash_api.cpp:941)
constexpr int kBlockN = 64;        // key-block size of the sparse mask (flash_api.cpp:706-710)

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4;
typedef uint16_t bf16_bits;

// Thread-local text of the last failure; every C entry point returns 0 on success.
void set_error(const char* fmt, ...);

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

}  // namespace infllmv2
