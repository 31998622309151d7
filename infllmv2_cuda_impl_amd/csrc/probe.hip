// Streaming probes: what one CU's vector-memory return path and LDS deliver when nothing else competes.
// Not part of the attention path: bench.py --probe runs them so that the rate the Stage-2 gather is held against
// (bytes a CU receives through its L1 from L2-resident data, by plain loads and by LDS-DMA) can be re-measured on any box.
#include "common.h"
#include "../../include/infllmv2_hip.h"

namespace infllmv2 {

// mode 0: global_load_dwordx4 into registers; mode 1: LDS-DMA (global_load_lds_dwordx4); mode 2: ds_read_b128;
// mode 3: ds_read_b64_tr_b16 (the transposing LDS read; half the bytes per instruction).
// Every workgroup (8 wavefronts) re-reads its own 128 KiB region `iters` times, so the data comes from L2 / L1 / LDS,
// never from HBM.  out[2 * workgroup] = cycle-counter ticks the workgroup took, out[2 * workgroup + 1] = bytes it moved.
template <int kMode>
__global__ __launch_bounds__(512)
void probe_stream_kernel(const uint4* __restrict__ src, unsigned long long* __restrict__ out, int iters) {
    extern __shared__ uint4 lds[];                             // 128 KiB
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint4* region = src + static_cast<size_t>(blockIdx.x) * 8192;
    for (int i = tid; i < 8192; i += 512) lds[i] = region[i];
    __syncthreads();
    uint4 acc = make_uint4(0, 0, 0, 0);
    const unsigned long long t0 = __builtin_readcyclecounter();
    for (int it = 0; it < iters; ++it) {
        if (kMode == 0) {
            uint4 v[16];
#pragma unroll
            for (int u = 0; u < 16; ++u) v[u] = region[((wave * 16 + u + it * 16) & 127) * 64 + lane];   // moves with `it`: not hoistable
#pragma unroll
            for (int u = 0; u < 16; ++u) { acc.x ^= v[u].x; acc.y ^= v[u].y; acc.z ^= v[u].z; acc.w ^= v[u].w; }
        } else if (kMode == 1) {
            const uint32_t lds_base = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(reinterpret_cast<uintptr_t>(
                (__attribute__((address_space(3))) const void*)lds)) + wave * 16384);
            const uint4* lane_src = region + wave * 1024 + lane;
#pragma unroll
            for (int u = 0; u < 4; ++u)
                asm volatile("s_mov_b32 m0, %1\n\t"
                             "global_load_lds_dwordx4 %0, off\n\t"
                             "global_load_lds_dwordx4 %0, off offset:1024\n\t"
                             "global_load_lds_dwordx4 %0, off offset:2048\n\t"
                             "global_load_lds_dwordx4 %0, off offset:3072"
                             : : "v"(lane_src + u * 256), "s"(lds_base + u * 4096) : "memory", "m0");
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        } else if (kMode == 2) {
            uint4 v[16];
#pragma unroll
            for (int u = 0; u < 16; ++u) v[u] = lds[((wave * 16 + u + it * 16) & 127) * 64 + lane];
#pragma unroll
            for (int u = 0; u < 16; ++u) { acc.x ^= v[u].x; acc.y ^= v[u].y; acc.z ^= v[u].z; acc.w ^= v[u].w; }
            asm volatile("" : "+v"(acc.x));
        } else {
            // 32 transposing reads of 8 bytes per lane = the same 16 KiB per wavefront and iteration
            typedef short short4p __attribute__((ext_vector_type(4)));
            short4p v[32];
            const unsigned char* base = reinterpret_cast<const unsigned char*>(lds) + lane * 8;
#pragma unroll
            for (int u = 0; u < 32; ++u)
                v[u] = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                    (__attribute__((address_space(3))) short4p*)(base + ((wave * 32 + u + it * 32) & 255) * 512));
#pragma unroll
            for (int u = 0; u < 32; ++u) { acc.x ^= static_cast<unsigned>(v[u][0]); acc.y ^= static_cast<unsigned>(v[u][2]); }
            asm volatile("" : "+v"(acc.x));
        }
    }
    const unsigned long long t1 = __builtin_readcyclecounter();
    __syncthreads();
    if (kMode == 1) acc = lds[tid];
    if (tid == 0) {
        out[2 * blockIdx.x] = t1 - t0;
        out[2 * blockIdx.x + 1] = static_cast<unsigned long long>(iters) * 131072ull;
    }
    if (acc.x == 0x12345678u && acc.y == 0x9abcdef0u) out[2 * blockIdx.x + 1] += acc.z + acc.w;   // keeps the loads alive
}

}  // namespace infllmv2

using namespace infllmv2;

extern "C" int infllmv2_probe_stream(void* stream, const void* src, size_t src_bytes, unsigned long long* out,
                                     int workgroups, int iters, int mode) {
    IV2_CHECK(src && out && workgroups > 0 && iters > 0, "probe_stream: bad arguments");
    IV2_CHECK(mode >= 0 && mode <= 3, "probe_stream: mode must be 0 (global loads), 1 (LDS-DMA), 2 (LDS reads) or 3 (transposing LDS reads)");
    IV2_CHECK(src_bytes >= static_cast<size_t>(workgroups) * 131072 && reinterpret_cast<uintptr_t>(src) % 16 == 0,
              "probe_stream: the source must hold 128 KiB per workgroup, 16-byte aligned");
    hipStream_t st = static_cast<hipStream_t>(stream);
    const uint4* s = static_cast<const uint4*>(src);
    constexpr int kProbeLds = 131072;
    const void* fns[4] = {reinterpret_cast<const void*>(&probe_stream_kernel<0>), reinterpret_cast<const void*>(&probe_stream_kernel<1>),
                          reinterpret_cast<const void*>(&probe_stream_kernel<2>), reinterpret_cast<const void*>(&probe_stream_kernel<3>)};
    hipError_t e = hipFuncSetAttribute(fns[mode], hipFuncAttributeMaxDynamicSharedMemorySize, kProbeLds);
    IV2_CHECK(e == hipSuccess, "probe_stream: cannot reserve LDS: %s", hipGetErrorString(e));
    if (mode == 0) hipLaunchKernelGGL(probe_stream_kernel<0>, dim3(workgroups), dim3(512), kProbeLds, st, s, out, iters);
    else if (mode == 1) hipLaunchKernelGGL(probe_stream_kernel<1>, dim3(workgroups), dim3(512), kProbeLds, st, s, out, iters);
    else if (mode == 2) hipLaunchKernelGGL(probe_stream_kernel<2>, dim3(workgroups), dim3(512), kProbeLds, st, s, out, iters);
    else hipLaunchKernelGGL(probe_stream_kernel<3>, dim3(workgroups), dim3(512), kProbeLds, st, s, out, iters);
    IV2_LAUNCH_CHECK();
    return 0;
}
