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

// Issue probes: what the arithmetic of one attention block costs when no memory instruction competes.  Two wavefronts
// per SIMD (a workgroup of 8 per CU, held to one per CU by its LDS request), operands in registers, `iters` rounds.
//  mode 0: 8 independent MFMA per round          mode 1: 32 fp32 multiply-adds          mode 2: 8 exp2
//  mode 3: 8 x (MFMA, 2 multiply-adds)           mode 4: 8 x (MFMA, 4 multiply-adds)
//  mode 5: one block as the forward kernel issues it: 16 S MFMA, 16 x (multiply-add, exp2, add), 8 conversions,
//          16 P.V MFMA                           mode 6: the same with a wavefront-uniform branch on the row sum
//          between the additions and the conversions
// out[workgroup] = cycle-counter ticks.
template <int kMode>
__global__ __launch_bounds__(512)
void probe_issue_kernel(unsigned long long* __restrict__ out, int iters, float scale, float limit) {
    extern __shared__ uint4 lds[];
    const int tid = threadIdx.x;
    floatx4 acc[8];
    float x[8];
    elem8 a, b;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        acc[j] = floatx4{0.f, 0.f, 0.f, 0.f};
        x[j] = tid * 1e-3f + j;
        a[j] = static_cast<elem_t>(tid * 1e-3f);
        b[j] = static_cast<elem_t>(j * 0.5f);
    }
    float l = 0.f;
    const unsigned long long t0 = __builtin_readcyclecounter();
    if (kMode <= 4) {
        constexpr int kMfma = (kMode == 0 || kMode >= 3) ? 8 : 0;
        constexpr int kValu = kMode == 1 ? 4 : kMode == 2 ? 1 : kMode == 3 ? 2 : kMode == 4 ? 4 : 0;
        for (int i = 0; i < iters; ++i) {
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                if (j < kMfma) acc[j] = IV2_MFMA(a, b, acc[j], 0, 0, 0);
#pragma unroll
                for (int r = 0; r < kValu; ++r) {
                    float& v = x[(j + r) & 7];
                    if (kMode == 2) v = __builtin_amdgcn_exp2f(v);
                    else v = __builtin_fmaf(v, scale, scale);
                    asm volatile("" : "+v"(v));                // one instruction each: no folding of the chain
                }
            }
        }
    } else {
        elem8 kf[16], vf[16], qf[4];
#pragma unroll
        for (int f = 0; f < 16; ++f)
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                kf[f][j] = static_cast<elem_t>(tid * 1e-3f + f);
                vf[f][j] = static_cast<elem_t>(j * 0.25f + f);
            }
#pragma unroll
        for (int c = 0; c < 4; ++c)
#pragma unroll
            for (int j = 0; j < 8; ++j) qf[c][j] = static_cast<elem_t>(tid * 2e-3f + c);
        for (int i = 0; i < iters; ++i) {
#pragma unroll
            for (int f = 0; f < 16; ++f) {                     // "fresh" operands every round
                asm volatile("" : "+v"(kf[f]));
                asm volatile("" : "+v"(vf[f]));
            }
            floatx4 s[4];
#pragma unroll
            for (int kt = 0; kt < 4; ++kt) s[kt] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int c = 0; c < 4; ++c)
#pragma unroll
                for (int kt = 0; kt < 4; ++kt) s[kt] = IV2_MFMA(kf[kt * 4 + c], qf[c], s[kt], 0, 0, 0);
            floatx4 pv[4];
            float rs = 0.f;
#pragma unroll
            for (int kt = 0; kt < 4; ++kt)
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    pv[kt][e] = __builtin_amdgcn_exp2f(__builtin_fmaf(s[kt][e], scale, -1.f));
                    rs += pv[kt][e];
                }
            if (kMode == 6 && __ballot(!(rs <= limit)) != 0ull) {   // never taken with the values used here
#pragma unroll
                for (int dt = 0; dt < 8; ++dt) acc[dt] *= scale;
            }
            l += rs;
            elem8 pf[2];
#pragma unroll
            for (int cc = 0; cc < 2; ++cc)
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    pf[cc][e] = static_cast<elem_t>(pv[2 * cc][e]);
                    pf[cc][4 + e] = static_cast<elem_t>(pv[2 * cc + 1][e]);
                }
#pragma unroll
            for (int cc = 0; cc < 2; ++cc)
#pragma unroll
                for (int dt = 0; dt < 8; ++dt) acc[dt] = IV2_MFMA(vf[dt * 2 + cc], pf[cc], acc[dt], 0, 0, 0);
        }
    }
    const unsigned long long t1 = __builtin_readcyclecounter();
    float t = l;
#pragma unroll
    for (int j = 0; j < 8; ++j) t += acc[j][0] + acc[j][1] + acc[j][2] + acc[j][3] + x[j];
    if (tid == 0) out[blockIdx.x] = t1 - t0;
    if (t == 123.456f) out[blockIdx.x] += lds[tid].x;          // keeps the arithmetic alive
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

extern "C" int infllmv2_probe_issue(void* stream, unsigned long long* out, int workgroups, int iters, int mode) {
    IV2_CHECK(out && workgroups > 0 && iters > 0, "probe_issue: bad arguments");
    IV2_CHECK(mode >= 0 && mode <= 6, "probe_issue: mode must be 0..6");
    hipStream_t st = static_cast<hipStream_t>(stream);
    constexpr int kIssueLds = 100 * 1024;                      // more than half a CU's LDS: one workgroup per CU
    const void* fns[7] = {reinterpret_cast<const void*>(&probe_issue_kernel<0>), reinterpret_cast<const void*>(&probe_issue_kernel<1>),
                          reinterpret_cast<const void*>(&probe_issue_kernel<2>), reinterpret_cast<const void*>(&probe_issue_kernel<3>),
                          reinterpret_cast<const void*>(&probe_issue_kernel<4>), reinterpret_cast<const void*>(&probe_issue_kernel<5>),
                          reinterpret_cast<const void*>(&probe_issue_kernel<6>)};
    hipError_t e = hipFuncSetAttribute(fns[mode], hipFuncAttributeMaxDynamicSharedMemorySize, kIssueLds);
    IV2_CHECK(e == hipSuccess, "probe_issue: cannot reserve LDS: %s", hipGetErrorString(e));
    const float scale = 0.01f, limit = 64.f;
    switch (mode) {
        case 0: hipLaunchKernelGGL(probe_issue_kernel<0>, dim3(workgroups), dim3(512), kIssueLds, st, out, iters, scale, limit); break;
        case 1: hipLaunchKernelGGL(probe_issue_kernel<1>, dim3(workgroups), dim3(512), kIssueLds, st, out, iters, scale, limit); break;
        case 2: hipLaunchKernelGGL(probe_issue_kernel<2>, dim3(workgroups), dim3(512), kIssueLds, st, out, iters, scale, limit); break;
        case 3: hipLaunchKernelGGL(probe_issue_kernel<3>, dim3(workgroups), dim3(512), kIssueLds, st, out, iters, scale, limit); break;
        case 4: hipLaunchKernelGGL(probe_issue_kernel<4>, dim3(workgroups), dim3(512), kIssueLds, st, out, iters, scale, limit); break;
        case 5: hipLaunchKernelGGL(probe_issue_kernel<5>, dim3(workgroups), dim3(512), kIssueLds, st, out, iters, scale, limit); break;
        default: hipLaunchKernelGGL(probe_issue_kernel<6>, dim3(workgroups), dim3(512), kIssueLds, st, out, iters, scale, limit); break;
    }
    IV2_LAUNCH_CHECK();
    return 0;
}
