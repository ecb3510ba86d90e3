// Measurement hook: the MFMA rate this chip sustains out of registers, with no memory traffic.
// bench.py places the HGEMM numbers against it next to the published peak, because the sustained
// rate depends on how much the operand bits toggle (the chip is power managed): constant operands
// run close to the published 2.5 PFLOP/s, operands that change with every instruction do not.
#include "tl_internal.h"

namespace tl {

constexpr int kChains = 8;  // independent accumulators per wavefront

// mode 0: the same operand registers for every instruction; mode 1: 8 pseudo-random operand pairs
// rotated so that both operands change with every instruction.
template <int MODE>
__global__ void __launch_bounds__(256) mfma_rate_kernel(float* out, int iters) {
    unsigned h = (threadIdx.x + blockIdx.x * 977u) * 2654435761u;
    half8_t av[kChains], bv[kChains];
#pragma unroll
    for (int j = 0; j < kChains; ++j)
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            h = h * 1664525u + 1013904223u;
            av[j][i] = (half_t)(((int)(h >> 16) % 2001 - 1000) * 0.001f);   // ~U(-1, 1)
            h = h * 1664525u + 1013904223u;
            bv[j][i] = (half_t)(((int)(h >> 16) % 2001 - 1000) * 0.00004f); // ~U(-0.04, 0.04)
        }
    float16_t acc[kChains];
#pragma unroll
    for (int j = 0; j < kChains; ++j)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[j][e] = 0.f;
    for (int it = 0; it < iters; it += kChains) {
#pragma unroll
        for (int r = 0; r < kChains; ++r)
#pragma unroll
            for (int j = 0; j < kChains; ++j) {
                if constexpr (MODE == 0)
                    acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(av[0], bv[0], acc[j], 0, 0, 0);
                else
                    acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(av[(j + 2 * r) % kChains], bv[(j + r) % kChains],
                                                                    acc[j], 0, 0, 0);
            }
    }
    float s = 0.f;
#pragma unroll
    for (int j = 0; j < kChains; ++j)
#pragma unroll
        for (int e = 0; e < 16; ++e) s += acc[j][e];
    out[blockIdx.x * 256 + threadIdx.x] = s;
}

// The same measurement with v_mfma_f32_16x16x32_f16 (mode 2: constant operands, mode 3: changing operands): half
// as many accumulator updates per flop as the 32x32x16 shape.  32 independent accumulators of four registers.
template <int MODE>
__global__ void __launch_bounds__(256) mfma_rate_16x16_kernel(float* out, int iters) {
    unsigned h = (threadIdx.x + blockIdx.x * 977u) * 2654435761u;
    half8_t av[kChains], bv[kChains];
#pragma unroll
    for (int j = 0; j < kChains; ++j)
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            h = h * 1664525u + 1013904223u;
            av[j][i] = (half_t)(((int)(h >> 16) % 2001 - 1000) * 0.001f);
            h = h * 1664525u + 1013904223u;
            bv[j][i] = (half_t)(((int)(h >> 16) % 2001 - 1000) * 0.00004f);
        }
    constexpr int kAcc = 32;
    float4_t acc[kAcc];
#pragma unroll
    for (int j = 0; j < kAcc; ++j) acc[j] = float4_t{0.f, 0.f, 0.f, 0.f};
    for (int it = 0; it < iters; it += kChains) {
#pragma unroll
        for (int r = 0; r < kChains; ++r)
#pragma unroll
            for (int j = 0; j < kAcc; ++j) {
                if constexpr (MODE == 0)
                    acc[j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(av[0], bv[0], acc[j], 0, 0, 0);
                else
                    acc[j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(av[(j + 2 * r) % kChains], bv[(j / 4 + r) % kChains],
                                                                    acc[j], 0, 0, 0);
            }
    }
    float s = 0.f;
#pragma unroll
    for (int j = 0; j < kAcc; ++j)
#pragma unroll
        for (int e = 0; e < 4; ++e) s += acc[j][e];
    out[blockIdx.x * 256 + threadIdx.x] = s;
}

}  // namespace tl

extern "C" int tl_measure_mfma_rate_f16(int mode, double* tflops) {
    TL_ENSURE_INIT();
    TL_REQUIRE(tflops != nullptr, "tl_measure_mfma_rate_f16: tflops is null");
    TL_REQUIRE(mode >= 0 && mode <= 3, "tl_measure_mfma_rate_f16: mode must be 0 .. 3");
    const int wgs = tl::device_info().cu_count * 4;
    const int iters = 8192;
    float* out = nullptr;
    TL_HIP_TRY(hipMalloc((void**)&out, (size_t)wgs * 256 * sizeof(float)));
    hipEvent_t e0, e1;
    TL_HIP_TRY(hipEventCreate(&e0));
    TL_HIP_TRY(hipEventCreate(&e1));
    hipStream_t st = tl::stream();
    float best_ms = 1e30f;
    for (int rep = 0; rep < 4; ++rep) {  // first repetition warms clocks up
        TL_HIP_TRY(hipEventRecord(e0, st));
        if (mode == 0)
            hipLaunchKernelGGL(tl::mfma_rate_kernel<0>, dim3(wgs), dim3(256), 0, st, out, iters);
        else if (mode == 1)
            hipLaunchKernelGGL(tl::mfma_rate_kernel<1>, dim3(wgs), dim3(256), 0, st, out, iters);
        else if (mode == 2)
            hipLaunchKernelGGL(tl::mfma_rate_16x16_kernel<0>, dim3(wgs), dim3(256), 0, st, out, iters);
        else
            hipLaunchKernelGGL(tl::mfma_rate_16x16_kernel<1>, dim3(wgs), dim3(256), 0, st, out, iters);
        TL_HIP_TRY(hipEventRecord(e1, st));
        TL_HIP_TRY(hipEventSynchronize(e1));
        float ms = 0.f;
        TL_HIP_TRY(hipEventElapsedTime(&ms, e0, e1));
        if (rep > 0 && ms < best_ms) best_ms = ms;
    }
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    TL_HIP_TRY(hipFree(out));
    // 4 wavefronts per workgroup; per iteration step kChains MFMAs of 2*32*32*16 flops or 32 of 2*16*16*32
    const double flops = (double)wgs * 4.0 * iters * (mode < 2 ? tl::kChains * 32768.0 : 32 * 16384.0);
    *tflops = flops / (best_ms * 1e-3) / 1e12;
    return TL_OK;
}
