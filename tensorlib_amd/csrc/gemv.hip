// fp16 GEMV for gfx950: y[N] = W[N,K] . x[K], fp32 accumulation, one rounding to fp16.
//
// Replaces gemv_v6 / gemv_v4 of the reference (tensorLib/src/device/cuda/gemv.cu:379-450,
// :260-300) behind Device<half>::matmul2d with M == 1 (tensorLib/src/device/cuda/gemm.cu:153-162).
//
// Design (HBM-bound, 2 bytes of W per multiply-add, every byte of W read exactly once):
//   * x is staged once per workgroup in LDS and read back with ds_read_b128;
//   * one 64-lane wavefront streams ROWS rows of W at a time with 16-byte loads, UNROLL
//     loads per row in flight per lane, so a wavefront keeps ROWS*UNROLL KiB outstanding;
//   * KSPLIT wavefronts of a workgroup may share a row group and split K between them
//     (used for the 11008-wide down-projection); partial sums meet in LDS, in a fixed order;
//   * the 64 partial sums of a wavefront are combined with DPP row operations and
//     four v_readlane, no LDS traffic.
#include "tl_internal.h"

namespace tl {

// ------------------------------------------------------------------ device helpers ----

__device__ __forceinline__ float dot8(const half8_t w, const half8_t x, float acc) {
#pragma unroll
    for (int i = 0; i < 8; ++i) acc = __builtin_fmaf((float)w[i], (float)x[i], acc);
    return acc;
}

template <int CTRL>
__device__ __forceinline__ float dpp_add(float v) {
    int t = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true);
    return v + __builtin_bit_cast(float, t);
}

// Sum over the 16 lanes of each DPP row; every lane of the row ends up with the row's sum.
__device__ __forceinline__ float row16_sum(float v) {
    v = dpp_add<0xB1>(v);   // quad_perm [1,0,3,2]
    v = dpp_add<0x4E>(v);   // quad_perm [2,3,0,1]
    v = dpp_add<0x141>(v);  // row_half_mirror
    v = dpp_add<0x140>(v);  // row_mirror
    return v;
}

// Sum over all 64 lanes, result uniform across the wavefront.
__device__ __forceinline__ float wave_sum(float v) {
    v = row16_sum(v);
    int b = __builtin_bit_cast(int, v);
    float s0 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 0));
    float s1 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 16));
    float s2 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 32));
    float s3 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 48));
    return (s0 + s1) + (s2 + s3);
}

// Sum over groups of LPR adjacent lanes (LPR in {8,16,32,64}).
template <int LPR>
__device__ __forceinline__ float group_sum(float v) {
    if constexpr (LPR == 64) {
        return wave_sum(v);
    } else if constexpr (LPR == 32) {
        v = row16_sum(v);
        return v + __shfl_xor(v, 16, 64);
    } else if constexpr (LPR == 16) {
        return row16_sum(v);
    } else {
        static_assert(LPR == 8, "unsupported lanes-per-row");
        v = dpp_add<0xB1>(v);
        v = dpp_add<0x4E>(v);
        v = dpp_add<0x141>(v);
        return v;
    }
}

template <bool NT>
__device__ __forceinline__ half8_t load16(const half8_t* p) {
    if constexpr (NT) {
        return __builtin_nontemporal_load(p);
    } else {
        return *p;
    }
}

// ------------------------------------------------------------------------ kernels ----

struct GemvArgs {
    const half8_t* x;
    const half8_t* W;
    half_t* y;
    int N;
    int K8;             // 16-byte chunks per row (K / 8)
    int num_row_blocks; // ceil(N / rows per workgroup pass)
    long sx8, sw8, sy;  // batch strides: x and W in 16-byte chunks, y in elements
};

// One wavefront per row group.  Dynamic LDS: K8 chunks of x (+ partial sums when KSPLIT > 1).
template <int WAVES, int ROWS, int UNROLL, int KSPLIT, bool NT>
__global__ void __launch_bounds__(WAVES * 64) gemv_f16_wave_kernel(GemvArgs a) {
    extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
    half8_t* xs = reinterpret_cast<half8_t*>(smem_raw);

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int batch = blockIdx.y;
    const half8_t* __restrict__ x = a.x + (size_t)batch * a.sx8;
    const half8_t* __restrict__ W = a.W + (size_t)batch * a.sw8;
    half_t* __restrict__ y = a.y + (size_t)batch * a.sy;
    const int K8 = a.K8;
    const int N = a.N;

    for (int c = tid; c < K8; c += WAVES * 64) xs[c] = x[c];
    __syncthreads();

    constexpr int RG = WAVES / KSPLIT;  // row groups a workgroup works on at once
    const int kpart = wave % KSPLIT;
    const int rgrp = wave / KSPLIT;
    const int seg = (K8 + KSPLIT - 1) / KSPLIT;
    const int c0 = kpart * seg;
    const int c1 = (c0 + seg < K8) ? (c0 + seg) : K8;

    float* part = reinterpret_cast<float*>(xs + K8);  // [RG][KSPLIT][ROWS], only if KSPLIT > 1

    for (int rb = blockIdx.x; rb < a.num_row_blocks; rb += gridDim.x) {
        const int row0 = (rb * RG + rgrp) * ROWS;
        const half8_t* wrow[ROWS];
#pragma unroll
        for (int r = 0; r < ROWS; ++r) {
            int row = row0 + r;
            row = row < N ? row : N - 1;  // clamp: rows past the end re-read the last row, result dropped
            wrow[r] = W + (size_t)row * K8;
        }
        float acc[ROWS];
#pragma unroll
        for (int r = 0; r < ROWS; ++r) acc[r] = 0.f;

        for (int cb = c0; cb < c1; cb += 64 * UNROLL) {
            half8_t w[ROWS][UNROLL];
            half8_t xv[UNROLL];
#pragma unroll
            for (int u = 0; u < UNROLL; ++u) {
                const int c = cb + u * 64 + lane;
                if (c < c1) {
#pragma unroll
                    for (int r = 0; r < ROWS; ++r) w[r][u] = load16<NT>(wrow[r] + c);
                } else {
#pragma unroll
                    for (int r = 0; r < ROWS; ++r) w[r][u] = half8_t{0, 0, 0, 0, 0, 0, 0, 0};
                }
            }
#pragma unroll
            for (int u = 0; u < UNROLL; ++u) {
                const int c = cb + u * 64 + lane;
                xv[u] = xs[c < c1 ? c : c1 - 1];
            }
#pragma unroll
            for (int u = 0; u < UNROLL; ++u)
#pragma unroll
                for (int r = 0; r < ROWS; ++r) acc[r] = dot8(w[r][u], xv[u], acc[r]);
        }

#pragma unroll
        for (int r = 0; r < ROWS; ++r) acc[r] = wave_sum(acc[r]);

        if constexpr (KSPLIT == 1) {
            if (lane < ROWS) {
                float v = acc[0];
#pragma unroll
                for (int r = 1; r < ROWS; ++r) v = (lane == r) ? acc[r] : v;
                if (row0 + lane < N) y[row0 + lane] = (half_t)v;
            }
        } else {
            if (lane == 0) {
#pragma unroll
                for (int r = 0; r < ROWS; ++r) part[(rgrp * KSPLIT + kpart) * ROWS + r] = acc[r];
            }
            __syncthreads();
            if (kpart == 0 && lane < ROWS) {
                float v = 0.f;
#pragma unroll
                for (int s = 0; s < KSPLIT; ++s) v += part[(rgrp * KSPLIT + s) * ROWS + lane];
                if (row0 + lane < N) y[row0 + lane] = (half_t)v;
            }
            __syncthreads();
        }
    }
}

// Short rows (K8 < 64 chunks): LPR lanes per row, 64/LPR rows per wavefront pass; x read
// straight from global memory (it is at most 1 KiB).  Serves attention's q.K^T (K = 128).
template <int LPR>
__global__ void __launch_bounds__(256) gemv_f16_short_kernel(GemvArgs a) {
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int batch = blockIdx.y;
    const half8_t* __restrict__ x = a.x + (size_t)batch * a.sx8;
    const half8_t* __restrict__ W = a.W + (size_t)batch * a.sw8;
    half_t* __restrict__ y = a.y + (size_t)batch * a.sy;
    constexpr int RPW = 64 / LPR;  // rows per wavefront pass
    const int sub = lane % LPR;
    const int rsub = lane / LPR;
    const int K8 = a.K8;
    for (int rb = blockIdx.x; rb < a.num_row_blocks; rb += gridDim.x) {
        const int row = (rb * 4 + wave) * RPW + rsub;
        const int rowc = row < a.N ? row : a.N - 1;
        const half8_t* wr = W + (size_t)rowc * K8;
        float acc = 0.f;
        for (int c = sub; c < K8; c += LPR) acc = dot8(wr[c], x[c], acc);
        acc = group_sum<LPR>(acc);
        if (sub == 0 && row < a.N) y[row] = (half_t)acc;
    }
}

// Any K, any alignment: one wavefront per row, 2-byte loads (the shape of the reference's
// gemv_v4, tensorLib/src/device/cuda/gemv.cu:260-300).
__global__ void __launch_bounds__(256)
gemv_f16_generic_kernel(const half_t* __restrict__ x0, const half_t* __restrict__ W0, half_t* __restrict__ y0,
                        int N, int K, long sx, long sw, long sy) {
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int batch = blockIdx.y;
    const half_t* x = x0 + (size_t)batch * sx;
    const half_t* W = W0 + (size_t)batch * sw;
    half_t* y = y0 + (size_t)batch * sy;
    for (int row = blockIdx.x * 4 + wave; row < N; row += gridDim.x * 4) {
        const half_t* wr = W + (size_t)row * K;
        float acc = 0.f;
        for (int k = lane; k < K; k += 64) acc = __builtin_fmaf((float)wr[k], (float)x[k], acc);
        acc = wave_sum(acc);
        if (lane == 0) y[row] = (half_t)acc;
    }
}

// ---------------------------------------------------------------------- dispatch ----

struct GemvVariant {
    const char* name;
    int waves, rows, unroll, ksplit;
    void (*kernel)(GemvArgs);
};

static const GemvVariant g_variants[] = {
    {"auto", 0, 0, 0, 0, nullptr},
    {"w4r2u4s1", 4, 2, 4, 1, gemv_f16_wave_kernel<4, 2, 4, 1, false>},     // 1
    {"w4r2u8s1", 4, 2, 8, 1, gemv_f16_wave_kernel<4, 2, 8, 1, false>},     // 2
    {"w4r4u8s1", 4, 4, 8, 1, gemv_f16_wave_kernel<4, 4, 8, 1, false>},     // 3
    {"w4r1u8s1", 4, 1, 8, 1, gemv_f16_wave_kernel<4, 1, 8, 1, false>},     // 4
    {"w4r4u4s1", 4, 4, 4, 1, gemv_f16_wave_kernel<4, 4, 4, 1, false>},     // 5
    {"w8r2u8s1", 8, 2, 8, 1, gemv_f16_wave_kernel<8, 2, 8, 1, false>},     // 6
    {"w4r2u4s2", 4, 2, 4, 2, gemv_f16_wave_kernel<4, 2, 4, 2, false>},     // 7
    {"w4r2u6s4", 4, 2, 6, 4, gemv_f16_wave_kernel<4, 2, 6, 4, false>},     // 8
    {"w4r4u6s4", 4, 4, 6, 4, gemv_f16_wave_kernel<4, 4, 6, 4, false>},     // 9
    {"w8r2u6s4", 8, 2, 6, 4, gemv_f16_wave_kernel<8, 2, 6, 4, false>},     // 10
    {"w4r2u11s2", 4, 2, 11, 2, gemv_f16_wave_kernel<4, 2, 11, 2, false>},  // 11
    {"w4r2u8s1nt", 4, 2, 8, 1, gemv_f16_wave_kernel<4, 2, 8, 1, true>},    // 12
    {"w4r4u8s1nt", 4, 4, 8, 1, gemv_f16_wave_kernel<4, 4, 8, 1, true>},    // 13
    {"w4r2u6s4nt", 4, 2, 6, 4, gemv_f16_wave_kernel<4, 2, 6, 4, true>},    // 14
    {"w8r4u8s1", 8, 4, 8, 1, gemv_f16_wave_kernel<8, 4, 8, 1, false>},     // 15
    {"w16r2u8s1", 16, 2, 8, 1, gemv_f16_wave_kernel<16, 2, 8, 1, false>},  // 16
};
static constexpr int kNumVariants = sizeof(g_variants) / sizeof(g_variants[0]);
static int g_forced_variant = 0;
static int g_grid_waves_per_cu = 0;  // 0 = automatic

static int pick_variant(size_t N, size_t K) {
    // Down-projection shape (long rows, few of them): split K across the workgroup.
    if (K >= 8192 && N <= 8192) return 8;
    if (N >= 16384) return 3;
    return 2;
}

int launch_gemv(const void* x, const void* W, void* y, size_t N, size_t K, size_t batch, size_t sx,
                size_t sw, size_t sy) {
    if (N == 0 || batch == 0) return TL_OK;
    TL_REQUIRE(N <= 0x7fffffffu && K <= 0x7fffffffu && batch <= 65535, "gemv: size out of range");
    const DeviceInfo& dev = device_info();
    hipStream_t st = stream();
    if (K == 0) {
        for (size_t b = 0; b < batch; ++b) {
            int rc = launch_fill_f16((half_t*)y + b * sy, 0, N);
            if (rc != TL_OK) return rc;
        }
        return TL_OK;
    }
    const bool vec_ok = (K % 8 == 0) && aligned16(x) && aligned16(W) &&
                        (batch == 1 || (sx % 8 == 0 && sw % 8 == 0));
    if (!vec_ok) {
        int blocks = (int)((N + 3) / 4);
        int cap = dev.cu_count * 16;
        if (blocks > cap) blocks = cap;
        hipLaunchKernelGGL(gemv_f16_generic_kernel, dim3(blocks, (unsigned)batch), dim3(256), 0, st,
                           (const half_t*)x, (const half_t*)W, (half_t*)y, (int)N, (int)K, (long)sx,
                           (long)sw, (long)sy);
        TL_CHECK_LAUNCH("gemv_f16_generic_kernel");
        return TL_OK;
    }
    GemvArgs a;
    a.x = (const half8_t*)x;
    a.W = (const half8_t*)W;
    a.y = (half_t*)y;
    a.N = (int)N;
    a.K8 = (int)(K / 8);
    a.sx8 = (long)(sx / 8);
    a.sw8 = (long)(sw / 8);
    a.sy = (long)sy;

    if (a.K8 < 64 && g_forced_variant == 0) {
        int lpr = a.K8 >= 32 ? 32 : a.K8 >= 16 ? 16 : 8;
        int rows_per_block = 4 * (64 / lpr);
        a.num_row_blocks = (int)((N + rows_per_block - 1) / rows_per_block);
        int blocks = a.num_row_blocks;
        int cap = dev.cu_count * 16;
        if (blocks > cap) blocks = cap;
        dim3 grid(blocks, (unsigned)batch);
        if (lpr == 32)
            hipLaunchKernelGGL(gemv_f16_short_kernel<32>, grid, dim3(256), 0, st, a);
        else if (lpr == 16)
            hipLaunchKernelGGL(gemv_f16_short_kernel<16>, grid, dim3(256), 0, st, a);
        else
            hipLaunchKernelGGL(gemv_f16_short_kernel<8>, grid, dim3(256), 0, st, a);
        TL_CHECK_LAUNCH("gemv_f16_short_kernel");
        return TL_OK;
    }

    int vi = g_forced_variant ? g_forced_variant : pick_variant(N, K);
    const GemvVariant& v = g_variants[vi];
    const int rg = v.waves / v.ksplit;
    const int rows_per_block = rg * v.rows;
    a.num_row_blocks = (int)((N + rows_per_block - 1) / rows_per_block);
    size_t lds = (size_t)a.K8 * 16 + (v.ksplit > 1 ? (size_t)rg * v.ksplit * v.rows * 4 : 0);
    if (lds > 64 * 1024) {
        // x does not fit the default LDS window: fall back to the generic kernel.
        int blocks = (int)((N + 3) / 4);
        int cap = dev.cu_count * 16;
        if (blocks > cap) blocks = cap;
        hipLaunchKernelGGL(gemv_f16_generic_kernel, dim3(blocks, (unsigned)batch), dim3(256), 0, st,
                           (const half_t*)x, (const half_t*)W, (half_t*)y, (int)N, (int)K, (long)sx,
                           (long)sw, (long)sy);
        TL_CHECK_LAUNCH("gemv_f16_generic_kernel");
        return TL_OK;
    }
    int blocks = a.num_row_blocks;
    int wpc = g_grid_waves_per_cu > 0 ? g_grid_waves_per_cu : 32;
    int cap = dev.cu_count * wpc / v.waves;
    if (cap < 1) cap = 1;
    if (blocks > cap) blocks = cap;
    hipLaunchKernelGGL(v.kernel, dim3(blocks, (unsigned)batch), dim3(v.waves * 64), lds, st, a);
    TL_CHECK_LAUNCH(v.name);
    return TL_OK;
}

}  // namespace tl

extern "C" {

int tl_gemv_f16(const void* x, const void* W, void* y, size_t N, size_t K) {
    TL_ENSURE_INIT();
    TL_REQUIRE(x && W && y, "tl_gemv_f16: null pointer");
    return tl::launch_gemv(x, W, y, N, K, 1, 0, 0, 0);
}

int tl_set_gemv_variant(int variant) {
    TL_REQUIRE(variant >= 0 && variant < tl::kNumVariants, "tl_set_gemv_variant: %d out of range [0,%d)",
               variant, tl::kNumVariants);
    tl::g_forced_variant = variant;
    return TL_OK;
}

const char* tl_gemv_variant_name(int variant) {
    if (variant < 0 || variant >= tl::kNumVariants) return nullptr;
    return tl::g_variants[variant].name;
}

int tl_set_gemv_grid_waves_per_cu(int waves) {
    tl::g_grid_waves_per_cu = waves;
    return TL_OK;
}

}  // extern "C"
