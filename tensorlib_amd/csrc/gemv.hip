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
#include <atomic>
#include <cstring>

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
    // XMODE 3 only: the vector that is multiplied is rmsnorm(x + x2) * g
    const half8_t* x2;  // may be null (no addend)
    const half8_t* g;   // norm weight
    half8_t* sum_out;   // may be null; receives half(x + x2), written by workgroup 0
    float eps;
    // stamped build of the streaming kernel only: stamps[2 * workgroup] / [2 * workgroup + 1] receive the constant
    // 100 MHz counter (s_memrealtime) at the workgroup's first instruction and after its last store
    unsigned long long* stamps;
};

// The kernels take GemvArgs' fields as separate scalar parameters, not the struct: the first 16 dwords of scalar kernel
// arguments (x, W, y, N, K8, the block count and the batch strides) are then preloaded into SGPRs when a wavefront is
// launched (-mllvm -amdgpu-kernarg-preload-count=16; a struct passed by value is not), and a wavefront's first address
// does not wait for a scalar load from the argument buffer.  On firmware without the feature the same code runs
// through the compiler's compatibility prologue, which loads them.
#define TL_GEMV_PARAMS                                                                                                 \
    const half8_t *p_x, const half8_t *p_W, half_t *p_y, int p_N, int p_K8, int p_blocks, long p_sx8, long p_sw8,     \
        long p_sy, const half8_t *p_x2, const half8_t *p_g, half8_t *p_sum_out, float p_eps, unsigned long long *p_stamps
#define TL_GEMV_ARGS_FROM_PARAMS \
    const GemvArgs a { p_x, p_W, p_y, p_N, p_K8, p_blocks, p_sx8, p_sw8, p_sy, p_x2, p_g, p_sum_out, p_eps, p_stamps }
#define TL_GEMV_PASS(a) \
    (a).x, (a).W, (a).y, (a).N, (a).K8, (a).num_row_blocks, (a).sx8, (a).sw8, (a).sy, (a).x2, (a).g, (a).sum_out, (a).eps, (a).stamps
typedef void (*GemvKernel)(TL_GEMV_PARAMS);

// One wavefront per row group.  Dynamic LDS: K8 chunks of x (+ partial sums when KSPLIT > 1).
template <int WAVES, int ROWS, int UNROLL, int KSPLIT, bool NT>
__global__ void __launch_bounds__(WAVES * 64) gemv_f16_wave_kernel(TL_GEMV_PARAMS) {
    TL_GEMV_ARGS_FROM_PARAMS;
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

// Single-tile streaming kernel: the K segment of a wavefront fits one register tile
// (segment <= 64*UNROLL chunks), so the chunk a lane owns is fixed for the whole kernel, the
// matching piece of x is read once and kept in registers, and row blocks are double buffered:
// the loads of row block i+1 are in flight while block i is reduced.
//   XMODE 0: x goes global -> LDS (whole vector, once per workgroup) -> registers;
//            the first W tile is requested before the staging barrier.
//   XMODE 1: every wavefront reads its own K segment of x straight into registers.
//   XMODE 2: like 1, but x is silu(a) * b of a [a | b] input (the SwiGLU gate fused into the load).
//   XMODE 3: like 1, but x is rmsnorm(h + d) * g: every wavefront forms half(h + d) of its K segment,
//            the KSPLIT segment sums of squares meet in LDS (fixed order), and the normalised, weighted
//            vector is rounded to fp16 once, as the separate add + RMSNorm kernel would have stored it.
//            Workgroup 0 also writes half(h + d) out (the new residual stream).
// Dynamic LDS: [K8 chunks of x when XMODE == 0] + 2*RG*KSPLIT*ROWS floats when KSPLIT > 1
//              (+ WAVES floats when XMODE == 3).
// STAMP: measurement build (tl_gemv_f16_stamped): thread 0 of every workgroup records the time at its first
// instruction and after the workgroup's last store; otherwise the same instructions.
template <int WAVES, int ROWS, int UNROLL, int KSPLIT, int XMODE, bool STAMP = false>
__global__ void __launch_bounds__(WAVES * 64) gemv_f16_stream_kernel(TL_GEMV_PARAMS) {
    TL_GEMV_ARGS_FROM_PARAMS;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
    half8_t* xs = reinterpret_cast<half8_t*>(smem_raw);

    unsigned long long t_start = 0;
    if constexpr (STAMP) t_start = __builtin_amdgcn_s_memrealtime();
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int batch = blockIdx.y;
    const half8_t* __restrict__ x = a.x + (size_t)batch * a.sx8;
    const half8_t* __restrict__ W = a.W + (size_t)batch * a.sw8;
    half_t* __restrict__ y = a.y + (size_t)batch * a.sy;
    const int K8 = a.K8;
    const int N = a.N;

    constexpr int RG = WAVES / KSPLIT;
    const int kpart = wave % KSPLIT;
    const int rgrp = wave / KSPLIT;
    const int seg = (K8 + KSPLIT - 1) / KSPLIT;
    const int c0 = kpart * seg;
    const int c1 = (c0 + seg < K8) ? (c0 + seg) : K8;
    float* part = reinterpret_cast<float*>(xs + (XMODE == 0 ? K8 : 0));  // [2][RG][KSPLIT][ROWS]

    int cidx[UNROLL];
    bool ok[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
        cidx[u] = c0 + u * 64 + lane;
        ok[u] = cidx[u] < c1;
    }
    const half8_t zero8 = {0, 0, 0, 0, 0, 0, 0, 0};

    half8_t xv[UNROLL];
    if constexpr (XMODE == 1) {
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) xv[u] = ok[u] ? x[cidx[u]] : zero8;
    }
    if constexpr (XMODE == 2) {
        // x is given as [a | b] (2*K halves); the vector that is multiplied is silu(a) * b, computed in
        // fp32 and rounded to fp16 once, exactly what tl_silu_mul_f16 would have written to memory
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            const half8_t va = ok[u] ? x[cidx[u]] : zero8;
            const half8_t vb = ok[u] ? x[K8 + cidx[u]] : zero8;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const float a = (float)va[i];
                xv[u][i] = (half_t)(a * (1.0f / (1.0f + expf(-a))) * (float)vb[i]);
            }
        }
    }

    half8_t gv[XMODE == 3 ? UNROLL : 1];
    float ss = 0.f;
    if constexpr (XMODE == 3) {
        const half8_t* __restrict__ x2 = a.x2;
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            const half8_t va = ok[u] ? x[cidx[u]] : zero8;
            const half8_t vb = (ok[u] && x2) ? x2[cidx[u]] : zero8;
            gv[u] = ok[u] ? a.g[cidx[u]] : zero8;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const half_t h = (half_t)((float)va[i] + (float)vb[i]);
                xv[u][i] = h;
                ss = __builtin_fmaf((float)h, (float)h, ss);
            }
        }
    }

    half8_t cur[ROWS][UNROLL], nxt[ROWS][UNROLL];
    auto load_tile = [&](half8_t (&t)[ROWS][UNROLL], int rb) {
        const int row0 = (rb * RG + rgrp) * ROWS;
#pragma unroll
        for (int r = 0; r < ROWS; ++r) {
            int row = row0 + r;
            row = row < N ? row : N - 1;
            const half8_t* wr = W + (size_t)row * K8;
#pragma unroll
            for (int u = 0; u < UNROLL; ++u) t[r][u] = ok[u] ? __builtin_nontemporal_load(wr + cidx[u]) : zero8;
        }
    };

    int rb = blockIdx.x;
    if (rb < a.num_row_blocks) load_tile(cur, rb);

    if constexpr (XMODE == 0) {
        for (int c = tid; c < K8; c += WAVES * 64) xs[c] = x[c];
        __syncthreads();
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) xv[u] = xs[ok[u] ? cidx[u] : 0];
    }
    if constexpr (XMODE == 3) {
        // the first W tile is already in flight; finish the norm under its latency
        float* nrm = part + (KSPLIT > 1 ? 2 * RG * KSPLIT * ROWS : 0);
        ss = wave_sum(ss);
        if (lane == 0) nrm[wave] = ss;
        __syncthreads();
        float total = 0.f;
#pragma unroll
        for (int sgm = 0; sgm < KSPLIT; ++sgm) total += nrm[rgrp * KSPLIT + sgm];
        const float rs = 1.0f / sqrtf(total / (float)(K8 * 8) + a.eps);
        const bool writer = blockIdx.x == 0 && rgrp == 0 && a.sum_out != nullptr;
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            if (writer && ok[u]) a.sum_out[cidx[u]] = xv[u];
#pragma unroll
            for (int i = 0; i < 8; ++i) xv[u][i] = (half_t)((float)xv[u][i] * rs * (float)gv[u][i]);
        }
    }

    int it = 0;
    for (; rb < a.num_row_blocks; rb += gridDim.x, ++it) {
        const int nrb = rb + gridDim.x;
        const bool has_next = nrb < a.num_row_blocks;
        if (has_next) load_tile(nxt, nrb);

        float acc[ROWS];
#pragma unroll
        for (int r = 0; r < ROWS; ++r) {
            acc[r] = 0.f;
#pragma unroll
            for (int u = 0; u < UNROLL; ++u) acc[r] = dot8(cur[r][u], xv[u], acc[r]);
            acc[r] = wave_sum(acc[r]);
        }
        const int row0 = (rb * RG + rgrp) * ROWS;
        if constexpr (KSPLIT == 1) {
            if (lane < ROWS) {
                float v = acc[0];
#pragma unroll
                for (int r = 1; r < ROWS; ++r) v = (lane == r) ? acc[r] : v;
                if (row0 + lane < N) y[row0 + lane] = (half_t)v;
            }
        } else {
            float* p = part + (it & 1) * (RG * KSPLIT * ROWS);
            if (lane == 0) {
#pragma unroll
                for (int r = 0; r < ROWS; ++r) p[(rgrp * KSPLIT + kpart) * ROWS + r] = acc[r];
            }
            __syncthreads();
            if (kpart == 0 && lane < ROWS) {
                float v = 0.f;
#pragma unroll
                for (int s = 0; s < KSPLIT; ++s) v += p[(rgrp * KSPLIT + s) * ROWS + lane];
                if (row0 + lane < N) y[row0 + lane] = (half_t)v;
            }
        }
        if (has_next) {
#pragma unroll
            for (int r = 0; r < ROWS; ++r)
#pragma unroll
                for (int u = 0; u < UNROLL; ++u) cur[r][u] = nxt[r][u];
        }
    }
    if constexpr (STAMP) {
        __syncthreads();   // the wavefronts that wrote y have passed their stores
        if (tid == 0) {
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            a.stamps[2 * blockIdx.x] = t_start;
            a.stamps[2 * blockIdx.x + 1] = __builtin_amdgcn_s_memrealtime();
        }
    }
}

// Short rows (K8 < 64 chunks): LPR lanes per row, 64/LPR rows per wavefront pass; x read
// straight from global memory (it is at most 1 KiB).  Serves attention's q.K^T (K = 128).
template <int LPR>
__global__ void __launch_bounds__(256) gemv_f16_short_kernel(TL_GEMV_PARAMS) {
    TL_GEMV_ARGS_FROM_PARAMS;
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
    int xmode;  // -1: looping kernel (any K), 0/1: single-tile streaming kernel
    GemvKernel kernel;
};

#define TL_LOOP(W_, R_, U_, S_, NT_) \
    { "loop_w" #W_ "r" #R_ "u" #U_ "s" #S_ "nt" #NT_, W_, R_, U_, S_, -1, gemv_f16_wave_kernel<W_, R_, U_, S_, NT_> }
#define TL_STREAM(W_, R_, U_, S_, X_) \
    { "stream_w" #W_ "r" #R_ "u" #U_ "s" #S_ "x" #X_, W_, R_, U_, S_, X_, gemv_f16_stream_kernel<W_, R_, U_, S_, X_> }
#define TL_STREAM2(W_, R_, U_, S_) TL_STREAM(W_, R_, U_, S_, 0), TL_STREAM(W_, R_, U_, S_, 1)

static const GemvVariant g_variants[] = {
    {"auto", 0, 0, 0, 0, 0, nullptr},
    // looping kernel, x staged in LDS (any K)
    TL_LOOP(4, 2, 8, 1, true),    // 1
    TL_LOOP(4, 2, 6, 4, false),   // 2
    TL_LOOP(4, 2, 6, 4, true),    // 3   K > 12288
    TL_LOOP(8, 2, 6, 4, true),    // 4
    // K = 4096 (512 chunks per row): x in LDS (x0) against x in registers (x1)
    TL_STREAM2(4, 2, 2, 4),       // 5, 6    6 = dispatch for K <= 4096
    TL_STREAM2(4, 4, 2, 4),       // 7, 8
    TL_STREAM2(4, 2, 4, 2),       // 9, 10
    TL_STREAM2(4, 2, 8, 1),       // 11, 12
    TL_STREAM2(8, 2, 2, 4),       // 13, 14
    // K = 11008 (1376 chunks per row)
    TL_STREAM2(8, 2, 3, 8),       // 15, 16  16 = dispatch for K <= 12288
    TL_STREAM2(4, 2, 6, 4),       // 17, 18
    TL_STREAM2(8, 2, 6, 4),       // 19, 20
    TL_STREAM2(4, 2, 11, 2),      // 21, 22
    TL_STREAM(4, 2, 2, 4, 2),     // 23  silu*mul prologue, K <= 4096
    TL_STREAM(8, 2, 3, 8, 2),     // 24  silu*mul prologue, K <= 12288
    TL_STREAM(4, 2, 2, 4, 3),     // 25  add + RMSNorm prologue, K <= 4096
    TL_STREAM(8, 2, 3, 8, 3),     // 26  add + RMSNorm prologue, K <= 12288
};

static constexpr int kNumVariants = sizeof(g_variants) / sizeof(g_variants[0]);
static std::atomic<int> g_forced_variant{0};
static std::atomic<int> g_grid_waves_per_cu{0};  // 0 = automatic

static int variant_index(const char* name) {
    for (int i = 0; i < (int)(sizeof(g_variants) / sizeof(g_variants[0])); ++i)
        if (strcmp(g_variants[i].name, name) == 0) return i;
    return -1;
}

// Measured on MI355X (rotating weights, HBM resident) over the Llama2-7B decode shapes:
//   K <= 4096  : 4 wavefronts split K, 2 rows each, one row block per workgroup
//                (4096<-4096 7.1 us, 11008<-4096 14.6 us, 32000<-4096 37.2 us)
//   K <= 12288 : 8 wavefronts split K, 2 rows each, 16 wavefronts per CU, grid-stride
//                (4096<-11008 15.1 us)
//   otherwise  : looping kernel with x staged in LDS.
// In both streaming picks x goes straight to registers: each wavefront needs only its own K
// segment, and skipping the LDS round trip and its barrier was 0.2-1.2 us faster per launch
// than the LDS-staged twin of the same kernel.
static int pick_variant(size_t N, size_t K, int* waves_per_cu) {
    (void)N;
    static const int v_k4096 = variant_index("stream_w4r2u2s4x1");
    static const int v_k12288 = variant_index("stream_w8r2u3s8x1");
    static const int v_loop = variant_index("loop_w4r2u6s4nttrue");
    const size_t K8 = K / 8;
    if (K8 <= 512) { *waves_per_cu = 1 << 20; return v_k4096; }
    if (K8 <= 1536) { *waves_per_cu = 16; return v_k12288; }
    *waves_per_cu = 16;
    return v_loop;
}

int launch_gemv(const void* x, const void* W, void* y, size_t N, size_t K, size_t batch, size_t sx,
                size_t sw, size_t sy, int prologue, const GemvNormPrologue* norm) {
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
    a.x2 = norm ? (const half8_t*)norm->addend : nullptr;
    a.g = norm ? (const half8_t*)norm->weight : nullptr;
    a.sum_out = norm ? (half8_t*)norm->sum_out : nullptr;
    a.eps = norm ? norm->eps : 0.f;
    a.stamps = nullptr;

    const int forced_variant = g_forced_variant.load();
    if (a.K8 < 64 && forced_variant == 0) {
        int lpr = a.K8 >= 32 ? 32 : a.K8 >= 16 ? 16 : 8;
        int rows_per_block = 4 * (64 / lpr);
        a.num_row_blocks = (int)((N + rows_per_block - 1) / rows_per_block);
        int blocks = a.num_row_blocks;
        int cap = dev.cu_count * 16;
        if (blocks > cap) blocks = cap;
        dim3 grid(blocks, (unsigned)batch);
        if (lpr == 32)
            hipLaunchKernelGGL(gemv_f16_short_kernel<32>, grid, dim3(256), 0, st, TL_GEMV_PASS(a));
        else if (lpr == 16)
            hipLaunchKernelGGL(gemv_f16_short_kernel<16>, grid, dim3(256), 0, st, TL_GEMV_PASS(a));
        else
            hipLaunchKernelGGL(gemv_f16_short_kernel<8>, grid, dim3(256), 0, st, TL_GEMV_PASS(a));
        TL_CHECK_LAUNCH("gemv_f16_short_kernel");
        return TL_OK;
    }

    int auto_wpc = 16;
    int vi = forced_variant ? forced_variant : pick_variant(N, K, &auto_wpc);
    if (prologue == 1) {
        static const int v_k4096 = variant_index("stream_w4r2u2s4x2");
        static const int v_k12288 = variant_index("stream_w8r2u3s8x2");
        if (a.K8 <= 512) { vi = v_k4096; auto_wpc = 1 << 20; }
        else if (a.K8 <= 1536) { vi = v_k12288; auto_wpc = 16; }
        else return set_error(TL_ELIMIT, "gemv with fused silu*mul: K=%zu exceeds 12288", K);
    }
    if (prologue == 2) {
        static const int v_k4096 = variant_index("stream_w4r2u2s4x3");
        static const int v_k12288 = variant_index("stream_w8r2u3s8x3");
        TL_REQUIRE(norm && norm->weight && batch == 1, "gemv with fused add + RMSNorm: needs a norm weight, batch 1");
        // every workgroup repeats the prologue (3 vectors from L2), so the grid is capped and loops
        if (a.K8 <= 512) { vi = v_k4096; auto_wpc = 32; }
        else if (a.K8 <= 1536) { vi = v_k12288; auto_wpc = 16; }
        else return set_error(TL_ELIMIT, "gemv with fused add + RMSNorm: K=%zu exceeds 12288", K);
    }
    TL_REQUIRE(g_variants[vi].xmode != 3 || prologue == 2,
               "gemv variant %s cannot hold a plain x: it needs the add + RMSNorm operands", g_variants[vi].name);
    TL_REQUIRE(g_variants[vi].xmode != 2 || prologue == 1,
               "gemv variant %s cannot hold a plain x: it reads an [a | b] input of 2*K halves", g_variants[vi].name);
    if (g_variants[vi].xmode >= 0) {
        // the streaming kernel needs a wavefront's K segment to fit one register tile
        const GemvVariant& sv = g_variants[vi];
        const int seg = (a.K8 + sv.ksplit - 1) / sv.ksplit;
        if (seg > 64 * sv.unroll) {
            TL_REQUIRE(forced_variant == 0, "gemv variant %s cannot hold K=%zu (segment %d chunks > %d)", sv.name, K,
                       seg, 64 * sv.unroll);
            vi = variant_index("loop_w4r2u6s4nttrue");
        }
    }
    const GemvVariant& v = g_variants[vi];
    const int rg = v.waves / v.ksplit;
    const int rows_per_block = rg * v.rows;
    a.num_row_blocks = (int)((N + rows_per_block - 1) / rows_per_block);
    size_t lds = (v.xmode >= 1 ? 0 : (size_t)a.K8 * 16) +
                 (v.ksplit > 1 ? (size_t)(v.xmode >= 0 ? 2 : 1) * rg * v.ksplit * v.rows * 4 : 0) +
                 (v.xmode == 3 ? (size_t)v.waves * 4 : 0);
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
    const int forced_wpc = g_grid_waves_per_cu.load();
    int wpc = forced_wpc > 0 ? forced_wpc : auto_wpc;
    long cap = (long)dev.cu_count * wpc / v.waves;
    if (cap < 1) cap = 1;
    if (blocks > cap) blocks = (int)cap;
    hipLaunchKernelGGL(v.kernel, dim3(blocks, (unsigned)batch), dim3(v.waves * 64), lds, st, TL_GEMV_PASS(a));
    TL_CHECK_LAUNCH(v.name);
    return TL_OK;
}

}  // namespace tl

extern "C" {

int tl_gemv_f16(const void* x, const void* W, void* y, size_t N, size_t K) {
    TL_ENSURE_INIT();
    TL_REQUIRE(x && W && y, "tl_gemv_f16: null pointer");
    return tl::launch_gemv(x, W, y, N, K, 1, 0, 0, 0, 0);
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

// The dispatch's kernel for K <= 4096 (<4,2,2,4,1>, one row block per workgroup) in its stamped build.
extern "C" int tl_gemv_f16_stamped(const void* x, const void* W, void* y, size_t N, size_t K, void* stamps,
                                   size_t stamps_capacity, int* workgroups) {
    TL_ENSURE_INIT();
    TL_REQUIRE(x && W && y && stamps && workgroups, "tl_gemv_f16_stamped: null pointer");
    TL_REQUIRE(K % 8 == 0 && K >= 512 && K <= 4096 && tl::aligned16(x) && tl::aligned16(W) && N >= 1 && N <= 0x7fffffffu,
               "tl_gemv_f16_stamped: needs 512 <= K <= 4096, K %% 8 == 0 and 16-byte aligned operands");
    constexpr int WAVES = 4, ROWS = 2, KSPLIT = 4;
    tl::GemvArgs a{};
    a.x = (const tl::half8_t*)x;
    a.W = (const tl::half8_t*)W;
    a.y = (tl::half_t*)y;
    a.N = (int)N;
    a.K8 = (int)(K / 8);
    a.num_row_blocks = (int)((N + ROWS - 1) / ROWS);
    a.stamps = (unsigned long long*)stamps;
    TL_REQUIRE((size_t)a.num_row_blocks * 2 <= stamps_capacity, "tl_gemv_f16_stamped: %d workgroups need %d stamps, the buffer holds %zu",
               a.num_row_blocks, 2 * a.num_row_blocks, stamps_capacity);
    *workgroups = a.num_row_blocks;
    const size_t lds = (size_t)2 * (WAVES / KSPLIT) * KSPLIT * ROWS * 4;
    hipLaunchKernelGGL((tl::gemv_f16_stream_kernel<WAVES, ROWS, 2, KSPLIT, 1, true>), dim3(a.num_row_blocks), dim3(WAVES * 64), lds,
                       tl::stream(), TL_GEMV_PASS(a));
    TL_CHECK_LAUNCH("gemv_f16_stream_kernel<stamped>");
    return TL_OK;
}

extern "C" int tl_gemv_silu_mul_f16(const void* ab, const void* W, void* y, size_t N, size_t K) {
    TL_ENSURE_INIT();
    TL_REQUIRE(ab && W && y, "tl_gemv_silu_mul_f16: null pointer");
    TL_REQUIRE(K % 8 == 0 && tl::aligned16(ab) && tl::aligned16(W),
               "tl_gemv_silu_mul_f16: needs K %% 8 == 0 and 16-byte aligned operands");
    TL_REQUIRE(K / 8 >= 64, "tl_gemv_silu_mul_f16: K=%zu too short for the fused kernel (K >= 512)", K);
    return tl::launch_gemv(ab, W, y, N, K, 1, 0, 0, 0, 1);
}

extern "C" int tl_gemv_add_rms_norm_f16(const void* x, const void* addend, const void* norm_weight, float eps,
                                        const void* W, void* y, void* sum_out, size_t N, size_t K) {
    TL_ENSURE_INIT();
    TL_REQUIRE(x && norm_weight && W && y, "tl_gemv_add_rms_norm_f16: null pointer");
    TL_REQUIRE(K % 8 == 0 && tl::aligned16(x) && tl::aligned16(W) && tl::aligned16(norm_weight) &&
                   (!addend || tl::aligned16(addend)) && (!sum_out || tl::aligned16(sum_out)),
               "tl_gemv_add_rms_norm_f16: needs K %% 8 == 0 and 16-byte aligned operands");
    TL_REQUIRE(K / 8 >= 64, "tl_gemv_add_rms_norm_f16: K=%zu too short for the fused kernel (K >= 512)", K);
    TL_REQUIRE(!sum_out || (sum_out != x && sum_out != addend), "tl_gemv_add_rms_norm_f16: sum_out must not alias an input");
    tl::GemvNormPrologue np{addend, norm_weight, sum_out, eps};
    return tl::launch_gemv(x, W, y, N, K, 1, 0, 0, 0, 2, &np);
}
