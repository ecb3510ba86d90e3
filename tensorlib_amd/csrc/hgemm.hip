// fp16 GEMM for gfx950 on the matrix cores: C[M,N] = A[M,K] . B[N,K]^T, fp32 accumulation
// in MFMA accumulators, one rounding to fp16 in the epilogue.
//
// Replaces hgemm_cublas (tensorLib/src/device/cuda/hgemm.cu:20-38) behind
// Device<half>::matmul2d with M > 1 (tensorLib/src/device/cuda/gemm.cu:163-171); numerics
// follow CPU<half>::matmul2d (tensorLib/src/device/cpu/CPU.cpp:76-89).
//
// Both operands are K-contiguous, which is exactly the register layout of
// v_mfma_f32_32x32x16_f16: lane l supplies 8 consecutive k values of row (l % 32), the two
// half-wavefronts supply k 0..7 and 8..15.  So a 16-byte global load, a 16-byte LDS write
// and a 16-byte LDS read move an operand fragment without any shuffling.
//
// Tiling: a workgroup of WM x WN wavefronts owns a BM x BN tile of C and walks K in steps
// of BK.  Tiles of A and B are staged in LDS rows of BK+8 halves (the 16-byte pad makes the
// 32 rows a ds_read_b128 touches fall in distinct bank groups), double buffered: while the
// MFMAs of step k run out of one buffer, the global loads of step k+1 are in flight in
// registers and are written to the other buffer before the single barrier of the step.
#include "tl_internal.h"

namespace tl {

struct HgemmArgs {
    const half_t* A;
    const half_t* B;
    half_t* C;
    int M, N, K;
    int tiles_m, tiles_n;
    long sa, sb, sc;  // batch strides in elements
};

constexpr int kPad = 8;  // halves of padding per LDS row

// Map the linear workgroup id to a tile so that workgroups resident on one XCD (ids
// congruent mod 8 are dispatched to the same XCD) work on neighbouring tiles that share a
// panel of B, and panels of B are walked once.
__device__ __forceinline__ void tile_of_block(int bid, int nblocks, int tiles_m, int& tm, int& tn) {
    int lid = bid;
    if ((nblocks & 7) == 0) {
        const int per_xcd = nblocks >> 3;
        lid = (bid & 7) * per_xcd + (bid >> 3);
    }
    tm = lid % tiles_m;
    tn = lid / tiles_m;
}

template <int BM, int BN, int BK, int WM, int WN>
__global__ void __launch_bounds__(WM* WN * 64) hgemm_f16_mfma_kernel(HgemmArgs a) {
    constexpr int THREADS = WM * WN * 64;
    constexpr int LDS_ROW = BK + kPad;          // halves
    constexpr int CPR = BK / 8;                 // 16-byte chunks per tile row
    constexpr int A_CHUNKS = BM * CPR / THREADS;  // per thread
    constexpr int B_CHUNKS = BN * CPR / THREADS;
    constexpr int ROWS_PER_PASS = THREADS / CPR;
    constexpr int TM = BM / WM, TN = BN / WN;   // wavefront tile
    constexpr int MT = TM / 32, NT = TN / 32;   // 32x32 MFMA tiles per wavefront
    static_assert(BM * CPR % THREADS == 0 && BN * CPR % THREADS == 0, "tile/threads mismatch");
    static_assert(TM % 32 == 0 && TN % 32 == 0 && BK % 16 == 0, "wave tile must be MFMA multiples");

    extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
    half_t* As = reinterpret_cast<half_t*>(smem_raw);          // [2][BM][LDS_ROW]
    half_t* Bs = As + 2 * BM * LDS_ROW;                        // [2][BN][LDS_ROW]

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wm = wave / WN, wn = wave % WN;

    int tile_m, tile_n;
    tile_of_block(blockIdx.x, gridDim.x, a.tiles_m, tile_m, tile_n);
    const int m0 = tile_m * BM, n0 = tile_n * BN;
    const int batch = blockIdx.y;
    const half_t* __restrict__ A = a.A + (size_t)batch * a.sa;
    const half_t* __restrict__ B = a.B + (size_t)batch * a.sb;
    half_t* __restrict__ C = a.C + (size_t)batch * a.sc;
    const int M = a.M, N = a.N, K = a.K;

    // global -> register staging assignment: chunk (tid % CPR) of rows (tid / CPR) + i*ROWS_PER_PASS
    const int ld_chunk = tid % CPR;
    const int ld_row = tid / CPR;
    const half_t* a_ptr[A_CHUNKS];
    const half_t* b_ptr[B_CHUNKS];
#pragma unroll
    for (int i = 0; i < A_CHUNKS; ++i) {
        int r = m0 + ld_row + i * ROWS_PER_PASS;
        r = r < M ? r : M - 1;
        a_ptr[i] = A + (size_t)r * K + ld_chunk * 8;
    }
#pragma unroll
    for (int i = 0; i < B_CHUNKS; ++i) {
        int r = n0 + ld_row + i * ROWS_PER_PASS;
        r = r < N ? r : N - 1;
        b_ptr[i] = B + (size_t)r * K + ld_chunk * 8;
    }

    half8_t a_reg[A_CHUNKS], b_reg[B_CHUNKS];
    const half8_t zero8 = {0, 0, 0, 0, 0, 0, 0, 0};

    auto load_global = [&](int kt) {
        const int k = kt * BK + ld_chunk * 8;
        const bool ok = k < K;
#pragma unroll
        for (int i = 0; i < A_CHUNKS; ++i)
            a_reg[i] = ok ? *reinterpret_cast<const half8_t*>(a_ptr[i] + (size_t)kt * BK) : zero8;
#pragma unroll
        for (int i = 0; i < B_CHUNKS; ++i)
            b_reg[i] = ok ? *reinterpret_cast<const half8_t*>(b_ptr[i] + (size_t)kt * BK) : zero8;
    };
    auto store_lds = [&](int buf) {
        half_t* as = As + buf * BM * LDS_ROW;
        half_t* bs = Bs + buf * BN * LDS_ROW;
#pragma unroll
        for (int i = 0; i < A_CHUNKS; ++i)
            *reinterpret_cast<half8_t*>(as + (ld_row + i * ROWS_PER_PASS) * LDS_ROW + ld_chunk * 8) = a_reg[i];
#pragma unroll
        for (int i = 0; i < B_CHUNKS; ++i)
            *reinterpret_cast<half8_t*>(bs + (ld_row + i * ROWS_PER_PASS) * LDS_ROW + ld_chunk * 8) = b_reg[i];
    };

    float16_t acc[MT][NT];
#pragma unroll
    for (int i = 0; i < MT; ++i)
#pragma unroll
        for (int j = 0; j < NT; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

    const int KT = (K + BK - 1) / BK;
    load_global(0);
    store_lds(0);
    __syncthreads();

    // fragment read addresses: row (lane % 32) of the MFMA tile, k offset 8 * (lane / 32)
    const int fr_row = lane & 31;
    const int fr_k = (lane >> 5) * 8;

    for (int kt = 0; kt < KT; ++kt) {
        const int buf = kt & 1;
        if (kt + 1 < KT) load_global(kt + 1);
        const half_t* as = As + buf * BM * LDS_ROW + (wm * TM + fr_row) * LDS_ROW + fr_k;
        const half_t* bs = Bs + buf * BN * LDS_ROW + (wn * TN + fr_row) * LDS_ROW + fr_k;
#pragma unroll
        for (int ks = 0; ks < BK / 16; ++ks) {
            half8_t af[MT], bf[NT];
#pragma unroll
            for (int i = 0; i < MT; ++i)
                af[i] = *reinterpret_cast<const half8_t*>(as + i * 32 * LDS_ROW + ks * 16);
#pragma unroll
            for (int j = 0; j < NT; ++j)
                bf[j] = *reinterpret_cast<const half8_t*>(bs + j * 32 * LDS_ROW + ks * 16);
#pragma unroll
            for (int i = 0; i < MT; ++i)
#pragma unroll
                for (int j = 0; j < NT; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[i], bf[j], acc[i][j], 0, 0, 0);
        }
        if (kt + 1 < KT) store_lds(buf ^ 1);
        __syncthreads();
    }

    // Epilogue.  Accumulator element e of lane l is C[8*(e/4) + 4*(l/32) + e%4][l%32] of its tile.
    const int c_col = lane & 31;
    const int c_row_base = (lane >> 5) * 4;
#pragma unroll
    for (int i = 0; i < MT; ++i) {
#pragma unroll
        for (int j = 0; j < NT; ++j) {
            const int col = n0 + wn * TN + j * 32 + c_col;
            if (col >= N) continue;
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const int row = m0 + wm * TM + i * 32 + 8 * (e / 4) + c_row_base + (e % 4);
                if (row < M) C[(size_t)row * N + col] = (half_t)acc[i][j][e];
            }
        }
    }
}

// Any shape, any alignment: 16x16 outputs per 256-thread workgroup through LDS tiles,
// fp32 accumulation.  Correctness path for K % 8 != 0 or unaligned operands.
template <typename T, typename AccOut>
__global__ void __launch_bounds__(256)
gemm_generic_kernel(const T* __restrict__ A0, const T* __restrict__ B0, T* __restrict__ C0, int M, int N, int K,
                    long sa, long sb, long sc) {
    __shared__ float As[16][17];
    __shared__ float Bs[16][17];
    const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;
    const int batch = blockIdx.z;
    const T* A = A0 + (size_t)batch * sa;
    const T* B = B0 + (size_t)batch * sb;
    T* C = C0 + (size_t)batch * sc;
    const int row = blockIdx.y * 16 + ty;
    const int col = blockIdx.x * 16 + tx;
    float acc = 0.f;
    for (int k0 = 0; k0 < K; k0 += 16) {
        const int ar = blockIdx.y * 16 + ty, ak = k0 + tx;
        As[ty][tx] = (ar < M && ak < K) ? (float)A[(size_t)ar * K + ak] : 0.f;
        const int br = blockIdx.x * 16 + ty;
        Bs[ty][tx] = (br < N && ak < K) ? (float)B[(size_t)br * K + ak] : 0.f;
        __syncthreads();
#pragma unroll
        for (int k = 0; k < 16; ++k) acc = __builtin_fmaf(As[ty][k], Bs[tx][k], acc);
        __syncthreads();
    }
    if (row < M && col < N) C[(size_t)row * N + col] = (T)(AccOut)acc;
}

// ---------------------------------------------------------------------- dispatch ----

struct HgemmVariant {
    const char* name;
    int bm, bn, bk, threads;
    void (*kernel)(HgemmArgs);
};

#define TL_HGEMM_VARIANT(BM, BN, BK, WM, WN) \
    { "t" #BM "x" #BN "x" #BK "w" #WM "x" #WN, BM, BN, BK, WM * WN * 64, hgemm_f16_mfma_kernel<BM, BN, BK, WM, WN> }

static const HgemmVariant g_variants[] = {
    {"auto", 0, 0, 0, 0, nullptr},
    TL_HGEMM_VARIANT(128, 128, 64, 2, 2),  // 1
    TL_HGEMM_VARIANT(256, 128, 64, 2, 2),  // 2
    TL_HGEMM_VARIANT(128, 256, 64, 2, 2),  // 3
    TL_HGEMM_VARIANT(256, 256, 64, 2, 2),  // 4
    TL_HGEMM_VARIANT(64, 64, 64, 2, 2),    // 5
    TL_HGEMM_VARIANT(256, 256, 32, 2, 2),  // 6
    TL_HGEMM_VARIANT(128, 128, 32, 2, 2),  // 7
    TL_HGEMM_VARIANT(64, 128, 64, 2, 2),   // 8
};
static constexpr int kNumVariants = sizeof(g_variants) / sizeof(g_variants[0]);
static int g_forced_variant = 0;
static bool g_attr_set[kNumVariants] = {false};

static size_t lds_bytes(const HgemmVariant& v) {
    return (size_t)2 * (v.bm + v.bn) * (v.bk + kPad) * sizeof(half_t);
}

static int pick_variant(size_t M, size_t N, size_t K, int cus) {
    (void)K;
    auto tiles = [&](int bm, int bn) { return ((M + bm - 1) / bm) * ((N + bn - 1) / bn); };
    if (M <= 64) return 8;
    if (tiles(256, 256) >= (size_t)cus * 2) return 4;
    if (tiles(256, 128) >= (size_t)cus && M >= 256) return 2;
    if (tiles(128, 128) >= (size_t)cus / 2) return 1;
    return 5;
}

int launch_hgemm(const void* A, const void* B, void* C, size_t M, size_t N, size_t K, size_t batch, size_t sa,
                 size_t sb, size_t sc) {
    if (M == 0 || N == 0 || batch == 0) return TL_OK;
    TL_REQUIRE(M <= 0x7fffffffu && N <= 0x7fffffffu && K <= 0x7fffffffu && batch <= 65535,
               "hgemm: size out of range");
    hipStream_t st = stream();
    if (K == 0) {
        for (size_t b = 0; b < batch; ++b) {
            int rc = launch_fill_f16((half_t*)C + b * sc, 0, M * N);
            if (rc != TL_OK) return rc;
        }
        return TL_OK;
    }
    const bool vec_ok = (K % 8 == 0) && aligned16(A) && aligned16(B) &&
                        (batch == 1 || (sa % 8 == 0 && sb % 8 == 0));
    if (!vec_ok) {
        dim3 grid((unsigned)((N + 15) / 16), (unsigned)((M + 15) / 16), (unsigned)batch);
        TL_REQUIRE(grid.y <= 65535, "hgemm generic path: M too large (%zu)", M);
        hipLaunchKernelGGL((gemm_generic_kernel<half_t, float>), grid, dim3(256), 0, st, (const half_t*)A,
                           (const half_t*)B, (half_t*)C, (int)M, (int)N, (int)K, (long)sa, (long)sb, (long)sc);
        TL_CHECK_LAUNCH("gemm_generic_kernel<half>");
        return TL_OK;
    }
    const int vi = g_forced_variant ? g_forced_variant : pick_variant(M, N, K, device_info().cu_count);
    const HgemmVariant& v = g_variants[vi];
    const size_t lds = lds_bytes(v);
    if (lds > 64 * 1024 && !g_attr_set[vi]) {
        TL_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(v.kernel),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
        g_attr_set[vi] = true;
    }
    HgemmArgs a;
    a.A = (const half_t*)A;
    a.B = (const half_t*)B;
    a.C = (half_t*)C;
    a.M = (int)M;
    a.N = (int)N;
    a.K = (int)K;
    a.tiles_m = (int)((M + v.bm - 1) / v.bm);
    a.tiles_n = (int)((N + v.bn - 1) / v.bn);
    a.sa = (long)sa;
    a.sb = (long)sb;
    a.sc = (long)sc;
    const size_t nblocks = (size_t)a.tiles_m * a.tiles_n;
    TL_REQUIRE(nblocks <= 0x7fffffffu, "hgemm: too many tiles");
    hipLaunchKernelGGL(v.kernel, dim3((unsigned)nblocks, (unsigned)batch), dim3(v.threads), lds, st, a);
    TL_CHECK_LAUNCH(v.name);
    return TL_OK;
}

}  // namespace tl

extern "C" {

int tl_hgemm_f16(const void* A, const void* B, void* C, size_t M, size_t N, size_t K) {
    TL_ENSURE_INIT();
    TL_REQUIRE(A && B && C, "tl_hgemm_f16: null pointer");
    return tl::launch_hgemm(A, B, C, M, N, K, 1, 0, 0, 0);
}

int tl_matmul2d_f16(const void* A, const void* B, void* C, size_t M, size_t N, size_t K) {
    TL_ENSURE_INIT();
    TL_REQUIRE(A && B && C, "tl_matmul2d_f16: null pointer");
    if (M == 1) return tl::launch_gemv(A, B, C, N, K, 1, 0, 0, 0);
    return tl::launch_hgemm(A, B, C, M, N, K, 1, 0, 0, 0);
}

int tl_matmul2d_batched_f16(const void* A, const void* B, void* C, size_t M, size_t N, size_t K, size_t batch,
                            size_t strideA, size_t strideB, size_t strideC) {
    TL_ENSURE_INIT();
    TL_REQUIRE(A && B && C, "tl_matmul2d_batched_f16: null pointer");
    TL_REQUIRE(batch <= 65535, "tl_matmul2d_batched_f16: batch %zu exceeds 65535", batch);
    if (M == 1) return tl::launch_gemv(A, B, C, N, K, batch, strideA, strideB, strideC);
    return tl::launch_hgemm(A, B, C, M, N, K, batch, strideA, strideB, strideC);
}

int tl_matmul2d_f32(const void* A, const void* B, void* C, size_t M, size_t N, size_t K) {
    TL_ENSURE_INIT();
    TL_REQUIRE(A && B && C, "tl_matmul2d_f32: null pointer");
    if (M == 0 || N == 0) return TL_OK;
    TL_REQUIRE(M <= 0x7fffffffu && N <= 0x7fffffffu && K <= 0x7fffffffu, "tl_matmul2d_f32: size out of range");
    dim3 grid((unsigned)((N + 15) / 16), (unsigned)((M + 15) / 16), 1);
    TL_REQUIRE(grid.y <= 65535, "tl_matmul2d_f32: M too large (%zu)", M);
    hipLaunchKernelGGL((tl::gemm_generic_kernel<float, float>), grid, dim3(256), 0, tl::stream(), (const float*)A,
                       (const float*)B, (float*)C, (int)M, (int)N, (int)K, 0L, 0L, 0L);
    TL_CHECK_LAUNCH("gemm_generic_kernel<float>");
    return TL_OK;
}

int tl_set_hgemm_variant(int variant) {
    TL_REQUIRE(variant >= 0 && variant < tl::kNumVariants, "tl_set_hgemm_variant: %d out of range [0,%d)",
               variant, tl::kNumVariants);
    tl::g_forced_variant = variant;
    return TL_OK;
}

const char* tl_hgemm_variant_name(int variant) {
    if (variant < 0 || variant >= tl::kNumVariants) return nullptr;
    return tl::g_variants[variant].name;
}

}  // extern "C"
