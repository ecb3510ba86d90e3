// fp16 GEMM for very few rows: C[M,N] = X[M,K] . W[N,K]^T with 2 <= M <= 32 (the prefill of a short prompt), fp32
// accumulation, one rounding to fp16.  Same contract as the M > 1 branch of the reference's CUDA<half>::matmul2d
// (tensorLib/src/device/cuda/gemm.cu:163-171 -> hgemm_cublas, tensorLib/src/device/cuda/hgemm.cu:20-38).
//
// With so few rows the product is a GEMV with a handful of right-hand sides: W has to stream from HBM once, and
// nothing else should move.  A tile kernel cannot do that (its tiles re-read X through every CU and are padded to 128
// rows), so this one is laid out like the GEMV:
//   * a workgroup of four wavefronts owns all of K (up to 4096: wavefront w the 1024 values from 1024 * w) and
//     every parts-th 16-row block of W; each wavefront keeps ITS slice of X, all rows x 1024 values of K, in
//     registers for the whole kernel, in the layout of the MFMA's second operand (MB x 128 registers per lane);
//   * X first and then W stream through a ring private to the wavefront: a piece is 16 rows x 512 bytes, requested
//     four pieces ahead with global_load_lds_dwordx4 (no barrier on the streaming path; the chunk a lane fetches is
//     permuted, slot = chunk ^ row, so the 16 rows of a fragment read fall into 16 different bank groups) and read
//     back once, the pieces of X into registers, a piece of W as the first operand of v_mfma_f32_16x16x32_f16;
//   * after the four pieces of a block the four K slices meet in LDS in wavefront order and leave as fp16: K up to
//     4096 needs no second pass, and longer rows are left to the tile kernels (their K would have to be split
//     over workgroups, and the fp32 slabs that costs were measured to eat the gain).
// The workgroups of the chip read a moving window of consecutive rows of W over all of K, so the requests spread
// over the memory channels the way a GEMV's do.
#include <atomic>
#include <type_traits>

#include "tl_internal.h"

namespace tl {

struct FewRowsArgs {
    const half_t* X;
    const half_t* W;
    half_t* C;
    int M, N, K;      // K <= 4096
    int ldc;
    int parts;        // workgroups: workgroup p takes blocks p, p + parts, ...
    int nblocks;      // N / 16
};

constexpr int kFrRing = 4;                                   // pieces per wavefront in the ring
constexpr int kFrPieceBytes = 16 * 512;                      // 16 rows x 256 halves
constexpr int kFrWaveRing = kFrRing * kFrPieceBytes;
constexpr int kFrRingBytes = 4 * kFrWaveRing;                // 128 KB
constexpr int kFrSub = 4;                                    // pieces per block and wavefront: 1024 values of K

template <int I, int N, typename F>
__device__ __forceinline__ void static_for(F&& f) {
    if constexpr (I < N) {
        f(std::integral_constant<int, I>{});
        static_for<I + 1, N>(f);
    }
}

template <int N>
__device__ __forceinline__ void wait_vmcnt() {
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

template <int MB>
constexpr int fewrows_lds_bytes() { return kFrRingBytes + 2 * 4 * MB * 1024; }   // ring + two buffers of slices

// MB: 16-row groups of X (M <= 16 * MB)
template <int MB>
__global__ void __launch_bounds__(256) hgemm_f16_fewrows_kernel(const half_t* p_X, const half_t* p_W, half_t* p_C, int p_M, int p_N,
                                                                 int p_K, int p_ldc, int p_parts, int p_nblocks) {
    // scalar parameters (preloaded into SGPRs with the wavefront), not the struct
    const FewRowsArgs a{p_X, p_W, p_C, p_M, p_N, p_K, p_ldc, p_parts, p_nblocks};
    static_assert(MB == 1 || MB == 2, "X[16*MB, 1024] per wavefront must fit its registers");
    extern __shared__ __attribute__((aligned(1024))) unsigned char smem_raw[];
    typedef __attribute__((address_space(3))) unsigned char lds_byte_t;
    const unsigned lds_base = (unsigned)(unsigned long)(lds_byte_t*)smem_raw;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int M = a.M, N = a.N, K = a.K, ldc = a.ldc;
    half_t* __restrict__ C = a.C;
    const int part = (int)blockIdx.x;
    const int nblk = (a.nblocks - part + a.parts - 1) / a.parts;   // blocks part, part + parts, ...
    const int bstride = a.parts;
    const size_t wstep = (size_t)bstride * 16 * K;          // halves between this workgroup's consecutive blocks
    const int k0 = wave * 1024;
    // K % 256 == 0: a wavefront has 0 .. 4 whole pieces of 256 values
    const int nsub = k0 >= K ? 0 : ((K - k0) / 256 < kFrSub ? (K - k0) / 256 : kFrSub);
    const half_t* wb = a.W + (size_t)part * 16 * K + k0;   // this wavefront's first piece of its first block
    const half_t* xb = a.X + k0;
    // every kernel argument sits in registers before the loop: a scalar load still pending there would turn the
    // waits for fragment reads into lgkmcnt(0)
    asm volatile("" ::"s"(xb), "s"(C), "s"(M), "s"(N), "s"(K), "s"(ldc), "s"(nblk), "s"(wb), "s"(bstride),
                 "s"(wstep), "s"(nsub));

    // ---- streaming side: request t of a piece covers rows 2t, 2t+1 (512 bytes each) ----
    unsigned voff[8];
#pragma unroll
    for (int t = 0; t < 8; ++t) {
        const int r = 2 * t + (lane >> 5);
        voff[t] = (unsigned)r * (unsigned)K * 2u + (unsigned)(((lane & 31) ^ r) * 16);
    }
    const unsigned ring = lds_base + (unsigned)wave * (unsigned)kFrWaveRing;
    auto issue_piece = [&](const half_t* base, const unsigned (&off)[8], int slot) {
#pragma unroll
        for (int t = 0; t < 8; ++t) load_16B_per_lane_to_lds(base, off[t], ring + (unsigned)(slot * kFrPieceBytes + t * 1024));
    };
    // Pieces are numbered in the order they pass through the ring: MB * nsub pieces of X (16-row group j, sub-range
    // s), then nsub pieces per block of W.  Rows of X past the end re-read the last row and are zeroed on the way
    // into the registers.
    const int xsteps = MB * nsub, steps = xsteps + nblk * nsub;
    int iss_j = 0, iss_s = 0, iss_blk = 0, iss_slot = 0;     // the next piece to request
    auto issue_next = [&]() {
        if (iss_j < MB) {
            unsigned xoff[8];
#pragma unroll
            for (int t = 0; t < 8; ++t) {
                const int r = 2 * t + (lane >> 5);
                const int row = 16 * iss_j + r < M ? 16 * iss_j + r : M - 1;
                xoff[t] = (unsigned)row * (unsigned)K * 2u + (unsigned)(((lane & 31) ^ r) * 16);
            }
            issue_piece(xb + 256 * iss_s, xoff, iss_slot);
        } else {
            issue_piece(wb + (size_t)iss_blk * wstep + 256 * iss_s, voff, iss_slot);
        }
        iss_slot = iss_slot + 1 >= kFrRing ? 0 : iss_slot + 1;
        if (++iss_s == nsub) {
            iss_s = 0;
            if (iss_j < MB) ++iss_j;
            else ++iss_blk;
        }
    };
    int issued = 0;
    for (; issued < kFrRing && issued < steps; ++issued) issue_next();

    // Piece `s` of the sequence has landed once at most the requests behind it are outstanding (the counter holds
    // loads and stores in issue order; stores are never counted here, which can only lengthen a wait).
    auto wait_piece = [&](int s) {
        const int rem = steps - 1 - s;
        if (rem >= 3) wait_vmcnt<24>();
        else if (rem == 2) wait_vmcnt<16>();
        else if (rem == 1) wait_vmcnt<8>();
        else wait_vmcnt<0>();
    };

    // A piece leaves the ring for registers in one go (eight fragment reads), and its slot is requested again at
    // once for the piece four ahead: all four slots of the ring are in flight while the MFMAs run from registers.
    auto refill = [&]() {
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // the slot has been read
        if (issued < steps) { issue_next(); ++issued; }
    };

    // fragment c of a piece: row lane%16, chunk 4c + lane/16 of its 512 bytes
    const int fi = lane & 15, fg = lane >> 4;
    int fro[8];
#pragma unroll
    for (int c = 0; c < 8; ++c) fro[c] = fi * 512 + (((4 * c + fg) ^ fi) * 16);
    const float4_t zero4 = {0.f, 0.f, 0.f, 0.f};
    const half8_t zero8 = {0, 0, 0, 0, 0, 0, 0, 0};

    // ---- X into registers: xr[j][s][c] = rows 16j + lane%16, values k0 + 256s + 32c + 8*(lane/16) .. +8 ----
    half8_t xr[MB][kFrSub][8];
#pragma unroll
    for (int j = 0; j < MB; ++j)
#pragma unroll
        for (int s = 0; s < kFrSub; ++s)
#pragma unroll
            for (int c = 0; c < 8; ++c) xr[j][s][c] = zero8;
    int slot = 0, done = 0;
    static_for<0, MB * kFrSub>([&](auto it) {
        constexpr int j = decltype(it)::value / kFrSub, s = decltype(it)::value % kFrSub;
        if (s < nsub) {
            wait_piece(done);
            const unsigned char* sl = smem_raw + wave * kFrWaveRing + slot * kFrPieceBytes;
            const bool keep = 16 * j + fi < M;
            half8_t f[8];
#pragma unroll
            for (int c = 0; c < 8; ++c) f[c] = *reinterpret_cast<const half8_t*>(sl + fro[c]);
            refill();
#pragma unroll
            for (int c = 0; c < 8; ++c) xr[j][s][c] = keep ? f[c] : zero8;
            slot = slot + 1 >= kFrRing ? 0 : slot + 1;
            ++done;
        }
    });

    // ---- W through the matrix cores ----
    float* const red_all = reinterpret_cast<float*>(smem_raw + kFrRingBytes);
    int par = 0;
    for (int i = 0; i < nblk; ++i) {
        float4_t acc[MB];
#pragma unroll
        for (int j = 0; j < MB; ++j) acc[j] = zero4;
        static_for<0, kFrSub>([&](auto st) {
            constexpr int s = decltype(st)::value;
            if (s < nsub) {
                wait_piece(done);
                const unsigned char* sl = smem_raw + wave * kFrWaveRing + slot * kFrPieceBytes;
                half8_t f[8];
#pragma unroll
                for (int c = 0; c < 8; ++c) f[c] = *reinterpret_cast<const half8_t*>(sl + fro[c]);
                refill();
#pragma unroll
                for (int c = 0; c < 8; ++c)
#pragma unroll
                    for (int j = 0; j < MB; ++j)
                        acc[j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(f[c], xr[j][s][c], acc[j], 0, 0, 0);
                slot = slot + 1 >= kFrRing ? 0 : slot + 1;
                ++done;
            }
        });
        // the four K slices meet (two buffers, so one barrier per block is enough: a wavefront writes block i+2
        // only behind the barrier of block i+1, which every reader of block i has passed its reads to reach)
        float* red = red_all + par * (4 * MB * 256);
        par ^= 1;
#pragma unroll
        for (int j = 0; j < MB; ++j) *reinterpret_cast<float4_t*>(red + (wave * MB + j) * 256 + lane * 4) = acc[j];
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
        if (wave < MB) {                                    // wavefront j sums 16-row group j
            float4_t v = *reinterpret_cast<const float4_t*>(red + (0 * MB + wave) * 256 + lane * 4);
#pragma unroll
            for (int w = 1; w < 4; ++w)                     // wavefront order: a fixed summation order
                v += *reinterpret_cast<const float4_t*>(red + (w * MB + wave) * 256 + lane * 4);
            // v[e] = D[W row 16*block + 4*(lane/16) + e][X row 16*wave + lane%16]
            const int m = 16 * wave + fi;
            const int n = 16 * (part + i * bstride) + 4 * fg;
            if (m < M) {
                const half4_t h = {(half_t)v[0], (half_t)v[1], (half_t)v[2], (half_t)v[3]};
                *reinterpret_cast<half4_t*>(C + (size_t)m * ldc + n) = h;
            }
        }
    }
}

static std::atomic<int> g_fewrows_mode{0};   // 0 = automatic, -1 = never

// Measured against the tile kernels with W from HBM: ahead by 20-30 % for up to 16 rows and N up to 12288, by 3-9 %
// for wider W; with 17 .. 32 rows ahead up to N = 12288 and behind from 22016; rows shorter than 2048 leave half the
// wavefronts without work.
bool hgemm_fewrows_applies(size_t M, size_t N, size_t K, size_t ldc, size_t batch) {
    if (g_fewrows_mode.load() < 0) return false;
    return batch == 1 && M >= 2 && M <= 32 && N >= 16 && N % 16 == 0 && N <= 0x7fffffffu && K >= 2048 && K <= 4096 &&
           K % 256 == 0 && ldc % 4 == 0 && (M <= 16 || N <= 16384);
}

template <int MB>
static int launch_fewrows_variant(const FewRowsArgs& a) {
    constexpr int lds = fewrows_lds_bytes<MB>();
    static std::atomic<bool> attr_set{false};
    if (!attr_set.load()) {
        TL_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(hgemm_f16_fewrows_kernel<MB>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, lds));
        attr_set.store(true);
    }
    hipLaunchKernelGGL((hgemm_f16_fewrows_kernel<MB>), dim3((unsigned)a.parts), dim3(256), lds, stream(), a.X, a.W, a.C, a.M, a.N, a.K,
                       a.ldc, a.parts, a.nblocks);
    TL_CHECK_LAUNCH("hgemm_f16_fewrows_kernel");
    return TL_OK;
}

int launch_hgemm_fewrows(const void* X, const void* W, void* C, size_t M, size_t N, size_t K, size_t ldc) {
    FewRowsArgs a;
    a.X = (const half_t*)X;
    a.W = (const half_t*)W;
    a.C = (half_t*)C;
    a.M = (int)M;
    a.N = (int)N;
    a.K = (int)K;
    a.ldc = (int)ldc;
    a.nblocks = (int)(N / 16);
    const int cus = device_info().cu_count > 0 ? device_info().cu_count : 1;
    a.parts = cus < a.nblocks ? cus : a.nblocks;   // one workgroup per CU (its LDS fills the CU), one round
    return M <= 16 ? launch_fewrows_variant<1>(a) : launch_fewrows_variant<2>(a);
}

}  // namespace tl

extern "C" int tl_set_hgemm_fewrows(int mode) {
    TL_REQUIRE(mode == 0 || mode == -1, "tl_set_hgemm_fewrows: mode %d is neither 0 (automatic) nor -1 (never)", mode);
    tl::g_fewrows_mode = mode;
    return TL_OK;
}
