// fp16 GEMM for many rows, one wavefront per SIMD: C[M,N] = A[M,K] . B[N,K]^T, fp32 accumulation in the MFMA
// accumulators, one rounding to fp16.  Same contract as the M > 1 branch of the reference's CUDA<half>::matmul2d
// (tensorLib/src/device/cuda/gemm.cu:163-171 -> hgemm_cublas, tensorLib/src/device/cuda/hgemm.cu:20-38); numerics
// follow CPU<half>::matmul2d (tensorLib/src/device/cpu/CPU.cpp:76-89).
//
// Why a second tile kernel.  The ring of hgemm_f16_dlds_kernel holds two 64 KB stages of a 256x256x64 tile in LDS,
// so a K tile has exactly one tile of MFMAs (about 1.4 us) between its requests and its barrier, while memory answers
// a request after 1-2 us under this load: the ring is bound by latency (bytes in flight over latency), not by
// bandwidth, and the 160 KB of LDS have no room for a third stage.  Here the bytes in flight live in registers:
//   * four wavefronts, one per SIMD, each owning a 128x128 piece of the 256x256 tile: 256 accumulator registers per
//     lane, pinned to the AGPR half of the register file by issuing the MFMA through inline assembly with an "a"
//     constraint (the compiler alone keeps accumulators where the other values live and spills), which leaves all
//     256 VGPRs for data in flight;
//   * the pieces of K tiles t+2 and t+3 (2 x 16 x 16 bytes per lane = 128 VGPRs, 128 KB per CU) are in flight while
//     tile t is multiplied: requested with buffer loads (the resource descriptor bounds them, so rows past the end
//     of a matrix read as zero instead of faulting), written to the LDS stage tile t-1 has left one tile later
//     (ds_write_b128, the layout of the other kernel: a wavefront-load is 8 rows x 128 bytes in lane order and the
//     chunk a lane fetches is permuted so that fragment reads are free of bank conflicts), and the register of a
//     piece takes the matching piece of the K tile three ahead at once;
//   * one request and one LDS write behind every third MFMA, fragment reads of K step s+1 behind the MFMAs of step s,
//     one barrier per K tile;
//   * four wavefronts of 128x128 read a third fewer fragment bytes from LDS than eight of 128x64.
// Everything but the MFMA is ordinary code, so the compiler counts the outstanding loads and LDS accesses itself.
#include <atomic>
#include <type_traits>

#include "hgemm_common.h"

namespace tl {

typedef unsigned u32x4_t __attribute__((ext_vector_type(4)));

// acc += b-fragment . a-fragment with the accumulator in AGPRs.  B's fragment goes in as the first operand: the
// accumulator then holds the tile transposed, lane l owning row (l % 32) of C and four consecutive columns per group
// of four accumulator registers.
__device__ __forceinline__ void mfma_agpr(float16_t& acc, const half8_t& b, const half8_t& a) {
    asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+a"(acc) : "v"(b), "v"(a));
}

// `nops` idle cycles that every access to the sixteen accumulators stays on its side of.  The MFMAs are hidden from
// the compiler, so it neither knows that the matrix core may still be writing an accumulator the vector ALU is about to
// read (a 16-pass MFMA needs 18 wait states) nor that a freshly written zero takes a few cycles to be readable by an
// MFMA: the accumulators are operands of this statement, which orders it against every producer and consumer.
#define TL_ACC_FENCE(acc, text)                                                                                          \
    asm volatile(text : "+a"(acc[0][0]), "+a"(acc[0][1]), "+a"(acc[0][2]), "+a"(acc[0][3]), "+a"(acc[1][0]),             \
                 "+a"(acc[1][1]), "+a"(acc[1][2]), "+a"(acc[1][3]), "+a"(acc[2][0]), "+a"(acc[2][1]), "+a"(acc[2][2]),   \
                 "+a"(acc[2][3]), "+a"(acc[3][0]), "+a"(acc[3][1]), "+a"(acc[3][2]), "+a"(acc[3][3]))

template <int BM, int BN, int WM, int WN>
__global__ void __launch_bounds__(WM* WN * 64) hgemm_f16_vstage_kernel(HgemmArgs a) {
    constexpr int BK = 64;
    constexpr int NW = WM * WN;
    constexpr int RB = BK * 2;                 // bytes per tile row
    constexpr int CPR = BK / 8;                // 16-byte chunks per tile row
    constexpr int RPL = 256 / RB;              // tile rows per 256-byte LDS line
    constexpr int RPW = 1024 / RB;             // tile rows written by one wavefront-load
    constexpr int A_LOADS = BM / RPW / NW;     // wavefront-loads per K tile, per wavefront
    constexpr int B_LOADS = BN / RPW / NW;
    constexpr int LPW = A_LOADS + B_LOADS;
    constexpr int A_BYTES = BM * RB;
    constexpr int STAGE_BYTES = (BM + BN) * RB;
    constexpr int TM = BM / WM, TN = BN / WN;
    constexpr int MT = TM / 32, NT = TN / 32;
    constexpr int KS = BK / 16;
    constexpr int NM = MT * NT;
    static_assert(BM % (RPW * NW) == 0 && BN % (RPW * NW) == 0, "tile rows must split over the wavefronts");
    static_assert((NW * RPW / RPL) % CPR == 0, "the chunk a lane fetches must not depend on the piece");
    static_assert(LPW * 3 <= (KS - 1) * NM && LPW * 4 <= KS * NM, "the pieces of a K tile must fit the steps before its barrier");
    static_assert(KS % 2 == 0, "fragment ping-pong needs an even number of K steps");
    static_assert(MT == 4 && NT == 4, "TL_ACC_FENCE names sixteen accumulators");

    extern __shared__ __attribute__((aligned(1024))) unsigned char smem_raw[];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave / WN, wn = wave % WN;
    const int M = a.M, N = a.N, K = a.K, ldc = a.ldc;
    half_t* __restrict__ C = a.C;
    const int KT = K / BK;              // even, at least 4 (host-checked)
    const int total_tiles = a.tiles_m * a.tiles_n;
    const int tiles_m = a.tiles_m, band_m = a.band_m;
    const unsigned rot_tile = (unsigned)a.rot_tile, rot_xcd = (unsigned)a.rot_xcd;

    // Requests: piece j of this wavefront covers tile rows (j * NW + wave) * RPW .. + RPW.  A lane's byte offset
    // inside a matrix is (row * K + chunk * 8) * 2 for piece 0 of tile (0, 0); the tile, the piece and the walk along
    // K add a wavefront-uniform amount.  The whole offset goes into the instruction's per-lane offset, the one the
    // buffer's bounds check looks at: rows past the end of a matrix then read as zero without touching memory,
    // and so does a request whose uniform part is kNoTile.
    constexpr unsigned kNoTile = 0x80000000u;
    const __amdgpu_buffer_rsrc_t a_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<half_t*>(a.A), 0, (int)((unsigned)M * (unsigned)K * 2u), 0x00020000);
    const __amdgpu_buffer_rsrc_t b_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<half_t*>(a.B), 0, (int)((unsigned)N * (unsigned)K * 2u), 0x00020000);
    const int r0 = wave * RPW + lane / CPR;                       // tile row of piece 0
    const int chunk = (lane % CPR) ^ ((r0 / RPL) % CPR);           // the same for every piece (static_assert above)
    const unsigned lane_off = ((unsigned)r0 * (unsigned)K + (unsigned)chunk * 8u) * 2u;
    const unsigned piece_stride = (unsigned)(NW * RPW) * (unsigned)K * 2u;
    unsigned char* const lds_lane = smem_raw + wave * 1024 + lane * 16;

    // the C tile being multiplied and the one after it (this workgroup walks tiles blockIdx.x, + gridDim.x, ...)
    struct Tile {
        unsigned a_off, b_off;   // byte offsets of the tile's first rows in A and B (kNoTile: there is no such tile)
        int rot;                 // first K tile of the walk
        int m0, n0;
    };
    auto tile_at = [&](int vb) {
        Tile t;
        if (vb < total_tiles) {
            int tm, tn;
            tile_of_block(vb, total_tiles, tiles_m, band_m, tm, tn);
            t.m0 = tm * BM;
            t.n0 = tn * BN;
            t.rot = (int)(((unsigned)tn * rot_tile + (blockIdx.x & 7u) * rot_xcd) % (unsigned)KT);
            t.a_off = (unsigned)t.m0 * (unsigned)K * 2u;
            t.b_off = (unsigned)t.n0 * (unsigned)K * 2u;
        } else {
            t.m0 = t.n0 = t.rot = 0;
            t.a_off = t.b_off = kNoTile;
        }
        return t;
    };
    // byte offset along a row of the kt-th K tile of a walk that starts at K tile `rot`
    auto k_of = [&](int kt, int rot) {
        int k = kt + rot;
        k = k >= KT ? k - KT : k;
        return (unsigned)k * (unsigned)(BK * 2);
    };

    // pieces of the two K tiles that are between memory and LDS: K tile t sits in set t % 2
    u32x4_t stg[2][LPW];
    auto piece_load = [&](auto set, int l, unsigned a_base, unsigned b_base) {
        if (l < A_LOADS)
            stg[decltype(set)::value][l] = __builtin_amdgcn_raw_buffer_load_b128(a_rsrc, (int)(lane_off + (a_base + (unsigned)l * piece_stride)), 0, 0);
        else
            stg[decltype(set)::value][l] = __builtin_amdgcn_raw_buffer_load_b128(b_rsrc, (int)(lane_off + (b_base + (unsigned)(l - A_LOADS) * piece_stride)), 0, 0);
    };
    // stage_lane: this lane's address in the stage that receives the tile (one addition per K tile, the piece's place
    // inside the stage is an immediate offset)
    auto piece_store = [&](auto set, int l, unsigned char* stage_lane) {
        const int in_stage = l < A_LOADS ? l * NW * 1024 : A_BYTES + (l - A_LOADS) * NW * 1024;
        *reinterpret_cast<u32x4_t*>(stage_lane + in_stage) = stg[decltype(set)::value][l];
    };

    // fragment reader: row (lane % 32) of a 32-row MFMA tile, chunk 2*ks + lane/32
    const int fr_row = lane & 31;
    const int fr_sw = (fr_row / RPL) % CPR;
    int fr_off[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) fr_off[ks] = fr_row * RB + (((ks * 2 + (lane >> 5)) ^ fr_sw) * 16);
    const int a_base = wm * TM * RB;
    const int b_base = A_BYTES + wn * TN * RB;

    float16_t acc[MT][NT];
    half8_t af[2][MT], bf[2][NT];
    using S0 = std::integral_constant<int, 0>;
    using S1 = std::integral_constant<int, 1>;
    // LDS writes and reads of this wavefront done, then the workgroup barrier; loads from memory stay in flight
    auto lds_barrier = [&]() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); };

    int vb = blockIdx.x;
    Tile cur = tile_at(vb);
    Tile nxt_tile = tile_at(vb + (int)gridDim.x);

    // prologue of the pipeline: K tiles 0 and 1 of the first C tile requested, tile 0 written to stage 0 as it
    // arrives while tile 2 takes over its registers
    {
        const unsigned k0 = k_of(0, cur.rot), k1 = k_of(1, cur.rot), k2 = k_of(2, cur.rot);
#pragma unroll
        for (int l = 0; l < LPW; ++l) piece_load(S0{}, l, cur.a_off + k0, cur.b_off + k0);
#pragma unroll
        for (int l = 0; l < LPW; ++l) piece_load(S1{}, l, cur.a_off + k1, cur.b_off + k1);
#pragma unroll
        for (int l = 0; l < LPW; ++l) {
            piece_store(S0{}, l, lds_lane);
            piece_load(S0{}, l, cur.a_off + k2, cur.b_off + k2);
        }
    }
    lds_barrier();
    {
        const unsigned char* sa = smem_raw + a_base;
        const unsigned char* sb = smem_raw + b_base;
        af[0][0] = *reinterpret_cast<const half8_t*>(sa + fr_off[0]);
#pragma unroll
        for (int j = 0; j < NT; ++j) bf[0][j] = *reinterpret_cast<const half8_t*>(sb + j * 32 * RB + fr_off[0]);
#pragma unroll
        for (int i = 1; i < MT; ++i) af[0][i] = *reinterpret_cast<const half8_t*>(sa + i * 32 * RB + fr_off[0]);
    }

    // One K tile of the pipeline, the same for every tile of every C tile: the K tile three positions ahead may
    // belong to the next C tile (or to none, then its requests fall outside the buffers and cost nothing), and the
    // fragments requested in the last step may be the first ones of the next C tile.
    // set: register set of K tile kt+1 (= (kt + 1) % 2), which the K tile three ahead takes over piece by piece.
    auto tile = [&](int kt, auto set) {
        const bool wrap = kt + 3 >= KT;
        const unsigned koff_fill = k_of(wrap ? kt + 3 - KT : kt + 3, wrap ? nxt_tile.rot : cur.rot);
        const unsigned fill_a = (wrap ? nxt_tile.a_off : cur.a_off) + koff_fill;
        const unsigned fill_b = (wrap ? nxt_tile.b_off : cur.b_off) + koff_fill;
        unsigned char* const stage_lane = lds_lane + ((kt + 1) & 1) * STAGE_BYTES;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            const int cur_f = ks & 1, nxt_f = cur_f ^ 1;
            const bool last = ks + 1 == KS;
            if (last) lds_barrier();   // tile kt+1 is complete in LDS, tile kt's stage is free
            const int rk = last ? kt + 1 : kt, rs = last ? 0 : ks + 1;
            const unsigned char* sa = smem_raw + (rk & 1) * STAGE_BYTES + a_base;
            const unsigned char* sb = smem_raw + (rk & 1) * STAGE_BYTES + b_base;
#pragma unroll
            for (int m = 0; m < NM; ++m) {
                const int i = m / NT, j = m % NT;
                mfma_agpr(acc[i][j], bf[cur_f][j], af[cur_f][i]);
                // fragment reads of the next step, in the order its MFMAs first need them: A0, B0 .. B(NT-1), A1 ..
                if (m % 2 == 0) {
                    const int r = m / 2;
                    if (r == 0) af[nxt_f][0] = *reinterpret_cast<const half8_t*>(sa + fr_off[rs]);
                    else if (r <= NT) bf[nxt_f][r - 1] = *reinterpret_cast<const half8_t*>(sb + (r - 1) * 32 * RB + fr_off[rs]);
                    else if (r < MT + NT) af[nxt_f][r - NT] = *reinterpret_cast<const half8_t*>(sa + (r - NT) * 32 * RB + fr_off[rs]);
                }
                // piece l moves register -> LDS behind MFMA 3*l + 1 of the tile (all before the barrier of the last
                // step), and its register takes the matching piece of the K tile three ahead behind MFMA 4*l + 3:
                // at most two memory instructions between two MFMAs
                const int q = ks * NM + m;
                if (q % 3 == 1 && q / 3 < LPW) piece_store(set, q / 3, stage_lane);
                if (q % 4 == 3 && q / 4 < LPW) piece_load(set, q / 4, fill_a, fill_b);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
    };

    for (;;) {   // C tiles of this workgroup
#pragma unroll
        for (int i = 0; i < MT; ++i)
#pragma unroll
            for (int j = 0; j < NT; ++j)
#pragma unroll
                for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;
        TL_ACC_FENCE(acc, "s_nop 7");

        for (int kt = 0; kt < KT; kt += 2) {
            tile(kt, S1{});
            tile(kt + 1, S0{});
        }
        TL_ACC_FENCE(acc, "s_nop 15\n\ts_nop 15");

        // ---- epilogue.  acc[i][j][4*g + r] = C[row i*32 + lane%32][col j*32 + 8*g + 4*(lane/32) + r] ----
        // fp16 output through LDS: every wavefront turns 32 x TN blocks of its accumulators into row-major halves in a
        // private region of stage 1 (free since the last barrier of the K loop; stage 0 already holds the first K tile
        // of the next C tile), 8-byte writes into rows padded by 16 bytes so that the 32 rows of one write land in
        // different banks, reads them back 16 bytes per lane and stores whole 16-byte pieces of C rows.  The host
        // guarantees N % 8 == 0, ldc % 8 == 0 and a 16-byte aligned C.
        const int e_row = lane & 31;
        const int e_col = (lane >> 5) * 4;
        const int row_base = cur.m0 + wm * TM, col_base = cur.n0 + wn * TN;
        constexpr int RS = TN * 2 + 16;
        constexpr int CH = TN / 8;               // 16-byte chunks per row
        constexpr int RPR = 64 / CH;             // rows per wavefront-wide read
        constexpr int PASSES = (32 + RPR - 1) / RPR;
        static_assert(NW * 32 * RS <= STAGE_BYTES, "staging area must fit one stage");
        unsigned char* region = smem_raw + STAGE_BYTES + wave * (32 * RS);
#pragma unroll
        for (int i = 0; i < MT; ++i) {
#pragma unroll
            for (int j = 0; j < NT; ++j)
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    half4_t h = {(half_t)acc[i][j][4 * g], (half_t)acc[i][j][4 * g + 1], (half_t)acc[i][j][4 * g + 2],
                                 (half_t)acc[i][j][4 * g + 3]};
                    *reinterpret_cast<half4_t*>(region + e_row * RS + (j * 32 + g * 8 + e_col) * 2) = h;
                }
#pragma unroll
            for (int q = 0; q < PASSES; ++q) {
                const int r = q * RPR + lane / CH, c = lane % CH;
                if (lane >= RPR * CH || r >= 32) continue;
                const half8_t v = *reinterpret_cast<const half8_t*>(region + r * RS + c * 16);
                const int row = row_base + i * 32 + r, col = col_base + c * 8;
                if (row < M && col < N) *reinterpret_cast<half8_t*>(C + (size_t)row * ldc + col) = v;
            }
        }
        vb += (int)gridDim.x;
        if (vb >= total_tiles) break;
        // the next K loop writes pieces into stage 1 at once: every wavefront must have read its staged C back
        lds_barrier();
        cur = nxt_tile;
        nxt_tile = tile_at(vb + (int)gridDim.x);
    }
}

struct VstageVariant {
    const char* name;
    int bm, bn, threads;
    void (*kernel)(HgemmArgs);
};
static const VstageVariant g_vstage[] = {
    {"v256x256x64w2x2", 256, 256, 256, hgemm_f16_vstage_kernel<256, 256, 2, 2>},
};
static std::atomic<bool> g_vstage_attr[sizeof(g_vstage) / sizeof(g_vstage[0])];

const char* hgemm_vstage_name(int index) {
    return index >= 0 && index < (int)(sizeof(g_vstage) / sizeof(g_vstage[0])) ? g_vstage[index].name : nullptr;
}

// Full contract of the kernel: an even number of K tiles of 64, at least four, both matrices below 2 GiB (32-bit buffer offsets), C rows that
// take 16-byte stores.
bool hgemm_vstage_applies(const void* A, const void* B, const void* C, size_t M, size_t N, size_t K, size_t ldc) {
    return M >= 1 && N >= 1 && K >= 256 && K % 128 == 0 && M * K * 2 < ((size_t)1 << 31) && N * K * 2 < ((size_t)1 << 31) &&
           N % 8 == 0 && ldc % 8 == 0 && aligned16(A) && aligned16(B) && aligned16(C) && M <= 0x7fffffffu && N <= 0x7fffffffu;
}

int launch_hgemm_vstage(int index, const void* A, const void* B, void* C, size_t M, size_t N, size_t K, size_t ldc, int band,
                        int rot_tile, int rot_xcd) {
    TL_REQUIRE(hgemm_vstage_name(index) != nullptr, "hgemm: no register-staged variant %d", index);
    TL_REQUIRE(hgemm_vstage_applies(A, B, C, M, N, K, ldc), "hgemm: %s does not serve this shape", g_vstage[index].name);
    const VstageVariant& v = g_vstage[index];
    const size_t lds = (size_t)2 * (v.bm + v.bn) * 64 * sizeof(half_t);
    if (!g_vstage_attr[index].load()) {
        TL_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(v.kernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
        g_vstage_attr[index].store(true);
    }
    HgemmArgs a{};
    a.A = (const half_t*)A;
    a.B = (const half_t*)B;
    a.C = (half_t*)C;
    a.M = (int)M;
    a.N = (int)N;
    a.K = (int)K;
    a.ldc = (int)ldc;
    a.tiles_m = (int)((M + v.bm - 1) / v.bm);
    a.tiles_n = (int)((N + v.bn - 1) / v.bn);
    a.kt_per_split = 0x7fffffff;
    a.band_m = band > 0 ? band : 8;
    a.rot_tile = rot_tile;
    a.rot_xcd = rot_xcd;
    const size_t nblocks = (size_t)a.tiles_m * a.tiles_n;
    TL_REQUIRE(nblocks <= 0x7fffffffu, "hgemm: too many tiles");
    // persistent: one workgroup per CU walks tiles blockIdx.x, + gridDim.x, ...
    size_t grid = nblocks;
    const size_t cus = (size_t)device_info().cu_count;
    if (cus > 0 && grid > cus) grid = cus;
    hipLaunchKernelGGL(v.kernel, dim3((unsigned)grid), dim3(v.threads), lds, stream(), a);
    TL_CHECK_LAUNCH(v.name);
    return TL_OK;
}

}  // namespace tl
