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
// Two kernels share that layout.  hgemm_f16_dlds_kernel (K % 64 == 0, the prefill shapes) moves tiles
// global -> LDS with global_load_lds_dwordx4 through a ring of stages, swizzles the chunk order instead of
// padding rows, pipelines fragment reads under the MFMAs of the previous K step and, for rings of two or
// three stages, is persistent over C tiles.  hgemm_f16_mfma_kernel (any K % 8 == 0) stages tiles through
// registers into LDS rows of BK+8 halves (the 16-byte pad makes the 32 rows a ds_read_b128 touches fall
// in distinct bank groups) and zero-fills the K tail.  gemm_generic_kernel covers everything else.
#include <atomic>
#include <cstring>
#include <mutex>
#include <numeric>
#include <type_traits>

#include "hgemm_common.h"

namespace tl {

constexpr int kPad = 8;  // halves of padding per LDS row

template <int BM, int BN, int BK, int WM, int WN>
__global__ void __launch_bounds__(WM* WN * 64) hgemm_f16_mfma_kernel(TL_HGEMM_PARAMS) {
    TL_HGEMM_ARGS_FROM_PARAMS;
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
    tile_of_block(blockIdx.x, gridDim.x, a.tiles_m, a.band_m, tile_m, tile_n);
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
                if (row < M) C[(size_t)row * a.ldc + col] = (half_t)acc[i][j][e];
            }
        }
    }
}

// ------------------------------------------------------------------------------------------
// Direct-to-LDS variant.  Tiles go HBM -> LDS with global_load_lds_dwordx4 (no VGPR staging,
// no ds_write), through a ring of STAGES LDS buffers, so the loads of tile k+STAGES-1 are in
// flight while tile k feeds the MFMAs.  A wavefront-load writes 1 KiB of LDS in lane order, so
// the bank-conflict-free layout is obtained by permuting WHICH 16-byte chunk of a row each lane
// fetches: the chunk stored at slot p of tile row r is chunk p ^ ((r / RPL) % CPR), where RPL
// rows fill one 256-byte LDS line and CPR is the number of chunks per row.  The 16 rows a
// ds_read_b128 group touches then land in 16 different 16-byte bank groups.
// Requirements: K % BK == 0 (no zero fill is possible on this path), K % 8 == 0, aligned operands.
// MODE 0: every wavefront reads the fragments of a K step, then issues its MFMAs.
// MODE 1: fragments double buffered in registers across K steps.
// MODE 2: MODE 1 with the SwiGLU gate in the epilogue: a B tile holds, for every wavefront column, TN/2 rows of the
//         first matrix followed by the TN/2 rows of the second that pair with them, so a wavefront finds both factors
//         of an output in the 32 x TN block it stages through LDS anyway; the tile then covers BN/2 output columns.
template <int BM, int BN, int BK, int WM, int WN, int STAGES, int MODE>
__global__ void __launch_bounds__(WM* WN * 64) hgemm_f16_dlds_kernel(TL_HGEMM_PARAMS) {
    TL_HGEMM_ARGS_FROM_PARAMS;
    constexpr int NW = WM * WN;
    constexpr int RB = BK * 2;                 // bytes per tile row
    constexpr int CPR = BK / 8;                // 16-byte chunks per tile row
    constexpr int RPL = 256 / RB;              // tile rows per 256-byte LDS line
    constexpr int RPW = 1024 / RB;             // tile rows written by one wavefront-load
    constexpr int A_LOADS = BM / RPW / NW;     // wavefront-loads per stage, per wavefront
    constexpr int B_LOADS = BN / RPW / NW;
    constexpr int LPW = A_LOADS + B_LOADS;
    constexpr int A_BYTES = BM * RB;
    constexpr int STAGE_BYTES = (BM + BN) * RB;
    constexpr int TM = BM / WM, TN = BN / WN;
    constexpr int MT = TM / 32, NT = TN / 32;
    constexpr int KS = BK / 16;
    constexpr bool GATED = MODE == 2;
    // the in-launch merge of split-K is compiled for tiles up to 128x256 (the ones a split launch uses; in the 256x256
    // kernels its registers would add to a budget that is already full)
    constexpr bool TICKETS = BM * BN <= 128 * 256;
    static_assert(!GATED || TN % 16 == 0, "a wavefront column holds two halves of whole 16-byte pieces");
    static_assert(BK == 32 || BK == 64, "BK must be 32 or 64");
    static_assert(BM % (RPW * NW) == 0 && BN % (RPW * NW) == 0, "tile rows must split over the wavefronts");
    static_assert(STAGES >= 2 && STAGES <= 5 && LPW * (STAGES - 2) < 64, "vmcnt is a 6-bit counter");
    // Pipelined variants with two or three stages are persistent: a workgroup walks tiles blockIdx.x,
    // + gridDim.x, ... and requests the first STAGES-1 K tiles of its next C tile before it stores the current
    // one (staged through the last stage's LDS), so the C stores and the cold start of the next tile overlap.
    // vmcnt counts loads and stores together on this ISA, so the stores are drained (vmcnt(0)) before the
    // next tile's loop resumes waiting with exact load counts.
    constexpr bool PERSIST = (STAGES <= 3 && MODE >= 1 && NW * 32 * (BN / WN * 2 + 16) <= (BM + BN) * BK * 2);

    extern __shared__ __attribute__((aligned(1024))) unsigned char smem_raw[];
    typedef __attribute__((address_space(3))) unsigned char lds_byte_t;
    lds_byte_t* lds = (lds_byte_t*)smem_raw;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave / WN, wn = wave % WN;

    const int total_tiles = a.tiles_m * a.tiles_n;
    int m0 = 0, n0 = 0;
    const int batch = blockIdx.y;
    const half_t* __restrict__ A = a.A + (size_t)batch * a.sa;
    const half_t* __restrict__ B = a.B + (size_t)batch * a.sb;
    half_t* __restrict__ C = a.C + (size_t)batch * a.sc;
    const int M = a.M, N = a.N, K = a.K;
    // Every kernel argument is pulled into registers here.  A scalar load still pending inside the main
    // loop would make the compiler treat lgkmcnt as unordered and turn every wait for LDS data into
    // lgkmcnt(0), which also waits for the fragment reads issued just before it.
    float* const partial = a.partial;
    unsigned* const tickets = a.tickets;
    const int ldc = a.ldc;
    const unsigned rot_tile = (unsigned)a.rot_tile, rot_xcd = (unsigned)a.rot_xcd;
    const int band_m = a.band_m;
    const int gate = GATED ? a.gate : 0;
    asm volatile("" ::"s"(partial), "s"(C), "s"(M), "s"(N), "s"(a.kt_per_split), "s"(rot_tile), "s"(rot_xcd), "s"(band_m), "s"(ldc),
                 "s"(gate), "s"(tickets));

    // ---- loader: wavefront-load j of this wavefront covers tile rows (j*NW + wave)*RPW .. +RPW ----
    // A request's address is a wavefront-uniform base (first row of the tile at the K tile wanted, in scalar
    // registers) plus a per-lane byte offset that is fixed for the whole C tile, and its LDS target a scalar
    // too: walking K costs a few scalar instructions per K tile and none per request.
    const int ld_row_in_group = lane / CPR;
    const int ld_slot = lane % CPR;
    unsigned a_voff[A_LOADS], b_voff[B_LOADS];
    const half_t* a_tile = A;
    const half_t* b_tile = B;
    const unsigned lds_wave = (unsigned)(unsigned long)lds + (unsigned)wave * 1024u;
    const int KT_all = K / BK;
    const int kt_begin = (int)blockIdx.z * a.kt_per_split;
    const int KT = (KT_all - kt_begin) < a.kt_per_split ? (KT_all - kt_begin) : a.kt_per_split;
    // tile `b` of the launch: sets m0, n0, the tile bases (at this split's first K tile) and the lane offsets
    int rot = 0;  // first K tile of this workgroup's walk (relative to its split)
    auto setup_tile = [&](int b) {
        int tile_m, tile_n;
        tile_of_block(b, total_tiles, a.tiles_m, band_m, tile_m, tile_n);
        m0 = tile_m * BM;
        n0 = GATED ? tile_n * (BN / 2) : tile_n * BN;   // first output column of the tile
        rot = KT > 0 ? (int)(((unsigned)tile_n * rot_tile + (blockIdx.x & 7u) * rot_xcd) % (unsigned)KT) : 0;
        a_tile = A + (size_t)m0 * K + (size_t)kt_begin * BK;
        b_tile = GATED ? B + (size_t)kt_begin * BK : B + (size_t)n0 * K + (size_t)kt_begin * BK;
#pragma unroll
        for (int j = 0; j < A_LOADS; ++j) {
            const int r = (j * NW + wave) * RPW + ld_row_in_group;  // tile row
            const int c = ld_slot ^ ((r / RPL) % CPR);              // chunk of that row this lane fetches
            const int rr = m0 + r < M ? r : M - 1 - m0;             // rows past the end re-read the last one
            a_voff[j] = (unsigned)(((size_t)rr * K + c * 8) * sizeof(half_t));
        }
#pragma unroll
        for (int j = 0; j < B_LOADS; ++j) {
            const int r = (j * NW + wave) * RPW + ld_row_in_group;
            const int c = ld_slot ^ ((r / RPL) % CPR);
            if constexpr (GATED) {
                // tile row r = wavefront column r / TN, inside it TN/2 rows of the first matrix, then their partners;
                // offsets are relative to B (the host checks that both matrices lie within 4 GB of it)
                const int in_wave = r % TN;
                const int ocol = n0 + (r / TN) * (TN / 2) + in_wave % (TN / 2);
                const size_t grow = (size_t)(ocol < N / 2 ? ocol : N / 2 - 1) + (in_wave >= TN / 2 ? (size_t)gate : 0);
                b_voff[j] = (unsigned)((grow * K + c * 8) * sizeof(half_t));
            } else {
                const int rr = n0 + r < N ? r : N - 1 - n0;
                b_voff[j] = (unsigned)(((size_t)rr * K + c * 8) * sizeof(half_t));
            }
        }
    };
    int vb = blockIdx.x;
    setup_tile(vb);
    auto a_off = [&](int kt) { return (kt % STAGES) * STAGE_BYTES; };
    auto b_off = [&](int kt) { return (kt % STAGES) * STAGE_BYTES + A_BYTES; };
    // element offset of the kt-th K tile of the walk
    auto k_of = [&](int kt) {
        int k = kt + rot;
        k = k >= KT ? k - KT : k;
        return (size_t)k * BK;
    };
    // wavefront-load l of a K tile whose bases and LDS stage the caller has worked out: l < A_LOADS from A
    auto issue_one_at = [&](const half_t* abase, const half_t* bbase, unsigned stage, int l) {
        if (l < A_LOADS)
            load_16B_per_lane_to_lds(abase, a_voff[l], stage + (unsigned)(l * NW * 1024));
        else
            load_16B_per_lane_to_lds(bbase, b_voff[l - A_LOADS], stage + (unsigned)(A_BYTES + (l - A_LOADS) * NW * 1024));
    };
    auto issue_tile = [&](int kt) {
        const size_t koff = k_of(kt);
        const unsigned stage = lds_wave + (unsigned)a_off(kt);
#pragma unroll
        for (int l = 0; l < LPW; ++l) issue_one_at(a_tile + koff, b_tile + koff, stage, l);
    };

    // ---- fragment reader: row (lane % 32) of a 32-row MFMA tile, chunk 2*ks + lane/32 ----
    const int fr_row = lane & 31;
    const int fr_sw = (fr_row / RPL) % CPR;
    int fr_off[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) fr_off[ks] = fr_row * RB + (((ks * 2 + (lane >> 5)) ^ fr_sw) * 16);
    const int a_base = wm * TM * RB;
    const int b_base = wn * TN * RB;

    float16_t acc[MT][NT];
#pragma unroll
    for (int s = 0; s < STAGES - 1; ++s)
        if (s < KT) issue_tile(s);

    // Wait until tile kt has landed in LDS for every wavefront.  Tiles requested after kt
    // (at most STAGES-2 of them) may stay in flight.
    auto sync_for = [&](int kt) {
        const int ahead = (KT - 1 - kt) < (STAGES - 2) ? (KT - 1 - kt) : (STAGES - 2);
        if (STAGES >= 5 && ahead >= 3) wait_vmcnt_and_barrier<3 * LPW>();
        else if (STAGES >= 4 && ahead == 2) wait_vmcnt_and_barrier<2 * LPW>();
        else if (STAGES >= 3 && ahead == 1) wait_vmcnt_and_barrier<LPW>();
        else wait_vmcnt_and_barrier<0>();
    };
    // After the barrier of tile kt every wavefront is done with tile kt-1: refill what it occupied.
    auto issue_after_sync = [&](int kt) {
        if (kt + STAGES - 1 < KT) issue_tile(kt + STAGES - 1);
    };
    // Fragment reads go out in the order the MFMAs of a step (A index outer, B index inner) first need them:
    // A0, B0 .. B(NT-1), A1 .. A(MT-1).  LDS returns data in order, so the wait in front of an MFMA then counts
    // only the reads that MFMA needs, and each read has had most of a step to land.
    auto load_frags = [&](half8_t (&af)[MT], half8_t (&bf)[NT], int kt, int ks) {
        const unsigned char* sa = smem_raw + a_off(kt) + a_base;
        const unsigned char* sb = smem_raw + b_off(kt) + b_base;
        af[0] = *reinterpret_cast<const half8_t*>(sa + fr_off[ks]);
#pragma unroll
        for (int j = 0; j < NT; ++j)
            bf[j] = *reinterpret_cast<const half8_t*>(sb + j * 32 * RB + fr_off[ks]);
#pragma unroll
        for (int i = 1; i < MT; ++i)
            af[i] = *reinterpret_cast<const half8_t*>(sa + i * 32 * RB + fr_off[ks]);
    };
    auto mfmas = [&](const half8_t (&af)[MT], const half8_t (&bf)[NT]) {
#pragma unroll
        for (int i = 0; i < MT; ++i)
#pragma unroll
            for (int j = 0; j < NT; ++j)
                // B's fragment goes in as the first operand: the accumulator then holds the tile
                // transposed, i.e. lane l owns row (l % 32) of C and, per group of four accumulator
                // registers, four CONSECUTIVE columns, which is what a vector store wants.
                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(bf[j], af[i], acc[i][j], 0, 0, 0);
    };

  for (;;) {  // tiles of this workgroup (one, unless PERSIST)
#pragma unroll
    for (int i = 0; i < MT; ++i)
#pragma unroll
        for (int j = 0; j < NT; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

    if constexpr (MODE >= 1) {
        // Fragments are double buffered in registers: the ds_reads of K step s+1 (or of the next tile's first
        // step, after the tile barrier) go out one by one behind the first MFMAs of step s, in the order
        // load_frags uses.
        //
        // Where the requests that refill the ring go.  With three or more stages they are spread over a whole K
        // tile of MFMAs: segment 0 of a tile's LPW requests goes out in the last step of the tile that frees
        // its stage (after the barrier), segments 1 .. KS-1 in steps 0 .. KS-2 of the next tile; all of them
        // are older than that next tile's barrier, so the vmcnt counts do not change.  With two stages a tile
        // has one K tile of time to land, and spreading its requests made every barrier wait 400-570 cycles
        // for data (measured), so there all LPW requests go out behind the MFMAs of the last step.
        static_assert(KS % 2 == 0, "fragment ping-pong needs an even number of K steps");
        constexpr int NM = MT * NT;
        half8_t af[2][MT], bf[2][NT];
        // requests [seg * LPW / KS, (seg + 1) * LPW / KS) of K tile kt, request i of them behind MFMA m
        constexpr bool SPREAD = STAGES >= 3;
        auto issue_segment = [&](int seg, int m, const half_t* abase, const half_t* bbase, unsigned stage) {
            const int l0 = SPREAD ? seg * LPW / KS : (seg == 0 ? 0 : LPW);
            const int l1 = SPREAD ? (seg + 1) * LPW / KS : LPW;
            const int n = l1 - l0;
#pragma unroll
            for (int i = 0; i < n; ++i) {
                const int at = n <= NM ? i * (NM / n) + (NM / n) / 2 : i % NM;
                if (at == m) issue_one_at(abase, bbase, stage, l0 + i);
            }
        };
        sync_for(0);
        if (STAGES - 1 < KT) {  // segment 0 of the tile that follows the prologue's; the rest inside tile(0)
            const size_t koff = k_of(STAGES - 1);
#pragma unroll
            for (int m = 0; m < NM; ++m) issue_segment(0, m, a_tile + koff, b_tile + koff, lds_wave + (unsigned)a_off(STAGES - 1));
        }
        load_frags(af[0], bf[0], 0, 0);
        // has_next: another K tile follows (its first fragments are requested in the last step);
        // fill: K tile kt + STAGES - 1 exists (its segments 1.. go out in steps 0 .. KS-2);
        // more: K tile kt + STAGES exists (its segment 0 goes out in the last step).
        // All compile-time, and the last K tile is peeled off, so every step is straight-line code and the
        // compiler knows how many reads are younger than the ones an MFMA needs.
        auto tile = [&](int kt, auto has_next, auto fill, auto more) {
            const size_t koff_fill = decltype(fill)::value ? k_of(kt + STAGES - 1) : 0;
            const half_t* abase_fill = a_tile + koff_fill;
            const half_t* bbase_fill = b_tile + koff_fill;
            const unsigned stage_fill = lds_wave + (unsigned)a_off(kt + STAGES - 1);
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                const int cur = ks & 1, nxt = cur ^ 1;
                const bool last = ks + 1 == KS;
                if (last && !decltype(has_next)::value) {
                    mfmas(af[cur], bf[cur]);
                    continue;
                }
                // where the fragments of the next step live: this tile's stage, or the next tile's after its barrier
                if (last) sync_for(kt + 1);  // every wavefront holds its last fragments of tile kt in registers
                const int rk = last ? kt + 1 : kt, rs = last ? 0 : ks + 1;
                const unsigned char* sa = smem_raw + a_off(rk) + a_base;
                const unsigned char* sb = smem_raw + b_off(rk) + b_base;
                const size_t koff = (last && decltype(more)::value) ? k_of(kt + STAGES) : 0;
                const half_t* abase = last ? a_tile + koff : abase_fill;
                const half_t* bbase = last ? b_tile + koff : bbase_fill;
                const unsigned stage = last ? lds_wave + (unsigned)a_off(kt + STAGES) : stage_fill;
#pragma unroll
                for (int m = 0; m < NM; ++m) {
                    const int i = m / NT, j = m % NT;
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(bf[cur][j], af[cur][i], acc[i][j], 0, 0, 0);
#pragma unroll
                    for (int r = m; r < MT + NT; r += NM) {  // same order as load_frags
                        if (r == 0) af[nxt][0] = *reinterpret_cast<const half8_t*>(sa + fr_off[rs]);
                        else if (r <= NT) bf[nxt][r - 1] = *reinterpret_cast<const half8_t*>(sb + (r - 1) * 32 * RB + fr_off[rs]);
                        else af[nxt][r - NT] = *reinterpret_cast<const half8_t*>(sa + (r - NT) * 32 * RB + fr_off[rs]);
                    }
                    if (last) {
                        if constexpr (decltype(more)::value) issue_segment(0, m, abase, bbase, stage);
                    } else {
                        if constexpr (decltype(fill)::value) issue_segment(ks + 1, m, abase, bbase, stage);
                    }
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
        };
        {
            using T = std::true_type;
            using F = std::false_type;
            int kt = 0;
            for (; kt + STAGES < KT; ++kt) tile(kt, T{}, T{}, T{});
            for (; kt + STAGES - 1 < KT && kt + 1 < KT; ++kt) tile(kt, T{}, T{}, F{});
            for (; kt + 1 < KT; ++kt) tile(kt, T{}, F{}, F{});
            if (KT > 0) tile(KT - 1, F{}, F{}, F{});
        }
    } else {
        for (int kt = 0; kt < KT; ++kt) {
            sync_for(kt);
            issue_after_sync(kt);
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                half8_t af[MT], bf[NT];
                load_frags(af, bf, kt, ks);
                mfmas(af, bf);
            }
        }
    }

    // ---- epilogue.  acc[i][j][4*g + r] = C[row i*32 + lane%32][col j*32 + 8*g + 4*(lane/32) + r] ----
    const int e_row = lane & 31;
    const int e_col = (lane >> 5) * 4;
    const int row_base = m0 + wm * TM, col_base = GATED ? n0 + wn * (TN / 2) : n0 + wn * TN;
    const int tile_m0 = m0, tile_n0 = n0;   // setup_tile() moves m0 and n0 on to the next tile before the stores
    constexpr int RS = TN * 2 + 16;          // bytes per staged row of the fp16 epilogue
    // (a gated launch is always staged: the host launches it only for 16-byte aligned rows of C and without split)
    const bool staged = GATED || (!partial && (N % 8) == 0 && (ldc % 8) == 0 && (reinterpret_cast<uintptr_t>(C) & 15u) == 0);
    const int next_vb = vb + (int)gridDim.x;
    const bool has_next_tile = PERSIST && next_vb < total_tiles;
    if (staged || has_next_tile) {
        // all wavefronts are done with the operand tiles before anyone overwrites them
        asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");
    }
    int stage_area = 0;
    if constexpr (PERSIST) {
        static_assert(!PERSIST || NW * 32 * RS <= STAGE_BYTES, "C staging must fit the last stage");
        if (has_next_tile) {
            // the first K tiles of the next C tile go to stages 0 .. STAGES-2 while this tile's C leaves
            // through the last stage
            setup_tile(next_vb);
#pragma unroll
            for (int st = 0; st < STAGES - 1; ++st)
                if (st < KT) issue_tile(st);
            stage_area = (STAGES - 1) * STAGE_BYTES;
        }
    }
    if constexpr (GATED) {
        // 32 x TN halves per block through the wavefront's LDS region as below; read back as pairs of 16-byte pieces
        // TN/2 columns apart: out = half(silu(a) * b) of the two rounded projections, the arithmetic of SiluMulOp.
        constexpr int TN2 = TN / 2, CHG = TN2 / 8, RPRG = 64 / CHG, PASSG = (32 + RPRG - 1) / RPRG;
        static_assert(NW * 32 * RS <= STAGES * STAGE_BYTES, "staging area must fit the ring");
        unsigned char* region = smem_raw + stage_area + wave * (32 * RS);
        const int n_out = N / 2;
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
            for (int q = 0; q < PASSG; ++q) {
                const int r = q * RPRG + lane / CHG, c = lane % CHG;
                const int row = row_base + i * 32 + r, col = col_base + c * 8;
                if (lane >= RPRG * CHG || r >= 32 || row >= M || col >= n_out) continue;
                const half8_t va = *reinterpret_cast<const half8_t*>(region + r * RS + c * 16);
                const half8_t vb = *reinterpret_cast<const half8_t*>(region + r * RS + TN2 * 2 + c * 16);
                half8_t o;
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    const float x = (float)va[e];
                    o[e] = (half_t)(x * (1.0f / (1.0f + expf(-x))) * (float)vb[e]);
                }
                *reinterpret_cast<half8_t*>(C + (size_t)row * ldc + col) = o;
            }
        }
    } else if (TICKETS && partial && tickets) {
        // split-K in one launch.  The fp32 partial sums of this split leave as device-coherent 16-byte stores (sc1:
        // written through to the level all XCDs share); every wavefront waits until its stores are acknowledged,
        // the workgroup barrier collects those waits, and then one thread draws the tile's ticket with a
        // device-scope atomic.  The workgroup that draws the last ticket of a tile reads all slabs of the tile back
        // with device-coherent loads, adds them in split order, exactly the sum and rounding of
        // splitk_reduce_kernel, writes fp16 C and sets the ticket back to zero for the next launch.  The ring is
        // drained at this point, so the waits cost nothing that the epilogue would not have waited for anyway.
        // The host guarantees N % 8 == 0, 16-byte aligned C and slabs, and byte offsets below 2^31.
        typedef unsigned u32x4_t __attribute__((ext_vector_type(4)));
        const unsigned slab_bytes = (unsigned)M * (unsigned)N * 4u;
        const __amdgpu_buffer_rsrc_t slabs = __builtin_amdgcn_make_buffer_rsrc(partial, 0, (int)(slab_bytes * gridDim.z), 0x00020000);
        constexpr int kCoherent = 16;   // sc1
#pragma unroll
        for (int i = 0; i < MT; ++i) {
            const int row = row_base + i * 32 + e_row;
            const unsigned row_off = (unsigned)blockIdx.z * slab_bytes + (unsigned)row * (unsigned)N * 4u;
#pragma unroll
            for (int j = 0; j < NT; ++j)
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    const int col = col_base + j * 32 + g * 8 + e_col;
                    if (row < M && col < N) {
                        float4_t v = {acc[i][j][4 * g], acc[i][j][4 * g + 1], acc[i][j][4 * g + 2], acc[i][j][4 * g + 3]};
                        __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4_t, v), slabs, (int)(row_off + (unsigned)col * 4u), 0, kCoherent);
                    }
                }
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        volatile int* flag = reinterpret_cast<volatile int*>(smem_raw + stage_area);
        if (tid == 0) {
            const unsigned t = __hip_atomic_fetch_add(tickets + vb, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            const int last = (t + 1u == gridDim.z);
            if (last) __hip_atomic_store(tickets + vb, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            *flag = last;
        }
        __syncthreads();
        const bool merge = *flag != 0;
        __syncthreads();   // the flag's word belongs to the next tile's ring once this workgroup moves on
        if (merge) {
            constexpr int C4 = BN / 4, THREADS = NW * 64, ITEMS = BM * C4 / THREADS, U = ITEMS < 4 ? ITEMS : 4;
            static_assert(BM * C4 % THREADS == 0 && ITEMS % U == 0, "tile must split evenly over the threads");
            const int splits = (int)gridDim.z;
            for (int it0 = 0; it0 < ITEMS; it0 += U) {
                float4_t sum[U];
                unsigned off[U];
                bool ok[U];
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    const int idx = (it0 + u) * THREADS + tid;
                    const int row = tile_m0 + idx / C4, col = tile_n0 + (idx % C4) * 4;
                    ok[u] = row < M && col < N;
                    off[u] = ok[u] ? ((unsigned)row * (unsigned)N + (unsigned)col) * 4u : 0u;
                }
                for (int s0 = 0; s0 < splits; s0 += 4) {
                    u32x4_t v[4][U];
#pragma unroll
                    for (int k = 0; k < 4; ++k)
                        if (s0 + k < splits) {
#pragma unroll
                            for (int u = 0; u < U; ++u)
                                v[k][u] = __builtin_amdgcn_raw_buffer_load_b128(slabs, (int)(off[u] + (unsigned)(s0 + k) * slab_bytes), 0, kCoherent);
                        }
#pragma unroll
                    for (int k = 0; k < 4; ++k)
                        if (s0 + k < splits) {
#pragma unroll
                            for (int u = 0; u < U; ++u) {
                                const float4_t f = __builtin_bit_cast(float4_t, v[k][u]);
                                sum[u] = (s0 + k == 0) ? f : sum[u] + f;
                            }
                        }
                }
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    if (!ok[u]) continue;
                    const int idx = (it0 + u) * THREADS + tid;
                    const int row = tile_m0 + idx / C4, col = tile_n0 + (idx % C4) * 4;
                    half4_t h = {(half_t)sum[u][0], (half_t)sum[u][1], (half_t)sum[u][2], (half_t)sum[u][3]};
                    *reinterpret_cast<half4_t*>(C + (size_t)row * ldc + col) = h;
                }
            }
        }
    } else if (partial) {
        // split-K with a second kernel: fp32 partial sums, four consecutive columns (16 bytes) per store where the row allows it
        const bool vec = (N % 4) == 0;
#pragma unroll
        for (int i = 0; i < MT; ++i) {
            const int row = row_base + i * 32 + e_row;
            if (row >= M) continue;
            float* prow = partial + ((size_t)blockIdx.z * M + row) * N;
#pragma unroll
            for (int j = 0; j < NT; ++j)
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    const int col = col_base + j * 32 + g * 8 + e_col;
                    if (vec && col + 3 < N) {
                        float4_t v = {acc[i][j][4 * g], acc[i][j][4 * g + 1], acc[i][j][4 * g + 2], acc[i][j][4 * g + 3]};
                        *reinterpret_cast<float4_t*>(prow + col) = v;
                    } else {
#pragma unroll
                        for (int r = 0; r < 4; ++r)
                            if (col + r < N) prow[col + r] = acc[i][j][4 * g + r];
                    }
                }
        }
    } else if (staged) {
        // fp16 output through LDS: every wavefront turns 32 x TN blocks of its accumulators into row-major
        // halves in a private LDS region (8-byte writes), reads them back 16 bytes per lane and stores
        // whole 16-byte pieces of C rows (TN = 64: full 128-byte lines).  Rows are padded by 16 bytes so
        // that the 32 rows of one write land in different banks.
        constexpr int CH = TN / 8;               // 16-byte chunks per row
        constexpr int RPR = 64 / CH;             // rows per wavefront-wide read (lanes beyond RPR * CH idle)
        constexpr int PASSES = (32 + RPR - 1) / RPR;
        static_assert(NW * 32 * RS <= STAGES * STAGE_BYTES, "staging area must fit the ring");
        unsigned char* region = smem_raw + stage_area + wave * (32 * RS);
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
    } else {
#pragma unroll
        for (int i = 0; i < MT; ++i) {
            const int row = row_base + i * 32 + e_row;
            if (row >= M) continue;
#pragma unroll
            for (int j = 0; j < NT; ++j)
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    const int col = col_base + j * 32 + (e / 4) * 8 + e_col + (e % 4);
                    if (col < N) C[(size_t)row * ldc + col] = (half_t)acc[i][j][e];
                }
        }
    }
    if (!has_next_tile) break;
    if constexpr (STAGES > 2) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    vb = next_vb;
  }
}

// out[i] = half(sum over splits, in split order, of partial[s][i]): second pass of split-K.
__global__ void __launch_bounds__(256)
splitk_reduce_kernel(half_t* __restrict__ out, const float* __restrict__ partial, size_t n, int splits) {
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t i = ((size_t)blockIdx.x * blockDim.x + threadIdx.x) * 4; i < n; i += stride * 4) {
        if (i + 4 <= n) {
            float4_t v = *reinterpret_cast<const float4_t*>(partial + i);
            for (int s = 1; s < splits; ++s) v += *reinterpret_cast<const float4_t*>(partial + (size_t)s * n + i);
            half4_t h = {(half_t)v[0], (half_t)v[1], (half_t)v[2], (half_t)v[3]};
            *reinterpret_cast<half4_t*>(out + i) = h;
        } else {
            for (size_t j = i; j < n; ++j) {
                float v = partial[j];
                for (int s = 1; s < splits; ++s) v += partial[(size_t)s * n + j];
                out[j] = (half_t)v;
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
    int stages;  // 0: register-staged kernel (any K % 8 == 0); >= 2: direct-to-LDS ring (K % bk == 0)
    HgemmKernel kernel;
    bool persistent;  // the kernel walks tiles blockIdx.x, + gridDim.x, ... (same predicate as PERSIST in the kernel)
    HgemmKernel gated_kernel;  // the same kernel with the SwiGLU gate in its epilogue (pipelined variants), else null
};

#define TL_HGEMM_VARIANT(BM, BN, BK, WM, WN) \
    { "t" #BM "x" #BN "x" #BK "w" #WM "x" #WN, BM, BN, BK, WM * WN * 64, 0, hgemm_f16_mfma_kernel<BM, BN, BK, WM, WN>, false, nullptr }
#define TL_HGEMM_DLDS(BM, BN, BK, WM, WN, ST) \
    { "d" #BM "x" #BN "x" #BK "w" #WM "x" #WN "s" #ST, BM, BN, BK, WM * WN * 64, ST, \
      hgemm_f16_dlds_kernel<BM, BN, BK, WM, WN, ST, 0>, false, nullptr }
#define TL_HGEMM_PIPE(BM, BN, BK, WM, WN, ST) \
    { "p" #BM "x" #BN "x" #BK "w" #WM "x" #WN "s" #ST, BM, BN, BK, WM * WN * 64, ST, \
      hgemm_f16_dlds_kernel<BM, BN, BK, WM, WN, ST, 1>, \
      (ST) <= 3 && (WM) * (WN) * 32 * ((BN) / (WN) * 2 + 16) <= ((BM) + (BN)) * (BK) * 2, \
      hgemm_f16_dlds_kernel<BM, BN, BK, WM, WN, ST, 2> }

static const HgemmVariant g_variants[] = {
    {"auto", 0, 0, 0, 0, 0, nullptr, false, nullptr},
    // register-staged kernel: serves K % 64 != 0 (index 1 is the fallback of launch_hgemm)
    TL_HGEMM_VARIANT(128, 128, 64, 2, 2),  // 1
    TL_HGEMM_VARIANT(256, 256, 64, 2, 4),  // 2
    TL_HGEMM_VARIANT(64, 64, 64, 2, 2),    // 3
    // direct-to-LDS ring, fragments read step by step (no register double buffering)
    TL_HGEMM_DLDS(256, 256, 64, 2, 4, 2),  // 4
    TL_HGEMM_DLDS(128, 128, 64, 2, 2, 4),  // 5
    TL_HGEMM_DLDS(256, 256, 32, 2, 4, 4),  // 6   BK = 32: half cache lines per row, measured slower
    // direct-to-LDS ring, pipelined (dispatch picks among these)
    TL_HGEMM_PIPE(256, 256, 64, 2, 4, 2),  // 7   8 wavefronts of 128x64
    TL_HGEMM_PIPE(256, 256, 64, 2, 2, 2),  // 8   4 wavefronts of 128x128
    TL_HGEMM_PIPE(128, 256, 64, 2, 4, 2),  // 9
    TL_HGEMM_PIPE(128, 256, 64, 2, 4, 3),  // 10
    TL_HGEMM_PIPE(256, 128, 64, 2, 4, 2),  // 11
    TL_HGEMM_PIPE(256, 128, 64, 2, 4, 3),  // 12
    TL_HGEMM_PIPE(128, 128, 64, 2, 4, 2),  // 13
    TL_HGEMM_PIPE(128, 128, 64, 2, 4, 4),  // 14
    TL_HGEMM_PIPE(128, 64, 64, 2, 2, 4),   // 15  few rows: narrow B tiles, deep ring
    TL_HGEMM_PIPE(128, 64, 64, 4, 1, 4),   // 16
    // 192 columns: tile counts that fit 256 CUs where 128 and 256 columns do not (N = 11008, 12288)
    TL_HGEMM_PIPE(128, 192, 64, 4, 2, 4),  // 17
    TL_HGEMM_PIPE(256, 192, 64, 2, 2, 2),  // 18
    // few rows: four wavefronts of 64x64 read a quarter fewer fragment bytes from LDS than eight of 64x32
    TL_HGEMM_PIPE(128, 128, 64, 2, 2, 4),  // 19
    // hgemm_agpr.hip: one wavefront per SIMD, 16x16x32 MFMAs, accumulators in AGPRs (stages < 0 marks it)
    {"a256x256x64w2x2", 256, 256, 64, 256, -1, nullptr, true, nullptr},  // 20
    {"a256x128x64w2x2", 256, 128, 64, 256, -2, nullptr, false, nullptr},  // 21
};

static constexpr int kNumVariants = sizeof(g_variants) / sizeof(g_variants[0]);
// Tuning knobs (tests and sweeps set them, any thread may read them while launching).
static std::atomic<int> g_forced_variant{0};
static std::atomic<bool> g_attr_set[kNumVariants], g_attr_set_gated[kNumVariants];

static std::atomic<int> g_forced_splits{0};  // 0 = automatic
static std::atomic<int> g_last_variant{0}, g_last_splits{0};   // what the most recent tile launch used
static std::atomic<bool> g_last_one_launch{false};             // its split-K was merged inside the launch
static std::atomic<int> g_forced_rot_tile{-1}, g_forced_rot_xcd{-1};  // -1 = automatic
static std::atomic<int> g_forced_band{0};                              // 0 = automatic
// Where the slabs of a split K are added up: 0 = automatic = 2 = by the second kernel; 1 = inside the GEMM launch, by the
// workgroup that finishes a tile's last split.  The second kernel is the default because it is faster (same box, W from
// HBM, second kernel against in-launch: 128x4096x4096 15.2 / 17.0 us, 128x11008x4096 29.9 / 36.1, 128x4096x11008
// 32.2 / 36.3, 256x4096x11008 40.8 / 47.2, 512x4096x11008 60.8 / 69.4): the slabs have to leave as write-through
// stores and come back through device-coherent loads, a serial chain of store acknowledgement, ticket and reload of
// about 4 us at the end of every tile, where the second kernel reads slabs that still sit in the L2s with every CU.
static std::atomic<int> g_splitk_merge_mode{0};
static std::atomic<int> g_agpr_mode{0};   // 0 = the dispatch may take the kernels of hgemm_agpr.hip, -1 = never

// Library-owned fp32 workspace for split-K partial sums, grown on demand (stream-ordered reuse).
static Workspace g_splitk;

static size_t lds_bytes(const HgemmVariant& v) {
    if (v.stages > 0) return (size_t)v.stages * (v.bm + v.bn) * v.bk * sizeof(half_t);
    return (size_t)2 * (v.bm + v.bn) * (v.bk + kPad) * sizeof(half_t);
}

static int hgemm_variant_index(const char* name) {
    for (int i = 0; i < kNumVariants; ++i)
        if (strcmp(g_variants[i].name, name) == 0) return i;
    return 1;
}

// Measured on MI355X over the Llama2-7B prefill shapes (M in {128, 512, 1024, 2048}), B streamed from HBM.
// More than 512 rows: the variant with the cheapest schedule and its cost in rounds of 256x256 tiles (see the
// comment above pick_variant for the constants).
struct HgemmPlan {
    int variant;
    double cost;
};
// more than 512 rows, few 128x256 tiles and a long K: split K instead of narrowing the tile
static bool hgemm_many_rows_split(size_t M, size_t N, size_t K, int cus) {
    const size_t t = ((M + 127) / 128) * ((N + 255) / 256);
    return M > 512 && K >= 8192 && t * 2 <= (size_t)cus && t * 22016 <= (size_t)cus * K;
}

// fast_big: the problem comes in whole 256x256 tiles that hgemm_agpr.hip's kernel can take (a round of them then costs
// 0.87 of a round of the ring kernel's: 2048x32000x4096 405 against 475 us on one box)
// fast_mid: the same for 128x256 tiles and the 256x128 kernel of that file (0.565 instead of 0.613: 2048x4096x11008 148
// against 167 us, 2048x2816x4096 50 against 54.5 us, 2048x4096x4096 64.6 against 66.4 us)
static HgemmPlan plan_many_rows(size_t M, size_t N, size_t K, int cus, bool can_split, bool fast_big = false, bool fast_mid = false) {
    static const int v_big = hgemm_variant_index("p256x256x64w2x4s2");
    static const int v_mid = hgemm_variant_index("p128x256x64w2x4s3");
    static const int v_small = hgemm_variant_index("p128x128x64w2x4s2");
    static const int v_few_128x128 = hgemm_variant_index("p128x128x64w2x2s4");
    static const int v_256x192 = hgemm_variant_index("p256x192x64w2x2s2");
    auto tiles = [&](int bm, int bn) { return ((M + bm - 1) / bm) * ((N + bn - 1) / bn); };
    auto cost = [&](size_t t, size_t slots, double round_cost) {
        const size_t full = t / slots, rem = t % slots;
        return round_cost * ((double)full + (rem ? 0.65 + 0.3 * (double)rem / (double)slots : 0.0));
    };
    const double c_small = cost(tiles(128, 128), (size_t)cus * 2, 0.66);
    // A problem that leaves half the CUs without a 128x256 tile: with a long K the tile stays and K is split over
    // two to four workgroups (launch_hgemm_cols), as long as a split keeps about 2700 values of K (640x4096x11008:
    // 72 against 103 us, 896x4096x11008: 97 against 103 us, 640x4096x8192: 57 against 67 us; from 1024x4096x11008
    // and 896x4096x8192 on the slabs cost what the split wins); otherwise it spreads wider as 128x128 tiles.
    if (tiles(128, 256) * 2 <= (size_t)cus) {
        if (can_split && hgemm_many_rows_split(M, N, K, cus)) return {v_mid, c_small};
        return {v_few_128x128, c_small};
    }
    const double c_big = cost(tiles(256, 256), (size_t)cus, fast_big ? 0.87 : 1.0);
    const double c_mid = cost(tiles(128, 256), (size_t)cus, fast_mid ? 0.565 : 0.613);
    const double c_192 = cost(tiles(256, 192), (size_t)cus, 0.865);   // three quarters of the work at 0.865 of the cost
    int best = v_big;
    double c = c_big;
    if (c_192 < c * 0.97) { best = v_256x192; c = c_192; }
    if (c_mid < c * 0.97) { best = v_mid; c = c_mid; }
    if (c_small < c * 0.97) { best = v_small; c = c_small; }
    return {best, c};
}

// Up to 512 rows the problem is bound by streaming B once: the largest tile shape that still gives one
// round of at least 0.6 x CUs workgroups, with a deep (3-4 stage) ring; if even 128x64 tiles are too few,
// K is split until the chip is full (see launch_hgemm).
// More rows: the tile shape with the cheapest schedule.  One round of 256x256 tiles on every CU costs R; a
// round of 128x256 tiles (one workgroup per CU, three-stage ring: with B streamed from HBM a 0.6 us tile step
// is shorter than the memory latency two stages can hide) does half the work in 0.61 R, a round of 128x128
// tiles (two per CU) in 0.66 R, a round of 256x192 tiles in 0.865 R, so the big tile wins unless its last round is
// mostly empty; a partly filled round of a fraction f of the CUs costs about (0.65 + 0.3 f) of a full one (fewer
// busy CUs clock higher).
// Splitting K or peeling the last round off into a second K-split launch lost to this on every shape tried.
// What does pay when whole rounds of 256x256 tiles are followed by a mostly empty one: launch the whole rounds as one
// column range of C and the remaining columns as a second launch with whatever tiles suit THAT problem
// (launch_hgemm; 2048x11008x4096: 344 big tiles = one round + 88 tiles, or one round + 176 tiles of 128x256).
// Up to 512 rows and from 5120 columns on, 128x128 tiles on four wavefronts, split over K until they fill one round
// of the chip, are as fast as or faster than the rules of pick_variant wherever they fill at least 67 % of the
// compute units (60 % from 192 rows on) with K loops of 1024 to 8192 (sweep of seven tile shapes x six split counts
// over 152 shapes, M = 48 .. 512, projections of Llama-size models 2048 to 8192 wide: 256x8192x8192 71.6 -> 52.8 us,
// 384x6144x4096 52.1 -> 37.7, 256x5120x5120 38.0 -> 29.7, 48x12288x4096 26.8 -> 23.9; at most 5 % slower on the shapes
// of that sweep it applies to).  With few rows
// the kernel is bound by HBM long before the K loop of one workgroup is: then the smallest split whose K loop
// (0.53 us per K tile of 64, less for a partly filled row tile) stays below the time HBM needs for W is enough, and
// every further split only adds slabs.  Returns the number of splits, 0 when the rule does not apply.
static int square_tile_splits(size_t M, size_t N, size_t K, int cus, bool can_split) {
    if (M > 512 || N < 5120 || K % 64 != 0) return 0;
    const size_t t = ((M + 127) / 128) * ((N + 127) / 128);
    if (t > (size_t)cus) return 0;
    const double hbm_us = (double)(N + M) * K * 2.0 / 5.5e6;
    const double per_k_us = M < 128 ? 0.53 * (0.69 * M + 0.31 * 128 + 128) / 256 : 0.53;
    const size_t KT = K / 64;
    int sp = 1;
    for (int s : {1, 2, 3, 4, 6}) {
        if (t * s > (size_t)cus) break;
        if (s > 1 && (!can_split || K < 4096 || K < (size_t)s * 1024)) break;
        sp = s;
        if ((double)((KT + s - 1) / s) * per_k_us <= hbm_us) break;
    }
    if (K > (size_t)sp * 8192 || t * sp * 100 < (size_t)cus * (M >= 192 ? 60 : 67)) return 0;
    return sp;
}

static int pick_variant(size_t M, size_t N, size_t K, int cus, bool can_split, bool fast_big = false, bool fast_mid = false) {
    static const int v_big = hgemm_variant_index("p256x256x64w2x4s2");
    static const int v_mid = hgemm_variant_index("p128x256x64w2x4s3");
    static const int v_few_256x128 = hgemm_variant_index("p256x128x64w2x4s3");
    static const int v_few_128x128 = hgemm_variant_index("p128x128x64w2x2s4");
    static const int v_few_128x64 = hgemm_variant_index("p128x64x64w4x1s4");
    static const int v_few_128x192 = hgemm_variant_index("p128x192x64w4x2s4");
    auto tiles = [&](int bm, int bn) { return ((M + bm - 1) / bm) * ((N + bn - 1) / bn); };
    if (M <= 512 && tiles(256, 256) <= (size_t)cus) {
        const size_t enough = (size_t)cus * 6 / 10;
        if (tiles(256, 256) >= enough) return v_big;
        // one round either way: 192 columns put more CUs to work than 256 (512x12288x4096: 58 vs 65 us)
        // (not with a very long K that two splits of 128x256 tiles cover in one round: 512x8192x28672 319 -> 237 us)
        const bool split_wide = can_split && K >= 16384 && M >= 256 && tiles(128, 256) * 2 <= (size_t)cus;
        if (M > 128 && tiles(128, 192) >= enough && tiles(128, 192) <= (size_t)cus && !split_wide) return v_few_128x192;
        // one row of 256-row tiles reads every row of W once; two rows of 128-row tiles read it twice (38 shapes with
        // 192 and 256 rows: 256x128 ahead of 128x256 by 1-9 %, 256x32000x4096 90.4 -> 82.3 us)
        if (M > 128 && M <= 256 && tiles(256, 128) >= enough) return v_few_256x128;
        if (M > 128 && tiles(128, 256) >= enough) return v_mid;   // from 257 rows on ahead of 256x128 at equal tile counts
        if (M > 128 && tiles(256, 128) >= enough) return v_few_256x128;
        // A long K is split instead of narrowing the tile: wider tiles pull fewer bytes through a CU per output, and
        // the slabs are small next to W (256x4096x11008: 128x128 tiles on four splits 40-43 us, 128x64 on two 48-49 us;
        // 384 and 512 rows: 128x256 on four splits 54 and 62 us against 61 and 65 us).  With fewer than 256 rows the
        // second row of 128-row tiles is mostly padding and the narrow tile stays ahead.
        if (can_split && K >= 8192 && M >= 256 && tiles(128, 256) * 4 >= enough) return v_mid;
        if (can_split && K >= 8192 && M >= 256 && tiles(128, 128) * 4 >= enough) return v_few_128x128;
        if (tiles(128, 128) >= enough || (K >= 8192 && tiles(128, 128) * 2 >= enough)) return v_few_128x128;
        // two rounds of narrow tiles lose to one partly filled round of square ones (384x6144x4096: 52 -> 38 us)
        if (tiles(128, 64) > (size_t)cus) return v_few_128x128;
        return v_few_128x64;
    }
    return plan_many_rows(M, N, K, cus, can_split, fast_big, fast_mid).variant;
}

// One launch (plus the ordered reduce when K is split) for columns [0, N) of a C whose rows are ldc elements apart.
// forced_vi: 0 = dispatch by shape.
// gate: 0, or the distance in rows between the two matrices stacked in B of a gated launch (HgemmArgs::gate); N then
// counts the rows of both and C has N / 2 columns.
static int launch_hgemm_cols(const void* A, const void* B, void* C, size_t M, size_t N, size_t K, size_t ldc, size_t batch,
                             size_t sa, size_t sb, size_t sc, float** partials_out, int* splits_out,
                             Workspace::Lease* lease_out, int forced_vi, size_t gate = 0);

int launch_hgemm(const void* A, const void* B, void* C, size_t M, size_t N, size_t K, size_t batch, size_t sa,
                 size_t sb, size_t sc, float** partials_out, int* splits_out, Workspace::Lease* lease_out, size_t gate) {
    const size_t ldc_all = gate ? N / 2 : N;   // row stride of C; a gated launch writes one column per pair of rows of B
    // Whole rounds of 256x256 tiles, then the remaining columns as a problem of their own, when the schedule model
    // says the two launches beat the best single one.  Only for many rows (no split-K there, so C is written
    // directly and a column range of it is just a pointer offset with the full row stride).
    if (batch == 1 && M > 512 && N <= 0x7fffffffu && K > 0 && K % 64 == 0 && K <= ((size_t)1 << 22) && N % 8 == 0 &&
        aligned16(A) && aligned16(B) && aligned16(C) && g_forced_variant.load() == 0 && g_forced_splits.load() <= 1) {
        static const int v_big = hgemm_variant_index("p256x256x64w2x4s2");
        const int cus = device_info().cu_count;
        const size_t tiles_m = (M + 255) / 256;
        if (cus > 0 && tiles_m <= (size_t)cus) {
            const size_t cols_per_round = (size_t)cus / tiles_m, col_tiles = (N + 255) / 256;
            const size_t full = col_tiles / cols_per_round, rem = col_tiles % cols_per_round;
            if (full >= 1 && rem > 0) {
                const size_t N1 = full * cols_per_round * 256;
                const size_t c1 = gate ? N1 / 2 : N1;   // first column of C (and row of B) of the second launch
                const bool agpr_ok = g_agpr_mode.load() == 0;   // (the 256x128 kernel has no gated build)
                const bool fast_all = agpr_ok && hgemm_big_applies(A, B, C, M, N, K, ldc_all, gate);
                const bool fast_first = agpr_ok && hgemm_big_applies(A, B, C, M, N1, K, ldc_all, gate);
                const bool fast_rest = agpr_ok && hgemm_big_applies(A, (const half_t*)B + c1 * K, (half_t*)C + c1, M, N - N1, K, ldc_all, gate);
                const bool mid_all = agpr_ok && gate == 0 && hgemm_mid_applies(A, B, C, M, N, K, ldc_all);
                const bool mid_rest = agpr_ok && gate == 0 && hgemm_mid_applies(A, (const half_t*)B + c1 * K, (half_t*)C + c1, M, N - N1, K, ldc_all);
                const double whole = plan_many_rows(M, N, K, cus, true, fast_all, mid_all).cost;
                const double split = (fast_first ? 0.87 : 1.0) * (double)full * (double)(tiles_m * cols_per_round) / (double)cus +
                                     plan_many_rows(M, N - N1, K, cus, false, fast_rest, mid_rest).cost + 0.04;   // 0.04: the second launch's ramp
                if (split < whole * 0.97) {
                    int rc = launch_hgemm_cols(A, B, C, M, N1, K, ldc_all, 1, 0, 0, 0, nullptr, nullptr, nullptr, v_big, gate);
                    if (rc != TL_OK) return rc;
                    if (splits_out) *splits_out = 1;
                    return launch_hgemm_cols(A, (const half_t*)B + c1 * K, (half_t*)C + c1, M, N - N1, K, ldc_all, 1, 0, 0, 0,
                                             nullptr, nullptr, nullptr, 0, gate);
                }
            }
        }
    }
    return launch_hgemm_cols(A, B, C, M, N, K, ldc_all, batch, sa, sb, sc, partials_out, splits_out, lease_out, 0, gate);
}

static int launch_hgemm_cols(const void* A, const void* B, void* C, size_t M, size_t N, size_t K, size_t ldc, size_t batch,
                             size_t sa, size_t sb, size_t sc, float** partials_out, int* splits_out,
                             Workspace::Lease* lease_out, int forced_vi, size_t gate) {
    Workspace::Lease own_lease;
    Workspace::Lease& lease = lease_out ? *lease_out : own_lease;
    if (splits_out) *splits_out = 1;
    if (M == 0 || N == 0 || batch == 0) return TL_OK;
    TL_REQUIRE(M <= 0x7fffffffu && N <= 0x7fffffffu && K <= 0x7fffffffu && batch <= 65535,
               "hgemm: size out of range");
    hipStream_t st = stream();
    if (K == 0) {
        for (size_t b = 0; b < batch; ++b) {
            int rc = launch_fill_f16((half_t*)C + b * sc, 0, gate ? M * (N / 2) : M * N);
            if (rc != TL_OK) return rc;
        }
        return TL_OK;
    }
    const bool vec_ok = (K % 8 == 0) && aligned16(A) && aligned16(B) &&
                        (batch == 1 || (sa % 8 == 0 && sb % 8 == 0));
    if (!vec_ok) {
        TL_REQUIRE(gate == 0, "hgemm: a gated launch needs K %% 8 == 0 and 16-byte aligned operands");
        TL_REQUIRE(ldc == N, "hgemm generic path: a column range of C is not supported");
        dim3 grid((unsigned)((N + 15) / 16), (unsigned)((M + 15) / 16), (unsigned)batch);
        TL_REQUIRE(grid.y <= 65535, "hgemm generic path: M too large (%zu)", M);
        hipLaunchKernelGGL((gemm_generic_kernel<half_t, float>), grid, dim3(256), 0, st, (const half_t*)A,
                           (const half_t*)B, (half_t*)C, (int)M, (int)N, (int)K, (long)sa, (long)sb, (long)sc);
        TL_CHECK_LAUNCH("gemm_generic_kernel<half>");
        return TL_OK;
    }
    const int forced_variant = forced_vi ? forced_vi : g_forced_variant.load();
    // a handful of rows and K up to 4096: X resident in registers, W streamed once, no split of K
    if (gate == 0 && forced_variant == 0 && g_forced_splits.load() == 0 && aligned16(C) &&
        hgemm_fewrows_applies(M, N, K, ldc, batch)) {
        g_last_variant = -1;
        g_last_splits = 1;
        return launch_hgemm_fewrows(A, B, C, M, N, K, ldc);
    }
    const bool can_split = batch == 1 && ldc == N;   // the second pass of a split K writes a dense C
    // whole 256x256 tiles of a single dense C: where the 256x256 ring kernel would run, hgemm_agpr.hip's kernel does
    const bool agpr_ok = batch == 1 && g_forced_variant.load() == 0 && g_agpr_mode.load() == 0;
    const bool fast_big = agpr_ok && hgemm_big_applies(A, B, C, M, N, K, ldc, gate);
    const bool fast_mid = agpr_ok && gate == 0 && M > 512 && hgemm_mid_applies(A, B, C, M, N, K, ldc);
    int vi = forced_variant ? forced_variant : pick_variant(M, N, K, device_info().cu_count, can_split, fast_big, fast_mid);
    {
        static const int v_big = hgemm_variant_index("p256x256x64w2x4s2");
        static const int v_fast = hgemm_variant_index("a256x256x64w2x2");
        static const int v_mid = hgemm_variant_index("p128x256x64w2x4s3");
        static const int v_fast_mid = hgemm_variant_index("a256x128x64w2x2");
        if (fast_big && vi == v_big) vi = v_fast;
        // (not where the 128x256 ring kernel is about to split K: the 256x128 kernel has no split)
        if (fast_mid && vi == v_mid && !(can_split && hgemm_many_rows_split(M, N, K, device_info().cu_count))) vi = v_fast_mid;
    }
    int square_splits = 0;
    if (forced_variant == 0 && g_forced_splits.load() == 0) {
        square_splits = square_tile_splits(M, N, K, device_info().cu_count, can_split);
        static const int v_square = hgemm_variant_index("p128x128x64w2x2s4");
        if (square_splits > 0) vi = v_square;
    }
    if (g_variants[vi].stages < 0) {
        // whole tiles of one fp16 C, no split (and no gate on the 256x128 tile); anything else falls back to the ring kernel
        const int forced_band = g_forced_band.load();
        const int rt = g_forced_rot_tile.load(), rx = g_forced_rot_xcd.load();
        const bool mid = g_variants[vi].stages == -2;
        // bands of four rows of tiles: the 32 tiles an XCD runs at a time then cover 4 panels of A and 8 of B (measured
        // against bands of 8, same box: 2048x32000x4096 392 -> 378 us, 2048x22016x4096 286 -> 275, 2048x4096x11008 147 -> 142,
        // 8192x8192x8192 equal)
        const int band = forced_band > 0 ? forced_band : 4, rot_tile = rt >= 0 ? rt : 0, rot_xcd = rx >= 0 ? rx : (int)(K / 64 / 8);
        if (batch == 1 && (mid ? gate == 0 && hgemm_mid_applies(A, B, C, M, N, K, ldc) : hgemm_big_applies(A, B, C, M, N, K, ldc, gate))) {
            g_last_variant = vi;
            g_last_splits = 1;
            g_last_one_launch = false;
            return mid ? launch_hgemm_mid(A, B, C, M, N, K, ldc, band, rot_tile, rot_xcd)
                       : launch_hgemm_big(A, B, C, M, N, K, ldc, band, rot_tile, rot_xcd, gate);
        }
        static const int v_big = hgemm_variant_index("p256x256x64w2x4s2");
        vi = v_big;
    }
    if (g_variants[vi].stages > 0 && K % g_variants[vi].bk != 0) vi = 1;  // direct-to-LDS path cannot zero-fill a K tail
    // its per-lane byte offsets inside a tile ((rows - 1) * K + 64 halves) are 32-bit
    if (g_variants[vi].stages > 0 && K > ((size_t)1 << 22)) vi = 1;
    const HgemmVariant& v = g_variants[vi];
    const size_t lds = lds_bytes(v);
    const HgemmKernel kernel = gate ? v.gated_kernel : v.kernel;
    if (gate) {
        // what hgemm_gated_applies checks, once more where a violation would fault: the pipelined kernel, a C the
        // staged epilogue can store to in 16-byte pieces, and 32-bit lane offsets that reach both matrices
        TL_REQUIRE(kernel != nullptr && v.stages > 0, "hgemm: variant %s has no gated kernel", v.name);
        TL_REQUIRE(batch == 1 && N % 16 == 0 && ldc % 8 == 0 && aligned16(C) && gate >= N / 2 &&
                       (gate + N / 2) * K * sizeof(half_t) < ((size_t)1 << 32),
                   "hgemm: gated launch outside its limits (N=%zu ldc=%zu gate=%zu K=%zu)", N, ldc, gate, K);
    }
    std::atomic<bool>& attr_set = gate ? g_attr_set_gated[vi] : g_attr_set[vi];
    if (lds > 64 * 1024 && !attr_set.load()) {
        TL_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
        attr_set.store(true);
    }
    HgemmArgs a;
    a.A = (const half_t*)A;
    a.B = (const half_t*)B;
    a.C = (half_t*)C;
    a.M = (int)M;
    a.N = (int)N;
    a.ldc = (int)ldc;
    a.K = (int)K;
    a.tiles_m = (int)((M + v.bm - 1) / v.bm);
    a.tiles_n = (int)((N + v.bn - 1) / v.bn);
    a.sa = (long)sa;
    a.sb = (long)sb;
    a.sc = (long)sc;
    const size_t nblocks = (size_t)a.tiles_m * a.tiles_n;
    TL_REQUIRE(nblocks <= 0x7fffffffu, "hgemm: too many tiles");
    a.kt_per_split = 0x7fffffff;
    a.partial = nullptr;
    a.tickets = nullptr;
    a.rot_tile = 0;
    a.rot_xcd = 0;
    a.gate = (int)gate;
    // band height that balances the panels of A and B an XCD's 32 tiles pull through its L2
    const int forced_band = g_forced_band.load();
    a.band_m = forced_band > 0 ? forced_band : (v.bm >= 2 * v.bn ? 4 : 8);
    int splits = 1;
    if (v.stages > 0) {
        // Split K when the tile grid alone cannot occupy the chip (prefill with few tokens: the
        // problem is then bound by streaming W, and every CU has to pull on it).
        const int KT = (int)(K / v.bk);
        const int cus = device_info().cu_count;
        splits = g_forced_splits.load();
        if (splits <= 0) {
            // aim at one workgroup per CU, keep at least 8 K tiles per split
            // (only for few rows: with more than 512 rows pick_variant already found a tile shape that
            // fills the chip well enough, and splitting measured slower there)
            splits = M <= 512 ? (int)((size_t)cus / nblocks) : 1;
            if (square_splits > 0) splits = square_splits;
            if (M > 512 && forced_variant == 0 && can_split && hgemm_many_rows_split(M, N, K, cus)) {
                splits = (int)((size_t)cus / nblocks);
                if (splits > 4) splits = 4;
            }
            const int max_by_k = KT / 8 > 0 ? KT / 8 : 1;
            if (splits > max_by_k) splits = max_by_k;
            if (splits > 16) splits = 16;
            if (splits < 1) splits = 1;
        }
        if (splits > KT) splits = KT;
        if (batch != 1 || ldc != N || gate) splits = 1;   // the reduce pass writes a dense C, and it does not gate
        if (splits > 1) {
            a.kt_per_split = (KT + splits - 1) / splits;
            splits = (KT + a.kt_per_split - 1) / a.kt_per_split;
            // [kSplitkTicketWords tile tickets][splits x M x N floats]
            int rc = g_splitk.acquire(kSplitkTicketWords + (size_t)splits * M * N, (size_t)8 << 20, "split-K workspace", &lease);
            if (rc != TL_OK) return rc;
            a.partial = lease.ptr + kSplitkTicketWords;
            // the last workgroup of a tile adds the slabs itself unless the caller folds that pass into its own kernel,
            // there are more tiles than tickets, or C cannot take its 8-byte stores / the slabs exceed 32-bit offsets
            const bool one_launch = !(partials_out && splits_out) && g_splitk_merge_mode.load() == 1 &&
                                    nblocks <= kSplitkTicketWords && N % 8 == 0 && aligned16(C) && v.bm * v.bn <= 128 * 256 &&
                                    (size_t)splits * M * N * sizeof(float) < ((size_t)1 << 31);
            if (one_launch) a.tickets = reinterpret_cast<unsigned*>(lease.ptr);
        }
    }
    g_last_variant = vi;
    g_last_splits = splits;
    // pipelined kernels with up to three stages are persistent: one workgroup per resident slot walks several tiles
    size_t grid_x = nblocks;
    if (v.persistent) {
        const size_t resident = (size_t)device_info().cu_count * ((160 * 1024) / lds > 0 ? (160 * 1024) / lds : 1);
        if (grid_x > resident) grid_x = resident;
    }
    if (v.stages > 0) {
        const int KT = (int)(K / v.bk);
        const int kt_walk = a.kt_per_split < KT ? a.kt_per_split : KT;
        if (M <= 512) {
            // rows of B are private to a column of tiles: spread the tiles over the K offsets
            for (int c : {5, 7, 11, 13, 3, 1})
                if (std::gcd(c, kt_walk) == 1) { a.rot_tile = c; break; }
        } else {
            a.rot_xcd = kt_walk / 8;  // tiles of one XCD keep walking K together (they share panels through its L2)
        }
        const int rt = g_forced_rot_tile.load(), rx = g_forced_rot_xcd.load();
        if (rt >= 0) a.rot_tile = rt;
        if (rx >= 0) a.rot_xcd = rx;
    }
    hipLaunchKernelGGL(kernel, dim3((unsigned)grid_x, (unsigned)batch, (unsigned)splits), dim3(v.threads), lds, st, TL_HGEMM_PASS(a));
    TL_CHECK_LAUNCH(v.name);
    if (splits > 1 && partials_out && splits_out) {
        // the caller folds the second pass of split-K into its own kernel
        *partials_out = a.partial;
        *splits_out = splits;
        return TL_OK;
    }
    g_last_one_launch = a.tickets != nullptr;
    if (splits > 1 && !a.tickets) {
        const size_t n = M * N;
        size_t blocks = (n / 4 + 255) / 256;
        const size_t cap = (size_t)device_info().cu_count * 8;
        if (blocks > cap) blocks = cap;
        if (blocks == 0) blocks = 1;
        hipLaunchKernelGGL(splitk_reduce_kernel, dim3((unsigned)blocks), dim3(256), 0, st, (half_t*)C, a.partial, n, splits);
        TL_CHECK_LAUNCH("splitk_reduce_kernel");
    }
    return TL_OK;
}

int splitk_reset_tickets() { return g_splitk.zero_head(kSplitkTicketWords); }

// One launch can apply the gate when the pipelined kernels serve the shape (K in whole tiles of 64, lane offsets within
// 32 bits over both matrices), C takes 16-byte stores, and no variant without a gated build is forced.
bool hgemm_gated_applies(const void* A, const void* B, const void* C, size_t M, size_t n_out, size_t K, size_t gate) {
    const int forced = g_forced_variant.load();
    return M >= 2 && n_out > 0 && n_out % 8 == 0 && gate >= n_out && K > 0 && K % 64 == 0 && K <= ((size_t)1 << 22) &&
           M <= 0x7fffffffu && 2 * n_out <= 0x7fffffffu && (gate + n_out) * K * sizeof(half_t) < ((size_t)1 << 32) &&
           aligned16(A) && aligned16(B) && aligned16(C) && (forced == 0 || g_variants[forced].gated_kernel != nullptr);
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
    if (M == 1) return tl::launch_gemv(A, B, C, N, K, 1, 0, 0, 0, 0);
    return tl::launch_hgemm(A, B, C, M, N, K, 1, 0, 0, 0);
}

int tl_hgemm_silu_mul_f16(const void* X, const void* W13, void* scratch, void* out, size_t M, size_t hidden, size_t K) {
    TL_ENSURE_INIT();
    if (M == 0 || hidden == 0) return TL_OK;
    TL_REQUIRE(X && W13 && out, "tl_hgemm_silu_mul_f16: null pointer");
    TL_REQUIRE(hidden % 8 == 0, "tl_hgemm_silu_mul_f16: hidden %% 8 != 0 (%zu)", hidden);
    // a handful of rows: the kernel that keeps X in registers plus the separate gate is the faster pair
    if (tl::hgemm_gated_applies(X, W13, out, M, hidden, K, hidden) && !tl::hgemm_fewrows_applies(M, 2 * hidden, K, 2 * hidden, 1))
        return tl::launch_hgemm(X, W13, out, M, 2 * hidden, K, 1, 0, 0, 0, nullptr, nullptr, nullptr, hidden);
    TL_REQUIRE(scratch, "tl_hgemm_silu_mul_f16: this shape takes the two-step path and needs the scratch buffer");
    int rc = tl_matmul2d_f16(X, W13, scratch, M, 2 * hidden, K);
    if (rc != TL_OK) return rc;
    return tl_silu_mul_rows_f16(out, scratch, M, hidden);
}

int tl_matmul2d_batched_f16(const void* A, const void* B, void* C, size_t M, size_t N, size_t K, size_t batch,
                            size_t strideA, size_t strideB, size_t strideC) {
    TL_ENSURE_INIT();
    TL_REQUIRE(A && B && C, "tl_matmul2d_batched_f16: null pointer");
    TL_REQUIRE(batch <= 65535, "tl_matmul2d_batched_f16: batch %zu exceeds 65535", batch);
    if (M == 1) return tl::launch_gemv(A, B, C, N, K, batch, strideA, strideB, strideC, 0);
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

int tl_set_hgemm_splits(int splits) {
    TL_REQUIRE(splits >= 0 && splits <= 64, "tl_set_hgemm_splits: %d out of range [0,64]", splits);
    tl::g_forced_splits = splits;
    return TL_OK;
}

int tl_set_hgemm_k_rotation(int per_tile, int per_xcd) {
    TL_REQUIRE(per_tile >= -1 && per_xcd >= -1, "tl_set_hgemm_k_rotation: negative step");
    tl::g_forced_rot_tile = per_tile;
    tl::g_forced_rot_xcd = per_xcd;
    return TL_OK;
}

int tl_set_hgemm_tile_band(int band) {
    TL_REQUIRE(band >= 0, "tl_set_hgemm_tile_band: negative band");
    tl::g_forced_band = band;
    return TL_OK;
}

int tl_set_hgemm_agpr_kernels(int mode) {
    TL_REQUIRE(mode == 0 || mode == -1, "tl_set_hgemm_agpr_kernels: %d is not 0 or -1", mode);
    tl::g_agpr_mode = mode;
    return TL_OK;
}

int tl_set_hgemm_stamps(void* stamps, size_t capacity) {
    tl::hgemm_agpr_set_stamps(stamps, capacity);
    return TL_OK;
}

int tl_set_hgemm_splitk_merge(int mode) {
    TL_REQUIRE(mode >= 0 && mode <= 2, "tl_set_hgemm_splitk_merge: %d out of range [0,2]", mode);
    tl::g_splitk_merge_mode = mode;
    return TL_OK;
}

int tl_hgemm_last_split_in_launch(void) { return tl::g_last_one_launch.load() ? 1 : 0; }

int tl_hgemm_last_plan(int* variant, int* splits) {
    TL_REQUIRE(variant && splits, "tl_hgemm_last_plan: null output");
    *variant = tl::g_last_variant.load();
    *splits = tl::g_last_splits.load();
    return TL_OK;
}

const char* tl_hgemm_variant_name(int variant) {
    if (variant < 0 || variant >= tl::kNumVariants) return nullptr;
    return tl::g_variants[variant].name;
}

}  // extern "C"
