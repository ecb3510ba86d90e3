// fp16 GEMM for many rows on 256x256 tiles, one wavefront per SIMD: C[M,N] = A[M,K] . B[N,K]^T, fp32 accumulation in the
// MFMA accumulators, one rounding to fp16.  Same contract as the M > 1 branch of the reference's CUDA<half>::matmul2d
// (tensorLib/src/device/cuda/gemm.cu:163-171 -> hgemm_cublas, tensorLib/src/device/cuda/hgemm.cu:20-38); numerics
// follow CPU<half>::matmul2d (tensorLib/src/device/cpu/CPU.cpp:76-89).
//
// What it does differently from hgemm_f16_dlds_kernel (hgemm.hip), and why:
//   * v_mfma_f32_16x16x32_f16 instead of 32x32x16.  The chip is power managed; out of registers, on operands that
//     change with every instruction, the 16x16x32 shape sustains 1.80 PFLOP/s where 32x32x16 sustains 1.64 (it
//     updates an accumulator half as often per flop), so the same schedule runs at a higher clock.
//   * four wavefronts, one per SIMD, each owning a 128x128 piece of the tile: a third fewer fragment bytes read from
//     LDS than eight wavefronts of 128x64.  That takes 256 accumulator registers per lane; they are pinned to the AGPR
//     half of the register file by issuing the MFMA through inline assembly with an "a" constraint (left to itself
//     the compiler keeps accumulators where the other values live, and spills), which leaves the VGPRs to fragments.
//   * operand tiles go global -> LDS with global_load_lds_dwordx4 into a ring of two 64 KB stages, in the layout of the
//     other kernel (a request is 8 rows x 128 bytes in lane order; the 16-byte chunk a lane fetches is permuted so that
//     the fragment reads are free of bank conflicts).  A wavefront issues its 16 requests per K tile one every fourth
//     MFMA (the CU's address path takes 16 cycles per request and four wavefronts share it), the first ones right
//     behind the barrier that frees their stage.
//   * the pipeline never drains between C tiles: a workgroup walks tiles blockIdx.x, + gridDim.x, ..., and the requests
//     and fragment reads that run ahead of the MFMAs simply continue into the next C tile's first K tiles while the
//     current tile's last MFMAs and its epilogue (staged through LDS behind the ring) are still under way.
//   * the K loop is one straight chain of MFMAs per accumulator (every register array is indexed at compile time), so
//     an accumulator never leaves the AGPR tuple it started in.
// Both operands must come in whole tiles (M % 256 == 0, N % 256 == 0: the direct path has no bounds check) and K in an
// even number of tiles of 64, at least four; the dispatch falls back to the other kernel otherwise.
//
// Measured on one MI355X (same box, W from HBM, random operands): 2048x32000x4096 412 us (1.30 PFLOP/s) against 470 us
// for hgemm_f16_dlds_kernel<256,256,64,2,4,2,1>; 8192x8192x8192 768 against 844 us.  The same kernel with the tiles
// travelling through registers (two K tiles in flight per wavefront, ds_write_b128 into the same ring) was built too,
// for either operand or both: 433 us on the first shape.  A ds_write_b128 occupies the LDS pipeline five times as long
// as a fragment read of the same size, which costs more than the deeper prefetch returns.
// What is left between the measured 0.77-0.81 matrix-core occupancy and 1: per K tile a workgroup writes 64 KB into LDS
// (DMA) and reads 128 KB of fragments out of it, 192 KB against 2048 MFMA cycles, i.e. 94 of the 128 bytes per clock the LDS
// moves; a 2x2 arrangement of 128x128 wavefront tiles is the one with the fewest LDS bytes per flop that 512 registers per
// lane allow.  Measured and ruled out: L2 miss latency (W resident in the memory-side cache, a prefetching fifth
// wavefront), the request spacing and barrier position, the four wavefronts issuing requests in the same slots.
#include <atomic>
#include <type_traits>

#include "hgemm_common.h"

namespace tl {

// f(integral_constant<int, I>) for I in [I0, N), expanded at compile time: every register array below is indexed with
// constants, whatever the optimiser's unrolling limits are.
template <int I, int N, typename F>
__device__ __forceinline__ void static_for(F&& f) {
    if constexpr (I < N) {
        f(std::integral_constant<int, I>{});
        static_for<I + 1, N>(f);
    }
}

// acc += b-fragment . a-fragment with the accumulator in AGPRs.  B's fragment goes in as the first operand: the
// accumulator then holds the tile transposed, lane l owning row (l % 16) of C and the four consecutive columns
// 4 * (l / 16) .. + 3.
__device__ __forceinline__ void mfma_agpr(float4_t& acc, const half8_t& b, const half8_t& a) {
    asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(acc) : "v"(b), "v"(a));
}
// acc = b-fragment . a-fragment: the first MFMA of a C tile starts the accumulator from the constant zero, so the
// 256 accumulator registers are never cleared by the vector ALU.
__device__ __forceinline__ void mfma_agpr_first(float4_t& acc, const half8_t& b, const half8_t& a) {
    asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, 0" : "=a"(acc) : "v"(b), "v"(a));
}

// One global_load_lds_dwordx4: lane l's 16 bytes at base + offset[l] go to LDS bytes [lds_base + lds_imm + 16 l, + 16).
template <int LDS_IMM>
__device__ __forceinline__ void request_16B_per_lane(const void* uniform_base, unsigned lane_offset, unsigned lds_base) {
    asm volatile("s_add_u32 m0, %2, %3\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %0"
                 ::"s"(uniform_base), "v"(lane_offset), "s"(lds_base), "n"(LDS_IMM) : "memory", "scc");
}

// Idle cycles that every access to two rows of accumulators stays on its side of.  The MFMAs are hidden from the
// compiler, so it neither knows that the matrix core may still be writing an accumulator the vector ALU is about to
// read (up to 18 wait states) nor that a freshly written zero takes a few cycles to be readable by an MFMA: the
// accumulators are operands of this statement, which orders it against every producer and consumer.
#define TL_ACC_FENCE2(acc, i, text)                                                                                       \
    asm volatile(text : "+a"(acc[i][0]), "+a"(acc[i][1]), "+a"(acc[i][2]), "+a"(acc[i][3]), "+a"(acc[i][4]),             \
                 "+a"(acc[i][5]), "+a"(acc[i][6]), "+a"(acc[i][7]), "+a"(acc[i + 1][0]), "+a"(acc[i + 1][1]),              \
                 "+a"(acc[i + 1][2]), "+a"(acc[i + 1][3]), "+a"(acc[i + 1][4]), "+a"(acc[i + 1][5]), "+a"(acc[i + 1][6]), \
                 "+a"(acc[i + 1][7]))
#define TL_ACC_FENCE(acc, text)       \
    do {                              \
        TL_ACC_FENCE2(acc, 0, text);  \
        TL_ACC_FENCE2(acc, 2, "");    \
        TL_ACC_FENCE2(acc, 4, "");    \
        TL_ACC_FENCE2(acc, 6, "");    \
    } while (0)

// A_AHEAD: how many iterations (of NT MFMAs) ahead of its use an A fragment is read; BAR_IT: the iteration in front of
// which the K tile's barrier stands; D_STEP: MFMAs between two requests.
// GATED: the SwiGLU gate in the epilogue, as in the gated build of hgemm_f16_dlds_kernel (HgemmArgs::gate).  A B tile
// then holds, per wavefront column, 64 rows of the first matrix followed by the 64 rows of the second one that pair
// with them, and covers 128 columns of C; the host passes tiles_n and ldc in output columns.
template <int A_AHEAD, int BAR_IT, int D_STEP, bool GATED>
__global__ void __launch_bounds__(256) hgemm_f16_big_kernel(TL_HGEMM_PARAMS) {
    TL_HGEMM_ARGS_FROM_PARAMS;
    constexpr int BM = 256, BN = 256, BK = 64, WN = 2, NW = 4;
    constexpr int RB = BK * 2;                 // bytes per tile row
    constexpr int CPR = BK / 8;                // 16-byte chunks per tile row
    constexpr int RPL = 256 / RB;              // tile rows per 256-byte LDS line
    constexpr int RPW = 1024 / RB;             // tile rows written by one request
    constexpr int A_REQS = BM / RPW / NW;      // requests per K tile, per wavefront and operand
    constexpr int B_REQS = BN / RPW / NW;
    constexpr int NREQ = A_REQS + B_REQS;
    constexpr int A_BYTES = BM * RB;
    constexpr int STAGE_BYTES = (BM + BN) * RB;
    constexpr int TM = 128, TN = 128;          // wavefront tile
    constexpr int MT = TM / 16, NT = TN / 16;  // 16x16 MFMA tiles per wavefront
    constexpr int KS = BK / 32;                // K steps of 32 per K tile
    constexpr int SLOTS = KS * MT * NT;        // MFMAs per K tile
    constexpr int NA = KS * MT;                // A fragments per K tile
    static_assert((NW * RPW / RPL) % CPR == 0, "the chunk a lane fetches must not depend on the request");
    static_assert(A_REQS == B_REQS, "one set of lane offsets serves both operands");
    // Slot of the K tile's barrier.  Every read of the tile's own stage is issued before it (A fragment n at iteration
    // n - A_AHEAD, the B fragments of step 1 during step 0), early enough that the data has arrived when the barrier
    // is reached; the first reads of the next tile's stage (its first A_AHEAD A fragments and the B fragments of its
    // step 0) stand behind it.
    constexpr int BARRIER_SLOT = BAR_IT * NT;
    static_assert(A_AHEAD >= 1 && NA - 1 - A_AHEAD < BAR_IT && BAR_IT < NA, "the last A fragment is requested before the barrier");
    static_assert(BARRIER_SLOT + 2 * (NT + A_AHEAD) <= SLOTS, "the next tile's first fragments are read behind the barrier");
    // request d < EARLY of K tile kt+2 goes out behind MFMA BARRIER_SLOT + 1 + D_STEP d of tile kt (the barrier has just
    // freed its stage), the others behind MFMA 1 + D_STEP (d - EARLY) of tile kt+1
    constexpr int EARLY_ROOM = (SLOTS - BARRIER_SLOT - 2) / D_STEP + 1;
    constexpr int EARLY = EARLY_ROOM < NREQ ? EARLY_ROOM : NREQ;
    constexpr int LATE = NREQ - EARLY;
    static_assert(LATE == 0 || 1 + D_STEP * (LATE - 1) + 32 < BARRIER_SLOT, "a request needs time to land before its tile's barrier");
    static_assert(NA % 4 == 0, "fragment counts");

    extern __shared__ __attribute__((aligned(1024))) unsigned char smem_raw[];

    const unsigned long long t_start = a.stamps ? __builtin_amdgcn_s_memrealtime() : 0ull;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave / WN, wn = wave % WN;
    const int N = a.N, K = a.K, ldc = a.ldc;
    half_t* __restrict__ C = a.C;
    const unsigned char* const Ag = reinterpret_cast<const unsigned char*>(a.A);
    const unsigned char* const Bg = reinterpret_cast<const unsigned char*>(a.B);
    const int KT = K / BK;              // even, at least 4 (host-checked)
    const int total_tiles = a.tiles_m * a.tiles_n;
    const int tiles_m = a.tiles_m, band_m = a.band_m;
    const unsigned rot_tile = (unsigned)a.rot_tile, rot_xcd = (unsigned)a.rot_xcd;
    const size_t row_bytes = (size_t)K * 2;

    // Requests: request d of an operand covers, for this wavefront, tile rows (d * NW + wave) * RPW .. + RPW.  The
    // lane's byte offset from the tile's first row at the K tile wanted is fixed for the whole kernel (one register
    // per request, the same for both operands); the tile and the walk along K move a base pointer in scalar registers.
    const int r0 = wave * RPW + lane / CPR;                       // tile row of request 0
    const int chunk = (lane % CPR) ^ ((r0 / RPL) % CPR);           // the same for every request (static_assert above)
    unsigned req_off[A_REQS];
#pragma unroll
    for (int d = 0; d < A_REQS; ++d) req_off[d] = (unsigned)(((size_t)(r0 + d * NW * RPW) * K + (size_t)chunk * 8) * 2);
    // gated: tile row r of B is row (r / TN) * (TN / 2) + r % (TN / 2) of the tile's 128 output columns, taken from the
    // first matrix for the first half of a wavefront column and `gate` rows further down for the second half
    unsigned req_off_gated[GATED ? B_REQS : 1];
    if constexpr (GATED) {
#pragma unroll
        for (int d = 0; d < B_REQS; ++d) {
            const int r = r0 + d * NW * RPW, in_wave = r % TN;
            const size_t row = (size_t)(r / TN) * (TN / 2) + (size_t)(in_wave % (TN / 2)) + (in_wave >= TN / 2 ? (size_t)a.gate : 0);
            req_off_gated[d] = (unsigned)((row * K + (size_t)chunk * 8) * 2);
        }
    }
    constexpr int B_TILE_ROWS = GATED ? BN / 2 : BN;   // rows of (either matrix of) B between two tiles
    const unsigned lds_wave = (unsigned)(unsigned long)(__attribute__((address_space(3))) unsigned char*)smem_raw + (unsigned)wave * 1024u;

    // The request stream: the K tile whose requests come next, as base pointers into A and B, and where it sits in its
    // C tile's walk (K tile k of the matrix, the w-th of the walk).  Past the last C tile the stream keeps asking for
    // the last tile's data, which lands in stages nobody reads.
    int req_vb = blockIdx.x, req_w = 0, req_k = 0;
    const unsigned char *req_a_tile = Ag, *req_b_tile = Bg;     // first row of the C tile's panels
    auto req_enter_tile = [&]() {
        int tm, tn;
        tile_of_block(req_vb, total_tiles, tiles_m, band_m, tm, tn);
        req_a_tile = Ag + (size_t)tm * BM * row_bytes;
        req_b_tile = Bg + (size_t)tn * B_TILE_ROWS * row_bytes;
        req_w = 0;
        req_k = (int)(((unsigned)tn * rot_tile + (blockIdx.x & 7u) * rot_xcd) % (unsigned)KT);
    };
    req_enter_tile();
    const unsigned char *req_a = req_a_tile + (size_t)req_k * (BK * 2), *req_b = req_b_tile + (size_t)req_k * (BK * 2);
    const unsigned char *late_a = req_a, *late_b = req_b;       // the K tile before it (its late requests are still due)
    auto req_advance = [&]() {
        late_a = req_a;
        late_b = req_b;
        ++req_w;
        ++req_k;
        if (req_k == KT) req_k = 0;
        if (req_w == KT) {
            if (req_vb + (int)gridDim.x < total_tiles) {
                req_vb += (int)gridDim.x;
                req_enter_tile();
            } else {
                req_w = 0;
            }
        }
        req_a = req_a_tile + (size_t)req_k * (BK * 2);
        req_b = req_b_tile + (size_t)req_k * (BK * 2);
    };
    // request d (A for d < A_REQS, else B) of the K tile at (pa, pb) into stage `stage` (a compile-time constant)
    auto request = [&](auto dd, auto stage, const unsigned char* pa, const unsigned char* pb) {
        constexpr int d = decltype(dd)::value, st = decltype(stage)::value;
        if constexpr (d < A_REQS)
            request_16B_per_lane<st * STAGE_BYTES + d * NW * 1024>(pa, req_off[d], lds_wave);
        else if constexpr (GATED)
            request_16B_per_lane<st * STAGE_BYTES + A_BYTES + (d - A_REQS) * NW * 1024>(pb, req_off_gated[d - A_REQS], lds_wave);
        else
            request_16B_per_lane<st * STAGE_BYTES + A_BYTES + (d - A_REQS) * NW * 1024>(pb, req_off[d - A_REQS], lds_wave);
    };

    // fragment reader: row (lane % 16) of a 16-row MFMA tile, chunk 4 * s + lane / 16 of K step s
    const int fr_row = lane & 15;
    const int fr_sw = (fr_row / RPL) % CPR;
    int fr_off[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) fr_off[ks] = fr_row * RB + (((ks * 4 + (lane >> 4)) ^ fr_sw) * 16);
    const unsigned char* const a_frag = smem_raw + wm * TM * RB;             // + stage, + 16-row block, + fr_off[s]
    const unsigned char* const b_frag = smem_raw + A_BYTES + wn * TN * RB;

    float4_t acc[MT][NT];
    half8_t abuf[NA];      // A fragment n of a K tile (n = s * MT + i)
    half8_t bbuf[2][NT];   // the B fragments of K step s stay in bbuf[s] for the whole step
    using S0 = std::integral_constant<int, 0>;
    using S1 = std::integral_constant<int, 1>;
    // This wavefront's requests have landed and its LDS reads are done, then the workgroup barrier.
    auto tile_barrier = [&]() { asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory"); };

    // prologue of the pipeline: K tile 0 of the first C tile into stage 0, the early requests of K tile 1 into stage 1
    // (its late ones go out in the first slots of tile 0, as in every tile)
    static_for<0, NREQ>([&](auto d) { request(d, S0{}, req_a, req_b); });
    req_advance();
    tile_barrier();
    static_for<0, EARLY>([&](auto d) { request(d, S1{}, req_a, req_b); });
    req_advance();
    abuf[0] = *reinterpret_cast<const half8_t*>(a_frag + fr_off[0]);
#pragma unroll
    for (int j = 0; j < NT; ++j) bbuf[0][j] = *reinterpret_cast<const half8_t*>(b_frag + j * 16 * RB + fr_off[0]);
#pragma unroll
    for (int n = 1; n < A_AHEAD; ++n) abuf[n] = *reinterpret_cast<const half8_t*>(a_frag + n * 16 * RB + fr_off[0]);

    // One K tile of the pipeline, the same for every tile of every C tile.  par: stage of this K tile (kt % 2).
    // Slot q = (s * MT + i) * NT + j of the tile holds the MFMA of A fragment (s, i) and B fragment (s, j), and behind it:
    //   j == 0: the read of A fragment n + A_AHEAD of this tile;  step 0, j == 4: the read of B fragment i of step 1;
    //   behind the barrier, every second slot: A fragment 0, the B fragments of step 0 and A fragments 1 .. A_AHEAD - 1 of
    //   the next tile, in the order its MFMAs need them;
    //   slots 1 + D_STEP d': the late requests of K tile kt+1;  slots BARRIER_SLOT + 1 + D_STEP d: the early requests of
    //   K tile kt+2, into the stage the barrier has just freed.
    // first: the K tile opens a C tile (its first K step starts the accumulators from zero)
    auto tile = [&](auto par, auto first) {
        constexpr int P = decltype(par)::value;
        constexpr bool FIRST = decltype(first)::value;
        using Cur = std::integral_constant<int, P>;
        using Nxt = std::integral_constant<int, 1 - P>;
        const unsigned char* const a_cur = a_frag + P * STAGE_BYTES;
        const unsigned char* const b_cur = b_frag + P * STAGE_BYTES;
        const unsigned char* const a_nxt = a_frag + (1 - P) * STAGE_BYTES;
        const unsigned char* const b_nxt = b_frag + (1 - P) * STAGE_BYTES;
        static_for<0, SLOTS>([&](auto slot) {
            constexpr int q = decltype(slot)::value;
            constexpr int s = q / (MT * NT), i = (q / NT) % MT, j = q % NT, n = s * MT + i;
            if constexpr (q == BARRIER_SLOT) tile_barrier();   // tile kt+1 is complete in LDS, nobody reads tile kt's stage any more
            if constexpr (FIRST && s == 0) mfma_agpr_first(acc[i][j], bbuf[s][j], abuf[n]);
            else mfma_agpr(acc[i][j], bbuf[s][j], abuf[n]);
            if constexpr (j == 0 && n + A_AHEAD < NA) {
                constexpr int n2 = n + A_AHEAD;
                abuf[n2] = *reinterpret_cast<const half8_t*>(a_cur + (n2 % MT) * 16 * RB + fr_off[n2 / MT]);
            }
            if constexpr (s + 1 < KS && j == 4)
                bbuf[(s + 1) % KS][i] = *reinterpret_cast<const half8_t*>(b_cur + i * 16 * RB + fr_off[(s + 1) % KS]);
            // r-th read behind the barrier: A0, B0 .. B(NT-1), A1 ..
            if constexpr (q > BARRIER_SLOT && (q - BARRIER_SLOT - 1) % 2 == 0 && (q - BARRIER_SLOT - 1) / 2 < NT + A_AHEAD) {
                constexpr int r = (q - BARRIER_SLOT - 1) / 2;
                if constexpr (r == 0) abuf[0] = *reinterpret_cast<const half8_t*>(a_nxt + fr_off[0]);
                else if constexpr (r <= NT) bbuf[0][r - 1] = *reinterpret_cast<const half8_t*>(b_nxt + (r - 1) * 16 * RB + fr_off[0]);
                else abuf[r - NT] = *reinterpret_cast<const half8_t*>(a_nxt + (r - NT) * 16 * RB + fr_off[0]);
            }
            if constexpr (q >= 1 && (q - 1) % D_STEP == 0 && (q - 1) / D_STEP < LATE)
                request(std::integral_constant<int, EARLY + (q - 1) / D_STEP>{}, Nxt{}, late_a, late_b);
            if constexpr (q > BARRIER_SLOT && (q - BARRIER_SLOT - 1) % D_STEP == 0 && (q - BARRIER_SLOT - 1) / D_STEP < EARLY)
                request(std::integral_constant<int, (q - BARRIER_SLOT - 1) / D_STEP>{}, Cur{}, req_a, req_b);
            __builtin_amdgcn_sched_barrier(0);
        });
        req_advance();
    };

    for (int vb = blockIdx.x;;) {   // C tiles of this workgroup
        tile(S0{}, std::true_type{});
        tile(S1{}, std::false_type{});
        for (int kt = 2; kt < KT; kt += 2) {
            tile(S0{}, std::false_type{});
            tile(S1{}, std::false_type{});
        }
        TL_ACC_FENCE(acc, "s_nop 15\n\ts_nop 15");

        // ---- epilogue.  acc[i][j][r] = C[row i*16 + lane%16][col j*16 + 4*(lane/16) + r] ----
        // fp16 output through LDS: every wavefront turns 16 x TN blocks of its accumulators into row-major halves in a
        // private region behind the ring (the ring itself already receives the next C tile's first K tiles), 8-byte
        // writes into rows padded by 16 bytes, reads them back 16 bytes per lane and stores whole 16-byte pieces of C
        // rows.  The host guarantees whole tiles, ldc % 8 == 0 and a 16-byte aligned C.
        int tm, tn;
        tile_of_block(vb, total_tiles, tiles_m, band_m, tm, tn);
        const int e_row = lane & 15;
        const int e_col = (lane >> 4) * 4;
        const int row_base = tm * BM + wm * TM, col_base = GATED ? tn * (BN / 2) + wn * (TN / 2) : tn * BN + wn * TN;
        constexpr int RS = TN * 2 + 16;
        constexpr int CH = (GATED ? TN / 2 : TN) / 8;   // 16-byte chunks per row of output
        constexpr int RPR = 64 / CH;             // rows per wavefront-wide read
        constexpr int PASSES = 16 / RPR;
        static_assert(64 % CH == 0 && 16 % RPR == 0, "a staged block is read back in whole wavefront-wide passes");
        unsigned char* region = smem_raw + 2 * STAGE_BYTES + wave * (16 * RS);
#pragma unroll
        for (int i = 0; i < MT; ++i) {
#pragma unroll
            for (int j = 0; j < NT; ++j) {
                half4_t h = {(half_t)acc[i][j][0], (half_t)acc[i][j][1], (half_t)acc[i][j][2], (half_t)acc[i][j][3]};
                *reinterpret_cast<half4_t*>(region + e_row * RS + (j * 16 + e_col) * 2) = h;
            }
#pragma unroll
            for (int q = 0; q < PASSES; ++q) {
                const int r = q * RPR + lane / CH, c = lane % CH;
                const int row = row_base + i * 16 + r, col = col_base + c * 8;
                if constexpr (GATED) {
                    // pairs of 16-byte pieces TN/2 columns apart: out = half(silu(x) * y) of the two rounded projections,
                    // the arithmetic of the separate gate kernel
                    const half8_t vx = *reinterpret_cast<const half8_t*>(region + r * RS + c * 16);
                    const half8_t vy = *reinterpret_cast<const half8_t*>(region + r * RS + TN + c * 16);
                    half8_t o;
#pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        const float x = (float)vx[e];
                        o[e] = (half_t)(x * (1.0f / (1.0f + expf(-x))) * (float)vy[e]);
                    }
                    *reinterpret_cast<half8_t*>(C + (size_t)row * ldc + col) = o;
                } else {
                    const half8_t v = *reinterpret_cast<const half8_t*>(region + r * RS + c * 16);
                    if (col < N) *reinterpret_cast<half8_t*>(C + (size_t)row * ldc + col) = v;
                }
            }
            // one block of accumulators at a time: without this the gate's arithmetic invites the scheduler to pull
            // every block's accumulators into VGPRs first
            if constexpr (GATED) __builtin_amdgcn_sched_barrier(0);
        }
        vb += (int)gridDim.x;
        if (vb >= total_tiles) break;
    }
    // requests that ran past the last tile may still be in flight towards LDS
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    if (a.stamps && tid == 0) {
        a.stamps[2 * blockIdx.x] = t_start;
        a.stamps[2 * blockIdx.x + 1] = __builtin_amdgcn_s_memrealtime();
    }
}

// The same ideas on a 256x128 tile for problems that have too few 256x256 tiles to fill the chip: four wavefronts of
// 128x64 (128 accumulator registers), a ring of three 48 KB stages (a K tile of this size is multiplied in 1024 cycles,
// less than a request takes to land, so requests run two tiles ahead), one C tile per workgroup.  Requests for K tiles
// past the end of K fetch the last K tile again into a stage nobody reads, so every tile of the loop is the same code
// and the barrier's wait count never changes.  Whole tiles only (M % 256 == 0, N % 128 == 0), K in tiles of 64, at
// least three.
#define TL_ACC_FENCE4(acc, i, text) \
    asm volatile(text : "+a"(acc[i][0]), "+a"(acc[i][1]), "+a"(acc[i][2]), "+a"(acc[i][3]), "+a"(acc[i + 1][0]), \
                 "+a"(acc[i + 1][1]), "+a"(acc[i + 1][2]), "+a"(acc[i + 1][3]))

template <int A_AHEAD, int BAR_IT, int D_STEP>
__global__ void __launch_bounds__(256) hgemm_f16_mid_kernel(TL_HGEMM_PARAMS) {
    TL_HGEMM_ARGS_FROM_PARAMS;
    constexpr int BM = 256, BN = 128, BK = 64, WN = 2, NW = 4, STAGES = 3;
    constexpr int RB = BK * 2;
    constexpr int CPR = BK / 8;
    constexpr int RPL = 256 / RB;
    constexpr int RPW = 1024 / RB;
    constexpr int A_REQS = BM / RPW / NW;      // 8
    constexpr int B_REQS = BN / RPW / NW;      // 4
    constexpr int NREQ = A_REQS + B_REQS;
    constexpr int A_BYTES = BM * RB;
    constexpr int STAGE_BYTES = (BM + BN) * RB;
    constexpr int TM = 128, TN = 64;           // wavefront tile
    constexpr int MT = TM / 16, NT = TN / 16;
    constexpr int KS = BK / 32;
    constexpr int SLOTS = KS * MT * NT;        // 64 MFMAs per K tile
    constexpr int NA = KS * MT;
    static_assert((NW * RPW / RPL) % CPR == 0, "the chunk a lane fetches must not depend on the request");
    constexpr int BARRIER_SLOT = BAR_IT * NT;
    static_assert(A_AHEAD >= 1 && NA - 1 - A_AHEAD < BAR_IT && BAR_IT < NA, "the last A fragment is requested before the barrier");
    static_assert(BARRIER_SLOT + 1 + NT + A_AHEAD <= SLOTS, "the next tile's first fragments are read behind the barrier");
    // request d < EARLY of K tile kt+3 goes out behind MFMA BARRIER_SLOT + 1 + D_STEP d of tile kt (the barrier has just
    // freed its stage), the others behind MFMA 1 + D_STEP (d - EARLY) of tile kt+1; at the barrier of tile kt+1 all of
    // them are out and may be in flight, everything older has to have landed
    constexpr int EARLY_ROOM = (SLOTS - BARRIER_SLOT - 2) / D_STEP + 1;
    constexpr int EARLY = EARLY_ROOM < NREQ ? EARLY_ROOM : NREQ;
    constexpr int LATE = NREQ - EARLY;
    static_assert(LATE == 0 || 1 + D_STEP * (LATE - 1) < BARRIER_SLOT, "a tile's requests are out before the next barrier");

    extern __shared__ __attribute__((aligned(1024))) unsigned char smem_raw[];

    const unsigned long long t_start = a.stamps ? __builtin_amdgcn_s_memrealtime() : 0ull;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave / WN, wn = wave % WN;
    const int K = a.K, ldc = a.ldc;
    half_t* __restrict__ C = a.C;
    const int KT = K / BK;
    const size_t row_bytes = (size_t)K * 2;

    int tm, tn;
    tile_of_block(blockIdx.x, a.tiles_m * a.tiles_n, a.tiles_m, a.band_m, tm, tn);
    const unsigned char* const a_tile = reinterpret_cast<const unsigned char*>(a.A) + (size_t)tm * BM * row_bytes;
    const unsigned char* const b_tile = reinterpret_cast<const unsigned char*>(a.B) + (size_t)tn * BN * row_bytes;
    const int rot = (int)(((unsigned)tn * (unsigned)a.rot_tile + (blockIdx.x & 7u) * (unsigned)a.rot_xcd) % (unsigned)KT);

    const int r0 = wave * RPW + lane / CPR;
    const int chunk = (lane % CPR) ^ ((r0 / RPL) % CPR);
    unsigned req_off[A_REQS];
#pragma unroll
    for (int d = 0; d < A_REQS; ++d) req_off[d] = (unsigned)(((size_t)(r0 + d * NW * RPW) * K + (size_t)chunk * 8) * 2);
    const unsigned lds_wave = (unsigned)(unsigned long)(__attribute__((address_space(3))) unsigned char*)smem_raw + (unsigned)wave * 1024u;

    // the request stream: K tile `req_pos` of the walk (clamped to the last one), as base pointers into A and B
    int req_pos = 0, req_k = rot;
    const unsigned char *req_a = a_tile + (size_t)req_k * (BK * 2), *req_b = b_tile + (size_t)req_k * (BK * 2);
    const unsigned char *late_a = req_a, *late_b = req_b;
    auto req_advance = [&]() {
        late_a = req_a;
        late_b = req_b;
        ++req_pos;
        if (req_pos < KT) {
            ++req_k;
            if (req_k == KT) req_k = 0;
            req_a = a_tile + (size_t)req_k * (BK * 2);
            req_b = b_tile + (size_t)req_k * (BK * 2);
        }
    };
    auto request = [&](auto dd, auto stage, const unsigned char* pa, const unsigned char* pb) {
        constexpr int d = decltype(dd)::value, st = decltype(stage)::value;
        if constexpr (d < A_REQS)
            request_16B_per_lane<st * STAGE_BYTES + d * NW * 1024>(pa, req_off[d], lds_wave);
        else
            request_16B_per_lane<st * STAGE_BYTES + A_BYTES + (d - A_REQS) * NW * 1024>(pb, req_off[d - A_REQS], lds_wave);
    };

    const int fr_row = lane & 15;
    const int fr_sw = (fr_row / RPL) % CPR;
    int fr_off[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) fr_off[ks] = fr_row * RB + (((ks * 4 + (lane >> 4)) ^ fr_sw) * 16);
    const unsigned char* const a_frag = smem_raw + wm * TM * RB;
    const unsigned char* const b_frag = smem_raw + A_BYTES + wn * TN * RB;

    float4_t acc[MT][NT];
    half8_t abuf[NA];
    half8_t bbuf[2][NT];
    using S0 = std::integral_constant<int, 0>;
    using S1 = std::integral_constant<int, 1>;
    using S2 = std::integral_constant<int, 2>;

    // prologue: K tiles 0 and 1 whole, the early requests of K tile 2; tile 0 has to have landed
    static_for<0, NREQ>([&](auto d) { request(d, S0{}, req_a, req_b); });
    req_advance();
    static_for<0, NREQ>([&](auto d) { request(d, S1{}, req_a, req_b); });
    req_advance();
    static_for<0, EARLY>([&](auto d) { request(d, S2{}, req_a, req_b); });
    req_advance();
    asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(NREQ + EARLY) : "memory");
    abuf[0] = *reinterpret_cast<const half8_t*>(a_frag + fr_off[0]);
#pragma unroll
    for (int j = 0; j < NT; ++j) bbuf[0][j] = *reinterpret_cast<const half8_t*>(b_frag + j * 16 * RB + fr_off[0]);
#pragma unroll
    for (int n = 1; n < A_AHEAD; ++n) abuf[n] = *reinterpret_cast<const half8_t*>(a_frag + n * 16 * RB + fr_off[0]);

    // One K tile in stage P; the next one is in stage (P + 1) % 3, the requests of the tile after that are finishing in
    // stage (P + 2) % 3, and behind the barrier stage P takes the first requests of the tile three ahead.
    auto tile = [&](auto par, auto first) {
        constexpr int P = decltype(par)::value;
        constexpr bool FIRST = decltype(first)::value;
        using Cur = std::integral_constant<int, P>;
        using Aft = std::integral_constant<int, (P + 2) % STAGES>;
        const unsigned char* const a_cur = a_frag + P * STAGE_BYTES;
        const unsigned char* const b_cur = b_frag + P * STAGE_BYTES;
        const unsigned char* const a_nxt = a_frag + ((P + 1) % STAGES) * STAGE_BYTES;
        const unsigned char* const b_nxt = b_frag + ((P + 1) % STAGES) * STAGE_BYTES;
        static_for<0, SLOTS>([&](auto slot) {
            constexpr int q = decltype(slot)::value;
            constexpr int s = q / (MT * NT), i = (q / NT) % MT, j = q % NT, n = s * MT + i;
            // tile kt+1 has landed for this wavefront (the NREQ requests of tile kt+2 may be in flight), its LDS reads
            // of tile kt are done; behind the barrier that holds for everyone
            if constexpr (q == BARRIER_SLOT) asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" ::"n"(NREQ) : "memory");
            if constexpr (FIRST && s == 0) mfma_agpr_first(acc[i][j], bbuf[s][j], abuf[n]);
            else mfma_agpr(acc[i][j], bbuf[s][j], abuf[n]);
            if constexpr (j == 0 && n + A_AHEAD < NA) {
                constexpr int n2 = n + A_AHEAD;
                abuf[n2] = *reinterpret_cast<const half8_t*>(a_cur + (n2 % MT) * 16 * RB + fr_off[n2 / MT]);
            }
            if constexpr (s + 1 < KS && j == 2 && i < NT)
                bbuf[(s + 1) % KS][i] = *reinterpret_cast<const half8_t*>(b_cur + i * 16 * RB + fr_off[(s + 1) % KS]);
            // r-th read behind the barrier: A0, B0 .. B(NT-1), A1 ..
            if constexpr (q > BARRIER_SLOT && q - BARRIER_SLOT - 1 < NT + A_AHEAD) {
                constexpr int r = q - BARRIER_SLOT - 1;
                if constexpr (r == 0) abuf[0] = *reinterpret_cast<const half8_t*>(a_nxt + fr_off[0]);
                else if constexpr (r <= NT) bbuf[0][r - 1] = *reinterpret_cast<const half8_t*>(b_nxt + (r - 1) * 16 * RB + fr_off[0]);
                else abuf[r - NT] = *reinterpret_cast<const half8_t*>(a_nxt + (r - NT) * 16 * RB + fr_off[0]);
            }
            if constexpr (q >= 1 && (q - 1) % D_STEP == 0 && (q - 1) / D_STEP < LATE)
                request(std::integral_constant<int, EARLY + (q - 1) / D_STEP>{}, Aft{}, late_a, late_b);
            if constexpr (q > BARRIER_SLOT && (q - BARRIER_SLOT - 1) % D_STEP == 0 && (q - BARRIER_SLOT - 1) / D_STEP < EARLY)
                request(std::integral_constant<int, (q - BARRIER_SLOT - 1) / D_STEP>{}, Cur{}, req_a, req_b);
            __builtin_amdgcn_sched_barrier(0);
        });
        req_advance();
    };

    {
        using T = std::true_type;
        using F = std::false_type;
        tile(S0{}, T{});
        int kt = 1;
        for (; kt + 3 <= KT; kt += 3) {
            tile(S1{}, F{});
            tile(S2{}, F{});
            tile(S0{}, F{});
        }
        if (kt < KT) {
            tile(S1{}, F{});
            if (kt + 1 < KT) tile(S2{}, F{});
        }
    }
    TL_ACC_FENCE4(acc, 0, "s_nop 15\n\ts_nop 15");
    TL_ACC_FENCE4(acc, 2, "");
    TL_ACC_FENCE4(acc, 4, "");
    TL_ACC_FENCE4(acc, 6, "");

    // ---- epilogue, as in the 256x256 kernel: 16 x TN blocks through a private LDS region behind the ring ----
    const int e_row = lane & 15;
    const int e_col = (lane >> 4) * 4;
    const int row_base = tm * BM + wm * TM, col_base = tn * BN + wn * TN;
    constexpr int RS = TN * 2 + 16;
    constexpr int CH = TN / 8;
    constexpr int RPR = 64 / CH;
    constexpr int PASSES = 16 / RPR;
    static_assert(64 % CH == 0 && 16 % RPR == 0, "a staged block is read back in whole wavefront-wide passes");
    unsigned char* region = smem_raw + STAGES * STAGE_BYTES + wave * (16 * RS);
#pragma unroll
    for (int i = 0; i < MT; ++i) {
#pragma unroll
        for (int j = 0; j < NT; ++j) {
            half4_t h = {(half_t)acc[i][j][0], (half_t)acc[i][j][1], (half_t)acc[i][j][2], (half_t)acc[i][j][3]};
            *reinterpret_cast<half4_t*>(region + e_row * RS + (j * 16 + e_col) * 2) = h;
        }
#pragma unroll
        for (int q = 0; q < PASSES; ++q) {
            const int r = q * RPR + lane / CH, c = lane % CH;
            const half8_t v = *reinterpret_cast<const half8_t*>(region + r * RS + c * 16);
            const int row = row_base + i * 16 + r, col = col_base + c * 8;
            *reinterpret_cast<half8_t*>(C + (size_t)row * ldc + col) = v;
        }
    }
    // the requests past the end of K may still be in flight towards LDS
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    if (a.stamps && tid == 0) {
        a.stamps[2 * blockIdx.x] = t_start;
        a.stamps[2 * blockIdx.x + 1] = __builtin_amdgcn_s_memrealtime();
    }
}

static std::atomic<bool> g_mid_attr{false};
// inspection: where the next launches of the two kernels write their workgroup time stamps (null: nowhere)
static std::atomic<unsigned long long*> g_stamps{nullptr};
static std::atomic<size_t> g_stamps_capacity{0};
void hgemm_agpr_set_stamps(void* buf, size_t capacity) {
    g_stamps_capacity = buf ? capacity : 0;
    g_stamps = (unsigned long long*)buf;
}
static unsigned long long* stamps_for(size_t workgroups) { return 2 * workgroups <= g_stamps_capacity.load() ? g_stamps.load() : nullptr; }


const char* hgemm_mid_name() { return "a256x128x64w2x2"; }

bool hgemm_mid_applies(const void* A, const void* B, const void* C, size_t M, size_t N, size_t K, size_t ldc) {
    return M >= 256 && N >= 128 && M % 256 == 0 && N % 128 == 0 && K >= 192 && K % 64 == 0 && K <= ((size_t)1 << 22) &&
           ldc % 8 == 0 && ldc >= N && aligned16(A) && aligned16(B) && aligned16(C) && M <= 0x7fffffffu && N <= 0x7fffffffu;
}

int launch_hgemm_mid(const void* A, const void* B, void* C, size_t M, size_t N, size_t K, size_t ldc, int band, int rot_tile,
                     int rot_xcd) {
    TL_REQUIRE(hgemm_mid_applies(A, B, C, M, N, K, ldc), "hgemm: %s does not serve this shape", hgemm_mid_name());
    const HgemmKernel kernel = hgemm_f16_mid_kernel<3, 13, 4>;
    // the three-stage ring and behind it the C staging of the epilogue (four wavefronts x 16 rows x (128 + 16) bytes)
    const size_t lds = (size_t)3 * (256 + 128) * 64 * sizeof(half_t) + (size_t)4 * 16 * (64 * 2 + 16);
    if (!g_mid_attr.load()) {
        TL_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
        g_mid_attr.store(true);
    }
    HgemmArgs a{};
    a.A = (const half_t*)A;
    a.B = (const half_t*)B;
    a.C = (half_t*)C;
    a.M = (int)M;
    a.N = (int)N;
    a.K = (int)K;
    a.ldc = (int)ldc;
    a.tiles_m = (int)(M / 256);
    a.tiles_n = (int)(N / 128);
    a.kt_per_split = 0x7fffffff;
    a.band_m = band > 0 ? band : 8;
    a.rot_tile = rot_tile;
    a.rot_xcd = rot_xcd;
    const size_t nblocks = (size_t)a.tiles_m * a.tiles_n;
    TL_REQUIRE(nblocks <= 0x7fffffffu, "hgemm: too many tiles");
    a.stamps = stamps_for(nblocks);
    hipLaunchKernelGGL(kernel, dim3((unsigned)nblocks), dim3(256), lds, stream(), TL_HGEMM_PASS(a));
    TL_CHECK_LAUNCH(hgemm_mid_name());
    return TL_OK;
}

static std::atomic<bool> g_big_attr{false}, g_big_gated_attr{false};

const char* hgemm_big_name() { return "a256x256x64w2x2"; }

// Full contract of the kernel: whole 256x256 tiles, an even number of K tiles of 64, at least four, lane offsets of a
// tile within 32 bits, C rows that take 16-byte stores.  gate != 0: N counts the rows of both matrices in B, C has N / 2
// columns in whole tiles of 128, and the lane offsets reach the second matrix.
bool hgemm_big_applies(const void* A, const void* B, const void* C, size_t M, size_t N, size_t K, size_t ldc, size_t gate) {
    const size_t n_out = gate ? N / 2 : N;
    return M >= 256 && N >= 256 && M % 256 == 0 && N % 256 == 0 && K >= 256 && K % 128 == 0 && K <= ((size_t)1 << 22) &&
           ldc % 8 == 0 && ldc >= n_out && aligned16(A) && aligned16(B) && aligned16(C) && M <= 0x7fffffffu && N <= 0x7fffffffu &&
           (gate == 0 || (gate >= n_out && gate <= 0x7fffffffu && (gate + n_out) * K * sizeof(half_t) < ((size_t)1 << 32)));
}

int launch_hgemm_big(const void* A, const void* B, void* C, size_t M, size_t N, size_t K, size_t ldc, int band, int rot_tile,
                     int rot_xcd, size_t gate) {
    TL_REQUIRE(hgemm_big_applies(A, B, C, M, N, K, ldc, gate), "hgemm: %s does not serve this shape", hgemm_big_name());
    // A fragments read three iterations ahead, the barrier in front of iteration 13 of 16, a request every fourth MFMA:
    // A_AHEAD 3 .. 6, barriers at 11 .. 13 and request spacings 3 and 4 measured within 1 % of each other
    const HgemmKernel kernel = gate ? hgemm_f16_big_kernel<3, 13, 4, true> : hgemm_f16_big_kernel<3, 13, 4, false>;
    // the two-stage ring and behind it the C staging of the epilogue (four wavefronts x 16 rows x (256 + 16) bytes)
    const size_t lds = (size_t)2 * (256 + 256) * 64 * sizeof(half_t) + (size_t)4 * 16 * (128 * 2 + 16);
    std::atomic<bool>& attr = gate ? g_big_gated_attr : g_big_attr;
    if (!attr.load()) {
        TL_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
        attr.store(true);
    }
    HgemmArgs a{};
    a.A = (const half_t*)A;
    a.B = (const half_t*)B;
    a.C = (half_t*)C;
    a.M = (int)M;
    a.N = (int)N;
    a.K = (int)K;
    a.ldc = (int)ldc;
    a.tiles_m = (int)(M / 256);
    a.tiles_n = (int)(N / 256);   // a gated tile covers 128 output columns: N / 2 / 128
    a.kt_per_split = 0x7fffffff;
    a.band_m = band > 0 ? band : 8;
    a.rot_tile = rot_tile;
    a.rot_xcd = rot_xcd;
    a.gate = (int)gate;
    const size_t nblocks = (size_t)a.tiles_m * a.tiles_n;
    TL_REQUIRE(nblocks <= 0x7fffffffu, "hgemm: too many tiles");
    // persistent: one workgroup per CU walks tiles blockIdx.x, + gridDim.x, ...
    size_t grid = nblocks;
    const size_t cus = (size_t)device_info().cu_count;
    if (cus > 0 && grid > cus) grid = cus;
    a.stamps = stamps_for(grid);
    hipLaunchKernelGGL(kernel, dim3((unsigned)grid), dim3(256), lds, stream(), TL_HGEMM_PASS(a));
    TL_CHECK_LAUNCH(hgemm_big_name());
    return TL_OK;
}

}  // namespace tl
