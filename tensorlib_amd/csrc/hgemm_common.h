// Shared by the translation units that hold the fp16 tile GEMM kernels: the kernel argument block and the
// workgroup-to-tile map.
#pragma once
#include "tl_internal.h"

namespace tl {

struct HgemmArgs {
    const half_t* A;
    const half_t* B;
    half_t* C;
    int M, N, K;
    int ldc;  // elements between rows of C (N, unless the launch covers a column range of a wider C)
    int tiles_m, tiles_n;
    long sa, sb, sc;  // batch strides in elements
    // split-K (direct-to-LDS kernel only): blockIdx.z walks K tiles [z*kt_per_split, ...) and writes
    // fp32 partial sums to partial[z][M][N]; a second kernel adds the splits in order.
    int kt_per_split;
    float* partial;
    // One-launch split-K: one counter per C tile, zero between launches.  The workgroup that finishes a tile's last
    // split adds the slabs in split order and writes C itself.  Null: a second kernel does that.
    unsigned* tickets;
    // K rotation: a workgroup walks its K tiles starting at (tile_n * rot_tile + xcd * rot_xcd) % KT and wraps.
    // Workgroups that run at the same time then touch different column offsets of the 8 KB-strided rows, which
    // spreads their requests over the memory channels (tile-shaped streaming of B from HBM: 4.3 -> 5.9 TB/s).
    int rot_tile, rot_xcd;
    // Tiles are numbered band by band: a band is band_m rows of tiles over all columns, walked column by column.
    int band_m;
    // Gated launches (kernels built with MODE 2): B holds two matrices `gate` rows apart, N counts the rows of both
    // (2 x the output columns), and C[m][n] = silu(A[m,:].B[n,:]) * (A[m,:].B[gate + n,:]) for n < N / 2.
    int gate;
    // Inspection (the kernels of hgemm_agpr.hip): when not null, stamps[2 * workgroup] / [2 * workgroup + 1] receive the
    // constant 100 MHz counter (s_memrealtime) at the workgroup's first instruction and after its last store.
    unsigned long long* stamps;
};

// The GEMM kernels take the fields of HgemmArgs as separate scalar parameters: the first 16 dwords of scalar kernel
// arguments (the three pointers, M, N, K, ldc, the tile counts and two strides) are preloaded into SGPRs when a wavefront
// is launched (-mllvm -amdgpu-kernarg-preload-count=16), which a struct passed by value is not, so a workgroup's first
// requests do not wait for a scalar load from the argument buffer.
#define TL_HGEMM_PARAMS                                                                                                   \
    const half_t *p_A, const half_t *p_B, half_t *p_C, int p_M, int p_N, int p_K, int p_ldc, int p_tiles_m, int p_tiles_n, \
        long p_sa, long p_sb, long p_sc, int p_kt_per_split, float *p_partial, unsigned *p_tickets, int p_rot_tile,        \
        int p_rot_xcd, int p_band_m, int p_gate, unsigned long long *p_stamps
#define TL_HGEMM_ARGS_FROM_PARAMS                                                                                          \
    const HgemmArgs a {                                                                                                    \
        p_A, p_B, p_C, p_M, p_N, p_K, p_ldc, p_tiles_m, p_tiles_n, p_sa, p_sb, p_sc, p_kt_per_split, p_partial, p_tickets, \
            p_rot_tile, p_rot_xcd, p_band_m, p_gate, p_stamps                                                              \
    }
#define TL_HGEMM_PASS(a)                                                                                                  \
    (a).A, (a).B, (a).C, (a).M, (a).N, (a).K, (a).ldc, (a).tiles_m, (a).tiles_n, (a).sa, (a).sb, (a).sc, (a).kt_per_split, \
        (a).partial, (a).tickets, (a).rot_tile, (a).rot_xcd, (a).band_m, (a).gate, (a).stamps
typedef void (*HgemmKernel)(TL_HGEMM_PARAMS);

// Map the linear workgroup id to a tile so that workgroups resident on one XCD (ids
// congruent mod 8 are dispatched to the same XCD) work on neighbouring tiles: XCD x takes a contiguous run of
// tile numbers, and tiles are numbered down a band of `band` rows of tiles, column after column, band after
// band.  The 32 tiles an XCD works on at a time then cover about band x 32/band panels of A and B, which its
// L2 serves to all of them; with more rows of tiles than `band` a whole column of tiles would share only its
// panel of B and pull every panel of A through the L2 for a single use.
__device__ __forceinline__ void tile_of_block(int bid, int nblocks, int tiles_m, int band, int& tm, int& tn) {
    // nblocks / 8 tiles per XCD, one more on the first nblocks % 8 XCDs
    const int x = bid & 7, base = nblocks >> 3, rem = nblocks & 7;
    const int lid = x * base + (x < rem ? x : rem) + (bid >> 3);
    if (band >= tiles_m) {
        tm = lid % tiles_m;
        tn = lid / tiles_m;
        return;
    }
    const int tiles_n = nblocks / tiles_m;
    const int per_band = band * tiles_n;
    const int b = lid / per_band;
    const int r = lid - b * per_band;
    const int rows = (tiles_m - b * band) < band ? (tiles_m - b * band) : band;  // the last band may be lower
    tm = b * band + r % rows;
    tn = r / rows;
}


// The kernel of hgemm_agpr.hip (256x256 tiles, one wavefront per SIMD, accumulators in AGPRs).  band / rot_*: as in
// HgemmArgs.
const char* hgemm_big_name();
// gate: 0, or HgemmArgs::gate of a gated launch (N then counts the rows of both matrices in B, C has N / 2 columns).
bool hgemm_big_applies(const void* A, const void* B, const void* C, size_t M, size_t N, size_t K, size_t ldc, size_t gate = 0);
int launch_hgemm_big(const void* A, const void* B, void* C, size_t M, size_t N, size_t K, size_t ldc, int band, int rot_tile,
                     int rot_xcd, size_t gate = 0);
// Inspection: the following launches of both kernels write 2 x workgroups time stamps (HgemmArgs::stamps) into buf when it
// holds that many 64-bit words; null switches it off.
void hgemm_agpr_set_stamps(void* buf, size_t capacity);
// and its 256x128 sibling (three-stage ring, one C tile per workgroup)
const char* hgemm_mid_name();
bool hgemm_mid_applies(const void* A, const void* B, const void* C, size_t M, size_t N, size_t K, size_t ldc);
int launch_hgemm_mid(const void* A, const void* B, void* C, size_t M, size_t N, size_t K, size_t ldc, int band, int rot_tile,
                     int rot_xcd);

}  // namespace tl
