// Internal helpers shared by the HIP translation units of libtensorlib_amd.so.
#pragma once
#include <hip/hip_runtime.h>
#include <cstdarg>
#include <cstddef>
#include <cstdint>
#include <cstdio>
#include <mutex>

#include "tensorlib_amd.h"

namespace tl {

typedef _Float16 half_t;
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));
typedef float float16_t __attribute__((ext_vector_type(16)));

constexpr int kWave = 64;  // CDNA wavefront width

// Per-thread last-error message; set_error returns `code` so call sites can `return set_error(...)`.
int set_error(int code, const char* fmt, ...) __attribute__((format(printf, 2, 3)));
void clear_error();

// Stream all kernels of this library are enqueued on.
hipStream_t stream();

// Device facts gathered by tl_init (lazily initialised on first use).
struct DeviceInfo {
    int ordinal = -1;
    int cu_count = 0;
    int wave_size = 0;
    size_t lds_per_block = 0;
    char arch[64] = {0};
};
const DeviceInfo& device_info();
int ensure_init();

// Library-owned fp32 device scratch that grows on demand (split-K partial sums, attention chunk partials).
// acquire() returns with the buffer's mutex held by the lease: the caller keeps the lease alive until every
// kernel that touches the pointer is enqueued, so no other host thread can grow (free) the buffer in between.
// Reuse is ordered by the library's stream; tl_set_stream drains the stream it replaces once a workspace has been
// used on it, so no stream handle outlives its owner here.  A buffer starts out all zero (written by a fill kernel,
// which a stream capture can record) and its first `head` floats hold the users' counters, which every kernel
// leaves at zero when it completes; zero_head() puts them back after a launch that did not.
class Workspace {
 public:
    struct Lease {
        std::unique_lock<std::mutex> lock;
        float* ptr = nullptr;
    };
    int acquire(size_t floats, size_t min_floats, const char* what, Lease* lease);
    int zero_head(size_t floats);

 private:
    std::mutex mu_;
    float* ptr_ = nullptr;
    size_t floats_ = 0;
};
// true once any workspace has been handed out since the library's stream was last drained by tl_set_stream
bool workspaces_in_use();

// Counter words at the head of the scratch buffers.  Decode attention: one ticket per head (launches with more
// heads merge with a second kernel).  Split-K GEMM: one ticket per C tile (launches with more tiles reduce with a
// second kernel).
constexpr size_t kAttnTicketWords = 1024;
constexpr size_t kSplitkTicketWords = 4096;
int attention_reset_tickets();   // zero the ticket words of both attention scratch buffers (workspace and static)
int splitk_reset_tickets();

// Looks up (once per device) the device address of the static scratch array behind
// tl_decode_attention_rope_static_f16 for the current device; `out` may be null.
int attention_static_scratch(float** out);

// out[i] = bits for i < n, as a kernel (safe to record into a HIP graph).
int launch_fill_f16(void* out, uint16_t bits, size_t n);

// Shared launchers (batch strides in elements; batch == 1 ignores them).
// prologue 0: plain x; 1: x is [a | b], the multiplied vector is silu(a) * b; 2: the multiplied vector is
// rmsnorm(x + norm->addend) * norm->weight and norm->sum_out receives half(x + addend).
struct GemvNormPrologue {
    const void* addend;  // may be null
    const void* weight;
    void* sum_out;       // may be null
    float eps;
};
int launch_gemv(const void* x, const void* W, void* y, size_t N, size_t K, size_t batch, size_t sx,
                size_t sw, size_t sy, int prologue, const GemvNormPrologue* norm = nullptr);
// partials_out / splits_out (both or neither): when K was split, the fp32 slabs [splits][M][N] are handed to the
// caller instead of being reduced into C (library-owned, valid until the next GEMM on the stream); *splits_out == 1
// means C holds the result.
// `lease` then keeps the slabs' buffer locked until the caller has enqueued its consumer.
int launch_hgemm(const void* A, const void* B, void* C, size_t M, size_t N, size_t K, size_t batch,
                 size_t sa, size_t sb, size_t sc, float** partials_out = nullptr, int* splits_out = nullptr,
                 Workspace::Lease* lease = nullptr, size_t gate = 0);
// gate != 0 (batch 1, no slabs): B stacks two matrices `gate` rows apart, N counts the rows of both, and
// C[M, N/2] = silu(A.B1^T) * (A.B2^T), the gate applied in the GEMM's epilogue.  Only where hgemm_gated_applies() says so.
bool hgemm_gated_applies(const void* A, const void* B, const void* C, size_t M, size_t n_out, size_t K, size_t gate);

// Very few rows (2 <= M <= 32, K <= 4096): X stays in registers, W streams through once (hgemm_fewrows.hip).
bool hgemm_fewrows_applies(size_t M, size_t N, size_t K, size_t ldc, size_t batch);
int launch_hgemm_fewrows(const void* X, const void* W, void* C, size_t M, size_t N, size_t K, size_t ldc);

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

#if defined(__HIPCC__)
// One global_load_lds_dwordx4: lane l's 16 bytes at `src` go to LDS bytes [dst + 16*l, +16).
// Written as inline assembly on purpose: the compiler models this instruction as a flat access that may
// touch LDS, and while one is outstanding (always, in a ring whose vmcnt waits it cannot see) it turns
// every wait for ds_read data into lgkmcnt(0), including reads issued an instant earlier.  Hidden from
// it, the ds_reads are the only lgkmcnt traffic and get exact in-order counts.
__device__ __forceinline__ void load_16B_per_lane_to_lds(const half_t* src,
                                                         __attribute__((address_space(3))) unsigned char* dst) {
    const unsigned lds_addr = (unsigned)(unsigned long)dst;
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(src), "s"(lds_addr) : "memory");
}

// The same instruction with the address split into a wavefront-uniform base (a scalar register pair) and a
// 32-bit byte offset per lane: a tile's per-lane offsets stay put while only the base moves along K, so a
// request costs no vector arithmetic.
__device__ __forceinline__ void load_16B_per_lane_to_lds(const void* uniform_base, unsigned lane_offset,
                                                         unsigned lds_addr) {
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %0"
                 ::"s"(uniform_base), "v"(lane_offset), "s"(lds_addr) : "memory");
}

// Rotary embedding, with every rounding of the reference's CPU loop (tensorLib/src/device/cpu/CPU.cpp:444-453):
// the angle is an fp32 quotient, cos and sin are rounded to half, each of the four products is rounded to half
// and so are their difference and sum.  cos, sin and the power are evaluated in double and rounded to fp32 once,
// i.e. they are the correctly rounded fp32 values a host libm returns for the same fp32 argument.
__device__ __forceinline__ void rope_cos_sin(int pos, int d, int head_dim, float& c, float& s) {
    const float base = (float)pow(10000.0, (double)((float)d / (float)head_dim));
    const float theta = (float)pos * 1.0f / base;
    float cf = (float)cos((double)theta), sf = (float)sin((double)theta);
    // the reference rounds double -> fp32 -> half; without this the compiler merges the two conversions into one
    // double -> half rounding, which differs when the fp32 value lands on a half-way point
    asm volatile("" : "+v"(cf), "+v"(sf));
    c = (float)(half_t)cf;
    s = (float)(half_t)sf;
}
__device__ __forceinline__ half2_t rope_rotate(float v0, float v1, float c, float s) {
#pragma clang fp contract(off)  // a fused multiply-add would skip the rounding of the second product
    const float p0 = (float)(half_t)(v0 * c), p1 = (float)(half_t)(v1 * s);
    const float p2 = (float)(half_t)(v0 * s), p3 = (float)(half_t)(v1 * c);
    half2_t r = {(half_t)(p0 - p1), (half_t)(p2 + p3)};
    return r;
}

template <int N_>
__device__ __forceinline__ void wait_vmcnt_and_barrier() {
    // waits until at most N_ of this wavefront's global->LDS loads are outstanding and all of its
    // LDS reads have returned, then joins the workgroup barrier; the "memory" clobber keeps LDS
    // accesses on their side of it
    asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" ::"n"(N_) : "memory");
}
#endif  // __HIPCC__

}  // namespace tl

#define TL_HIP_TRY(expr)                                                                        \
    do {                                                                                        \
        hipError_t _e = (expr);                                                                 \
        if (_e != hipSuccess)                                                                   \
            return tl::set_error(TL_EHIP, "%s failed: %s (%s:%d)", #expr, hipGetErrorString(_e), \
                                 __FILE__, __LINE__);                                           \
    } while (0)

// After a kernel launch: surfaces launch-configuration errors without synchronising.
#define TL_CHECK_LAUNCH(name)                                                                       \
    do {                                                                                            \
        hipError_t _e = hipGetLastError();                                                          \
        if (_e != hipSuccess)                                                                       \
            return tl::set_error(TL_EHIP, "launch of %s failed: %s", name, hipGetErrorString(_e));  \
    } while (0)

#define TL_REQUIRE(cond, ...)                                   \
    do {                                                        \
        if (!(cond)) return tl::set_error(TL_EINVAL, __VA_ARGS__); \
    } while (0)

#define TL_ENSURE_INIT()                 \
    do {                                 \
        int _rc = tl::ensure_init();     \
        if (_rc != TL_OK) return _rc;    \
    } while (0)
