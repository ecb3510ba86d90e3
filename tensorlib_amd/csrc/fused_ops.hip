// The small kernels that sit between the matmuls of a Llama2 decode step, so the loop never
// leaves the GPU: RMSNorm, RoPE, softmax, SiLU, elementwise add/sub/mul/div, strided
// gather/scatter (contiguous / setItemEwise), argmax, embedding lookup, fill.
// All HBM-trivial; written for 64-lane wavefronts with 16-byte accesses where alignment allows.
#include <cstring>

#include "tl_internal.h"

namespace tl {

// ------------------------------------------------------------------ reductions ----

template <int CTRL>
__device__ __forceinline__ float dpp_f(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true));
}
__device__ __forceinline__ float readlane_f(float v, int l) {
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), l));
}
__device__ __forceinline__ float wave_sum_f(float v) {
    v += dpp_f<0xB1>(v);
    v += dpp_f<0x4E>(v);
    v += dpp_f<0x141>(v);
    v += dpp_f<0x140>(v);
    return (readlane_f(v, 0) + readlane_f(v, 16)) + (readlane_f(v, 32) + readlane_f(v, 48));
}
__device__ __forceinline__ float wave_max_f(float v) {
    v = fmaxf(v, dpp_f<0xB1>(v));
    v = fmaxf(v, dpp_f<0x4E>(v));
    v = fmaxf(v, dpp_f<0x141>(v));
    v = fmaxf(v, dpp_f<0x140>(v));
    return fmaxf(fmaxf(readlane_f(v, 0), readlane_f(v, 16)), fmaxf(readlane_f(v, 32), readlane_f(v, 48)));
}

// Workgroup-wide sum / max for up to 16 wavefronts; `red` is 16 floats of LDS.
__device__ __forceinline__ float block_sum_f(float v, float* red) {
    v = wave_sum_f(v);
    const int nw = blockDim.x >> 6;
    if (nw == 1) return v;
    __syncthreads();
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
    __syncthreads();
    float s = 0.f;
    for (int w = 0; w < nw; ++w) s += red[w];
    return s;
}
__device__ __forceinline__ float block_max_f(float v, float* red) {
    v = wave_max_f(v);
    const int nw = blockDim.x >> 6;
    if (nw == 1) return v;
    __syncthreads();
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
    __syncthreads();
    float s = red[0];
    for (int w = 1; w < nw; ++w) s = fmaxf(s, red[w]);
    return s;
}

// --------------------------------------------------------------------- RMSNorm ----

// One workgroup per token.  fp32 sum of squares, out = x * w * rsqrt(mean + eps), one rounding.
template <bool VEC>
__global__ void __launch_bounds__(256)
rms_norm_kernel(half_t* out, const half_t* in, const half_t* w, float eps,
                int hidden) {
    __shared__ float red[16];
    const size_t base = (size_t)blockIdx.x * hidden;
    const half_t* x = in + base;
    half_t* o = out + base;
    float ss = 0.f;
    if constexpr (VEC) {
        const half8_t* x8 = reinterpret_cast<const half8_t*>(x);
        for (int c = threadIdx.x; c < hidden / 8; c += blockDim.x) {
            half8_t v = x8[c];
#pragma unroll
            for (int i = 0; i < 8; ++i) ss = __builtin_fmaf((float)v[i], (float)v[i], ss);
        }
    } else {
        for (int i = threadIdx.x; i < hidden; i += blockDim.x) ss = __builtin_fmaf((float)x[i], (float)x[i], ss);
    }
    ss = block_sum_f(ss, red);
    const float r = 1.0f / sqrtf(ss / (float)hidden + eps);
    if constexpr (VEC) {
        const half8_t* x8 = reinterpret_cast<const half8_t*>(x);
        const half8_t* w8 = reinterpret_cast<const half8_t*>(w);
        half8_t* o8 = reinterpret_cast<half8_t*>(o);
        for (int c = threadIdx.x; c < hidden / 8; c += blockDim.x) {
            half8_t v = x8[c], g = w8[c], res;
#pragma unroll
            for (int i = 0; i < 8; ++i) res[i] = (half_t)((float)v[i] * r * (float)g[i]);
            o8[c] = res;
        }
    } else {
        for (int i = threadIdx.x; i < hidden; i += blockDim.x) o[i] = (half_t)((float)x[i] * r * (float)w[i]);
    }
}

// ------------------------------------------------------------------------ RoPE ----

// One thread per (even, odd) pair of a contiguous [B,T,H,D] tensor.
__global__ void __launch_bounds__(256)
rope_kernel(const half_t* in, half_t* out, int start_pos, int T, int n_heads, int head_dim,
            size_t n_pairs) {
    const size_t p = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (p >= n_pairs) return;
    const int half_d = head_dim / 2;
    const int dp = (int)(p % half_d);
    const size_t bth = p / half_d;           // (b*T + t)*H + h
    const int t = (int)((bth / n_heads) % T);
    const int d = dp * 2;
    float c, s;
    rope_cos_sin(start_pos + t, d, head_dim, c, s);
    const half2_t v = *reinterpret_cast<const half2_t*>(in + 2 * p);
    const half2_t r = rope_rotate((float)v[0], (float)v[1], c, s);
    *reinterpret_cast<half2_t*>(out + 2 * p) = r;
}

// --------------------------------------------------------------------- softmax ----

// One workgroup (64..256 threads) per row; fp32 max and sum.
__global__ void __launch_bounds__(256)
softmax_kernel(half_t* out, const half_t* in, size_t cols) {
    __shared__ float red[16];
    const half_t* x = in + (size_t)blockIdx.x * cols;
    half_t* o = out + (size_t)blockIdx.x * cols;
    float mx = -INFINITY;
    for (size_t j = threadIdx.x; j < cols; j += blockDim.x) mx = fmaxf(mx, (float)x[j]);
    mx = block_max_f(mx, red);
    float sum = 0.f;
    for (size_t j = threadIdx.x; j < cols; j += blockDim.x) sum += expf((float)x[j] - mx);
    sum = block_sum_f(sum, red);
    const float inv = 1.0f / sum;
    for (size_t j = threadIdx.x; j < cols; j += blockDim.x) o[j] = (half_t)(expf((float)x[j] - mx) * inv);
}

// ----------------------------------------------------------------- elementwise ----

struct SiluOp {
    __device__ static half_t apply(half_t a, half_t) {
        const float x = (float)a;
        return (half_t)(x * (1.0f / (1.0f + expf(-x))));
    }
};
struct SiluMulOp {
    __device__ static half_t apply(half_t a, half_t b) {
        const float x = (float)a;
        return (half_t)(x * (1.0f / (1.0f + expf(-x))) * (float)b);
    }
};
struct AddOp { __device__ static half_t apply(half_t a, half_t b) { return (half_t)((float)a + (float)b); } };
struct SubOp { __device__ static half_t apply(half_t a, half_t b) { return (half_t)((float)a - (float)b); } };
struct MulOp { __device__ static half_t apply(half_t a, half_t b) { return (half_t)((float)a * (float)b); } };
struct DivOp { __device__ static half_t apply(half_t a, half_t b) { return (half_t)((float)a / (float)b); } };

// In-place softmax over rows of attention scores with the two elementwise steps that precede it in
// Attention::forward folded into the load: v = half(x / divisor) (ScalarDiv), columns beyond
// start_pos + (row % seqlen) are -inf (the causal mask EwiseAdd would have made them -inf).  The values
// entering the softmax are the same halves the three-kernel chain would have read.
__global__ void __launch_bounds__(256)
scaled_causal_softmax_kernel(half_t* scores, half_t divisor, int seqlen, int start_pos, size_t cols) {
    __shared__ float red[16];
    half_t* x = scores + (size_t)blockIdx.x * cols;
    const size_t limit = (size_t)start_pos + (blockIdx.x % (unsigned)seqlen);  // last visible column
    const float d = (float)divisor;
    auto val = [&](size_t j) { return j <= limit ? (float)(half_t)((float)x[j] / d) : -INFINITY; };
    float mx = -INFINITY;
    for (size_t j = threadIdx.x; j < cols; j += blockDim.x) mx = fmaxf(mx, val(j));
    mx = block_max_f(mx, red);
    float sum = 0.f;
    for (size_t j = threadIdx.x; j < cols; j += blockDim.x) sum += expf(val(j) - mx);
    sum = block_sum_f(sum, red);
    const float inv = 1.0f / sum;
    for (size_t j = threadIdx.x; j < cols; j += blockDim.x) x[j] = (half_t)(expf(val(j) - mx) * inv);
}

// out[r][j] = silu(ab[r][j]) * ab[r][hidden + j]: SwiGLU gate on the rows of a fused w1|w3 projection.
__global__ void __launch_bounds__(256)
silu_mul_rows_kernel(half_t* out, const half_t* ab, int hidden, size_t n8) {
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    const size_t h8 = (size_t)hidden / 8;
    for (size_t c = (size_t)blockIdx.x * blockDim.x + threadIdx.x; c < n8; c += stride) {
        const size_t r = c / h8, j = c % h8;
        const half8_t va = reinterpret_cast<const half8_t*>(ab)[r * 2 * h8 + j];
        const half8_t vb = reinterpret_cast<const half8_t*>(ab)[r * 2 * h8 + h8 + j];
        half8_t o;
#pragma unroll
        for (int e = 0; e < 8; ++e) o[e] = SiluMulOp::apply(va[e], vb[e]);
        reinterpret_cast<half8_t*>(out)[c] = o;
    }
}

// out[i] = Op(a[i], b[i])  (B_MODE 0: no second operand, 1: tensor, 2: scalar)
template <typename Op, int B_MODE, bool VEC>
__global__ void __launch_bounds__(256)
ewise_kernel(half_t* out, const half_t* a, const half_t* b, half_t scalar,
             size_t n) {
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if constexpr (VEC) {
        const size_t n8 = n / 8;
        for (size_t c = i; c < n8; c += stride) {
            half8_t va = reinterpret_cast<const half8_t*>(a)[c], vb, r;
            if constexpr (B_MODE == 1) vb = reinterpret_cast<const half8_t*>(b)[c];
#pragma unroll
            for (int e = 0; e < 8; ++e)
                r[e] = Op::apply(va[e], B_MODE == 1 ? vb[e] : scalar);
            reinterpret_cast<half8_t*>(out)[c] = r;
        }
        for (size_t j = n8 * 8 + i; j < n; j += stride) out[j] = Op::apply(a[j], B_MODE == 1 ? b[j] : scalar);
    } else {
        for (; i < n; i += stride) out[i] = Op::apply(a[i], B_MODE == 1 ? b[i] : scalar);
    }
}

__global__ void __launch_bounds__(256) fill_kernel(half_t* out, half_t v, size_t n) {
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) out[i] = v;
}

static inline unsigned ewise_blocks(size_t work_items) {
    size_t b = (work_items + 255) / 256;
    const size_t cap = (size_t)device_info().cu_count * 16;
    if (b > cap) b = cap;
    if (b == 0) b = 1;
    return (unsigned)b;
}

template <typename Op, int B_MODE>
static int launch_ewise(void* out, const void* a, const void* b, uint16_t scalar_bits, size_t n, const char* name) {
    if (n == 0) return TL_OK;
    half_t scalar = __builtin_bit_cast(half_t, scalar_bits);
    const bool vec = aligned16(out) && aligned16(a) && (B_MODE != 1 || aligned16(b)) && n >= 8;
    if (vec) {
        hipLaunchKernelGGL((ewise_kernel<Op, B_MODE, true>), dim3(ewise_blocks(n / 8)), dim3(256), 0, stream(),
                           (half_t*)out, (const half_t*)a, (const half_t*)b, scalar, n);
    } else {
        hipLaunchKernelGGL((ewise_kernel<Op, B_MODE, false>), dim3(ewise_blocks(n)), dim3(256), 0, stream(),
                           (half_t*)out, (const half_t*)a, (const half_t*)b, scalar, n);
    }
    TL_CHECK_LAUNCH(name);
    return TL_OK;
}

int launch_fill_f16(void* out, uint16_t bits, size_t n) {
    if (n == 0) return TL_OK;
    hipLaunchKernelGGL(fill_kernel, dim3(ewise_blocks(n)), dim3(256), 0, stream(), (half_t*)out,
                       __builtin_bit_cast(half_t, bits), n);
    TL_CHECK_LAUNCH("fill_kernel");
    return TL_OK;
}

// ---------------------------------------------------------- strided gather/scatter ----

constexpr int kMaxDims = 8;
struct StridedView {
    int ndim;
    int shape[kMaxDims];
    int stride[kMaxDims];
    size_t offset;
};

__device__ __forceinline__ size_t view_index(size_t lin, const StridedView& v) {
    size_t r = v.offset;
    for (int d = v.ndim - 1; d >= 0; --d) {
        const size_t s = (size_t)v.shape[d];
        const size_t id = lin % s;
        lin /= s;
        r += id * (size_t)(long)v.stride[d];
    }
    return r;
}

// GATHER: out[i] = base[view(i)];  !GATHER: base[view(i)] = src[i].  VEC moves 8 halves per
// thread and requires a unit-stride last dimension whose extent, like every other stride
// and the offset, is a multiple of 8.
template <bool GATHER, bool VEC>
__global__ void __launch_bounds__(256)
strided_copy_kernel(half_t* dense, half_t* base, StridedView v, size_t n) {
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if constexpr (VEC) {
        for (size_t c = i; c < n / 8; c += stride) {
            const size_t src = view_index(c * 8, v);
            if constexpr (GATHER)
                reinterpret_cast<half8_t*>(dense)[c] = *reinterpret_cast<const half8_t*>(base + src);
            else
                *reinterpret_cast<half8_t*>(base + src) = reinterpret_cast<const half8_t*>(dense)[c];
        }
    } else {
        for (; i < n; i += stride) {
            const size_t src = view_index(i, v);
            if constexpr (GATHER)
                dense[i] = base[src];
            else
                base[src] = dense[i];
        }
    }
}

template <bool GATHER>
static int launch_strided(void* dense, void* base, const int* shape, const int* stride, int ndim, size_t offset,
                          size_t n, const char* name) {
    if (n == 0) return TL_OK;
    TL_REQUIRE(dense && base, "%s: null pointer", name);
    TL_REQUIRE(ndim >= 1 && ndim <= kMaxDims, "%s: ndim %d not in [1,%d]", name, ndim, kMaxDims);
    TL_REQUIRE(shape && stride, "%s: null shape/stride", name);
    StridedView v;
    v.ndim = ndim;
    v.offset = offset;
    size_t total = 1;
    bool vec = aligned16(dense) && aligned16(base) && (offset % 8 == 0) && stride[ndim - 1] == 1 &&
               shape[ndim - 1] % 8 == 0;
    for (int d = 0; d < ndim; ++d) {
        TL_REQUIRE(shape[d] > 0, "%s: shape[%d] = %d must be positive", name, d, shape[d]);
        TL_REQUIRE(stride[d] >= 0, "%s: negative stride[%d] = %d", name, d, stride[d]);
        v.shape[d] = shape[d];
        v.stride[d] = stride[d];
        total *= (size_t)shape[d];
        if (d != ndim - 1 && stride[d] % 8 != 0) vec = false;
    }
    for (int d = ndim; d < kMaxDims; ++d) { v.shape[d] = 1; v.stride[d] = 0; }
    TL_REQUIRE(total == n, "%s: num_elements %zu does not match the shape product %zu", name, n, total);
    if (vec)
        hipLaunchKernelGGL((strided_copy_kernel<GATHER, true>), dim3(ewise_blocks(n / 8)), dim3(256), 0, stream(),
                           (half_t*)dense, (half_t*)base, v, n);
    else
        hipLaunchKernelGGL((strided_copy_kernel<GATHER, false>), dim3(ewise_blocks(n)), dim3(256), 0, stream(),
                           (half_t*)dense, (half_t*)base, v, n);
    TL_CHECK_LAUNCH(name);
    return TL_OK;
}

// ---------------------------------------------------------------------- argmax ----

// One workgroup per row; ties resolve to the smallest index (the CPU backend's strict '>',
// tensorLib/src/device/cpu/CPU.cpp:356-372).  A row with no element above -inf returns 0.
template <bool VEC>
__global__ void __launch_bounds__(1024)
argmax_kernel(int* out, const half_t* in, size_t reduce_size) {
    __shared__ float sv[1024];
    __shared__ int si[1024];
    constexpr int kNone = 0x7fffffff;
    const half_t* x = in + (size_t)blockIdx.x * reduce_size;
    float best = -INFINITY;
    int bi = kNone;
    if constexpr (VEC) {
        // 16-byte loads; a thread visits its chunks, and the elements of a chunk, in increasing index order
        const size_t chunks = reduce_size / 8;
        for (size_t c = threadIdx.x; c < chunks; c += blockDim.x) {
            const half8_t v8 = reinterpret_cast<const half8_t*>(x)[c];
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const float v = (float)v8[e];
                if (v > best) { best = v; bi = (int)(c * 8 + e); }
            }
        }
    } else {
        for (size_t j = threadIdx.x; j < reduce_size; j += blockDim.x) {
            const float v = (float)x[j];
            if (v > best) { best = v; bi = (int)j; }
        }
    }
    sv[threadIdx.x] = best;
    si[threadIdx.x] = bi;
    __syncthreads();
    for (int s = blockDim.x / 2; s > 0; s >>= 1) {
        if ((int)threadIdx.x < s) {
            const float ov = sv[threadIdx.x + s], mv = sv[threadIdx.x];
            const int oi = si[threadIdx.x + s], mi = si[threadIdx.x];
            if (ov > mv || (ov == mv && oi < mi)) {
                sv[threadIdx.x] = ov;
                si[threadIdx.x] = oi;
            }
        }
        __syncthreads();
    }
    if (threadIdx.x == 0) out[blockIdx.x] = si[0] == kNone ? 0 : si[0];
}

// ------------------------------------------------------------------- embedding ----

__global__ void __launch_bounds__(256)
embedding_kernel(half_t* out, const half_t* table, const int* ids, int dim,
                 int vocab) {
    int id = ids[blockIdx.x];
    id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);
    const half_t* src = table + (size_t)id * dim;
    half_t* dst = out + (size_t)blockIdx.x * dim;
    if ((dim & 7) == 0) {
        for (int c = threadIdx.x; c < dim / 8; c += blockDim.x)
            reinterpret_cast<half8_t*>(dst)[c] = reinterpret_cast<const half8_t*>(src)[c];
    } else {
        for (int i = threadIdx.x; i < dim; i += blockDim.x) dst[i] = src[i];
    }
}

}  // namespace tl

// ======================================================================== C ABI ====

extern "C" {

int tl_rms_norm_f16(void* out, const void* in, const void* weight, float eps, int hidden_size, int num_tokens) {
    TL_ENSURE_INIT();
    TL_REQUIRE(out && in && weight, "tl_rms_norm_f16: null pointer");
    TL_REQUIRE(hidden_size > 0 && num_tokens >= 0, "tl_rms_norm_f16: bad sizes hidden=%d tokens=%d", hidden_size,
               num_tokens);
    if (num_tokens == 0) return TL_OK;
    const bool vec = (hidden_size % 8 == 0) && tl::aligned16(out) && tl::aligned16(in) && tl::aligned16(weight);
    if (vec)
        hipLaunchKernelGGL((tl::rms_norm_kernel<true>), dim3(num_tokens), dim3(256), 0, tl::stream(), (tl::half_t*)out,
                           (const tl::half_t*)in, (const tl::half_t*)weight, eps, hidden_size);
    else
        hipLaunchKernelGGL((tl::rms_norm_kernel<false>), dim3(num_tokens), dim3(256), 0, tl::stream(),
                           (tl::half_t*)out, (const tl::half_t*)in, (const tl::half_t*)weight, eps, hidden_size);
    TL_CHECK_LAUNCH("rms_norm_kernel");
    return TL_OK;
}

int tl_apply_rotary_emb_f16(const void* in, void* out, int start_pos, int B, int T, int n_heads, int head_dim) {
    TL_ENSURE_INIT();
    TL_REQUIRE(in && out, "tl_apply_rotary_emb_f16: null pointer");
    TL_REQUIRE(B >= 0 && T >= 0 && n_heads >= 0 && head_dim >= 0 && head_dim % 2 == 0,
               "tl_apply_rotary_emb_f16: bad sizes B=%d T=%d H=%d D=%d (D must be even)", B, T, n_heads, head_dim);
    TL_REQUIRE(((uintptr_t)in & 3) == 0 && ((uintptr_t)out & 3) == 0, "tl_apply_rotary_emb_f16: pointers must be 4-byte aligned");
    const size_t n_pairs = (size_t)B * T * n_heads * (head_dim / 2);
    if (n_pairs == 0) return TL_OK;
    const size_t blocks = (n_pairs + 255) / 256;
    TL_REQUIRE(blocks <= 0x7fffffffu, "tl_apply_rotary_emb_f16: tensor too large");
    hipLaunchKernelGGL(tl::rope_kernel, dim3((unsigned)blocks), dim3(256), 0, tl::stream(), (const tl::half_t*)in,
                       (tl::half_t*)out, start_pos, T, n_heads, head_dim, n_pairs);
    TL_CHECK_LAUNCH("rope_kernel");
    return TL_OK;
}

int tl_softmax_f16(void* out, const void* in, size_t rows, size_t cols) {
    TL_ENSURE_INIT();
    TL_REQUIRE(out && in, "tl_softmax_f16: null pointer");
    if (rows == 0 || cols == 0) return TL_OK;
    TL_REQUIRE(rows <= 0x7fffffffu, "tl_softmax_f16: too many rows (%zu)", rows);
    const int threads = cols <= 64 ? 64 : cols <= 128 ? 128 : 256;
    hipLaunchKernelGGL(tl::softmax_kernel, dim3((unsigned)rows), dim3(threads), 0, tl::stream(), (tl::half_t*)out,
                       (const tl::half_t*)in, cols);
    TL_CHECK_LAUNCH("softmax_kernel");
    return TL_OK;
}

int tl_scaled_causal_softmax_f16(void* scores, uint16_t divisor_bits, int n_heads, int seqlen, int start_pos) {
    TL_ENSURE_INIT();
    TL_REQUIRE(n_heads >= 0 && seqlen >= 0 && start_pos >= 0, "tl_scaled_causal_softmax_f16: negative size");
    const size_t rows = (size_t)n_heads * seqlen, cols = (size_t)start_pos + seqlen;
    if (rows == 0) return TL_OK;
    TL_REQUIRE(scores, "tl_scaled_causal_softmax_f16: null pointer");
    TL_REQUIRE(rows <= 0x7fffffffu, "tl_scaled_causal_softmax_f16: too many rows (%zu)", rows);
    tl::half_t d;
    memcpy(&d, &divisor_bits, 2);
    const int threads = cols <= 64 ? 64 : cols <= 128 ? 128 : 256;
    hipLaunchKernelGGL(tl::scaled_causal_softmax_kernel, dim3((unsigned)rows), dim3(threads), 0, tl::stream(),
                       (tl::half_t*)scores, d, seqlen, start_pos, cols);
    TL_CHECK_LAUNCH("scaled_causal_softmax_kernel");
    return TL_OK;
}

int tl_silu_mul_rows_f16(void* out, const void* ab, size_t rows, size_t hidden) {
    TL_ENSURE_INIT();
    if (rows == 0 || hidden == 0) return TL_OK;
    TL_REQUIRE(out && ab, "tl_silu_mul_rows_f16: null pointer");
    TL_REQUIRE(hidden % 8 == 0 && hidden <= 0x7fffffffu && tl::aligned16(out) && tl::aligned16(ab),
               "tl_silu_mul_rows_f16: needs hidden %% 8 == 0 and 16-byte aligned operands");
    const size_t n8 = rows * hidden / 8;
    size_t blocks = (n8 + 255) / 256;
    const size_t cap = (size_t)tl::device_info().cu_count * 16;
    if (blocks > cap) blocks = cap;
    hipLaunchKernelGGL(tl::silu_mul_rows_kernel, dim3((unsigned)blocks), dim3(256), 0, tl::stream(), (tl::half_t*)out,
                       (const tl::half_t*)ab, (int)hidden, n8);
    TL_CHECK_LAUNCH("silu_mul_rows_kernel");
    return TL_OK;
}

int tl_silu_f16(void* out, const void* in, size_t n) {
    TL_ENSURE_INIT();
    TL_REQUIRE(n == 0 || (out && in), "tl_silu_f16: null pointer");
    return tl::launch_ewise<tl::SiluOp, 0>(out, in, nullptr, 0, n, "silu");
}

int tl_silu_mul_f16(void* out, const void* a, const void* b, size_t n) {
    TL_ENSURE_INIT();
    TL_REQUIRE(n == 0 || (out && a && b), "tl_silu_mul_f16: null pointer");
    return tl::launch_ewise<tl::SiluMulOp, 1>(out, a, b, 0, n, "silu_mul");
}

int tl_binary_f16(void* out, const void* a, const void* b, size_t n, int op) {
    TL_ENSURE_INIT();
    TL_REQUIRE(n == 0 || (out && a && b), "tl_binary_f16: null pointer");
    switch (op) {
        case 0: return tl::launch_ewise<tl::AddOp, 1>(out, a, b, 0, n, "add");
        case 1: return tl::launch_ewise<tl::SubOp, 1>(out, a, b, 0, n, "sub");
        case 2: return tl::launch_ewise<tl::MulOp, 1>(out, a, b, 0, n, "mul");
        case 3: return tl::launch_ewise<tl::DivOp, 1>(out, a, b, 0, n, "div");
        default: return tl::set_error(TL_EINVAL, "tl_binary_f16: unknown op %d", op);
    }
}

int tl_binary_scalar_f16(void* out, const void* a, uint16_t scalar_bits, size_t n, int op) {
    TL_ENSURE_INIT();
    TL_REQUIRE(n == 0 || (out && a), "tl_binary_scalar_f16: null pointer");
    switch (op) {
        case 0: return tl::launch_ewise<tl::AddOp, 2>(out, a, nullptr, scalar_bits, n, "add_scalar");
        case 1: return tl::launch_ewise<tl::SubOp, 2>(out, a, nullptr, scalar_bits, n, "sub_scalar");
        case 2: return tl::launch_ewise<tl::MulOp, 2>(out, a, nullptr, scalar_bits, n, "mul_scalar");
        case 3: return tl::launch_ewise<tl::DivOp, 2>(out, a, nullptr, scalar_bits, n, "div_scalar");
        default: return tl::set_error(TL_EINVAL, "tl_binary_scalar_f16: unknown op %d", op);
    }
}

int tl_contiguous_f16(void* out, const void* base, const int* host_shape, const int* host_stride, int ndim,
                      size_t offset, size_t n) {
    TL_ENSURE_INIT();
    return tl::launch_strided<true>(out, const_cast<void*>(base), host_shape, host_stride, ndim, offset, n,
                                    "tl_contiguous_f16");
}

int tl_set_item_ewise_f16(void* base, const void* src, const int* host_shape, const int* host_stride, int ndim,
                          size_t offset, size_t n) {
    TL_ENSURE_INIT();
    return tl::launch_strided<false>(const_cast<void*>(src), base, host_shape, host_stride, ndim, offset, n,
                                     "tl_set_item_ewise_f16");
}

int tl_argmax_f16(int* out, const void* in, size_t reduce_size, size_t num_elements) {
    TL_ENSURE_INIT();
    TL_REQUIRE(out && in, "tl_argmax_f16: null pointer");
    TL_REQUIRE(reduce_size > 0 && num_elements % reduce_size == 0,
               "tl_argmax_f16: num_elements %zu is not a multiple of reduce_size %zu", num_elements, reduce_size);
    const size_t rows = num_elements / reduce_size;
    if (rows == 0) return TL_OK;
    TL_REQUIRE(rows <= 0x7fffffffu && reduce_size <= 0x7fffffffu, "tl_argmax_f16: size out of range");
    const bool vec = reduce_size % 8 == 0 && tl::aligned16(in);
    const int threads = reduce_size >= 8192 ? 1024 : 256;
    if (vec)
        hipLaunchKernelGGL(tl::argmax_kernel<true>, dim3((unsigned)rows), dim3(threads), 0, tl::stream(), out,
                           (const tl::half_t*)in, reduce_size);
    else
        hipLaunchKernelGGL(tl::argmax_kernel<false>, dim3((unsigned)rows), dim3(threads), 0, tl::stream(), out,
                       (const tl::half_t*)in, reduce_size);
    TL_CHECK_LAUNCH("argmax_kernel");
    return TL_OK;
}

int tl_embedding_f16(void* out, const void* table, const int* ids, int n_tokens, int dim, int vocab) {
    TL_ENSURE_INIT();
    TL_REQUIRE(out && table && ids, "tl_embedding_f16: null pointer");
    TL_REQUIRE(n_tokens >= 0 && dim > 0 && vocab > 0, "tl_embedding_f16: bad sizes");
    if (n_tokens == 0) return TL_OK;
    TL_REQUIRE((dim % 8 != 0) || (tl::aligned16(out) && tl::aligned16(table)),
               "tl_embedding_f16: 16-byte aligned buffers required when dim %% 8 == 0");
    hipLaunchKernelGGL(tl::embedding_kernel, dim3(n_tokens), dim3(256), 0, tl::stream(), (tl::half_t*)out,
                       (const tl::half_t*)table, ids, dim, vocab);
    TL_CHECK_LAUNCH("embedding_kernel");
    return TL_OK;
}

int tl_full_f16(void* out, uint16_t value_bits, size_t n) {
    TL_ENSURE_INIT();
    TL_REQUIRE(n == 0 || out, "tl_full_f16: null pointer");
    return tl::launch_fill_f16(out, value_bits, n);
}

}  // extern "C"
