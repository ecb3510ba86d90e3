// Attention helpers for the Llama2 driver.
//
// tl_decode_attention_f16: single-token attention that reads the KV cache in place.  The
// reference (model/llama2_7b/src/Transformer.cpp:55-109) re-gathers the whole K and V cache
// into contiguous scratch every step, then issues 2*n_heads GEMV launches, a scalar divide
// and a softmax.  Here one launch covers all heads: the T cached positions are cut into
// chunks, each (head, chunk) workgroup produces a partial (max, sum, weighted V) triple in
// fp32, and a second tiny launch merges the chunks (the split keeps >= 256 workgroups busy
// although there are only n_heads independent rows).
//
// tl_causal_mask_f16: the additive mask of Transformer::get_mask
// (model/llama2_7b/src/Transformer.cpp:231-261) written by one kernel instead of one
// host-to-device copy per element.
#include <atomic>
#include <mutex>
#include <type_traits>

#include "tl_internal.h"

namespace tl {

// 0: automatic, 1: one wavefront per 32 query rows, 2: LDS-tiled workgroups of 128 query rows (tuning hook)
static std::atomic<int> g_prefill_attention_variant{0};
// where the chunk partials of a head are merged: 0 = automatic, 1 = by the workgroup that finishes the head's last
// chunk, 2 = by a second launch, 3 = like 1 with a release/acquire ticket and plain accesses to the partials
static std::atomic<int> g_decode_merge_mode{0};
// Up to this many chunks the in-kernel merge is ahead (384 positions: 7.6 against 10.2 us for the pair of launches;
// 1024 positions: equal; 1951 positions: 14.7 against 13.2 us, the merging workgroup's serial walk over 31 partials
// through device-coherent loads then costs more than a launch).
constexpr int kMergeInKernelMaxChunks = 8;

template <int CTRL>
__device__ __forceinline__ float dppf(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true));
}

// Sum over groups of LPR adjacent lanes, LPR in {8,16,32}; all lanes of a group get the sum.
template <int LPR>
__device__ __forceinline__ float lanes_sum(float v) {
    v += dppf<0xB1>(v);
    v += dppf<0x4E>(v);
    v += dppf<0x141>(v);
    if constexpr (LPR >= 16) v += dppf<0x140>(v);
    if constexpr (LPR == 32) v += __shfl_xor(v, 16, 64);
    return v;
}

constexpr int kAttnThreads = 256;
constexpr int kAttnChunk = 64;  // cached positions per workgroup when a context is cut into many chunks
// tuning hook: cached positions per workgroup, 0 = automatic, else 64, 128 or 256
static std::atomic<int> g_decode_chunk{0};

// partial layout per (head, chunk): [0] = max, [1] = sum, [2 .. 2+head_dim) = sum_t p_t * V[t]
// Rotate the 4 (even, odd) pairs of one 16-byte chunk of a head vector; `d0` is the index of the
// chunk's first element inside the head.  Same arithmetic as rope_kernel (rope_cos_sin, rope_rotate).
__device__ __forceinline__ half8_t rope_chunk(half8_t v, int pos, int d0, int head_dim) {
    half8_t r;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        float c, s;
        rope_cos_sin(pos, d0 + 2 * i, head_dim, c, s);
        const half2_t o = rope_rotate((float)v[2 * i], (float)v[2 * i + 1], c, s);
        r[2 * i] = o[0];
        r[2 * i + 1] = o[1];
    }
    return r;
}

// Same rotation with (cos, sin) pairs read from a table built by rope_table_kernel.
__device__ __forceinline__ half8_t rope_chunk_cs(half8_t v, half8_t cs) {
    half8_t r;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const half2_t o = rope_rotate((float)v[2 * i], (float)v[2 * i + 1], (float)cs[2 * i], (float)cs[2 * i + 1]);
        r[2 * i] = o[0];
        r[2 * i + 1] = o[1];
    }
    return r;
}

// table[pos][pair] = (half(cos(theta)), half(sin(theta))), theta = pos / 10000^(2*pair/head_dim) in fp32
// (rope_cos_sin): the values every RoPE kernel of this library computes on the fly.
__global__ void __launch_bounds__(256) rope_table_kernel(half_t* table, int max_seq, int head_dim) {
    const int half_d = head_dim / 2;
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= (size_t)max_seq * half_d) return;
    const int pos = (int)(i / half_d), pair = (int)(i % half_d);
    float c, s;
    rope_cos_sin(pos, 2 * pair, head_dim, c, s);
    half2_t cs = {(half_t)c, (half_t)s};
    *reinterpret_cast<half2_t*>(table + 2 * i) = cs;
}

// Merge of the chunk partials of head h for output dimension d (base: the head's first partial).  COHERENT: the
// partials were written by other workgroups of the SAME launch and are read with device-coherent loads.
template <bool COHERENT>
__device__ __forceinline__ void merge_head(half_t* out, const float* base, int h, int D, int n_chunks, int d) {
    auto ldp = [](const float* p) {
        if constexpr (COHERENT) return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        else return *p;
    };
    // Sixteen chunks per round trip (a long context has dozens of chunks, and a dependent load per chunk would
    // cost a memory latency each), folded in with the online-softmax update, so the maxima need no pass of their
    // own; the sums run over the chunks in ascending order.
    constexpr int U = 16;
    float m = -INFINITY, l = 0.f, o = 0.f;
    for (int c0 = 0; c0 < n_chunks; c0 += U) {
        float pm[U], pl[U], po[U];
#pragma unroll
        for (int j = 0; j < U; ++j) {
            const float* p = base + (size_t)(c0 + j < n_chunks ? c0 + j : c0) * (D + 2);
            pm[j] = ldp(p);
            pl[j] = ldp(p + 1);
            po[j] = ldp(p + 2 + d);
        }
        float m_new = m;
#pragma unroll
        for (int j = 0; j < U; ++j)
            if (c0 + j < n_chunks) m_new = fmaxf(m_new, pm[j]);
        const float scale = expf(m - m_new);   // 0 on the first round (m = -inf), 1 when the maximum stays
        l *= scale;
        o *= scale;
        m = m_new;
#pragma unroll
        for (int j = 0; j < U; ++j) {
            if (c0 + j < n_chunks) {
                const float w = expf(pm[j] - m);
                l = __builtin_fmaf(pl[j], w, l);
                o = __builtin_fmaf(po[j], w, o);
            }
        }
    }
    out[(size_t)h * D + d] = (half_t)(o / l);
}

// FUSE_ROPE: `q` points at the raw q|k|v projection of the new token (position T-1).  q is rotated
// on load; the workgroup that owns the last chunk rotates the new k row, uses it, and writes it and
// the new v row into the caches (each head's workgroup writes only its own head slice).
// ROPE: 0 = q is already rotated and the caches hold position T-1; 1 = rotate with the table's (cos, sin);
// 2 = rotate with cos/sin evaluated in the kernel (no table given).
// CHUNK: cached positions per workgroup (64, 128 or 256; every thread holds CHUNK / GROUPS rows of K and of V).
template <int LPR, int ROPE, int CHUNK>
__global__ void __launch_bounds__(kAttnThreads)
decode_attn_partial_kernel(half_t* out, float* partial, const half_t* q, half_t* cache_k,
                           half_t* cache_v, const half_t* rope_table, int T, int n_heads, float inv_scale,
                           int n_chunks, unsigned* tickets, int ordered) {
    constexpr int D = LPR * 8;
    constexpr int GROUPS = kAttnThreads / LPR;
    static_assert(CHUNK % 64 == 0 && CHUNK <= kAttnThreads && CHUNK % (kAttnThreads / LPR) == 0, "chunk size");
    __shared__ float sc[CHUNK];
    __shared__ float red[16];
    __shared__ float obuf[GROUPS][D];

    const int h = blockIdx.x;
    const int chunk = blockIdx.y;
    const int t0 = chunk * CHUNK;
    const int t1 = (t0 + CHUNK < T) ? (t0 + CHUNK) : T;
    const int tid = threadIdx.x;
    const int sub = tid % LPR;
    const int grp = tid / LPR;
    const size_t row_stride = (size_t)n_heads * D;

    half8_t qv = *reinterpret_cast<const half8_t*>(q + (size_t)h * D + sub * 8);
    half8_t cs = {0, 0, 0, 0, 0, 0, 0, 0};  // (cos, sin) of the 4 pairs of this thread's chunk at position T-1
    constexpr bool FUSE_ROPE = ROPE != 0;
    if constexpr (ROPE == 1) {
        cs = *reinterpret_cast<const half8_t*>(rope_table + ((size_t)(T - 1) * (D / 2) + sub * 4) * 2);
        qv = rope_chunk_cs(qv, cs);
    } else if constexpr (ROPE == 2) {
        qv = rope_chunk(qv, T - 1, sub * 8, D);
    }

    // All K and V rows this thread will touch are requested up front (NIT rows each), so the whole
    // kernel pays one global round trip instead of one per phase.
    constexpr int NIT = CHUNK / GROUPS;
    half8_t kreg[NIT], vreg[NIT];
    const half8_t zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
    const size_t head_off = (size_t)h * D + sub * 8;
#pragma unroll
    for (int it = 0; it < NIT; ++it) {
        const int t = t0 + grp + it * GROUPS;
        if (t < t1) {
            if (FUSE_ROPE && t == T - 1) {
                kreg[it] = *reinterpret_cast<const half8_t*>(q + row_stride + head_off);
                vreg[it] = *reinterpret_cast<const half8_t*>(q + 2 * row_stride + head_off);
            } else {
                kreg[it] = *reinterpret_cast<const half8_t*>(cache_k + (size_t)t * row_stride + head_off);
                vreg[it] = *reinterpret_cast<const half8_t*>(cache_v + (size_t)t * row_stride + head_off);
            }
        } else {
            kreg[it] = zero8;
            vreg[it] = zero8;
        }
    }

    // scores
#pragma unroll
    for (int it = 0; it < NIT; ++it) {
        const int t = t0 + grp + it * GROUPS;
        if (t < t1) {
            if (FUSE_ROPE && t == T - 1) {
                if constexpr (ROPE == 1) kreg[it] = rope_chunk_cs(kreg[it], cs);
                else kreg[it] = rope_chunk(kreg[it], T - 1, sub * 8, D);
                *reinterpret_cast<half8_t*>(cache_k + (size_t)t * row_stride + head_off) = kreg[it];
                *reinterpret_cast<half8_t*>(cache_v + (size_t)t * row_stride + head_off) = vreg[it];
            }
            float s = 0.f;
#pragma unroll
            for (int i = 0; i < 8; ++i) s = __builtin_fmaf((float)qv[i], (float)kreg[it][i], s);
            s = lanes_sum<LPR>(s);
            if (sub == 0) sc[t - t0] = s * inv_scale;
        }
    }
    __syncthreads();

    // chunk max and sum: thread t holds the score of position t0 + t; 64 positions are reduced by wavefront 0 alone,
    // more by one wavefront per 64 and a second step over the wavefronts' results in ascending order
    float m, l;
    {
        const int n = t1 - t0;
        float v = (tid < n) ? sc[tid] : -INFINITY;
        auto wave_max = [](float x) {
            x = fmaxf(x, dppf<0xB1>(x));
            x = fmaxf(x, dppf<0x4E>(x));
            x = fmaxf(x, dppf<0x141>(x));
            x = fmaxf(x, dppf<0x140>(x));
            x = fmaxf(x, __shfl_xor(x, 16, 64));
            x = fmaxf(x, __shfl_xor(x, 32, 64));
            return x;
        };
        auto wave_sum = [](float x) {
            x += dppf<0xB1>(x);
            x += dppf<0x4E>(x);
            x += dppf<0x141>(x);
            x += dppf<0x140>(x);
            x += __shfl_xor(x, 16, 64);
            x += __shfl_xor(x, 32, 64);
            return x;
        };
        if constexpr (CHUNK == 64) {
            if (tid < 64) {
                const float mx = wave_max(v);
                const float p = (tid < n) ? expf(v - mx) : 0.f;
                const float sm = wave_sum(p);
                if (tid < n) sc[tid] = p;
                if (tid == 0) { red[0] = mx; red[1] = sm; }
            }
            __syncthreads();
            m = red[0];
            l = red[1];
        } else {
            constexpr int RW = CHUNK / 64;
            const int wave = tid / 64;
            float mx = wave_max(v);
            if (tid % 64 == 0) red[wave] = mx;
            __syncthreads();
            mx = red[0];
#pragma unroll
            for (int w = 1; w < RW; ++w) mx = fmaxf(mx, red[w]);
            const float p = (tid < n) ? expf(v - mx) : 0.f;
            const float sm = wave_sum(p);
            if (tid < n) sc[tid] = p;
            if (tid % 64 == 0) red[8 + wave] = sm;
            __syncthreads();
            m = mx;
            l = red[8];
#pragma unroll
            for (int w = 1; w < RW; ++w) l += red[8 + w];
        }
    }

    // weighted sum of V rows: thread (grp, sub) accumulates dims [sub*8, sub*8+8) over its positions
    float acc[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[i] = 0.f;
#pragma unroll
    for (int it = 0; it < NIT; ++it) {
        const int t = t0 + grp + it * GROUPS;
        if (t < t1) {
            const float p = sc[t - t0];
#pragma unroll
            for (int i = 0; i < 8; ++i) acc[i] = __builtin_fmaf(p, (float)vreg[it][i], acc[i]);
        }
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) obuf[grp][sub * 8 + i] = acc[i];
    __syncthreads();
    if (tid < D) {
        float o = 0.f;
#pragma unroll
        for (int g = 0; g < GROUPS; ++g) o += obuf[g][tid];
        if (n_chunks == 1) {
            out[(size_t)h * D + tid] = (half_t)(o / l);
        } else {
            float* p = partial + ((size_t)h * n_chunks + chunk) * (D + 2);
            if (tickets && !ordered) {
                // device-coherent stores: the workgroup that merges may sit on another XCD, behind another L2
                __hip_atomic_store(p + 2 + tid, o, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                if (tid == 0) {
                    __hip_atomic_store(p, m, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    __hip_atomic_store(p + 1, l, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                }
            } else {
                p[2 + tid] = o;
                if (tid == 0) { p[0] = m; p[1] = l; }
            }
        }
    }
    if (tickets == nullptr || n_chunks == 1) return;
    // One launch instead of two: the workgroup that finishes a head's last chunk merges the head, walking the chunks
    // in index order, so the result has the bits of the two-launch path.
    // What orders the partials before the merge (ordered == 0, the default): the partials leave as device-coherent
    // stores (write-through, sc1), every wavefront waits until its stores are acknowledged (s_waitcnt vmcnt(0):
    // on this ISA a store counts as done when the coherent level holds it), the workgroup barrier collects those
    // waits, and only then is the ticket drawn; the workgroup that draws the last ticket reads the partials with
    // device-coherent loads issued after the ticket's value has returned.  That is an ordering by instruction
    // completion, which the HIP memory model does not spell out for relaxed atomics.  ordered == 1 is the same
    // protocol in the model's own terms: plain stores, a release/acquire read-modify-write at device scope on the
    // ticket, plain loads.  It costs a write-back of this XCD's L2 per workgroup and an invalidate in the merging
    // one (32 heads of 128, K and V from HBM, us per call for 256 / 384 / 512 / 1024 cached positions: 7.8 / 9.1 / 10.7 /
    // 16.1 against 7.4 / 7.6 / 7.7 / 10.0 for the default and 10.0 / 10.4 / 10.1 / 10.1 for the second launch), so it is
    // kept as the tested alternative (tl_set_decode_attention_merge(3)), not the default.
    __shared__ int s_last;
    if (!ordered) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (tid == 0) {
        const unsigned t = ordered ? __hip_atomic_fetch_add(tickets + h, 1u, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_AGENT)
                                   : __hip_atomic_fetch_add(tickets + h, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        const int last = (t + 1u == (unsigned)n_chunks);
        if (last) __hip_atomic_store(tickets + h, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);   // ready for the next call
        s_last = last;
    }
    __syncthreads();
    if (!s_last || tid >= D) return;
    if (ordered) merge_head<false>(out, partial + (size_t)h * n_chunks * (D + 2), h, D, n_chunks, tid);
    else merge_head<true>(out, partial + (size_t)h * n_chunks * (D + 2), h, D, n_chunks, tid);
}

// Second pass for long contexts: merge the chunk partials of one head.  (Short contexts merge inside the first
// launch, see the ticket at the end of decode_attn_partial_kernel.  Doing that with device-scope fences around
// plain accesses instead of device-coherent accesses cost 18 us against 12.6 us for two launches: the fences write
// back and invalidate whole L2s.  One 1024-thread workgroup per head covering up to 512 positions alone was slower
// too: 32 workgroups pull a context through 32 CUs' L2 ports instead of 256, and a whole decode step lost 6 %.)
__global__ void __launch_bounds__(256)
decode_attn_merge_kernel(half_t* out, const float* partial, int D, int n_chunks) {
    const int h = blockIdx.x;
    const int d = threadIdx.x;
    if (d >= D) return;
    merge_head<false>(out, partial + (size_t)h * n_chunks * (D + 2), h, D, n_chunks, d);
}

// mask[r, i, j] = (j > start_pos + i) ? -inf : 0 for r < reps, i < seqlen, j < start_pos + seqlen
__global__ void __launch_bounds__(256)
causal_mask_kernel(half_t* mask, int seqlen, int start_pos, size_t n) {
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    const int cols = start_pos + seqlen;
    for (size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x; idx < n; idx += stride) {
        const int j = (int)(idx % cols);
        const int i = (int)((idx / cols) % seqlen);
        mask[idx] = (j > start_pos + i) ? (half_t)(-INFINITY) : (half_t)0.f;
    }
}

// Prefill glue after the q, k, v projections of n_tokens rows (row stride `ld`, e.g. 3*dim for a fused
// q|k|v GEMM): one thread per (token, head, pair).  q is rotated and written head-major [H, S, D] (the
// layout the per-head score matmul wants), k is rotated into cache_k[start_pos + s], v copied into cache_v.
// Same arithmetic as rope_kernel with the table's half-rounded cos/sin.
__global__ void __launch_bounds__(256)
prefill_rope_qkv_kernel(half_t* q_out, const half_t* q, const half_t* k, const half_t* v, size_t ld, half_t* cache_k,
                        half_t* cache_v, const half_t* rope_table, int start_pos, int n_tokens, int n_heads,
                        int head_dim) {
    const int half_d = head_dim / 2;
    const size_t total = (size_t)n_tokens * n_heads * half_d;
    const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= total) return;
    const int pair = (int)(idx % half_d);
    const int h = (int)((idx / half_d) % n_heads);
    const int s = (int)(idx / ((size_t)half_d * n_heads));
    const half2_t cs = *reinterpret_cast<const half2_t*>(rope_table + ((size_t)(start_pos + s) * half_d + pair) * 2);
    const float c = (float)cs[0], sn = (float)cs[1];
    const size_t in_off = (size_t)s * ld + (size_t)h * head_dim + 2 * pair;
    const half2_t qv = *reinterpret_cast<const half2_t*>(q + in_off);
    const half2_t kv = *reinterpret_cast<const half2_t*>(k + in_off);
    const half2_t vv = *reinterpret_cast<const half2_t*>(v + in_off);
    const half2_t qr = rope_rotate((float)qv[0], (float)qv[1], c, sn);
    const half2_t kr = rope_rotate((float)kv[0], (float)kv[1], c, sn);
    *reinterpret_cast<half2_t*>(q_out + ((size_t)h * n_tokens + s) * head_dim + 2 * pair) = qr;
    const size_t c_off = ((size_t)(start_pos + s) * n_heads + h) * head_dim + 2 * pair;
    *reinterpret_cast<half2_t*>(cache_k + c_off) = kr;
    *reinterpret_cast<half2_t*>(cache_v + c_off) = vv;
}

// prefill_rope_qkv_kernel and gather_vt_kernel in one pass for a fresh context (start_pos 0, so the new tokens are
// all there is to transpose): workgroup (64-token tile, head), 16-byte accesses throughout; the tile of v goes
// through LDS and leaves transposed, 128 contiguous bytes per head_dim row, zero beyond the last token.
// SLABS: the projection's K was split and its fp32 partial sums [splits][n_tokens][ld] have not been added up yet; q, k
// and v then only carry the column where their section starts (the column number times two as the pointer's value) and every value read is
// half(partial[0] + partial[1] + ...), the sum and rounding of splitk_reduce_kernel.
template <int D, bool SLABS>
__global__ void __launch_bounds__(256)
prefill_rope_qkv_vt_kernel(half_t* q_out, const half_t* q, const half_t* k, const half_t* v, size_t ld, half_t* cache_k,
                           half_t* cache_v, const half_t* rope_table, half_t* vT, int ldv, int n_tokens, int n_heads,
                           const float* slabs, int splits, size_t slab_elems) {
    auto load8 = [&](const half_t* base, size_t off) -> half8_t {
        if constexpr (SLABS) {
            const float* p = slabs + reinterpret_cast<uintptr_t>(base) / sizeof(half_t) + off;   // base: a column, not an address
            float4_t lo = *reinterpret_cast<const float4_t*>(p), hi = *reinterpret_cast<const float4_t*>(p + 4);
            for (int sp = 1; sp < splits; ++sp) {
                lo += *reinterpret_cast<const float4_t*>(p + (size_t)sp * slab_elems);
                hi += *reinterpret_cast<const float4_t*>(p + (size_t)sp * slab_elems + 4);
            }
            const half8_t r = {(half_t)lo[0], (half_t)lo[1], (half_t)lo[2], (half_t)lo[3],
                               (half_t)hi[0], (half_t)hi[1], (half_t)hi[2], (half_t)hi[3]};
            return r;
        } else {
            return *reinterpret_cast<const half8_t*>(base + off);
        }
    };
    constexpr int CH = D / 8;                     // 16-byte chunks per head row
    __shared__ __attribute__((aligned(16))) half_t vt_tile[64][D + 8];
    const int h = blockIdx.y;
    const int s0 = blockIdx.x * 64;
    // a grid three deep gives q, k and v a workgroup each (short prompts: three times the workgroups pull on the slabs)
    const bool do_q = gridDim.z == 1 || blockIdx.z == 0, do_k = gridDim.z == 1 || blockIdx.z == 1,
               do_v = gridDim.z == 1 || blockIdx.z == 2;
    const half8_t zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
    for (int it = threadIdx.x; it < 64 * CH; it += 256) {
        const int sl = it / CH, c = it % CH;
        const int s = s0 + sl;
        half8_t vv = zero8;
        if (s < n_tokens) {
            const size_t in_off = (size_t)s * ld + (size_t)h * D + c * 8;
            const size_t c_off = ((size_t)s * n_heads + h) * D + c * 8;
            half8_t cs = zero8;
            if (do_q || do_k) cs = *reinterpret_cast<const half8_t*>(rope_table + ((size_t)s * (D / 2) + c * 4) * 2);
            if (do_q)
                *reinterpret_cast<half8_t*>(q_out + ((size_t)h * n_tokens + s) * D + c * 8) = rope_chunk_cs(load8(q, in_off), cs);
            if (do_k) *reinterpret_cast<half8_t*>(cache_k + c_off) = rope_chunk_cs(load8(k, in_off), cs);
            if (do_v) {
                vv = load8(v, in_off);
                *reinterpret_cast<half8_t*>(cache_v + c_off) = vv;
            }
        }
        if (do_v) *reinterpret_cast<half8_t*>(&vt_tile[sl][c * 8]) = vv;
    }
    if (!do_v) return;
    __syncthreads();
    for (int it = threadIdx.x; it < D * 8; it += 256) {
        const int d = it / 8, j = it % 8;
        half8_t o;
#pragma unroll
        for (int i = 0; i < 8; ++i) o[i] = vt_tile[8 * j + i][d];
        *reinterpret_cast<half8_t*>(vT + ((size_t)h * D + d) * ldv + s0 + 8 * j) = o;
    }
}

// vT[h][d][t] = cache_v[t][h][d] for t < T, zero for T <= t < ldv: the value operand of the prefill attention,
// rows of `ldv` elements (a multiple of 8, so that groups of four positions can be read with 8-byte loads).
__global__ void __launch_bounds__(256)
gather_vt_kernel(half_t* vT, const half_t* cache_v, int T, int ldv, int n_heads, int head_dim) {
    __shared__ half_t tile[64][65];
    const int h = blockIdx.z;
    const int t0 = blockIdx.x * 64, d0 = blockIdx.y * 64;
    const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;  // 64 x 4
    for (int r = ty; r < 64; r += 4) {
        const int t = t0 + r, d = d0 + tx;
        tile[r][tx] = (t < T && d < head_dim) ? cache_v[((size_t)t * n_heads + h) * head_dim + d] : (half_t)0.f;
    }
    __syncthreads();
    for (int r = ty; r < 64; r += 4) {
        const int d = d0 + r, t = t0 + tx;
        if (d < head_dim && t < ldv) vT[((size_t)h * head_dim + d) * ldv + t] = tile[tx][r];
    }
}

// Scores of one block of 32 keys x 32 query rows -> probabilities, online-softmax state update.
// sacc[4g + r] of lane (lr, lh) is the fp32 score of key t0 + 8g + 4*lh + r against the lane's query row.
// Rounding follows the reference chain: score to fp16, fp16 quotient by half(sqrt(head_dim)) (the quotient
// is formed as x*r corrected by one fused Newton step, which rounds to the same fp16 value as the fp32
// division for every fp16 x and both supported divisors; exhaustively checked on the host), -inf above the
// diagonal (MASK: only blocks that reach the diagonal pay for it), exp in fp32, probability to fp16 (summed by attn_add_row_sums).
// The softmax is bound by vector-ALU instructions (1024 scores per 16 MFMAs), so the work per score is kept
// to conversions the hardware fuses into fma_mix, a packed-fp16 maximum, one fma + exp2 and the fp32 sum.
// The row maximum is finite from the first block on (key 0 is visible to every query), so exp2(-inf) = 0
// covers the first block without a guard.  Returns the factor by which the running output is to be rescaled
// (1 when the maximum did not move).
template <bool MASK>
__device__ __forceinline__ float attn_block_softmax(const float16_t& sacc, int t0, int lh, int limit, float dv,
                                                    float rdv, float& m, half8_t (&pf)[2]) {
    constexpr float kLog2e = 1.4426950408889634f;
    half_t sh[16];
#pragma unroll
    for (int e = 0; e < 16; ++e) {
        const half_t xh = (half_t)sacc[e];
        const float qv = (float)xh * rdv;
        sh[e] = (half_t)__builtin_fmaf(__builtin_fmaf(-qv, dv, (float)xh), rdv, qv);
        if constexpr (MASK) {
            const int kk = t0 + 8 * (e / 4) + 4 * lh + (e % 4);
            sh[e] = kk <= limit ? sh[e] : (half_t)-INFINITY;
        }
    }
    half2_t mx = {sh[0], sh[1]};
#pragma unroll
    for (int e = 2; e < 16; e += 2) {
        const half2_t t = {sh[e], sh[e + 1]};
        mx = __builtin_elementwise_max(mx, t);
    }
    float bm = (float)(mx[0] > mx[1] ? mx[0] : mx[1]);
    bm = fmaxf(bm, __shfl_xor(bm, 32, 64));
    const float m_new = fmaxf(m, bm);
    const float corr = __builtin_amdgcn_exp2f((m - m_new) * kLog2e);
    const float nm = -m_new * kLog2e;
#pragma unroll
    for (int e = 0; e < 16; ++e)      // MFMA step s = e / 8 holds g = 2s (slots 0..3) and g = 2s + 1 (slots 4..7)
        pf[e / 8][e % 8] = (half_t)__builtin_amdgcn_exp2f(__builtin_fmaf((float)sh[e], kLog2e, nm));
    m = m_new;
    return corr;
}

// Row sums of the fp16 probabilities of a block, added to the running sums: an MFMA whose A operand is all
// ones leaves sum_key P^T[key][q] in every row of column q, i.e. in element 0 of both lanes that own query
// row q (the matrix core is idle while the softmax runs; a vector-ALU sum costs 32 instructions and a lane
// exchange).  Only element 0 is kept meaningful: it alone is rescaled.
__device__ __forceinline__ void attn_add_row_sums(float16_t& lacc, const half8_t (&pf)[2], float corr, bool rescale) {
    const half8_t ones = {(half_t)1.f, (half_t)1.f, (half_t)1.f, (half_t)1.f, (half_t)1.f, (half_t)1.f, (half_t)1.f, (half_t)1.f};
    if (rescale) lacc[0] *= corr;
    lacc = __builtin_amdgcn_mfma_f32_32x32x16_f16(ones, pf[0], lacc, 0, 0, 0);
    lacc = __builtin_amdgcn_mfma_f32_32x32x16_f16(ones, pf[1], lacc, 0, 0, 0);
}

// Causal attention of n_tokens new tokens against cache positions [0, start_pos + n_tokens): one wavefront per
// (head, 32 query rows), no LDS, no score matrix in memory.  Per block of 32 keys:
//   S^T[key][q] = sum_d K[key][d] Q[q][d]        8 MFMAs, A = K rows straight from the cache, B = Q (registers)
//   lane l then holds 16 keys of ONE query row (l % 32): the row maximum is in-lane plus one exchange with
//   lane l ^ 32; scores are rounded like the reference chain (fp16 score, fp16 quotient by
//   half(sqrt(head_dim)), -inf above the diagonal); the row sums of the fp16 probabilities come from an MFMA
//   with an all-ones operand;
//   O^T[d][q] += sum_key vT[d][key] P^T[key][q]   A = vT with the key order the accumulator layout dictates
//   (lane half h of MFMA step s owns keys 16s+4h+{0..3} and 16s+8+4h+{0..3}: two 8-byte loads), B = P^T taken
//   from the score accumulators of the same lane without any shuffle.
// q: [n_heads, n_tokens, D] (rotated), out: [n_tokens, n_heads, D].
// One wavefront per workgroup: the kernel is bound by memory latency, so the (head, query block) units are
// spread over as many CUs as possible, the K rows of the next key block and the value fragments of the
// current one are requested before the score MFMAs of the current block start.
template <int D>
__global__ void __launch_bounds__(64)
prefill_attention_kernel(half_t* out, const half_t* q, const half_t* cache_k, const half_t* vT, int ldv, int start_pos,
                         int n_tokens, int n_heads, half_t divisor) {
    constexpr int KS = D / 16;    // MFMA steps over head_dim for Q.K
    constexpr int DB = D / 32;    // 32-row blocks of O^T
    const int lane = threadIdx.x & 63;
    const int h = blockIdx.y;
    const int qb = blockIdx.x;                      // block of 32 query rows
    const int q0 = qb * 32;
    if (q0 >= n_tokens) return;
    const int T = start_pos + n_tokens;
    const int lr = lane & 31, lh = lane >> 5;
    const int my_q = q0 + lr;                       // the query row this lane owns in S^T / O^T
    const int my_q_c = my_q < n_tokens ? my_q : n_tokens - 1;
    const int limit = start_pos + my_q;             // last visible key
    const float dv = (float)divisor, rdv = 1.0f / dv;

    half8_t qf[KS];
    const half_t* qrow = q + ((size_t)h * n_tokens + my_q_c) * D + lh * 8;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) qf[ks] = *reinterpret_cast<const half8_t*>(qrow + ks * 16);

    float16_t o[DB];
#pragma unroll
    for (int b = 0; b < DB; ++b)
#pragma unroll
        for (int e = 0; e < 16; ++e) o[b][e] = 0.f;
    float m = -INFINITY;
    float16_t lacc;
#pragma unroll
    for (int e = 0; e < 16; ++e) lacc[e] = 0.f;

    const int last_key = start_pos + (q0 + 31 < n_tokens ? q0 + 31 : n_tokens - 1);  // of the whole wavefront
    const size_t krow_stride = (size_t)n_heads * D;
    auto load_k = [&](half8_t (&dst)[KS], int t0) {
        int key = t0 + lr;
        key = key < T ? key : T - 1;
        const half_t* krow = cache_k + (size_t)key * krow_stride + (size_t)h * D + lh * 8;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) dst[ks] = *reinterpret_cast<const half8_t*>(krow + ks * 16);
    };
    half8_t kf[KS], kn[KS];
    load_k(kf, 0);
    for (int t0 = 0; t0 <= last_key; t0 += 32) {
        // requests for the next block's K rows and this block's value fragments go out first
        if (t0 + 32 <= last_key) load_k(kn, t0 + 32);
        half4_t vraw[DB][2][2];
#pragma unroll
        for (int b = 0; b < DB; ++b) {
            const half_t* vrow = vT + ((size_t)h * D + b * 32 + lr) * ldv + t0 + 4 * lh;
#pragma unroll
            for (int st = 0; st < 2; ++st) {
                vraw[b][st][0] = *reinterpret_cast<const half4_t*>(vrow + 16 * st);
                vraw[b][st][1] = *reinterpret_cast<const half4_t*>(vrow + 16 * st + 8);
            }
        }
        // ---- S^T block ----
        float16_t sacc;
#pragma unroll
        for (int e = 0; e < 16; ++e) sacc[e] = 0.f;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) sacc = __builtin_amdgcn_mfma_f32_32x32x16_f16(kf[ks], qf[ks], sacc, 0, 0, 0);
        half8_t pf[2];
        const float corr = t0 + 31 > start_pos + q0 ? attn_block_softmax<true>(sacc, t0, lh, limit, dv, rdv, m, pf)
                                                    : attn_block_softmax<false>(sacc, t0, lh, limit, dv, rdv, m, pf);
        const bool rescale = __builtin_amdgcn_ballot_w64(corr != 1.0f) != 0;
        attn_add_row_sums(lacc, pf, corr, rescale);
        // ---- O^T += vT . P^T ----
#pragma unroll
        for (int b = 0; b < DB; ++b) {
            if (rescale) {
#pragma unroll
                for (int e = 0; e < 16; ++e) o[b][e] *= corr;
            }
#pragma unroll
            for (int st = 0; st < 2; ++st) {
                const half4_t v0 = vraw[b][st][0], v1 = vraw[b][st][1];
                const half8_t vf = {v0[0], v0[1], v0[2], v0[3], v1[0], v1[1], v1[2], v1[3]};
                o[b] = __builtin_amdgcn_mfma_f32_32x32x16_f16(vf, pf[st], o[b], 0, 0, 0);
            }
        }
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) kf[ks] = kn[ks];
    }
    if (my_q >= n_tokens) return;
    const float inv = 1.0f / lacc[0];
    half_t* orow = out + ((size_t)my_q * n_heads + h) * D;
#pragma unroll
    for (int b = 0; b < DB; ++b)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            half4_t r = {(half_t)(o[b][4 * g] * inv), (half_t)(o[b][4 * g + 1] * inv), (half_t)(o[b][4 * g + 2] * inv),
                         (half_t)(o[b][4 * g + 3] * inv)};
            *reinterpret_cast<half4_t*>(orow + b * 32 + 8 * g + 4 * lh) = r;
        }
}

// The same attention for long prompts: a workgroup of four wavefronts owns 128 query rows of one head and
// walks the keys in tiles of 64, K rows and vT rows of a tile staged once in LDS (direct global->LDS loads, two
// stages) and read from there by all four wavefronts.  Per wavefront and block of 32 keys the arithmetic and
// its order are exactly those of prefill_attention_kernel (results are bit-identical); what changes is the
// traffic: that kernel re-reads a head's K and V for every 32 query rows (1.1 GB per layer at 2048 tokens),
// this one for every 128.  LDS layout, 16-byte chunks swizzled so that the 16 rows one ds_read phase touches
// fall into different banks: K tile [64 keys][256 B], chunk c of row r at slot c ^ (r % 16); vT tile
// [128 d][128 B], chunk c of row r at slot c ^ ((r / 2) % 8).  Needs vT rows that cover the context rounded up
// to 64.
// Registers are capped for two workgroups per CU (each hides the other's barriers and softmax); the cap also gave
// the faster code when only one is resident.
template <int D, bool PAIRED>
__global__ void __launch_bounds__(256, 2)
prefill_attention_tiled_kernel(half_t* out, const half_t* q, const half_t* cache_k, const half_t* vT, int ldv,
                               int start_pos, int n_tokens, int n_heads, half_t divisor, int slots) {
    static_assert(D == 128, "tile layout is written for head_dim 128");
    constexpr int KS = D / 16, DB = D / 32, TK = 64, NWQ = 4;
    constexpr int K_BYTES = TK * D * 2, V_BYTES = D * TK * 2, STAGE_BYTES = K_BYTES + V_BYTES;
    constexpr int K_LOADS = K_BYTES / 1024 / NWQ, V_LOADS = V_BYTES / 1024 / NWQ;   // wavefront-loads per wavefront
    extern __shared__ __attribute__((aligned(1024))) unsigned char smem_raw[];
    typedef __attribute__((address_space(3))) unsigned char lds_byte_t;
    lds_byte_t* lds = (lds_byte_t*)smem_raw;

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    // One-dimensional grid of n_heads * slots workgroups (slots = query-group slots per head); ids congruent mod 8
    // run on the same XCD, so XCD x takes a contiguous run of (head, slot) pairs and the workgroups that read one
    // head's K and V share an L2.
    const int nwg = (int)gridDim.x;
    const int bid = (int)blockIdx.x;
    const int xcd = bid & 7, per = nwg >> 3, rem = nwg & 7;
    const int lid = xcd * per + (xcd < rem ? xcd : rem) + (bid >> 3);
    const int h = lid / slots;
    const int slot = lid % slots;
    const int T = start_pos + n_tokens;
    const int lr = lane & 31, lh = lane >> 5;
    const float dv = (float)divisor, rdv = 1.0f / dv;

    // loader: K wavefront-load u covers tile rows 4u..4u+3, vT wavefront-load u covers d rows 8u..8u+7
    const size_t krow_stride = (size_t)n_heads * D;
    int k_row[K_LOADS], k_chunk[K_LOADS];
    const half_t* v_src[V_LOADS];
#pragma unroll
    for (int j = 0; j < K_LOADS; ++j) {
        const int u = j * NWQ + wave;
        k_row[j] = 4 * u + lane / 16;
        k_chunk[j] = (lane % 16) ^ (k_row[j] % 16);
    }
#pragma unroll
    for (int j = 0; j < V_LOADS; ++j) {
        const int u = j * NWQ + wave;
        const int r = 8 * u + lane / 8;
        const int c = (lane % 8) ^ ((r / 2) % 8);
        v_src[j] = vT + ((size_t)h * D + r) * ldv + c * 8;
    }
    auto issue = [&](int tile, int stage) {
        const int t0 = tile * TK;
        lds_byte_t* base = lds + stage * STAGE_BYTES;
#pragma unroll
        for (int j = 0; j < K_LOADS; ++j) {
            int key = t0 + k_row[j];
            key = key < T ? key : T - 1;
            load_16B_per_lane_to_lds(cache_k + (size_t)key * krow_stride + (size_t)h * D + k_chunk[j] * 8,
                                     base + (j * NWQ + wave) * 1024);
        }
#pragma unroll
        for (int j = 0; j < V_LOADS; ++j)
            load_16B_per_lane_to_lds(v_src[j] + t0, base + K_BYTES + (j * NWQ + wave) * 1024);
    };

    // Query groups are issued longest first.  With more groups than the chip holds at once (PAIRED) a workgroup
    // takes two of them, the longest with the shortest, so that every workgroup walks the same number of key
    // tiles and the kernel does not end on a few long walks.
    const int n_groups = (n_tokens + 32 * NWQ - 1) / (32 * NWQ);
    for (int job = 0; job < 2; ++job) {
        const int group = job == 0 ? n_groups - 1 - slot : slot;
        if (job == 1) {
            if (!PAIRED || group >= n_groups - 1 - slot) break;   // odd count: the middle group has no partner
            asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");   // the stages are free again
        }
        const int qg0 = group * (32 * NWQ);                                    // first query row of the group
        const int q0 = qg0 + 32 * wave;                                       // of this wavefront
        const int wg_last_key = start_pos + (qg0 + 32 * NWQ - 1 < n_tokens ? qg0 + 32 * NWQ - 1 : n_tokens - 1);
        const int ntiles = wg_last_key / TK + 1;
        const bool active = q0 < n_tokens;
        const int my_q = q0 + lr;
        const int my_q_c = my_q < n_tokens ? my_q : n_tokens - 1;
        const int limit = start_pos + my_q;
        const int last_key = start_pos + (q0 + 31 < n_tokens ? q0 + 31 : n_tokens - 1);

        half8_t qf[KS];
        const half_t* qrow = q + ((size_t)h * n_tokens + my_q_c) * D + lh * 8;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) qf[ks] = *reinterpret_cast<const half8_t*>(qrow + ks * 16);

        float16_t o[DB];
#pragma unroll
        for (int b = 0; b < DB; ++b)
#pragma unroll
            for (int e = 0; e < 16; ++e) o[b][e] = 0.f;
        float m = -INFINITY;
        float16_t lacc;
#pragma unroll
        for (int e = 0; e < 16; ++e) lacc[e] = 0.f;

        issue(0, 0);
        if (ntiles > 1) issue(1, 1);
        for (int i = 0; i < ntiles; ++i) {
            if (i + 1 < ntiles) wait_vmcnt_and_barrier<K_LOADS + V_LOADS>();
            else wait_vmcnt_and_barrier<0>();
            const unsigned char* kt = smem_raw + (i & 1) * STAGE_BYTES;
            const unsigned char* vt = kt + K_BYTES;
            if (active && i * TK <= last_key) {
                // scores of a block: one MFMA per 16 values of head_dim, K fragments read from the swizzled tile
                auto score_step = [&](float16_t& sacc, int kb, int ks) {
                    const int kr = 32 * kb + lr;
                    const half8_t kf = *reinterpret_cast<const half8_t*>(kt + kr * (D * 2) + (((2 * ks + lh) ^ (kr % 16)) * 16));
                    sacc = __builtin_amdgcn_mfma_f32_32x32x16_f16(kf, qf[ks], sacc, 0, 0, 0);
                };
                auto finish_block = [&](const float16_t& sacc, int kb) {
                    const int t0 = i * TK + 32 * kb;
                    half8_t pf[2];
                    const float corr = t0 + 31 > start_pos + q0 ? attn_block_softmax<true>(sacc, t0, lh, limit, dv, rdv, m, pf)
                                                                : attn_block_softmax<false>(sacc, t0, lh, limit, dv, rdv, m, pf);
                    const bool rescale = __builtin_amdgcn_ballot_w64(corr != 1.0f) != 0;
                    attn_add_row_sums(lacc, pf, corr, rescale);
                    // ---- O^T += vT . P^T ----
#pragma unroll
                    for (int b = 0; b < DB; ++b) {
                        if (rescale) {
#pragma unroll
                            for (int e = 0; e < 16; ++e) o[b][e] *= corr;
                        }
                        const int vr = 32 * b + lr;
                        const unsigned char* vrow = vt + vr * (TK * 2) + 8 * lh;
                        const int sw = (vr / 2) % 8;
#pragma unroll
                        for (int st = 0; st < 2; ++st) {
                            const int c0 = 4 * kb + 2 * st;
                            const half4_t v0 = *reinterpret_cast<const half4_t*>(vrow + ((c0 ^ sw) * 16));
                            const half4_t v1 = *reinterpret_cast<const half4_t*>(vrow + (((c0 + 1) ^ sw) * 16));
                            const half8_t vf = {v0[0], v0[1], v0[2], v0[3], v1[0], v1[1], v1[2], v1[3]};
                            o[b] = __builtin_amdgcn_mfma_f32_32x32x16_f16(vf, pf[st], o[b], 0, 0, 0);
                        }
                    }
                };
#pragma unroll
                for (int kb = 0; kb < TK / 32; ++kb) {
                    if (i * TK + 32 * kb > last_key) break;
                    float16_t sacc;
#pragma unroll
                    for (int e = 0; e < 16; ++e) sacc[e] = 0.f;
#pragma unroll
                    for (int ks = 0; ks < KS; ++ks) score_step(sacc, kb, ks);
                    finish_block(sacc, kb);
                }
            }
            if (i + 2 < ntiles) {
                // everyone is done reading this stage before the tile after next lands in it
                asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
                issue(i + 2, i & 1);
            }
        }
        if (active && my_q < n_tokens) {
            const float inv = 1.0f / lacc[0];
            half_t* orow = out + ((size_t)my_q * n_heads + h) * D;
#pragma unroll
            for (int b = 0; b < DB; ++b)
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    half4_t r = {(half_t)(o[b][4 * g] * inv), (half_t)(o[b][4 * g + 1] * inv), (half_t)(o[b][4 * g + 2] * inv),
                                 (half_t)(o[b][4 * g + 3] * inv)};
                    *reinterpret_cast<half4_t*>(orow + b * 32 + 8 * g + 4 * lh) = r;
                }
        }
    }
}

// Decode-step glue after the fused q|k|v GEMV: rotate q in place, rotate k and write it to
// cache_k[pos], copy v to cache_v[pos].  One thread per (even, odd) pair of the 3*dim vector.
__global__ void __launch_bounds__(256)
rope_qk_store_kv_kernel(half_t* qkv, half_t* cache_k, half_t* cache_v, int pos, int n_heads, int head_dim) {
    const int dim = n_heads * head_dim;
    const int p = blockIdx.x * blockDim.x + threadIdx.x;  // pair index in [0, 3*dim/2)
    if (p >= 3 * dim / 2) return;
    const int which = p / (dim / 2);                       // 0 q, 1 k, 2 v
    const int e = (p % (dim / 2)) * 2;                     // element index within the dim vector
    half2_t v = *reinterpret_cast<const half2_t*>(qkv + which * dim + e);
    if (which < 2) {
        const int d = e % head_dim;
        float c, s;
        rope_cos_sin(pos, d, head_dim, c, s);
        v = rope_rotate((float)v[0], (float)v[1], c, s);
    }
    if (which == 0)
        *reinterpret_cast<half2_t*>(qkv + e) = v;
    else if (which == 1)
        *reinterpret_cast<half2_t*>(cache_k + (size_t)pos * dim + e) = v;
    else
        *reinterpret_cast<half2_t*>(cache_v + (size_t)pos * dim + e) = v;
}

// sum = a + b (one rounding, like the reference's EwiseAdd) and norm = rmsnorm(sum) * w in
// one pass per token: the residual add of one sub-block and the RMSNorm that opens the next.
__global__ void __launch_bounds__(256)
add_rms_norm_kernel(half_t* sum_out, half_t* norm_out, const half_t* a, const half_t* b, const half_t* w, float eps,
                    int hidden) {
    __shared__ float red[4];
    const size_t base = (size_t)blockIdx.x * hidden;
    float ss = 0.f;
    for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
        const half_t s = (half_t)((float)a[base + i] + (float)b[base + i]);
        sum_out[base + i] = s;
        ss = __builtin_fmaf((float)s, (float)s, ss);
    }
    // wavefront then workgroup reduction
    ss += dppf<0xB1>(ss);
    ss += dppf<0x4E>(ss);
    ss += dppf<0x141>(ss);
    ss += dppf<0x140>(ss);
    ss += __shfl_xor(ss, 16, 64);
    ss += __shfl_xor(ss, 32, 64);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = ss;
    __syncthreads();
    const float total = (red[0] + red[1]) + (red[2] + red[3]);
    const float r = 1.0f / sqrtf(total / (float)hidden + eps);
    // every thread re-reads the elements it wrote itself
    for (int i = threadIdx.x; i < hidden; i += blockDim.x)
        norm_out[base + i] = (half_t)((float)sum_out[base + i] * r * (float)w[i]);
}

// Same operation with every element held in registers between the two phases: one 16-byte load of
// a, b and w per chunk, one global round trip in total.  512 threads, CPT chunks of 8 halves each.
// SLABS: b is not in memory yet: it is the result of a split-K GEMM whose fp32 slabs [splits][tokens][hidden] are
// added here in split order and rounded to fp16, exactly what the GEMM's own second pass would have stored.
template <int CPT, bool SLABS = false>
__global__ void __launch_bounds__(512)
add_rms_norm_vec_kernel(half_t* sum_out, half_t* norm_out, const half_t* a, const half_t* b, const half_t* w, float eps,
                        int hidden, const float* slabs, int splits, size_t slab_stride) {
    __shared__ float red[8];
    const size_t base = (size_t)blockIdx.x * hidden;
    const int chunks = hidden / 8;
    half8_t va[CPT], vb[CPT], vw[CPT];
    const half8_t zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
    for (int j = 0; j < CPT; ++j) {
        const int c = threadIdx.x + j * 512;
        const bool ok = c < chunks;
        va[j] = ok ? reinterpret_cast<const half8_t*>(a + base)[c] : zero8;
        if constexpr (SLABS) {
            vb[j] = zero8;
            if (ok) {
                const float4_t* p = reinterpret_cast<const float4_t*>(slabs + base) + 2 * c;
                float4_t lo = p[0], hi = p[1];
                for (int sp = 1; sp < splits; ++sp) {
                    const float4_t* q = reinterpret_cast<const float4_t*>(slabs + (size_t)sp * slab_stride + base) + 2 * c;
                    lo += q[0];
                    hi += q[1];
                }
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    vb[j][i] = (half_t)lo[i];
                    vb[j][4 + i] = (half_t)hi[i];
                }
            }
        } else {
            vb[j] = ok ? reinterpret_cast<const half8_t*>(b + base)[c] : zero8;
        }
        vw[j] = ok ? reinterpret_cast<const half8_t*>(w)[c] : zero8;
    }
    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < CPT; ++j)
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const half_t s = (half_t)((float)va[j][i] + (float)vb[j][i]);
            va[j][i] = s;
            ss = __builtin_fmaf((float)s, (float)s, ss);
        }
    ss += dppf<0xB1>(ss);
    ss += dppf<0x4E>(ss);
    ss += dppf<0x141>(ss);
    ss += dppf<0x140>(ss);
    ss += __shfl_xor(ss, 16, 64);
    ss += __shfl_xor(ss, 32, 64);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = ss;
    __syncthreads();
    float total = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) total += red[i];
    const float r = 1.0f / sqrtf(total / (float)hidden + eps);
#pragma unroll
    for (int j = 0; j < CPT; ++j) {
        const int c = threadIdx.x + j * 512;
        if (c < chunks) {
            half8_t n;
#pragma unroll
            for (int i = 0; i < 8; ++i) n[i] = (half_t)((float)va[j][i] * r * (float)vw[j][i]);
            reinterpret_cast<half8_t*>(sum_out + base)[c] = va[j];
            reinterpret_cast<half8_t*>(norm_out + base)[c] = n;
        }
    }
}

// Cached positions per workgroup of the decode attention.  Every launch boundary in a decode step costs about 3 us and
// merging chunk partials another 2-2.5 us, so a context that one workgroup per head can hold in registers is not cut:
// up to 128 positions one chunk of 128 (4.0-4.7 us against 5.5-5.8 us for two chunks of 64 merged in the kernel), up
// to 192 one chunk of 256 (4.9-5.6 against 5.6-5.8 us).  Beyond that a single workgroup per head is bound by what one
// CU takes in (256 positions: 6.2 us) and chunks of 64 over many CUs win again; from 1280 positions on chunks of 128
// halve the partials the second launch merges (2048 positions: 10.0 against 11.5 us).  Times: one attention launch
// between dependent 4096x4096 GEMVs, 32 heads of 128.
static int decode_attention_chunk(int T, int head_dim) {
    (void)head_dim;
    if (T <= 64) return 64;
    if (T <= 128) return 128;
    if (T <= 192) return 256;
    return T < 1280 ? 64 : 128;
}

// Library-owned fp32 workspace for the chunk partials, grown on demand.
static Workspace g_partials;

}  // namespace tl

// Chunk partials of tl_decode_attention_rope_static_f16, the entry point that allocates nothing: the memory is part
// of the code object, so every GPU the library runs on holds its own copy from load time until the process ends.
// `scratch` is a host-side stand-in for the symbol, not a device address: host code only ever passes the pointer
// hipGetSymbolAddress returned for the current device.
static __device__ __align__(256) float scratch[TL_DECODE_ATTENTION_STATIC_SCRATCH_FLOATS];

namespace tl {

constexpr int kMaxDevices = 64;
static std::mutex g_scratch_mu;
static float* g_scratch_ptr[kMaxDevices] = {nullptr};   // device address of `scratch`, per device ordinal

// Resolves the current device's copy of `scratch` (once per device; called from the library's init and, for a
// device the library was not initialised on, from the entry point's first call there).
int attention_static_scratch(float** out) {
    int dev = -1;
    TL_HIP_TRY(hipGetDevice(&dev));
    TL_REQUIRE(dev >= 0 && dev < kMaxDevices, "static attention scratch: device ordinal %d not supported", dev);
    std::lock_guard<std::mutex> lk(g_scratch_mu);
    if (!g_scratch_ptr[dev]) {
        float* p = nullptr;
        TL_HIP_TRY(hipGetSymbolAddress((void**)&p, HIP_SYMBOL(scratch)));
        TL_REQUIRE(p != nullptr, "static attention scratch: hipGetSymbolAddress returned a null address");
        g_scratch_ptr[dev] = p;
    }
    if (out) *out = g_scratch_ptr[dev];
    return TL_OK;
}

// Puts the ticket words of both scratch buffers back to zero (after a launch that did not complete).
int attention_reset_tickets() {
    int rc = g_partials.zero_head(kAttnTicketWords);
    if (rc != TL_OK) return rc;
    float* st = nullptr;
    rc = attention_static_scratch(&st);
    if (rc != TL_OK) return rc;
    return launch_fill_f16(st, 0, kAttnTicketWords * 2);
}

}  // namespace tl

extern "C" {

// static_ws: null = partials go to the library's grown-on-demand workspace; else the caller's buffer of
// static_ws_floats floats (no allocation on this path).
static int launch_decode_attention(void* out, const void* q, void* cache_k, void* cache_v, const void* rope_table,
                                   int T, int n_heads, int head_dim, bool fuse_rope, const char* name,
                                   float* static_ws = nullptr, size_t static_ws_floats = 0) {
    TL_ENSURE_INIT();
    TL_REQUIRE(out && q && cache_k && cache_v, "%s: null pointer", name);
    TL_REQUIRE(T >= 1 && n_heads >= 1, "%s: bad sizes T=%d n_heads=%d", name, T, n_heads);
    TL_REQUIRE(head_dim == 64 || head_dim == 128 || head_dim == 256, "%s: head_dim %d not supported (64, 128 or 256)",
               name, head_dim);
    TL_REQUIRE(tl::aligned16(q) && tl::aligned16(cache_k) && tl::aligned16(cache_v),
               "%s: q and the caches must be 16-byte aligned", name);
    TL_REQUIRE(n_heads <= 65535, "%s: too many heads", name);
    int chunk = tl::g_decode_chunk.load();
    if (chunk == 0) chunk = tl::decode_attention_chunk(T, head_dim);
    if (head_dim == 256) chunk = tl::kAttnChunk;   // 32 rows of K and V per thread do not fit the registers
    const int n_chunks = (T + chunk - 1) / chunk;
    TL_REQUIRE(n_chunks <= 65535, "%s: T=%d too long", name, T);
    tl::Workspace::Lease lease;   // held until both kernels are enqueued
    // [kAttnTicketWords ticket words, one per head][partials]; tickets are zero between calls.  The ticket region has
    // one size for every call, so partials of one call never land where another call keeps tickets.
    const size_t ticket_words = tl::kAttnTicketWords;
    const size_t ws_floats = ticket_words + (size_t)n_heads * n_chunks * (head_dim + 2);
    float* ws = static_ws;
    if (static_ws) {
        TL_REQUIRE(ws_floats <= static_ws_floats,
                   "%s: %d heads x %d chunks of %d positions x (%d + 2) floats (+ tickets) = %zu floats of partial results exceed the "
                   "static scratch of %zu floats; use tl_decode_attention_rope_f16 for this size",
                   name, n_heads, n_chunks, chunk, head_dim, ws_floats, static_ws_floats);
    } else if (n_chunks > 1) {
        int rc = tl::g_partials.acquire(ws_floats, (size_t)1 << 20, "attention workspace", &lease);
        if (rc != TL_OK) return rc;
        ws = lease.ptr;
    }
    const int merge_mode = tl::g_decode_merge_mode.load();
    // more heads than ticket words: the second kernel merges
    const bool in_kernel = (size_t)n_heads <= ticket_words &&
                           (merge_mode == 1 || merge_mode == 3 || (merge_mode == 0 && n_chunks <= tl::kMergeInKernelMaxChunks));
    unsigned* tickets = (ws && in_kernel) ? reinterpret_cast<unsigned*>(ws) : nullptr;
    float* partials = ws ? ws + ticket_words : nullptr;
    // the reference divides the scores by half(sqrt(head_dim)) (Transformer.cpp:94)
    const float scale = (float)(tl::half_t)sqrtf((float)head_dim);
    const float inv_scale = 1.0f / scale;
    dim3 grid(n_heads, n_chunks);
    hipStream_t st = tl::stream();
    auto launch = [&](auto kernel) {
        hipLaunchKernelGGL(kernel, grid, dim3(tl::kAttnThreads), 0, st, (tl::half_t*)out, partials,
                           (const tl::half_t*)q, (tl::half_t*)cache_k, (tl::half_t*)cache_v,
                           (const tl::half_t*)rope_table, T, n_heads, inv_scale, n_chunks, tickets, merge_mode == 3 ? 1 : 0);
    };
    const int rope = fuse_rope ? (rope_table ? 1 : 2) : 0;
    auto launch_chunk = [&](auto lpr, auto rp) {
        constexpr int LPR = decltype(lpr)::value, RP = decltype(rp)::value;
        if constexpr (LPR == 32) {
            launch(tl::decode_attn_partial_kernel<LPR, RP, 64>);
        } else {
            if (chunk == 64) launch(tl::decode_attn_partial_kernel<LPR, RP, 64>);
            else if (chunk == 128) launch(tl::decode_attn_partial_kernel<LPR, RP, 128>);
            else launch(tl::decode_attn_partial_kernel<LPR, RP, 256>);
        }
    };
    auto launch_rope = [&](auto lpr) {
        if (rope == 0) launch_chunk(lpr, std::integral_constant<int, 0>{});
        else if (rope == 1) launch_chunk(lpr, std::integral_constant<int, 1>{});
        else launch_chunk(lpr, std::integral_constant<int, 2>{});
    };
    if (head_dim == 64) launch_rope(std::integral_constant<int, 8>{});
    else if (head_dim == 128) launch_rope(std::integral_constant<int, 16>{});
    else launch_rope(std::integral_constant<int, 32>{});
    TL_CHECK_LAUNCH("decode_attn_partial_kernel");
    if (n_chunks > 1 && !tickets) {
        hipLaunchKernelGGL(tl::decode_attn_merge_kernel, dim3(n_heads), dim3(256), 0, st, (tl::half_t*)out, partials, head_dim,
                           n_chunks);
        TL_CHECK_LAUNCH("decode_attn_merge_kernel");
    }
    return TL_OK;
}

int tl_decode_attention_f16(void* out, const void* q, const void* cache_k, const void* cache_v, int T, int n_heads,
                            int head_dim) {
    return launch_decode_attention(out, q, const_cast<void*>(cache_k), const_cast<void*>(cache_v), nullptr, T, n_heads,
                                   head_dim, false, "tl_decode_attention_f16");
}

int tl_decode_attention_rope_f16(void* out, const void* qkv, void* cache_k, void* cache_v, const void* rope_table,
                                 int pos, int n_heads, int head_dim) {
    TL_REQUIRE(pos >= 0, "tl_decode_attention_rope_f16: negative position");
    TL_REQUIRE(rope_table == nullptr || tl::aligned16(rope_table), "tl_decode_attention_rope_f16: misaligned table");
    return launch_decode_attention(out, qkv, cache_k, cache_v, rope_table, pos + 1, n_heads, head_dim, true,
                                   "tl_decode_attention_rope_f16");
}

int tl_decode_attention_rope_static_f16(void* out, const void* qkv, void* cache_k, void* cache_v, const void* rope_table,
                                        int pos, int n_heads, int head_dim) {
    TL_ENSURE_INIT();
    TL_REQUIRE(pos >= 0, "tl_decode_attention_rope_static_f16: negative position");
    TL_REQUIRE(rope_table == nullptr || tl::aligned16(rope_table), "tl_decode_attention_rope_static_f16: misaligned table");
    float* ws = nullptr;
    int rc = tl::attention_static_scratch(&ws);   // a table lookup after the first call on a device
    if (rc != TL_OK) return rc;
    return launch_decode_attention(out, qkv, cache_k, cache_v, rope_table, pos + 1, n_heads, head_dim, true,
                                   "tl_decode_attention_rope_static_f16", ws,
                                   (size_t)TL_DECODE_ATTENTION_STATIC_SCRATCH_FLOATS);
}

int tl_set_decode_attention_chunk(int positions) {
    TL_REQUIRE(positions == 0 || positions == 64 || positions == 128 || positions == 256,
               "tl_set_decode_attention_chunk: %d is not 0, 64, 128 or 256", positions);
    tl::g_decode_chunk = positions;
    return TL_OK;
}

int tl_rope_table_f16(void* table, int max_seq, int head_dim) {
    TL_ENSURE_INIT();
    TL_REQUIRE(table, "tl_rope_table_f16: null pointer");
    TL_REQUIRE(max_seq >= 1 && head_dim >= 2 && head_dim % 2 == 0, "tl_rope_table_f16: bad sizes");
    const size_t n = (size_t)max_seq * (head_dim / 2);
    hipLaunchKernelGGL(tl::rope_table_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, tl::stream(),
                       (tl::half_t*)table, max_seq, head_dim);
    TL_CHECK_LAUNCH("rope_table_kernel");
    return TL_OK;
}

int tl_prefill_rope_qkv_f16(void* q_out, const void* q, const void* k, const void* v, size_t row_stride, void* cache_k,
                            void* cache_v, const void* rope_table, int start_pos, int n_tokens, int n_heads,
                            int head_dim) {
    TL_ENSURE_INIT();
    TL_REQUIRE(q_out && q && k && v && cache_k && cache_v && rope_table, "tl_prefill_rope_qkv_f16: null pointer");
    TL_REQUIRE(start_pos >= 0 && n_tokens >= 0 && n_heads >= 1 && head_dim >= 2 && head_dim % 2 == 0,
               "tl_prefill_rope_qkv_f16: bad sizes");
    TL_REQUIRE(row_stride % 2 == 0 && row_stride >= (size_t)n_heads * head_dim,
               "tl_prefill_rope_qkv_f16: row stride %zu too small or odd", row_stride);
    auto al4 = [](const void* p) { return ((uintptr_t)p & 3) == 0; };
    TL_REQUIRE(al4(q_out) && al4(q) && al4(k) && al4(v) && al4(cache_k) && al4(cache_v) && al4(rope_table),
               "tl_prefill_rope_qkv_f16: pointers must be 4-byte aligned");
    const size_t total = (size_t)n_tokens * n_heads * (head_dim / 2);
    if (total == 0) return TL_OK;
    TL_REQUIRE((total + 255) / 256 <= 0x7fffffffu, "tl_prefill_rope_qkv_f16: too many elements");
    hipLaunchKernelGGL(tl::prefill_rope_qkv_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, tl::stream(),
                       (tl::half_t*)q_out, (const tl::half_t*)q, (const tl::half_t*)k, (const tl::half_t*)v, row_stride,
                       (tl::half_t*)cache_k, (tl::half_t*)cache_v, (const tl::half_t*)rope_table, start_pos, n_tokens,
                       n_heads, head_dim);
    TL_CHECK_LAUNCH("prefill_rope_qkv_kernel");
    return TL_OK;
}

int tl_prefill_rope_qkv_vt_f16(void* q_out, const void* q, const void* k, const void* v, size_t row_stride, void* cache_k,
                               void* cache_v, const void* rope_table, void* vT, int ldv, int n_tokens, int n_heads,
                               int head_dim) {
    TL_ENSURE_INIT();
    TL_REQUIRE(q_out && q && k && v && cache_k && cache_v && rope_table && vT, "tl_prefill_rope_qkv_vt_f16: null pointer");
    TL_REQUIRE(n_tokens >= 1 && n_heads >= 1 && n_heads <= 65535, "tl_prefill_rope_qkv_vt_f16: bad sizes");
    TL_REQUIRE(head_dim == 64 || head_dim == 128, "tl_prefill_rope_qkv_vt_f16: head_dim %d not supported (64 or 128)", head_dim);
    TL_REQUIRE(ldv % 64 == 0 && ldv >= n_tokens, "tl_prefill_rope_qkv_vt_f16: ldv=%d must be a multiple of 64 that covers the tokens", ldv);
    TL_REQUIRE(row_stride % 8 == 0 && row_stride >= (size_t)n_heads * head_dim,
               "tl_prefill_rope_qkv_vt_f16: row stride %zu too small or not a multiple of 8", row_stride);
    TL_REQUIRE(tl::aligned16(q_out) && tl::aligned16(q) && tl::aligned16(k) && tl::aligned16(v) && tl::aligned16(cache_k) &&
                   tl::aligned16(cache_v) && tl::aligned16(rope_table) && tl::aligned16(vT),
               "tl_prefill_rope_qkv_vt_f16: pointers must be 16-byte aligned");
    dim3 grid((unsigned)(ldv / 64), (unsigned)n_heads);
    auto launch = [&](auto kernel) {
        hipLaunchKernelGGL(kernel, grid, dim3(256), 0, tl::stream(), (tl::half_t*)q_out, (const tl::half_t*)q,
                           (const tl::half_t*)k, (const tl::half_t*)v, row_stride, (tl::half_t*)cache_k, (tl::half_t*)cache_v,
                           (const tl::half_t*)rope_table, (tl::half_t*)vT, ldv, n_tokens, n_heads, (const float*)nullptr, 1,
                           (size_t)0);
    };
    if (head_dim == 64) launch(tl::prefill_rope_qkv_vt_kernel<64, false>);
    else launch(tl::prefill_rope_qkv_vt_kernel<128, false>);
    TL_CHECK_LAUNCH("prefill_rope_qkv_vt_kernel");
    return TL_OK;
}

int tl_hgemm_prefill_rope_qkv_vt_f16(const void* X, const void* Wqkv, void* qkv, void* q_out, void* cache_k, void* cache_v,
                                     const void* rope_table, void* vT, int ldv, int n_tokens, int n_heads, int head_dim,
                                     size_t K) {
    TL_ENSURE_INIT();
    // every argument of both steps is checked before the first launch: a rejected call has written nothing
    TL_REQUIRE(X && Wqkv && qkv && q_out && cache_k && cache_v && rope_table && vT, "tl_hgemm_prefill_rope_qkv_vt_f16: null pointer");
    TL_REQUIRE(n_tokens >= 1 && n_heads >= 1 && (head_dim == 64 || head_dim == 128),
               "tl_hgemm_prefill_rope_qkv_vt_f16: bad sizes");
    TL_REQUIRE(n_heads <= 65535 && ldv % 64 == 0 && ldv >= n_tokens,
               "tl_hgemm_prefill_rope_qkv_vt_f16: ldv=%d must be a multiple of 64 that covers the tokens", ldv);
    TL_REQUIRE(tl::aligned16(q_out) && tl::aligned16(qkv) && tl::aligned16(cache_k) && tl::aligned16(cache_v) &&
                   tl::aligned16(rope_table) && tl::aligned16(vT),
               "tl_hgemm_prefill_rope_qkv_vt_f16: pointers must be 16-byte aligned");
    const size_t dim = (size_t)n_heads * head_dim, N = 3 * dim, M = (size_t)n_tokens;
    float* slabs = nullptr;
    int splits = 1;
    tl::Workspace::Lease lease;   // keeps the split-K slabs in place until the kernel that reads them is enqueued
    int rc = M == 1 ? tl::launch_gemv(X, Wqkv, qkv, N, K, 1, 0, 0, 0, 0)
                    : tl::launch_hgemm(X, Wqkv, qkv, M, N, K, 1, 0, 0, 0, &slabs, &splits, &lease);
    if (rc != TL_OK) return rc;
    const tl::half_t* base = (const tl::half_t*)qkv;
    if (splits <= 1)
        return tl_prefill_rope_qkv_vt_f16(q_out, base, base + dim, base + 2 * dim, N, cache_k, cache_v, rope_table, vT, ldv,
                                          n_tokens, n_heads, head_dim);
    // the projections read from the slabs
    TL_REQUIRE(tl::aligned16(slabs), "tl_hgemm_prefill_rope_qkv_vt_f16: the split-K slabs must be 16-byte aligned");
    dim3 grid((unsigned)(ldv / 64), (unsigned)n_heads, 3);
    auto column = [](size_t col) { return reinterpret_cast<const tl::half_t*>((uintptr_t)(col * sizeof(tl::half_t))); };
    auto launch = [&](auto kernel) {
        hipLaunchKernelGGL(kernel, grid, dim3(256), 0, tl::stream(), (tl::half_t*)q_out, column(0), column(dim),
                           column(2 * dim), N, (tl::half_t*)cache_k, (tl::half_t*)cache_v, (const tl::half_t*)rope_table,
                           (tl::half_t*)vT, ldv, n_tokens, n_heads, (const float*)slabs, splits, M * N);
    };
    if (head_dim == 64) launch(tl::prefill_rope_qkv_vt_kernel<64, true>);
    else launch(tl::prefill_rope_qkv_vt_kernel<128, true>);
    TL_CHECK_LAUNCH("prefill_rope_qkv_vt_kernel<slabs>");
    return TL_OK;
}

int tl_gather_vt_f16(void* vT, const void* cache_v, int T, int ldv, int n_heads, int head_dim) {
    TL_ENSURE_INIT();
    TL_REQUIRE(vT && cache_v, "tl_gather_vt_f16: null pointer");
    TL_REQUIRE(T >= 1 && ldv >= T && ldv % 8 == 0 && n_heads >= 1 && head_dim >= 1, "tl_gather_vt_f16: bad sizes");
    TL_REQUIRE(n_heads <= 65535, "tl_gather_vt_f16: too many heads");
    dim3 grid((unsigned)((ldv + 63) / 64), (unsigned)((head_dim + 63) / 64), (unsigned)n_heads);
    hipLaunchKernelGGL(tl::gather_vt_kernel, grid, dim3(256), 0, tl::stream(), (tl::half_t*)vT, (const tl::half_t*)cache_v,
                       T, ldv, n_heads, head_dim);
    TL_CHECK_LAUNCH("gather_vt_kernel");
    return TL_OK;
}

int tl_prefill_attention_f16(void* out, const void* q, const void* cache_k, const void* vT, int ldv, int start_pos,
                             int n_tokens, int n_heads, int head_dim) {
    TL_ENSURE_INIT();
    TL_REQUIRE(out && q && cache_k && vT, "tl_prefill_attention_f16: null pointer");
    TL_REQUIRE(start_pos >= 0 && n_tokens >= 1 && n_heads >= 1 && n_heads <= 65535, "tl_prefill_attention_f16: bad sizes");
    TL_REQUIRE(head_dim == 64 || head_dim == 128, "tl_prefill_attention_f16: head_dim %d not supported (64 or 128)",
               head_dim);
    // the value reads run to the end of the last block of 32 keys
    TL_REQUIRE(ldv % 8 == 0 && ldv >= ((start_pos + n_tokens + 31) / 32) * 32,
               "tl_prefill_attention_f16: ldv=%d must be a multiple of 8 and cover the context rounded up to 32", ldv);
    TL_REQUIRE(tl::aligned16(q) && tl::aligned16(cache_k) && tl::aligned16(vT) && tl::aligned16(out),
               "tl_prefill_attention_f16: operands must be 16-byte aligned");
    const float sq = sqrtf((float)head_dim);
    const tl::half_t divisor = (tl::half_t)sq;  // the reference divides by half(sqrt(head_dim)) (Transformer.cpp:94)
    const int variant = tl::g_prefill_attention_variant;
    const bool tiled_ok = head_dim == 128 && ldv >= ((start_pos + n_tokens + 63) / 64) * 64;
    if (variant == 2) TL_REQUIRE(tiled_ok, "tl_prefill_attention_f16: the tiled kernel needs head_dim 128 and ldv covering the context rounded up to 64");
    if (tiled_ok && (variant == 2 || (variant == 0 && n_tokens >= 128))) {
        static bool attr_set = false;
        constexpr int lds_bytes = 2 * (64 * 128 * 2 + 128 * 64 * 2);
        if (!attr_set) {
            TL_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(tl::prefill_attention_tiled_kernel<128, false>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes));
            TL_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(tl::prefill_attention_tiled_kernel<128, true>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes));
            attr_set = true;
        }
        const unsigned groups = (unsigned)((n_tokens + 127) / 128);
        // two workgroups fit a CU; beyond that a workgroup takes a long and a short group of 128 query rows
        const bool paired = (size_t)groups * (size_t)n_heads >= 2 * (size_t)tl::device_info().cu_count;
        const unsigned slots = paired ? (groups + 1) / 2 : groups;   // workgroups per head
        TL_REQUIRE((size_t)slots * (size_t)n_heads <= 0x7fffffffu, "tl_prefill_attention_f16: too many workgroups");
        auto kernel = paired ? tl::prefill_attention_tiled_kernel<128, true> : tl::prefill_attention_tiled_kernel<128, false>;
        hipLaunchKernelGGL(kernel, dim3(slots * (unsigned)n_heads), dim3(256), lds_bytes, tl::stream(), (tl::half_t*)out,
                           (const tl::half_t*)q, (const tl::half_t*)cache_k, (const tl::half_t*)vT, ldv, start_pos, n_tokens,
                           n_heads, divisor, (int)slots);
        TL_CHECK_LAUNCH("prefill_attention_tiled_kernel");
        return TL_OK;
    }
    dim3 grid((unsigned)((n_tokens + 31) / 32), (unsigned)n_heads);
    if (head_dim == 64)
        hipLaunchKernelGGL(tl::prefill_attention_kernel<64>, grid, dim3(64), 0, tl::stream(), (tl::half_t*)out,
                           (const tl::half_t*)q, (const tl::half_t*)cache_k, (const tl::half_t*)vT, ldv, start_pos, n_tokens,
                           n_heads, divisor);
    else
        hipLaunchKernelGGL(tl::prefill_attention_kernel<128>, grid, dim3(64), 0, tl::stream(), (tl::half_t*)out,
                           (const tl::half_t*)q, (const tl::half_t*)cache_k, (const tl::half_t*)vT, ldv, start_pos, n_tokens,
                           n_heads, divisor);
    TL_CHECK_LAUNCH("prefill_attention_kernel");
    return TL_OK;
}

int tl_set_decode_attention_merge(int mode) {
    TL_REQUIRE(mode >= 0 && mode <= 3, "tl_set_decode_attention_merge: %d out of range [0,3]", mode);
    tl::g_decode_merge_mode = mode;
    return TL_OK;
}

int tl_set_prefill_attention_variant(int variant) {
    TL_REQUIRE(variant >= 0 && variant <= 2, "tl_set_prefill_attention_variant: %d out of range [0,2]", variant);
    tl::g_prefill_attention_variant = variant;
    return TL_OK;
}

int tl_rope_qk_store_kv_f16(void* qkv, void* cache_k, void* cache_v, int pos, int n_heads, int head_dim) {
    TL_ENSURE_INIT();
    TL_REQUIRE(qkv && cache_k && cache_v, "tl_rope_qk_store_kv_f16: null pointer");
    TL_REQUIRE(pos >= 0 && n_heads >= 1 && head_dim >= 2 && head_dim % 2 == 0,
               "tl_rope_qk_store_kv_f16: bad sizes pos=%d n_heads=%d head_dim=%d", pos, n_heads, head_dim);
    TL_REQUIRE(((uintptr_t)qkv & 3) == 0 && ((uintptr_t)cache_k & 3) == 0 && ((uintptr_t)cache_v & 3) == 0,
               "tl_rope_qk_store_kv_f16: pointers must be 4-byte aligned");
    const int pairs = 3 * n_heads * head_dim / 2;
    hipLaunchKernelGGL(tl::rope_qk_store_kv_kernel, dim3((pairs + 255) / 256), dim3(256), 0, tl::stream(),
                       (tl::half_t*)qkv, (tl::half_t*)cache_k, (tl::half_t*)cache_v, pos, n_heads, head_dim);
    TL_CHECK_LAUNCH("rope_qk_store_kv_kernel");
    return TL_OK;
}

int tl_add_rms_norm_f16(void* sum_out, void* norm_out, const void* a, const void* b, const void* weight, float eps,
                        int hidden_size, int num_tokens) {
    TL_ENSURE_INIT();
    TL_REQUIRE(sum_out && norm_out && a && b && weight, "tl_add_rms_norm_f16: null pointer");
    TL_REQUIRE(hidden_size > 0 && num_tokens >= 0, "tl_add_rms_norm_f16: bad sizes");
    if (num_tokens == 0) return TL_OK;
    const bool vec = hidden_size % 8 == 0 && hidden_size <= 512 * 8 * 4 && tl::aligned16(sum_out) &&
                     tl::aligned16(norm_out) && tl::aligned16(a) && tl::aligned16(b) && tl::aligned16(weight);
    if (vec) {
        const int cpt = (hidden_size / 8 + 511) / 512;
        auto launch = [&](auto kernel) {
            hipLaunchKernelGGL(kernel, dim3(num_tokens), dim3(512), 0, tl::stream(), (tl::half_t*)sum_out,
                               (tl::half_t*)norm_out, (const tl::half_t*)a, (const tl::half_t*)b,
                               (const tl::half_t*)weight, eps, hidden_size, (const float*)nullptr, 0, (size_t)0);
        };
        if (cpt <= 1) launch(tl::add_rms_norm_vec_kernel<1>);
        else if (cpt == 2) launch(tl::add_rms_norm_vec_kernel<2>);
        else launch(tl::add_rms_norm_vec_kernel<4>);
    } else {
        hipLaunchKernelGGL(tl::add_rms_norm_kernel, dim3(num_tokens), dim3(256), 0, tl::stream(), (tl::half_t*)sum_out,
                           (tl::half_t*)norm_out, (const tl::half_t*)a, (const tl::half_t*)b,
                           (const tl::half_t*)weight, eps, hidden_size);
    }
    TL_CHECK_LAUNCH("add_rms_norm_kernel");
    return TL_OK;
}

int tl_hgemm_add_rms_norm_f16(const void* A, const void* W, const void* residual, const void* norm_weight, float eps,
                              void* sum_out, void* norm_out, size_t M, size_t N, size_t K) {
    TL_ENSURE_INIT();
    TL_REQUIRE(A && W && residual && norm_weight && sum_out && norm_out, "tl_hgemm_add_rms_norm_f16: null pointer");
    TL_REQUIRE(N >= 1 && N <= 0x7fffffffu && M <= 0x7fffffffu, "tl_hgemm_add_rms_norm_f16: bad sizes");
    if (M == 0) return TL_OK;
    const bool vec = N % 8 == 0 && N <= 512 * 8 * 4 && tl::aligned16(sum_out) && tl::aligned16(norm_out) &&
                     tl::aligned16(residual) && tl::aligned16(norm_weight);
    float* slabs = nullptr;
    int splits = 1;
    tl::Workspace::Lease lease;   // keeps the split-K slabs in place until the norm kernel that reads them is enqueued
    // the product goes to norm_out (overwritten by the normalised rows afterwards) unless K was split
    int rc = M == 1 ? tl::launch_gemv(A, W, norm_out, N, K, 1, 0, 0, 0, 0)
                    : tl::launch_hgemm(A, W, norm_out, M, N, K, 1, 0, 0, 0, vec ? &slabs : nullptr, vec ? &splits : nullptr,
                                       &lease);
    if (rc != TL_OK) return rc;
    if (splits <= 1) return tl_add_rms_norm_f16(sum_out, norm_out, residual, norm_out, norm_weight, eps, (int)N, (int)M);
    const int cpt = (int)((N / 8 + 511) / 512);
    auto launch = [&](auto kernel) {
        hipLaunchKernelGGL(kernel, dim3((unsigned)M), dim3(512), 0, tl::stream(), (tl::half_t*)sum_out, (tl::half_t*)norm_out,
                           (const tl::half_t*)residual, (const tl::half_t*)nullptr, (const tl::half_t*)norm_weight, eps, (int)N,
                           (const float*)slabs, splits, M * N);
    };
    if (cpt <= 1) launch(tl::add_rms_norm_vec_kernel<1, true>);
    else if (cpt == 2) launch(tl::add_rms_norm_vec_kernel<2, true>);
    else launch(tl::add_rms_norm_vec_kernel<4, true>);
    TL_CHECK_LAUNCH("add_rms_norm_vec_kernel<slabs>");
    return TL_OK;
}

int tl_causal_mask_f16(void* mask, int reps, int seqlen, int start_pos) {
    TL_ENSURE_INIT();
    TL_REQUIRE(mask, "tl_causal_mask_f16: null pointer");
    TL_REQUIRE(reps >= 0 && seqlen >= 0 && start_pos >= 0, "tl_causal_mask_f16: negative size");
    const size_t n = (size_t)reps * seqlen * ((size_t)start_pos + seqlen);
    if (n == 0) return TL_OK;
    size_t blocks = (n + 255) / 256;
    const size_t cap = (size_t)tl::device_info().cu_count * 16;
    if (blocks > cap) blocks = cap;
    hipLaunchKernelGGL(tl::causal_mask_kernel, dim3((unsigned)blocks), dim3(256), 0, tl::stream(), (tl::half_t*)mask,
                       seqlen, start_pos, n);
    TL_CHECK_LAUNCH("causal_mask_kernel");
    return TL_OK;
}

}  // extern "C"
