/*
 * tensorlib_amd.h : C ABI of the MI355X (gfx950) device backend for tensorLib's
 * matrix-multiplication hot path.
 *
 * Every entry point is what a `Device<dtype>` subclass of the reference
 * (tensorLib/include/device/Device.hpp:5-110) forwards to: plain device pointers and
 * sizes, no C++ types, no exceptions across the boundary.  "f16" buffers hold IEEE
 * binary16 values (the reference's `half`); element counts are in elements, not bytes.
 *
 * Conventions
 *   - Return value: 0 on success, a negative TL_E* code otherwise; tl_last_error()
 *     returns the message of the calling thread's last failure.
 *   - All pointers named A/B/C/x/W/y/in/out/src/dst are DEVICE pointers unless the
 *     parameter is called host_*.
 *   - Work is enqueued on one in-order HIP stream (the null stream unless
 *     tl_set_stream() was called) and is asynchronous w.r.t. the host, like the
 *     reference's default-stream launches (tensorLib/src/device/cuda/CUDA.cu).
 *   - Matrices are dense row-major.  The matmul operand contract is the reference's:
 *     A[M,K], B[N,K] ("col-major B"), C[M,N] (tensorLib/src/ops/matmul.cpp:265-268).
 */
#ifndef TENSORLIB_AMD_H
#define TENSORLIB_AMD_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define TL_OK 0
#define TL_EINVAL (-1)   /* bad argument (null pointer, misaligned, size out of range) */
#define TL_EHIP (-2)     /* a HIP runtime call failed */
#define TL_ENOMEM (-3)   /* device allocation failed */
#define TL_ELIMIT (-4)   /* size exceeds a documented limit of the entry point */

/* ---------------------------------------------------------------- runtime ---- */

/* Select the GPU, read its properties, create library state.  Idempotent.
 * Replaces the implicit CUDA context creation of the first cudaMalloc
 * (tensorLib/src/device/cuda/CUDA.cu:16-19). */
int tl_init(int device_ordinal);

/* Message of the calling thread's last failing tl_* call ("" if none).
 * Replaces the print-and-exit of CUDA_CHECK (tensorLib/include/device/cuda/CUDA.cuh:131-151). */
const char* tl_last_error(void);

/* Library version string, e.g. "tensorlib_amd 0.1 gfx950". */
const char* tl_version(void);

/* Number of compute units and wavefront size of the selected GPU (0 before tl_init). */
int tl_device_cu_count(void);

/* Enqueue all later work on `hip_stream` (a hipStream_t; NULL = null stream).
 * The reference uses the default stream everywhere (tensorLib/src/device/cuda/gemm.cu).
 * When the stream changes and the stream being replaced has used the library's scratch buffers (split-K GEMM,
 * decode attention with more than one chunk), this call waits for that stream to drain, so the buffers are free
 * when the first call on the new stream reuses them; the stream being replaced must therefore still exist when
 * this is called, and may be destroyed right after. */
int tl_set_stream(void* hip_stream);
void* tl_get_stream(void);

/* Device memory: CUDA<dtype>::CUDA(size) / ~CUDA() (tensorLib/src/device/cuda/CUDA.cu:16-32). */
int tl_malloc(void** dev_ptr, size_t bytes);
int tl_free(void* dev_ptr);

/* Copies.  h2d/d2h synchronise with the stream before returning, like the 1-element
 * cudaMemcpy of getDataLinear/setDataLinear (tensorLib/src/device/cuda/CUDA.cu:71-81)
 * and the weight loader's cudaMemcpy (model/llama2_7b/src/main.cpp:53-57). */
int tl_memcpy_h2d(void* dst, const void* host_src, size_t bytes);
int tl_memcpy_d2h(void* host_dst, const void* src, size_t bytes);
int tl_memcpy_d2d(void* dst, const void* src, size_t bytes);
int tl_synchronize(void);

/* Zeroes the counters the library keeps in its own device scratch between calls: the per-head tickets of the decode
 * attention (grown-on-demand workspace and static array) and the per-tile tickets of the one-launch split-K GEMM.
 * Every kernel leaves them at zero when it completes, so this is only needed after a launch that did not complete
 * (a device error reported by a later call, a stream destroyed with work pending): a ticket left set would make
 * later calls merge early, silently.  Enqueues fill kernels on the library's stream; no allocation, no host wait.
 * No counterpart in the reference (its kernels keep no state between launches). */
int tl_reset_scratch(void);

/* ------------------------------------------------------- the hot path ---- */

/* C[M,N] = A[M,K] . B[N,K]^T, fp32 accumulation, one rounding to fp16 at the end.
 * Replaces Device<half>::matmul2d (tensorLib/include/device/Device.hpp:22) as
 * implemented by CUDA<half>::matmul2d (tensorLib/src/device/cuda/gemm.cu:153-172);
 * numerics follow CPU<half>::matmul2d (tensorLib/src/device/cpu/CPU.cpp:76-89).
 * M == 1 takes the GEMV path, M > 1 the MFMA GEMM path; any M,N,K >= 1 is accepted
 * (unaligned shapes take a slower generic kernel).  C must not alias A or B. */
int tl_matmul2d_f16(const void* A, const void* B, void* C, size_t M, size_t N, size_t K);

/* y[N] = W[N,K] . x[K].  Replaces gemv_v6 / gemv_v4
 * (tensorLib/src/device/cuda/gemv.cu:379-450, :260-300).  Fast path needs K % 8 == 0
 * and 16-byte aligned x and W; otherwise a scalar-load kernel runs. */
int tl_gemv_f16(const void* x, const void* W, void* y, size_t N, size_t K);

/* C[M,N] = A[M,K] . B[N,K]^T on the matrix cores.  Replaces hgemm_cublas
 * (tensorLib/src/device/cuda/hgemm.cu:20-38) but keeps fp32 accumulation, which the
 * cuBLAS call with fp16 alpha/beta does not guarantee. */
int tl_hgemm_f16(const void* A, const void* B, void* C, size_t M, size_t N, size_t K);

/* Batched form of the loop in ops::matmul<dtype>::call2
 * (tensorLib/src/ops/matmul.cpp:297-321): for b in [0,batch):
 *   C + b*strideC = matmul2d(A + b*strideA, B + b*strideB), strides in elements
 * (0 = operand broadcast over the batch).  One launch instead of `batch` launches. */
int tl_matmul2d_batched_f16(const void* A, const void* B, void* C, size_t M, size_t N, size_t K,
                            size_t batch, size_t strideA, size_t strideB, size_t strideC);

/* fp32 / int32 matmul2d for Device<float> / Device<int> (same operand contract;
 * tensorLib/src/device/cpu/CPU.cpp:76-89 with dtype=float/int: fp32 accumulate then
 * cast).  Plain tiled kernels; not part of the fp16 hot path. */
int tl_matmul2d_f32(const void* A, const void* B, void* C, size_t M, size_t N, size_t K);

/* Force a kernel variant for benchmarking/tests: 0 = automatic dispatch.  The variant
 * names are listed by tl_gemv_variant_name()/tl_hgemm_variant_name() (NULL past the end). */
int tl_set_gemv_variant(int variant);
int tl_set_hgemm_variant(int variant);
const char* tl_gemv_variant_name(int variant);
const char* tl_hgemm_variant_name(int variant);
/* Measurement hook (no reference counterpart): fp16 MFMA rate sustained out of registers, in
 * TFLOP/s.  mode 0: constant operands; mode 1: both operands change with every instruction (v_mfma_f32_32x32x16_f16);
 * modes 2 and 3: the same two with v_mfma_f32_16x16x32_f16.
 * Synchronises the stream.  Used by bench.py to place HGEMM against the power-managed ceiling. */
int tl_measure_mfma_rate_f16(int mode, double* tflops);
/* Measurement hook (no reference counterpart): the GEMV kernel the dispatch uses for K <= 4096, built with time stamps.
 * Same arithmetic and stores as tl_gemv_f16; in addition workgroup g writes the GPU's constant 100 MHz counter at its
 * first instruction to stamps[2 g] and after its last store to stamps[2 g + 1] (device memory, uint64, capacity in
 * elements); *workgroups receives the number of workgroups launched.  bench.py --workload gemv_timeline turns the
 * stamps of a sequence of launches into the launch time line (ramp, streaming phase, tail, time between launches). */
int tl_gemv_f16_stamped(const void* x, const void* W, void* y, size_t N, size_t K, void* stamps,
                        size_t stamps_capacity, int* workgroups);
/* Tuning hook: force the number of K splits of the MFMA GEMM (0 = automatic). */
int tl_set_hgemm_splits(int splits);
/* Inspection hook (no reference counterpart): the kernel variant (index into tl_hgemm_variant_name(); -1 = the
 * kernel for at most 32 rows) and the number of K splits the most recent fp16 GEMM launch of this process used. */
int tl_hgemm_last_plan(int* variant, int* splits);
/* Tuning hook: 0 = the dispatch takes the kernels with 16x16x32 MFMAs and accumulators in AGPRs (variants
 * a256x256x64w2x2, a256x128x64w2x2) wherever whole tiles of theirs cover the problem, -1 = never (the ring kernels with
 * 32x32x16 MFMAs serve every shape, as they do for partly filled tiles). */
int tl_set_hgemm_agpr_kernels(int mode);
/* Inspection hook (no reference counterpart): while `stamps` is not NULL, every launch of those two kernels with at most
 * capacity / 2 workgroups writes stamps[2 * w] / stamps[2 * w + 1] = the GPU's constant 100 MHz counter at workgroup w's
 * first instruction and after its last store (device memory, `capacity` 64-bit words).  bench.py --workload
 * hgemm_timeline turns them into the time line of a launch.  NULL switches it off. */
int tl_set_hgemm_stamps(void* stamps, size_t capacity);
/* Tuning hook: where the fp32 partial sums of a split-K GEMM are added up.  0 = automatic and 2 = by a second kernel
 * (the default: measured faster on every split shape); 1 = inside the GEMM launch, by the workgroup that finishes a
 * C tile's last split (one counter per tile in the library's scratch, zero between launches), whenever C takes 8-byte
 * stores (N % 8 == 0, 16-byte aligned C), the tile is at most 128x256, the launch has at most 4096 tiles and the
 * partial sums stay below 2 GiB, else the second kernel.  Both add the splits in split order: same bits.
 * tl_hgemm_last_split_in_launch() tells which one the most recent GEMM launch used (1 = inside the launch). */
int tl_set_hgemm_splitk_merge(int mode);
int tl_hgemm_last_split_in_launch(void);
/* Tuning hook: the MFMA GEMM's workgroups start their walk over K at K tile
 * (tile_column * per_tile + xcd * per_xcd) % tiles and wrap (-1 = automatic, 0 = no rotation). */
int tl_set_hgemm_k_rotation(int per_tile, int per_xcd);
/* Tuning hook: the MFMA GEMM numbers its tiles down bands of `band` rows of tiles (0 = automatic; a value of
 * at least the number of tile rows numbers them down whole columns). */
int tl_set_hgemm_tile_band(int band);
/* Tuning hook: the kernel for 2 <= M <= 32 that keeps X in registers and streams W once (0 = automatic, -1 = never:
 * such shapes then take the tile kernels). */
int tl_set_hgemm_fewrows(int mode);
/* Tuning hook: prefill attention kernel, 0 = automatic, 1 = one wavefront per 32 query rows,
 * 2 = LDS-tiled workgroups of 128 query rows (head_dim 128, ldv covering the context rounded up to 64). */
int tl_set_prefill_attention_variant(int variant);
/* Tuning hook: where the chunk partials of the decode attention are merged: 0 = automatic (inside the one launch
 * up to 512 cached positions), 1 = always inside the launch, by the workgroup that finishes a head's last chunk,
 * 2 = always by a second launch, 3 = like 1 but ordered by a release/acquire read-modify-write on the ticket and plain
 * accesses to the partials (the HIP memory model's own terms; slower, kept as the tested alternative).  Same bits
 * in every mode. */
int tl_set_decode_attention_merge(int mode);
/* Tuning hook: cached positions per workgroup of the decode attention: 0 = automatic, else 64, 128 or 256
 * (head_dim 256 always uses 64). */
int tl_set_decode_attention_chunk(int positions);
/* Tuning hook: cap the GEMV grid at `waves` resident wavefronts per compute unit (0 = default). */
int tl_set_gemv_grid_waves_per_cu(int waves);

/* ------------------------------- small kernels that keep decode on the GPU ---- */

/* out[t,:] = in[t,:] * weight[:] / sqrt(mean(in[t,:]^2) + eps), fp32 math, one rounding.
 * Replaces CUDA<dtype>::rms_norm (tensorLib/include/device/cuda/CUDA.cuh:108,
 * tensorLib/src/device/cuda/rms_norm.cu:139-184), called from
 * nn::RMSNorm::forward_fused_cuda (tensorLib/src/nn/rmsNorm.cpp:62-94). */
int tl_rms_norm_f16(void* out, const void* in, const void* weight, float eps,
                    int hidden_size, int num_tokens);

/* Interleaved-pair rotary embedding on a contiguous [B,T,n_heads,head_dim] tensor;
 * in == out is allowed.  Replaces Device::apply_rotary_emb
 * (tensorLib/include/device/Device.hpp:94-101; tensorLib/src/device/cuda/CUDA.cu:405-437;
 * numerics per tensorLib/src/device/cpu/CPU.cpp:427-461). */
int tl_apply_rotary_emb_f16(const void* in, void* out, int start_pos, int B, int T,
                            int n_heads, int head_dim);

/* Row softmax over the last dimension of a contiguous [rows, cols] matrix; in == out
 * allowed.  Replaces Device::softmax (Device.hpp:79; tensorLib/src/device/cuda/softmax.cu:21-82;
 * tensorLib/src/device/cpu/softmax.cpp:9-31).  Max/sum are carried in fp32. */
int tl_softmax_f16(void* out, const void* in, size_t rows, size_t cols);

/* Elementwise: out = silu(in) = in / (1 + exp(-in)) evaluated in fp32
 * (tensorLib/src/device/cuda/CUDA.cu:334-347; Device.hpp:57). */
int tl_silu_f16(void* out, const void* in, size_t n);

/* Elementwise binary ops on halves, one rounding each (Device.hpp:62-65;
 * tensorLib/include/device/cuda/binary.cuh:3-74).  op: 0 add, 1 sub, 2 mul, 3 div. */
int tl_binary_f16(void* out, const void* a, const void* b, size_t n, int op);
/* Same with a scalar right operand given as the 16 bits of a half (Device.hpp:66-70). */
int tl_binary_scalar_f16(void* out, const void* a, uint16_t scalar_bits, size_t n, int op);

/* out[i] = base[offset + sum_d idx_d(i) * stride[d]] for the row-major index i over
 * `shape` (Device::contiguous, Device.hpp:30-35; tensorLib/src/device/cuda/CUDA.cu:83-116).
 * ndim <= 8.  host_shape/host_stride are HOST arrays of ndim ints. */
int tl_contiguous_f16(void* out, const void* base, const int* host_shape, const int* host_stride,
                      int ndim, size_t offset, size_t n);
/* base[offset + sum_d idx_d(i) * stride[d]] = src[i] (Device::setItemEwise,
 * Device.hpp:36-41; tensorLib/src/device/cuda/CUDA.cu:118-151). */
int tl_set_item_ewise_f16(void* base, const void* src, const int* host_shape, const int* host_stride,
                          int ndim, size_t offset, size_t n);

/* out[r] = index of the first maximum of in[r*reduce_size .. +reduce_size)
 * (Device::argmax, Device.hpp:77; first-max-wins like tensorLib/src/device/cpu/CPU.cpp:356-372). */
int tl_argmax_f16(int* out, const void* in, size_t reduce_size, size_t num_elements);

/* out[t,:] = table[ids[t],:] for t < n_tokens; ids is a DEVICE int32 array.
 * Replaces the per-token select+setItem loop of nn::Embedding::forward
 * (tensorLib/src/nn/embedding.cpp:47-81) without the per-token host read. */
int tl_embedding_f16(void* out, const void* table, const int* ids, int n_tokens, int dim, int vocab);

/* out[i] = value for i < n (Device::full, Device.hpp:25). */
int tl_full_f16(void* out, uint16_t value_bits, size_t n);

/* ------------------------------------------ fused forms used by the driver ---- */

/* out = silu(a) * b in fp32, one rounding: FeedForward's silu + EwiseMul
 * (model/llama2_7b/src/Transformer.cpp:137-141) in one pass. */
int tl_silu_mul_f16(void* out, const void* a, const void* b, size_t n);

/* Single-token attention over a [max_seq, n_heads, head_dim] KV cache read in place:
 * out[h,:] = softmax(q[h,:] . K[0:T,h,:]^T / half(sqrt(head_dim))) . V[0:T,h,:].
 * Replaces the gather + 2*n_heads gemv_v4 launches + scale + softmax of
 * Attention::forward at seqlen 1 (model/llama2_7b/src/Transformer.cpp:55-109). */
int tl_decode_attention_f16(void* out, const void* q, const void* cache_k, const void* cache_v,
                            int T, int n_heads, int head_dim);

/* y[N] = W[N,K] . (silu(ab[0:K]) * ab[K:2K]): FeedForward's silu, EwiseMul and w2 projection
 * (model/llama2_7b/src/Transformer.cpp:137-143) in one launch; the gated vector is rounded to
 * fp16 once, as tl_silu_mul_f16 would store it.  Needs 512 <= K <= 12288, K % 8 == 0. */
int tl_gemv_silu_mul_f16(const void* ab, const void* W, void* y, size_t N, size_t K);

/* y[N] = W[N,K] . (rmsnorm(x + addend) * norm_weight) and sum_out = x + addend: the residual EwiseAdd of
 * TransformerBlock::forward, the RMSNorm that follows it and the Linear that consumes the norm
 * (model/llama2_7b/src/Transformer.cpp:165-175, tensorLib/src/nn/rmsNorm.cpp:85-106) in one launch.
 * The sum is rounded to fp16 before it is squared and the normalised vector is rounded to fp16 once, as
 * tl_add_rms_norm_f16 stores them.  addend may be NULL (plain RMSNorm), sum_out may be NULL; sum_out must
 * not alias x or addend.  Needs 512 <= K <= 12288, K % 8 == 0, 16-byte aligned operands. */
int tl_gemv_add_rms_norm_f16(const void* x, const void* addend, const void* norm_weight, float eps,
                             const void* W, void* y, void* sum_out, size_t N, size_t K);

/* sum_out[M,N] = residual + A[M,K] . W[N,K]^T and norm_out = rmsnorm(sum_out) * norm_weight: a Linear, the residual
 * EwiseAdd and the RMSNorm that follow it in TransformerBlock::forward (model/llama2_7b/src/Transformer.cpp:165-175)
 * for M token rows.  Same values as tl_matmul2d_f16 followed by tl_add_rms_norm_f16 (product rounded to fp16, sum
 * rounded to fp16, fp32 mean of squares); when the GEMM splits K, its second pass is folded into the add + norm
 * kernel.  norm_out also serves as the scratch for the product; it must not alias A or residual. */
int tl_hgemm_add_rms_norm_f16(const void* A, const void* W, const void* residual, const void* norm_weight, float eps,
                              void* sum_out, void* norm_out, size_t M, size_t N, size_t K);

/* tl_rope_qk_store_kv_f16 + tl_decode_attention_f16 in one launch pair: qkv is the raw q|k|v
 * projection of the token at position `pos`; q is rotated on load, the rotated k and the v row
 * are written to cache_k[pos] / cache_v[pos], and out[h,:] attends to positions 0..pos.
 * rope_table: NULL, or a table from tl_rope_table_f16 covering `pos` (saves the sin/cos/pow). */
int tl_decode_attention_rope_f16(void* out, const void* qkv, void* cache_k, void* cache_v,
                                 const void* rope_table, int pos, int n_heads, int head_dim);

/* tl_decode_attention_rope_f16 for callers that cannot allocate (code under HIP-graph capture, tight serving loops,
 * harnesses that forbid hipMalloc).  It has no counterpart in the reference.  Same kernels, same arguments, same
 * results; the per-chunk partial results go to a static device array of TL_DECODE_ATTENTION_STATIC_SCRATCH_FLOATS
 * floats that is part of the library's code object (each GPU holds its copy until the process ends) instead of the
 * grown-on-demand workspace, and the call makes no hipMalloc / hipFree.  Limit:
 *   1024 + n_heads * ceil((pos + 1) / 64) * (head_dim + 2) <= TL_DECODE_ATTENTION_STATIC_SCRATCH_FLOATS
 * (32 heads of 128: 16064 positions) is always accepted; what exceeds the array returns TL_EINVAL (contexts from 1280
 * positions on with head_dim up to 128 are cut into chunks of 128 positions and need half of that).  Every call on a GPU shares that GPU's array:
 * calls that overlap on one GPU (two streams, two host threads) race; calls on one stream do not.  The caller clears
 * nothing: every partial a call reads was written by the same call, and the per-head tickets in the first 1024 words
 * of the array (one per head whatever the head count; launches with more than 1024 heads merge with a second kernel
 * and use none) are zero when the library is loaded and are set back to zero by the workgroup that draws a head's
 * last one.  Only a launch that did not run to completion (a device error, a process that tore the stream down)
 * can leave a ticket set; tl_reset_scratch() clears them. */
#define TL_DECODE_ATTENTION_STATIC_SCRATCH_FLOATS (1u << 20)
int tl_decode_attention_rope_static_f16(void* out, const void* qkv, void* cache_k, void* cache_v,
                                        const void* rope_table, int pos, int n_heads, int head_dim);

/* table[pos][pair] = (half(cos), half(sin)) of pos / 10000^(2*pair/head_dim) for pos < max_seq:
 * max_seq * head_dim halves.  The same values every RoPE entry point computes on the fly
 * (tensorLib/src/device/cpu/CPU.cpp:444-447); the reference's own precompute_freqs table is unused
 * (model/llama2_7b/src/Transformer.cpp:203-216). */
int tl_rope_table_f16(void* table, int max_seq, int head_dim);

/* Decode-step glue after a fused q|k|v projection (qkv = [q | k | v], each n_heads*head_dim
 * halves): rotary-embed q in place, rotary-embed k into cache_k[pos], copy v into cache_v[pos]
 * (caches are [max_seq, n_heads, head_dim]).  Replaces two apply_rotary_emb launches and two
 * setItem launches (model/llama2_7b/src/Transformer.cpp:47-53). */
int tl_rope_qk_store_kv_f16(void* qkv, void* cache_k, void* cache_v, int pos, int n_heads, int head_dim);

/* sum_out = a + b (one rounding) and norm_out = rmsnorm(sum_out) * weight per token: the
 * residual EwiseAdd and the RMSNorm that follows it
 * (model/llama2_7b/src/Transformer.cpp:167-171).  sum_out may alias a or b. */
int tl_add_rms_norm_f16(void* sum_out, void* norm_out, const void* a, const void* b, const void* weight,
                        float eps, int hidden_size, int num_tokens);

/* Prefill glue after the q, k, v projections of n_tokens rows with row stride `row_stride` elements
 * (dim, or 3*dim for one fused q|k|v GEMM): q is rotated and written head-major [n_heads, n_tokens,
 * head_dim], k is rotated into cache_k[start_pos + s], v copied into cache_v[start_pos + s].  Replaces two
 * apply_rotary_emb, two setItem and one transpose+contiguous of Attention::forward
 * (model/llama2_7b/src/Transformer.cpp:47-60).  rope_table as built by tl_rope_table_f16. */
int tl_prefill_rope_qkv_f16(void* q_out, const void* q, const void* k, const void* v, size_t row_stride,
                            void* cache_k, void* cache_v, const void* rope_table, int start_pos, int n_tokens,
                            int n_heads, int head_dim);

/* tl_prefill_rope_qkv_f16 for a fresh context (start_pos 0) that also writes the transposed value operand
 * tl_gather_vt_f16 would build (vT[h][d][t] = v[t][h][d], zero for n_tokens <= t < ldv): one launch instead of two.
 * head_dim 64 or 128, ldv a multiple of 64, row_stride a multiple of 8, 16-byte aligned pointers. */
int tl_prefill_rope_qkv_vt_f16(void* q_out, const void* q, const void* k, const void* v, size_t row_stride, void* cache_k,
                               void* cache_v, const void* rope_table, void* vT, int ldv, int n_tokens, int n_heads,
                               int head_dim);

/* The fused q|k|v projection of a fresh context followed by tl_prefill_rope_qkv_vt_f16: X[n_tokens, K] .
 * Wqkv[3*n_heads*head_dim, K]^T, then RoPE, cache rows and the transposed values.  When the GEMM splits K (short
 * prompts), the kernel that rotates reads the fp32 partial sums and adds them itself in split order, so the separate
 * second pass of the split and one launch are saved; same bits as the two entries called one after the other.
 * qkv: [n_tokens, 3*n_heads*head_dim] halves, receives the projection when K is not split. */
int tl_hgemm_prefill_rope_qkv_vt_f16(const void* X, const void* Wqkv, void* qkv, void* q_out, void* cache_k, void* cache_v,
                                     const void* rope_table, void* vT, int ldv, int n_tokens, int n_heads, int head_dim,
                                     size_t K);

/* vT[h][d][t] = cache_v[t][h][d] for t < T and 0 for T <= t < ldv (ldv % 8 == 0): the transposed value operand
 * of tl_prefill_attention_f16; the reference builds the same tensor with transpose + contiguous
 * (model/llama2_7b/src/Transformer.cpp:66-80). */
int tl_gather_vt_f16(void* vT, const void* cache_v, int T, int ldv, int n_heads, int head_dim);

/* Causal attention of n_tokens new tokens over cache positions [0, start_pos + n_tokens) in one launch:
 * scores, ScalarDiv by half(sqrt(head_dim)), mask, softmax and the product with the values
 * (Attention::forward, model/llama2_7b/src/Transformer.cpp:92-109) without a score matrix in memory.
 * q: [n_heads, n_tokens, head_dim] (rotated, as tl_prefill_rope_qkv_f16 writes it); cache_k: [.., n_heads,
 * head_dim]; vT from tl_gather_vt_f16 with ldv >= the context rounded up to 32; out: [n_tokens, n_heads,
 * head_dim].  head_dim 64 or 128.  With head_dim 128, at least 128 new tokens and ldv >= the context rounded up
 * to 64, workgroups of 128 query rows share key tiles through LDS (same results bit for bit). */
int tl_prefill_attention_f16(void* out, const void* q, const void* cache_k, const void* vT, int ldv, int start_pos,
                             int n_tokens, int n_heads, int head_dim);

/* In place on scores [n_heads, seqlen, start_pos + seqlen]: ScalarDiv by `divisor` (fp16 bits), the causal
 * mask add and softmax(3) of Attention::forward (model/llama2_7b/src/Transformer.cpp:94-105) in one launch;
 * the quotient is rounded to fp16 before the softmax, as the separate kernels store it. */
int tl_scaled_causal_softmax_f16(void* scores, uint16_t divisor_bits, int n_heads, int seqlen, int start_pos);

/* out[r, j] = silu(ab[r, j]) * ab[r, hidden + j] for rows of a fused w1|w3 projection [rows, 2*hidden]
 * (FeedForward::forward, model/llama2_7b/src/Transformer.cpp:137-141).  hidden % 8 == 0. */
int tl_silu_mul_rows_f16(void* out, const void* ab, size_t rows, size_t hidden);

/* out[M, hidden] = silu(X . W1^T) * (X . W3^T) for W13 = [W1; W3] stored as one [2*hidden, K] matrix: the two
 * projections and the gate of FeedForward::forward (model/llama2_7b/src/Transformer.cpp:136-141) in one launch, the
 * gate applied to the fp16-rounded projections in the GEMM's epilogue: the arithmetic of tl_matmul2d_f16 into a
 * [M, 2*hidden] buffer followed by tl_silu_mul_rows_f16.  The bits agree with that pair when both add the products
 * of a row in the same order (the same kernel family, K walked from the same first tile, K not split: what
 * tl_set_hgemm_k_rotation(0, 0) and tl_set_hgemm_splits(1) force); the default dispatch picks tiles and K walks per
 * launch, so the two generally differ by the rounding of the fp32 sums, within the tolerance of the GEMM.  Shapes the one-launch kernel does not serve (K % 64 != 0,
 * unaligned pointers, at most 32 rows, M == 1) take exactly that two-step path through `scratch`
 * ([M, 2*hidden] halves; may be NULL when the caller knows the one-launch path applies).  hidden % 8 == 0. */
int tl_hgemm_silu_mul_f16(const void* X, const void* W13, void* scratch, void* out, size_t M, size_t hidden, size_t K);

/* mask[r,i,j] = (j > start_pos + i) ? -inf : 0 for r < reps, i < seqlen, j < start_pos+seqlen.
 * Replaces the element-by-element host loop of Transformer::get_mask
 * (model/llama2_7b/src/Transformer.cpp:231-261). */
int tl_causal_mask_f16(void* mask, int reps, int seqlen, int start_pos);

#ifdef __cplusplus
}
#endif
#endif /* TENSORLIB_AMD_H */
