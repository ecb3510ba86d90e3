/*
 * tensorlib_llama2.h : C ABI of the host-side Llama2 driver (libtensorlib_llama2.so).
 *
 * The driver is this repository's own C++ caller of the matmul hot path.  It issues the op
 * sequence of the reference's model code through the Device-shaped backend
 * (include/tl_hip_device.hpp over include/tensorlib_amd.h):
 *   Transformer::forward / TransformerBlock::forward / Attention::forward /
 *   FeedForward::forward     model/llama2_7b/src/Transformer.cpp:26-178,263-299
 *   Llama2::generate          model/llama2_7b/src/llama2.cpp:15-101
 *   ActivationBuffer          model/llama2_7b/include/ActivationBuffer.hpp:10-36
 * Weights are borrowed device pointers (fp16, row-major [out_features, in_features], as
 * nn::Linear stores them, tensorLib/src/nn/linear.cpp:43-49).
 *
 * All functions return 0 on success, negative on failure; tlm_last_error() has the message.
 */
#ifndef TENSORLIB_LLAMA2_H
#define TENSORLIB_LLAMA2_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct tlm_model tlm_model;

/* Weight slots for tlm_set_weight. Per-layer kinds take a layer index, the others ignore it. */
enum {
    TLM_W_TOK_EMB = 0,    /* [vocab, dim] */
    TLM_W_ATT_NORM = 1,   /* [dim]            per layer */
    TLM_W_WQ = 2,         /* [dim, dim]       per layer */
    TLM_W_WK = 3,
    TLM_W_WV = 4,
    TLM_W_WO = 5,
    TLM_W_FFN_NORM = 6,   /* [dim]            per layer */
    TLM_W_W1 = 7,         /* [hidden, dim]    per layer */
    TLM_W_W2 = 8,         /* [dim, hidden]    per layer */
    TLM_W_W3 = 9,         /* [hidden, dim]    per layer */
    TLM_W_FINAL_NORM = 10,/* [dim] */
    TLM_W_CLASSIFIER = 11 /* [vocab, dim] */
};

/* Execution modes of tlm_forward / tlm_generate. */
enum {
    /* The reference's op list one for one (Appendix-B order): separate q/k/v GEMVs, two RoPE
     * launches, setItem cache writes, full K/V re-gather with `contiguous`, per-head matmul2d
     * (as one batched launch), ScalarDiv, mask add, softmax, EwiseAdd/EwiseMul, silu. */
    TLM_MODE_REFERENCE_CHAIN = 0,
    /* Same mathematics with the decode step fused: q|k|v and w1|w3 as single GEMVs when the
     * weights are adjacent in memory, RoPE + cache write in one launch, attention read from the
     * cache in place, residual-add + RMSNorm in one launch, silu*mul in one launch. */
    TLM_MODE_FUSED = 1
};

/* Buffers exposed to tests by tlm_get_buffer. */
enum { TLM_BUF_X = 0, TLM_BUF_LOGITS = 1, TLM_BUF_CACHE_K = 2, TLM_BUF_CACHE_V = 3, TLM_BUF_NEXT_TOKEN = 4 };

const char* tlm_last_error(void);

/* Allocates activation buffers and a [max_seq_len, n_heads, head_dim] fp16 K and V cache per
 * layer (batch 1).  max_tokens = largest number of tokens one tlm_forward call will process. */
int tlm_create(tlm_model** out, int dim, int hidden_dim, int n_layers, int n_heads, int vocab_size,
               int max_seq_len, float norm_eps, int max_tokens);
int tlm_destroy(tlm_model* m);

int tlm_set_weight(tlm_model* m, int kind, int layer, const void* dev_ptr);

/* Create a model from a llama2.c legacy fp16 checkpoint, the file the reference's read_checkpoint
 * loads (model/llama2_7b/src/main.cpp:36-228; writer script/export.py:138-190).  The model owns
 * the weight memory.  max_seq_len > 0 caps the KV cache below the file's seq_len. */
int tlm_load_checkpoint(const char* path, int max_tokens, int max_seq_len, tlm_model** out);

/* out7 = {dim, hidden_dim, n_layers, n_heads, vocab_size, max_seq_len, max_tokens}. */
int tlm_get_config(tlm_model* m, int* out7);

/* Forward `n_tokens` tokens (device int32 ids) at positions [start_pos, start_pos + n_tokens).
 * all_logits != 0: logits for every token ([n_tokens, vocab], as Transformer::forward does);
 * all_logits == 0: only the last token's row is projected.  *logits_out receives the device
 * pointer of the fp16 logits (row 0 = first computed row).  Asynchronous on the library stream. */
int tlm_forward(tlm_model* m, const int* dev_tokens, int n_tokens, int start_pos, int mode, int all_logits,
                void** logits_out);

/* Llama2::generate: prefill the prompt at position 0, then n_generate greedy steps.
 * host_out_tokens receives n_generate ids (the first comes from the prefill logits).
 * Seconds are host wall-clock around each phase, synchronised at both ends.  No early stop on
 * BOS/EOS (random-weight runs would stop at arbitrary points). */
int tlm_generate(tlm_model* m, const int* host_prompt, int n_prompt, int n_generate, int mode,
                 int* host_out_tokens, double* prefill_seconds, double* decode_seconds);

/* Llama2::text_completion and one turn of Llama2::chat (model/llama2_7b/src/llama2.cpp:103-107,120-148) on
 * top of Llama2::generate (llama2.cpp:15-101), with the tokenizer of include/tensorlib_tokenizer.h.
 *   chat_template != 0 renders "[INST] <text> [/INST]" first (llama2.cpp:131,137);
 *   the text is encoded with BOS and without EOS (llama2.cpp:105,143) and must fit max_tokens;
 *   *position is the reference's process-wide `total_len` (llama2.cpp:13), owned by the caller here: the prompt
 *   is prefilled at [*position, *position + n_prompt), and *position advances by the prompt length plus the
 *   number of decode steps run (llama2.cpp:52,83), so the next turn continues in the same KV cache;
 *   the token picked from the prefill logits is always emitted (llama2.cpp:57-63); each of the up to
 *   n_generate decode steps (the reference runs 256) picks the next token and stops, without emitting it, on
 *   BOS (1) or EOS (2) (llama2.cpp:88-91);
 *   every emitted token goes to on_piece (may be NULL) with its piece decoded as the reference prints it,
 *   tokenizer.decode(-1, token) (llama2.cpp:63,93); the bytes are not terminated and only valid during the call.
 * *n_decode_steps receives the number of decode steps run (the reference's generate_cnt).  The host reads one
 * token id per step, as the reference does (llama2.cpp:85); benchmarks use tlm_generate, which does not.
 * Declared with an opaque tokenizer pointer so this header does not depend on the tokenizer's. */
struct tlt_tokenizer;
typedef void (*tlm_piece_fn)(const char* bytes, size_t n_bytes, int token, void* user);
int tlm_text_completion(tlm_model* m, const struct tlt_tokenizer* tok, const char* text, int chat_template,
                        int* position, int n_generate, int mode, tlm_piece_fn on_piece, void* user,
                        int* n_decode_steps, double* prefill_seconds, double* decode_seconds);

int tlm_get_buffer(tlm_model* m, int which, int layer, void** dev_ptr);

#ifdef __cplusplus
}
#endif
#endif /* TENSORLIB_LLAMA2_H */
