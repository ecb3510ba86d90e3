/*
 * tensorlib_tokenizer.h : C ABI of the llama2.c-format tokenizer (part of libtensorlib_llama2.so).
 *
 * Host-side text <-> token ids for the Llama2 driver; replaces the reference's Tokenizer class
 *   Tokenizer::Tokenizer   model/llama2_7b/src/Tokenizer.cpp:7-60   (tokenizer.bin reader)
 *   Tokenizer::encode      model/llama2_7b/src/Tokenizer.cpp:62-154 (UTF-8 grouping, byte fallback, score-ordered merges)
 *   Tokenizer::decode      model/llama2_7b/src/Tokenizer.cpp:156-169
 * as called by Llama2::generate / text_completion (model/llama2_7b/src/llama2.cpp:63,93,105).
 *
 * File format (llama2.c tokenizer.bin): int32 max_token_length, then per token float32 score,
 * int32 byte length, bytes.  Ids 1 and 2 are BOS and EOS, ids 3..258 the byte tokens "<0x00>".."<0xFF>".
 *
 * All functions return 0 on success, negative on failure; tlt_last_error() has the message.
 */
#ifndef TENSORLIB_TOKENIZER_H
#define TENSORLIB_TOKENIZER_H

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct tlt_tokenizer tlt_tokenizer;

const char* tlt_last_error(void);

/* Tokenizer::Tokenizer(path, vocab_size) (Tokenizer.cpp:7-60). */
int tlt_load(const char* path, int vocab_size, tlt_tokenizer** out);
int tlt_destroy(tlt_tokenizer* t);
int tlt_vocab_size(const tlt_tokenizer* t);

/* Tokenizer::encode(text, bos, eos) (Tokenizer.cpp:62-154).  Writes at most `capacity` ids to out_tokens and
 * the number of ids of the full encoding to *n_tokens; fails (nothing usable written) if capacity is too small. */
int tlt_encode(const tlt_tokenizer* t, const char* text, size_t text_len, int bos, int eos, int* out_tokens,
               size_t capacity, size_t* n_tokens);

/* Tokenizer::decode(prev_token, token) (Tokenizer.cpp:156-169): the piece of `token`, without its leading
 * space when it follows BOS, byte tokens turned into their byte.  Unlike the reference it does not modify the
 * stored vocabulary (the reference strips the space from the stored piece for good).  Writes the bytes (no
 * terminator) to out and their count to *n_bytes; fails if capacity is too small. */
int tlt_decode(const tlt_tokenizer* t, int prev_token, int token, char* out, size_t capacity, size_t* n_bytes);

#ifdef __cplusplus
}
#endif
#endif /* TENSORLIB_TOKENIZER_H */
