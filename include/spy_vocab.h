/*
 * SentencePiece vocabulary of a GGUF file: text -> token ids before the token loop, ids -> text after it.
 *
 * Follows spy::SentencePieceVocab (model/include/llm/vocab/sentence_piece_vocab.h:67-263 in the Spy tree) over the
 * tables spy::Vocab builds from the file (model/include/llm/vocab/abstract_vocab.h:57-126: `tokenizer.ggml.tokens`,
 * optional `.scores`, `.token_type`, `.bos_token_id` / `.eos_token_id` / `.unknown_token_id` /
 * `.seperator_token_id` / `.padding_token_id`): a leading space, spaces escaped to U+2581, the text split into UTF-8
 * characters, adjacent pairs merged greedily by token score (ties: the leftmost pair), pieces that are no token
 * re-split along their merges and finally spelled as <0xXX> byte tokens.
 *
 * Two things are done the way that code means rather than the way it runs: every call starts from empty merge
 * state (the reference keeps its symbol list, queue and merge map in the object, so only the first call of an
 * object tokenizes its own text), and `special` is accepted but changes nothing, as in the reference, whose table of
 * special tokens is never filled (init_special_token_cache is not called).
 *
 * Plain C.  Library: spy_amd/libspy_backend.so.  Errors: negative SPY_GGUF_E* codes, text from spy_gguf_last_error().
 */
#ifndef SPY_VOCAB_H
#define SPY_VOCAB_H

#include <stdint.h>

#include "spy_gguf.h"

#ifdef __cplusplus
extern "C" {
#endif

/* ModelTokenType (model/include/llm/vocab/type.h) */
enum { SPY_TOKEN_UNDEFINED = 0, SPY_TOKEN_NORMAL = 1, SPY_TOKEN_UNKNOWN = 2, SPY_TOKEN_CONTROL = 3, SPY_TOKEN_USER_DEFINED = 4,
       SPY_TOKEN_UNUSED = 5, SPY_TOKEN_BYTE = 6 };

typedef struct spy_vocab spy_vocab;

/* copies what it needs: the file may be closed afterwards */
int spy_vocab_from_gguf(const spy_gguf *g, spy_vocab **out);
void spy_vocab_free(spy_vocab *v);
int32_t spy_vocab_size(const spy_vocab *v);
/* bos (default 1), eos (2), unknown (0), separator (-1), padding (-1), linefeed (the token of byte 0x0A, 13 if there is none) */
int spy_vocab_special_ids(const spy_vocab *v, int32_t *bos, int32_t *eos, int32_t *unk, int32_t *sep, int32_t *pad, int32_t *linefeed);
int spy_vocab_token(const spy_vocab *v, int32_t id, const char **text, uint64_t *len, float *score, int32_t *type);
/* SentencePieceVocab::tokenize(text, bos, special): returns the number of ids (at most `cap` are written), or a
 * negative code when a character has neither a token nor a byte token */
int64_t spy_vocab_tokenize(const spy_vocab *v, const char *text, uint64_t len, int32_t add_bos, int32_t special, int32_t *ids, uint64_t cap);
/* SentencePieceVocab::token_to_piece: bytes of one token as text (normal: U+2581 back to spaces; byte tokens: the
 * byte; unknown: U+2585; control: nothing).  Returns the length (at most `cap` bytes are written). */
int64_t spy_vocab_token_to_piece(const spy_vocab *v, int32_t id, char *buf, uint64_t cap);
/* the pieces of n ids one after the other */
int64_t spy_vocab_detokenize(const spy_vocab *v, const int32_t *ids, uint64_t n, char *buf, uint64_t cap);

#ifdef __cplusplus
}
#endif
#endif
