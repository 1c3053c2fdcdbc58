/*
 * GGUF ingest: the file format on the step before the token loop.
 *
 * Reads what spy::GGUFAdapter::init_from_file reads (storage/src/adapter/gguf_adapter.cpp:90-190 in the
 * Spy tree: magic "GGUF", u32 version, u64 tensor count, u64 key/value count, the key/value section, the
 * tensor infos {name, u32 n_dim, u64 ne[n_dim], u32 type, u64 offset}, data aligned to `general.alignment`,
 * default 32) and does what its SimpleModelLoader + the scheduler's constant fetch do together
 * (storage/include/loader/simple_loader.h:36-70, backend/distributor/include/scheduler/default_scheduler.h:
 * 120-156): maps the file and hands every weight tensor to the backend -- here ONE upload per tensor into
 * HBM, in the file's own block layout, before the first pass.
 *
 * The hyper-parameters are the ones spy::HyperParam / LLAMAModel take from the file
 * (model/include/llm/model/abstract_model.h:72-144, model/include/llm/model/llama.h:55-62): the
 * `<arch>.*` keys below must be stored as UInt32 and the epsilon as Float32, as the reference's strict
 * std::get<> demands.
 *
 * Plain C, POD only.  Library: spy_amd/libspy_backend.so.  Every function returns 0 or a negative
 * SPY_GGUF_E* code (or a HIP / spy_hip error code > 0 from the upload); spy_gguf_last_error() gives the text of
 * the calling thread's last failure.
 */
#ifndef SPY_GGUF_H
#define SPY_GGUF_H

#include <stddef.h>
#include <stdint.h>

#include "spy_hip.h"

#ifdef __cplusplus
extern "C" {
#endif

#define SPY_GGUF_EIO          (-1)   /* cannot open / map the file */
#define SPY_GGUF_EFORMAT      (-2)   /* not GGUF, truncated, or inconsistent */
#define SPY_GGUF_EKEY         (-3)   /* key absent or of another type */
#define SPY_GGUF_EUNSUPPORTED (-4)   /* a model this backend does not run (architecture, tensor type, grouped-query attention) */
#define SPY_GGUF_EINVAL       (-5)

/* metadata value types of the file format (ModelMetaDataType, storage/include/adapter/type.h) */
enum { SPY_GGUF_U8 = 0, SPY_GGUF_I8, SPY_GGUF_U16, SPY_GGUF_I16, SPY_GGUF_U32, SPY_GGUF_I32, SPY_GGUF_F32, SPY_GGUF_BOOL,
       SPY_GGUF_STRING, SPY_GGUF_ARRAY, SPY_GGUF_U64, SPY_GGUF_I64, SPY_GGUF_F64 };

typedef struct spy_gguf spy_gguf;

const char *spy_gguf_last_error(void);

/* ---- the file (GGUFAdapter::init_from_file) ---- */
int spy_gguf_open(const char *path, spy_gguf **out);
void spy_gguf_close(spy_gguf *g);
/* version, counts, `general.alignment` (default 32), file offset of the data section, bytes of the data
 * section as the reference sums them (every tensor rounded up to the alignment) */
int spy_gguf_header(const spy_gguf *g, uint32_t *version, uint64_t *n_tensors, uint64_t *n_kv, uint32_t *alignment,
                    uint64_t *data_offset, uint64_t *data_bytes);
/* type of a key (SPY_GGUF_*), for arrays also element type and length; SPY_GGUF_EKEY when absent */
int spy_gguf_kv_type(const spy_gguf *g, const char *key, int32_t *type, int32_t *elem_type, uint64_t *n);
/* strict getters: the stored type must be exactly the one asked for */
int spy_gguf_get_u32(const spy_gguf *g, const char *key, uint32_t *out);
int spy_gguf_get_f32(const spy_gguf *g, const char *key, float *out);
int spy_gguf_get_str(const spy_gguf *g, const char *key, const char **ptr, uint64_t *len);      /* not NUL-terminated: points into the map */
int spy_gguf_get_arr_str(const spy_gguf *g, const char *key, uint64_t i, const char **ptr, uint64_t *len);
int spy_gguf_get_arr_data(const spy_gguf *g, const char *key, const void **ptr, uint64_t *n);  /* numeric arrays: packed elements */
/* tensors in file order; ne[] is padded with 1, nbytes = row size of `type` over all elements */
int spy_gguf_tensor_info(const spy_gguf *g, uint64_t index, const char **name, int32_t *type, int32_t *n_dim, int64_t ne[4],
                         uint64_t *offset, uint64_t *nbytes);
int64_t spy_gguf_find_tensor(const spy_gguf *g, const char *name);                             /* index or -1 */
int spy_gguf_tensor_data(const spy_gguf *g, uint64_t index, const void **ptr);                 /* host pointer into the map */

/* ---- file -> HBM -> token loop ---- */
typedef struct spy_gguf_model spy_gguf_model;

/* Opens the file, checks that it is a LLaMA model this backend runs (architecture "llama", head_count_kv ==
 * head_count, 128-wide heads, matrices Q4_0 / Q8_0 / Q4_K / Q6_K, embeddings F32 or Q8_0, norms F32), uploads every
 * tensor once and creates the token loop (spy_hip_llama_create).  n_ctx: context to allocate KV caches for, 0 =
 * `<arch>.context_length`; rounded up to a multiple of 8.  spy_hip_init must have been called. */
int spy_gguf_model_load(const char *path, int32_t n_ctx, spy_gguf_model **out);
spy_hip_llama *spy_gguf_model_engine(spy_gguf_model *m);           /* owned by the model */
const spy_gguf *spy_gguf_model_file(const spy_gguf_model *m);      /* the parsed file (vocabulary etc.), owned by the model */
/* hyper-parameters as passed to spy_hip_llama_create (device pointers inside), bytes uploaded, and the times spent
 * parsing, uploading (host -> HBM, synchronised) and creating the token loop, in milliseconds */
int spy_gguf_model_info(const spy_gguf_model *m, spy_hip_llama_desc *desc, uint64_t *weight_bytes, double *parse_ms, double *upload_ms,
                        double *create_ms);
void spy_gguf_model_free(spy_gguf_model *m);

#ifdef __cplusplus
}
#endif
#endif
