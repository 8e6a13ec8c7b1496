/*
 * oxq_files.h - C ABI for the on-disk formats that feed the quantized matmul
 * library: GGUF files, safetensors files, and the `quantization_config` block
 * of a Hugging Face config.json.
 *
 * The reference maps a checkpoint, indexes its tensors by name and hands the
 * packed tensors to the layer constructors (src/common/gguf_weights.rs,
 * src/common/weights.rs); the GGUF container itself is parsed by candle-core
 * 0.11's `quantized::gguf_file`, the safetensors container by the
 * `safetensors` crate.  This interface does the same on the host: a file (or a
 * set of shards) is memory-mapped read-only and indexed; tensor payloads are
 * exposed as pointers into the mapping, never copied.  oxq_upload() moves a
 * payload into caller-allocated device memory.
 *
 * Status codes, oxq_last_error() and the threading rules are those of oxq.h.
 * Nothing here needs a GPU except oxq_upload().
 */
#ifndef OXQ_FILES_H
#define OXQ_FILES_H

#include "oxq.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Element type of a tensor as stored in the file. */
typedef enum oxq_file_dtype {
    OXQ_FILE_F32 = 0,
    OXQ_FILE_F16 = 1,
    OXQ_FILE_BF16 = 2,
    OXQ_FILE_F64 = 3,
    OXQ_FILE_U8 = 4,
    OXQ_FILE_I8 = 5,
    OXQ_FILE_U16 = 6,
    OXQ_FILE_I16 = 7,
    OXQ_FILE_U32 = 8,
    OXQ_FILE_I32 = 9,
    OXQ_FILE_U64 = 10,
    OXQ_FILE_I64 = 11,
    OXQ_FILE_BOOL = 12,
    OXQ_FILE_F8_E4M3 = 13,
    OXQ_FILE_F8_E5M2 = 14,
    OXQ_FILE_GGML_BLOCK = 15 /* GGUF block-quantized rows; see ggml_type / gguf_quant */
} oxq_file_dtype;

#define OXQ_FILE_MAX_RANK 8

typedef struct oxq_file_tensor {
    const char *name;    /* NUL-terminated, valid until the file is closed */
    int32_t file_dtype;  /* oxq_file_dtype */
    int32_t ggml_type;   /* GGUF only: the ggml type id stored in the file; -1 for safetensors */
    int32_t gguf_quant;  /* oxq_gguf_quant when the library has kernels for the block format, else -1 */
    int32_t rank;
    int64_t dims[OXQ_FILE_MAX_RANK]; /* row-major, outermost first (GGUF's stored order reversed, as
                                        candle reports it: a [out, in] weight has dims {out, in}) */
    const void *data;    /* host pointer into the read-only mapping; valid until the file is closed */
    uint64_t nbytes;
    int32_t shard;       /* index of the path the tensor came from */
    int32_t reserved;
} oxq_file_tensor;

typedef struct oxq_tensor_file oxq_tensor_file;

/* ---- GGUF ------------------------------------------------------------------
 * gguf_weights.rs:36-64 GgufWeights::load and 153-206 load_shards: versions 1-3,
 * little endian; tensors of every shard are merged by name (a later shard
 * replaces an earlier tensor of the same name), metadata is taken from the
 * first shard.  A tensor whose element count is not a multiple of its block
 * size, or whose payload reaches past the end of the file, fails the open
 * (gguf_weights.rs:318-345).  n_paths must be >= 1. */
int oxq_gguf_open(const char *const *paths, int n_paths, oxq_tensor_file **out);

/* ---- safetensors -------------------------------------------------------------
 * weights.rs:314-325 ModelWeights::load (MmapedSafetensors::multi): every file's
 * header is parsed and the tensors merged by name.  No tensor is converted or
 * filtered; the caller decides what to skip and what to cast. */
int oxq_safetensors_open(const char *const *paths, int n_paths, oxq_tensor_file **out);

int oxq_tensor_file_close(oxq_tensor_file *f);

/* Tensors are enumerated in the order of their names (byte-wise ascending). */
int64_t oxq_tensor_file_count(const oxq_tensor_file *f);
int oxq_tensor_file_at(const oxq_tensor_file *f, int64_t index, oxq_file_tensor *out);

/* gguf_weights.rs:70-81 get/try_get (exact name) and weights.rs:452-514
 * resolve_name/get/try_get for safetensors: the exact name first, then the
 * multimodal aliases (`model.X` -> `model.language_model.X`,
 * `model.language_model.model.X`, `language_model.X`, `language_model.model.X`,
 * `model.model.X`; `lm_head.weight` and `lm_head.weight_scale_inv` under the
 * same nestings).  *found = 0 and OXQ_OK when nothing resolves. */
int oxq_tensor_file_find(const oxq_tensor_file *f, const char *name, oxq_file_tensor *out, int *found);

/* gguf_weights.rs:84-89 total_size_bytes / weights.rs:576-581 runtime_size_bytes:
 * the sum of the stored payload sizes. */
uint64_t oxq_tensor_file_total_bytes(const oxq_tensor_file *f);

/* weights.rs:568-572 has_packed_quantized_weights: any `*.qweight` or `*.weight_packed`. */
int oxq_tensor_file_has_packed_quantized_weights(const oxq_tensor_file *f);

/* ---- GGUF metadata -----------------------------------------------------------
 * gguf_weights.rs:95-144: typed getters over the key/value map.  A key that is
 * missing, or whose stored type is not exactly the one asked for, gives
 * *found = 0 (the reference returns Err for both; its `_or` forms fall back to
 * a default for both). */
typedef enum oxq_gguf_value_type {
    OXQ_GGUF_U8 = 0,
    OXQ_GGUF_I8 = 1,
    OXQ_GGUF_U16 = 2,
    OXQ_GGUF_I16 = 3,
    OXQ_GGUF_U32 = 4,
    OXQ_GGUF_I32 = 5,
    OXQ_GGUF_F32 = 6,
    OXQ_GGUF_BOOL = 7,
    OXQ_GGUF_STRING = 8,
    OXQ_GGUF_ARRAY = 9,
    OXQ_GGUF_U64 = 10,
    OXQ_GGUF_I64 = 11,
    OXQ_GGUF_F64 = 12
} oxq_gguf_value_type;

int64_t oxq_gguf_metadata_count(const oxq_tensor_file *f);
/* key i in file order; *value_type its oxq_gguf_value_type; for arrays *elem_type and *elem_count too. */
int oxq_gguf_metadata_at(const oxq_tensor_file *f, int64_t index, const char **key, int *value_type,
                         int *elem_type, uint64_t *elem_count);
int oxq_gguf_metadata_u32(const oxq_tensor_file *f, const char *key, uint32_t *value, int *found);
int oxq_gguf_metadata_f32(const oxq_tensor_file *f, const char *key, float *value, int *found);
/* *value points at the string's bytes (NUL-terminated copy owned by the file). */
int oxq_gguf_metadata_string(const oxq_tensor_file *f, const char *key, const char **value, uint64_t *len,
                             int *found);
/* Any scalar integer, boolean or float value widened to double / int64 (no reference
 * counterpart: lets a caller read keys whose writer chose another width). */
int oxq_gguf_metadata_number(const oxq_tensor_file *f, const char *key, double *value, int *found);
/* gguf_weights.rs:216-218 architecture(): the `general.architecture` string. */
int oxq_gguf_architecture(const oxq_tensor_file *f, const char **value, uint64_t *len, int *found);
/* gguf_weights.rs:222-240 eos_token_ids(): `tokenizer.ggml.eos_token_id` (u32) followed by the
 * u32 elements of `tokenizer.ggml.eos_token_ids` not already listed.  Writes at most `cap` ids,
 * *count receives how many there are. */
int oxq_gguf_eos_token_ids(const oxq_tensor_file *f, uint32_t *ids, uint64_t cap, uint64_t *count);

/* ---- quantization scheme of a Hugging Face checkpoint ---------------------------
 * weights.rs:22-26 QuantScheme and hf_parser.rs:451-585 validate_quantization_config. */
typedef enum oxq_scheme_kind {
    OXQ_SCHEME_NONE = 0,               /* dense, FP8 (scale_inv companions) or MXFP4 (GPT-OSS experts) */
    OXQ_SCHEME_AWQ = 1,                /* bits 4 | 8, GEMM version */
    OXQ_SCHEME_GPTQ = 2,               /* bits 4 | 8, desc_act = false */
    OXQ_SCHEME_COMPRESSED_TENSORS4 = 3 /* pack-quantized symmetric int4, one group config */
} oxq_scheme_kind;

typedef struct oxq_quant_scheme {
    int32_t kind; /* oxq_scheme_kind */
    uint32_t bits;
    int32_t sym;  /* GPTQ only */
} oxq_quant_scheme;

/* `json` is the text of the `quantization_config` value (or of a whole config.json when
 * whole_config != 0, in which case its "quantization_config" member is looked up; absent =
 * null).  A recognised but unsupported combination returns OXQ_ERR_UNSUPPORTED with the
 * reason in oxq_last_error(); malformed JSON returns OXQ_ERR_FORMAT. */
int oxq_validate_quantization_config(const char *json, int whole_config, oxq_quant_scheme *out);

/* weights.rs:523-565 try_get_awq / try_get_gptq / try_get_compressed / try_get_quant:
 * the packed tensors of the projection at `prefix` under `scheme`.
 *   AWQ   `prefix.qweight`, `prefix.qzeros`, `prefix.scales`: all three or *found = 0
 *   GPTQ  `prefix.qweight`, `prefix.scales` required, `prefix.qzeros` optional
 *         (qzeros->data = NULL when absent)
 *   compressed-tensors  qweight <- `prefix.weight_packed`, scales <- `prefix.weight_scale`,
 *         qzeros->data = NULL; the caller converts with oxq_compressed_to_awq
 *   NONE  *found = 0
 * Names resolve as in oxq_tensor_file_find. */
int oxq_safetensors_try_get_quant(const oxq_tensor_file *f, const oxq_quant_scheme *scheme, const char *prefix,
                                  oxq_file_tensor *qweight, oxq_file_tensor *qzeros, oxq_file_tensor *scales,
                                  int *found);

/* Copies `nbytes` from host memory (typically oxq_file_tensor.data) to device memory on the
 * ctx's device, ordered on `stream`; returns once the host range has been read.  The reference
 * moves each tensor with Tensor::to_device / qtensor_from_ggml (weights.rs:392-404,
 * gguf_weights.rs:352-358). */
int oxq_upload(oxq_ctx *ctx, void *stream, void *dst_device, const void *src_host, uint64_t nbytes);

#ifdef __cplusplus
}
#endif
#endif /* OXQ_FILES_H */
