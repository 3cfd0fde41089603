/* GGUF files: the header parser and the step from a file's tensor to what the operators take.
 * Replaces, for the verify step's weights, the reference's model::GgufFile / GgufTensor / GgufMetadata
 * (runtime/model/GgufFile.hpp:24-150) and the image preparation of runtime/model/GgufImage.cpp: a tensor
 * of a projection format (Q4_K, Q5_K, Q6_K, Q8_0, IQ4_XS, IQ4_NL) becomes the weight image spo_projection_create takes,
 * a 16- or 32-bit float vector the bf16 weights of a norm. Status codes and the thread-local message of
 * sp_last_error are those of splash_hip.h; a malformed file is SP_BACKEND_ERROR with the parser's message. */
#pragma once
#include "splash_hip.h"
#include "splash_ops.h"

#ifdef __cplusplus
extern "C" {
#endif

typedef struct spg_file spg_file; /* model::GgufFile: the mapped file and its parsed header */

/* GgufFile::GgufFile (GgufFile.hpp:117): GGUF version 3, one file. */
sp_status spg_open(const char *path, spg_file **out);
/* The parts of a split GGUF (NAME-0000K-of-0000N.gguf, K = 1..N) in split order, which is their name order
 * (GgufFile.hpp:118-124, GgufFile.cpp:167-201, GgufTarget.cpp:19-46): the first part's metadata is the file's, and its
 * split.count and split.tensors.count, where stated, must be the parts and tensors read, so a part alone is refused; a
 * later part's split.no must be its place; a part of no tensors may end at its header. Tensors keep one numbering
 * across the parts. count 1 is spg_open. */
sp_status spg_open_parts(const char *const *paths, uint32_t count, spg_file **out);
void spg_close(spg_file *file);

/* GgufMetadata (GgufFile.hpp:95-107): integers and booleans as unsigned, floats as double, strings.
 * A getter returns 0 when the key is absent or of another kind; spg_metadata_string returns the
 * string's size with its terminator and copies up to `capacity` bytes. */
int spg_metadata_unsigned(const spg_file *file, const char *key, uint64_t *value);
int spg_metadata_float(const spg_file *file, const char *key, double *value);
size_t spg_metadata_string(const spg_file *file, const char *key, char *out, size_t capacity);

/* GgufFile::tensors / find (GgufFile.hpp:131-133). */
typedef struct spg_tensor {
  uint32_t ggml_type;   /* as the file stores it (ggml-common.h) */
  uint32_t dimensions;  /* 1..4 */
  uint64_t dims[4];     /* dims[0] is the row length */
  uint64_t bytes;
  uint32_t format;      /* the weight-image format (GGUF_FMT_* numbering) or 0xFFFFFFFF when the projections do not read the type */
  uint32_t reserved;
} spg_tensor;
uint64_t spg_tensor_count(const spg_file *file);
/* The tensor's name (size with terminator, copied up to `capacity`) and description; index below the count. */
size_t spg_tensor_name(const spg_file *file, uint64_t index, char *out, size_t capacity);
sp_status spg_tensor_info(const spg_file *file, uint64_t index, spg_tensor *out);
/* Index of the tensor of that name, or -1. */
int64_t spg_find(const spg_file *file, const char *name);
/* The tensor's bytes in the mapped file, valid until spg_close. */
const void *spg_tensor_data(const spg_file *file, uint64_t index);

/* Rows [first_row, first_row + rows) (rows 0: all) of a two-dimensional tensor of a projection format, packed
 * as the weight image and uploaded: whole 16-row tiles of whole 256-input super-blocks. The caller releases
 * the buffer; format, rows and input size are what spo_projection_create takes beside it. */
sp_status spg_load_image(sp_backend *backend, const spg_file *file, uint64_t index, uint32_t first_row, uint32_t rows,
                         sp_buffer **image, uint32_t *format, uint32_t *out_rows, uint32_t *input_size);
/* An F32, F16 or BF16 tensor as bf16 in device memory (a norm's weights). The caller releases the buffer. */
sp_status spg_load_bf16(sp_backend *backend, const spg_file *file, uint64_t index, sp_buffer **out, uint64_t *elements);

/* A dense decoder from a file (the reference's GgufTargetLoader and planImages for its targets, GgufTarget.hpp:24-75,
 * GgufImage.cpp:474-520, :696-713). spg_dense_dimensions reads the geometry from the metadata of the file's
 * architecture (block_count, embedding_length, feed_forward_length, attention.head_count / head_count_kv / key_length,
 * rope.freq_base; the vocabulary is token_embd.weight's rows; per-head q/k norms when blk.0.attn_q_norm.weight exists);
 * spo_dense_verify_load_gguf then loads every weight of a driver created with those dimensions: blk.N.attn_norm,
 * attn_q | attn_k | attn_v as one projection of three segments, each of its tensor's format, attn_q_norm, attn_k_norm,
 * attn_output, ffn_norm, ffn_gate, ffn_up, ffn_down, output_norm, token_embd (native rows, for the token gather) and
 * output.weight, or the token table again when the file ties them. A malformed file, a missing tensor, a type the
 * path does not read or a tensor the loader would ignore (a bias) is SP_BACKEND_ERROR naming all of them. */
sp_status spg_dense_dimensions(const spg_file *file, spo_dense_dimensions *out);
sp_status spo_dense_verify_load_gguf(spo_dense_verify *verify, const spg_file *file);

/* A hybrid decoder from a file (the reference's HybridGguf family: architectures qwen35 and qwen35moe, GgufImage.cpp:474-520
 * mixerImage and ffnImage, :541-557, :874-936). spg_hybrid_dimensions reads the geometry: the dense driver's keys, and
 * full_attention_interval, ssm.group_count (key heads), ssm.time_step_rank (value heads), ssm.state_size (128),
 * ssm.conv_kernel (4), ssm.inner_size, expert_count, expert_used_count, expert_feed_forward_length and
 * expert_shared_feed_forward_length, or without experts feed_forward_length; block_count less nextn_predict_layers
 * layers; gated attention when attn_q holds two rows a query dimension. spo_hybrid_verify_load_gguf loads a driver
 * created with those dimensions: an attention layer's attn_q | attn_k | attn_v, head norms and attn_output; a Gated
 * DeltaNet layer's attn_qkv | attn_gate with the value heads' rows regrouped by key head (llama.cpp stores them tiled,
 * GgufImage.hpp:29-38), ssm_beta and ssm_alpha as rows of floats the fp32 projection runs, ssm_conv1d, ssm_a, ssm_dt.bias,
 * ssm_norm (fp32) and ssm_out, whose input columns keep the file's order (the driver's GDN rows then leave tiled);
 * ffn_gate_inp as rows of floats, the routed experts of ffn_gate_exps and ffn_up_exps (or the fused ffn_gate_up_exps)
 * and ffn_down_exps an image an expert, the shared expert's slices after them, ffn_gate_inp_shexp; or a dense SwiGLU.
 * Errors as the dense loader's. */
sp_status spg_hybrid_dimensions(const spg_file *file, spo_hybrid_dimensions *out);
sp_status spo_hybrid_verify_load_gguf(spo_hybrid_verify *verify, const spg_file *file);

#ifdef __cplusplus
}
#endif
