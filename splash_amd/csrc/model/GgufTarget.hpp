// A dense decoder's weights from a GGUF file: the counterpart, for the dense verify driver, of the reference's
// GgufTargetLoader and planImages (runtime/model/GgufTarget.hpp:24-75, GgufImage.cpp:474-520, :696-713): the
// geometry from the file's metadata, each layer's projections as weight images (q|k|v one projection of three segments,
// each of its tensor's format), the norms as bf16, the token table as native rows and the head, tied to the token table
// when the file holds no output.weight.
#pragma once
#include "model/DenseVerify.hpp"
#include "model/GgufFile.hpp"
#include "model/HybridVerify.hpp"

namespace splash::model {

// The geometry the file's metadata names (<architecture>.block_count, .embedding_length, .feed_forward_length,
// .attention.head_count, .attention.head_count_kv, .attention.key_length, .rope.freq_base; the vocabulary is the token
// table's rows). Throws GgufError for a missing key, an RMS epsilon other than 1e-6 or a geometry the kernels do not
// take.
[[nodiscard]] DenseDimensions ggufDenseDimensions(const GgufFile &file);
// Loads every weight of `verify` (built with ggufDenseDimensions(file)) from the file. Throws GgufError naming every
// tensor that is missing, of a type or shape the path does not read, or that the file holds and the loader does not
// read (biases, for one).
void loadGgufDenseWeights(hip::Backend &backend, const GgufFile &file, DenseVerify &verify);

// The hybrid targets' files (the reference's HybridGguf family, architectures qwen35 and qwen35moe: GgufImage.cpp:474-520
// mixerImage and ffnImage, :541-557, :874-936 requireMetadata). The geometry: Gated DeltaNet mixers with every
// <arch>.full_attention_interval-th layer an attention layer, <arch>.ssm.group_count key heads and .ssm.time_step_rank value
// heads of .ssm.state_size = 128 with .ssm.conv_kernel = 4 taps, and a mixture of .expert_count experts
// (.expert_used_count a row, .expert_feed_forward_length wide, .expert_shared_feed_forward_length of shared slices) or,
// without experts, a dense SwiGLU of .feed_forward_length. Layers past block_count - nextn_predict_layers are the
// multi-token prediction blocks the target does not run.
[[nodiscard]] HybridDimensions ggufHybridDimensions(const GgufFile &file);
// Loads every weight of `verify` (built with ggufHybridDimensions(file)): an attention layer's attn_q | attn_k | attn_v and
// attn_output; a GDN layer's attn_qkv | attn_gate with the value heads' rows regrouped by key head (llama.cpp stores
// them tiled), ssm_beta and ssm_alpha as rows of floats for the fp32 projection, ssm_conv1d, ssm_a, ssm_dt.bias,
// ssm_norm and ssm_out, whose input columns stay in the file's tiled order (the driver's GDN rows then leave tiled:
// setTiledGdnHeads); the router as rows of floats, the routed experts of ffn_gate_exps and ffn_up_exps (or the fused
// ffn_gate_up_exps) and ffn_down_exps an image an expert, the shared expert's slices after them and its scalar gate.
// Throws GgufError naming every tensor that is missing, of a type or shape the path does not read, or unread.
void loadGgufHybridWeights(hip::Backend &backend, const GgufFile &file, HybridVerify &verify);

} // namespace splash::model
