// Parameters of the acceptance kernels (the reference's abi/Sampling.h:50-67, :314-317 and
// abi/VerifyTree.h:40-45).
#pragma once
#include <stdint.h>

#define SAMPLING_SHARDS 32u          // vocabulary shards of one row's scan (one workgroup each)
#define SAMPLING_THREADS 256u
#define SAMPLING_RANGES 256u         // id-ordered ranges a sampled row's draw sums
#define SAMPLING_MAXIMUM_LANES 8u
#define SAMPLING_MAXIMUM_ROWS 16u    // rows of a lane's verify block
#define SAMPLING_STOP_TOKENS 4u
#define SAMPLING_NO_TOKEN 0xFFFFFFFFu  // a row with no selectable logit selects it (SPLASH_NO_TOKEN)

// A lane's rows of the packed rows (SplashLaneRows).
struct SamplingLaneRows {
  uint32_t first;
  uint32_t rows;
};

// decode_sample_argmax_sharded / _reduce, decode_sample_mass_sharded, decode_sample_residual_sharded,
// decode_sample_draw: one dispatch over `rows` packed logits rows of `vocabulary` fp32 logits.
struct TargetSamplingParams {
  uint32_t vocabulary;
  uint32_t rows;          // packed rows
  uint32_t lanes;
  uint32_t logits_stride; // floats between logits rows
  float temperature[SAMPLING_MAXIMUM_LANES];
  uint32_t sampling_mask; // lanes that sample; the others take the argmax
  uint32_t reserved[3];
  struct SamplingLaneRows lane[SAMPLING_MAXIMUM_LANES];
};

// decode_accept_tree: one thread per lane (AcceptBatchParams).
struct AcceptBatchParams {
  uint32_t lanes;
  uint32_t reserved[3];
  uint32_t remaining[SAMPLING_MAXIMUM_LANES];
  uint32_t stop_tokens[SAMPLING_STOP_TOKENS];
  struct SamplingLaneRows lane[SAMPLING_MAXIMUM_LANES];
};

#ifdef __cplusplus
static_assert(sizeof(TargetSamplingParams) == 16 + 32 + 16 + 64, "target sampling parameters are 128 bytes on both sides");
static_assert(sizeof(AcceptBatchParams) == 16 + 32 + 16 + 64, "acceptance parameters are 128 bytes on both sides");
#endif
