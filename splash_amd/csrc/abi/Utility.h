// Parameters of the utility kernels: a plain 128-bit copy and a streaming read, which calibrate
// the memory counters and measure the achievable HBM rate next to the operators' kernels.
#pragma once
#include <stdint.h>

struct UtilityCopyParams {
  uint64_t vectors;  // 16-byte vectors to move
};
#ifdef __cplusplus
static_assert(sizeof(UtilityCopyParams) == 8, "copy parameters are 8 bytes on both sides");
#endif
