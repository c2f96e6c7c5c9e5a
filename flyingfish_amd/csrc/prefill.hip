// Prefill path (token-sorted grouped FP8 GEMM on MFMA) and the W8A8 block linear.
#include "common.cuh"
#include "api.h"

extern "C" __attribute__((visibility("default"))) int ffmoe_linear_fp8_block_w8a8(const void*, const float*, const void*, const float*, void*, int, int, int, void*) {
  return ffmoe::ff_fail(FFMOE_ERR_UNSUPPORTED, "ffmoe_linear_fp8_block_w8a8 is not built yet");
}
extern "C" __attribute__((visibility("default"))) uint64_t ffmoe_prefill_scratch_bytes(int, int, int, int, int) { return 0; }
extern "C" __attribute__((visibility("default"))) int ffmoe_prefill_contribute(const ffmoe_expert_table*, const ffmoe_prefill*, void*) {
  return ffmoe::ff_fail(FFMOE_ERR_UNSUPPORTED, "ffmoe_prefill_contribute is not built yet");
}
