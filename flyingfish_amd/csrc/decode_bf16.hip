// Decode stages for FmtBf16 experts.
#include "decode_kernel.cuh"

namespace ffmoe {
int decode_launch_bf16(const DecodeParams& p, int rg, int stage_mask, hipStream_t st) { return launch_format<FmtBf16>(p, rg, stage_mask, st); }
}  // namespace ffmoe
