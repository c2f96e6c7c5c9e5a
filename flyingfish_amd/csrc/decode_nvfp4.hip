// Decode stages for FmtNvfp4 experts.
#include "decode_kernel.cuh"

namespace ffmoe {
int decode_launch_nvfp4(const DecodeParams& p, int rg, int stage_mask, hipStream_t st) { return launch_format<FmtNvfp4>(p, rg, stage_mask, st); }
}  // namespace ffmoe
