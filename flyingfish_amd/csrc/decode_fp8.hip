// Decode stages for FmtFp8 experts.
#include "decode_kernel.cuh"

namespace ffmoe {
int decode_launch_fp8(const DecodeParams& p, int rg, int stage_mask, hipStream_t st) { return launch_format<FmtFp8>(p, rg, stage_mask, st); }
}  // namespace ffmoe
