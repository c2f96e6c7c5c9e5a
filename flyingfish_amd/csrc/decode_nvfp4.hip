// Decode stages for FmtNvfp4 experts.
#include "finish_kernel.cuh"
#include "token_layer.cuh"

namespace ffmoe {
int decode_launch_nvfp4(const DecodeParams& p, int rg, int stage_mask, hipStream_t st) { return launch_format<FmtNvfp4>(p, rg, stage_mask, st); }
int decode_finish_nvfp4(const FinishParams& q, hipStream_t st) { return launch_finish<FmtNvfp4>(q, st); }
int decode_token_layer_nvfp4(const FinishParams& q, hipStream_t st) { return launch_token_layer<FmtNvfp4>(q, st); }
}  // namespace ffmoe
