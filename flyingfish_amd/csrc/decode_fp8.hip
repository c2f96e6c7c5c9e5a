// Decode stages for FmtFp8 experts.
#include "finish_kernel.cuh"
#include "token_layer.cuh"

namespace ffmoe {
int decode_launch_fp8(const DecodeParams& p, int rg, int stage_mask, hipStream_t st) { return launch_format<FmtFp8>(p, rg, stage_mask, st); }
int decode_finish_fp8(const FinishParams& q, hipStream_t st) { return launch_finish<FmtFp8>(q, st); }
int decode_token_layer_fp8(const FinishParams& q, hipStream_t st) { return launch_token_layer<FmtFp8>(q, st); }
}  // namespace ffmoe
