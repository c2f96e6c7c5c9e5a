// Decode stages for FmtBf16 experts.
#include "finish_kernel.cuh"
#include "token_layer.cuh"

namespace ffmoe {
int decode_launch_bf16(const DecodeParams& p, int rg, int stage_mask, hipStream_t st) { return launch_format<FmtBf16>(p, rg, stage_mask, st); }
int decode_finish_bf16(const FinishParams& q, hipStream_t st) { return launch_finish<FmtBf16>(q, st); }
int decode_token_layer_bf16(const FinishParams& q, hipStream_t st) { return launch_token_layer<FmtBf16>(q, st); }
}  // namespace ffmoe
