// Decode stages for FmtFp8Channel experts (E4M3 codes, one BF16 scale per output row).
#include "finish_kernel.cuh"
#include "token_layer.cuh"

namespace ffmoe {
int decode_launch_fp8c(const DecodeParams& p, int rg, int stage_mask, hipStream_t st) { return launch_format<FmtFp8Channel>(p, rg, stage_mask, st); }
int decode_finish_fp8c(const FinishParams& q, hipStream_t st) { return launch_finish<FmtFp8Channel>(q, st); }
int decode_token_layer_fp8c(const FinishParams& q, hipStream_t st) { return launch_token_layer<FmtFp8Channel>(q, st); }
}  // namespace ffmoe
