// Decode stages for FmtNvfp4 experts.
#include "finish_kernel.cuh"
#include "token_layer.cuh"

namespace ffmoe {
int decode_launch_nvfp4(const DecodeParams& p, int rg, int stage_mask, hipStream_t st) { return launch_format<FmtNvfp4>(p, rg, stage_mask, st); }
int decode_finish_nvfp4(const FinishParams& q, hipStream_t st) { return launch_finish<FmtNvfp4>(q, st); }
// the same with a BF16 shared expert, whose down rows the finish streams in their own format
int decode_finish_nvfp4_bf16_shared(const FinishParams& q, hipStream_t st) { return launch_finish<FmtNvfp4>(q, st, true); }
int decode_token_layer_nvfp4(const FinishParams& q, hipStream_t st) { return launch_token_layer<FmtNvfp4>(q, st); }

// One token, NVFP4 routed experts next to a BF16 shared expert: the gate/up launch with the selection in its prologue
// takes the shared expert's rows as every block's first slice, in BF16 (k_decode_stage's FSH / SSH). The step counts of
// both formats are template parameters, so the launch exists for the pairs of the common hidden sizes (2048, 4096, 7168,
// 8192); for any other size the caller keeps the shared expert's gate/up launch of its own.
static bool mixed_steps(int hidden, int* s_routed, int* s_shared) {
  auto steps_of = [](int k, int epl, int smax) {
    const int steps = (k / epl + 63) / 64;
    const int nslabs = (steps + smax - 1) / smax;
    return (steps + nslabs - 1) / nslabs;
  };
  *s_routed = steps_of(hidden, FmtNvfp4::EPL, Policy<FmtNvfp4>::S0);
  *s_shared = steps_of(hidden, FmtBf16::EPL, Policy<FmtBf16>::S0);
  const int a = *s_routed, b = *s_shared;
  return (a == 1 && b == 4) || (a == 2 && b == 8) || (a == 4 && b == 7) || (a == 4 && b == 8);
}
bool decode_gate_up_nvfp4_bf16_shared_available(int hidden) {
  int a, b;
  return mixed_steps(hidden, &a, &b);
}
int decode_gate_up_nvfp4_bf16_shared(const DecodeParams& p, hipStream_t st) {
  int a, b;
  if (!mixed_steps(p.hidden, &a, &b)) return ff_fail(FFMOE_ERR_UNSUPPORTED, "no mixed gate/up launch for hidden=%d", p.hidden);
  const size_t lds = size_t(p.hidden) * 2;
  const int blocks = decode_num_cus() * 2;
  constexpr int NR = Policy<FmtNvfp4>::NR0;
  static_assert(Policy<FmtNvfp4>::NR0 == Policy<FmtBf16>::NR0, "one unit shape for both formats");
  if (a == 1) hipLaunchKernelGGL((k_decode_stage<FmtNvfp4, 1, 0, 1, NR, FmtBf16, 4>), dim3(blocks), dim3(256), lds, st, p);
  else if (a == 2) hipLaunchKernelGGL((k_decode_stage<FmtNvfp4, 2, 0, 1, NR, FmtBf16, 8>), dim3(blocks), dim3(256), lds, st, p);
  else if (b == 7) hipLaunchKernelGGL((k_decode_stage<FmtNvfp4, 4, 0, 1, NR, FmtBf16, 7>), dim3(blocks), dim3(256), lds, st, p);
  else hipLaunchKernelGGL((k_decode_stage<FmtNvfp4, 4, 0, 1, NR, FmtBf16, 8>), dim3(blocks), dim3(256), lds, st, p);
  return ff_launch_status();
}
}  // namespace ffmoe
