// Decode expert FFN in the reference's Lane16 / Lane8 reduction orders (form_kernel.cuh) for the BF16 and per-channel
// FP8 expert formats.
#include "form_kernel.cuh"

namespace ffmoe {
int decode_form_launch(int fmt, int form, const DecodeParams& p, int stage_mask, hipStream_t st) {
  if (fmt == FFMOE_FMT_BF16)
    return form == FFMOE_FORM_LANE16 ? launch_form<FmtBf16, FFMOE_FORM_LANE16_>(p, stage_mask, st) : launch_form<FmtBf16, FFMOE_FORM_LANE8_>(p, stage_mask, st);
  return form == FFMOE_FORM_LANE16 ? launch_form<FmtFp8Channel, FFMOE_FORM_LANE16_>(p, stage_mask, st)
                                   : launch_form<FmtFp8Channel, FFMOE_FORM_LANE8_>(p, stage_mask, st);
}
}  // namespace ffmoe
