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

template <class F>
static int form_grouped_fmt(int form, int rg, const DecodeParams& p, unsigned max_groups, int stage_mask, hipStream_t st) {
  const bool l16 = form == FFMOE_FORM_LANE16;
  switch (rg) {
    case 8: return l16 ? launch_form_grouped<F, FFMOE_FORM_LANE16_, 8>(p, max_groups, stage_mask, st) : launch_form_grouped<F, FFMOE_FORM_LANE8_, 8>(p, max_groups, stage_mask, st);
    case 4: return l16 ? launch_form_grouped<F, FFMOE_FORM_LANE16_, 4>(p, max_groups, stage_mask, st) : launch_form_grouped<F, FFMOE_FORM_LANE8_, 4>(p, max_groups, stage_mask, st);
    default: return l16 ? launch_form_grouped<F, FFMOE_FORM_LANE16_, 2>(p, max_groups, stage_mask, st) : launch_form_grouped<F, FFMOE_FORM_LANE8_, 2>(p, max_groups, stage_mask, st);
  }
}
// groups of rg = 2, 4 or 8 assignments per expert (p.groups / p.counters filled by k_group_assignments)
int decode_form_grouped_launch(int fmt, int form, int rg, const DecodeParams& p, unsigned max_groups, int stage_mask, hipStream_t st) {
  if (fmt == FFMOE_FMT_BF16) return form_grouped_fmt<FmtBf16>(form, rg, p, max_groups, stage_mask, st);
  return form_grouped_fmt<FmtFp8Channel>(form, rg, p, max_groups, stage_mask, st);
}
}  // namespace ffmoe
