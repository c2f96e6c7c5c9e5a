// Entry points of the E8M0 block-32 expert path (W4A8 routed experts, W8A8 shared expert, exact arithmetic); the
// kernels are in e8m0_kernel.cuh.
#include "e8m0_kernel.cuh"

using namespace ffmoe;

namespace {
struct E8m0Layout {
  uint64_t xq, xs, h, hq, hs, live, total;
};
E8m0Layout e8m0_layout(int rows, int top_k, int hidden, int inter, int shared_inter) {
  const uint64_t R = rows, A = uint64_t(rows) * top_k, S = A + R;
  const uint64_t imax = uint64_t(inter > shared_inter ? inter : shared_inter);
  auto up = [](uint64_t v) { return (v + 255) & ~uint64_t(255); };
  E8m0Layout l;
  uint64_t at = 0;
  l.xq = at; at = up(at + R * hidden);
  l.xs = at; at = up(at + R * (hidden / 32));
  l.h = at; at = up(at + S * imax * 2);
  l.hq = at; at = up(at + S * imax);
  l.hs = at; at = up(at + S * (imax / 32));
  l.live = at; at = up(at + S * 4);
  l.total = at;
  return l;
}
}  // namespace

extern "C" __attribute__((visibility("default"))) uint64_t ffmoe_e8m0_scratch_bytes(int rows, int top_k, int hidden, int inter, int shared_inter) {
  if (rows < 1 || top_k < 0 || hidden < 32 || inter < 32) return 0;
  return e8m0_layout(rows, top_k, hidden, inter, shared_inter).total;
}

extern "C" __attribute__((visibility("default"))) int ffmoe_act_quant_e8m0(const void* x, void* codes, void* scales, int rows, int k, void* stream) {
  FF_REQUIRE(x && codes && scales, FFMOE_ERR_NULL, "x/codes/scales is NULL");
  FF_REQUIRE(rows >= 1 && rows <= 65535 && k >= 32 && k % 32 == 0, FFMOE_ERR_SHAPE, "rows=%d k=%d: k must be a positive multiple of 32", rows, k);
  FF_PTR16(x); FF_PTR_ALIGNED(codes, 8);
  hipLaunchKernelGGL(k_act_quant_e8m0, dim3((k / 32 + 63) / 64, rows), dim3(256), 0, (hipStream_t)stream, (const uint16_t*)x, k, (uint8_t*)codes, k,
                     (uint8_t*)scales, k / 32, k, (const uint32_t*)nullptr);
  return ff_launch_status();
}

extern "C" __attribute__((visibility("default"))) int ffmoe_decode_contribute_e8m0(const ffmoe_expert_table* table, const ffmoe_shared_expert* shared,
                                                                                  const ffmoe_decode* args, void* stream) {
  FF_REQUIRE(table && args, FFMOE_ERR_NULL, "table/args is NULL");
  const int R = args->rows, K = args->top_k, E = table->experts, H = table->hidden, I = table->inter;
  FF_REQUIRE(table->format == FFMOE_FMT_E2M1_E8M0, FFMOE_ERR_UNSUPPORTED, "routed experts must be FFMOE_FMT_E2M1_E8M0 (format %d)", table->format);
  FF_REQUIRE(!shared || shared->format == FFMOE_FMT_E4M3_E8M0_32, FFMOE_ERR_UNSUPPORTED, "the shared expert must be FFMOE_FMT_E4M3_E8M0_32 (format %d)",
             shared ? shared->format : -1);
  FF_REQUIRE(R >= 1 && R <= 65535 && K >= 0 && (K >= 1 || shared) && K <= FFMOE_MAX_TOP_K && E >= 1 && E <= FFMOE_MAX_EXPERTS, FFMOE_ERR_SHAPE,
             "rows=%d top_k=%d experts=%d out of range", R, K, E);
  const int SI = shared ? shared->inter : I;
  FF_REQUIRE(H >= 32 && I >= 32 && SI >= 32 && H % 32 == 0 && I % 32 == 0 && SI % 32 == 0, FFMOE_ERR_SHAPE,
             "hidden=%d inter=%d shared inter=%d must be positive multiples of 32", H, I, SI);
  FF_REQUIRE(args->act_mode == FFMOE_ACT_E4M3_E8M0_32 || args->act_mode == FFMOE_ACT_E4M3_E8M0_32_F32, FFMOE_ERR_UNSUPPORTED,
             "act_mode %d: this path quantizes activations to E4M3 with E8M0 scales per 32", args->act_mode);
  const bool exact = args->act_mode == FFMOE_ACT_E4M3_E8M0_32;
  FF_REQUIRE(args->swiglu_limit > 0.0f && args->swiglu_limit < INFINITY, FFMOE_ERR_SHAPE, "the contract clamps the SwiGLU inputs: limit %g",
             (double)args->swiglu_limit);
  FF_REQUIRE(args->routed_weight == FFMOE_WEIGHT_BEFORE_DOWN_F32 && args->weights_f32 == 1, FFMOE_ERR_UNSUPPORTED,
             "the routed weight is an f32 applied before the down projection (FFMOE_WEIGHT_BEFORE_DOWN_F32)");
  FF_PTR16(args->x); FF_PTR4(args->ids); FF_PTR4(args->weights); FF_PTR16(args->contributions); FF_PTR16(table->slots);
  if (shared) {
    FF_PTR16(args->shared_out);
    for (int i = 0; i < 6; ++i)
      FF_REQUIRE(shared->slot[i] != 0 && (i % 2 == 1 || shared->slot[i] % 16 == 0), FFMOE_ERR_ALIGN, "shared expert slot[%d] is NULL or misaligned", i);
  }
  if (args->done) FF_PTR4(args->done);
  const E8m0Layout l = e8m0_layout(R, K, H, I, shared ? SI : 0);
  FF_PTR_ALIGNED(args->scratch, 256);
  FF_REQUIRE(args->scratch_bytes >= l.total, FFMOE_ERR_SCRATCH, "scratch holds %llu bytes, %llu needed (ffmoe_e8m0_scratch_bytes)",
             (unsigned long long)args->scratch_bytes, (unsigned long long)l.total);
  const int imax = I > (shared ? SI : 0) ? I : SI;
  FF_REQUIRE(size_t((H > imax ? H : imax) / 32) * 33 * 4 <= 64 * 1024, FFMOE_ERR_SHAPE, "a row of %d activations does not fit the LDS staging", H > imax ? H : imax);
  uint8_t* sc = (uint8_t*)args->scratch;
  E8m0Params q;
  DecodeParams& p = q.d;
  p.route = RouteInline{nullptr, nullptr, 0, 1, 1, 1.0f};
  p.rows = R; p.top_k = K; p.experts = E; p.hidden = H; p.inter = I; p.shared_inter = SI; p.has_shared = shared ? 1 : 0;
  p.swiglu = FFMOE_SWIGLU_CLAMPED_ONCE; p.routed_weight = args->routed_weight; p.weights_f32 = 1; p.swiglu_limit = args->swiglu_limit;
  p.x = (const uint16_t*)args->x; p.ids = args->ids; p.active = args->active; p.weights = args->weights;
  p.slots = table->slots; p.valid = table->valid; p.generation = table->generation; p.assignment_gen = args->assignment_gen;
  p.global_scales = nullptr;
  for (int i = 0; i < 6; ++i) p.shared_slot[i] = shared ? shared->slot[i] : 0;
  for (int i = 0; i < 3; ++i) p.shared_global[i] = 1.0f;
  p.contributions = (uint16_t*)args->contributions; p.shared_out = (uint16_t*)args->shared_out; p.done = args->done;
  p.h = (uint16_t*)(sc + l.h); p.h_stride = imax; p.groups = nullptr; p.counters = nullptr;
  q.xq = sc + l.xq; q.xs = sc + l.xs; q.hq = sc + l.hq; q.hs = sc + l.hs;
  uint32_t* live = (uint32_t*)(sc + l.live);
  hipStream_t st = (hipStream_t)stream;
  const int S = R * K + R;
  hipLaunchKernelGGL(k_act_quant_e8m0, dim3((H / 32 + 63) / 64, R), dim3(256), 0, st, p.x, H, sc + l.xq, H, sc + l.xs, H / 32, H, (const uint32_t*)nullptr);
  hipLaunchKernelGGL(k_e8m0_live, dim3((S + 255) / 256), dim3(256), 0, st, p, live);
  if (exact) hipLaunchKernelGGL((k_e8m0_stage<0>), dim3((imax + 7) / 8, R, K + 1), dim3(256), size_t(H / 32) * 33 * 4, st, q);
  else hipLaunchKernelGGL((k_e8m0_stage_f32<0>), dim3((imax + 7) / 8, R, K + 1), dim3(256), size_t(H) * 4 + size_t(H / 32) * 4, st, q);
  FF_TRY(ff_launch_status());
  // every live down-input row is quantized over imax elements (a shorter row leaves its tail unused)
  if (K > 0)
    hipLaunchKernelGGL(k_act_quant_e8m0, dim3((I / 32 + 63) / 64, R * K), dim3(256), 0, st, p.h, imax, sc + l.hq, imax, sc + l.hs, imax / 32, I,
                       (const uint32_t*)live);
  if (shared)
    hipLaunchKernelGGL(k_act_quant_e8m0, dim3((SI / 32 + 63) / 64, R), dim3(256), 0, st, p.h + size_t(R) * K * imax, imax,
                       sc + l.hq + size_t(R) * K * imax, imax, sc + l.hs + size_t(R) * K * (imax / 32), imax / 32, SI, (const uint32_t*)(live + R * K));
  if (exact) hipLaunchKernelGGL((k_e8m0_stage<1>), dim3((H + 7) / 8, R, K + 1), dim3(256), size_t(imax / 32) * 33 * 4, st, q);
  else hipLaunchKernelGGL((k_e8m0_stage_f32<1>), dim3((H + 7) / 8, R, K + 1), dim3(256), size_t(imax) * 4 + size_t(imax / 32) * 4, st, q);
  return ff_launch_status();
}
