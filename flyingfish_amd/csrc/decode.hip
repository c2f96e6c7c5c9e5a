// Decode expert contribution: entry points, argument checks and the kernel that groups assignments by expert.
// The streaming kernels live in decode_kernel.cuh and are instantiated per weight format.
#include "common.cuh"
#include "api.h"
#include "decode.h"
#include <atomic>
#include <stdlib.h>

namespace ffmoe {

int decode_launch_fp8(const DecodeParams& p, int rg, int stage_mask, hipStream_t st);
int decode_launch_nvfp4(const DecodeParams& p, int rg, int stage_mask, hipStream_t st);
int decode_launch_bf16(const DecodeParams& p, int rg, int stage_mask, hipStream_t st);
int decode_launch_fp8c(const DecodeParams& p, int rg, int stage_mask, hipStream_t st);
bool decode_gate_up_nvfp4_bf16_shared_available(int hidden);
int decode_gate_up_nvfp4_bf16_shared(const DecodeParams& p, hipStream_t st);
int decode_finish_fp8(const FinishParams& q, hipStream_t st);
int decode_finish_nvfp4(const FinishParams& q, hipStream_t st);
int decode_finish_nvfp4_bf16_shared(const FinishParams& q, hipStream_t st);
int decode_finish_bf16(const FinishParams& q, hipStream_t st);
int decode_finish_fp8c(const FinishParams& q, hipStream_t st);
int decode_token_layer_fp8(const FinishParams& q, hipStream_t st);
int decode_token_layer_nvfp4(const FinishParams& q, hipStream_t st);
int decode_token_layer_bf16(const FinishParams& q, hipStream_t st);
int decode_token_layer_fp8c(const FinishParams& q, hipStream_t st);
int decode_form_launch(int fmt, int form, const DecodeParams& p, int stage_mask, hipStream_t st);
int decode_form_grouped_launch(int fmt, int form, int rg, const DecodeParams& p, unsigned max_groups, int stage_mask, hipStream_t st);
int prefill_impl(const ffmoe_expert_table* table, const ffmoe_prefill* args, int stages, void* stream);
int shared_expert_w16(const ffmoe_shared_expert* shared, const void* x, int R, int H, int swiglu, float limit, void* act, void* shared_out,
                      int stage_mask, void* stream_);
}  // namespace ffmoe

namespace ffmoe {

// Device-side state of the one-launch token layer, zero when the module is loaded: 16 slots of {exit counter, 128 claim
// counters}, every counter on its own 128-byte line. Calls take slots round-robin and get their activation tag from the
// same host-side ticket, so launches in flight on different streams share neither counters nor a tag. Every launch
// leaves its slot at zero.
#define FFMOE_TOKEN_SLOTS 16
#define FFMOE_TOKEN_SLOT_WORDS (129 * 32)
static __device__ __align__(256) unsigned int g_token_state[32 + FFMOE_TOKEN_SLOTS * FFMOE_TOKEN_SLOT_WORDS];

static bool token_layer_sync(FinishParams* q) {
  static std::atomic<unsigned int*> base[16];
  static std::atomic<unsigned int> next{0};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 16) return false;
  unsigned int* b = base[dev].load(std::memory_order_acquire);
  if (!b) {
    if (hipGetSymbolAddress((void**)&b, HIP_SYMBOL(g_token_state)) != hipSuccess || !b) {
      (void)hipGetLastError();
      return false;
    }
    base[dev].store(b, std::memory_order_release);
  }
  const char* le = getenv("FFMOE_TOKEN_SPIN_LIMIT");  // read per call, so a process can change it
  const unsigned int limit = le ? (unsigned int)strtoul(le, nullptr, 10) : 100000u;
  const unsigned int ticket = next.fetch_add(1, std::memory_order_relaxed);
  const unsigned int slot = ticket % FFMOE_TOKEN_SLOTS;
  q->tag = 1u + ticket % 65535u;
  q->exited = b + 32 + slot * FFMOE_TOKEN_SLOT_WORDS;
  q->claims = q->exited + 32;
  q->spin_limit = limit;
  static const int dynamic = [] { const char* e = getenv("FFMOE_TOKEN_STATIC"); return (e && e[0] == '1') ? 0 : 1; }();
  q->dynamic = dynamic;
  return true;
}

// ---------------------------------------------------------------------------------------------
// Gather assignments by expert into groups of at most RGMAX rows (single block; A <= FFMOE_DECODE_MAX_ASSIGN).
// Groups are ordered by expert id, rows inside a group by assignment index, so the result does not
// depend on scheduling. counters[0] = routed groups, counters[1] = shared groups.
__global__ __launch_bounds__(1024) void k_group_assignments(const int* __restrict__ ids, const uint32_t* __restrict__ active,
                                                            const uint32_t* __restrict__ valid, const uint64_t* __restrict__ generation,
                                                            const uint64_t* __restrict__ assignment_gen,
                                                            GroupDesc* __restrict__ groups, int* __restrict__ counters,
                                                            int rows, int top_k, int experts, int has_shared, int rgmax) {
  extern __shared__ int s_ids[];  // [A] expert id or -1
  __shared__ int s_scan[FFMOE_MAX_EXPERTS];
  const int tid = threadIdx.x;
  const int A = rows * top_k;
  for (int a = tid; a < A; a += blockDim.x) {
    int e = (!active || active[a]) ? ids[a] : -1;
    if ((unsigned)e >= (unsigned)experts || (valid && valid[e] == 0u)) e = -1;
    else if (generation && assignment_gen && generation[e] != assignment_gen[a]) e = -1;  // stale choice
    s_ids[a] = e;
  }
  __syncthreads();
  int cnt = 0;
  if (tid < experts)
    for (int a = 0; a < A; ++a) cnt += s_ids[a] == tid;
  const int chunks = (cnt + rgmax - 1) / rgmax;
  // inclusive scan over experts (blockDim == 1024 >= experts)
  s_scan[tid] = tid < experts ? chunks : 0;
  __syncthreads();
  for (int off = 1; off < 1024; off <<= 1) {
    const int v = tid >= off ? s_scan[tid - off] : 0;
    __syncthreads();
    s_scan[tid] += v;
    __syncthreads();
  }
  const int base = s_scan[tid] - chunks;
  const int n_routed = s_scan[1023];
  if (tid < experts && cnt > 0) {
    int filled = 0, gi = base;
    for (int a = 0; a < A; ++a) {
      if (s_ids[a] != tid) continue;
      GroupDesc& gd = groups[gi];
      if (filled == 0) { gd.expert = tid; gd.n = cnt - (gi - base) * rgmax < rgmax ? cnt - (gi - base) * rgmax : rgmax; }
      gd.row[filled] = a / top_k;
      gd.slot[filled] = a;
      if (++filled == rgmax) { filled = 0; ++gi; }
    }
  }
  const int n_shared = has_shared ? (rows + rgmax - 1) / rgmax : 0;
  for (int t = tid; t < n_shared; t += blockDim.x) {
    GroupDesc& gd = groups[n_routed + t];
    gd.expert = -1;
    const int r0 = t * rgmax;
    gd.n = rows - r0 < rgmax ? rows - r0 : rgmax;
    for (int r = 0; r < gd.n; ++r) { gd.row[r] = r0 + r; gd.slot[r] = A + r0 + r; }
  }
  if (tid == 0) { counters[0] = n_routed; counters[1] = n_shared; }
}

}  // namespace ffmoe

using namespace ffmoe;


extern "C" __attribute__((visibility("default"))) uint64_t ffmoe_decode_scratch_bytes(int rows, int top_k, int experts, int hidden, int inter, int shared_inter) {
  (void)hidden;
  if (rows < 1 || top_k < 1 || experts < 1 || inter < 1) return 0;
  const uint64_t A = uint64_t(rows) * top_k;
  const uint64_t imax = uint64_t(inter > shared_inter ? inter : shared_inter);
  // one token: the one-launch layer keeps its activations as 32-bit tagged words
  const uint64_t h = ((A + rows) * imax * (rows == 1 ? 4 : 2) + 255) & ~uint64_t(255);
  (void)experts;
  const uint64_t max_groups = A + rows + 2;  // worst case: one row per group
  const uint64_t groups = (max_groups * sizeof(GroupDesc) + 255) & ~uint64_t(255);
  // FFMOE_ACT_FP8_BLOCK128 runs on the grouped matrix-core path, which lays the arena out differently
  const uint64_t w8a8 = ffmoe_prefill_scratch_bytes(rows, top_k, experts, hidden, inter, shared_inter);
  // a shared expert served by the matrix-core path (large batches) keeps its activations behind the decode arena
  const uint64_t shared_act = shared_inter > 0 ? ((uint64_t(rows) * shared_inter * 2 + 255) & ~uint64_t(255)) : 0;
  const uint64_t own = h + groups + 256 + shared_act;
  uint64_t need = own > w8a8 ? own : w8a8;
  // a cohort of routed experts on the matrix cores with a shared expert of another format on the streaming kernels: the
  // shared pass gets an arena of its own behind the cohort's, so the two may also be issued stage by stage
  if (shared_inter > 0) {
    const uint64_t routed = ffmoe_prefill_scratch_bytes(rows, top_k, experts, hidden, inter, 0);
    const uint64_t mixed = routed + (top_k == 1 ? need : ffmoe_decode_scratch_bytes(rows, 1, experts, hidden, inter, shared_inter));
    if (top_k > 1 && mixed > need) need = mixed;
  }
  return need;
}

// layout_k >= 0: the call processes args->top_k choices per row (0 = the shared expert only) but lays the scratch
// arena out for layout_k choices and for rows of max(inter, shared inter, arena_shared_inter) activations, so a routed
// pass and a shared pass of another weight format share one arena with the same row stride and the same offsets.
// Pass 1 keeps its group descriptors and counters behind those of pass 0: the passes may be issued stage by stage
// (both gate/up launches, then both down launches), so neither may overwrite the other's grouping.
static int decode_impl(const ffmoe_expert_table* table, const ffmoe_shared_expert* shared, const ffmoe_decode* args,
                       int stage_mask, void* stream, int layout_k = -1, int pass = 0, const FinishParams* fin = nullptr,
                       const RouteInline* route = nullptr, int form = -1, int arena_shared_inter = 0, bool mixed_gate_up = false,
                       bool finish_record = false, bool mixed_finish = false) {
  FF_REQUIRE(table && args, FFMOE_ERR_NULL, "table/args is NULL");
  const int R = args->rows, K = args->top_k, E = table->experts, H = table->hidden, I = table->inter;
  const int LK = layout_k < 0 ? K : layout_k;
  FF_REQUIRE(R >= 1 && K >= 0 && (K >= 1 || shared) && K <= FFMOE_MAX_TOP_K && LK >= K && E >= 1 && E <= FFMOE_MAX_EXPERTS, FFMOE_ERR_SHAPE,
             "decode rows=%d top_k=%d experts=%d out of range", R, K, E);
  // the reduction-order kernels take one launch block per (row, choice) and no grouping pass: any cohort the grid holds
  if (form < 0)
    FF_REQUIRE((long long)R * K <= FFMOE_DECODE_MAX_ASSIGN, FFMOE_ERR_SHAPE,
               "decode handles at most %d assignments per call (got %lld); use ffmoe_prefill_contribute", FFMOE_DECODE_MAX_ASSIGN,
               (long long)R * K);
  const int fmt = table->format;
  FF_REQUIRE(fmt == FFMOE_FMT_FP8_BLOCK128 || fmt == FFMOE_FMT_NVFP4 || fmt == FFMOE_FMT_BF16 || fmt == FFMOE_FMT_FP8_CHANNEL, FFMOE_ERR_UNSUPPORTED,
             "unknown expert format %d", fmt);
  // every format's granule is a multiple of 4, the largest number of output rows a wave handles per unit
  const int gran = fmt == FFMOE_FMT_FP8_BLOCK128 ? 128 : (fmt == FFMOE_FMT_NVFP4 ? 32 : (fmt == FFMOE_FMT_FP8_CHANNEL ? 16 : 8));
  FF_REQUIRE(H >= gran && I >= gran && H % gran == 0 && I % gran == 0, FFMOE_ERR_SHAPE,
             "hidden=%d inter=%d must be positive multiples of %d for this format", H, I, gran);
  FF_REQUIRE(args->act_mode == FFMOE_ACT_BF16, FFMOE_ERR_UNSUPPORTED,
             "decode act_mode %d is not implemented (only FFMOE_ACT_BF16)", args->act_mode);
  FF_REQUIRE(args->swiglu >= 0 && args->swiglu <= FFMOE_SWIGLU_GELU_TWICE, FFMOE_ERR_UNSUPPORTED, "unknown SwiGLU mode %d", args->swiglu);
  if (args->swiglu == FFMOE_SWIGLU_CLAMPED_TWICE || args->swiglu == FFMOE_SWIGLU_CLAMPED_ONCE)
    FF_REQUIRE(args->swiglu_limit > 0.0f && args->swiglu_limit < INFINITY, FFMOE_ERR_SHAPE, "invalid SwiGLU limit %g",
               (double)args->swiglu_limit);
  FF_REQUIRE(args->routed_weight == 0 || args->routed_weight == 1, FFMOE_ERR_UNSUPPORTED, "unknown routed-weight boundary %d",
             args->routed_weight);
  FF_PTR16(args->x); FF_PTR4(args->ids); FF_PTR16(args->contributions); FF_PTR16(table->slots);
  if (args->weights_f32) { FF_PTR4(args->weights); } else { FF_PTR2(args->weights); }
  if (fmt == FFMOE_FMT_NVFP4 && K > 0) FF_PTR4(table->global_scales);
  int SI = I;
  if (shared) {
    // mixed_gate_up: NVFP4 experts and a BF16 shared expert in one gate/up launch (one token, selection in the prologue)
    // mixed_finish: the same pair in the one-token finish launch
    FF_REQUIRE(shared->format == fmt || (mixed_gate_up && fmt == FFMOE_FMT_NVFP4 && shared->format == FFMOE_FMT_BF16 && route && stage_mask == 1) ||
                   (mixed_finish && fmt == FFMOE_FMT_NVFP4 && shared->format == FFMOE_FMT_BF16 && fin && !fin->whole && R == 1),
               FFMOE_ERR_UNSUPPORTED, "shared expert format %d differs from the table format %d", shared->format, fmt);
    SI = shared->inter;
    FF_REQUIRE(SI >= gran && SI % gran == 0, FFMOE_ERR_SHAPE, "shared inter=%d must be a positive multiple of %d", SI, gran);
    FF_PTR16(args->shared_out);
    for (int i = 0; i < 6; i += 2)
      FF_REQUIRE(shared->slot[i] != 0 && shared->slot[i] % 16 == 0, FFMOE_ERR_ALIGN, "shared expert slot[%d] is NULL or misaligned", i);
  }
  const int arena_si = shared ? (SI > arena_shared_inter ? SI : arena_shared_inter) : arena_shared_inter;
  const uint64_t need = ffmoe_decode_scratch_bytes(R, LK > 0 ? LK : 1, E, H, I, arena_si);
  FF_PTR_ALIGNED(args->scratch, 256);
  FF_REQUIRE(args->scratch_bytes >= need, FFMOE_ERR_SCRATCH, "decode scratch holds %llu bytes, %llu needed",
             (unsigned long long)args->scratch_bytes, (unsigned long long)need);
  const size_t A = size_t(R) * K;
  const size_t xb = size_t(R) * H * 2, cb = A * H * 2;
  FF_NO_OVERLAP(args->contributions, cb, args->x, xb);
  FF_NO_OVERLAP(args->contributions, cb, args->ids, A * 4);
  FF_NO_OVERLAP(args->contributions, cb, args->weights, A * (args->weights_f32 ? 4 : 2));
  FF_NO_OVERLAP(args->contributions, cb, args->scratch, args->scratch_bytes);
  FF_NO_OVERLAP(args->scratch, args->scratch_bytes, args->x, xb);
  if (shared) {
    FF_NO_OVERLAP(args->shared_out, xb, args->x, xb);
    FF_NO_OVERLAP(args->shared_out, xb, args->contributions, cb);
    FF_NO_OVERLAP(args->shared_out, xb, args->scratch, args->scratch_bytes);
  }
  if (args->done) {
    FF_PTR4(args->done);
    FF_NO_OVERLAP(args->done, A * 4, args->contributions, cb);
    FF_NO_OVERLAP(args->done, A * 4, args->scratch, args->scratch_bytes);
  }

  const int imax = I > arena_si ? I : arena_si;
  const int kmax_lds = H > imax ? H : imax;
  FF_REQUIRE(size_t(kmax_lds) * 2 <= 160 * 1024 / 2, FFMOE_ERR_SHAPE, "row of %d BF16 does not fit the LDS staging", kmax_lds);

  DecodeParams p;
  p.route = route ? *route : RouteInline{nullptr, nullptr, 0, 1, 1, 1.0f, 0};
  p.rows = R; p.top_k = K; p.experts = E; p.hidden = H; p.inter = I; p.shared_inter = SI;
  p.has_shared = shared ? 1 : 0;
  p.swiglu = args->swiglu; p.swiglu_limit = args->swiglu_limit; p.routed_weight = args->routed_weight;
  p.weights_f32 = args->weights_f32;
  p.x = (const uint16_t*)args->x; p.ids = args->ids; p.active = args->active; p.weights = args->weights;
  p.slots = table->slots; p.valid = table->valid; p.global_scales = table->global_scales;
  p.generation = table->generation; p.assignment_gen = args->assignment_gen;
  if (p.generation) FF_PTR_ALIGNED(p.generation, 8);
  if (p.assignment_gen) FF_PTR_ALIGNED(p.assignment_gen, 8);
  for (int i = 0; i < 6; ++i) p.shared_slot[i] = shared ? shared->slot[i] : 0;
  for (int i = 0; i < 3; ++i) p.shared_global[i] = shared ? shared->global_scales[i] : 1.0f;
  p.contributions = (uint16_t*)args->contributions; p.shared_out = (uint16_t*)args->shared_out; p.done = args->done;
  uint8_t* sc = (uint8_t*)args->scratch;
  const size_t LA = size_t(R) * LK;
  p.h = (uint16_t*)sc + (LA - A) * imax;  // slot s of this call -> arena row (LA - A) + s
  p.h_stride = imax;
  const uint64_t hbytes = ((uint64_t(LA) + R) * imax * 2 + 255) & ~uint64_t(255);
  hipStream_t st = (hipStream_t)stream;
  if (form >= 0) {
    // The reference's reduction orders. Several rows: assignments sorted by expert into groups that share one pass over
    // the expert's weights (the same bits as one block per (row, choice), which one row, cohorts beyond the grouping
    // kernel's LDS and FFMOE_FORM_GROUPED=0 keep).
    int frg = FFMOE_DECODE_RG;
    while (frg > 1 && size_t(frg) * kmax_lds * 2 > 64 * 1024) frg >>= 1;
    const bool can_group = R > 1 && frg > 1 && size_t(A) * sizeof(int) <= 64 * 1024 && uint64_t(LA) + R + 2 <= 65535;
    // it pays from about two rows per expert on (per-channel FP8, hidden 4096, 32 experts top-4: 64 rows 0.89 against
    // 1.56 ms in the Lane16 order, 512 rows 3.6 against 13.0 ms; 8 rows 0.41 against 0.30 ms)
    bool grouped = can_group && A >= 2 * E;
    if (const char* f = getenv("FFMOE_FORM_GROUPED")) grouped = can_group && atoi(f) != 0;
    if (!grouped) {
      p.groups = nullptr;
      p.counters = nullptr;
      return decode_form_launch(fmt, form, p, stage_mask, st);
    }
    p.groups = (GroupDesc*)(sc + hbytes);
    const uint64_t max_groups = uint64_t(LA) + R + 2;
    p.counters = (int*)(sc + hbytes + ((max_groups * sizeof(GroupDesc) + 255) & ~uint64_t(255)));
    if (stage_mask & 1) hipLaunchKernelGGL(k_group_assignments, dim3(1), dim3(1024), A * sizeof(int), st, args->ids, args->active, table->valid, p.generation,
                                           p.assignment_gen, p.groups, p.counters, R, K, E, p.has_shared, frg);
    FF_TRY(ff_launch_status());
    // at most one group per assignment and per shared row, so A + R bounds what the counters can hold
    return decode_form_grouped_launch(fmt, form, frg, p, unsigned(A + R), stage_mask, st);
  }
  int rg = 1;
  // LDS budget per block: rg rows of the widest contraction; two blocks per CU must fit in 160 KiB
  if (R > 1) {
    rg = FFMOE_DECODE_RG;
    while (rg > 1 && size_t(rg) * kmax_lds * 2 > 64 * 1024) rg >>= 1;
  }
  if (rg > 1) {
    p.groups = (GroupDesc*)(sc + hbytes) + (pass ? LA + 1 : 0);
    const uint64_t max_groups = uint64_t(LA) + R + 2;
    p.counters = (int*)(sc + hbytes + ((max_groups * sizeof(GroupDesc) + 255) & ~uint64_t(255))) + 2 * pass;
    if (stage_mask & 1) hipLaunchKernelGGL(k_group_assignments, dim3(1), dim3(1024), A * sizeof(int), st, args->ids, args->active, table->valid, p.generation, p.assignment_gen, p.groups,
                       p.counters, R, K, E, p.has_shared, rg);
    FF_TRY(ff_launch_status());
  } else {
    p.groups = nullptr;
    p.counters = nullptr;
    // one row: the group tables are unused, and the gate/up launch with the selection in its prologue leaves the record
    // of the live choices there for the finish launch of the same call
    if (finish_record) p.route.finish_desc = (FinishDesc*)(sc + hbytes);
  }
  if (fin) {
    FinishParams q = *fin;
    q.d = p;
    q.d.route.finish_desc = nullptr;
    q.desc = finish_record && rg == 1 ? (const FinishDesc*)(sc + hbytes) : nullptr;
    if (q.whole) {
      if (!token_layer_sync(&q)) return ff_fail(FFMOE_ERR_UNSUPPORTED, "one-launch token layer: no device counters on this device");
      q.h32 = (uint32_t*)sc;
      q.d.h_stride = imax;
      switch (fmt) {
        case FFMOE_FMT_FP8_BLOCK128: return decode_token_layer_fp8(q, st);
        case FFMOE_FMT_NVFP4: return decode_token_layer_nvfp4(q, st);
        case FFMOE_FMT_FP8_CHANNEL: return decode_token_layer_fp8c(q, st);
        default: return decode_token_layer_bf16(q, st);
      }
    }
    if (mixed_finish) return decode_finish_nvfp4_bf16_shared(q, st);
    switch (fmt) {
      case FFMOE_FMT_FP8_BLOCK128: return decode_finish_fp8(q, st);
      case FFMOE_FMT_NVFP4: return decode_finish_nvfp4(q, st);
      case FFMOE_FMT_FP8_CHANNEL: return decode_finish_fp8c(q, st);
      default: return decode_finish_bf16(q, st);
    }
  }
  if (mixed_gate_up) return decode_gate_up_nvfp4_bf16_shared(p, st);
  switch (fmt) {
    case FFMOE_FMT_FP8_BLOCK128: return decode_launch_fp8(p, rg, stage_mask, st);
    case FFMOE_FMT_NVFP4: return decode_launch_nvfp4(p, rg, stage_mask, st);
    case FFMOE_FMT_FP8_CHANNEL: return decode_launch_fp8c(p, rg, stage_mask, st);
    default: return decode_launch_bf16(p, rg, stage_mask, st);
  }
}

// A shared expert stored in another weight format than the routed experts (NVFP4 experts next to a BF16 shared expert)
// runs as two passes over one arena: the routed choices with the table's kernels, then the shared expert alone with the
// kernels of its own format.
static int decode_dispatch(const ffmoe_expert_table* table, const ffmoe_shared_expert* shared, const ffmoe_decode* args,
                           int stage_mask, void* stream) {
  if (table && args && args->act_mode == FFMOE_ACT_FP8_BLOCK128) {
    // W8A8 (the reference's block-F32 model path, kernels/moe_ffn.cu:870-908): activations are quantized per 128 and
    // the dot products run on the FP8 matrix cores through the grouped kernels of the prefill path, whatever the
    // row count; the shared expert goes through the same kernels as one dense group.
    ffmoe_prefill pf{};
    pf.rows = args->rows; pf.top_k = args->top_k; pf.act_mode = args->act_mode;
    pf.swiglu = args->swiglu; pf.swiglu_limit = args->swiglu_limit; pf.routed_weight = args->routed_weight; pf.weights_f32 = args->weights_f32;
    pf.x = args->x; pf.ids = args->ids; pf.active = args->active; pf.weights = args->weights;
    pf.contributions = args->contributions; pf.done = args->done; pf.scratch = args->scratch; pf.scratch_bytes = args->scratch_bytes;
    pf.shared = shared; pf.shared_out = args->shared_out; pf.assignment_gen = args->assignment_gen;
    return prefill_impl(table, &pf, (stage_mask & 1 ? 3 : 0) | (stage_mask & 2 ? 12 : 0), stream);
  }
  // Row counts from which the matrix-core cohort kernels take over for block-FP8 experts (same effective weights and BF16
  // boundaries, the dot products in the matrix instruction's FP32 order instead of the wave's). The whole batch goes there
  // from FFMOE_DECODE_COHORT_ROWS on: 3 when a block-FP8 shared expert rides in the routed launches (same format and width, or no
  // shared expert; with the four-block line kernel: 2 rows 186 / 166 us, 3 rows 220 / 235, 4 rows 264 / 312), 32 when it needs
  // launches of its own, a few dozen blocks each. Per layer at hidden 7168 / 256 experts
  // with a riding shared expert, cohort (whole-line kernel) against streaming kernels: 2 rows 200 / 166 us, 3 rows 236 / 235,
  // 4 rows 277 / 313, 6 rows 368 / 433, 8 rows 485 / 554, 16 rows 810 / 939, 32 rows 1278 / 1550, 64 rows 1730 / 2402. Below
  // that a block-FP8 shared expert alone from FFMOE_DECODE_SHARED_COHORT_ROWS on (it has every row: streamed once instead of
  // once per row group that fits LDS).
  // NVFP4 experts whose rows are whole 128-byte lines of codes (hidden and inter multiples of 256) take the line-wise
  // cohort kernel from FFMOE_DECODE_COHORT_ROWS on as well (4 rows 266 / 282 us, 6 rows 352 / 406); next to them a shared expert of another format stays on the
  // streaming kernels up to FFMOE_DECODE_SHARED_STREAM_ROWS = 24 rows and runs on one-wave blocks on the matrix cores
  // beyond (BF16 next to NVFP4 experts at hidden 7168, streaming against matrix cores: 16 rows 725 / 736 us per layer, 32 rows
  // 1123 / 1109, 64 rows 1524 / 1489) and gets an arena of its own behind the cohort's.
  // (0 switches a rule off; read at every call)
  const char* ce = getenv("FFMOE_DECODE_COHORT_ROWS");
  const char* se = getenv("FFMOE_DECODE_SHARED_COHORT_ROWS");
  const char* te = getenv("FFMOE_DECODE_SHARED_STREAM_ROWS");
  const bool rides = !shared || (table && shared->format == table->format && shared->inter == table->inter);
  const bool nv_lines = table && table->format == FFMOE_FMT_NVFP4 && table->hidden % 256 == 0 && table->inter % 256 == 0;
  const bool fp8_rides = rides && table && table->format == FFMOE_FMT_FP8_BLOCK128;
  const int cohort_rows = ce ? atoi(ce) : (fp8_rides ? 3 : (rides || nv_lines ? 4 : 32)), shared_rows = se ? atoi(se) : 16;
  // a BF16 shared expert that the split-contraction kernel takes (dense_splitk.cuh) leaves the streaming kernels with the
  // routed choices, at 4 rows: hidden 7168 next to NVFP4 experts, 4 / 8 / 16 / 24 rows: 249 / 413 / 665 / 859 us per layer
  // against 263 / 434 / 691 / 917 with the shared expert streaming
  const char* ke = getenv("FFMOE_SHARED_SPLITK");
  const bool shared_splits = table && shared && shared->format == FFMOE_FMT_BF16 && !(ke && atoi(ke) == 0) && table->hidden % 256 == 0 &&
                             shared->inter % 256 == 0;
  const int stream_rows = te ? atoi(te) : (shared_splits ? 0 : 24);
  if (table && args && args->act_mode == FFMOE_ACT_BF16 && args->rows > 1) {
    const int fmt = table->format, H = table->hidden, I = table->inter, R = args->rows;
    auto on_matrix_cores = [&](int f, int inter) {
      const int gran = f == FFMOE_FMT_FP8_BLOCK128 ? 128 : 64;
      return (f == FFMOE_FMT_FP8_BLOCK128 || f == FFMOE_FMT_NVFP4 || f == FFMOE_FMT_BF16 || f == FFMOE_FMT_FP8_CHANNEL) && H % gran == 0 && inter % gran == 0 &&
             H >= gran && inter >= gran;
    };
    const bool shared_ok = !shared || on_matrix_cores(shared->format, shared->inter);
    const bool shared_streams = nv_lines && shared && !rides && R <= stream_rows && args->top_k > 1;
    if (cohort_rows > 0 && R >= cohort_rows && (fmt == FFMOE_FMT_FP8_BLOCK128 || nv_lines) && args->top_k >= 1 && on_matrix_cores(fmt, I) &&
        (shared_ok || shared_streams)) {
      ffmoe_prefill pf{};
      pf.rows = args->rows; pf.top_k = args->top_k; pf.act_mode = FFMOE_ACT_BF16;
      pf.swiglu = args->swiglu; pf.swiglu_limit = args->swiglu_limit; pf.routed_weight = args->routed_weight; pf.weights_f32 = args->weights_f32;
      pf.x = args->x; pf.ids = args->ids; pf.active = args->active; pf.weights = args->weights;
      pf.contributions = args->contributions; pf.done = args->done; pf.scratch = args->scratch; pf.scratch_bytes = args->scratch_bytes;
      pf.shared = shared_streams ? nullptr : shared; pf.shared_out = args->shared_out; pf.assignment_gen = args->assignment_gen;
      if (!shared_streams) return prefill_impl(table, &pf, (stage_mask & 1 ? 3 : 0) | (stage_mask & 2 ? 12 : 0), stream);
      const uint64_t routed = ffmoe_prefill_scratch_bytes(R, args->top_k, table->experts, H, I, 0);
      FF_REQUIRE(args->scratch_bytes >= ffmoe_decode_scratch_bytes(R, args->top_k, table->experts, H, I, shared->inter), FFMOE_ERR_SCRATCH,
                 "decode scratch holds %llu bytes, %llu needed", (unsigned long long)args->scratch_bytes,
                 (unsigned long long)ffmoe_decode_scratch_bytes(R, args->top_k, table->experts, H, I, shared->inter));
      pf.scratch_bytes = routed;
      FF_TRY(prefill_impl(table, &pf, (stage_mask & 1 ? 3 : 0) | (stage_mask & 2 ? 12 : 0), stream));
      ffmoe_expert_table as_shared = *table;
      as_shared.format = shared->format;
      ffmoe_decode only_shared = *args;
      only_shared.top_k = 0;
      only_shared.done = nullptr;
      only_shared.scratch = (uint8_t*)args->scratch + routed;
      only_shared.scratch_bytes = args->scratch_bytes - routed;
      return decode_impl(&as_shared, shared, &only_shared, stage_mask, stream, 0, 0);
    }
    if (shared && shared_rows > 0 && R >= shared_rows && args->top_k >= 1 && shared_ok && shared->format == FFMOE_FMT_FP8_BLOCK128) {
      // routed choices on the streaming kernels, the shared expert on the matrix cores with its activations behind the arena
      FF_TRY(decode_impl(table, nullptr, args, stage_mask, stream, args->top_k, 0, nullptr, nullptr, -1, shared->inter));
      const int SI = shared->inter;
      FF_REQUIRE(SI >= 64, FFMOE_ERR_SHAPE, "shared inter=%d", SI);
      FF_PTR16(args->shared_out);
      for (int i = 0; i < 6; i += 2)
        FF_REQUIRE(shared->slot[i] != 0 && shared->slot[i] % 16 == 0, FFMOE_ERR_ALIGN, "shared expert slot[%d] is NULL or misaligned", i);
      const size_t xb = size_t(R) * H * 2;
      FF_NO_OVERLAP(args->shared_out, xb, args->x, xb);
      FF_NO_OVERLAP(args->shared_out, xb, args->contributions, size_t(R) * args->top_k * H * 2);
      FF_NO_OVERLAP(args->shared_out, xb, args->scratch, args->scratch_bytes);
      const uint64_t act_bytes = (uint64_t(R) * SI * 2 + 255) & ~uint64_t(255);
      const uint64_t need = ffmoe_decode_scratch_bytes(R, args->top_k, table->experts, H, I, SI);
      FF_REQUIRE(args->scratch_bytes >= need, FFMOE_ERR_SCRATCH, "decode scratch holds %llu bytes, %llu needed", (unsigned long long)args->scratch_bytes,
                 (unsigned long long)need);
      // the last act_bytes of what ffmoe_decode_scratch_bytes asks for lie behind everything decode_impl lays out
      const uint64_t A = uint64_t(R) * args->top_k, imax = uint64_t(I > SI ? I : SI);
      const uint64_t own = (((A + R) * imax * 2 + 255) & ~uint64_t(255)) + (((A + R + 2) * sizeof(GroupDesc) + 255) & ~uint64_t(255)) + 256;
      uint8_t* act = (uint8_t*)args->scratch + own;
      FF_REQUIRE(own + act_bytes <= args->scratch_bytes, FFMOE_ERR_SCRATCH, "decode scratch too small for the shared expert's activations");
      return shared_expert_w16(shared, args->x, R, H, args->swiglu, args->swiglu_limit, act, args->shared_out, stage_mask, stream);
    }
  }
  if (!table || !args || !shared || shared->format == table->format) return decode_impl(table, shared, args, stage_mask, stream);
  FF_TRY(decode_impl(table, nullptr, args, stage_mask, stream, args->top_k, 0, nullptr, nullptr, -1, shared->inter));
  ffmoe_expert_table as_shared = *table;
  as_shared.format = shared->format;
  ffmoe_decode only_shared = *args;
  only_shared.top_k = 0;
  only_shared.done = nullptr;
  return decode_impl(&as_shared, shared, &only_shared, stage_mask, stream, args->top_k, 1);
}

extern "C" __attribute__((visibility("default"))) int ffmoe_decode_contribute(const ffmoe_expert_table* table, const ffmoe_shared_expert* shared,
                                       const ffmoe_decode* args, void* stream) {
  return decode_dispatch(table, shared, args, 3, stream);
}

// ---------------------------------------------------------------------------------------------
// The same call for callers that cannot allocate (HIP graph capture, serving loops that forbid hipMalloc): the
// scratch arena is a fixed array in device memory instead of a caller buffer. Every GPU holds its own copy of the
// array at its own address, looked up once per device with that device current. Nothing in the arena has to start
// at zero: the grouping kernel writes descriptors and counters before any reader, and the gate/up launch writes every
// activation row the down launch reads. Calls on one GPU share the array, so calls that overlap in time race.
static __device__ __align__(256) unsigned char g_static_scratch[FFMOE_STATIC_SCRATCH_BYTES];

static int static_scratch(void** out) {
  static std::atomic<void*> base[64];
  int dev = 0;
  const hipError_t de = hipGetDevice(&dev);
  if (de != hipSuccess) return ff_fail(int(de), "hipGetDevice failed: %s", hipGetErrorString(de));
  FF_REQUIRE(dev >= 0 && dev < 64, FFMOE_ERR_UNSUPPORTED, "device ordinal %d is outside the per-device table", dev);
  void* b = base[dev].load(std::memory_order_acquire);
  if (!b) {
    const hipError_t se = hipGetSymbolAddress(&b, HIP_SYMBOL(g_static_scratch));
    if (se != hipSuccess || !b) {
      (void)hipGetLastError();
      return ff_fail(se != hipSuccess ? int(se) : FFMOE_ERR_NULL, "hipGetSymbolAddress(static scratch) failed: %s", hipGetErrorString(se));
    }
    base[dev].store(b, std::memory_order_release);
  }
  *out = b;
  return 0;
}

extern "C" __attribute__((visibility("default"))) uint64_t ffmoe_decode_static_scratch_bytes(void) { return FFMOE_STATIC_SCRATCH_BYTES; }

extern "C" __attribute__((visibility("default"))) int ffmoe_decode_contribute_static(const ffmoe_expert_table* table, const ffmoe_shared_expert* shared,
                                                                                    const ffmoe_decode* args, void* stream) {
  FF_REQUIRE(table && args, FFMOE_ERR_NULL, "table/args is NULL");
  const uint64_t need = ffmoe_decode_scratch_bytes(args->rows, args->top_k > 0 ? args->top_k : 1, table->experts, table->hidden, table->inter,
                                                   shared ? shared->inter : 0);
  FF_REQUIRE(need != 0, FFMOE_ERR_SHAPE, "decode rows=%d top_k=%d experts=%d out of range", args->rows, args->top_k, table->experts);
  FF_REQUIRE(need <= FFMOE_STATIC_SCRATCH_BYTES, FFMOE_ERR_SCRATCH,
             "this shape needs %llu bytes of scratch, the built-in arena holds %llu: use ffmoe_decode_contribute with a caller arena",
             (unsigned long long)need, (unsigned long long)FFMOE_STATIC_SCRATCH_BYTES);
  void* arena = nullptr;
  FF_TRY(static_scratch(&arena));
  ffmoe_decode own = *args;
  own.scratch = arena;
  own.scratch_bytes = FFMOE_STATIC_SCRATCH_BYTES;
  return decode_dispatch(table, shared, &own, 3, stream);
}

extern "C" __attribute__((visibility("default"))) int ffmoe_decode_contribute_stage(const ffmoe_expert_table* table, const ffmoe_shared_expert* shared,
                                             const ffmoe_decode* args, int stage, void* stream) {
  FF_REQUIRE(stage == 0 || stage == 1, FFMOE_ERR_SHAPE, "decode stage %d is neither 0 (gate/up) nor 1 (down)", stage);
  return decode_dispatch(table, shared, args, 1 << stage, stream);
}

extern "C" __attribute__((visibility("default"))) int ffmoe_decode_finish(const ffmoe_expert_table* table, const ffmoe_shared_expert* shared,
                                                                         const ffmoe_decode* args, const void* scale, void* y, uint32_t* status,
                                                                         int combine_mode, void* stream) {
  FF_REQUIRE(table && args, FFMOE_ERR_NULL, "table/args is NULL");
  FF_REQUIRE(args->rows == 1, FFMOE_ERR_UNSUPPORTED, "ffmoe_decode_finish handles one token row (rows=%d)", args->rows);
  FF_REQUIRE(!shared || shared->format == table->format, FFMOE_ERR_UNSUPPORTED, "ffmoe_decode_finish needs the shared expert in the table's format");
  FF_REQUIRE(!shared || shared->inter == table->inter, FFMOE_ERR_UNSUPPORTED, "ffmoe_decode_finish needs shared inter == inter");
  FF_REQUIRE(combine_mode >= 0 && combine_mode <= FFMOE_COMBINE_ROUTED, FFMOE_ERR_UNSUPPORTED, "unknown combine mode %d", combine_mode);
  FF_REQUIRE(shared || combine_mode == FFMOE_COMBINE_ROUTED, FFMOE_ERR_SHAPE, "combine mode %d needs a shared expert", combine_mode);
  FF_PTR16(y);
  if (combine_mode == FFMOE_COMBINE_GATED) FF_PTR2(scale);
  if (status) FF_PTR4(status);
  FF_NO_OVERLAP(y, size_t(table->hidden) * 2, args->scratch, args->scratch_bytes);
  FF_NO_OVERLAP(y, size_t(table->hidden) * 2, args->x, size_t(table->hidden) * 2);
  FinishParams fin{};
  fin.scale = (const uint16_t*)scale; fin.y = (uint16_t*)y; fin.status = status; fin.mode = combine_mode;
  // the shared expert takes part only in the modes that add it
  const ffmoe_shared_expert* sh = combine_mode == FFMOE_COMBINE_ROUTED ? nullptr : shared;
  return decode_impl(table, sh, args, 0, stream, -1, 0, &fin);
}

extern "C" __attribute__((visibility("default"))) int ffmoe_decode_contribute_from_logits(const ffmoe_expert_table* table, const ffmoe_shared_expert* shared,
                                                                                         const ffmoe_decode* args, const float* logits, const float* bias,
                                                                                         int score_mode, float routed_scaling, int n_group, int topk_group,
                                                                                         void* stream) {
  FF_REQUIRE(table && args, FFMOE_ERR_NULL, "table/args is NULL");
  FF_REQUIRE(args->rows == 1, FFMOE_ERR_UNSUPPORTED, "selection inside the gate/up launch handles one token row (rows=%d)", args->rows);
  FF_REQUIRE(args->act_mode == FFMOE_ACT_BF16, FFMOE_ERR_UNSUPPORTED, "selection inside the gate/up launch needs FFMOE_ACT_BF16");
  FF_REQUIRE(!shared || shared->format == table->format, FFMOE_ERR_UNSUPPORTED, "selection inside the gate/up launch needs the shared expert in the table's format");
  FF_REQUIRE(args->weights_f32 == 1 && args->active == nullptr && args->assignment_gen == nullptr, FFMOE_ERR_UNSUPPORTED,
             "selection inside the gate/up launch writes f32 weights and takes no active mask or epochs");
  const int E = table->experts, K = args->top_k;
  FF_REQUIRE(E == 64 || E == 128 || E == 256 || E == 512 || E == 1024, FFMOE_ERR_UNSUPPORTED, "experts=%d is not 64 * 2^n", E);
  FF_REQUIRE(K >= 1 && K <= FFMOE_MAX_TOP_K && K < E, FFMOE_ERR_SHAPE, "top_k=%d out of range", K);
  FF_REQUIRE(score_mode == FFMOE_NOAUX_SIGMOID || score_mode == FFMOE_NOAUX_SQRTSOFTPLUS, FFMOE_ERR_UNSUPPORTED, "unknown score mode %d", score_mode);
  FF_REQUIRE(routed_scaling > 0.0f && routed_scaling < INFINITY, FFMOE_ERR_SHAPE, "routed_scaling=%g", (double)routed_scaling);
  FF_REQUIRE(n_group >= 1 && topk_group >= 1 && topk_group <= n_group && E % n_group == 0, FFMOE_ERR_SHAPE, "n_group=%d topk_group=%d", n_group, topk_group);
  if (n_group > 1) {
    const int c = E / 64, per = E / n_group;
    FF_REQUIRE(per % c == 0 && ((per / c) & (per / c - 1)) == 0 && topk_group * per >= K, FFMOE_ERR_UNSUPPORTED,
               "groups of %d experts do not tile the wave, or the kept groups hold fewer than top_k experts", per);
  }
  FF_PTR4(logits);
  if (bias) FF_PTR4(bias);
  const RouteInline route{logits, bias, score_mode, n_group, topk_group, routed_scaling};
  return decode_impl(table, shared, args, 3, stream, -1, 0, nullptr, &route);
}

// One token in two launches: top-k selection in the prologue of the gate/up launch (behind the shared expert's rows,
// which need no routing), then down + routing weight + ordered combine in one launch.
static int token_forward(const ffmoe_expert_table* table, const ffmoe_shared_expert* shared, const ffmoe_decode* args, const float* logits,
                         const float* bias, int score_mode, float routed_scaling, int n_group, int topk_group, const void* scale, void* y,
                         uint32_t* status, int combine_mode, int stage_mask, void* stream) {
  FF_REQUIRE(table && args, FFMOE_ERR_NULL, "table/args is NULL");
  FF_REQUIRE(args->rows == 1, FFMOE_ERR_UNSUPPORTED, "ffmoe_decode_token_forward handles one token row (rows=%d)", args->rows);
  FF_REQUIRE(args->act_mode == FFMOE_ACT_BF16, FFMOE_ERR_UNSUPPORTED, "ffmoe_decode_token_forward needs FFMOE_ACT_BF16");
  FF_REQUIRE(combine_mode >= 0 && combine_mode <= FFMOE_COMBINE_ROUTED, FFMOE_ERR_UNSUPPORTED, "unknown combine mode %d", combine_mode);
  FF_REQUIRE(shared || combine_mode == FFMOE_COMBINE_ROUTED, FFMOE_ERR_SHAPE, "combine mode %d needs a shared expert", combine_mode);
  FF_REQUIRE(args->weights_f32 == 1 && args->active == nullptr && args->assignment_gen == nullptr, FFMOE_ERR_UNSUPPORTED,
             "selection inside the gate/up launch writes f32 weights and takes no active mask or epochs");
  const int E = table->experts, K = args->top_k;
  FF_REQUIRE(E == 64 || E == 128 || E == 256 || E == 512 || E == 1024, FFMOE_ERR_UNSUPPORTED, "experts=%d is not 64 * 2^n", E);
  FF_REQUIRE(K >= 1 && K <= 8 && K < E, FFMOE_ERR_UNSUPPORTED, "top_k=%d: the one-token finish holds up to 8 routed choices", K);
  FF_REQUIRE(score_mode == FFMOE_NOAUX_SIGMOID || score_mode == FFMOE_NOAUX_SQRTSOFTPLUS, FFMOE_ERR_UNSUPPORTED, "unknown score mode %d", score_mode);
  FF_REQUIRE(routed_scaling > 0.0f && routed_scaling < INFINITY, FFMOE_ERR_SHAPE, "routed_scaling=%g", (double)routed_scaling);
  FF_REQUIRE(n_group >= 1 && topk_group >= 1 && topk_group <= n_group && E % n_group == 0, FFMOE_ERR_SHAPE, "n_group=%d topk_group=%d", n_group, topk_group);
  if (n_group > 1) {
    const int c = E / 64, per = E / n_group;
    FF_REQUIRE(per % c == 0 && ((per / c) & (per / c - 1)) == 0 && topk_group * per >= K, FFMOE_ERR_UNSUPPORTED,
               "groups of %d experts do not tile the wave, or the kept groups hold fewer than top_k experts", per);
  }
  // rows of the down matrix beyond two 64-lane steps are outside the finish kernel's register buffers
  {
    const int epl = table->format == FFMOE_FMT_NVFP4 ? 32 : (table->format == FFMOE_FMT_BF16 ? 8 : 16);
    FF_REQUIRE((table->inter / epl + 63) / 64 <= 2, FFMOE_ERR_UNSUPPORTED, "inter=%d is beyond the one-token finish's row buffers", table->inter);
  }
  FF_PTR4(logits);
  if (bias) FF_PTR4(bias);
  FF_PTR16(y);
  if (combine_mode == FFMOE_COMBINE_GATED) FF_PTR2(scale);
  if (status) FF_PTR4(status);
  FF_NO_OVERLAP(y, size_t(table->hidden) * 2, args->scratch, args->scratch_bytes);
  FF_NO_OVERLAP(y, size_t(table->hidden) * 2, args->x, size_t(table->hidden) * 2);
  // the shared expert takes part only in the modes that add it
  const ffmoe_shared_expert* sh = combine_mode == FFMOE_COMBINE_ROUTED ? nullptr : shared;
  const RouteInline route{logits, bias, score_mode, n_group, topk_group, routed_scaling};
  FinishParams fin{};
  fin.scale = (const uint16_t*)scale; fin.y = (uint16_t*)y; fin.status = status; fin.mode = combine_mode;
  if (sh && !(sh->format == table->format && sh->inter == table->inter)) {
    // A shared expert of another format or width (BF16 next to NVFP4 experts) cannot share the routed launches: its
    // two launches run with the kernels of its own format (second pass of the arena, as in ffmoe_decode_contribute) and
    // leave the BF16 row in shared_out, which the finish adds where its own shared group's row would go - the same
    // value, rounded at the same boundary. The selection runs in the prologue of the shared expert's gate/up launch
    // (wave 0 of every block, next to the three waves that stream the shared rows), so the routed gate/up launch starts
    // with its ids in memory. Five launches per layer with the logits instead of seven.
    // NVFP4 experts and a BF16 shared expert of their width: the finish launch streams the shared expert's down rows too, in
    // BF16, as every wave's first units - three launches with the logits (FFMOE_DECODE_MIXED_FINISH=0: four)
    const char* mf = getenv("FFMOE_DECODE_MIXED_FINISH");
    const char* mg = getenv("FFMOE_DECODE_MIXED_GATE_UP");
    const int sh_steps = (sh->inter / 8 + 63) / 64;
    const bool finish_shared = table->format == FFMOE_FMT_NVFP4 && sh->format == FFMOE_FMT_BF16 && sh->inter == table->inter &&
                               table->inter <= 2048 && (sh_steps == 1 || sh_steps == 2 || sh_steps == 4) && !(mf && atoi(mf) == 0) &&
                               !(mg && atoi(mg) == 0) && decode_gate_up_nvfp4_bf16_shared_available(table->hidden);
    if (stage_mask & 1) {
      ffmoe_expert_table as_shared = *table;
      as_shared.format = sh->format;
      ffmoe_decode only_shared = *args;
      only_shared.top_k = 0;
      const char* me = getenv("FFMOE_DECODE_MIXED_GATE_UP");
      if (sh->format == table->format && !(me && atoi(me) == 0)) {
        // same format, another width: the gate/up launch takes shared rows of any width as it is; only the finish cannot
        FF_TRY(decode_impl(table, sh, args, 1, stream, K, 0, nullptr, &route, -1, sh->inter));
        FF_TRY(decode_impl(&as_shared, sh, &only_shared, 2, stream, K, 1));
      } else if (table->format == FFMOE_FMT_NVFP4 && sh->format == FFMOE_FMT_BF16 && !(me && atoi(me) == 0) &&
                 decode_gate_up_nvfp4_bf16_shared_available(table->hidden)) {
        // the shared expert's gate/up rows as every block's first slice of the routed gate/up launch, in BF16, next to the
        // selection; only its down launch is its own: four launches with the logits (FFMOE_DECODE_MIXED_GATE_UP=0: five)
        FF_TRY(decode_impl(table, sh, args, 1, stream, K, 0, nullptr, &route, -1, sh->inter, true));
        if (!finish_shared) FF_TRY(decode_impl(&as_shared, sh, &only_shared, 2, stream, K, 1));
      } else {
        RouteInline select = route;
        select.select_k = K;
        FF_TRY(decode_impl(&as_shared, sh, &only_shared, 3, stream, K, 1, nullptr, &select));
        FF_TRY(decode_impl(table, nullptr, args, 1, stream, K, 0, nullptr, nullptr, -1, sh->inter));
      }
    }
    if ((stage_mask & 2) && finish_shared) {
      FF_TRY(decode_impl(table, sh, args, 0, stream, K, 0, &fin, nullptr, -1, sh->inter, false, false, true));
    } else if (stage_mask & 2) {
      FF_PTR16(args->shared_out);
      FF_NO_OVERLAP(y, size_t(table->hidden) * 2, args->shared_out, size_t(table->hidden) * 2);
      fin.shared_ready = (const uint16_t*)args->shared_out;
      FF_TRY(decode_impl(table, nullptr, args, 0, stream, K, 0, &fin, nullptr, -1, sh->inter));
    }
    return 0;
  }
  // both launches in one call: block 0 of the gate/up launch resolves the live choices (combine order, down matrices,
  // routing weights) for the finish, which then starts from that record instead of the chain ids -> slot table. A stage
  // issued alone works from ids and weights in memory, as ffmoe_decode_finish does.
  const bool record = stage_mask == 3 && K <= FFMOE_FINISH_ROUTED;
  RouteInline route_rec = route;
  route_rec.finish_ordered = !(combine_mode == FFMOE_COMBINE_ACCUM_FP32 || combine_mode == FFMOE_COMBINE_ACCUM_BF16);
  if (stage_mask & 1) FF_TRY(decode_impl(table, sh, args, 1, stream, -1, 0, nullptr, &route_rec, -1, 0, false, record));
  if (stage_mask & 2) FF_TRY(decode_impl(table, sh, args, 0, stream, -1, 0, &fin, nullptr, -1, 0, false, record));
  return 0;
}

extern "C" __attribute__((visibility("default"))) int ffmoe_decode_token_forward(const ffmoe_expert_table* table, const ffmoe_shared_expert* shared,
                                                                                const ffmoe_decode* args, const float* logits, const float* bias,
                                                                                int score_mode, float routed_scaling, int n_group, int topk_group,
                                                                                const void* scale, void* y, uint32_t* status, int combine_mode,
                                                                                void* stream) {
  return token_forward(table, shared, args, logits, bias, score_mode, routed_scaling, n_group, topk_group, scale, y, status, combine_mode, 3, stream);
}

extern "C" __attribute__((visibility("default"))) int ffmoe_decode_token_forward_stage(const ffmoe_expert_table* table, const ffmoe_shared_expert* shared,
                                                                                      const ffmoe_decode* args, const float* logits, const float* bias,
                                                                                      int score_mode, float routed_scaling, int n_group, int topk_group,
                                                                                      const void* scale, void* y, uint32_t* status, int combine_mode,
                                                                                      int stage, void* stream) {
  FF_REQUIRE(stage == 0 || stage == 1, FFMOE_ERR_SHAPE, "token forward stage %d is neither 0 (selection + gate/up) nor 1 (down + combine)", stage);
  return token_forward(table, shared, args, logits, bias, score_mode, routed_scaling, n_group, topk_group, scale, y, status, combine_mode, 1 << stage, stream);
}

extern "C" __attribute__((visibility("default"))) int ffmoe_decode_token_layer(const ffmoe_expert_table* table, const ffmoe_shared_expert* shared,
                                                                              const ffmoe_decode* args, const float* logits, const float* bias,
                                                                              int score_mode, float routed_scaling, int n_group, int topk_group,
                                                                              const void* scale, void* y, uint32_t* status, int combine_mode,
                                                                              void* stream) {
  FF_REQUIRE(table && args, FFMOE_ERR_NULL, "table/args is NULL");
  FF_REQUIRE(args->rows == 1, FFMOE_ERR_UNSUPPORTED, "ffmoe_decode_token_layer handles one token row (rows=%d)", args->rows);
  FF_REQUIRE(args->act_mode == FFMOE_ACT_BF16, FFMOE_ERR_UNSUPPORTED, "ffmoe_decode_token_layer needs FFMOE_ACT_BF16");
  FF_REQUIRE(!shared || shared->format == table->format, FFMOE_ERR_UNSUPPORTED, "ffmoe_decode_token_layer needs the shared expert in the table's format");
  FF_REQUIRE(combine_mode >= 0 && combine_mode <= FFMOE_COMBINE_ROUTED, FFMOE_ERR_UNSUPPORTED, "unknown combine mode %d", combine_mode);
  FF_REQUIRE(shared || combine_mode == FFMOE_COMBINE_ROUTED, FFMOE_ERR_SHAPE, "combine mode %d needs a shared expert", combine_mode);
  FF_PTR16(y);
  if (combine_mode == FFMOE_COMBINE_GATED) FF_PTR2(scale);
  if (status) FF_PTR4(status);
  FF_NO_OVERLAP(y, size_t(table->hidden) * 2, args->scratch, args->scratch_bytes);
  FF_NO_OVERLAP(y, size_t(table->hidden) * 2, args->x, size_t(table->hidden) * 2);
  RouteInline route{nullptr, nullptr, 0, 1, 1, 1.0f};
  if (logits) {
    FF_REQUIRE(args->weights_f32 == 1 && args->active == nullptr && args->assignment_gen == nullptr, FFMOE_ERR_UNSUPPORTED,
               "selection inside the launch writes f32 weights and takes no active mask or epochs");
    const int E = table->experts, K = args->top_k;
    FF_REQUIRE(E == 64 || E == 128 || E == 256 || E == 512 || E == 1024, FFMOE_ERR_UNSUPPORTED, "experts=%d is not 64 * 2^n", E);
    FF_REQUIRE(K >= 1 && K <= FFMOE_MAX_TOP_K && K < E, FFMOE_ERR_SHAPE, "top_k=%d out of range", K);
    FF_REQUIRE(score_mode == FFMOE_NOAUX_SIGMOID || score_mode == FFMOE_NOAUX_SQRTSOFTPLUS, FFMOE_ERR_UNSUPPORTED, "unknown score mode %d", score_mode);
    FF_REQUIRE(routed_scaling > 0.0f && routed_scaling < INFINITY, FFMOE_ERR_SHAPE, "routed_scaling=%g", (double)routed_scaling);
    FF_REQUIRE(n_group >= 1 && topk_group >= 1 && topk_group <= n_group && E % n_group == 0, FFMOE_ERR_SHAPE, "n_group=%d topk_group=%d", n_group, topk_group);
    if (n_group > 1) {
      const int c = E / 64, per = E / n_group;
      FF_REQUIRE(per % c == 0 && ((per / c) & (per / c - 1)) == 0 && topk_group * per >= K, FFMOE_ERR_UNSUPPORTED,
                 "groups of %d experts do not tile the wave, or the kept groups hold fewer than top_k experts", per);
    }
    FF_PTR4(logits);
    if (bias) FF_PTR4(bias);
    route = RouteInline{logits, bias, score_mode, n_group, topk_group, routed_scaling};
  }
  FinishParams fin{};
  fin.scale = (const uint16_t*)scale; fin.y = (uint16_t*)y; fin.status = status; fin.mode = combine_mode; fin.whole = 1;
  // the shared expert takes part only in the modes that add it
  const ffmoe_shared_expert* sh = combine_mode == FFMOE_COMBINE_ROUTED ? nullptr : shared;
  return decode_impl(table, sh, args, 0, stream, -1, 0, &fin, logits ? &route : nullptr);
}

extern "C" __attribute__((visibility("default"))) int ffmoe_decode_contribute_form(const ffmoe_expert_table* table, const ffmoe_shared_expert* shared,
                                                                                  const ffmoe_decode* args, int form, void* stream) {
  FF_REQUIRE(table && args, FFMOE_ERR_NULL, "table/args is NULL");
  FF_REQUIRE(form == FFMOE_FORM_LANE16 || form == FFMOE_FORM_LANE8, FFMOE_ERR_UNSUPPORTED, "unknown reduction form %d", form);
  FF_REQUIRE(table->format == FFMOE_FMT_BF16 || table->format == FFMOE_FMT_FP8_CHANNEL, FFMOE_ERR_UNSUPPORTED,
             "the reference's reduction orders are built for BF16 and per-channel FP8 experts (format %d)", table->format);
  FF_REQUIRE(!shared || shared->format == table->format, FFMOE_ERR_UNSUPPORTED, "shared expert format %d differs from the table format %d",
             shared ? shared->format : -1, table->format);
  FF_REQUIRE(args->act_mode == FFMOE_ACT_BF16, FFMOE_ERR_UNSUPPORTED, "the reference's reduction orders need FFMOE_ACT_BF16");
  FF_REQUIRE(args->rows <= 65535 && args->top_k + 1 <= 65535, FFMOE_ERR_SHAPE, "rows=%d top_k=%d exceed the launch grid", args->rows, args->top_k);
  return decode_impl(table, shared, args, 3, stream, -1, 0, nullptr, nullptr, form);
}
