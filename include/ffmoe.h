/*
 * libffmoe — MI355X (gfx950) kernels for the quantized MoE expert-FFN path of GreatV/flyingfish:
 * router top-k, block-scaled FP8 E4M3 / NVFP4 expert SwiGLU FFN for decode, token-sorted grouped
 * GEMM prefill, and the ordered weighted combine.
 *
 * Conventions (they restate the reference's operator contract,
 * src/backend/cuda/contracts.rs:80-137 and the per-op validators cited below):
 *   - every tensor argument is a raw DEVICE pointer to a dense row-major array; the caller owns
 *     all of them, including scratch, `contributions` and `done`;
 *   - base pointers of BF16/FP8/FP4 tensors are 16-byte aligned, f32/i32/u32 tensors 4-byte;
 *   - BF16 values are passed as uint16 bit patterns (`void*` in the signatures);
 *   - `stream` is a hipStream_t (NULL = the default stream); calls only enqueue work;
 *   - return value: 0 = ok, > 0 = hipError_t of a failed runtime call, < 0 = contract violation
 *     detected on the host before anything was launched (`ffmoe_last_error()` has the text);
 *   - nothing here allocates device memory.
 */
#ifndef FFMOE_H
#define FFMOE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define FFMOE_VERSION 1

/* contract-violation codes (negative) */
#define FFMOE_ERR_NULL        (-1)  /* required pointer is NULL */
#define FFMOE_ERR_ALIGN       (-2)  /* base pointer misaligned */
#define FFMOE_ERR_SHAPE       (-3)  /* extent out of range or inconsistent */
#define FFMOE_ERR_OVERLAP     (-4)  /* an output aliases an input, scratch or another output */
#define FFMOE_ERR_UNSUPPORTED (-5)  /* format / mode combination not implemented */
#define FFMOE_ERR_SCRATCH     (-6)  /* scratch arena too small */

/* limits of the routing contract (kernels/moe_route.cu:23-30, :462-466) */
#define FFMOE_MAX_EXPERTS 1024
#define FFMOE_MAX_TOP_K   32

/* expert weight formats (src/model_spec.rs ExpertFormat / LinearFormat) */
#define FFMOE_FMT_FP8_BLOCK128 0  /* E4M3 codes [N,K] + f32 scales [ceil(N/128), ceil(K/128)] (src/fp8.rs:31-36) */
#define FFMOE_FMT_NVFP4        1  /* E2M1 pairs [N,K/2] (low nibble = even k) + E4M3 scales [N,K/16] + f32 global */
#define FFMOE_FMT_BF16         2  /* BF16 [N,K] */
#define FFMOE_FMT_FP8_CHANNEL  3  /* E4M3 codes [N,K] + one BF16 scale per output row [N] (src/experts/catalogue.rs:31-39) */
#define FFMOE_FMT_E2M1_E8M0     4  /* E2M1 pairs [N,K/2] (low nibble = even k) + E8M0 scales [N,K/32] (kernels/moe_ffn.cu:398-403) */
#define FFMOE_FMT_E4M3_E8M0_32  5  /* E4M3 codes [N,K] + E8M0 scales [ceil(N/32), K/32], one per 32x32 block (kernels/moe_ffn.cu:743-747) */

/* activation arithmetic of the FP8 linears */
#define FFMOE_ACT_BF16         0  /* W8A16: w = bf16(e4m3(code) * scale), FP32 accumulate against BF16 activations
                                     (src/fp8.rs:138-140, src/cpu/expert_ffn.rs:592-679) */
#define FFMOE_ACT_FP8_BLOCK128 1  /* W8A8: activations quantized per 128 to E4M3 with an f32 scale, per-128 dot then
                                     one scale product (kernels/fp8_linear.cu:12-48, kernels/q38_contract.cuh:239-279);
                                     on NVFP4 tables W4A8: the weights rounded to E4M3 first (ffmoe_prefill_contribute) */
#define FFMOE_ACT_E4M3_E8M0_32  2  /* activations quantized per 32 to E4M3 with a power-of-two (E8M0) scale, exact integer dots
                                     (ffmoe_decode_contribute_e8m0 only) */
#define FFMOE_ACT_E4M3_E8M0_32_F32 3  /* the same quantizer with the FP32 fma chains and 32-lane order of the reference's
                                        moe_ffn_dispatch_*_e2m1_e8m0 / moe_ffn_*_e4m3_block32 (kernels/moe_ffn.cu:469-576,764-865) */

/* SwiGLU rounding (src/model_spec.rs:61-69; src/cpu/expert_ffn.rs:58-100) */
#define FFMOE_SWIGLU_TWICE          0  /* a = bf16(bf16(silu(g)) * u) */
#define FFMOE_SWIGLU_ONCE           1  /* a = bf16(silu(g) * u) */
#define FFMOE_SWIGLU_CLAMPED_TWICE  2  /* g = min(g,L), u = clamp(u,+-L), then TWICE */
#define FFMOE_SWIGLU_CLAMPED_ONCE   3
/* a = bf16(bf16(gelu(g)) * u), gelu(g) = 0.5 g (1 + tanh(0.7978846 (g + 0.044715 g^3))) in FP32 with one rounding per
   operation and no clamp (SwigluRounding::GeluTwice, src/cpu/expert_ffn.rs:65,87-91,110-113; kernels/act.cu:16-22).
   The reference takes tanh from libm or the CUDA math library; this library uses one fixed FP32 tanh within 3 ulp of
   the exact function. Not available with FFMOE_ACT_FP8_BLOCK128 (the reference binds it to BF16 experts only,
   src/backend/cuda/engine_diffusion.rs:1135-1141). */
#define FFMOE_SWIGLU_GELU_TWICE     4

/* routed-weight boundary (src/model_spec.rs:70-75) */
#define FFMOE_WEIGHT_AFTER_DOWN_BF16          0  /* c = bf16(bf16(d) * w) */
#define FFMOE_WEIGHT_BEFORE_CONTRIBUTION_BF16 1  /* c = bf16(d * w) */
#define FFMOE_WEIGHT_BEFORE_DOWN_F32          2  /* the f32 weight multiplies the SwiGLU product before its BF16 cast, i.e. before
                                                  the down projection (E8M0 contract, kernels/moe_ffn.cu:411-414) */

/* router score */
#define FFMOE_SCORE_SOFTMAX      0
#define FFMOE_SCORE_SIGMOID      1
#define FFMOE_NOAUX_SIGMOID      0  /* score_mode of the noaux kernels (kernels/moe_route.cu:329-336) */
#define FFMOE_NOAUX_SQRTSOFTPLUS 1

/* combine variants (kernels/moe_combine.cu) */
#define FFMOE_COMBINE_GATED      0  /* moe_combine         :71-93   */
#define FFMOE_COMBINE_UNGATED    1  /* moe_combine_ungated :95-116  */
#define FFMOE_COMBINE_BF16       2  /* moe_combine_bf16    :592-613 */
#define FFMOE_COMBINE_ACCUM_FP32 3  /* moe_combine_accum, fp32_accum = 1 :541-591 */
#define FFMOE_COMBINE_ACCUM_BF16 4  /* moe_combine_accum, fp32_accum = 0 */
#define FFMOE_COMBINE_ROUTED     5  /* moe_combine_routed  :176-196 */

const char* ffmoe_last_error(void);
int ffmoe_version(void);

/* ------------------------------------------------------------------------------------------------
 * Router. Replaces RouteOps (src/backend/cuda/moe/route.rs:450-499, :505-562, :721-769, :808-905)
 * and the kernels of kernels/moe_route.cu.
 */

/* logits[r,e] = bf16(ascending FP32 fma chain over x[r,:] * router[e,:]).
 * Replaces moe_route_logits_bf16 (kernels/moe_route.cu:408-457). hidden % 8 == 0. */
int ffmoe_route_logits_bf16(const void* x, const void* router, void* logits,
                            int rows, int experts, int hidden, void* stream);

/* FP32 logits (replaces RouteOps::logits_f32, route.rs:505-562, a BLAS GEMM of undefined order).
 * Order used here: 256 partial chains, partial p chaining fma over the 8-element vectors p, p+256, ... in
 * ascending order, summed by a balanced pairwise tree in natural order. hidden % 8 == 0. */
int ffmoe_route_logits_f32(const void* x, const void* router, float* logits,
                           int rows, int experts, int hidden, void* stream);

/* Softmax or sigmoid top-k over BF16 logits; ids [rows,top_k] i32, weights [rows,top_k] BF16.
 * Replaces moe_route_topk / moe_route_topk_sigmoid (kernels/moe_route.cu:459-491).
 * 1 <= top_k <= 32, top_k < experts <= 1024. */
int ffmoe_route_topk(const void* logits, int* ids, void* weights,
                     int rows, int experts, int top_k, int score, void* stream);

/* noaux_tc selection over FP32 logits: select on score+bias, weight = score/(sum+1e-20)*routed_scaling.
 * Replaces moe_route_topk_noaux(_f32) (kernels/moe_route.cu:579-628; route.rs:721-769).
 * bias may be NULL; bias_row_stride is `experts` for a [rows,experts] bias or 0 to broadcast one [experts] row.
 * weights_f32 != 0 stores f32 weights, else BF16. n_group > 1 adds a group filter that the reference does not
 * have (group score = sum of the two largest score+bias in the group; keep topk_group groups; ties to the
 * lower group id); n_group == 1 is the reference kernel. experts % n_group == 0. */
int ffmoe_route_topk_noaux(const float* logits, const float* bias, int bias_row_stride,
                           int* ids, void* weights, int weights_f32,
                           int rows, int experts, int top_k, int score_mode, float routed_scaling,
                           int n_group, int topk_group, void* stream);

/* Decode route of the noaux_tc models: FP32 logits (ffmoe_route_logits_f32) then the noaux selection, which also
 * clears `done` (optional, [rows, top_k]) for the rows routed, so the contribution that follows starts from a clean
 * slate. Replaces NativeMoe::enqueue_route (src/backend/cuda/moe/decode.rs:1145-1168: logits GEMM +
 * moe_route_topk_noaux_f32). Two launches: on this multi-die GPU a cross-block hand-over inside one kernel costs more
 * than a kernel boundary. Results are bit-identical to ffmoe_route_logits_f32 followed by ffmoe_route_topk_noaux. */
int ffmoe_route_noaux_decode(const void* x, const void* router, const float* bias, int bias_row_stride,
                             float* logits, int* ids, void* weights, int weights_f32, uint32_t* done,
                             int rows, int experts, int hidden, int top_k, int score_mode, float routed_scaling,
                             int n_group, int topk_group, void* stream);

/* Fused decode route: BF16 logits (stored) then softmax/sigmoid top-k.
 * Replaces RouteOps::route / moe_route_decode_bf16 (route.rs:450-499; kernels/moe_route.cu:496-568). With at most 64
 * experts it is ONE launch, as in the reference: the wave that runs a row's 64 logit chains holds the row's logits one per
 * lane and selects right away; with more experts a row's logits come from several blocks and the selection is a launch of
 * its own. logits, ids and weights are the bits of ffmoe_route_logits_bf16 followed by ffmoe_route_topk either way. */
int ffmoe_route_decode(const void* x, const void* router, void* logits, int* ids, void* weights,
                       int rows, int experts, int hidden, int top_k, int score, void* stream);

/* ------------------------------------------------------------------------------------------------
 * Expert tables. All experts stay resident in HBM. A slot is six device addresses per expert, as
 * NativeMoe's `slots[E,6]` (kernels/moe_ffn.cu:869-885; src/backend/cuda/moe/decode.rs:683-698):
 *   {gate codes, gate scales, up codes, up scales, down codes, down scales}
 * gate/up are [inter, hidden], down is [hidden, inter]. For FFMOE_FMT_BF16 the scale entries are ignored.
 * For NVFP4 `global_scales` holds weight_scale_2 of gate, up, down per expert.
 */
typedef struct ffmoe_expert_table {
  int format;                 /* FFMOE_FMT_* */
  int experts, hidden, inter;
  const uint64_t* slots;      /* device [experts, 6] */
  const uint32_t* valid;      /* device [experts], 0 = not resident; NULL = all valid */
  const float* global_scales; /* device [experts, 3] (NVFP4) or NULL */
  const uint64_t* generation; /* device [experts] residency epoch of each slot (ffmoe_slot_publish), or NULL */
} ffmoe_expert_table;

/* One always-on shared expert (MoeDecode::shared_gate/up/down, decode.rs:26-44). Addresses by value. */
typedef struct ffmoe_shared_expert {
  int format;                 /* FFMOE_FMT_* */
  int inter;
  uint64_t slot[6];           /* device addresses, same order as a table slot */
  float global_scales[3];     /* NVFP4 only */
} ffmoe_shared_expert;

/* ------------------------------------------------------------------------------------------------
 * Decode contribution: for every active (row, choice) the expert SwiGLU FFN output times the routing
 * weight, plus the shared expert per row. Replaces DecodeOps::contribute(_routed,_shared,_w8a16)
 * (src/backend/cuda/moe/decode.rs:421-589) and NativeMoe's dispatch (decode.rs:1187-1262), i.e. kernels
 * moe_ffn_gate_up/_down(+_w8a16) and moe_ffn_dispatch_e4m3_f32_128 + moe_ffn_weight_f32 (kernels/moe_ffn.cu).
 * Unlike the reference (rows <= 8/16) any row count is accepted; rows routed to the same expert share one
 * pass over that expert's weights.
 */
typedef struct ffmoe_decode {
  int rows, top_k;
  int act_mode;        /* FFMOE_ACT_* (FP8 formats) */
  int swiglu;          /* FFMOE_SWIGLU_* */
  float swiglu_limit;  /* clamped modes: finite, > 0 */
  int routed_weight;   /* FFMOE_WEIGHT_* */
  int weights_f32;     /* routing weights are f32 (else BF16) */
  const void* x;       /* [rows, hidden] BF16 */
  const int* ids;      /* [rows, top_k] */
  const uint32_t* active; /* [rows, top_k] or NULL = all active */
  const void* weights; /* [rows, top_k] BF16 or f32 */
  void* contributions; /* [rows, top_k, hidden] BF16 */
  void* shared_out;    /* [rows, hidden] BF16 (NULL when there is no shared expert) */
  uint32_t* done;      /* [rows, top_k]; set to 1 for every contributed slot (NULL = not tracked) */
  void* scratch;       /* ffmoe_decode_scratch_bytes() bytes, 256-byte aligned */
  uint64_t scratch_bytes;
  const uint64_t* assignment_gen; /* [rows, top_k] epoch each choice was routed against (ffmoe_route_mask), or NULL.
                                     With table->generation: a choice whose expert has been replaced since (epochs
                                     differ) contributes nothing and keeps done = 0, where the reference traps
                                     (kernels/moe_ffn.cu:140-154) */
} ffmoe_decode;

/* Scratch needed by ffmoe_decode_contribute (mirrors decode_scratch_bytes_mixed, decode.rs:52-59,
 * plus the assignment-grouping tables and the quantized activations of FFMOE_ACT_FP8_BLOCK128). */
uint64_t ffmoe_decode_scratch_bytes(int rows, int top_k, int experts, int hidden, int inter, int shared_inter);

int ffmoe_decode_contribute(const ffmoe_expert_table* table, const ffmoe_shared_expert* shared,
                            const ffmoe_decode* args, void* stream);

/* ffmoe_decode_contribute for callers that cannot allocate device memory or hand over a scratch arena (code under HIP
 * graph capture, serving loops and harnesses that forbid hipMalloc). No counterpart in the reference. args->scratch and
 * args->scratch_bytes are ignored: the arena is a fixed array of ffmoe_decode_static_scratch_bytes() bytes (8 MiB) in
 * the library's device image, one copy per GPU, held until the process ends. Everything else (arguments, arithmetic,
 * outputs, errors) is ffmoe_decode_contribute's, and the results are bit-identical to it. A shape whose
 * ffmoe_decode_scratch_bytes() exceeds the arena is rejected with FFMOE_ERR_SCRATCH and nothing is launched (at the
 * DeepSeek-V3 dimensions the arena holds up to 128 rows x top-8). The call allocates nothing and clears nothing
 * (no stage reads arena bytes that an earlier launch of the same call has not written). All calls on one GPU share
 * that GPU's array: two calls that overlap in time on one GPU (different streams) race. Under HIP graph capture: make
 * the first call on each GPU outside capture (it looks the array's address up with hipGetSymbolAddress, which may load
 * the code object), and note that the environment switches that pick the kernels (FFMOE_DECODE_COHORT_ROWS and the
 * like) are read when the call is made, i.e. at capture, not at replay. */
uint64_t ffmoe_decode_static_scratch_bytes(void);
int ffmoe_decode_contribute_static(const ffmoe_expert_table* table, const ffmoe_shared_expert* shared,
                                   const ffmoe_decode* args, void* stream);

/* The two launches of the contribution as separate calls, like the reference's gate_up and down launches
 * (src/backend/cuda/moe/decode.rs:486-490 and :513-517): stage 0 = gate/up + SwiGLU into scratch (and the
 * grouping of assignments by expert), stage 1 = down + routing weight from scratch. Stage 0 then stage 1 with the
 * same arguments equals ffmoe_decode_contribute. */
int ffmoe_decode_contribute_stage(const ffmoe_expert_table* table, const ffmoe_shared_expert* shared,
                                  const ffmoe_decode* args, int stage, void* stream);

/* Expert contributions in the reference's own summation orders, bit for bit: the same call as ffmoe_decode_contribute,
 * but every dot product follows Form::Lane16 or Form::Lane8 of the reference's CPU path
 * (src/cpu/expert_ffn.rs:689-776; GPU: the invariant kernels moe_ffn_*_lane16, kernels/moe_ffn.cu:364-393, and the
 * production kernels moe_gate_up / moe_down, kernels/moe_ffn.cu:98-302), with the SiLU form that goes with it, so
 * contributions and shared_out equal the CPU path's to the last bit (mixed CPU / GPU expert tiering stays
 * reproducible). Replaces DecodeOps::new_invariant_with_boundaries + contribute (src/backend/cuda/moe/decode.rs:342-520).
 * FFMOE_FMT_BF16 and FFMOE_FMT_FP8_CHANNEL tables only (the formats the CPU path executes); slower than
 * ffmoe_decode_contribute, whose 64-lane sums match these orders to 2 BF16 ulp. No limit on rows * top_k beyond the
 * launch grid (rows <= 65535): a prefill cohort in these orders, the arithmetic of moe_gemm_lane16*
 * (kernels/moe_prefill.cu:13-71), is this call with the cohort's rows. */
#define FFMOE_FORM_LANE16 0
#define FFMOE_FORM_LANE8  1
int ffmoe_decode_contribute_form(const ffmoe_expert_table* table, const ffmoe_shared_expert* shared, const ffmoe_decode* args,
                                 int form, void* stream);

/* Experts of the E8M0 block-32 contract (DeepSeek-V4.1 formats) in exact arithmetic. Routed experts are W4A8
 * (FFMOE_FMT_E2M1_E8M0), the shared expert W8A8 with 32x32 block scales (FFMOE_FMT_E4M3_E8M0_32); every activation row
 * is quantized to E4M3 with one E8M0 scale per 32 elements (amax floored at 1e-4, scale 2^ceil(log2(amax / 448))); a
 * 32-element group dot is an exact integer, the groups are accumulated in ascending order by an FP64 fma and the total
 * takes one BF16 rounding with the double-rounding tie repaired; gate is clamped from above and up on both sides by
 * swiglu_limit, the FP32 SiLU * up * routed weight takes one BF16 cast and that row is quantized again for the down
 * projection. Replaces moe_act_quant_e4m0, moe_ffn_dispatch_{gate_up,down}_e2m1_e8m0_exact and
 * moe_ffn_{gate_up,down}_e4m3_block32_exact (kernels/moe_ffn.cu:463-467,601-700; kernels/q38_contract.cuh:53-101,
 * 153-170; host: MoeExpertW4A8 / w8a8, src/backend/cuda/moe/w4a8.rs:248-420), for rows x top_k choices in one call.
 * act_mode = FFMOE_ACT_E4M3_E8M0_32_F32 selects the reference's FP32-chain kernels instead (per 8-element chunk an fma
 * chain, chunk sums scaled in FP32, 32-lane xor-butterfly sum; moe_ffn_dispatch_{gate_up,down}_e2m1_e8m0 and
 * moe_ffn_{gate_up,down}_e4m3_block32), reproduced lane for lane.
 * args: act_mode as above, routed_weight = FFMOE_WEIGHT_BEFORE_DOWN_F32, weights_f32 = 1,
 * swiglu_limit > 0; swiglu is ignored (the contract fixes it). contributions[row, choice, :] already carry the routed
 * weight. A choice that is inactive, out of range, not valid or stale writes nothing and keeps done = 0 (the reference
 * traps). scratch: ffmoe_e8m0_scratch_bytes. */
uint64_t ffmoe_e8m0_scratch_bytes(int rows, int top_k, int hidden, int inter, int shared_inter);
int ffmoe_decode_contribute_e8m0(const ffmoe_expert_table* table, const ffmoe_shared_expert* shared, const ffmoe_decode* args,
                                 void* stream);
/* x [rows, k] BF16 -> codes [rows, k] E4M3, scales [rows, k / 32] E8M0 (moe_act_quant_e4m0, kernels/moe_ffn.cu:444-467). */
int ffmoe_act_quant_e8m0(const void* x, void* codes, void* scales, int rows, int k, void* stream);

/* One token, selection inside the gate/up launch: logits [experts] FP32 (from ffmoe_route_logits_f32) go in, and the
 * top-k selection of ffmoe_route_topk_noaux (same arithmetic, bit for bit) runs in the prologue of every block of the
 * gate/up launch instead of a launch of its own; args->ids and args->weights (f32) are OUTPUTS here, written for the
 * down launch and the combine, and args->done is cleared. Replaces moe_route_select_noaux + moe_gate_up + moe_down for
 * rows == 1 (kernels/moe_route.cu:315-390, kernels/moe_ffn.cu:98-302) with one launch less. Needs experts = 64 * 2^n,
 * FFMOE_ACT_BF16, f32 weights, no active mask; FFMOE_ERR_UNSUPPORTED otherwise (use the separate calls). */
int ffmoe_decode_contribute_from_logits(const ffmoe_expert_table* table, const ffmoe_shared_expert* shared,
                                        const ffmoe_decode* args, const float* logits, const float* bias,
                                        int score_mode, float routed_scaling, int n_group, int topk_group, void* stream);

/* One token, everything after the router logits in ONE launch: top-k selection (when logits != NULL; same arithmetic as
 * ffmoe_route_topk_noaux, args->ids and args->weights (f32) are then OUTPUTS), gate/up + SwiGLU, down, routing weight
 * and the ordered combine into y [hidden] BF16. Replaces the launches moe_route_select_noaux, moe_gate_up, moe_down /
 * moe_ffn_weight_f32 and moe_combine* of NativeMoe::run for one token (src/backend/cuda/moe/decode.rs:1187-1297); ids,
 * weights and y are bit-identical to those launches. logits == NULL: args->ids / weights / active are inputs as in
 * ffmoe_decode_contribute. The grid stays resident and hands activations between its blocks through args->scratch
 * (ffmoe_decode_scratch_bytes bytes, which must be zero-filled ONCE before the first call that uses it: a word of
 * the arena counts as an activation of the launch only if its upper half carries the launch's non-zero 16-bit tag,
 * and the last block of every launch hands the arena back zero-filled. The arena belongs to this entry point: the
 * other entry points store untagged BF16 pairs in their scratch, whose upper halves can equal a tag, so zero-fill it
 * again after lending it to one of them);
 * contributions, shared_out and done are not written. Bit 0 of *status is set for
 * a live choice naming an expert that is out of range or not valid (its contribution is skipped), bit 1 if a block
 * gave up waiting for another (y is then not valid; happens only when the grid cannot be resident at once, e.g. two
 * such launches running concurrently on one GPU, each holding part of the CUs; FFMOE_TOKEN_SPIN_LIMIT, read at every
 * call, sets the number of polls a block makes before it gives up, default 100000). Do not capture this call into a
 * HIP graph: the tag is a kernel argument drawn from a host-side counter at call time, so every replay of a captured
 * launch would carry the same tag and could take a late word of the replay before for its own. FFMOE_ERR_UNSUPPORTED
 * (nothing launched): rows != 1, a shape outside the kernel's register buffers, or a shared expert of another format; use
 * the separate calls then. */
int ffmoe_decode_token_layer(const ffmoe_expert_table* table, const ffmoe_shared_expert* shared, const ffmoe_decode* args,
                             const float* logits, const float* bias, int score_mode, float routed_scaling, int n_group,
                             int topk_group, const void* scale, void* y, uint32_t* status, int combine_mode, void* stream);

/* One token, everything after the router logits in TWO launches (the default of the host mirror's NativeMoe for one row):
 * launch 1 = top-k selection (same arithmetic as ffmoe_route_topk_noaux; args->ids and args->weights (f32) are OUTPUTS,
 * args->done is cleared) in the prologue of the gate/up + SwiGLU launch, hidden behind the shared expert's rows, which
 * need no routing; launch 2 = ffmoe_decode_finish (down, routing weight and the ordered combine into y [hidden] BF16).
 * Replaces moe_route_select_noaux, moe_gate_up, moe_down / moe_ffn_weight_f32 and moe_combine* of NativeMoe::run for one
 * token (src/backend/cuda/moe/decode.rs:1187-1297; kernels/moe_route.cu:315-390, kernels/moe_ffn.cu:98-302,894-908,
 * kernels/moe_combine.cu:51-116,541-613); ids, weights and y are bit-identical to the separate calls. contributions,
 * shared_out are not written. Arguments as ffmoe_decode_token_layer; the scratch arena needs no preparation.
 * A shared expert of another format or width than the table's (BF16 next to NVFP4 experts) cannot share the routed
 * launches: its gate/up and down launches run first with the kernels of its own format (the selection then sits in the
 * prologue of ITS gate/up launch), args->shared_out receives its BF16 row and the finish adds that row - four launches,
 * the same bits. (NVFP4 experts next to a BF16 shared expert at hidden 2048 / 4096 / 7168 / 8192: the shared gate/up rows run
 * inside the routed gate/up launch, in BF16, and only the shared down launch is its own - three launches.)
 * FFMOE_ERR_UNSUPPORTED (nothing launched): rows != 1, top_k > 8, experts not 64 * 2^n, an active mask or epochs, or
 * down rows beyond the kernel's register buffers. */
int ffmoe_decode_token_forward(const ffmoe_expert_table* table, const ffmoe_shared_expert* shared, const ffmoe_decode* args,
                               const float* logits, const float* bias, int score_mode, float routed_scaling, int n_group,
                               int topk_group, const void* scale, void* y, uint32_t* status, int combine_mode, void* stream);
/* One launch of the same call, for timing a kernel alone: stage 0 = selection + gate/up, stage 1 = down + combine
 * (stage 0 then stage 1 with the same arguments equals ffmoe_decode_token_forward; with a shared expert of another
 * format or width stage 0 also holds that expert's two launches). No counterpart in the reference. */
int ffmoe_decode_token_forward_stage(const ffmoe_expert_table* table, const ffmoe_shared_expert* shared, const ffmoe_decode* args,
                                     const float* logits, const float* bias, int score_mode, float routed_scaling, int n_group,
                                     int topk_group, const void* scale, void* y, uint32_t* status, int combine_mode, int stage,
                                     void* stream);

/* One-token finish: the down projection of every live choice and of the shared expert, the routing weight and the
 * ordered combine in ONE launch, for rows == 1. Call after ffmoe_decode_contribute_stage(table, shared, args, 0, stream)
 * with the same table / shared / args (the gate/up activations are taken from args->scratch); writes y[hidden] and
 * nothing else (contributions, shared_out and done stay untouched). y is bit-identical to
 * ffmoe_decode_contribute_stage(.., 1, ..) followed by ffmoe_combine(mode): it replaces moe_down + moe_ffn_weight_f32 +
 * moe_combine{,_ungated,_bf16,_accum,_routed} (kernels/moe_ffn.cu:211-302,894-908; kernels/moe_combine.cu:51-116,
 * 541-613) of NativeMoe::run (src/backend/cuda/moe/decode.rs:1187-1297). args->active plays the role of final_active;
 * *status |= 1 when a live choice names an expert that is out of range or not valid.
 * Returns FFMOE_ERR_UNSUPPORTED (nothing launched) when the shape is outside the fast path (rows != 1, top_k > 8,
 * shared expert of another format or width, rows of the down matrix longer than two 64-lane steps): run the
 * two separate calls then. */
int ffmoe_decode_finish(const ffmoe_expert_table* table, const ffmoe_shared_expert* shared, const ffmoe_decode* args,
                        const void* scale, void* y, uint32_t* status, int combine_mode, void* stream);

/* ------------------------------------------------------------------------------------------------
 * Expert residency protocol (src/experts/arena.rs:220-483). With every expert resident the table is constant and
 * none of this is needed; an engine that swaps experts in and out publishes each change on the stream and masks
 * the routing against the table before the expert launches.
 */

/* Replaces moe_slot_publish (kernels/moe_route.cu:650-670): stream-ordered publication of expert `incoming` (its six
 * slot addresses and a strictly increasing epoch) and retirement of `victim` (-1 = none): valid[victim] = 0,
 * generation[victim] = 0, its slot row cleared. Contract violations (bad ids, NULL or misaligned addresses, epoch 0,
 * epoch not above the one of a slot that is already valid) are reported on the host where the arguments show them and
 * through *status |= 1 where only the device table does. */
int ffmoe_slot_publish(uint64_t* slots, uint32_t* valid, uint64_t* generation, int experts, int incoming, int victim,
                       const uint64_t incoming_slot[6], uint64_t epoch, uint32_t* status, void* stream);

/* Replaces moe_route_mask (kernels/moe_route.cu:672-681): active[a] = valid[ids[a]], assignment_gen[a] = its epoch
 * (0 when not resident). *status |= 1 for an id out of range or a table entry that is valid without an epoch. */
int ffmoe_route_mask(const int* ids, const uint32_t* valid, const uint64_t* generation, uint32_t* active,
                     uint64_t* assignment_gen, uint32_t* status, int assignments, int experts, void* stream);

/* ------------------------------------------------------------------------------------------------
 * Standalone linears, M <= 16 "skinny" and beyond. y[M,N] = x[M,K] * W[N,K]^T, BF16 in / BF16 out.
 */

/* Replaces fp8_quant_f32_128 (kernels/fp8_linear.cu:12-48): per (row, 128-group) scale = amax*(1/448),
 * codes = e4m3_rne(clamp(x / max(scale,1e-12), +-448)). scales [m, ceil(k/128)] f32. */
int ffmoe_quant_fp8_f32_128(const void* x, void* codes, float* scales, int m, int k, void* stream);

/* Replaces Fp8Ops::bind_block + Fp8BlockPlan::run (src/backend/cuda/linear.rs:571-660) on pre-quantized
 * activations: kernels fp8_block_f32_128_decode/_mma (kernels/fp8_linear.cu:194-206). */
int ffmoe_linear_fp8_block_w8a8(const void* w_codes, const float* w_scales, const void* x_codes,
                                const float* x_scales, void* y, int m, int n, int k, void* stream);

/* BF16 activations against a 128x128-f32 block-scaled FP8 weight.
 * act_mode FFMOE_ACT_BF16: w = bf16(e4m3*scale) in registers (the W8A16 contract of fp8_gemv_bf16 /
 * fp8_skinny_bf16_mM, kernels/fp8_linear.cu:353-511, with f32 instead of BF16 scales). Up to 4 rows are FP32 fma
 * chains per weight row; more rows (k % 64 == 0, n % 16 == 0) take the same effective weights through the BF16 matrix
 * cores, 16 rows per pass over the weights: FP32 accumulation in the instruction's order, same tolerance.
 * act_mode FFMOE_ACT_FP8_BLOCK128: NativeProjection::run (linear.rs:1352-1405): quantize then W8A8;
 * needs scratch of m*k + 4*m*ceil(k/128) bytes (256-byte aligned), otherwise scratch may be NULL. */
int ffmoe_linear_fp8_block(const void* w_codes, const float* w_scales, const void* x, void* y,
                           int m, int n, int k, int act_mode, void* scratch, uint64_t scratch_bytes, void* stream);

/* Several independent block-FP8 skinny linears of one shape in ONE launch, W8A16 arithmetic (act_mode FFMOE_ACT_BF16 of
 * ffmoe_linear_fp8_block): the projections a decoder layer applies side by side (the reference plans them one
 * Fp8BlockPlan each, src/linear_plan.rs, src/backend/cuda/linear.rs:571-660, and launches fp8_gemv_bf16 /
 * fp8_skinny_bf16_mM per projection, kernels/fp8_linear.cu:353-511; it has no batched launch). A 14.7 MB matrix streams for
 * about 2.3 us on this GPU against 2 - 3 us of launch start-up, so single calls cannot pass ~40 % of the HBM rate;
 * a batch pays the start-up once. `items` is a DEVICE array of `count` descriptors (device addresses of codes [n,k],
 * f32 block scales, x [m,k] BF16, y [m,n] BF16), caller-owned like a slot table; 1 <= m <= 4. Every item's y is
 * bit-identical to its own ffmoe_linear_fp8_block call. Items must not alias each other's outputs. */
typedef struct ffmoe_linear_item { uint64_t w_codes, w_scales, x, y; } ffmoe_linear_item;
int ffmoe_linear_fp8_block_batch(const ffmoe_linear_item* items, int count, int m, int n, int k, void* stream);

/* Replaces NvFp4Ops::gemm (linear.rs:488-551; kernels/nvfp4_linear.cu:50-252): W4A16,
 * w = bf16(e2m1 * (e4m3(scale) * global)). global_scale is a device pointer to one f32. k % 16 == 0. Up to 16 rows
 * run the direct kernel (the reference's host mirror order); more rows with k % 128 == 0 and n % 16 == 0 the BF16
 * matrix cores, as the reference switches to its MMA kernel there (kernels/nvfp4_linear.cu:262-573). */
int ffmoe_linear_nvfp4(const void* w_codes, const void* w_scales, const float* global_scale,
                       const void* x, void* y, int m, int n, int k, void* stream);

/* Replaces gemm_skinny_bf16 (kernels/gemm_skinny.cu:509-675): BF16 weights [n,k]. More than 4 rows with k % 32 == 0
 * and n % 16 == 0 run on the BF16 matrix cores (FP32 accumulation in the instruction's order). */
int ffmoe_gemm_skinny_bf16(const void* w, const void* x, void* y, int m, int n, int k, void* stream);

/* Replaces silu_mul_split / silu_mul_split_clamped (kernels/act.cu:65-99, :125-159):
 * y = swiglu(gate, up) over dense [rows, width] BF16 regions, width % 8 == 0. */
int ffmoe_swiglu(const void* gate, const void* up, void* y, int rows, int width, int mode, float limit, void* stream);

/* ------------------------------------------------------------------------------------------------
 * Combine. Replaces CombineOps (src/backend/cuda/moe/combine.rs:440-760; kernels/moe_combine.cu).
 */

/* scale[r] = bf16(sigmoid(bf16(x[r,:] . seg))). Replaces moe_shared_scale (kernels/moe_combine.cu:21-49). */
int ffmoe_shared_scale(const void* x, const void* seg, void* scale, int rows, int hidden, void* stream);

/* y[r,:] from contributions [rows,top_k,hidden] and shared_out [rows,hidden] in the order of `mode`.
 * ids/done/final_active are [rows,top_k]; a slot with done != final_active is a protocol violation: the
 * reference traps (kernels/moe_combine.cu:56-58); here the row is still combined over final_active and bit 0
 * of *status (device u32, may be NULL) is set. final_active NULL = all active; done NULL = not checked.
 * ACCUM modes ignore ids/done/final_active. */
int ffmoe_combine(const void* contributions, const void* shared_out, const void* scale, const int* ids,
                  const uint32_t* done, const uint32_t* final_active, void* y, uint32_t* status,
                  int rows, int top_k, int hidden, int mode, void* stream);

/* Combine group with the residual add, and the peer-join form. Replaces moe_combine_residual{,_scalar} and
 * moe_join_routed_residual{,_scalar} (kernels/moe_combine.cu:246-533; CombineOps::combine_residual / join_routed*,
 * src/backend/cuda/moe/combine.rs:608-760):
 *   ff = BF16(BF16(routed) + gated),  gated = BF16(scale_row * shared) if seg != NULL else shared,
 *   scale_row = ffmoe_shared_scale(x_row, seg) computed in the same launch,
 *   routed = ordered FP32 sum of the row's live contributions (contributions != NULL) or routed_in (the sum a peer
 *   computed; exactly one of the two is given),
 *   y_out != NULL: y_out = ff; else residual = BF16(residual + ff) in place.
 * x row r starts at x + r * x_stride elements. */
int ffmoe_combine_residual(const void* contributions, const void* routed_in, const void* shared_out, const void* seg,
                           const void* x, long long x_stride, const int* ids, const uint32_t* done,
                           const uint32_t* final_active, void* residual, void* y_out, uint32_t* status,
                           int rows, int top_k, int hidden, void* stream);

/* ------------------------------------------------------------------------------------------------
 * Prefill: many tokens, grouped by expert on the device (no host synchronisation: grids are sized from upper
 * bounds and kernels read the device-side counts), then two grouped GEMMs on the FP8 matrix cores in
 * FFMOE_ACT_FP8_BLOCK128 arithmetic: x is quantized per (row, 128) once, gate/up + SwiGLU (two-branch sigmoid,
 * kernels/act.cu:125-159) writes BF16 activations in expert order, they are re-quantized, and down x routing
 * weight is scattered to contributions[row, choice, :] with done[row, choice] = 1. Per assignment the arithmetic
 * equals the reference's <=16-row block-FP8 pipeline (NativeMoe::run, src/backend/cuda/moe/decode.rs:1187-1297;
 * kernels/moe_ffn.cu:870-908), which is how the reference runs block-FP8 prefill (in 16-row chunks).
 * Replaces PrefillOps::prefill_contribute (src/backend/cuda/moe/prefill.rs:1033-1408) and kernels moe_count_scan /
 * moe_permute / moe_gemm_* / silu_mul / moe_scatter_rows (kernels/moe_prefill.cu:364-553).
 * That is act_mode FFMOE_ACT_FP8_BLOCK128 (W8A8) on FFMOE_FMT_FP8_BLOCK128 tables, hidden and inter multiples of 128.
 * The same act_mode on an FFMOE_FMT_NVFP4 table is W4A8 on the FP8 matrix cores: the kernels turn every NVFP4 weight
 * into E4M3 on its way through LDS - E2M1 value x E4M3 group scale / 8, rounded to nearest even (6 x 448 / 8 = 336 stays
 * inside E4M3) - and use 8 x the matrix's f32 global scale where a block-FP8 matrix has its 128 x 128 scales; everything
 * else (activation quantizer, per-128 dots, SwiGLU, re-quantization, routing weight) is the W8A8 pipeline above. The
 * second rounding of the weights makes this an arithmetic of its own (the reference's NVFP4 GEMM dequantizes to BF16,
 * kernels/nvfp4_linear.cu:262-573, and has no FP8 form): results equal, bit for bit, a block-FP8 cohort on those derived
 * codes. The shared expert may be FFMOE_FMT_FP8_BLOCK128 or FFMOE_FMT_NVFP4 then.
 * act_mode FFMOE_ACT_BF16 runs the cohort in the decode path's W*A16 arithmetic instead: experts of any format
 * (block FP8, NVFP4, per-channel FP8, BF16; the shared expert may have another format than the table) are
 * dequantized in registers to the BF16 effective weights of ffmoe_decode_contribute, activations stay BF16 between
 * the stages, and the grouped GEMMs run on the BF16 matrix cores with FP32 accumulation: what the reference's prefill
 * computes for its per-channel FP8 and BF16 experts (moe_gemm_w8a16 and the BF16 grouped GEMM,
 * kernels/moe_prefill.cu:157-350, whose summation order is bounded by tolerance only), with the decode path's SwiGLU
 * roundings and routing-weight boundaries; hidden and inter multiples of 64 (128 for block FP8).
 * FFMOE_FMT_E2M1_E8M0 tables with act_mode FFMOE_ACT_E4M3_E8M0_32 run the W4A8 contract of ffmoe_decode_contribute_e8m0
 * for a cohort on the MX matrix cores (v_mfma_scale_f32_16x16x128_f8f6f4 takes E2M1 / E4M3 operands with E8M0 scales
 * per 32 columns as they are): x is quantized per 32, gate/up dots are rounded to BF16, clamped SwiGLU x the f32
 * routing weight (routed_weight = FFMOE_WEIGHT_BEFORE_DOWN_F32, weights_f32 = 1, swiglu_limit > 0) gives the BF16
 * activations, they are quantized per 32 again, and the down dots are stored as BF16 contributions; the shared expert
 * must be FFMOE_FMT_E4M3_E8M0_32. Same operands and stage boundaries as the exact entry, but the matrix core adds
 * the products in FP32 in its own order: this is the tolerance-checked variant (kernels/moe_ffn.cu:398-867 is the
 * contract; the reference has no cohort kernel for it). hidden, inter multiples of 128; rows * top_k <= 65535.
 * Assignments whose id is out of range, whose expert is not valid or whose active flag is 0 contribute nothing and
 * keep done = 0.
 */
typedef struct ffmoe_prefill {
  int rows, top_k;
  int act_mode;            /* FFMOE_ACT_FP8_BLOCK128, FFMOE_ACT_BF16, or FFMOE_ACT_E4M3_E8M0_32 (E2M1/E8M0 tables) */
  int swiglu; float swiglu_limit;
  int routed_weight;
  int weights_f32;
  const void* x;           /* [rows, hidden] BF16 */
  const int* ids;          /* [rows, top_k] */
  const uint32_t* active;  /* [rows, top_k] or NULL */
  const void* weights;     /* [rows, top_k] */
  void* contributions;     /* [rows, top_k, hidden] BF16 */
  uint32_t* done;          /* [rows, top_k] or NULL */
  void* scratch; uint64_t scratch_bytes;
  const ffmoe_shared_expert* shared; /* always-on expert (W8A8: FFMOE_FMT_FP8_BLOCK128), or NULL */
  void* shared_out;        /* [rows, hidden] BF16 = bf16(down output), no routing weight (with shared) */
  const uint64_t* assignment_gen; /* as in ffmoe_decode, or NULL */
} ffmoe_prefill;

uint64_t ffmoe_prefill_scratch_bytes(int rows, int top_k, int experts, int hidden, int inter, int shared_inter);
int ffmoe_prefill_contribute(const ffmoe_expert_table* table, const ffmoe_prefill* args, void* stream);
/* One step of the same call, for timing a kernel alone (the steps of one cohort must run in order once before any of
 * them is repeated): 0 = count / scan / fill + quantize x, 1 = gate/up GEMM + SwiGLU, 2 = re-quantize activations,
 * 3 = down GEMM + routing weight + scatter. No counterpart in the reference. */
int ffmoe_prefill_contribute_stage(const ffmoe_expert_table* table, const ffmoe_prefill* args, int stage, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* FFMOE_H */
