// Internal structures of the decode path (not part of the C ABI).
#pragma once
#include <stdint.h>

#define FFMOE_DECODE_RG 8              /* rows of one expert served by one pass over its weights */
#define FFMOE_DECODE_MAX_ASSIGN 4096   /* rows * top_k handled by the single-block grouping kernel */
#define FFMOE_STATIC_SCRATCH_BYTES (8ull << 20)  /* built-in arena of ffmoe_decode_contribute_static, per GPU */

namespace ffmoe {

struct GroupDesc {
  int expert;                 // expert id, -1 = shared expert
  int n;                      // rows in this group (0 = nothing to do)
  int row[FFMOE_DECODE_RG];   // token row of each member
  int slot[FFMOE_DECODE_RG];  // activation / contribution slot: assignment index, or rows*top_k + row for the shared expert
  int pad[2];
};

// What the one-token finish needs to know about the live choices, in combine order, resolved by the gate/up launch that
// selected them (block 0, right behind the selection): the finish then starts from one load of this record instead of the
// chain ids -> slot table, and ranks nothing.
#define FFMOE_FINISH_ROUTED 8
struct FinishDesc {
  int n;       // live routed groups
  int bad;     // 1: a selected expert is out of range or not valid (the finish reports it in its status word)
  int pad[2];
  uint64_t codes[FFMOE_FINISH_ROUTED], scales[FFMOE_FINISH_ROUTED];  // down matrix of group g
  float glob[FFMOE_FINISH_ROUTED], wk[FFMOE_FINISH_ROUTED];          // its global scale (NVFP4) and routing weight
  int slot[FFMOE_FINISH_ROUTED];                                     // its choice index = activation row
};

// Top-k selection inside the gate/up kernel (one token row): every block selects from the FP32 logits in its prologue,
// block 0 publishes ids and weights for the later launches. logits == NULL: ids and weights are inputs.
struct RouteInline {
  const float* logits;  // [experts]
  const float* bias;    // [experts] or NULL
  int score_mode, n_group, topk_group;
  float routed_scaling;
  int select_k;         // choices to select; 0: the launch's own top_k (a shared-expert-only launch has top_k = 0)
  FinishDesc* finish_desc;  // block 0 also resolves the live choices for the finish launch of the same call, or NULL
  int finish_ordered;       // their order: 1 ascending expert id (stable), 0 choice order (the accumulate combine modes)
};

struct DecodeParams {
  RouteInline route;
  int rows, top_k, experts, hidden, inter, shared_inter, has_shared;
  int swiglu, routed_weight, weights_f32;
  float swiglu_limit;
  const uint16_t* x;
  const int* ids;
  const uint32_t* active;
  const void* weights;
  const uint64_t* slots;
  const uint32_t* valid;
  const uint64_t* generation;      // per expert, or NULL
  const uint64_t* assignment_gen;  // per assignment, or NULL
  const float* global_scales;
  uint64_t shared_slot[6];
  float shared_global[3];
  uint16_t* contributions;
  uint16_t* shared_out;
  uint32_t* done;
  uint16_t* h;       // [rows*top_k + rows, h_stride] BF16 activations between the two stages
  int h_stride;
  GroupDesc* groups;        // NULL = one group per assignment, built on the fly
  int* counters;            // {routed groups, shared groups} when groups != NULL
};

// one-token finish (down + routing weight + combine in one launch)
struct FinishParams {
  DecodeParams d;
  const uint16_t* scale;  // [1] BF16 shared-expert gate (FFMOE_COMBINE_GATED)
  uint16_t* y;            // [hidden]
  uint32_t* status;       // |= 1 when a live choice names an expert that is out of range or not valid
  int mode;               // FFMOE_COMBINE_*
  const FinishDesc* desc;  // the live choices as the gate/up launch of the same call resolved them, or NULL: from ids
  const uint16_t* shared_ready;  // [hidden] BF16 output of a shared expert that other launches computed (another format or
                                 // width than the table's), or NULL: the finish computes d.has_shared's expert itself
  // the whole token layer in one launch (k_token_layer)
  int whole;              // 0: one-token finish, 1: selection, gate/up, down and combine
  uint32_t* h32;          // [(top_k + 1), d.h_stride] activations as (launch tag << 16 | BF16) words; row top_k = shared expert
  uint32_t tag;           // 1 .. 65535, the tag of this launch's activation words (host-side launch counter)
  unsigned int* exited;   // blocks that left the kernel; the last one clears it and advances gen
  unsigned int* claims;   // 128 claim counters, 32 words apart: gate/up and down phase of up to 64 grid partitions
  unsigned int spin_limit;
  int dynamic;            // 1: work items claimed from the counters, 0: fixed round-robin shares
};

}  // namespace ffmoe
