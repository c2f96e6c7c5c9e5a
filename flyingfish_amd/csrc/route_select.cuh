// Single-wave top-k selection for the noaux router (sigmoid / sqrt-softplus scores + selection bias, optional group
// filter), shared by the routing kernels and by the decode kernel that selects in its own prologue.
#pragma once
#include "common.cuh"
#include "../../include/ffmoe.h"

namespace ffmoe {

// ---------------------------------------------------------------------------------------------
// Single-wave selection, everything in registers: lane L holds the C = experts / 64 candidates L*C .. L*C+C-1 as
// 64-bit keys (orderable score bits, ~id), so "higher score, then lower id" is one unsigned compare and keys are
// unique. top_k rounds of (lane-local max, DPP wave max, retire the winner) reproduce the reference's block-wide
// arg-max rounds (kernels/moe_route.cu:349-377) without LDS or barriers.
__device__ __forceinline__ uint32_t orderable(float f) {
  const uint32_t b = __float_as_uint(f);
  return b ^ ((b >> 31) ? 0xffffffffu : 0x80000000u);
}
__device__ __forceinline__ uint64_t max_u64(uint64_t a, uint64_t b) { return a > b ? a : b; }
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ uint64_t dpp_u64(uint64_t v) {
  const int lo = dpp_or<CTRL, ROW_MASK>(int(uint32_t(v)), int(uint32_t(v)));
  const int hi = dpp_or<CTRL, ROW_MASK>(int(uint32_t(v >> 32)), int(uint32_t(v >> 32)));
  return (uint64_t(uint32_t(hi)) << 32) | uint32_t(lo);
}
__device__ __forceinline__ uint64_t wave_max_u64(uint64_t v) {
  v = max_u64(v, dpp_u64<DPP_QUAD_SWAP1, 0xf>(v));
  v = max_u64(v, dpp_u64<DPP_QUAD_SWAP2, 0xf>(v));
  v = max_u64(v, dpp_u64<DPP_ROW_HALF_MIRROR, 0xf>(v));
  v = max_u64(v, dpp_u64<DPP_ROW_MIRROR, 0xf>(v));
  v = max_u64(v, dpp_u64<DPP_ROW_BCAST15, 0xa>(v));
  v = max_u64(v, dpp_u64<DPP_ROW_BCAST31, 0xc>(v));
  const uint32_t lo = uint32_t(__builtin_amdgcn_readlane(int(uint32_t(v)), 63));
  const uint32_t hi = uint32_t(__builtin_amdgcn_readlane(int(uint32_t(v >> 32)), 63));
  return (uint64_t(hi) << 32) | lo;
}

// Wave maximum, returned in a scalar register. The cross-lane modes ride on the max itself (the compiler emits a move with
// the mode and a separate max); the waits the cross-lane reads need behind a vector write are spelled out, the
// compiler does not look into the block.
__device__ __forceinline__ uint32_t wave_max_u32(uint32_t v) {
  uint32_t out;
  asm volatile(
      "s_nop 1\n\tv_max_u32_dpp %1, %1, %1 quad_perm:[1,0,3,2] row_mask:0xf bank_mask:0xf\n\t"
      "s_nop 1\n\tv_max_u32_dpp %1, %1, %1 quad_perm:[2,3,0,1] row_mask:0xf bank_mask:0xf\n\t"
      "s_nop 1\n\tv_max_u32_dpp %1, %1, %1 row_half_mirror row_mask:0xf bank_mask:0xf\n\t"
      "s_nop 1\n\tv_max_u32_dpp %1, %1, %1 row_mirror row_mask:0xf bank_mask:0xf\n\t"
      "s_nop 1\n\tv_max_u32_dpp %1, %1, %1 row_bcast:15 row_mask:0xa bank_mask:0xf\n\t"
      "s_nop 1\n\tv_max_u32_dpp %1, %1, %1 row_bcast:31 row_mask:0xc bank_mask:0xf\n\t"
      "s_nop 1\n\tv_readlane_b32 %0, %1, 63\n\ts_nop 3"
      : "=s"(out), "+v"(v));
  return out;
}

// One wave selects for one row, in two parts so that a caller can do the first before something it has to wait for and the
// second behind it. Requires experts == 64 * C and, with groups, experts / n_group a multiple of C whose lane span is a
// power of two. score[] = unbiased scores, select[] = score + bias of the lane's C candidates.
template <int C>
struct NoauxState {
  float score[C], select[C];
  uint32_t key[C];  // heads form: the lane's candidates in pick order, barred and retired ones 0
  int pos[C];       // the register index (id % C) that goes with key[]
  bool allowed;     // the lane's group passed the group filter
  bool heads;       // wave-uniform: enough candidates for top_k picks and few enough per lane to sort them
};

// Part one: group filter, keys, the lane's candidates sorted.
template <int C>
__device__ __forceinline__ void wave_select_prepare(NoauxState<C>& st, int lane, int experts, int top_k, int n_group, int topk_group) {
  const float (&select)[C] = st.select;
  bool allowed = true;
  if (n_group > 1) {
    // the two largest selection scores of the lane, then of the lanes of its group (values only: the group score
    // is their sum, so ties between members do not matter)
    float a = -INFINITY, b = -INFINITY;
#pragma unroll
    for (int j = 0; j < C; ++j) {
      const float v = select[j];
      b = fmaxf(b, fminf(a, v));
      a = fmaxf(a, v);
    }
    const int span = (experts / n_group) / C;  // lanes per group
    // Merging the two largest of two disjoint sets of lanes is symmetric, and after a level all lanes of a merged set hold
    // the same pair, so the partner may be any lane of the neighbouring set: the cross-lane modes of the vector ALU reach
    // one for sets of up to 8 lanes (pairs, quads, the mirrored half row, the mirrored row); wider sets go through LDS.
    auto merge = [&](float oa, float ob) {
      const float na = fmaxf(a, oa);
      b = fmaxf(fminf(a, oa), fmaxf(b, ob));
      a = na;
    };
    auto fdpp = [](auto ctrl, float v) {
      return __builtin_bit_cast(float, dpp_or<decltype(ctrl)::value, 0xf>(__builtin_bit_cast(int, v), __builtin_bit_cast(int, v)));
    };
    if (span > 1) merge(fdpp(std::integral_constant<int, DPP_QUAD_SWAP1>{}, a), fdpp(std::integral_constant<int, DPP_QUAD_SWAP1>{}, b));
    if (span > 2) merge(fdpp(std::integral_constant<int, DPP_QUAD_SWAP2>{}, a), fdpp(std::integral_constant<int, DPP_QUAD_SWAP2>{}, b));
    if (span > 4) merge(fdpp(std::integral_constant<int, DPP_ROW_HALF_MIRROR>{}, a), fdpp(std::integral_constant<int, DPP_ROW_HALF_MIRROR>{}, b));
    if (span > 8) merge(fdpp(std::integral_constant<int, DPP_ROW_MIRROR>{}, a), fdpp(std::integral_constant<int, DPP_ROW_MIRROR>{}, b));
    for (int off = 16; off < span; off <<= 1) merge(__shfl_xor(a, off, 64), __shfl_xor(b, off, 64));
    const float gscore = __fadd_rn(a, b);
    const int g = lane / span;
    // rank of the lane's group among the groups under (score desc, id asc)
    int rank = 0;
    for (int og = 0; og < n_group; ++og) {
      const float os = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, gscore), og * span));
      rank += (os > gscore || (os == gscore && og < g)) ? 1 : 0;
    }
    allowed = rank < topk_group;
  }
  st.allowed = allowed;
  const int candidates = __builtin_popcountll(__ballot(allowed)) * C;
  st.heads = C <= 8 && candidates >= top_k;
#pragma unroll
  for (int j = 0; j < C; ++j) { st.key[j] = allowed ? orderable(select[j]) : 0u; st.pos[j] = j; }  // 0: below every score, also -inf
  if (st.heads) {
    // The lane's candidates sorted once (score descending, id ascending: exchanges of neighbours only, so equal scores keep
    // their order).
#pragma unroll
    for (int pass = 0; pass < C - 1; ++pass) {
#pragma unroll
      for (int i = 0; i < C - 1 - pass; ++i) {
        const bool sw = st.key[i + 1] > st.key[i];
        const uint32_t ka = sw ? st.key[i + 1] : st.key[i], kb = sw ? st.key[i] : st.key[i + 1];
        const int pa = sw ? st.pos[i + 1] : st.pos[i], pb = sw ? st.pos[i] : st.pos[i + 1];
        st.key[i] = ka; st.key[i + 1] = kb; st.pos[i] = pa; st.pos[i + 1] = pb;
      }
    }
  }
}

// Part two: top_k rounds, normalized weights, ids and weights written by the lanes 0 .. top_k-1.
template <int C>
__device__ __forceinline__ void wave_select_pick(NoauxState<C>& st, int lane, int top_k, float routed_scaling,
                                                 int* __restrict__ ids_row, void* __restrict__ weights_row, int weights_f32) {
  const float (&score)[C] = st.score;
  const float (&select)[C] = st.select;
  const bool allowed = st.allowed;
  float tsum = 0.0f;
  float my_w = 0.0f;  // lane r keeps the score of the r-th pick
  int my_id = 0;
  // Enough candidates for top_k picks (every sane configuration): rounds on 32-bit orderable scores with "the lowest id that
  // has the maximum" - the order of the 64-bit keys at the bottom (score descending, id ascending: ids ascend with the lane
  // and inside the lane).
  const int candidates = __builtin_popcountll(__ballot(allowed)) * C;
  if (st.heads) {
    // A round looks at the lanes' heads only: wave maximum, the lowest lane whose head has it, that lane pops its head.
    // The picks' scores are fetched once at the end.
    uint32_t (&key)[C] = st.key;
    int (&pos)[C] = st.pos;
    for (int r = 0; r < top_k; ++r) {
      const uint32_t win = wave_max_u32(key[0]);
      const int wl = __builtin_ctzll(__ballot(key[0] == win));  // a retired or barred head (0) never equals a live maximum
      const int id = wl * C + __builtin_amdgcn_readlane(pos[0], wl);
      const bool me = lane == wl;
#pragma unroll
      for (int j = 0; j < C - 1; ++j) {
        key[j] = me ? key[j + 1] : key[j];
        pos[j] = me ? pos[j + 1] : pos[j];
      }
      key[C - 1] = me ? 0u : key[C - 1];
      my_id = lane == r ? id : my_id;
    }
    // lane r < top_k: the score of pick r sits in lane id / C, register id % C
#pragma unroll
    for (int j = 0; j < C; ++j) {
      const float sj = __shfl(score[j], my_id / C, 64);
      my_w = (my_id % C) == j ? sj : my_w;
    }
    for (int r = 0; r < top_k; ++r)
      tsum = __fadd_rn(tsum, __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, my_w), r)));
  } else if (C > 8 && candidates >= top_k) {
    // more than eight candidates per lane: a round is the wave maximum of the 32-bit orderable scores and then the lowest
    // id that has it
    uint32_t (&k32)[C] = st.key;
    for (int r = 0; r < top_k; ++r) {
      uint32_t m = k32[0];
#pragma unroll
      for (int j = 1; j < C; ++j) m = max(m, k32[j]);
      const uint32_t win = wave_max_u32(m);
      int first = C;
      float sc = 0.0f;
#pragma unroll
      for (int j = C - 1; j >= 0; --j) {
        const bool hit = k32[j] == win;
        first = hit ? j : first;
        sc = hit ? score[j] : sc;
      }
      const unsigned long long hits = __ballot(first < C);
      const int wl = __builtin_ctzll(hits);  // a retired or barred candidate (0) never equals a live maximum
      const int jw = __builtin_amdgcn_readlane(first, wl);
      const int id = wl * C + jw;
#pragma unroll
      for (int j = 0; j < C; ++j) k32[j] = (lane == wl && j == jw) ? 0u : k32[j];
      const float wsc = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, sc), wl));
      tsum = __fadd_rn(tsum, wsc);
      if (lane == r) { my_w = wsc; my_id = id; }
    }
  } else {
  uint64_t key[C];
#pragma unroll
  for (int j = 0; j < C; ++j)
    key[j] = allowed ? (uint64_t(orderable(select[j])) << 32) | uint32_t(~uint32_t(lane * C + j)) : 0ull;
  for (int r = 0; r < top_k; ++r) {
    uint64_t best = key[0];
#pragma unroll
    for (int j = 1; j < C; ++j) best = max_u64(best, key[j]);
    const uint64_t win = wave_max_u64(best);
    const int id = int(~uint32_t(win));
    float sc = 0.0f;
#pragma unroll
    for (int j = 0; j < C; ++j) {
      const bool hit = key[j] == win;
      sc = hit ? score[j] : sc;
      key[j] = hit ? 0ull : key[j];
    }
    const float wsc = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, sc), id / C));
    tsum = __fadd_rn(tsum, wsc);
    if (lane == r) { my_w = wsc; my_id = id; }
  }
  }
  if (lane < top_k) {
    const float w = __fmul_rn(__fdiv_rn(my_w, __fadd_rn(tsum, 1.0e-20f)), routed_scaling);
    ids_row[lane] = my_id;
    if (weights_f32) reinterpret_cast<float*>(weights_row)[lane] = w;
    else reinterpret_cast<uint16_t*>(weights_row)[lane] = f32_to_bf16(w);
  }
}

template <int C>
__device__ __forceinline__ void wave_select_noaux(const float (&score)[C], const float (&select)[C], int lane, int experts,
                                                  int top_k, float routed_scaling, int n_group, int topk_group,
                                                  int* __restrict__ ids_row, void* __restrict__ weights_row, int weights_f32) {
  NoauxState<C> st;
#pragma unroll
  for (int j = 0; j < C; ++j) { st.score[j] = score[j]; st.select[j] = select[j]; }
  wave_select_prepare<C>(st, lane, experts, top_k, n_group, topk_group);
  wave_select_pick<C>(st, lane, top_k, routed_scaling, ids_row, weights_row, weights_f32);
}

__device__ __forceinline__ float noaux_score(float l, int score_mode) {
  if (score_mode == FFMOE_NOAUX_SIGMOID) return sigmoid1(l);
  const float softplus = __fadd_rn(fmaxf(l, 0.0f), det_log1pf_unit(det_expf(-fabsf(l))));
  return __builtin_sqrtf(softplus);  // correctly rounded (hipcc default); __fsqrt_rn is the approximate native sqrt
}

template <int C>
__device__ __forceinline__ void wave_route_row(const float* __restrict__ logits_row, const float* __restrict__ bias_row,
                                               int lane, int experts, int top_k, int score_mode, float routed_scaling,
                                               int n_group, int topk_group, int* ids_row, void* weights_row, int weights_f32) {
  float score[C], select[C];
#pragma unroll
  for (int j = 0; j < C; ++j) {
    const int e = lane * C + j;
    const float l = logits_row[e];
    score[j] = noaux_score(l, score_mode);
    select[j] = __fadd_rn(score[j], bias_row ? bias_row[e] : 0.0f);
  }
  wave_select_noaux<C>(score, select, lane, experts, top_k, routed_scaling, n_group, topk_group, ids_row, weights_row, weights_f32);
}

// the same with the lane's C logits and biases already in registers (fetched early by the caller)
template <int C>
__device__ __forceinline__ void wave_route_row_preloaded(const float (&l)[C], const float (&b)[C], int lane, int experts, int top_k, int score_mode,
                                                         float routed_scaling, int n_group, int topk_group, int* ids_row, void* weights_row,
                                                         int weights_f32) {
  float score[C], select[C];
#pragma unroll
  for (int j = 0; j < C; ++j) {
    score[j] = noaux_score(l[j], score_mode);
    select[j] = __fadd_rn(score[j], b[j]);
  }
  wave_select_noaux<C>(score, select, lane, experts, top_k, routed_scaling, n_group, topk_group, ids_row, weights_row, weights_f32);
}

// Part one of the same from registers: scores, group filter, sorted candidates (part two is wave_select_pick)
template <int C>
__device__ __forceinline__ void wave_route_prepare_preloaded(NoauxState<C>& st, const float (&l)[C], const float (&b)[C], int lane, int experts,
                                                             int top_k, int score_mode, int n_group, int topk_group) {
#pragma unroll
  for (int j = 0; j < C; ++j) {
    st.score[j] = noaux_score(l[j], score_mode);
    st.select[j] = __fadd_rn(st.score[j], b[j]);
  }
  wave_select_prepare<C>(st, lane, experts, top_k, n_group, topk_group);
}

__device__ __forceinline__ void wave_route_dispatch(const float* logits_row, const float* bias_row, int lane, int experts,
                                                    int top_k, int score_mode, float routed_scaling, int n_group,
                                                    int topk_group, int* ids_row, void* weights_row, int weights_f32) {
  switch (experts >> 6) {
    case 1: wave_route_row<1>(logits_row, bias_row, lane, experts, top_k, score_mode, routed_scaling, n_group, topk_group, ids_row, weights_row, weights_f32); break;
    case 2: wave_route_row<2>(logits_row, bias_row, lane, experts, top_k, score_mode, routed_scaling, n_group, topk_group, ids_row, weights_row, weights_f32); break;
    case 4: wave_route_row<4>(logits_row, bias_row, lane, experts, top_k, score_mode, routed_scaling, n_group, topk_group, ids_row, weights_row, weights_f32); break;
    case 8: wave_route_row<8>(logits_row, bias_row, lane, experts, top_k, score_mode, routed_scaling, n_group, topk_group, ids_row, weights_row, weights_f32); break;
    default: wave_route_row<16>(logits_row, bias_row, lane, experts, top_k, score_mode, routed_scaling, n_group, topk_group, ids_row, weights_row, weights_f32); break;
  }
}

}  // namespace ffmoe
