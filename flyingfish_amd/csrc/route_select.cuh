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

__device__ __forceinline__ uint32_t wave_max_u32(uint32_t v) {
  v = max(v, uint32_t(dpp_or<DPP_QUAD_SWAP1, 0xf>(int(v), int(v))));
  v = max(v, uint32_t(dpp_or<DPP_QUAD_SWAP2, 0xf>(int(v), int(v))));
  v = max(v, uint32_t(dpp_or<DPP_ROW_HALF_MIRROR, 0xf>(int(v), int(v))));
  v = max(v, uint32_t(dpp_or<DPP_ROW_MIRROR, 0xf>(int(v), int(v))));
  v = max(v, uint32_t(dpp_or<DPP_ROW_BCAST15, 0xa>(int(v), int(v))));
  v = max(v, uint32_t(dpp_or<DPP_ROW_BCAST31, 0xc>(int(v), int(v))));
  return uint32_t(__builtin_amdgcn_readlane(int(v), 63));
}

// One wave selects for one row. Requires experts == 64 * C and, with groups, experts / n_group a multiple of C whose
// lane span is a power of two. score[] = unbiased scores, select[] = score + bias of the lane's C candidates.
template <int C>
__device__ __forceinline__ void wave_select_noaux(const float (&score)[C], const float (&select)[C], int lane, int experts,
                                                  int top_k, float routed_scaling, int n_group, int topk_group,
                                                  int* __restrict__ ids_row, void* __restrict__ weights_row, int weights_f32) {
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
  float tsum = 0.0f;
  float my_w = 0.0f;  // lane r keeps the score of the r-th pick
  int my_id = 0;
  // Enough candidates for top_k picks (every sane configuration): a round is the wave maximum of the 32-bit orderable scores
  // and then the lowest id that has it - the order of the 64-bit keys below (score descending, id ascending: ids ascend
  // with the lane and inside the lane), in a quarter of the dependent instructions.
  const int candidates = __builtin_popcountll(__ballot(allowed)) * C;
  if (candidates >= top_k) {
    uint32_t k32[C];
#pragma unroll
    for (int j = 0; j < C; ++j) k32[j] = allowed ? orderable(select[j]) : 0u;  // 0: below every score, also -inf
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
