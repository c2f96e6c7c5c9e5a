// One-token finish: down projection of every live choice and of the shared expert, routing weight and the ordered
// combine in a single launch (the last two launches of the decode layer, src/backend/cuda/moe/decode.rs:1187-1297:
// moe_down / moe_ffn_weight_f32 and moe_combine*, kernels/moe_ffn.cu:211-302,894-908, kernels/moe_combine.cu:51-116,
// 541-613).
//
// A unit is ONE output column d for ALL groups: the wave streams row d of every live expert's down matrix (and of the
// shared expert's) in combine order, so the per-expert results of a column meet in one lane and the combine needs no
// second pass over memory: contributions are neither written nor re-read and the combine launch disappears.
// The groups are visited in the order the combine adds them (ascending expert id, stable; choice order for the
// accumulate modes), so the parked sums are already in summation order. Per row the dot product is the same chunk ->
// lane mapping, step order and wave reduction as k_decode_stage, and the rounding boundaries are those of
// k_decode_stage + k_combine, so y is bit-identical to the three-launch path.
#pragma once
#include "decode_kernel.cuh"

namespace ffmoe {

template <class F, int S, int GMAX>
__global__ __launch_bounds__(256) void k_decode_finish(const FinishParams q) {
  const DecodeParams& p = q.d;
  extern __shared__ __align__(16) uint8_t xs[];  // [groups][inter] BF16 activations
  __shared__ int s_choice[FFMOE_MAX_TOP_K + 1];
  __shared__ int s_groups;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = uni(tid >> 6);
  const int K = p.top_k, I = p.inter, H = p.hidden;
  const bool ordered = !(q.mode == FFMOE_COMBINE_ACCUM_FP32 || q.mode == FFMOE_COMBINE_ACCUM_BF16);

  // live choices in combine order
  auto is_live = [&](int c) {
    const int e = p.ids[c];
    if (p.active && p.active[c] == 0u) return false;
    if ((unsigned)e >= (unsigned)p.experts || (p.valid && p.valid[e] == 0u)) return false;
    return !(p.generation && p.assignment_gen && p.generation[e] != p.assignment_gen[c]);
  };
  if (tid < K) {
    const int mine = p.ids[tid];
    const bool live = is_live(tid);
    if (!live && (!p.active || p.active[tid] != 0u) && q.status && blockIdx.x == 0) atomicOr(q.status, 1u);  // bad expert id
    int rank = 0;
    for (int c = 0; c < K; ++c) {
      const int other = p.ids[c];
      const bool before = ordered ? (other < mine || (other == mine && c < tid)) : c < tid;
      rank += (is_live(c) && before) ? 1 : 0;
    }
    if (live) s_choice[rank] = tid;
  }
  if (tid == 0) {
    int total = 0;
    for (int c = 0; c < K; ++c) total += is_live(c) ? 1 : 0;
    if (p.has_shared) s_choice[total] = -1;
    s_groups = total + (p.has_shared ? 1 : 0);
  }
  __syncthreads();
  const int ng = uni(s_groups);
  const int nr = ng - (p.has_shared ? 1 : 0);  // routed groups come first
  if (ng == 0) {  // nothing contributes: y = 0
    for (int d = blockIdx.x * 256 + tid; d < H; d += gridDim.x * 256) q.y[d] = 0;
    return;
  }

  // per-group constants: thread g gathers group g (ids -> slot table, two dependent loads, all groups in parallel) into
  // LDS; every wave then reads them back as wave-uniform scalars. Entries past the last group repeat it (their loads hit
  // the same lines, their sums are never used).
  __shared__ uint64_t s_codes[GMAX], s_scales[GMAX];
  __shared__ float s_glob[GMAX], s_wk[GMAX];
  __shared__ int s_slot[GMAX];
  if (tid < GMAX) {
    const int gg = tid < ng ? tid : ng - 1;
    const int c = s_choice[gg];
    if (c >= 0) {
      const int e = p.ids[c];
      s_codes[tid] = p.slots[size_t(e) * 6 + 4];
      s_scales[tid] = p.slots[size_t(e) * 6 + 5];
      s_glob[tid] = p.global_scales ? p.global_scales[size_t(e) * 3 + 2] : 1.0f;
      s_wk[tid] = p.weights_f32 ? reinterpret_cast<const float*>(p.weights)[c] : bf16_to_f32(reinterpret_cast<const uint16_t*>(p.weights)[c]);
      s_slot[tid] = c;
    } else {
      s_codes[tid] = p.shared_slot[4]; s_scales[tid] = p.shared_slot[5]; s_glob[tid] = p.shared_global[2];
      s_wk[tid] = 1.0f;
      s_slot[tid] = K;  // rows == 1: the shared expert's activations follow the K routed slots
    }
  }
  __syncthreads();
  uint64_t codes[GMAX], scales[GMAX];
  float glob[GMAX], wk[GMAX];
  int slot[GMAX];
#pragma unroll
  for (int g = 0; g < GMAX; ++g) {
    codes[g] = uni64(s_codes[g]); scales[g] = uni64(s_scales[g]);
    glob[g] = unif(s_glob[g]); wk[g] = unif(s_wk[g]);
    slot[g] = uni(s_slot[g]);
  }

  // this wave's contiguous run of output columns
  const int b_lo = int((long long)H * blockIdx.x / gridDim.x), b_hi = int((long long)H * (blockIdx.x + 1) / gridDim.x);
  const int count = b_hi - b_lo;
  const int w_lo = count * wave / 4, w_hi = count * (wave + 1) / 4;
  const int my_units = w_hi - w_lo;
  const int d0 = b_lo + w_lo;
  const int nchunks = I / F::EPL;

  typename F::Chunk buf[GMAX][1][S];
  auto issue = [&](int t, int g, int s) {
    const int chunk = s * 64 + lane;
    const int cc = chunk < nchunks ? chunk : nchunks - 1;
    F::load(buf[g][0][s], F::row(codes[g], scales[g], glob[g], d0 + t, I), cc);
  };
  if (my_units > 0) {
#pragma unroll
    for (int g = 0; g < GMAX; ++g)
#pragma unroll
      for (int s = 0; s < S; ++s) issue(0, g, s);
  }
  // activations of every group -> LDS, behind the first weight requests
  {
    const int row_words = I >> 3;
#pragma unroll
    for (int g = 0; g < GMAX; ++g) {
      if (g < ng) {
        u32x4* dst = reinterpret_cast<u32x4*>(xs + size_t(g) * I * 2);
        const uint16_t* src = p.h + size_t(slot[g]) * p.h_stride;
        for (int v = tid; v < row_words; v += 256) dst[v] = load16(src + size_t(v) * 8);
      }
    }
  }
  __syncthreads();
  if (my_units <= 0) return;

  const float sc = (q.mode == FFMOE_COMBINE_GATED) ? bf16_to_f32(q.scale[0]) : 0.0f;
  float park[GMAX];
#pragma unroll
  for (int g = 0; g < GMAX; ++g) park[g] = 0.0f;

  auto flush = [&](int ub, int nu) {
    if (lane < nu) {
      float sum = 0.0f, sh = 0.0f;
#pragma unroll
      for (int g = 0; g < GMAX; ++g) {
        if (g < nr) {
          const float v = __fmul_rn(p.routed_weight == FFMOE_WEIGHT_AFTER_DOWN_BF16 ? bround(park[g]) : park[g], wk[g]);
          const float c = bround(v);  // the BF16 contribution
          sum = q.mode == FFMOE_COMBINE_BF16 ? bround(__fadd_rn(sum, c)) : __fadd_rn(sum, c);
        } else if (g == nr && g < ng) {
          sh = bround(park[g]);       // the BF16 shared output
        }
      }
      float v;
      switch (q.mode) {
        case FFMOE_COMBINE_GATED: v = __fadd_rn(bround(sum), bround(__fmul_rn(sc, sh))); break;
        case FFMOE_COMBINE_UNGATED:
        case FFMOE_COMBINE_ACCUM_BF16: v = __fadd_rn(bround(sum), sh); break;
        case FFMOE_COMBINE_BF16:
        case FFMOE_COMBINE_ACCUM_FP32: v = __fadd_rn(sum, sh); break;
        default: v = sum; break;
      }
      q.y[d0 + ub + lane] = f32_to_bf16(v);
    }
  };

  for (int t = 0; t < my_units; ++t) {
    const int tn = t + 1 < my_units ? t + 1 : t;  // the last unit re-requests its own rows; nothing reads them
    const int slot_lane = t & 63;
    float part[GMAX];
#pragma unroll
    for (int g = 0; g < GMAX; ++g) {
      float acc[1][1] = {{0.0f}};
#pragma unroll
      for (int s = 0; s < S; ++s) {
        if (g < ng) step_compute<F, 1, 1, S>(buf[g], s, xs + size_t(g) * I * 2, I, nchunks, s * 64 + lane, 1, acc);
        issue(tn, g, s);
      }
      part[g] = acc[0][0];
    }
    // the reductions of the groups are independent chains: issued together they overlap each other's latency
#pragma unroll
    for (int g = 0; g < GMAX; ++g) {
      const float total = wave_sum(part[g]);
      park[g] = lane == slot_lane ? total : park[g];
    }
    if (slot_lane == 63) flush(t - 63, 64);
  }
  if (my_units & 63) flush(my_units & ~63, my_units & 63);
}

template <class F, int GMAX, int SMAX, int S = 1>
void launch_finish_steps(int want, const FinishParams& q, int blocks, size_t lds, hipStream_t st) {
  if constexpr (S <= SMAX) {
    if (want == S) hipLaunchKernelGGL((k_decode_finish<F, S, GMAX>), dim3(blocks), dim3(256), lds, st, q);
    else launch_finish_steps<F, GMAX, SMAX, S + 1>(want, q, blocks, lds, st);
  }
}

// Returns FFMOE_ERR_UNSUPPORTED when the shape is outside what the kernel holds in registers; the caller then runs the
// separate down and combine launches.
template <class F>
int launch_finish(const FinishParams& q, hipStream_t st) {
  const DecodeParams& p = q.d;
  const int groups = p.top_k + (p.has_shared ? 1 : 0);
  const int steps = (p.inter / F::EPL + 63) / 64;
  if (steps > 2 || groups > 9)
    return ff_fail(FFMOE_ERR_UNSUPPORTED, "one-token finish holds at most 9 groups and 2 steps per row (groups=%d, steps=%d)", groups, steps);
  const size_t lds = size_t(groups) * p.inter * 2;
  const int blocks = decode_num_cus() * 2;
  if (groups <= 4) launch_finish_steps<F, 4, 2>(steps, q, blocks, lds, st);
  else launch_finish_steps<F, 9, 2>(steps, q, blocks, lds, st);
  return ff_launch_status();
}

}  // namespace ffmoe
