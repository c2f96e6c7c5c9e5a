// One-token finish: down projection of every live choice and of the shared expert, routing weight and the ordered
// combine in a single launch (the last two launches of the decode layer, src/backend/cuda/moe/decode.rs:1187-1297:
// moe_down / moe_ffn_weight_f32 and moe_combine*, kernels/moe_ffn.cu:211-302,894-908, kernels/moe_combine.cu:51-116,
// 541-613).
//
// A block owns a run of output columns for ALL groups (live choices + shared expert), so the per-expert results of a
// column meet in the block's LDS and the combine needs no second pass over memory: contributions are neither written
// nor re-read and the combine launch disappears. Inside the block the work is the down stage's: a unit is NR
// consecutive rows of one group's down matrix, the units (group-major) are split evenly over the block's waves, each wave
// streams whole rows one unit ahead. The number of waves per block is chosen by the host so that the units divide
// evenly. Per row the dot product is the same chunk -> lane mapping, step order and wave reduction as k_decode_stage,
// and the groups are combined in the order the combine kernel adds them (ascending expert id, stable; choice order for
// the accumulate modes) with the rounding boundaries of k_decode_stage + k_combine, so y is bit-identical to the
// three-launch path.
#pragma once
#include "decode_kernel.cuh"
#include <cstdio>
#include <cstdlib>

namespace ffmoe {

#define FFMOE_FINISH_GROUPS 9  /* 8 routed choices + the shared expert */

// MAXT: the largest block the instantiation is launched with. Blocks of eight waves (the usual shape) are compiled for two
// waves per SIMD, i.e. with the whole register file of 256 registers per lane; 12 and 16 waves need the 128-register build.
// FSH / SSH: format and steps per row of the shared expert's down matrix when they differ from the routed experts' (a BF16
// shared expert next to NVFP4 experts): its units are every wave's first units, streamed and multiplied in their own
// format, so such a shared expert needs no down launch of its own.
template <class F, int S, int NR, int MAXT = 1024, class FSH = F, int SSH = S>
__global__ __launch_bounds__(MAXT) void k_decode_finish(const FinishParams q, const int cmax) {
  const DecodeParams& p = q.d;
  constexpr int GT = FFMOE_FINISH_GROUPS;
  extern __shared__ __align__(16) uint8_t xs[];  // [GT][inter] BF16 activations, then [GT][cmax] f32 row sums
  __shared__ int s_expert[FFMOE_MAX_TOP_K];      // expert of choice c, -1 = not live
  __shared__ int s_choice[FFMOE_MAX_TOP_K];      // live choices in combine order
  __shared__ int s_groups;
  __shared__ int s_next;  // the block's next unclaimed routed unit
  __shared__ uint64_t s_codes[GT], s_scales[GT];
  __shared__ float s_glob[GT], s_wk[GT];
  __shared__ int s_slot[GT];
  // NVFP4: the split dot's constants per scale code, one table per group's down matrix
  constexpr bool NV = std::is_same<F, FmtNvfp4>::value;
  __shared__ u32x2 s_lut[NV ? GT * FmtNvfp4::LUT_ENTRIES : 1];
  const int tid = threadIdx.x, lane = tid & 63, nthreads = blockDim.x;
  const int wave = uni(tid >> 6), nw = uni(int(blockDim.x >> 6));
  const int K = p.top_k, I = p.inter, H = p.hidden;
  float* s_part = reinterpret_cast<float*>(xs + size_t(GT) * I * 2);
  const bool ordered = !(q.mode == FFMOE_COMBINE_ACCUM_FP32 || q.mode == FFMOE_COMBINE_ACCUM_BF16);
  const bool has_shared = p.has_shared != 0;

  // this block's columns; a unit is NR consecutive rows of one group's down matrix inside them
  const int b_lo = int((long long)H * blockIdx.x / gridDim.x), b_hi = int((long long)H * (blockIdx.x + 1) / gridDim.x);
  const int C = b_hi - b_lo;
  const int P = (C + NR - 1) / NR;  // units per group
  const int nchunks = I / F::EPL;
  // One register buffer per wave: as soon as step s of a unit has been consumed, step s of the wave's next unit is requested
  // into the same registers. A second buffer, two units ahead, is slower for both formats measured (FP8 at hidden 7168:
  // 28.5 against 27.0 us, more requests in flight than the memory system takes; NVFP4: 24.1 against 22.1 us - its launch
  // takes 21.9 us with the dot work removed and 17.2 us with the requests removed, so it is the requests there too).
  constexpr int NB = 1;
  constexpr bool MIXED = !std::is_same<F, FSH>::value;
  typename F::Chunk buf[NB][NR][S];
  typename FSH::Chunk sbuf[MIXED ? NR : 1][MIXED ? SSH : 1];  // MIXED: the shared expert's unit in flight
  const int nchunks_sh = I / FSH::EPL;
  auto issue_shared_rows = [&](int i, int s) {  // MIXED: step s of the shared expert's unit i
    const int j = b_lo + i * NR;
    const int chunk = s * 64 + lane;
    const int cc = chunk < nchunks_sh ? chunk : nchunks_sh - 1;
#pragma unroll
    for (int m = 0; m < NR; ++m) {
      const int row = j + m < b_hi ? j + m : b_hi - 1;
      FSH::load(sbuf[MIXED ? m : 0][MIXED ? s : 0], FSH::row(uni64(p.shared_slot[4]), uni64(p.shared_slot[5]), unif(p.shared_global[2]), row, I), cc);
    }
  };
  // spare: a request behind the wave's last unit. It keeps the loop free of branches around its loads and nothing reads it;
  // every lane then asks for the row's first chunk (one line per load) instead of the unit's rows once more, which, streamed,
  // have left L2 by then and would come from HBM a second time (an eighth of the launch's bytes).
  auto issue_rows = [&](auto which, uint64_t codes, uint64_t scales, float glob, int i, int s, bool spare = false) {
    constexpr int b_ = decltype(which)::value;
    const int j = b_lo + i * NR;
    const int chunk = s * 64 + lane;
    const int cc = spare ? 0 : (chunk < nchunks ? chunk : nchunks - 1);
#pragma unroll
    for (int m = 0; m < NR; ++m) {
      const int row = j + m < b_hi ? j + m : b_hi - 1;  // a ragged last unit repeats the block's last row
      F::load(buf[b_][m][s], F::row(codes, scales, glob, row, I), cc);
    }
  };
  using B0 = std::integral_constant<int, 0>;
  // The shared expert's down matrix is a kernel argument, the routed ones are two dependent loads away (ids, then the slot
  // table): the shared expert's units w, w + nw, ... < P are wave w's first units, and it requests the first of them before
  // anything else, so the first weights are on their way while the block finds out which experts were chosen.
  const bool first_shared = has_shared && wave < P;
  if (first_shared) {
    if constexpr (MIXED) {
#pragma unroll
      for (int s = 0; s < SSH; ++s) issue_shared_rows(wave, s);
    } else {
#pragma unroll
      for (int s = 0; s < S; ++s) issue_rows(B0{}, uni64(p.shared_slot[4]), uni64(p.shared_slot[5]), unif(p.shared_global[2]), wave, s);
    }
  }
  // Activations: row c of the arena belongs to choice c, row K to the shared expert, whichever experts were chosen, so
  // all K + 1 rows are requested right here, in front of everything that depends on the ids, and go to LDS in arena
  // order (a group finds its row through s_slot). Rows of choices that turn out not to be live are never read.
  constexpr int HV = 8;  // 16-byte words per thread: (K + 1) * inter * 2 <= 64 KiB of LDS over >= 512 threads
  const int row_words = I >> 3;
  const int h_rows = K + (has_shared ? 1 : 0);
  const int h_words = h_rows * row_words;
  u32x4 hv[HV];
#pragma unroll
  for (int i = 0; i < HV; ++i) {
    const int v = tid + i * nthreads;
    const int vc = v < h_words ? v : 0;
    const int row = vc / row_words;
    hv[i] = load16(p.h + size_t(row) * p.h_stride + size_t(vc - row * row_words) * 8);
  }
  auto stage_activations = [&]() {
    u32x4* dst = reinterpret_cast<u32x4*>(xs);
#pragma unroll
    for (int i = 0; i < HV; ++i) {
      const int v = tid + i * nthreads;
      if (v < h_words) dst[v] = hv[i];
    }
    for (int v = tid + HV * nthreads; v < h_words; v += nthreads) {  // blocks below 512 threads with long rows
      const int row = v / row_words;
      dst[v] = load16(p.h + size_t(row) * p.h_stride + size_t(v - row * row_words) * 8);
    }
  };

  int nr_;
  if (q.desc) {
    // the gate/up launch of the same call has resolved the live choices: one record instead of ids -> slot table
    if (tid < FFMOE_FINISH_ROUTED) {
      s_codes[tid] = q.desc->codes[tid]; s_scales[tid] = q.desc->scales[tid];
      s_glob[tid] = q.desc->glob[tid]; s_wk[tid] = q.desc->wk[tid]; s_slot[tid] = q.desc->slot[tid];
    }
    if (tid == 0) {
      s_groups = q.desc->n;
      s_next = 0;
      if (q.desc->bad && q.status && blockIdx.x == 0) atomicOr(q.status, 1u);
    }
    __syncthreads();
    nr_ = uni(s_groups);
    if (tid == 0 && has_shared) {
      s_codes[nr_] = p.shared_slot[4]; s_scales[nr_] = p.shared_slot[5]; s_glob[nr_] = p.shared_global[2];
      s_wk[nr_] = 1.0f;
      s_slot[nr_] = K;
    }
  } else {
    // live choices in combine order
    if (tid < K) {
      const int e = p.ids[tid];
      bool live = !(p.active && p.active[tid] == 0u);
      const bool wanted = live;
      if (live) live = (unsigned)e < (unsigned)p.experts && !(p.valid && p.valid[e] == 0u);
      if (live && p.generation && p.assignment_gen && p.generation[e] != p.assignment_gen[tid]) live = false;
      if (wanted && !live && q.status && blockIdx.x == 0) atomicOr(q.status, 1u);  // bad or stale expert id
      s_expert[tid] = live ? e : -1;
    }
    __syncthreads();
    if (tid < K) {
      const int mine = s_expert[tid];
      int rank = 0;
      for (int c = 0; c < K; ++c) {
        const int other = s_expert[c];
        const bool before = ordered ? (other < mine || (other == mine && c < tid)) : c < tid;
        rank += (other >= 0 && before) ? 1 : 0;
      }
      if (mine >= 0) s_choice[rank] = tid;
    }
    if (tid == 0) {
      int total = 0;
      for (int c = 0; c < K; ++c) total += s_expert[c] >= 0 ? 1 : 0;
      s_groups = total;
      s_next = 0;
    }
    __syncthreads();
    nr_ = uni(s_groups);
    // per-group constants: thread g gathers group g (ids -> slot table, two dependent loads, all groups in parallel)
    if (tid < nr_ + (has_shared ? 1 : 0)) {
      if (tid < nr_) {
        const int c = s_choice[tid];
        const int e = s_expert[c];
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
  }
  const int nr = nr_;                           // routed groups, in combine order
  const int G = nr + (has_shared ? 1 : 0);      // group nr = the shared expert
  if (G == 0 && !q.shared_ready) {  // nothing contributes: y = 0
    for (int d = blockIdx.x * nthreads + tid; d < H; d += gridDim.x * nthreads) q.y[d] = 0;
    return;
  }
  __syncthreads();

  // This wave's units: the shared expert's units wave, wave + nw, ... < P first (the first of them is on its way since
  // entry), then routed units claimed one at a time from the block's counter (unit u = rows b_lo + NR * (u % P) .. of
  // group u / P). The two waves of a SIMD do not run at the same pace - the one placed first issues first and, with equal
  // shares, is done a fifth earlier - so equal shares leave every SIMD with one wave for the last microseconds. Which wave
  // computes a unit does not change its result.
  const int Ur = nr * P;
  auto claim = [&](int& g, int& i) -> bool {
    int u = 0;
    if (lane == 0) u = atomicAdd(&s_next, 1);
    u = uni(u);
    if (u >= Ur) return false;
    g = u / P;
    i = u - g * P;
    return true;
  };
  // the unit after (g, i): the wave's next shared unit, else a claim
  auto next_unit = [&](int& g, int& i) -> bool {
    if (!MIXED && g == nr && first_shared && i + nw < P) { i += nw; return true; }
    return claim(g, i);
  };
  auto issue_unit = [&](auto which, int g, int i, int s, bool spare) {
    issue_rows(which, uni64(s_codes[g]), uni64(s_scales[g]), unif(s_glob[g]), i, s, spare);
  };
  // (ug, ui): the unit whose rows are in flight in buf
  int ug = nr, ui = wave;
  bool uvalid = first_shared && !MIXED;
  if (!uvalid) {
    uvalid = claim(ug, ui);  // MIXED: the first routed unit goes out next to the shared ones, into its own registers
    if (uvalid) {
#pragma unroll
      for (int s = 0; s < S; ++s) issue_unit(B0{}, ug, ui, s, false);
    }
  }
  // NVFP4: the split dot's constants of every group's down matrix; then the activations, which were requested first
  if constexpr (NV) {
    for (int g = 0; g < (MIXED ? nr : G); ++g) FmtNvfp4::build_lut(s_lut + g * FmtNvfp4::LUT_ENTRIES, s_glob[g], tid, nthreads);
  }
  stage_activations();
  __syncthreads();
  if constexpr (MIXED) {
    // the shared expert's units of this wave in their own format; the first routed unit is already on its way
    const int lead = first_shared ? (P - wave + nw - 1) / nw : 0;
    for (int t = 0; t < lead; ++t) {
      const int i = wave + t * nw;
      float acc[NR][1];
#pragma unroll
      for (int m = 0; m < NR; ++m) acc[m][0] = 0.0f;
#pragma unroll
      for (int s = 0; s < SSH; ++s) {
        step_compute<FSH, NR, 1, SSH, false>(sbuf, s, xs + size_t(K) * I * 2, I, nchunks_sh, s * 64 + lane, 1, acc);
        if (t + 1 < lead) issue_shared_rows(i + nw, s);
      }
      float total[NR];
#pragma unroll
      for (int m = 0; m < NR; ++m) total[m] = wave_sum(acc[m][0]);
      if (lane == 0) {
#pragma unroll
        for (int m = 0; m < NR; ++m)
          if (i * NR + m < C) s_part[nr * cmax + i * NR + m] = total[m];
      }
    }
  }
  while (uvalid) {
    int ng = ug, ni = ui;
    const bool nvalid = next_unit(ng, ni);
    const int arow = uni(s_slot[ug]);  // the group's activation row in LDS (arena order)
    float acc[NR][1];
#pragma unroll
    for (int m = 0; m < NR; ++m) acc[m][0] = 0.0f;
#pragma unroll
    for (int s = 0; s < S; ++s) {
      step_compute<F, NR, 1, S, NV>(buf[0], s, xs + size_t(arow) * I * 2, I, nchunks, s * 64 + lane, 1, acc, s_lut + (NV ? ug * FmtNvfp4::LUT_ENTRIES : 0));
      // behind the last unit a request that nothing reads keeps the loop free of branches around its loads
      issue_unit(B0{}, nvalid ? ng : ug, nvalid ? ni : ui, s, !nvalid);
    }
    float total[NR];
#pragma unroll
    for (int m = 0; m < NR; ++m) total[m] = wave_sum(acc[m][0]);
    if (lane == 0) {
#pragma unroll
      for (int m = 0; m < NR; ++m)
        if (ui * NR + m < C) s_part[ug * cmax + ui * NR + m] = total[m];
    }
    ug = ng; ui = ni; uvalid = nvalid;
  }
  __syncthreads();
  // ordered combine of the block's columns
  const float sc = (q.mode == FFMOE_COMBINE_GATED) ? bf16_to_f32(q.scale[0]) : 0.0f;
  for (int col = tid; col < C; col += nthreads) {
    float sum = 0.0f;
    for (int g = 0; g < nr; ++g) {
      const float d = s_part[g * cmax + col];
      const float v = __fmul_rn(p.routed_weight == FFMOE_WEIGHT_AFTER_DOWN_BF16 ? bround(d) : d, s_wk[g]);
      const float c = bround(v);  // the BF16 contribution
      sum = q.mode == FFMOE_COMBINE_BF16 ? bround(__fadd_rn(sum, c)) : __fadd_rn(sum, c);
    }
    // the BF16 shared output: this launch's own down row, or the row other launches left in memory
    const float sh = q.shared_ready ? bf16_to_f32(q.shared_ready[b_lo + col]) : (has_shared ? bround(s_part[nr * cmax + col]) : 0.0f);
    float v;
    switch (q.mode) {
      case FFMOE_COMBINE_GATED: v = __fadd_rn(bround(sum), bround(__fmul_rn(sc, sh))); break;
      case FFMOE_COMBINE_UNGATED:
      case FFMOE_COMBINE_ACCUM_BF16: v = __fadd_rn(bround(sum), sh); break;
      case FFMOE_COMBINE_BF16:
      case FFMOE_COMBINE_ACCUM_FP32: v = __fadd_rn(sum, sh); break;
      default: v = sum; break;
    }
    q.y[b_lo + col] = f32_to_bf16(v);
  }
}

// NVFP4 routed experts next to a BF16 shared expert of the same width: steps per row are (S, SSH) = (inter / 2048, inter / 512)
template <int S, int SSH>
void launch_finish_mixed(const FinishParams& q, int blocks, int threads, int cmax, size_t lds, hipStream_t st) {
  hipLaunchKernelGGL((k_decode_finish<FmtNvfp4, S, 4, 512, FmtBf16, SSH>), dim3(blocks), dim3(threads), lds, st, q, cmax);
}

template <class F, int NR, int SMAX, int S = 1>
void launch_finish_steps(int want, const FinishParams& q, int blocks, int threads, int cmax, size_t lds, hipStream_t st) {
  if constexpr (S <= SMAX) {
    if (want == S) {
      if (threads <= 512) hipLaunchKernelGGL((k_decode_finish<F, S, NR, 512>), dim3(blocks), dim3(threads), lds, st, q, cmax);
      else hipLaunchKernelGGL((k_decode_finish<F, S, NR, 1024>), dim3(blocks), dim3(threads), lds, st, q, cmax);
    }
    else launch_finish_steps<F, NR, SMAX, S + 1>(want, q, blocks, threads, cmax, lds, st);
  }
}

// Grid and block size: one block per CU with 8, 12 or 16 waves (the same number on each of the CU's four SIMDs: the
// dequantization keeps the vector ALUs busy enough that a SIMD with one wave more than its neighbours finishes last;
// measured at hidden 7168: 8 waves 28.3 us, 9 waves 31.5 us), whichever divides the block's units most evenly (a wave with
// 6 units against waves with 5 holds the launch for a fifth longer); ties go to fewer waves.
inline void finish_shape(int columns, int groups, int nr_rows, int cus, int* blocks, int* waves) {
  *blocks = columns < cus ? columns : cus;
  const int per_block = (columns + *blocks - 1) / *blocks;
  const int units = groups * ((per_block + nr_rows - 1) / nr_rows);
  double best = 1e30;
  *waves = 8;
  for (int w = 8; w <= 16; w += 4) {
    const int busiest = (units + w - 1) / w;
    const double cost = double(busiest) * w / double(units);
    if (cost < best - 1e-9) { best = cost; *waves = w; }
  }
}

// Returns FFMOE_ERR_UNSUPPORTED when the shape is outside what the kernel holds in registers; the caller then runs the
// separate down and combine launches.
template <class F>
int launch_finish(const FinishParams& q, hipStream_t st, bool bf16_shared = false) {
  const DecodeParams& p = q.d;
  const int steps = (p.inter / F::EPL + 63) / 64;
  const int steps_sh = (p.inter / FmtBf16::EPL + 63) / 64;
  if (bf16_shared && !(std::is_same<F, FmtNvfp4>::value && steps == 1 && (steps_sh == 1 || steps_sh == 2 || steps_sh == 4) && p.shared_inter == p.inter))
    return ff_fail(FFMOE_ERR_UNSUPPORTED, "one-token finish with a BF16 shared expert: NVFP4 experts of the same width, at most 2048 columns (inter=%d)", p.inter);
  if (steps > 2 || p.top_k > FFMOE_FINISH_GROUPS - 1)
    return ff_fail(FFMOE_ERR_UNSUPPORTED, "one-token finish holds at most %d routed groups and 2 steps per row (top_k=%d, steps=%d)",
                   FFMOE_FINISH_GROUPS - 1, p.top_k, steps);
  constexpr int NR = 4;
  int blocks, waves;
  finish_shape(p.hidden, p.top_k + (p.has_shared ? 1 : 0), NR, decode_num_cus(), &blocks, &waves);
  if (const char* e = getenv("FFMOE_FINISH_SHAPE")) {  // "blocks,waves": measurement override
    int b = 0, w = 0;
    if (sscanf(e, "%d,%d", &b, &w) == 2 && b >= 1 && w >= 1 && w <= 16) { blocks = b; waves = w; }
  }
  // NVFP4 rows of two steps hold their split-dot operands in more registers than the 128 of a 12- or 16-wave block
  if (std::is_same<F, FmtNvfp4>::value && steps == 2 && waves > 8) waves = 8;
  const int cmax = (p.hidden + blocks - 1) / blocks;
  const size_t lds = size_t(FFMOE_FINISH_GROUPS) * p.inter * 2 + size_t(FFMOE_FINISH_GROUPS) * cmax * 4;
  const size_t tables = std::is_same<F, FmtNvfp4>::value ? size_t(FFMOE_FINISH_GROUPS) * FmtNvfp4::LUT_ENTRIES * 8 : 0;  // static, next to lds
  if (lds + tables + 512 > 64 * 1024) return ff_fail(FFMOE_ERR_UNSUPPORTED, "one-token finish: %zu bytes of LDS per block", lds + tables);
  if (bf16_shared) {
    if constexpr (std::is_same<F, FmtNvfp4>::value) {
      waves = 8;  // the instantiation is built for eight-wave blocks
      if (steps_sh == 4) launch_finish_mixed<1, 4>(q, blocks, waves * 64, cmax, lds, st);
      else if (steps_sh == 2) launch_finish_mixed<1, 2>(q, blocks, waves * 64, cmax, lds, st);
      else launch_finish_mixed<1, 1>(q, blocks, waves * 64, cmax, lds, st);
    }
    return ff_launch_status();
  }
  launch_finish_steps<F, NR, 2>(steps, q, blocks, waves * 64, cmax, lds, st);
  return ff_launch_status();
}

}  // namespace ffmoe
