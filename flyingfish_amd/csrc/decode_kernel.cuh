// Decode expert FFN kernel (both stages) and its launch policy, instantiated once per weight format in
// decode_fp8.hip / decode_nvfp4.hip / decode_bf16.hip.
//
// Work model. Assignments (row, choice) that hit the same expert are gathered into groups of at most RG rows, so
// one pass over an expert's weights serves all of them. A "unit" is NR consecutive output rows of one group. The
// unit space is split evenly over a fixed grid; every block walks a contiguous unit range, so each wave streams
// whole weight rows with 16-byte loads per lane (a wave covers 1 KiB of a row per load instruction), dequantizes
// in registers and keeps one FP32 accumulator per (row-of-group, weight row), reduced across the wave at the end
// of the unit. Activations of the group live in LDS.
//
// Arithmetic (FFMOE_ACT_BF16): effective weight = bf16(decode(code) * scale) as in the reference's CPU path
// (src/fp8.rs:138-145), FP32 accumulation, BF16 boundaries at gate, up, SiLU, product, down and weighted
// contribution (src/cpu/expert_ffn.rs:592-679; kernels/moe_ffn.cu:198-209,293-301).
#pragma once
#include "gemv.cuh"
#include "route_select.cuh"
#include "api.h"
#include "decode.h"

namespace ffmoe {

// ---------------------------------------------------------------------------------------------

// Group g as wave-uniform scalars. Without a descriptor table (one row per call) every assignment is its own
// group and the shared expert follows the routed ones.
template <int RG>
__device__ __forceinline__ void load_group(const DecodeParams& p, int g, int& expert, int& n, int (&row)[RG], int (&slot)[RG],
                                           const int* inline_ids = nullptr) {
  if (p.groups) {
    const int* gd = reinterpret_cast<const int*>(p.groups + g);
    expert = load_uniform<int>(gd);
    n = load_uniform<int>(gd + 1);
#pragma unroll
    for (int r = 0; r < RG; ++r) {
      row[r] = load_uniform<int>(gd + 2 + r);
      slot[r] = load_uniform<int>(gd + 2 + FFMOE_DECODE_RG + r);
    }
    return;
  }
  const int A = p.rows * p.top_k;
#pragma unroll
  for (int r = 0; r < RG; ++r) { row[r] = 0; slot[r] = 0; }
  n = 1;
  if (g < A) {
    expert = inline_ids ? uni(inline_ids[g]) : load_uniform<int>(p.ids + g);
    row[0] = g / p.top_k;
    slot[0] = g;
    if (p.active && int(load_uniform<uint32_t>(p.active + g)) == 0) n = 0;
    if ((unsigned)expert >= (unsigned)p.experts) n = 0;  // out-of-range id: contribute nothing, done stays 0
    else if (p.valid && int(load_uniform<uint32_t>(p.valid + expert)) == 0) n = 0;
    else if (p.generation && p.assignment_gen &&
             load_uniform<uint64_t>(p.generation + expert) != load_uniform<uint64_t>(p.assignment_gen + g)) n = 0;  // stale choice
  } else {
    expert = -1;
    row[0] = g - A;
    slot[0] = g;
  }
}

// STAGE 0: gate/up + SwiGLU -> h[slot, j].   STAGE 1: down (+ routing weight) -> contributions / shared_out.
// A unit is NR consecutive output rows of one group: stage 0 streams NR gate rows and the NR matching up rows
// (2*NR weight rows sharing every activation read), stage 1 streams NR down rows.
//
// Every quantity that decides an address (group, expert, row index, slab) is wave-uniform and lives in scalar
// registers, so a weight load is a scalar base plus one per-lane offset. A wave owns a contiguous run of units
// of the segment and keeps ONE register buffer of S steps per weight row: as soon as step s of the current item
// has been consumed, step s of the next item is requested into the same registers, so a full row per weight
// matrix is in flight at all times and the first requests of a segment go out before the activations are even
// staged. Reduced sums of up to 64 units are parked one per lane; the epilogue (SwiGLU or weighting, BF16
// rounding, store) runs once per 64 units with coalesced stores.
// FSH / SSH: format and steps of the shared expert's rows when they differ from the routed experts' (one token with the
// selection in the prologue: every block takes its slice of the shared expert first, in that expert's own format, so a
// BF16 shared expert next to NVFP4 experts needs no gate/up launch of its own). Everything else runs as F / S.
template <class FF_, int SS_>
struct SegmentKind { using fmt = FF_; static constexpr int steps = SS_; };

template <class F, int S, int STAGE, int RG, int NR, class FSH = F, int SSH = S>
__global__ __launch_bounds__(256) void k_decode_stage(const DecodeParams p) {
  constexpr int NROWS = STAGE == 0 ? 2 * NR : NR;
  extern __shared__ __align__(16) uint8_t xs[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = uni(tid >> 6);
  const int A = p.rows * p.top_k;
  // one token, selection in the prologue: wave 0 selects into LDS, block 0 publishes ids, weights and clean done flags
  __shared__ int s_route_ids[FFMOE_MAX_TOP_K];
  __shared__ float s_route_w[FFMOE_MAX_TOP_K];
  // NVFP4: the split dot's constants per scale code, one table per matrix of the segment (gate, up | down)
  constexpr bool NV = std::is_same<F, FmtNvfp4>::value || std::is_same<FSH, FmtNvfp4>::value;
  __shared__ u32x2 s_lut[NV ? 2 * FmtNvfp4::LUT_ENTRIES : 1];
  // One token with the selection in this launch (256 experts, a shared expert): no block barrier behind the slice's first
  // one. Wave 0 selects as soon as its logits are there and hands the choices over through a flag in LDS; the other waves
  // stage the token row, compute their slice units and pick the flag up when they are done - a wave starts on its routed
  // rows as soon as its own slice units are finished. FP8 / BF16 rows: the token row is staged by the three slice waves
  // alone, counted in s_staged (with wave 0 in that barrier either it waits four microseconds for rows it does not need
  // before it may select, or the slice waves wait for the selection). NVFP4 rows: every wave keeps split-dot tables of
  // its own for its routed segments, built with its own lanes, so those segments need no barrier either.
  constexpr bool FREE = STAGE == 0 && RG == 1;
  __shared__ int s_staged;  // slice waves whose share of the token row is in LDS
  __shared__ u32x2 s_lut_wave[FREE && NV ? 4 * 2 * FmtNvfp4::LUT_ENTRIES : 1];
  __shared__ int s_selected;
  const bool inline_route = STAGE == 0 && RG == 1 && p.route.logits != nullptr;
  // With a shared expert the selection hides behind it: its units need no routing, so every block first takes its slice
  // of the shared expert's rows on waves 1..3 while wave 0 selects, and the routed units follow once the ids are known.
  const bool shared_first = inline_route && p.has_shared;
  const int n_routed = p.counters ? uni(load_global<int>(p.counters)) : A;
  const int n_shared = p.counters ? uni(load_global<int>(p.counters + 1)) : (p.has_shared ? p.rows : 0);
  // units per group
  const int out_r = (STAGE == 0 ? p.inter : p.hidden) / NR;
  const int out_s = (STAGE == 0 ? p.shared_inter : p.hidden) / NR;
  const long long routed_units = (long long)n_routed * out_r;

  // 256 experts: wave 0 asks for its four logits and biases per lane before anything else of this CU is in the memory
  // pipeline; asked for behind the shared slice they wait for the waves' first weight rows, which the vector memory
  // pipeline of the CU serves first (2 - 4 us in front of the selection)
  constexpr int PC = 4;
  float pre_l[PC] = {0.0f, 0.0f, 0.0f, 0.0f}, pre_b[PC] = {0.0f, 0.0f, 0.0f, 0.0f};
  const bool preloaded = STAGE == 0 && RG == 1 && inline_route && shared_first && p.experts == 64 * PC;
  if (preloaded && wave == 0) {
    if (((reinterpret_cast<uintptr_t>(p.route.logits) | reinterpret_cast<uintptr_t>(p.route.bias)) & 15) == 0) {
      // one 16-byte request per lane and array
      const u32x4 vl = load16(p.route.logits + lane * PC);
      u32x4 vb = {0u, 0u, 0u, 0u};
      if (p.route.bias) vb = load16(p.route.bias + lane * PC);
#pragma unroll
      for (int j = 0; j < PC; ++j) {
        const uint32_t lj = vl[j], bj = vb[j];  // a bit cast of the vector element itself reads element 0
        pre_l[j] = __uint_as_float(lj);
        pre_b[j] = __uint_as_float(bj);
      }
    } else {
#pragma unroll
      for (int j = 0; j < PC; ++j) {
        pre_l[j] = load_global<float>(p.route.logits + lane * PC + j);
        if (p.route.bias) pre_b[j] = load_global<float>(p.route.bias + lane * PC + j);
      }
    }
  }
  const int select_k = p.route.select_k > 0 ? p.route.select_k : p.top_k;
  NoauxState<PC> sel;
  // The usual router (256 experts in 8 groups of which 4 stay, sigmoid scores, 8 picks) runs a copy of the selection with
  // these numbers as literals: two thirds of the instructions of the general one (no integer divisions, loops unrolled).
  const bool usual_router = p.experts == 256 && p.route.n_group == 8 && p.route.topk_group == 4 && select_k == 8 &&
                            p.route.score_mode == FFMOE_NOAUX_SIGMOID;
  auto select_preloaded = [&]() {
    if (usual_router) {
      wave_route_prepare_preloaded<PC>(sel, pre_l, pre_b, lane, 256, 8, FFMOE_NOAUX_SIGMOID, 8, 4);
      wave_select_pick<PC>(sel, lane, 8, p.route.routed_scaling, s_route_ids, s_route_w, 1);
    } else {
      wave_route_prepare_preloaded<PC>(sel, pre_l, pre_b, lane, p.experts, select_k, p.route.score_mode, p.route.n_group, p.route.topk_group);
      wave_select_pick<PC>(sel, lane, select_k, p.route.routed_scaling, s_route_ids, s_route_w, 1);
    }
  };
  bool slice3_used = false;  // the slice's token row was staged by the three slice waves alone, counted in s_staged
  const bool free_run = FREE && preloaded && p.rows == 1;  // block-uniform
  if (free_run && tid == 0) { s_selected = 0; s_staged = 0; }  // in front of the slice's first barrier; read behind it
  int slice_first_units = 0;  // > 0 while the block's first routed segment is dealt out: the units of its shared slice

  // One segment: `count` units of group g from unit j0 on, split over the waves wv = 0 .. nw-1 (wv < 0: this wave only
  // takes part in the staging and the barriers).
  // staged: the group's activation row is in LDS already (one token: the routed segments behind the shared slice read the
  // same token row) - no second copy behind the segment's first weight requests, and without a table to build no barrier
  auto segment = [&](auto kind, int g, int j0, int count, int nw, int wv, const int* inline_ids, bool staged = false, bool slice_free = false) {
    using FF = typename decltype(kind)::fmt;
    constexpr int SS = decltype(kind)::steps;
    constexpr bool NVF = std::is_same<FF, FmtNvfp4>::value;
    int expert, gn, grow[RG], gslot[RG];
    // One row per call: the slot entries of the choice are requested next to the checks of its id (valid flag, epoch), not
    // behind them - one round trip to L2 in front of the first weight request instead of two.
    uint64_t slv[6] = {0, 0, 0, 0, 0, 0};
    float glv[3] = {1.0f, 1.0f, 1.0f};
    bool early = false;
    if (!p.groups && g < A) {
      const int e = inline_ids ? uni(inline_ids[g]) : load_uniform<int>(p.ids + g);
      if ((unsigned)e < (unsigned)p.experts) {
        early = true;
#pragma unroll
        for (int i = 0; i < 6; ++i) slv[i] = load_uniform<uint64_t>(p.slots + size_t(e) * 6 + i);
        if (p.global_scales) {
#pragma unroll
          for (int i = 0; i < 3; ++i) glv[i] = load_uniform<float>(p.global_scales + size_t(e) * 3 + i);
        }
      }
    }
    load_group<RG>(p, g, expert, gn, grow, gslot, inline_ids);
    const bool shared = expert < 0;
    const int Kg = STAGE == 0 ? p.hidden : (shared ? p.shared_inter : p.inter);
    // the six slot addresses through scalar-friendly paths (kernel argument or global table), never a generic pointer
    uint64_t sl[6] = {0, 0, 0, 0, 0, 0};
    float gl3[3] = {1.0f, 1.0f, 1.0f};
    if (gn > 0) {
      if (shared) {
#pragma unroll
        for (int i = 0; i < 6; ++i) sl[i] = p.shared_slot[i];
#pragma unroll
        for (int i = 0; i < 3; ++i) gl3[i] = p.shared_global[i];
      } else if (early) {
#pragma unroll
        for (int i = 0; i < 6; ++i) sl[i] = uni64(slv[i]);
#pragma unroll
        for (int i = 0; i < 3; ++i) gl3[i] = unif(glv[i]);
      } else {
#pragma unroll
        for (int i = 0; i < 6; ++i) sl[i] = load_uniform<uint64_t>(p.slots + size_t(expert) * 6 + i);
        if (p.global_scales) {
#pragma unroll
          for (int i = 0; i < 3; ++i) gl3[i] = load_uniform<float>(p.global_scales + size_t(expert) * 3 + i);
        }
      }
    }
    // weight row m of a unit comes from matrix m / NR (stage 0: gate, up; stage 1: down)
    uint64_t codes[2], scales[2];
    float global[2];
    if (STAGE == 0) {
      codes[0] = sl[0]; scales[0] = sl[1]; global[0] = gl3[0];
      codes[1] = sl[2]; scales[1] = sl[3]; global[1] = gl3[1];
    } else {
      codes[0] = codes[1] = sl[4]; scales[0] = scales[1] = sl[5]; global[0] = global[1] = gl3[2];
    }
    // routing weights of the group's rows (stage 1), fetched up front so the epilogue never waits on them
    float wk[RG];
#pragma unroll
    for (int r = 0; r < RG; ++r) {
      wk[r] = 1.0f;
      if (STAGE == 1 && !shared && r < gn) {
        wk[r] = p.weights_f32 ? unif(load_global<float>(reinterpret_cast<const float*>(p.weights) + gslot[r]))
                              : bf16_to_f32(uint16_t(uni(int(load_global<uint16_t>(reinterpret_cast<const uint16_t*>(p.weights) + gslot[r])))));
      }
    }
    const int nchunks = Kg / FF::EPL;
    const int nslabs = (nchunks + SS * 64 - 1) / (SS * 64);
    // this wave's contiguous run of units inside the segment
    int w_lo = wv >= 0 ? count * wv / nw : 0, w_hi = wv >= 0 ? count * (wv + 1) / nw : 0;
    if (slice_first_units > 0 && wv >= 0 && nw == 4) {
      // the block's first routed segment behind its slice of the shared expert: shares that even out slice units plus
      // routed units per wave (wave 0 took no slice unit and has been streaming routed rows since the selection, the
      // wave with two slice units starts last) - 9 / 8 / 8 / 7 units for a slice of 4 and 32 routed units
      const int all = count + slice_first_units;
      auto cut = [&](int w) {  // routed units of the waves below w
        const int slice_below = w == 0 ? 0 : slice_first_units * (w - 1) / 3;
        const int c = all * w / 4 - slice_below;
        return c < 0 ? 0 : (c > count ? count : c);
      };
      w_lo = cut(wv); w_hi = wv == 3 ? count : cut(wv + 1);
      if (w_hi < w_lo) w_hi = w_lo;
    }
    const int my_units = gn > 0 ? w_hi - w_lo : 0;
    const int items = my_units * nslabs;
    const int jw = j0 + w_lo;  // first unit of the run
    typename FF::Chunk buf[NROWS][SS];
    auto issue_step = [&](int t, int s) {
      const int j = (jw + t / nslabs) * NR;  // first output row of the unit
      const int chunk = (t % nslabs) * (SS * 64) + s * 64 + lane;
      const int cc = chunk < nchunks ? chunk : nchunks - 1;
#pragma unroll
      for (int m = 0; m < NROWS; ++m) {
        const int mat = m / NR;
        FF::load(buf[m][s], FF::row(codes[mat], scales[mat], global[mat], j + (m % NR), Kg), cc);
      }
    };
    if (items > 0) {
#pragma unroll
      for (int s = 0; s < SS; ++s) issue_step(0, s);
    }
    // activations of the group -> LDS (row r at r*Kg*2), behind the first weight requests
    const bool own_tables = FREE && NVF && staged && free_run;  // block-uniform
    const bool skip_staging = staged && (!NVF || own_tables);  // wave-uniform, block-uniform
    const bool slice3 = FREE && !NV && slice_free && gn == 1;  // block-uniform
    if (slice3) slice3_used = true;  // block-uniform
    const u32x2* lut = s_lut;
    if constexpr (FREE && NVF) {
      if (own_tables && gn > 0) {
        u32x2* mine = s_lut_wave + wave * 2 * FmtNvfp4::LUT_ENTRIES;
        FmtNvfp4::build_lut(mine, global[0], lane, 64);
        FmtNvfp4::build_lut(mine + FmtNvfp4::LUT_ENTRIES, global[1], lane, 64);
        lut = mine;
      }
    }
    if (!skip_staging) __syncthreads();  // the previous segment's readers are done with xs
    if (gn > 0 && !skip_staging) {
      const uint16_t* src = STAGE == 0 ? p.x : p.h;
      const int row_words = Kg >> 3;  // 16-byte words per row
#pragma unroll
      for (int r = 0; r < RG; ++r) {
        if (r < gn && !staged) {
          const size_t base = STAGE == 0 ? size_t(grow[r]) * p.hidden : size_t(gslot[r]) * p.h_stride;
          u32x4* d4 = reinterpret_cast<u32x4*>(xs + size_t(r) * Kg * 2);
          if (slice3) {
            // the three slice waves stage the row; the selecting wave takes no part and does not wait for it here
            if (wave != 0) {
              for (int v = tid - 64; v < row_words; v += 192) d4[v] = load16(src + base + size_t(v) * 8);
              if (lane == 0) atomicAdd(&s_staged, 1);  // behind the wave's writes: its LDS operations land in program order
            }
          } else {
            for (int v = tid; v < row_words; v += 256) d4[v] = load16(src + base + size_t(v) * 8);
          }
        }
      }
      if constexpr (NVF) {
        FmtNvfp4::build_lut(s_lut, global[0], tid, 256);
        if (STAGE == 0) FmtNvfp4::build_lut(s_lut + FmtNvfp4::LUT_ENTRIES, global[1], tid, 256);
      }
    }
    if (slice3) {
      // bounded by the other slice waves, which are on their way to the same point
      if (wave != 0) while (uni(*reinterpret_cast<volatile int*>(&s_staged)) < 3) __builtin_amdgcn_s_sleep(1);
    } else if (!skip_staging) {
      __syncthreads();
    }
    if (items > 0) {
      float acc[NROWS][RG];
      float park[NROWS][RG];  // lane L keeps the sums of unit (batch base + L)
#pragma unroll
      for (int m = 0; m < NROWS; ++m)
#pragma unroll
        for (int r = 0; r < RG; ++r) { acc[m][r] = 0.0f; park[m][r] = 0.0f; }
      // epilogue for the units [ub, ub + nu) of the run, one unit per lane
      auto flush = [&](int ub, int nu) {
        if (lane < nu) {
          const int j = (jw + ub + lane) * NR;
#pragma unroll
          for (int r = 0; r < RG; ++r) {
            if (RG == 1 || r < gn) {
              if (STAGE == 0) {
                uint16_t* dst = p.h + size_t(gslot[r]) * p.h_stride + j;
#pragma unroll
                for (int m = 0; m < NR; ++m)
                  dst[m] = swiglu_bf16(bround(park[m][r]), bround(park[NR + m][r]), p.swiglu, p.swiglu_limit);
              } else {
                float v[NR];
#pragma unroll
                for (int m = 0; m < NR; ++m) {
                  if (shared) v[m] = park[m][r];
                  else v[m] = __fmul_rn(p.routed_weight == FFMOE_WEIGHT_AFTER_DOWN_BF16 ? bround(park[m][r]) : park[m][r], wk[r]);
                }
                uint16_t* dst = shared ? p.shared_out + size_t(grow[r]) * p.hidden + j : p.contributions + size_t(gslot[r]) * p.hidden + j;
                if (NR == 4) {
                  u32x2 o = {pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2 % NR], v[3 % NR])};
                  *reinterpret_cast<u32x2*>(dst) = o;
                } else {
#pragma unroll
                  for (int m = 0; m < NR; ++m) dst[m] = f32_to_bf16(v[m]);
                }
                if (!shared && j == 0 && p.done) p.done[gslot[r]] = 1u;
              }
            }
          }
        }
      };
      auto compute_step = [&](int t, int s) {
        const int chunk = (t % nslabs) * (SS * 64) + s * 64 + lane;
        step_compute<FF, NROWS, RG, SS, NVF>(buf, s, xs, Kg, nchunks, chunk, gn, acc, lut, lut + (NVF ? FmtNvfp4::LUT_ENTRIES : 0), NR);
      };
      auto item_end = [&](int t) {
        const int unit = t / nslabs;
        if (t % nslabs != nslabs - 1) return;
        const int slot_lane = unit & 63;
#pragma unroll
        for (int m = 0; m < NROWS; ++m)
#pragma unroll
          for (int r = 0; r < RG; ++r) {
            if (RG == 1 || r < gn) {
              const float total = wave_sum(acc[m][r]);
              park[m][r] = lane == slot_lane ? total : park[m][r];
            }
            acc[m][r] = 0.0f;
          }
        if (slot_lane == 63) flush(unit - 63, 64);
      };
      for (int t = 0; t + 1 < items; ++t) {
#pragma unroll
        for (int s = 0; s < SS; ++s) {
          compute_step(t, s);
          issue_step(t + 1, s);
        }
        item_end(t);
      }
#pragma unroll
      for (int s = 0; s < SS; ++s) compute_step(items - 1, s);
      item_end(items - 1);
      if (my_units & 63) flush(my_units & ~63, my_units & 63);
    }
  };

  if (STAGE == 0 && RG == 1) {
    if (shared_first) {
      // this block's slice of the shared expert (group A: rows == 1), waves 1..3; wave 0 selects meanwhile
      const int s_lo = int((long long)out_s * blockIdx.x / gridDim.x), s_hi = int((long long)out_s * (blockIdx.x + 1) / gridDim.x);
      segment(SegmentKind<FSH, SSH>{}, A, s_lo, s_hi - s_lo, 3, wave - 1, nullptr, false, free_run);
      if (free_run) slice_first_units = s_hi - s_lo;
    }
    if (inline_route) {
      if (wave == 0 && preloaded) {
        select_preloaded();
        if (free_run && lane == 0) s_selected = 1;  // behind the ids and weights: a wave's LDS writes land in program order
      } else if (wave == 0)
        wave_route_dispatch(p.route.logits, p.route.bias, lane, p.experts, select_k, p.route.score_mode, p.route.routed_scaling,
                            p.route.n_group, p.route.topk_group, s_route_ids, s_route_w, 1);
      if (free_run) {
        // bounded by wave 0, which selects right behind the slice's staging barrier
        while (uni(*reinterpret_cast<volatile int*>(&s_selected)) == 0) __builtin_amdgcn_s_sleep(1);
        // the selecting wave took no part in the staging of the slice: the row has to be there before its routed units
        if (slice3_used && wave == 0) while (uni(*reinterpret_cast<volatile int*>(&s_staged)) < 3) __builtin_amdgcn_s_sleep(1);
      } else {
        __syncthreads();
      }
      if (blockIdx.x == 0 && tid < select_k) {
        const_cast<int*>(p.ids)[tid] = s_route_ids[tid];
        reinterpret_cast<float*>(const_cast<void*>(p.weights))[tid] = s_route_w[tid];
        if (p.done) p.done[tid] = 0u;
      }
      // the finish launch of the same call: live choices in combine order with their down matrices resolved
      if (blockIdx.x == 0 && p.route.finish_desc && tid < 64) {
        FinishDesc* fd = p.route.finish_desc;
        const int mine = tid < select_k ? s_route_ids[tid] : -1;
        const bool in_range = tid < select_k && (unsigned)mine < (unsigned)p.experts;
        const bool live = in_range && !(p.valid && p.valid[mine] == 0u);
        const unsigned long long lives = __ballot(live);
        int rank = 0;
        for (int c = 0; c < select_k; ++c) {
          const int other = s_route_ids[c];
          const bool before = p.route.finish_ordered ? (other < mine || (other == mine && c < tid)) : c < tid;
          rank += (((lives >> c) & 1ull) && before) ? 1 : 0;
        }
        if (live && rank < FFMOE_FINISH_ROUTED) {
          fd->codes[rank] = p.slots[size_t(mine) * 6 + 4];
          fd->scales[rank] = p.slots[size_t(mine) * 6 + 5];
          fd->glob[rank] = p.global_scales ? p.global_scales[size_t(mine) * 3 + 2] : 1.0f;
          fd->wk[rank] = s_route_w[tid];
          fd->slot[rank] = tid;
        }
        if (tid == 0) {
          fd->n = __builtin_popcountll(lives);
          fd->bad = __builtin_popcountll(lives) != select_k ? 1 : 0;
        }
      }
    }
  }
  const long long total = shared_first ? routed_units : routed_units + (long long)n_shared * out_s;
  const long long lo = total * blockIdx.x / gridDim.x, hi = total * (blockIdx.x + 1) / gridDim.x;
  long long u0 = lo;
  while (u0 < hi) {
    // group segment containing u0
    int g, j0, width;
    if (u0 < routed_units) { g = int(u0 / out_r); j0 = int(u0 % out_r); width = out_r; }
    else { const long long v = u0 - routed_units; g = n_routed + int(v / out_s); j0 = int(v % out_s); width = out_s; }
    const long long seg_end = u0 + (width - j0) < hi ? u0 + (width - j0) : hi;
    segment(SegmentKind<F, S>{}, g, j0, int(seg_end - u0), 4, wave, inline_route ? s_route_ids : nullptr,
            STAGE == 0 && RG == 1 && shared_first && p.rows == 1 && g < A);
    u0 = seg_end;
    slice_first_units = 0;
  }
}

// ---------------------------------------------------------------------------------------------
// Launch policy. A weight row needs steps = ceil(K / (64 * EPL)) 16-byte loads per lane. S of them are kept in
// flight per weight row (one slab); rows longer than the format's cap take several slabs. The caps keep every
// instantiation inside the register file without spills: stage 0 holds 2 weight rows per unit, stage 1 holds
// Policy::NR1 rows; with several rows of a group per pass (RG > 1) the cap is halved.
template <class F> struct Policy { static constexpr int S0 = 8, S0G = 8, NR0 = 1, NR1 = 4, NR1G = 4, S1 = 2, S1G = 2; };
// NVFP4: two gate and two up rows per unit (NR0 = 2, as many bytes in flight per wave as FP8) measured slower
// (96 against 91 us per C4 layer): its gate/up stage is bound by the conversion work, not by requests in flight
template <> struct Policy<FmtNvfp4> { static constexpr int S0 = 4, S0G = 4, NR0 = 1, NR1 = 4, NR1G = 2, S1 = 2, S1G = 2; };

inline int decode_num_cus() {
  static int cus = 0;
  if (cus == 0) {
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) == hipSuccess && hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && n > 0)
      cus = n;
    else
      cus = 256;
  }
  return cus;
}

template <class F, int STAGE, int RG, int NR, int SMAX, int S = 1>
void launch_steps(int want, const DecodeParams& p, int blocks, size_t lds, hipStream_t st) {
  if constexpr (S <= SMAX) {
    if (want == S) hipLaunchKernelGGL((k_decode_stage<F, S, STAGE, RG, NR>), dim3(blocks), dim3(256), lds, st, p);
    else launch_steps<F, STAGE, RG, NR, SMAX, S + 1>(want, p, blocks, lds, st);
  }
}

template <class F, int STAGE>
int launch_stage(const DecodeParams& p, int rg, hipStream_t st) {
  const int kr = STAGE == 0 ? p.hidden : p.inter;
  const int ks = STAGE == 0 ? p.hidden : (p.has_shared ? p.shared_inter : p.inter);
  const int kmax = kr > ks ? kr : ks;
  const size_t lds = size_t(rg) * kmax * 2;
  // blocks per CU: two for the long rows of the gate/up stage, three for the shorter down rows
  const int blocks = decode_num_cus() * (STAGE == 0 ? 2 : 3);
  constexpr int NR = STAGE == 0 ? Policy<F>::NR0 : Policy<F>::NR1;
  constexpr int NRG = STAGE == 0 ? 1 : Policy<F>::NR1G;
  constexpr int SMAX1 = STAGE == 0 ? Policy<F>::S0 : Policy<F>::S1;
  constexpr int SMAXG = STAGE == 0 ? Policy<F>::S0G : Policy<F>::S1G;
  const int steps = (kmax / F::EPL + 63) / 64;
  const int smax = rg == 1 ? SMAX1 : SMAXG;
  const int nslabs = (steps + smax - 1) / smax;
  const int S = (steps + nslabs - 1) / nslabs;
  if (rg == 1) launch_steps<F, STAGE, 1, NR, SMAX1>(S, p, blocks, lds, st);
  else launch_steps<F, STAGE, FFMOE_DECODE_RG, NRG, SMAXG>(S, p, blocks, lds, st);
  return ff_launch_status();
}

template <class F>
int launch_format(const DecodeParams& p, int rg, int stage_mask, hipStream_t st) {
  if (stage_mask & 1) FF_TRY((launch_stage<F, 0>(p, rg, st)));
  if (stage_mask & 2) FF_TRY((launch_stage<F, 1>(p, rg, st)));
  return 0;
}

}  // namespace ffmoe
