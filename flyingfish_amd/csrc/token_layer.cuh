// One token, the expert part of the layer in ONE launch: top-k selection, gate/up + SwiGLU, down, routing weight and the
// ordered combine (src/backend/cuda/moe/decode.rs:1187-1297 of the reference runs moe_route_select_noaux, moe_gate_up,
// moe_down / moe_ffn_weight_f32 and moe_combine* as separate launches; kernels/moe_route.cu:315-390,
// kernels/moe_ffn.cu:98-302,894-908, kernels/moe_combine.cu:51-116,541-613).
//
// Why one launch. With one token every launch of the layer is a pure weight stream, and each launch boundary drains
// the memory pipe: the next kernel has to start, find its expert ids, chase them through the slot table and only then
// request weights. Here the grid is resident for the whole layer:
//
//   * Gate/up phase. The work items are the output rows of every live group, the shared expert's first: its addresses
//     are kernel arguments, so its rows are requested in the first instructions of the kernel, and the selection
//     (wave 0 of every block, from the FP32 logits) and the walk through the slot table run underneath that stream.
//   * Hand-over without a barrier instruction. Each activation h[g][j] is stored as one 32-bit word
//     (launch tag << 16 | BF16 value) with a device-coherent store. A reader accepts a word only when its tag is this
//     launch's, so data and "ready" flag are one atomic store: no waiting for stores to be acknowledged and no
//     cache-wide operations (a release / acquire pair at device scope writes back and invalidates whole L2s; with
//     2048 waves doing that the layer took 60 us longer). The arena starts zero-filled (tag 0 is never used) and the
//     last block to leave clears the words again, so a launch never meets words of an earlier one.
//   * Down phase. A work item is one OUTPUT row of y with the rows of every group's down matrix that produce it, in
//     combine order, so the per-expert results of a row meet in one wave: weighting and the ordered combine happen in
//     registers, contributions are neither written nor read back. The first down rows are requested before the block
//     looks at the activations, so the memory pipe stays busy while the last gate/up items of the grid finish.
//   * Items are claimed from device-wide counters, two items ahead of the one being computed (see the kernel).
//
// Arithmetic: per weight row the chunk -> lane mapping, the step order and the wave reduction are those of
// k_decode_stage, and the rounding boundaries those of k_decode_stage + k_combine, so ids, weights and y are bit-identical
// to the separate launches.
//
// Measured on MI355X at the DeepSeek-V3 shape (8 of 256 experts + shared, FP8): 91 us per launch against 79 us for
// the gate/up, down and combine launches it replaces, so the layer does not use it by default. Where the time goes,
// from per-block timestamps: the gate/up phase ends 6 us later than the stand-alone gate/up kernel, and reading the
// 74 KB of tagged activations coherently from every block (38 MB out of a handful of memory channels) takes 15 us.
//
// The grid must be co-resident (the launcher sizes it from the occupancy query). Every wait is bounded: a block that
// gives up sets bit 1 of *status and still leaves the kernel.
#pragma once
#include "decode_kernel.cuh"
#include <stdlib.h>

namespace ffmoe {

// groups (live choices + shared expert) whose weight rows a wave keeps in flight in the down phase
#define FFMOE_TOKEN_GROUPS 9

template <class F, int S0, int S1>
__global__ __launch_bounds__(256) void k_token_layer(const FinishParams q) {
  const DecodeParams& p = q.d;
  extern __shared__ __align__(16) uint8_t lds[];
  const int H = p.hidden, K = p.top_k, I = p.inter, SI = p.shared_inter;
  const int imax = I > SI ? I : SI;
  uint8_t* xs = lds;                  // [hidden] BF16 token
  uint8_t* hs = lds + size_t(H) * 2;  // [top_k + 1][imax] BF16 activations, one row per down-phase position
  __shared__ int s_ids[FFMOE_MAX_TOP_K];
  __shared__ float s_w[FFMOE_MAX_TOP_K];
  __shared__ int s_choice[FFMOE_MAX_TOP_K];  // live choices in combine order
  __shared__ uint64_t s_slot[FFMOE_MAX_TOP_K][6];
  __shared__ float s_glob[FFMOE_MAX_TOP_K][3];
  __shared__ float s_wk[FFMOE_MAX_TOP_K];
  __shared__ int s_nr, s_gave_up, s_last;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = uni(tid >> 6);
  // launch tag, 1 .. 65535: never 0, so a zero-filled arena holds no word that looks valid
  const uint32_t tag = q.tag;  // chosen by the host per launch: launches in flight on different streams never share one
  const bool ordered = !(q.mode == FFMOE_COMBINE_ACCUM_FP32 || q.mode == FFMOE_COMBINE_ACCUM_BF16);
  const bool select_here = p.route.logits != nullptr;
  const int has_shared = p.has_shared;
  if (tid == 0) s_gave_up = 0;

  // Work is claimed, not assigned: waves differ in speed (a wave that became resident later loses instruction issue
  // to the older wave of its SIMD for the whole kernel), and with fixed shares the slow half of the grid finishes long
  // after the fast half has gone idle. The grid is split into NP partitions (block index mod NP), each with its own
  // claim counters: a device-wide atomic on one address takes tens of nanoseconds, so the claims are spread over NP
  // addresses; item_of() below says which items a partition owns. A wave's first
  // two items per phase are fixed (claims 0 .. 2 * waves - 1 of its partition), the rest come from the counter, always
  // two items ahead of the one being computed, so the atomic's round trip is never waited for.
  const int NP = (gridDim.x & 63) == 0 ? 64 : ((gridDim.x & 7) == 0 ? 8 : 1);
  const int part = int(blockIdx.x % NP);
  const int bp = int(blockIdx.x / NP);           // block index inside the partition
  const int pwaves = int(gridDim.x / NP) * 4;    // waves of the partition
  const int pw = bp * 4 + wave;                  // this wave inside the partition
  unsigned int* cnt_gu = q.claims + part * 32;   // every counter on its own 128-byte line
  unsigned int* cnt_dn = q.claims + (64 + part) * 32;
  // The claim is an atomic INCREMENT (wrap bound 2^32 - 1), not an add: the compiler rewrites a wave's atomic adds
  // into one aggregated add whose result it needs at once, and that wait would drain the wave's weight requests.
  // Work item of claim c of this partition: the item space is cut into runs of `pwaves` consecutive items dealt
  // round-robin to the partitions, so the waves of a block (and the blocks of a partition, which share an XCD) work on
  // neighbouring weight rows at the same time.
  auto item_of = [&](int c) { return ((c / pwaves) * NP + part) * pwaves + (c % pwaves); };
  auto claim_request = [&](unsigned int* cnt, int& pend) {
    if (lane == 0) pend = int(__builtin_amdgcn_atomic_inc32(cnt, 0xffffffffu, __ATOMIC_RELAXED, "agent"));
  };

  // ---- gate/up phase ------------------------------------------------------------------------------------------
  // flat unit space: the shared expert's rows first (their addresses are kernel arguments), then the live choices in
  // combine order; unit f of group position pos, row j
  const int nchunks0 = H / F::EPL;
  const int SIu = has_shared ? SI : 0;
  typename F::Chunk gbuf[2][S0];
  typename F::Row crow[2], nrow[2];
  auto gu_decode = [&](int f, int& pos, int& j) {
    if (f < SIu) { pos = 0; j = f; }
    else { const int g = (f - SIu) / I; pos = has_shared + g; j = f - SIu - g * I; }
  };
  auto gu_rows = [&](int pos, int j, typename F::Row (&r)[2]) {
    if (has_shared && pos == 0) {
      r[0] = F::row(p.shared_slot[0], p.shared_slot[1], p.shared_global[0], j, H);
      r[1] = F::row(p.shared_slot[2], p.shared_slot[3], p.shared_global[1], j, H);
    } else {
      const int i = pos - has_shared;
      r[0] = F::row(uni64(s_slot[i][0]), uni64(s_slot[i][1]), unif(s_glob[i][0]), j, H);
      r[1] = F::row(uni64(s_slot[i][2]), uni64(s_slot[i][3]), unif(s_glob[i][1]), j, H);
    }
  };
  auto gu_issue = [&](const typename F::Row (&r)[2], int s) {
    const int chunk = s * 64 + lane;
    const int cc = chunk < nchunks0 ? chunk : nchunks0 - 1;
    F::load(gbuf[0][s], r[0], cc);
    F::load(gbuf[1][s], r[1], cc);
  };
  int f_cur = item_of(pw);            // fixed claims 0 and 1
  int f_nxt = item_of(pwaves + pw);
  int f_claim = pwaves + pw;          // claim index of f_nxt (fixed shares only)
  int cpos = 0, cj = 0;
  // the token is requested ahead of the weights (loads return in order) and written to LDS behind them
  constexpr int XV = 4;
  u32x4 xv[XV];
#pragma unroll
  for (int i = 0; i < XV; ++i) {
    const int v = i * 256 + tid;
    xv[i] = load16(p.x + size_t(v < (H >> 3) ? v : 0) * 8);
  }
  // a first item in the shared expert goes out before anything else
  const bool early = f_cur < SIu;
  if (early) { cj = f_cur; gu_rows(0, cj, crow); }
  // Wave 0 prepares the block before it requests any weights, so none of its loads queue behind a weight stream:
  // selection, live choices in combine order, and the slot-table entries of the live experts. The other waves are
  // already streaming the shared expert.
  if (wave == 0) {
    if (select_here) {
      wave_route_dispatch(p.route.logits, p.route.bias, lane, p.experts, K, p.route.score_mode, p.route.routed_scaling,
                          p.route.n_group, p.route.topk_group, s_ids, s_w, 1);
    } else if (lane < K) {
      s_ids[lane] = p.ids[lane];
      s_w[lane] = p.weights_f32 ? reinterpret_cast<const float*>(p.weights)[lane] : bf16_to_f32(reinterpret_cast<const uint16_t*>(p.weights)[lane]);
    }
    wave_lds_fence();
    // live choices in combine order (ascending expert id, stable; choice order for the accumulate modes)
    auto is_live = [&](int c) {
      const int e = s_ids[c];
      if (p.active && p.active[c] == 0u) return false;
      if ((unsigned)e >= (unsigned)p.experts || (p.valid && p.valid[e] == 0u)) return false;
      return !(p.generation && p.assignment_gen && p.generation[e] != p.assignment_gen[c]);
    };
    bool live = false;
    if (lane < K) {
      const int mine = s_ids[lane];
      live = is_live(lane);
      if (!live && (!p.active || p.active[lane] != 0u) && q.status && blockIdx.x == 0) atomicOr(q.status, 1u);  // bad expert id
      int rank = 0;
      for (int c = 0; c < K; ++c) {
        const int other = s_ids[c];
        const bool before = ordered ? (other < mine || (other == mine && c < lane)) : c < lane;
        rank += (is_live(c) && before) ? 1 : 0;
      }
      if (live) s_choice[rank] = lane;
      if (select_here && blockIdx.x == 0) {
        const_cast<int*>(p.ids)[lane] = mine;
        reinterpret_cast<float*>(const_cast<void*>(p.weights))[lane] = s_w[lane];
      }
    }
    const int live_count = __builtin_popcountll(__ballot(live));
    if (lane == 0) s_nr = live_count;
    wave_lds_fence();
    if (lane < live_count) {
      const int c = s_choice[lane];
      const int e = s_ids[c];
#pragma unroll
      for (int i = 0; i < 6; ++i) s_slot[lane][i] = p.slots[size_t(e) * 6 + i];
#pragma unroll
      for (int i = 0; i < 3; ++i) s_glob[lane][i] = p.global_scales ? p.global_scales[size_t(e) * 3 + i] : 1.0f;
      s_wk[lane] = s_w[c];
    }
  }
  if (early) {
#pragma unroll
    for (int s = 0; s < S0; ++s) gu_issue(crow, s);
  }
  {
    u32x4* d4 = reinterpret_cast<u32x4*>(xs);
#pragma unroll
    for (int i = 0; i < XV; ++i)
      if (i * 256 + tid < (H >> 3)) d4[i * 256 + tid] = xv[i];
    for (int v = XV * 256 + tid; v < (H >> 3); v += 256) d4[v] = load16(p.x + size_t(v) * 8);
  }
  __syncthreads();
  const int nr = uni(s_nr);
  const int ng = nr + has_shared;
  const int Utot = SIu + nr * I;

  int pend = 0;  // lane 0: the claim of the current pass
  bool have = f_cur < Utot;
  if (have && !early) {
    gu_decode(f_cur, cpos, cj);
    gu_rows(cpos, cj, crow);
#pragma unroll
    for (int s = 0; s < S0; ++s) gu_issue(crow, s);
  }
  auto gu_finish_item = [&](float (&acc)[2][1]) {
    const float g = wave_sum(acc[0][0]), u = wave_sum(acc[1][0]);
    const uint32_t hv = swiglu_bf16(bround(g), bround(u), p.swiglu, p.swiglu_limit);
    const int row = (has_shared && cpos == 0) ? K : cpos - has_shared;
    if (lane == 0) store_agent(q.h32 + size_t(row) * p.h_stride + cj, (tag << 16) | hv);
  };
  // Every pass computes item f_cur while requesting the weights of f_nxt, and claims the item after that: the claim
  // goes out first (ahead of the pass's weight requests, so it returns before them) and is read at the end of the
  // same pass, so no memory operation other than the weight requests is in flight across the loop edge.
  while (have) {
    if (f_nxt >= Utot) break;
    if (q.dynamic) claim_request(cnt_gu, pend);
    int npos, nj;
    gu_decode(f_nxt, npos, nj);
    gu_rows(npos, nj, nrow);
    float acc[2][1] = {{0.0f}, {0.0f}};
#pragma unroll
    for (int s = 0; s < S0; ++s) {
      step_compute<F, 2, 1, S0>(gbuf, s, xs, H, nchunks0, s * 64 + lane, 1, acc);
      gu_issue(nrow, s);
    }
    gu_finish_item(acc);
    cpos = npos; cj = nj;
    f_cur = f_nxt;
    if (q.dynamic) {
      f_nxt = item_of(2 * pwaves + uni(pend));
    } else {
      f_claim += pwaves;
      f_nxt = item_of(f_claim);
    }
    crow[0] = nrow[0]; crow[1] = nrow[1];
  }
  // ---- down phase: first rows requested before the activations are looked at ---------------------------------
  // positions: the live choices in combine order, then the shared expert. A work item is ONE output row of y with
  // the rows of every group's down matrix that produce it, so the per-expert results meet in one wave and weighting
  // and the ordered combine happen in registers; the next item's weight rows are requested slot by slot as the
  // current item's are consumed (about ng * 2 * inter bytes in flight per wave).
  constexpr int G = FFMOE_TOKEN_GROUPS;
  typename F::Chunk dbuf[G][1][S1];
  int d_cur = item_of(pw);            // fixed claims 0 and 1
  int d_nxt = item_of(pwaves + pw);
  int d_claim = pwaves + pw;
  // Straight-line requests: a position past the last group reads one 16-byte word of the token instead (the same
  // word for every lane), so the number of loads in flight never depends on a branch and the waits stay exact.
  auto d_issue = [&](auto slot_c, int d) {
    constexpr int pos = decltype(slot_c)::value;
    const bool live = pos < ng;
    const bool sh = pos == nr;  // only with has_shared
    const int lp = live && !sh ? pos : 0;
    const uint64_t codes = !live ? uint64_t(p.x) : (sh ? p.shared_slot[4] : uni64(s_slot[lp][4]));
    const uint64_t scales = !live ? uint64_t(p.x) : (sh ? p.shared_slot[5] : uni64(s_slot[lp][5]));
    const float glob = !live ? 1.0f : (sh ? p.shared_global[2] : unif(s_glob[lp][2]));
    const int Kg = sh ? SI : I;
    const int nchunks = Kg / F::EPL;
    const typename F::Row row = F::row(codes, scales, glob, live ? d : 0, Kg);
#pragma unroll
    for (int s = 0; s < S1; ++s) {
      const int chunk = s * 64 + lane;
      const int cc = !live ? 0 : (chunk < nchunks ? chunk : nchunks - 1);
      F::load(dbuf[pos][0][s], row, cc);
    }
  };
  if (have) {  // the wave's last gate/up item, with the first down row requested underneath it
    float acc[2][1] = {{0.0f}, {0.0f}};
#pragma unroll
    for (int s = 0; s < S0; ++s) step_compute<F, 2, 1, S0>(gbuf, s, xs, H, nchunks0, s * 64 + lane, 1, acc);
    gu_finish_item(acc);
  }
  if (d_cur < H) static_for<G>([&](auto pc) { d_issue(pc, d_cur); });
  // Activations of every group: tagged words -> BF16 rows in LDS, by the whole block. A word is accepted only with
  // this launch's tag; the last words arrive when the slowest wave of the grid has finished its last gate/up item,
  // and until then the rows requested above keep the memory pipe busy.
  {
    constexpr int HWB = 12;  // 64-bit words per thread and round trip
    const int row_pairs = imax >> 1;  // slots per group row; a shorter row leaves its tail unused
    const int total = ng * row_pairs;
    for (int v0 = 0; v0 < total; v0 += 256 * HWB) {
      uint64_t hw[HWB];
      bool mine[HWB];
      for (unsigned int spins = 0;; ++spins) {
#pragma unroll
        for (int i = 0; i < HWB; ++i) {
          const int v = v0 + i * 256 + tid;
          const int pos = v / row_pairs, w = v - pos * row_pairs;
          mine[i] = v < total && w < (((pos == nr) ? SI : I) >> 1);
          const uint64_t* src = reinterpret_cast<const uint64_t*>(q.h32 + size_t(pos == nr ? K : pos) * p.h_stride) + w;
          hw[i] = mine[i] ? __hip_atomic_load(src, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : 0ull;
        }
        bool ok = true;
#pragma unroll
        for (int i = 0; i < HWB; ++i)
          ok = ok && (!mine[i] || (((uint32_t(hw[i]) >> 16) == tag) && (uint32_t(hw[i] >> 48) == tag)));
        if (ok) break;
        if (spins >= q.spin_limit) { s_gave_up = 1; break; }
        __builtin_amdgcn_s_sleep(8);
      }
#pragma unroll
      for (int i = 0; i < HWB; ++i) {
        const int v = v0 + i * 256 + tid;
        const int pos = v / row_pairs, w = v - pos * row_pairs;
        if (mine[i]) reinterpret_cast<uint32_t*>(hs + size_t(pos) * imax * 2)[w] = (uint32_t(hw[i]) & 0xffffu) | (uint32_t(hw[i] >> 32) << 16);
      }
    }
  }
  __syncthreads();

  // ---- down phase + combine --------------------------------------------------------------------------------------
  const float sc = (q.mode == FFMOE_COMBINE_GATED) ? bf16_to_f32(q.scale[0]) : 0.0f;
  auto down_row = [&](auto last_c) {
    constexpr bool LAST = decltype(last_c)::value;  // nothing left to request
    float sum = 0.0f, shv = 0.0f;  // running combine and shared output of row d_cur (wave-uniform)
    static_for<G>([&](auto pc) {
      constexpr int pos = decltype(pc)::value;
      if (pos < ng) {
        const bool sh = pos == nr;
        const int Kg = sh ? SI : I;
        float acc[1][1] = {{0.0f}};
#pragma unroll
        for (int s = 0; s < S1; ++s)
          step_compute<F, 1, 1, S1>(dbuf[pos], s, hs + size_t(pos) * imax * 2, Kg, Kg / F::EPL, s * 64 + lane, 1, acc);
        const float total = wave_sum(acc[0][0]);
        if (sh) {
          shv = bround(total);  // the BF16 shared output
        } else {
          const float v = __fmul_rn(p.routed_weight == FFMOE_WEIGHT_AFTER_DOWN_BF16 ? bround(total) : total, unif(s_wk[pos]));
          const float c = bround(v);  // the BF16 contribution
          sum = q.mode == FFMOE_COMBINE_BF16 ? bround(__fadd_rn(sum, c)) : __fadd_rn(sum, c);
        }
      }
      if (!LAST) d_issue(pc, d_nxt);  // the register slot is free: the same group's row of the next item
    });
    float v;
    switch (q.mode) {
      case FFMOE_COMBINE_GATED: v = __fadd_rn(bround(sum), bround(__fmul_rn(sc, shv))); break;
      case FFMOE_COMBINE_UNGATED:
      case FFMOE_COMBINE_ACCUM_BF16: v = __fadd_rn(bround(sum), shv); break;
      case FFMOE_COMBINE_BF16:
      case FFMOE_COMBINE_ACCUM_FP32: v = __fadd_rn(sum, shv); break;
      default: v = sum; break;
    }
    if (lane == 0) q.y[d_cur] = f32_to_bf16(v);
  };
  while (d_nxt < H) {  // d_cur < d_nxt: both valid
    if (q.dynamic) claim_request(cnt_dn, pend);  // the item after d_nxt; read at the end of this pass
    down_row(std::false_type{});
    d_cur = d_nxt;
    if (q.dynamic) {
      d_nxt = item_of(2 * pwaves + uni(pend));
    } else {
      d_claim += pwaves;
      d_nxt = item_of(d_claim);
    }
  }
  if (d_cur < H) down_row(std::true_type{});
  __syncthreads();
  if (tid == 0) {
    if (s_gave_up && q.status) atomicOr(q.status, 2u);
    const unsigned int left = __hip_atomic_fetch_add(q.exited, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    s_last = left + 1 == gridDim.x;
    if (s_last) {  // last block out: clear the claim counters
      for (int i = 0; i < 128; ++i) __hip_atomic_store(q.claims + i * 32, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      __hip_atomic_store(q.exited, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
  }
  __syncthreads();
  // Every other block has left, so nobody reads the arena any more: the last block hands it back zero-filled, as it
  // found it. A launch therefore never meets a word of an earlier one, whatever their shapes and however often the
  // 16-bit tag has come round.
  if (s_last) {
    const int words = (K + 1) * p.h_stride;
    for (int i = tid; i < words; i += 256) q.h32[i] = 0u;
  }
}

template <class F, int S0, int S1MAX, int S1 = 1>
int launch_token_layer_s1(int want1, const FinishParams& q, size_t lds, hipStream_t st) {
  if constexpr (S1 <= S1MAX) {
    if (want1 != S1) return launch_token_layer_s1<F, S0, S1MAX, S1 + 1>(want1, q, lds, st);
    auto kernel = k_token_layer<F, S0, S1>;
    static int per_cu = -1;  // co-resident blocks per CU for this instantiation
    static size_t per_cu_lds = 0;
    if (per_cu < 0 || per_cu_lds != lds) {
      int nb = 0;
      per_cu = hipOccupancyMaxActiveBlocksPerMultiprocessor(&nb, kernel, 256, lds) == hipSuccess ? nb : 0;
      per_cu_lds = lds;
    }
    if (per_cu < 1) return FFMOE_ERR_UNSUPPORTED;
    const int blocks = decode_num_cus() * (per_cu < 2 ? per_cu : 2);
    hipLaunchKernelGGL(kernel, dim3(blocks), dim3(256), lds, st, q);
    return ff_launch_status();
  }
  return FFMOE_ERR_UNSUPPORTED;
}

template <class F, int S0MAX, int S0 = 1>
int launch_token_layer_s0(int want0, int want1, const FinishParams& q, size_t lds, hipStream_t st) {
  if constexpr (S0 <= S0MAX) {
    if (want0 == S0) return launch_token_layer_s1<F, S0, Policy<F>::S1>(want1, q, lds, st);
    return launch_token_layer_s0<F, S0MAX, S0 + 1>(want0, want1, q, lds, st);
  }
  return FFMOE_ERR_UNSUPPORTED;
}

// FFMOE_ERR_UNSUPPORTED (nothing launched): a weight row needs more loads per lane than the register buffers hold, or
// the wave's slice of y does not fit one row per lane; the caller then runs the separate launches.
template <class F>
int launch_token_layer(const FinishParams& q, hipStream_t st) {
  const DecodeParams& p = q.d;
  const int imax = p.inter > p.shared_inter ? p.inter : p.shared_inter;
  const int steps0 = (p.hidden / F::EPL + 63) / 64, steps1 = (imax / F::EPL + 63) / 64;
  if (steps0 > Policy<F>::S0 || steps1 > Policy<F>::S1)
    return ff_fail(FFMOE_ERR_UNSUPPORTED, "one-launch token layer: rows of %d / %d elements exceed the register buffers", p.hidden, imax);
  if (p.top_k + (p.has_shared ? 1 : 0) > FFMOE_TOKEN_GROUPS)
    return ff_fail(FFMOE_ERR_UNSUPPORTED, "one-launch token layer: %d groups exceed the %d a wave keeps in flight", p.top_k + (p.has_shared ? 1 : 0), FFMOE_TOKEN_GROUPS);
  const size_t lds = size_t(p.hidden) * 2 + size_t(p.top_k + 1) * imax * 2;
  if (lds > 72 * 1024)
    return ff_fail(FFMOE_ERR_UNSUPPORTED, "one-launch token layer: %zu bytes of LDS per block", lds);
  return launch_token_layer_s0<F, Policy<F>::S0>(steps0, steps1, q, lds, st);
}

}  // namespace ffmoe
