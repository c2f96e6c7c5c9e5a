// Router kernels: logits (BF16 chain contract / FP32 wave-reduced) and deterministic top-k.
// Behaviour follows kernels/moe_route.cu of the reference; the mapping to wave64 is new.
#include "common.cuh"
#include "route_select.cuh"
#include "api.h"
#include <stdlib.h>
#include <algorithm>

namespace ffmoe {

// ---------------------------------------------------------------------------------------------
// logits[r,e] = bf16(fma chain over k ascending). One lane owns one (row, expert) chain
// (kernels/moe_route.cu:392-403, :536-544): 2 * hidden dependent fmas, serial by contract. What the lane must not also
// do is fetch its router row itself - 64 lanes reading 16 bytes each of 64 different rows is 64 cache lines per load
// instruction, and that, not the chain, was the kernel's time (22.8 us for 64 experts x 2048). A block is five waves: four
// of them move the router tile of 64 experts x 256 columns through LDS with coalesced requests (32 lanes per 512-byte row
// segment), one chunk ahead, multiplied by the token's values on the way (see the kernel), and wave 0 does nothing but run
// the 64 chains out of LDS (rows padded by 16 bytes, so the 16 lanes of a quarter wave read 16 different LDS slots). A
// dependent FP32 add or fma takes 8 cycles on this machine; fed from LDS the chain runs at 8.7 cycles per element with one
// operand per element and at 12.1 with two (2048 elements: 7.5 and 10.3 us); the chain wave is kept clear of everything else.
__device__ __forceinline__ int rank_of(const float* s_key, int padded, float mine, int e);

// Softmax / sigmoid top-k of at most 64 experts by the wave whose lane e holds expert e's BF16 logit: the arithmetic of
// k_route_topk for a block of one wave, operation for operation (the softmax denominator as the reference's 32-lane trees
// and the tree over the two 32-lane sums, selection by rank, weights = score / sum of the picked scores in pick order), with
// the block-wide exchanges replaced by the wave's own LDS scratch (LDS operations of one wave execute in order).
// s_key: 64 floats, 16-byte aligned; s_sel / s_selid: FFMOE_MAX_TOP_K entries.
__device__ __forceinline__ void wave_topk64(float logit, bool live, int lane, int top_k, int score_mode, float* s_key, float* s_sel,
                                            int* s_selid, int* __restrict__ ids_row, uint16_t* __restrict__ weights_row) {
  float score;
  if (score_mode == FFMOE_SCORE_SOFTMAX) {
    const float m = wave_max(logit);
    const float ev = live ? det_expf(__fsub_rn(logit, m)) : 0.0f;
    float v = ev;
#pragma unroll
    for (int off = 16; off > 0; off >>= 1) {
      const float o = __shfl_down(v, off, 32);
      v = __fadd_rn(v, ((lane & 31) + off < 32) ? o : 0.0f);
    }
    const float upper = __shfl(v, 32);  // the second 32-lane group's sum
    v = lane == 0 ? v : (lane == 1 ? upper : 0.0f);
#pragma unroll
    for (int off = 16; off > 0; off >>= 1) {
      const float o = __shfl_down(v, off, 32);
      v = __fadd_rn(v, ((lane & 31) + off < 32) ? o : 0.0f);
    }
    const float den = __shfl(v, 0);
    score = live ? __fdiv_rn(ev, den) : -INFINITY;
  } else {
    score = live ? sigmoid1(logit) : -INFINITY;
  }
  s_key[lane] = score;
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  if (live) {
    const int rank = rank_of(s_key, 64, score, lane);
    if (rank < top_k) { s_sel[rank] = score; s_selid[rank] = lane; }
  }
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  if (lane < top_k) {
    float tsum = 0.0f;
    for (int r = 0; r < top_k; ++r) tsum = __fadd_rn(tsum, s_sel[r]);
    const float den = score_mode == FFMOE_SCORE_SOFTMAX ? tsum : __fadd_rn(tsum, 1.0e-20f);
    ids_row[lane] = s_selid[lane];
    weights_row[lane] = f32_to_bf16(__fdiv_rn(s_sel[lane], den));
  }
}

constexpr int LOGIT_CHUNK = 256;                      // columns per chunk
constexpr int LOGIT_ROW_BYTES = LOGIT_CHUNK * 4 + 16;  // a row of the tile as FP32, padded by one 16-byte slot
// SELECT (at most 64 experts, i.e. one block per row): the chain wave goes on to the top-k of its row, whose logits it holds
// one per lane - the selection launch and the logits' round trip through memory fall away.
template <bool SELECT>
__global__ __launch_bounds__(320) void k_route_logits_bf16(const uint16_t* __restrict__ x, const uint16_t* __restrict__ router,
                                                           uint16_t* __restrict__ logits, int rows, int experts, int hidden,
                                                           int* __restrict__ ids, uint16_t* __restrict__ weights, int top_k, int score_mode) {
  // The waves that move the router tile leave PRODUCTS in LDS: x[k] * w[e][k] of two BF16 values has at most 16 significant
  // bits and is exact in FP32 unless it falls below the normal range, and then fma(x, w, acc) = acc + product, one rounding
  // either way. The chain wave's step is one dependent add with one LDS operand per four elements (8.7 cycles per element
  // against 12.1 for the fma with the token and the router element read separately). A product that is zero or subnormal -
  // an exact zero in the token or the router, or an underflow - flags its chunk, and the chain wave then runs that chunk
  // as fmas on the BF16 values themselves: the same bits for every input.
  __shared__ __attribute__((aligned(16))) uint8_t tile[2][64 * LOGIT_ROW_BYTES];
  __shared__ int s_inexact[2];
  const int lane = threadIdx.x & 63, wave = uni(int(threadIdx.x >> 6));
  const int tid = int(threadIdx.x) - 64;                  // index among the 256 moving threads (wave 0: negative, moves nothing)
  const bool mover = wave != 0;
  const int e0 = blockIdx.x * 64;
  const int row = blockIdx.y;
  const int words = hidden >> 3;                          // 16-byte pieces (8 columns) per row
  const int chunks = (words + 31) >> 5;
  // piece (r, q) of a chunk for i = 0 .. 7: r = (tid + 256 i) / 32, q = (tid + 256 i) % 32 = tid % 32: a thread moves the same
  // eight columns of eight router rows and needs the token's eight values of those columns. Pieces past the end of the row
  // repeat its last piece; nothing adds them.
  // The movers run two chunks ahead in two register sets (chunk c in set c % 2): a chunk's chains take about 0.9 us, less than a
  // request that misses the caches.
  u32x4 regs[2][8], xreg[2];
  auto request = [&](auto set, int c) {
    constexpr int S = decltype(set)::value;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int idx = tid + 256 * i;
      const int r = idx >> 5, q = idx & 31;
      const int er = min(e0 + r, experts - 1);
      const int piece = min(32 * c + q, words - 1);
      regs[S][i] = load16(router + size_t(er) * hidden + size_t(piece) * 8);
    }
    xreg[S] = load16(x + size_t(row) * hidden + size_t(min(32 * c + (tid & 31), words - 1)) * 8);
  };
  auto publish = [&](auto set) {  // chunk c sits in set c % 2 and goes to buffer c % 2
    constexpr int S = decltype(set)::value;
    float xf[8];
#pragma unroll
    for (int j = 0; j < 4; ++j) { xf[2 * j] = bf16lo(xreg[S][j]); xf[2 * j + 1] = bf16hi(xreg[S][j]); }
    float smallest = INFINITY;  // of the products' magnitudes
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int idx = tid + 256 * i;
      const u32x4 v = regs[S][i];
      float pr[8];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        pr[2 * j] = __fmul_rn(xf[2 * j], bf16lo(v[j]));
        pr[2 * j + 1] = __fmul_rn(xf[2 * j + 1], bf16hi(v[j]));
      }
#pragma unroll
      for (int j = 0; j < 8; ++j) smallest = fminf(smallest, fabsf(pr[j]));
      uint8_t* dst = &tile[S][(idx >> 5) * LOGIT_ROW_BYTES + (idx & 31) * 32];
      const u32x4 lo = {__float_as_uint(pr[0]), __float_as_uint(pr[1]), __float_as_uint(pr[2]), __float_as_uint(pr[3])};
      const u32x4 hi = {__float_as_uint(pr[4]), __float_as_uint(pr[5]), __float_as_uint(pr[6]), __float_as_uint(pr[7])};
      *reinterpret_cast<u32x4*>(dst) = lo;
      *reinterpret_cast<u32x4*>(dst + 16) = hi;
    }
    if (smallest < 1.17549435e-38f) s_inexact[S] = 1;  // a zero or a subnormal product
  };
  using S0 = std::integral_constant<int, 0>;
  using S1 = std::integral_constant<int, 1>;
  if (threadIdx.x < 2) s_inexact[threadIdx.x] = 0;
  __syncthreads();
  if (mover) {
    request(S0{}, 0);
    if (chunks > 1) request(S1{}, 1);
    publish(S0{});
    if (chunks > 2) request(S0{}, 2);
  }
  __syncthreads();
  float acc = 0.0f;
  // stage c: the chain wave reads buffer c % 2; the movers publish chunk c + 1 into the other buffer and request chunk c + 3
  auto stage = [&](auto other, int c) {
    if (mover) {
      if (c + 1 < chunks) publish(other);
      if (c + 3 < chunks) request(other, c + 3);
    } else {
      const int nquads = 2 * min(32, words - 32 * c);  // groups of four columns
      if (uni(s_inexact[c & 1]) == 0) {
        const uint8_t* prow = &tile[c & 1][lane * LOGIT_ROW_BYTES];
#pragma unroll 8
        for (int q = 0; q < nquads; ++q) {
          const u32x4 pv = *reinterpret_cast<const u32x4*>(prow + q * 16);
#pragma unroll
          for (int j = 0; j < 4; ++j) acc = __fadd_rn(acc, __uint_as_float(pv[j]));
        }
      } else {
        // a product of this chunk is not exact (or is an exact zero, which looks the same): the fmas on the values themselves
        const uint16_t* wr = router + size_t(min(e0 + lane, experts - 1)) * hidden + size_t(c) * LOGIT_CHUNK;
        const uint16_t* xr = x + size_t(row) * hidden + size_t(c) * LOGIT_CHUNK;
        for (int q = 0; q < nquads; q += 2) {
          const u32x4 wv = load16(wr + q * 4), xv = load16(xr + q * 4);
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            acc = __fmaf_rn(bf16lo(xv[j]), bf16lo(wv[j]), acc);
            acc = __fmaf_rn(bf16hi(xv[j]), bf16hi(wv[j]), acc);
          }
        }
        if (lane == 0) s_inexact[c & 1] = 0;  // the buffer's next chunk starts clean (the movers write behind the barrier)
      }
    }
    __syncthreads();
  };
  for (int c = 0; c < chunks; c += 2) {
    stage(S1{}, c);
    if (c + 1 < chunks) stage(S0{}, c + 1);
  }
  if (!mover) {
    const bool live = e0 + lane < experts;
    const uint16_t lb = f32_to_bf16(acc);
    if (live) logits[size_t(row) * experts + e0 + lane] = lb;
    if constexpr (SELECT) {
      // the tiles are no longer read (every wave is past the last barrier): the head of buffer 0 is the wave's scratch
      float* s_key = reinterpret_cast<float*>(&tile[0][0]);
      float* s_sel = s_key + 64;
      int* s_selid = reinterpret_cast<int*>(s_sel + FFMOE_MAX_TOP_K);
      wave_topk64(live ? bf16_to_f32(lb) : -INFINITY, live, lane, top_k, score_mode, s_key, s_sel, s_selid, ids + size_t(row) * top_k,
                  weights + size_t(row) * top_k);
    }
  }
}

// FP32 logits. One block of 256 threads per expert: thread p chains the 8-element vectors p, p+256, ... in ascending
// order; the 256 partials are summed by a balanced pairwise tree in natural order (adjacent pairs, then pairs of
// pairs, ...), which is what the DPP wave sum followed by ((w0+w1)+(w2+w3)) computes. The router row stays in
// registers while the block walks over the token rows.
__device__ __forceinline__ float logit_block_sum(float acc, float* s_part) {
  const float w = wave_sum(acc);
  const int wave = threadIdx.x >> 6;
  if ((threadIdx.x & 63) == 0) s_part[wave] = w;
  __syncthreads();
  const float total = __fadd_rn(__fadd_rn(s_part[0], s_part[1]), __fadd_rn(s_part[2], s_part[3]));
  __syncthreads();
  return total;
}

constexpr int LOGIT_ROWS = 8;  // token rows per block
constexpr int LOGIT_PF = 4;  // vectors per thread held in registers: covers hidden <= 8192 in one batch

__device__ __forceinline__ void logits_f32_rows(const uint16_t* __restrict__ x, const uint16_t* __restrict__ router,
                                                float* __restrict__ logits, int e, int r0, int r1, int experts, int hidden,
                                                float* s_part) {
  const int tid = threadIdx.x;
  const int words = hidden >> 3;
  const uint16_t* wr = router + size_t(e) * hidden;
  const bool one_batch = words <= 256 * LOGIT_PF;
  u32x4 wv[LOGIT_PF];
  if (one_batch) {
#pragma unroll
    for (int i = 0; i < LOGIT_PF; ++i) {
      const int v = tid + 256 * i;
      wv[i] = load16(wr + size_t(v < words ? v : words - 1) * 8);
    }
  }
  if (one_batch && r1 - r0 <= LOGIT_ROWS) {
    // The router row stays in registers; the next token row is requested while this one is multiplied, and the block-wide
    // sums of all the block's rows share one barrier (same products, same order, same tree per row).
    u32x4 xv[LOGIT_PF], xn[LOGIT_PF];
    float accs[LOGIT_ROWS];
    float wf[LOGIT_PF][8];  // the router row widened once, not once per token row
#pragma unroll
    for (int i = 0; i < LOGIT_PF; ++i)
#pragma unroll
      for (int q = 0; q < 4; ++q) { wf[i][2 * q] = bf16lo(wv[i][q]); wf[i][2 * q + 1] = bf16hi(wv[i][q]); }
#pragma unroll
    for (int i = 0; i < LOGIT_PF; ++i) {
      const int v = tid + 256 * i;
      xn[i] = load16(x + size_t(r0) * hidden + size_t(v < words ? v : words - 1) * 8);
    }
#pragma unroll
    for (int k = 0; k < LOGIT_ROWS; ++k) {
      accs[k] = 0.0f;
      if (r0 + k < r1) {
#pragma unroll
        for (int i = 0; i < LOGIT_PF; ++i) xv[i] = xn[i];
        if (r0 + k + 1 < r1) {
#pragma unroll
          for (int i = 0; i < LOGIT_PF; ++i) {
            const int v = tid + 256 * i;
            xn[i] = load16(x + size_t(r0 + k + 1) * hidden + size_t(v < words ? v : words - 1) * 8);
          }
        }
        float acc = 0.0f;
#pragma unroll
        for (int i = 0; i < LOGIT_PF; ++i) {
          if (tid + 256 * i < words) {
#pragma unroll
            for (int q = 0; q < 4; ++q) {
              acc = __fmaf_rn(bf16lo(xv[i][q]), wf[i][2 * q], acc);
              acc = __fmaf_rn(bf16hi(xv[i][q]), wf[i][2 * q + 1], acc);
            }
          }
        }
        accs[k] = acc;
      }
    }
#pragma unroll
    for (int k = 0; k < LOGIT_ROWS; ++k) {
      if (r0 + k < r1) {
        const float w = wave_sum(accs[k]);
        if ((tid & 63) == 0) s_part[4 * k + (tid >> 6)] = w;
      }
    }
    __syncthreads();
    if (tid < r1 - r0)
      logits[size_t(r0 + tid) * experts + e] =
          __fadd_rn(__fadd_rn(s_part[4 * tid], s_part[4 * tid + 1]), __fadd_rn(s_part[4 * tid + 2], s_part[4 * tid + 3]));
    return;
  }
  for (int r = r0; r < r1; ++r) {
    const uint16_t* xr = x + size_t(r) * hidden;
    float acc = 0.0f;
    for (int v0 = tid; v0 < words; v0 += 256 * LOGIT_PF) {
      u32x4 xv[LOGIT_PF];
      if (!one_batch) {
#pragma unroll
        for (int i = 0; i < LOGIT_PF; ++i) {
          const int v = v0 + 256 * i;
          wv[i] = load16(wr + size_t(v < words ? v : words - 1) * 8);
        }
      }
#pragma unroll
      for (int i = 0; i < LOGIT_PF; ++i) {
        const int v = v0 + 256 * i;
        xv[i] = load16(xr + size_t(v < words ? v : words - 1) * 8);
      }
#pragma unroll
      for (int i = 0; i < LOGIT_PF; ++i) {
        if (v0 + 256 * i < words) {
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            acc = __fmaf_rn(bf16lo(xv[i][q]), bf16lo(wv[i][q]), acc);
            acc = __fmaf_rn(bf16hi(xv[i][q]), bf16hi(wv[i][q]), acc);
          }
        }
      }
    }
    const float total = logit_block_sum(acc, s_part);
    if (tid == 0) logits[size_t(r) * experts + e] = total;
  }
}

__global__ __launch_bounds__(256) void k_route_logits_f32(const uint16_t* __restrict__ x, const uint16_t* __restrict__ router,
                                                          float* __restrict__ logits, int rows, int experts, int hidden) {
  __shared__ float s_part[4 * LOGIT_ROWS];
  const int r0 = blockIdx.y * LOGIT_ROWS;
  const int r1 = r0 + LOGIT_ROWS < rows ? r0 + LOGIT_ROWS : rows;
  logits_f32_rows(x, router, logits, blockIdx.x, r0, r1, experts, hidden, s_part);
}

// FP32 logits for many token rows (a prefill cohort: 4096 x 256 x 7168 is 15 GFLOP, and with eight rows per pass over a
// router row the kernel above re-reads the 3.67 MB router 512 times). Same products, same order, same tree per logit
// as k_route_logits_f32: partial chain p (0 .. 255) walks the 16-byte vectors p, p + 256, ... element by element, the
// 256 partials meet in the adjacent-pair tree. A block owns a tile of ME experts, whose router rows stay in LDS as BF16
// for the whole launch, and a run of token rows; it is TEAMS teams of 256 threads, thread t of a team = chain t. A
// team takes MR rows at a time: per vector it widens its slice of the MR rows once (registers) and walks the ME
// experts out of LDS, MR x 8 fmas per 16-byte LDS read, so the widening costs a fifth of the fmas. Row chunks map to
// XCDs (block index mod 8), so the blocks that read the same token rows at about the same time share an L2.
constexpr int LG_ME = 8, LG_MR = 8, LG_TEAMS = 3;

__global__ __launch_bounds__(256 * LG_TEAMS) void k_route_logits_f32_rows(const uint16_t* __restrict__ x, const uint16_t* __restrict__ router,
                                                                           float* __restrict__ logits, int rows, int experts, int hidden,
                                                                           int row_chunks) {
  extern __shared__ __align__(16) uint8_t lg_lds[];
  const int tid = threadIdx.x, team = uni(tid >> 8), t = tid & 255, lane = tid & 63, wave_in_team = uni((tid >> 6) & 3);
  const int words = hidden >> 3;
  const int nvec = (words + 255) >> 8;  // vectors per chain
  u32x4* wl = reinterpret_cast<u32x4*>(lg_lds);                                   // [ME][words] router tile
  float* part = reinterpret_cast<float*>(lg_lds + size_t(LG_ME) * words * 16);   // [TEAMS][4 waves][MR * ME]
  const int chunk = blockIdx.x % row_chunks, etile = blockIdx.x / row_chunks;
  const int e0 = etile * LG_ME;
  const int per_chunk = (rows + row_chunks - 1) / row_chunks;
  const int r_lo = chunk * per_chunk, r_hi = min(rows, r_lo + per_chunk);
  for (int v = tid; v < LG_ME * words; v += 256 * LG_TEAMS) {
    const int e = v / words, w = v - e * words;
    wl[v] = load16(router + size_t(min(e0 + e, experts - 1)) * hidden + size_t(w) * 8);
  }
  __syncthreads();
  for (int rb = r_lo; rb < r_hi; rb += LG_MR * LG_TEAMS) {  // uniform trip count over the block: the barriers below are block-wide
    const int r0 = rb + team * LG_MR;
    float acc[LG_MR * LG_ME];
#pragma unroll
    for (int j = 0; j < LG_MR * LG_ME; ++j) acc[j] = 0.0f;
    for (int i = 0; i < nvec; ++i) {
      const int v = t + 256 * i;
      if (v < words) {  // a chain that ends early skips the step: its lanes are switched off, its sums stay as they are
        float xf[LG_MR][8];
#pragma unroll
        for (int r = 0; r < LG_MR; ++r) {
          const int row = min(r0 + r, rows - 1);
          const u32x4 xv = load16(x + size_t(row) * hidden + size_t(v) * 8);
#pragma unroll
          for (int q = 0; q < 4; ++q) { xf[r][2 * q] = bf16lo(xv[q]); xf[r][2 * q + 1] = bf16hi(xv[q]); }
        }
#pragma unroll
        for (int e = 0; e < LG_ME; ++e) {
          const u32x4 wv = wl[e * words + v];
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            const float w0 = bf16lo(wv[q]), w1 = bf16hi(wv[q]);
#pragma unroll
            for (int r = 0; r < LG_MR; ++r) acc[r * LG_ME + e] = __fmaf_rn(xf[r][2 * q], w0, acc[r * LG_ME + e]);
#pragma unroll
            for (int r = 0; r < LG_MR; ++r) acc[r * LG_ME + e] = __fmaf_rn(xf[r][2 * q + 1], w1, acc[r * LG_ME + e]);
          }
        }
      }
    }
    // the adjacent-pair tree over the 256 chains: the 64 lanes of a wave (lane L ends with the sum of value bitrev6(L)),
    // then the team's four waves
    float* mine = part + (team * 4 + wave_in_team) * (LG_MR * LG_ME);
    static_assert(LG_MR * LG_ME == 64, "one value per lane");
    const float wsum = wave_reduce_scatter64(acc, lane);
    mine[bitrev6(lane)] = wsum;
    __syncthreads();
    if (t < LG_MR * LG_ME) {
      const int r = t / LG_ME, e = t - r * LG_ME;
      const float* pt = part + team * 4 * (LG_MR * LG_ME) + t;
      const float total = __fadd_rn(__fadd_rn(pt[0], pt[LG_MR * LG_ME]), __fadd_rn(pt[2 * LG_MR * LG_ME], pt[3 * LG_MR * LG_ME]));
      if (r0 + r < r_hi && e0 + e < experts) logits[size_t(r0 + r) * experts + e0 + e] = total;
    }
    __syncthreads();
  }
}

// ---------------------------------------------------------------------------------------------
// Selection by rank. The reference runs top_k rounds of a block-wide arg-max under (score desc, id asc)
// (kernels/moe_route.cu:205-235); that order is total, so the r-th pick is the candidate with exactly r
// candidates ahead of it. Every thread counts the candidates ahead of its own in one pass over LDS.
// s_key[e] = selection score of expert e, -inf for experts that cannot be picked; padded to a multiple of 4.
__device__ __forceinline__ int rank_of(const float* s_key, int padded, float mine, int e) {
  int rank = 0;
#pragma unroll 8
  for (int i = 0; i < padded; i += 4) {  // unrolled so that several LDS reads are in flight; one per trip is latency-bound
    const float4 v = *reinterpret_cast<const float4*>(s_key + i);
    rank += (v.x > mine || (v.x == mine && i + 0 < e)) ? 1 : 0;
    rank += (v.y > mine || (v.y == mine && i + 1 < e)) ? 1 : 0;
    rank += (v.z > mine || (v.z == mine && i + 2 < e)) ? 1 : 0;
    rank += (v.w > mine || (v.w == mine && i + 3 < e)) ? 1 : 0;
  }
  return rank;
}

// Softmax / sigmoid top-k over BF16 logits (kernels/moe_route.cu:154-301). One block per row, thread e
// owns expert e. The softmax denominator is summed exactly as the reference's 32-lane warp trees.
__global__ void k_route_topk(const uint16_t* __restrict__ logits, int* __restrict__ ids, uint16_t* __restrict__ weights,
                             int experts, int top_k, int score_mode) {
  __shared__ float s_red[32];
  __shared__ float s_v[16];
  __shared__ float s_sel[FFMOE_MAX_TOP_K];
  __shared__ int s_selid[FFMOE_MAX_TOP_K];
  __shared__ __align__(16) float s_key[FFMOE_MAX_EXPERTS];
  const int tid = threadIdx.x, row = blockIdx.x;
  const int e = tid;
  const bool live = e < experts;
  const int nwaves = blockDim.x >> 6;
  const int nw32 = blockDim.x >> 5;  // 32-lane groups, the reference's warps
  const float logit = live ? bf16_to_f32(logits[size_t(row) * experts + e]) : -INFINITY;
  float score;
  if (score_mode == FFMOE_SCORE_SOFTMAX) {
    float m = wave_max(logit);
    if ((tid & 63) == 0) s_v[tid >> 6] = m;
    __syncthreads();
    for (int w = 0; w < nwaves; ++w) m = fmaxf(m, s_v[w]);
    __syncthreads();
    const float ev = live ? det_expf(__fsub_rn(logit, m)) : 0.0f;
    float v = ev;
#pragma unroll
    for (int off = 16; off > 0; off >>= 1) {
      const float o = __shfl_down(v, off, 32);
      v = __fadd_rn(v, ((tid & 31) + off < 32) ? o : 0.0f);
    }
    if (tid < 32) s_red[tid] = 0.0f;
    __syncthreads();
    if ((tid & 31) == 0) s_red[tid >> 5] = v;
    __syncthreads();
    if (tid < 32) {
      v = tid < nw32 ? s_red[tid] : 0.0f;
#pragma unroll
      for (int off = 16; off > 0; off >>= 1) {
        const float o = __shfl_down(v, off, 32);
        v = __fadd_rn(v, (tid + off < 32) ? o : 0.0f);
      }
      if (tid == 0) s_red[0] = v;
    }
    __syncthreads();
    score = live ? __fdiv_rn(ev, s_red[0]) : -INFINITY;
  } else {
    score = live ? sigmoid1(logit) : -INFINITY;
  }
  s_key[tid] = score;  // blockDim is a multiple of 64 covering every expert
  __syncthreads();
  if (live) {
    const int rank = rank_of(s_key, blockDim.x, score, e);
    if (rank < top_k) { s_sel[rank] = score; s_selid[rank] = e; }
  }
  __syncthreads();
  if (tid < top_k) {
    float tsum = 0.0f;
    for (int r = 0; r < top_k; ++r) tsum = __fadd_rn(tsum, s_sel[r]);
    const float den = score_mode == FFMOE_SCORE_SOFTMAX ? tsum : __fadd_rn(tsum, 1.0e-20f);
    ids[size_t(row) * top_k + tid] = s_selid[tid];
    weights[size_t(row) * top_k + tid] = f32_to_bf16(__fdiv_rn(s_sel[tid], den));
  }
}

// noaux_tc selection over FP32 logits (kernels/moe_route.cu:315-390), with the optional group filter.
__global__ void k_route_topk_noaux(const float* __restrict__ logits, const float* __restrict__ bias, int bias_row_stride,
                                   int* __restrict__ ids, void* __restrict__ weights, int weights_f32, int experts,
                                   int top_k, int score_mode, float routed_scaling, int n_group, int topk_group) {
  __shared__ float s_sel[FFMOE_MAX_TOP_K];
  __shared__ int s_selid[FFMOE_MAX_TOP_K];
  __shared__ __align__(16) float s_key[FFMOE_MAX_EXPERTS];
  __shared__ float s_top[2 * FFMOE_MAX_EXPERTS / 2];
  __shared__ __align__(16) float s_group[FFMOE_MAX_EXPERTS / 2 + 4];
  const int tid = threadIdx.x, row = blockIdx.x;
  const int e = tid;
  const bool live = e < experts;
  float score = -1.0f, select = -INFINITY;
  if (live) {
    const float l = logits[size_t(row) * experts + e];
    if (score_mode == FFMOE_NOAUX_SIGMOID) {
      score = sigmoid1(l);
    } else {
      const float softplus = __fadd_rn(fmaxf(l, 0.0f), det_log1pf_unit(det_expf(-fabsf(l))));
      score = __builtin_sqrtf(softplus);  // correctly rounded (hipcc default); __fsqrt_rn is the approximate native sqrt
    }
    select = __fadd_rn(score, bias ? bias[size_t(row) * bias_row_stride + e] : 0.0f);
  }
  s_key[tid] = select;
  __syncthreads();
  bool allowed = live;
  if (n_group > 1) {
    // the two largest selection scores of every group, by rank inside the group
    const int per = experts / n_group;
    const int g = live ? e / per : 0;
    if (live) {
      int rank = 0;
#pragma unroll 8
      for (int i = g * per; i < (g + 1) * per; ++i) {
        const float v = s_key[i];
        rank += (v > select || (v == select && i < e)) ? 1 : 0;
      }
      if (rank < 2) s_top[2 * g + rank] = select;
    }
    __syncthreads();
    const int gpad = (n_group + 3) & ~3;
    if (tid < gpad) s_group[tid] = tid < n_group ? __fadd_rn(s_top[2 * tid], s_top[2 * tid + 1]) : -INFINITY;
    __syncthreads();
    if (live) allowed = rank_of(s_group, gpad, s_group[g], g) < topk_group;
    __syncthreads();
    s_key[tid] = allowed ? select : -INFINITY;
    __syncthreads();
  }
  if (allowed) {
    const int rank = rank_of(s_key, blockDim.x, select, e);
    if (rank < top_k) { s_sel[rank] = score; s_selid[rank] = e; }
  }
  __syncthreads();
  if (tid < top_k) {
    float tsum = 0.0f;
    for (int r = 0; r < top_k; ++r) tsum = __fadd_rn(tsum, s_sel[r]);
    const float w = __fmul_rn(__fdiv_rn(s_sel[tid], __fadd_rn(tsum, 1.0e-20f)), routed_scaling);
    ids[size_t(row) * top_k + tid] = s_selid[tid];
    if (weights_f32) reinterpret_cast<float*>(weights)[size_t(row) * top_k + tid] = w;
    else reinterpret_cast<uint16_t*>(weights)[size_t(row) * top_k + tid] = f32_to_bf16(w);
  }
}

__global__ void k_fill_u32(uint32_t* p, uint32_t v, long long n) {
  const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) p[i] = v;
}

// Host-side test for the register path: experts in {64,128,256,512,1024}; groups must tile the lanes.
static bool wave_select_ok(int experts, int n_group) {
  if (experts != 64 && experts != 128 && experts != 256 && experts != 512 && experts != 1024) return false;
  if (n_group == 1) return true;
  const int c = experts / 64, per = experts / n_group;
  if (per % c) return false;
  const int span = per / c;
  return span >= 1 && span <= 64 && (span & (span - 1)) == 0;
}

// noaux selection, one wave per row (register path).
__global__ __launch_bounds__(64) void k_route_topk_noaux_wave(const float* __restrict__ logits, const float* __restrict__ bias,
                                                              int bias_row_stride, int* __restrict__ ids, void* __restrict__ weights,
                                                              int weights_f32, uint32_t* __restrict__ done, int experts, int top_k,
                                                              int score_mode, float routed_scaling, int n_group, int topk_group) {
  const int row = blockIdx.x, lane = threadIdx.x;
  if (done && lane < top_k) done[size_t(row) * top_k + lane] = 0u;  // the contribution of this row starts from a clean slate
  void* wrow = weights_f32 ? (void*)(reinterpret_cast<float*>(weights) + size_t(row) * top_k)
                           : (void*)(reinterpret_cast<uint16_t*>(weights) + size_t(row) * top_k);
  const float* brow = bias ? bias + size_t(row) * bias_row_stride : nullptr;
  // the usual router (256 experts in 8 groups of which 4 stay, sigmoid scores, 8 picks) with its numbers as literals: two
  // thirds of the general selection's instructions, the same ids and weights
  if (experts == 256 && top_k == 8 && n_group == 8 && topk_group == 4 && score_mode == FFMOE_NOAUX_SIGMOID)
    wave_route_row<4>(logits + size_t(row) * 256, brow, lane, 256, 8, FFMOE_NOAUX_SIGMOID, routed_scaling, 8, 4, ids + size_t(row) * 8, wrow, weights_f32);
  else
    wave_route_dispatch(logits + size_t(row) * experts, brow, lane, experts, top_k, score_mode, routed_scaling, n_group, topk_group,
                        ids + size_t(row) * top_k, wrow, weights_f32);
}

}  // namespace ffmoe

using namespace ffmoe;

static int decode_cus() {
  static int cus = 0;
  if (cus == 0) {
    int dev = 0, n = 0;
    cus = (hipGetDevice(&dev) == hipSuccess && hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && n > 0) ? n : 256;
  }
  return cus;
}

static int check_route_dims(int rows, int experts, int hidden) {
  FF_REQUIRE(rows >= 1 && experts >= 1 && experts <= FFMOE_MAX_EXPERTS, FFMOE_ERR_SHAPE,
             "router rows=%d experts=%d outside [1, %d]", rows, experts, FFMOE_MAX_EXPERTS);
  FF_REQUIRE(hidden >= 8 && (hidden & 7) == 0, FFMOE_ERR_SHAPE, "router hidden=%d must be a positive multiple of 8", hidden);
  return 0;
}

extern "C" __attribute__((visibility("default"))) int ffmoe_route_logits_bf16(const void* x, const void* router, void* logits, int rows, int experts, int hidden,
                                       void* stream) {
  FF_TRY(check_route_dims(rows, experts, hidden));
  FF_PTR16(x); FF_PTR16(router); FF_PTR16(logits);
  FF_NO_OVERLAP(logits, size_t(rows) * experts * 2, x, size_t(rows) * hidden * 2);
  FF_NO_OVERLAP(logits, size_t(rows) * experts * 2, router, size_t(experts) * hidden * 2);
  hipLaunchKernelGGL(k_route_logits_bf16<false>, dim3((experts + 63) / 64, rows), dim3(320), 0, (hipStream_t)stream,
                     (const uint16_t*)x, (const uint16_t*)router, (uint16_t*)logits, rows, experts, hidden, (int*)nullptr, (uint16_t*)nullptr, 0, 0);
  return ff_launch_status();
}

extern "C" __attribute__((visibility("default"))) int ffmoe_route_logits_f32(const void* x, const void* router, float* logits, int rows, int experts, int hidden,
                                      void* stream) {
  FF_TRY(check_route_dims(rows, experts, hidden));
  FF_PTR16(x); FF_PTR16(router); FF_PTR4(logits);
  FF_NO_OVERLAP(logits, size_t(rows) * experts * 4, x, size_t(rows) * hidden * 2);
  FF_NO_OVERLAP(logits, size_t(rows) * experts * 4, router, size_t(experts) * hidden * 2);
  // Many rows: the kernel that keeps a tile of router rows in LDS (from FFMOE_ROUTE_LOGITS_TILE_ROWS rows on, default 96 - 15.8 against 18.4 us there at 256 x 7168, 13.2 against 15.5 us at 64 rows;
  // 0 = never), when the tile and the partial sums fit. Same bits either way.
  {
    static const int tile_rows = [] { const char* e = getenv("FFMOE_ROUTE_LOGITS_TILE_ROWS"); return e ? atoi(e) : 96; }();
    const size_t lds = size_t(LG_ME) * hidden * 2 + size_t(LG_TEAMS) * 4 * LG_MR * LG_ME * 4;
    if (tile_rows > 0 && rows >= tile_rows && lds <= 150 * 1024) {
      static int lds_ok = -1;
      if (lds_ok < 0)
        lds_ok = hipFuncSetAttribute(reinterpret_cast<const void*>(k_route_logits_f32_rows), hipFuncAttributeMaxDynamicSharedMemorySize, 150 * 1024) == hipSuccess ? 1 : 0;
      if (lds_ok == 1) {
        const int etiles = (experts + LG_ME - 1) / LG_ME;
        // a block takes LG_MR * LG_TEAMS rows per pass and one block fits a CU: as many row chunks as keep the grid within
        // one round of blocks, eight (one per XCD) for a cohort
        const int per_pass = LG_MR * LG_TEAMS;
        const int max_chunks = std::max(1, decode_cus() / etiles);
        const int row_chunks = std::max(1, std::min(max_chunks, (rows + per_pass - 1) / per_pass));
        hipLaunchKernelGGL(k_route_logits_f32_rows, dim3(unsigned(etiles) * unsigned(row_chunks)), dim3(256 * LG_TEAMS), lds, (hipStream_t)stream,
                           (const uint16_t*)x, (const uint16_t*)router, logits, rows, experts, hidden, row_chunks);
        return ff_launch_status();
      }
    }
  }
  FF_REQUIRE((rows + LOGIT_ROWS - 1) / LOGIT_ROWS <= 65535, FFMOE_ERR_SHAPE, "too many rows (%d) for one logits launch", rows);
  hipLaunchKernelGGL(k_route_logits_f32, dim3(experts, (rows + LOGIT_ROWS - 1) / LOGIT_ROWS), dim3(256), 0, (hipStream_t)stream,
                     (const uint16_t*)x, (const uint16_t*)router, logits, rows, experts, hidden);
  return ff_launch_status();
}

static int check_topk_dims(int rows, int experts, int top_k, bool allow_all) {
  FF_REQUIRE(rows >= 1 && experts >= 1 && experts <= FFMOE_MAX_EXPERTS, FFMOE_ERR_SHAPE,
             "router rows=%d experts=%d outside [1, %d]", rows, experts, FFMOE_MAX_EXPERTS);
  FF_REQUIRE(top_k >= 1 && top_k <= FFMOE_MAX_TOP_K && (allow_all ? top_k <= experts : top_k < experts), FFMOE_ERR_SHAPE,
             "top_k=%d outside [1, %d] or not below experts=%d", top_k, FFMOE_MAX_TOP_K, experts);
  return 0;
}

extern "C" __attribute__((visibility("default"))) int ffmoe_route_topk(const void* logits, int* ids, void* weights, int rows, int experts, int top_k, int score,
                                void* stream) {
  FF_TRY(check_topk_dims(rows, experts, top_k, false));
  FF_REQUIRE(score == FFMOE_SCORE_SOFTMAX || score == FFMOE_SCORE_SIGMOID, FFMOE_ERR_UNSUPPORTED, "unknown router score %d", score);
  FF_PTR16(logits); FF_PTR4(ids); FF_PTR2(weights);
  FF_NO_OVERLAP(ids, size_t(rows) * top_k * 4, logits, size_t(rows) * experts * 2);
  FF_NO_OVERLAP(weights, size_t(rows) * top_k * 2, logits, size_t(rows) * experts * 2);
  FF_NO_OVERLAP(ids, size_t(rows) * top_k * 4, weights, size_t(rows) * top_k * 2);
  const int threads = (experts + 63) & ~63;
  hipLaunchKernelGGL(k_route_topk, dim3(rows), dim3(threads), 0, (hipStream_t)stream, (const uint16_t*)logits, ids,
                     (uint16_t*)weights, experts, top_k, score);
  return ff_launch_status();
}

extern "C" __attribute__((visibility("default"))) int ffmoe_route_topk_noaux(const float* logits, const float* bias, int bias_row_stride, int* ids, void* weights,
                                      int weights_f32, int rows, int experts, int top_k, int score_mode,
                                      float routed_scaling, int n_group, int topk_group, void* stream) {
  FF_TRY(check_topk_dims(rows, experts, top_k, true));
  FF_REQUIRE(score_mode == 0 || score_mode == 1, FFMOE_ERR_UNSUPPORTED, "unknown noaux score mode %d", score_mode);
  FF_REQUIRE(routed_scaling > 0.0f && routed_scaling < INFINITY, FFMOE_ERR_SHAPE, "invalid routed scaling %g", (double)routed_scaling);
  FF_REQUIRE(bias_row_stride == 0 || bias_row_stride == experts, FFMOE_ERR_SHAPE, "bias row stride %d must be 0 or experts", bias_row_stride);
  FF_REQUIRE(n_group >= 1 && topk_group >= 1 && topk_group <= n_group && experts % n_group == 0, FFMOE_ERR_SHAPE,
             "invalid grouping n_group=%d topk_group=%d experts=%d", n_group, topk_group, experts);
  FF_REQUIRE(n_group == 1 || (experts / n_group >= 2 && top_k <= topk_group * (experts / n_group)), FFMOE_ERR_SHAPE,
             "groups of %d experts cannot supply top_k=%d from %d groups", experts / n_group, top_k, topk_group);
  FF_PTR4(logits); FF_PTR4(ids);
  if (bias) FF_PTR4(bias);
  if (weights_f32) { FF_PTR4(weights); } else { FF_PTR2(weights); }
  const size_t wbytes = size_t(rows) * top_k * (weights_f32 ? 4 : 2);
  FF_NO_OVERLAP(ids, size_t(rows) * top_k * 4, logits, size_t(rows) * experts * 4);
  FF_NO_OVERLAP(weights, wbytes, logits, size_t(rows) * experts * 4);
  FF_NO_OVERLAP(ids, size_t(rows) * top_k * 4, weights, wbytes);
  if (wave_select_ok(experts, n_group)) {
    hipLaunchKernelGGL(k_route_topk_noaux_wave, dim3(rows), dim3(64), 0, (hipStream_t)stream, logits, bias, bias_row_stride, ids,
                       weights, weights_f32, (uint32_t*)nullptr, experts, top_k, score_mode, routed_scaling, n_group, topk_group);
    return ff_launch_status();
  }
  const int threads = (experts + 63) & ~63;
  hipLaunchKernelGGL(k_route_topk_noaux, dim3(rows), dim3(threads), 0, (hipStream_t)stream, logits, bias, bias_row_stride,
                     ids, weights, weights_f32, experts, top_k, score_mode, routed_scaling, n_group, topk_group);
  return ff_launch_status();
}

extern "C" __attribute__((visibility("default"))) int ffmoe_route_decode(const void* x, const void* router, void* logits, int* ids, void* weights, int rows,
                                  int experts, int hidden, int top_k, int score, void* stream) {
  FF_TRY(check_topk_dims(rows, experts, top_k, false));
  // up to 64 experts the wave that runs a row's chains holds all its logits and selects right away: one launch
  // (FFMOE_ROUTE_FUSED=0: the two launches; same bits)
  static const bool fused = [] { const char* e = getenv("FFMOE_ROUTE_FUSED"); return !(e && atoi(e) == 0); }();
  if (fused && experts <= 64) {
    FF_TRY(check_route_dims(rows, experts, hidden));
    FF_REQUIRE(score == FFMOE_SCORE_SOFTMAX || score == FFMOE_SCORE_SIGMOID, FFMOE_ERR_UNSUPPORTED, "unknown router score %d", score);
    FF_PTR16(x); FF_PTR16(router); FF_PTR16(logits); FF_PTR4(ids); FF_PTR2(weights);
    FF_NO_OVERLAP(logits, size_t(rows) * experts * 2, x, size_t(rows) * hidden * 2);
    FF_NO_OVERLAP(logits, size_t(rows) * experts * 2, router, size_t(experts) * hidden * 2);
    FF_NO_OVERLAP(ids, size_t(rows) * top_k * 4, logits, size_t(rows) * experts * 2);
    FF_NO_OVERLAP(weights, size_t(rows) * top_k * 2, logits, size_t(rows) * experts * 2);
    FF_NO_OVERLAP(ids, size_t(rows) * top_k * 4, weights, size_t(rows) * top_k * 2);
    FF_NO_OVERLAP(ids, size_t(rows) * top_k * 4, x, size_t(rows) * hidden * 2);
    FF_NO_OVERLAP(weights, size_t(rows) * top_k * 2, x, size_t(rows) * hidden * 2);
    hipLaunchKernelGGL(k_route_logits_bf16<true>, dim3(1, rows), dim3(320), 0, (hipStream_t)stream, (const uint16_t*)x, (const uint16_t*)router,
                       (uint16_t*)logits, rows, experts, hidden, ids, (uint16_t*)weights, top_k, score);
    return ff_launch_status();
  }
  int rc = ffmoe_route_logits_bf16(x, router, logits, rows, experts, hidden, stream);
  if (rc) return rc;
  return ffmoe_route_topk(logits, ids, weights, rows, experts, top_k, score, stream);
}

extern "C" __attribute__((visibility("default"))) int ffmoe_route_noaux_decode(const void* x, const void* router, const float* bias, int bias_row_stride, float* logits, int* ids,
                                        void* weights, int weights_f32, uint32_t* done, int rows, int experts, int hidden,
                                        int top_k, int score_mode, float routed_scaling, int n_group, int topk_group,
                                        void* stream) {
  FF_TRY(ffmoe_route_logits_f32(x, router, logits, rows, experts, hidden, stream));
  if (done) FF_PTR4(done);
  if (wave_select_ok(experts, n_group)) {
    // same checks as ffmoe_route_topk_noaux, then the register-path kernel, which also clears `done`
    FF_TRY(check_topk_dims(rows, experts, top_k, true));
    FF_REQUIRE(score_mode == 0 || score_mode == 1, FFMOE_ERR_UNSUPPORTED, "unknown noaux score mode %d", score_mode);
    FF_REQUIRE(routed_scaling > 0.0f && routed_scaling < INFINITY, FFMOE_ERR_SHAPE, "invalid routed scaling %g", (double)routed_scaling);
    FF_REQUIRE(bias_row_stride == 0 || bias_row_stride == experts, FFMOE_ERR_SHAPE, "bias row stride %d must be 0 or experts", bias_row_stride);
    FF_REQUIRE(topk_group >= 1 && topk_group <= n_group && top_k <= topk_group * (experts / n_group), FFMOE_ERR_SHAPE,
               "invalid grouping n_group=%d topk_group=%d top_k=%d", n_group, topk_group, top_k);
    FF_PTR4(ids);
    if (bias) FF_PTR4(bias);
    if (weights_f32) { FF_PTR4(weights); } else { FF_PTR2(weights); }
    const size_t wbytes = size_t(rows) * top_k * (weights_f32 ? 4 : 2), lbytes = size_t(rows) * experts * 4;
    FF_NO_OVERLAP(ids, size_t(rows) * top_k * 4, logits, lbytes);
    FF_NO_OVERLAP(weights, wbytes, logits, lbytes);
    FF_NO_OVERLAP(ids, size_t(rows) * top_k * 4, weights, wbytes);
    hipLaunchKernelGGL(k_route_topk_noaux_wave, dim3(rows), dim3(64), 0, (hipStream_t)stream, logits, bias, bias_row_stride, ids,
                       weights, weights_f32, done, experts, top_k, score_mode, routed_scaling, n_group, topk_group);
    return ff_launch_status();
  }
  if (done) {  // a fill kernel, not a memset node: callers may capture this call into a HIP graph
    const long long n = (long long)rows * top_k;
    hipLaunchKernelGGL(k_fill_u32, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, (hipStream_t)stream, done, 0u, n);
    FF_TRY(ff_launch_status());
  }
  return ffmoe_route_topk_noaux(logits, bias, bias_row_stride, ids, weights, weights_f32, rows, experts, top_k, score_mode,
                                routed_scaling, n_group, topk_group, stream);
}

// ---------------------------------------------------------------------------------------------
// expert residency protocol
namespace ffmoe {
__global__ void k_slot_publish(uint64_t* slots, uint32_t* valid, uint64_t* generation, int incoming, int victim,
                               uint64_t s0, uint64_t s1, uint64_t s2, uint64_t s3, uint64_t s4, uint64_t s5, uint64_t epoch, uint32_t* status) {
  if (blockIdx.x != 0 || threadIdx.x != 0) return;
  if (valid[incoming] == 1u && generation[incoming] >= epoch) {  // an epoch must move forward
    if (status) atomicOr(status, 1u);
    return;
  }
  if (victim >= 0) {
    valid[victim] = 0u;
    generation[victim] = 0;
    for (int i = 0; i < 6; ++i) slots[size_t(victim) * 6 + i] = 0;
  }
  const uint64_t in[6] = {s0, s1, s2, s3, s4, s5};
  for (int i = 0; i < 6; ++i) slots[size_t(incoming) * 6 + i] = in[i];
  generation[incoming] = epoch;
  valid[incoming] = 1u;
}

__global__ __launch_bounds__(256) void k_route_mask(const int* __restrict__ ids, const uint32_t* __restrict__ valid,
                                                    const uint64_t* __restrict__ generation, uint32_t* __restrict__ active,
                                                    uint64_t* __restrict__ assignment_gen, uint32_t* __restrict__ status, int assignments, int experts) {
  const int a = blockIdx.x * 256 + threadIdx.x;
  if (a >= assignments) return;
  const int e = ids[a];
  if ((unsigned)e >= (unsigned)experts || valid[e] > 1u || (valid[e] == 1u && generation[e] == 0)) {
    if (status) atomicOr(status, 1u);
    active[a] = 0u;
    assignment_gen[a] = 0;
    return;
  }
  active[a] = valid[e];
  assignment_gen[a] = valid[e] ? generation[e] : 0;
}
}  // namespace ffmoe

extern "C" __attribute__((visibility("default"))) int ffmoe_slot_publish(uint64_t* slots, uint32_t* valid, uint64_t* generation, int experts, int incoming,
                                                                        int victim, const uint64_t incoming_slot[6], uint64_t epoch, uint32_t* status,
                                                                        void* stream) {
  FF_PTR16(slots); FF_PTR4(valid); FF_PTR_ALIGNED(generation, 8);
  FF_REQUIRE(incoming_slot != nullptr, FFMOE_ERR_NULL, "incoming_slot is NULL");
  FF_REQUIRE(experts >= 1 && experts <= FFMOE_MAX_EXPERTS && incoming >= 0 && incoming < experts && victim >= -1 && victim < experts && victim != incoming,
             FFMOE_ERR_SHAPE, "slot_publish experts=%d incoming=%d victim=%d", experts, incoming, victim);
  FF_REQUIRE(epoch != 0, FFMOE_ERR_SHAPE, "slot_publish epoch must not be 0");
  for (int i = 0; i < 6; i += 2)
    FF_REQUIRE(incoming_slot[i] != 0 && incoming_slot[i] % 16 == 0, FFMOE_ERR_ALIGN, "incoming_slot[%d] is NULL or misaligned", i);
  if (status) FF_PTR4(status);
  hipLaunchKernelGGL(ffmoe::k_slot_publish, dim3(1), dim3(1), 0, (hipStream_t)stream, slots, valid, generation, incoming, victim, incoming_slot[0],
                     incoming_slot[1], incoming_slot[2], incoming_slot[3], incoming_slot[4], incoming_slot[5], epoch, status);
  return ffmoe::ff_launch_status();
}

extern "C" __attribute__((visibility("default"))) int ffmoe_route_mask(const int* ids, const uint32_t* valid, const uint64_t* generation, uint32_t* active,
                                                                      uint64_t* assignment_gen, uint32_t* status, int assignments, int experts, void* stream) {
  FF_PTR4(ids); FF_PTR4(valid); FF_PTR_ALIGNED(generation, 8); FF_PTR4(active); FF_PTR_ALIGNED(assignment_gen, 8);
  FF_REQUIRE(assignments >= 1 && experts >= 1 && experts <= FFMOE_MAX_EXPERTS, FFMOE_ERR_SHAPE, "route_mask assignments=%d experts=%d", assignments, experts);
  if (status) FF_PTR4(status);
  FF_NO_OVERLAP(active, size_t(assignments) * 4, ids, size_t(assignments) * 4);
  hipLaunchKernelGGL(ffmoe::k_route_mask, dim3((assignments + 255) / 256), dim3(256), 0, (hipStream_t)stream, ids, valid, generation, active,
                     assignment_gen, status, assignments, experts);
  return ffmoe::ff_launch_status();
}
