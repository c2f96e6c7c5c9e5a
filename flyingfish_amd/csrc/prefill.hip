// Prefill path: device-side grouping of (row, choice) assignments by expert, then the two grouped W8A8 GEMMs on the
// FP8 matrix cores (gate/up + SwiGLU, down x routing weight scattered to contributions), and the standalone W8A8
// block linear that shares the GEMM kernel.
//
// Reference shape of the pipeline: kernels/moe_prefill.cu:364-553 (count / scan / permute / grouped GEMM / scatter),
// src/backend/cuda/moe/prefill.rs:1053-1408 (host orchestration). The reference reads the counts back to the host
// between scan and GEMM (prefill.rs:1146-1147); here grids are sized from upper bounds and every kernel reads the
// device-side totals, so the call enqueues without a host synchronisation.
// Arithmetic: the reference's block-F32 W8A8 path (kernels/fp8_linear.cu:12-48, kernels/q38_contract.cuh:239-279,
// kernels/act.cu:125-159, kernels/moe_ffn.cu:870-908) applied per assignment, so results do not depend on which
// other rows share an expert.
#include "w8a8_gemm.cuh"
#include "w16_gemm.cuh"
#include "mx_gemm.cuh"
#include "dense_splitk.cuh"
#include "api.h"
#include <algorithm>
#include <cstdlib>

namespace ffmoe {

struct PrefillBook {
  uint32_t* counts;   // [E]
  uint32_t* offsets;  // [E + 1]
  uint32_t* gbase;    // [E + 1] first group of each expert
  uint32_t* totals;   // [0] units of the gate/up GEMM, [1] units of the down GEMM, [2] groups, [3] active assignments
  int* perm;          // [A]
  GemmGroup* groups;
  u32x2* units0;
  u32x2* units1;
};

__global__ void k_prefill_zero(uint32_t* counts, int experts, uint32_t* totals) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < experts) counts[i] = 0u;
  if (i < 4) totals[i] = 0u;
}

struct LiveTest { const int* ids; const uint32_t* active; const uint32_t* valid; const uint64_t* generation; const uint64_t* assignment_gen; int experts; };
__device__ __forceinline__ bool assignment_live(const LiveTest& t, long long a, int& e) {
  e = t.ids[a];
  if ((unsigned)e >= (unsigned)t.experts) return false;
  if (t.active && t.active[a] == 0u) return false;
  if (t.valid && t.valid[e] == 0u) return false;
  if (t.generation && t.assignment_gen && t.generation[e] != t.assignment_gen[a]) return false;  // stale choice
  return true;
}

// histogram of live assignments per expert (kernels/moe_prefill.cu:364-420): per block in LDS over 1024 assignments, then
// one global add per expert the block has seen (a global add per assignment serializes on the popular experts' counters)
constexpr int FFMOE_COUNT_PER_BLOCK = 1024;
__global__ __launch_bounds__(256) void k_prefill_count(const LiveTest t, uint32_t* __restrict__ counts, long long A) {
  __shared__ uint32_t s_hist[FFMOE_MAX_EXPERTS];
  for (int e = threadIdx.x; e < t.experts; e += 256) s_hist[e] = 0u;
  __syncthreads();
  const long long first = (long long)blockIdx.x * FFMOE_COUNT_PER_BLOCK;
#pragma unroll
  for (int i = 0; i < FFMOE_COUNT_PER_BLOCK / 256; ++i) {
    const long long a = first + i * 256 + threadIdx.x;
    int e;
    if (a < A && assignment_live(t, a, e)) atomicAdd(&s_hist[e], 1u);
  }
  __syncthreads();
  for (int e = threadIdx.x; e < t.experts; e += 256) {
    const uint32_t c = s_hist[e];
    if (c != 0u) atomicAdd(counts + e, c);
  }
}

// exclusive scans over experts (row offsets and group offsets), group descriptors and the two unit lists
// (kernels/moe_prefill.cu:421-472; unit order = expert, column tile, row group, so neighbours share weights)
// shared_rows > 0 appends the always-on expert as groups of expert id `experts` over rows 0 .. shared_rows - 1, their units
// behind the routed ones (column tile outermost, so the row groups of a tile are neighbours and share its weights in L2):
// the launches that run the routed experts then run the shared one as well.
struct PlanShared { uint32_t rows[1025], groups[1025], tmp[1024]; };

// unit u of a list with `tiles` column tiles per group -> (group, tile); s_groups = exclusive scan of the experts' group
// counts, G routed groups, GS groups of the riding shared expert behind them
__device__ __forceinline__ u32x2 plan_unit(const uint32_t* s_groups, int experts, uint32_t tiles, int rgb, int tgb, uint32_t G, uint32_t GS, uint32_t u) {
  if (u >= G * tiles) {
    const uint32_t v = u - G * tiles;
    return u32x2{G + v % GS, v / GS};
  }
  const uint32_t key = u / tiles;
  int lo = 0, hi = experts;  // last e with s_groups[e] <= key
  while (hi - lo > 1) { const int mid = (lo + hi) >> 1; if (s_groups[mid] <= key) lo = mid; else hi = mid; }
  // An expert's units run over blocks of rgb row groups, inside a row block over blocks of tgb column tiles, inside those
  // over the tiles, innermost over the row groups. The blocks of an XCD work on neighbouring units at the same time (64 of
  // them with two blocks per CU), so a window of rgb x tgb units fetches rgb token tiles and tgb weight tiles into that
  // XCD's L2 and shares each among tgb resp. rgb blocks.
  const uint32_t ge = s_groups[lo + 1] - s_groups[lo];
  const uint32_t v = u - s_groups[lo] * tiles;
  const uint32_t per = uint32_t(rgb) * tiles;
  const uint32_t j = min(v / per, (ge - 1u) / uint32_t(rgb));
  const uint32_t w = v - j * per;
  const uint32_t rb = min(uint32_t(rgb), ge - j * uint32_t(rgb));
  const uint32_t tg = min(uint32_t(tgb), tiles);
  const uint32_t per2 = rb * tg;
  const uint32_t q = min(w / per2, (tiles - 1u) / tg);
  const uint32_t w2 = w - q * per2;
  return u32x2{s_groups[lo] + j * uint32_t(rgb) + w2 % rb, q * tg + w2 / rb};
}

__device__ __forceinline__ void prefill_plan_body(PlanShared& sh, const PrefillBook& b, int experts, int tm, int tiles0, int tiles1, int rgb,
                                                  int tgb, int shared_rows, uint32_t c, bool with_units) {
  uint32_t* s_rows = sh.rows;
  uint32_t* s_groups = sh.groups;
  uint32_t* s_tmp = sh.tmp;
  const int tid = threadIdx.x;
  const uint32_t g = (c + tm - 1) / tm;
  // Inclusive scans of the row and group counts over the block's 1024 threads: inside each wave by six cross-lane steps,
  // then the sixteen wave totals by the first wave, two barriers for both scans (forty barrier pairs as a block-wide
  // Hillis-Steele scan, which was most of this block's time)
  uint32_t vr = c, vg = g;
  const int lane = tid & 63, wv = tid >> 6;
#pragma unroll
  for (int off = 1; off < 64; off <<= 1) {
    const uint32_t ar = uint32_t(__builtin_amdgcn_ds_bpermute(((lane - off) & 63) << 2, int(vr)));
    const uint32_t ag = uint32_t(__builtin_amdgcn_ds_bpermute(((lane - off) & 63) << 2, int(vg)));
    if (lane >= off) { vr += ar; vg += ag; }
  }
  if (lane == 63) { s_tmp[wv] = vr; s_tmp[16 + wv] = vg; }
  __syncthreads();
  if (wv == 0) {
    uint32_t tr = lane < 16 ? s_tmp[lane] : 0u, tg = lane < 16 ? s_tmp[16 + lane] : 0u;
#pragma unroll
    for (int off = 1; off < 16; off <<= 1) {
      const uint32_t ar = uint32_t(__builtin_amdgcn_ds_bpermute(((lane - off) & 63) << 2, int(tr)));
      const uint32_t ag = uint32_t(__builtin_amdgcn_ds_bpermute(((lane - off) & 63) << 2, int(tg)));
      if (lane >= off) { tr += ar; tg += ag; }
    }
    if (lane < 16) { s_tmp[32 + lane] = tr; s_tmp[48 + lane] = tg; }  // inclusive totals of waves 0 .. lane
  }
  __syncthreads();
  if (wv > 0) { vr += s_tmp[32 + wv - 1]; vg += s_tmp[48 + wv - 1]; }
  s_rows[tid + 1] = vr; s_groups[tid + 1] = vg;
  if (tid == 0) { s_rows[0] = 0u; s_groups[0] = 0u; }
  __syncthreads();
  if (tid < experts) { b.offsets[tid] = s_rows[tid]; b.gbase[tid] = s_groups[tid]; }
  if (tid == 0) { b.offsets[experts] = s_rows[experts]; b.gbase[experts] = s_groups[experts]; }
  const uint32_t G = s_groups[experts];
  const uint32_t GS = shared_rows > 0 ? uint32_t((shared_rows + tm - 1) / tm) : 0u;
  if (tid == 0) { b.totals[0] = (G + GS) * tiles0; b.totals[1] = (G + GS) * tiles1; b.totals[2] = G; b.totals[3] = s_rows[experts]; }
  for (uint32_t q = tid; q < GS; q += 1024) {
    GemmGroup gd;
    gd.expert = experts; gd.start = int(q) * tm; gd.n = min(tm, shared_rows - int(q) * tm); gd.pad = 0;
    b.groups[G + q] = gd;
  }
  // group descriptors
  for (uint32_t q = tid; q < G; q += 1024) {
    int lo = 0, hi = experts;  // last e with s_groups[e] <= q
    while (hi - lo > 1) { const int mid = (lo + hi) >> 1; if (s_groups[mid] <= q) lo = mid; else hi = mid; }
    const uint32_t i = q - s_groups[lo];
    const uint32_t cnt = s_rows[lo + 1] - s_rows[lo];
    GemmGroup gd;
    gd.expert = lo; gd.start = int(s_rows[lo] + i * tm); gd.n = int(min(uint32_t(tm), cnt - i * tm)); gd.pad = 0;
    b.groups[q] = gd;
  }
  // unit lists
  if (!with_units) return;
  for (int pass = 0; pass < 2; ++pass) {
    const uint32_t tiles = pass == 0 ? tiles0 : tiles1;
    u32x2* units = pass == 0 ? b.units0 : b.units1;
    for (uint32_t u = tid; u < (G + GS) * tiles; u += 1024) units[u] = plan_unit(s_groups, experts, tiles, rgb, tgb, G, GS, u);
  }
}

__global__ __launch_bounds__(1024) void k_prefill_plan(PrefillBook b, int experts, int tm, int tiles0, int tiles1, int rgb, int tgb, int shared_rows) {
  __shared__ PlanShared sh;
  prefill_plan_body(sh, b, experts, tm, tiles0, tiles1, rgb, tgb, shared_rows, int(threadIdx.x) < experts ? b.counts[threadIdx.x] : 0u, false);
}

// the two unit lists behind k_prefill_plan, one unit per thread over as many blocks as the lists can need (blocks past the
// device-side totals leave at once): tens of thousands of units are too many for the plan's single block
__global__ __launch_bounds__(256) void k_prefill_units(PrefillBook b, int experts, int tm, int tiles0, int tiles1, int rgb, int tgb, int shared_rows) {
  __shared__ uint32_t s_groups[1025];
  const uint32_t n0 = b.totals[0], n1 = b.totals[1];
  const uint32_t u = blockIdx.x * 256u + threadIdx.x;
  if (blockIdx.x * 256u >= n0 + n1) return;
  for (int e = threadIdx.x; e <= experts; e += 256) s_groups[e] = b.gbase[e];
  __syncthreads();
  if (u >= n0 + n1) return;
  const uint32_t G = s_groups[experts];
  const uint32_t GS = shared_rows > 0 ? uint32_t((shared_rows + tm - 1) / tm) : 0u;
  if (u < n0) b.units0[u] = plan_unit(s_groups, experts, uint32_t(tiles0), rgb, tgb, G, GS, u);
  else b.units1[u - n0] = plan_unit(s_groups, experts, uint32_t(tiles1), rgb, tgb, G, GS, u - n0);
}

// Small cohorts (at most FFMOE_BOOK_SMALL_MAX assignments, one per thread): count, plan and stable fill in ONE launch of one
// block, instead of four launches that each cost a launch more than they compute. The ids of the live assignments are kept
// in LDS; an assignment's place in its expert's segment is the number of earlier assignments of that expert.
constexpr int FFMOE_BOOK_SMALL_MAX = 1024;
__global__ __launch_bounds__(1024) void k_prefill_book_small(const LiveTest lt, PrefillBook b, int A, int experts, int tm, int tiles0, int tiles1,
                                                             int rgb, int tgb, int shared_rows, int with_units) {
  __shared__ PlanShared sh;
  __shared__ uint32_t s_cnt[1024];
  __shared__ __attribute__((aligned(16))) int s_id[FFMOE_BOOK_SMALL_MAX];
  const int tid = threadIdx.x;
  s_cnt[tid] = 0u;
  __syncthreads();
  int my = -1;  // thread a holds assignment a (A <= 1024 = the block)
  if (tid < A) {
    int id;
    if (assignment_live(lt, tid, id)) { my = id; atomicAdd(&s_cnt[id], 1u); }
  }
  s_id[tid] = my;
  __syncthreads();
  const uint32_t c = tid < experts ? s_cnt[tid] : 0u;
  if (tid < experts) b.counts[tid] = c;
  prefill_plan_body(sh, b, experts, tm, tiles0, tiles1, rgb, tgb, shared_rows, c, with_units != 0);
  // position inside the expert's segment = number of earlier assignments of the same expert; every thread walks the same
  // LDS words (broadcast reads), four at a time
  uint32_t rank = 0;
  const int upto = my >= 0 ? (tid + 3) & ~3 : 0;  // only earlier assignments count, and only live ones look
  for (int q = 0; q < upto; q += 4) {
    const int4 v = *reinterpret_cast<const int4*>(&s_id[q]);
    rank += uint32_t(v.x == my && q < tid) + uint32_t(v.y == my && q + 1 < tid) + uint32_t(v.z == my && q + 2 < tid) + uint32_t(v.w == my && q + 3 < tid);
  }
  if (my >= 0) b.perm[sh.rows[my] + rank] = tid;
}

// stable fill: block e lists its assignments in ascending assignment order (the reference permutes with an atomic
// cursor, kernels/moe_prefill.cu:475-510; per-row results make the order irrelevant, a fixed one keeps runs repeatable).
// Each of the four waves owns a contiguous quarter of the assignments: it counts its hits, the block exchanges the four
// counts once, and the wave walks its quarter again writing positions - no block-wide step per 256 assignments. The
// per-assignment words are all loaded unconditionally (independent, coalesced requests: one memory latency per 2048
// assignments of a wave), and while a quarter has at most 8192 assignments a lane keeps its 128 hit bits in registers, so
// the second walk reads nothing.
__global__ __launch_bounds__(256) void k_prefill_fill(const LiveTest lt, PrefillBook b, long long A) {
  __shared__ uint32_t s_wave[4];
  const int e = blockIdx.x;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const uint32_t cnt = b.counts[e];
  if (cnt == 0u) return;
  const bool gens = lt.generation && lt.assignment_gen;
  const uint64_t gen_e = gens ? lt.generation[e] : 0ull;
  const long long quarter = ((A + 255) / 256) * 64;  // a multiple of 64, four of them cover A
  const long long lo = quarter * wave, hi = lo + quarter < A ? lo + quarter : A;
  // 32 assignments of this lane starting at a0: bit j = assignment a0 + 64 j + lane is a live choice of expert e
  // (the conditions of assignment_live; the expert's valid flag is implied by its non-zero count)
  auto hits32 = [&](long long a0) {
    int id[32];
    uint32_t act[32];
    uint64_t ag[32];
#pragma unroll
    for (int j = 0; j < 32; ++j) {
      const long long a = a0 + 64 * j + lane;
      const bool in = a < hi;
      id[j] = in ? lt.ids[a] : -1;
      act[j] = (in && lt.active) ? lt.active[a] : 1u;
      ag[j] = (in && gens) ? lt.assignment_gen[a] : gen_e;
    }
    uint32_t bits = 0;
#pragma unroll
    for (int j = 0; j < 32; ++j) bits |= uint32_t(id[j] == e && act[j] != 0u && ag[j] == gen_e) << j;
    return bits;
  };
  const bool cached = quarter <= 8192;
  uint32_t keep[4] = {0u, 0u, 0u, 0u};
  uint32_t mine = 0;
  {
    int w = 0;
    for (long long a0 = lo; a0 < hi; a0 += 2048, ++w) {
      const uint32_t bits = hits32(a0);
      if (cached) {
#pragma unroll
        for (int q = 0; q < 4; ++q) keep[q] = w == q ? bits : keep[q];
      }
#pragma unroll
      for (int j = 0; j < 32; ++j) mine += __popcll(__ballot((bits >> j) & 1u));
    }
  }
  if (lane == 0) s_wave[wave] = mine;
  __syncthreads();
  uint32_t run = b.offsets[e];
  for (int w = 0; w < wave; ++w) run += s_wave[w];
  int w = 0;
  for (long long a0 = lo; a0 < hi; a0 += 2048, ++w) {
    uint32_t bits;
    if (cached) {
      bits = keep[0];
#pragma unroll
      for (int q = 1; q < 4; ++q) bits = w == q ? keep[q] : bits;
    } else {
      bits = hits32(a0);
    }
#pragma unroll
    for (int j = 0; j < 32; ++j) {
      const bool h = (bits >> j) & 1u;
      const uint64_t mask = __ballot(h);
      if (h) b.perm[run + __popcll(mask & ((uint64_t(1) << lane) - 1))] = int(a0 + 64 * j + lane);
      run += __popcll(mask);
    }
  }
}

// rows beyond the live count keep whatever the scratch held: quantize only live rows
__global__ __launch_bounds__(256) void k_quant_live(const uint16_t* __restrict__ x, uint8_t* __restrict__ codes, float* __restrict__ scales,
                                                    const uint32_t* __restrict__ live_rows, int k) {
  const int groups = k >> 7;
  const long long cell = (long long)blockIdx.x * 16 + (threadIdx.x >> 4);
  if (cell >= (long long)(*live_rows) * groups) return;
  const int sub = threadIdx.x & 15;
  const long long row = cell / groups;
  const int first = int(cell % groups) * 128 + sub * 8;
  float v[8];
  const u32x4 w = load16(x + row * k + first);
#pragma unroll
  for (int q = 0; q < 4; ++q) { v[2 * q] = bf16lo(w[q]); v[2 * q + 1] = bf16hi(w[q]); }
  float amax = 0.0f;
#pragma unroll
  for (int i = 0; i < 8; ++i) amax = fmaxf(amax, fabsf(v[i]));
#pragma unroll
  for (int off = 8; off > 0; off >>= 1) amax = fmaxf(amax, __shfl_xor(amax, off, 16));
  const float scale = __fmul_rn(amax, 1.0f / 448.0f);
  if (sub == 0) scales[cell] = scale;
  const float divisor = fmaxf(scale, 1.0e-12f);
  float q[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) q[i] = fminf(448.0f, fmaxf(-448.0f, __fdiv_rn(v[i], divisor)));
  const uint32_t out[2] = {e4m3x4_encode_finite(q[0], q[1], q[2], q[3]), e4m3x4_encode_finite(q[4], q[5], q[6], q[7])};
  const u32x2 o = {out[0], out[1]};
  *reinterpret_cast<u32x2*>(codes + row * k + first) = o;
}

}  // namespace ffmoe

using namespace ffmoe;

namespace {
int g_cus_p = 0;
int num_cus_p() {
  if (g_cus_p == 0) {
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) == hipSuccess && hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && n > 0)
      g_cus_p = n;
    else
      g_cus_p = 256;
  }
  return g_cus_p;
}

inline uint64_t up256(uint64_t v) { return (v + 255) & ~uint64_t(255); }

// rows per group for an average of `avg` rows per expert
// (cap: the largest group a path's kernels are built for, in units of 16 rows; anything else in the variable is ignored)
int pick_mf(double avg, int cap, bool w8a8 = false) {
  if (const char* f = getenv("FFMOE_PREFILL_MF")) {
    const int v = atoi(f);
    if (v == 1 || v == 2 || v == 4 || v == 8) return std::min(v, cap);
  }
  // W8A8: the 64-row kernel with eight waves per block is ahead at every cohort size measured (top-8 of 256 experts at
  // hidden 7168, 32 / 128 / 512 / 2048 tokens: 0.74 / 1.42 / 2.04 / 2.65 ms against 0.77 / 1.54 / 2.30 / 4.17 ms with 32-row
  // groups and 0.77 / 1.55 / 2.71 / 6.79 ms with 16-row groups). The W*A16 and MX kernels dequantize per row group
  // and keep the short groups for short segments (64 rows, 16-row groups: 1.89 ms, 64-row groups: 2.17 ms).
  if (w8a8) return 4;
  return avg > 24.0 ? 4 : avg > 12.0 ? 2 : 1;
}

// column tiles per block of the unit order (k_prefill_plan)
int pick_tgb() {
  if (const char* f = getenv("FFMOE_PREFILL_TGB")) return max(1, atoi(f));
  return 1 << 20;
}

// row groups of one expert that share a run of units (k_prefill_plan)
int pick_rgb() {
  if (const char* f = getenv("FFMOE_PREFILL_RGB")) return max(1, atoi(f));
  return 32;  // measured at 4096 tokens, top-8 of 256, Zipf: 32 is 1 to 4 % ahead of unblocked on the gate/up launch (two seeded routings), 8 and below lose
}

// wide: 64-row groups with eight waves per block (twice the columns per unit and token tile), one block per CU
template <int MODE>
int launch_gemm(const GemmParams& p, int mf, unsigned blocks, hipStream_t stream, bool wide = false, bool nv = false) {
  if (nv) {  // NVFP4 weights turned into E4M3 on their way through LDS: the eight-wave 64-row kernel only
    hipLaunchKernelGGL((k_w8a8_grouped<4, MODE, 2, 8, true>), dim3(blocks), dim3(512), 0, stream, p);
    return ff_launch_status();
  }
  if (wide) {
    hipLaunchKernelGGL((k_w8a8_grouped<4, MODE, 2, 8>), dim3(blocks), dim3(512), 0, stream, p);
    return ff_launch_status();
  }
  switch (mf) {
    case 1: hipLaunchKernelGGL((k_w8a8_grouped<1, MODE, 4>), dim3(blocks), dim3(256), 0, stream, p); break;
    case 2: hipLaunchKernelGGL((k_w8a8_grouped<2, MODE, 4>), dim3(blocks), dim3(256), 0, stream, p); break;
    case 4: hipLaunchKernelGGL((k_w8a8_grouped<4, MODE, 2>), dim3(blocks), dim3(256), 0, stream, p); break;
    default: hipLaunchKernelGGL((k_w8a8_grouped<8, MODE, 2>), dim3(blocks), dim3(256), 0, stream, p); break;
  }
  return ff_launch_status();
}

// read at every call
bool nvfp4_lines_enabled() {
  const char* le = getenv("FFMOE_PREFILL_NVFP4_LINES");
  return !(le && atoi(le) == 0);
}

// 16-row groups of the NVFP4 line kernel: one set of lines ahead and three blocks per CU (FFMOE_PREFILL_LINES_THREE_BLOCKS=0: two
// sets ahead, two blocks; same bits); read at every call
bool lines_three_blocks() {
  const char* e = getenv("FFMOE_PREFILL_LINES_THREE_BLOCKS");
  return !(e && atoi(e) == 0);
}

template <class F, int MODE>
int launch_w16(const W16Params& p, int mf, unsigned blocks, hipStream_t stream, bool wide = false) {
  if constexpr (std::is_same<F, FmtFp8>::value) {
    // 16- and 32-row groups (decode batches): whole 128-byte code lines per request (FFMOE_PREFILL_FP8_LINES=0 keeps the
    // per-K-block kernel; same bits). 64-row groups keep the per-K-block kernel: two sets ahead do not fit their registers
    const char* le = getenv("FFMOE_PREFILL_FP8_LINES");
    if (!(le && atoi(le) == 0) && !wide && mf == 1) {
      // one set of lines ahead and four blocks per CU for gate/up, three for down (FFMOE_FP8_LINES_OCC=2: two sets ahead, two
      // blocks; 3 / 4: that many blocks for both launches; same bits). 8 tokens, gate/up | down: 308 | 161 us with two, 299 | 148
      // with three, 292 | 153 with four blocks; 64 tokens: 1116 | 600, 1080 | 568, 1051 | 569
      const char* oe = getenv("FFMOE_FP8_LINES_OCC");
      const int occ = oe ? atoi(oe) : (MODE == 0 ? 4 : 3);
      if (occ == 3) hipLaunchKernelGGL((k_w16_fp8_lines<1, MODE, 1, 4, 3>), dim3((blocks * 3 / 2 + 7u) & ~7u), dim3(256), 0, stream, p);
      else if (occ == 4) hipLaunchKernelGGL((k_w16_fp8_lines<1, MODE, 1, 4, 4>), dim3(blocks * 2), dim3(256), 0, stream, p);
      else hipLaunchKernelGGL((k_w16_fp8_lines<1, MODE, 2>), dim3(blocks), dim3(256), 0, stream, p);
      return ff_launch_status();
    }
  }
  if constexpr (std::is_same<F, FmtNvfp4>::value) {
    // rows of whole 128-byte code lines: the line-wise kernel (FFMOE_PREFILL_NVFP4_LINES=0 keeps the per-K-block one)
    if (p.K % 256 == 0 && nvfp4_lines_enabled()) {
      if (wide) hipLaunchKernelGGL((k_w16_nvfp4_lines<4, MODE, 1, 8>), dim3(blocks), dim3(512), 0, stream, p);
      else if (mf == 1 && lines_three_blocks()) hipLaunchKernelGGL((k_w16_nvfp4_lines<1, MODE, 1, 4, 3>), dim3((blocks * 3 / 2 + 7u) & ~7u), dim3(256), 0, stream, p);  // whole blocks per XCD
      else if (mf == 1) hipLaunchKernelGGL((k_w16_nvfp4_lines<1, MODE, 2>), dim3(blocks), dim3(256), 0, stream, p);
      else if (mf == 2) hipLaunchKernelGGL((k_w16_nvfp4_lines<2, MODE, 2>), dim3(blocks), dim3(256), 0, stream, p);
      else hipLaunchKernelGGL((k_w16_nvfp4_lines<4, MODE, 1>), dim3(blocks), dim3(256), 0, stream, p);
      return ff_launch_status();
    }
  }
  if (wide) {  // 64-row groups, eight waves per block, one block per CU
    hipLaunchKernelGGL((k_w16_grouped<F, 4, MODE, 2, 8>), dim3(blocks), dim3(512), 0, stream, p);
    return ff_launch_status();
  }
  switch (mf) {
    case 1: hipLaunchKernelGGL((k_w16_grouped<F, 1, MODE, 2>), dim3(blocks), dim3(256), 0, stream, p); break;
    case 2: hipLaunchKernelGGL((k_w16_grouped<F, 2, MODE, 2>), dim3(blocks), dim3(256), 0, stream, p); break;
    default: hipLaunchKernelGGL((k_w16_grouped<F, 4, MODE, 2>), dim3(blocks), dim3(256), 0, stream, p); break;
  }
  return ff_launch_status();
}
template <int MODE>
int launch_w16_fmt(int format, const W16Params& p, int mf, unsigned blocks, hipStream_t stream, bool wide = false) {
  switch (format) {
    case FFMOE_FMT_FP8_BLOCK128: return launch_w16<FmtFp8, MODE>(p, mf, blocks, stream, wide);
    case FFMOE_FMT_NVFP4: return launch_w16<FmtNvfp4, MODE>(p, mf, blocks, stream, wide);
    case FFMOE_FMT_FP8_CHANNEL: return launch_w16<FmtFp8Channel, MODE>(p, mf, blocks, stream, wide);
    default: return launch_w16<FmtBf16, MODE>(p, mf, blocks, stream, wide);
  }
}

// One wave per block and a quarter of the tile's columns: for one dense group over few rows (the always-on expert), whose
// four-wave tiles would be a few dozen blocks on 256 CUs (a lone wave per CU is bound by the one-stage lead of its token
// tile, not by its weight loads: four K blocks ahead measured the same as two). Block-FP8 and BF16 weights.
template <int MODE>
bool launch_w16_narrow(int format, const W16Params& p, int mf, unsigned blocks, hipStream_t stream) {
#define FF_NARROW(F_)                                                                                              \
  switch (mf) {                                                                                                    \
    case 1: hipLaunchKernelGGL((k_w16_grouped<F_, 1, MODE, 2, 1>), dim3(blocks), dim3(64), 0, stream, p); break;   \
    case 2: hipLaunchKernelGGL((k_w16_grouped<F_, 2, MODE, 2, 1>), dim3(blocks), dim3(64), 0, stream, p); break;   \
    default: hipLaunchKernelGGL((k_w16_grouped<F_, 4, MODE, 2, 1>), dim3(blocks), dim3(64), 0, stream, p); break;  \
  }
  if (format == FFMOE_FMT_BF16) { FF_NARROW(FmtBf16) return true; }
  if (format == FFMOE_FMT_FP8_BLOCK128) { FF_NARROW(FmtFp8) return true; }
#undef FF_NARROW
  return false;
}

template <int MODE, int PACKED>
int launch_mx(const MxParams& p, int mf, unsigned blocks, hipStream_t stream, bool wide = false) {
  if (wide) {
    hipLaunchKernelGGL((k_mx_grouped<4, MODE, PACKED, 2, 8>), dim3(blocks), dim3(512), 0, stream, p);
    return ff_launch_status();
  }
  switch (mf) {
    case 1: hipLaunchKernelGGL((k_mx_grouped<1, MODE, PACKED, 2>), dim3(blocks), dim3(256), 0, stream, p); break;
    case 2: hipLaunchKernelGGL((k_mx_grouped<2, MODE, PACKED, 2>), dim3(blocks), dim3(256), 0, stream, p); break;
    default: hipLaunchKernelGGL((k_mx_grouped<4, MODE, PACKED, 2>), dim3(blocks), dim3(256), 0, stream, p); break;
  }
  return ff_launch_status();
}

struct PrefillLayout {
  uint64_t xq, sx, act, aq, sa, counts, offsets, gbase, totals, perm, groups, units0, units1, sh_act, sh_aq, sh_sa, total;
  uint64_t max_groups;
};
PrefillLayout prefill_layout(int rows, int top_k, int experts, int hidden, int inter, int shared_inter) {
  PrefillLayout l{};
  const uint64_t A = uint64_t(rows) * top_k;
  l.max_groups = uint64_t(experts) + (A + 15) / 16 + (shared_inter > 0 ? (uint64_t(rows) + 15) / 16 : 0);
  uint64_t off = 0;
  auto take = [&](uint64_t bytes) { const uint64_t at = off; off += up256(bytes); return at; };
  l.xq = take(uint64_t(rows) * hidden);
  l.sx = take(uint64_t(rows) * (hidden / 128) * 4);
  l.act = take(A * inter * 2);
  l.aq = take(A * inter);
  l.sa = take(A * (inter / 128) * 4);
  l.counts = take(uint64_t(experts) * 4);
  l.offsets = take(uint64_t(experts + 1) * 4);
  l.gbase = take(uint64_t(experts + 1) * 4);
  l.totals = take(16);
  l.perm = take(A * 4);
  l.groups = take(l.max_groups * sizeof(GemmGroup));
  l.units0 = take(l.max_groups * uint64_t((inter + 127) / 128) * 8);
  l.units1 = take(l.max_groups * uint64_t((hidden + 255) / 256) * 8);
  if (shared_inter > 0) {
    l.sh_act = take(uint64_t(rows) * shared_inter * 2);
    l.sh_aq = take(uint64_t(rows) * shared_inter);
    l.sh_sa = take(uint64_t(rows) * (shared_inter / 128) * 4);
  }
  l.total = off;
  return l;
}
}  // namespace

extern "C" __attribute__((visibility("default"))) int ffmoe_linear_fp8_block_w8a8(const void* w_codes, const float* w_scales, const void* x_codes,
                                                                                 const float* x_scales, void* y, int m, int n, int k, void* stream) {
  FF_REQUIRE(m >= 1 && n >= 16 && n % 16 == 0 && k >= 128 && k % 128 == 0, FFMOE_ERR_SHAPE,
             "w8a8 linear m=%d n=%d k=%d (n must be a multiple of 16, k a multiple of 128)", m, n, k);
  FF_PTR16(w_codes); FF_PTR4(w_scales); FF_PTR16(x_codes); FF_PTR4(x_scales); FF_PTR16(y);
  FF_NO_OVERLAP(y, size_t(m) * n * 2, x_codes, size_t(m) * k);
  FF_NO_OVERLAP(y, size_t(m) * n * 2, x_scales, size_t(m) * (k / 128) * 4);
  const int mf = m > 32 ? 4 : m > 16 ? 2 : 1;
  const int tm = 16 * mf;
  GemmParams p{};
  p.a_codes = (const uint8_t*)x_codes; p.a_scales = x_scales;
  p.w0_codes = (uint64_t)(uintptr_t)w_codes; p.w0_scales = (uint64_t)(uintptr_t)w_scales;
  p.total_units = uint32_t(((m + tm - 1) / tm) * ((n + 255) / 256));
  p.out = (uint16_t*)y; p.rows_total = m; p.K = k; p.N = n; p.top_k = 1;
  const unsigned blocks = (unsigned)std::min<uint32_t>((p.total_units + 7u) & ~7u, uint32_t(num_cus_p()) * 2u) & ~7u;
  return launch_gemm<2>(p, mf, blocks, (hipStream_t)stream);
}

extern "C" __attribute__((visibility("default"))) uint64_t ffmoe_prefill_scratch_bytes(int rows, int top_k, int experts, int hidden, int inter, int shared_inter) {
  if (rows < 1 || top_k < 1 || experts < 1 || hidden < 128 || inter < 128 || shared_inter < 0) return 0;
  return prefill_layout(rows, top_k, experts, hidden, inter, shared_inter).total;
}

namespace ffmoe {
int prefill_impl(const ffmoe_expert_table* table, const ffmoe_prefill* args, int stages, void* stream_);

// The always-on expert over all rows in the decode path's W*A16 arithmetic on the BF16 matrix cores, as one dense group
// per 16 .. 64 rows: the weights stream once however many rows there are. act [rows, shared inter] BF16 holds the SwiGLU
// activations between the two launches; stage_mask bit 0 = gate/up + SwiGLU, bit 1 = down. Arguments are checked by the
// callers.
int shared_expert_w16(const ffmoe_shared_expert* shared, const void* x, int R, int H, int swiglu, float limit, void* act, void* shared_out,
                      int stage_mask, void* stream_) {
  hipStream_t stream = (hipStream_t)stream_;
  const int SI = shared->inter;
  const unsigned blocks = ((unsigned)num_cus_p() * 2u) & ~7u;
  const int smf = R > 32 ? 4 : R > 16 ? 2 : 1;
  const int stm = 16 * smf;
  const uint32_t sgroups = uint32_t((R + stm - 1) / stm);
  W16Params q{};
  q.rows_total = R; q.top_k = 1; q.shared_expert = -1;
  q.swiglu = swiglu; q.limit = limit;
  // fewer four-wave tiles than CUs: one-wave blocks over a quarter of the columns each (FFMOE_PREFILL_SHARED_NARROW=0
  // keeps the four-wave tiles; same bits)
  const char* ne = getenv("FFMOE_PREFILL_SHARED_NARROW");
  const bool may_narrow = (shared->format == FFMOE_FMT_BF16 || shared->format == FFMOE_FMT_FP8_BLOCK128) && !(ne && atoi(ne) == 0);
  const unsigned nblocks = ((unsigned)num_cus_p() * 8u) & ~7u;
  // A BF16 expert over so few rows that the grouped kernels would give it fewer tiles than CUs: blocks of eight waves that
  // split the contraction (dense_splitk.cuh; FFMOE_SHARED_SPLITK=0 keeps the grouped kernels). Hidden 7168 / intermediate
  // 2048, 32 rows: 62 + 19 us on one-wave tiles.
  const char* se = getenv("FFMOE_SHARED_SPLITK");
  const bool splitk = shared->format == FFMOE_FMT_BF16 && !(se && atoi(se) == 0) && H % 256 == 0 && SI % 256 == 0 &&
                      sgroups * uint32_t((SI + 127) / 128) < (unsigned)num_cus_p();
  if (splitk) {
    // 8 activation columns (gate + up rows in one fragment) or 16 output columns per block; tiles of half that size, for
    // twice the blocks, measured slower (32 rows: 52 + 34 against 32 + 20 us): every block reads the whole token panel
    const int mft = R > 32 ? 4 : 2;
    const unsigned gy = unsigned((R + 16 * mft - 1) / (16 * mft));
    DenseParams d{};
    d.rows = R; d.swiglu = swiglu; d.limit = limit;
    // up to 32 rows the token panel goes through LDS (two buffers of 32 rows x 2 KB, a round ahead); it needs every wave's steps
    // in whole chunks of four, i.e. contractions that are multiples of 1024 (FFMOE_SPLITK_LDS=0: requested in lane order; same bits)
    const char* xe = getenv("FFMOE_SPLITK_LDS");
    constexpr size_t xl_bytes = size_t(2) * 32 * (2048 + 16);
    static int xl_ok = -1;
    if (xl_ok < 0) {
      xl_ok = hipFuncSetAttribute(reinterpret_cast<const void*>(k_dense_bf16_splitk<0, 2, 8, 1, true>), hipFuncAttributeMaxDynamicSharedMemorySize, int(xl_bytes)) == hipSuccess &&
              hipFuncSetAttribute(reinterpret_cast<const void*>(k_dense_bf16_splitk<2, 2, 16, 2, true>), hipFuncAttributeMaxDynamicSharedMemorySize, int(xl_bytes)) == hipSuccess ? 1 : 0;
      if (!xl_ok) (void)hipGetLastError();
    }
    const bool xl = mft == 2 && xl_ok == 1 && !(xe && atoi(xe) == 0);
    if (stage_mask & 1) {
      d.x = (const uint16_t*)x; d.w0 = (const uint16_t*)shared->slot[0]; d.w1 = (const uint16_t*)shared->slot[2];
      d.out = (uint16_t*)act; d.K = H; d.N = SI;
      const dim3 grid(unsigned(SI / 8), gy);
      if (mft == 4) hipLaunchKernelGGL((k_dense_bf16_splitk<0, 4, 8>), grid, dim3(512), 0, stream, d);
      else if (xl && H % 1024 == 0) hipLaunchKernelGGL((k_dense_bf16_splitk<0, 2, 8, 1, true>), grid, dim3(512), xl_bytes, stream, d);
      else hipLaunchKernelGGL((k_dense_bf16_splitk<0, 2, 8>), grid, dim3(512), 0, stream, d);
      FF_TRY(ff_launch_status());
    }
    if (stage_mask & 2) {
      d.x = (const uint16_t*)act; d.w0 = (const uint16_t*)shared->slot[4]; d.w1 = nullptr;
      d.out = (uint16_t*)shared_out; d.K = SI; d.N = H;
      // two fragments = 32 output columns per block (32 rows at hidden 7168: 15.2 us against 20.6 with one and 20.7 with four)
      const dim3 grid(unsigned(H / 32), gy);
      if (mft == 4) hipLaunchKernelGGL((k_dense_bf16_splitk<2, 4, 16, 2>), grid, dim3(512), 0, stream, d);
      else if (xl && SI % 1024 == 0) hipLaunchKernelGGL((k_dense_bf16_splitk<2, 2, 16, 2, true>), grid, dim3(512), xl_bytes, stream, d);
      else hipLaunchKernelGGL((k_dense_bf16_splitk<2, 2, 16, 2>), grid, dim3(512), 0, stream, d);
      FF_TRY(ff_launch_status());
    }
    return 0;
  }
  if (stage_mask & 1) {
    q.a = (const uint16_t*)x;
    q.w0_codes = shared->slot[0]; q.w0_scales = shared->slot[1]; q.w1_codes = shared->slot[2]; q.w1_scales = shared->slot[3];
    q.g0 = shared->global_scales[0]; q.g1 = shared->global_scales[1];
    q.total_units = sgroups * uint32_t((SI + 127) / 128);
    q.out = (uint16_t*)act; q.K = H; q.N = SI;
    if (may_narrow && q.total_units < (unsigned)num_cus_p()) {
      q.total_units = sgroups * uint32_t((SI + 31) / 32);
      launch_w16_narrow<0>(shared->format, q, smf, std::min<unsigned>(nblocks, (q.total_units + 7u) & ~7u), stream);
      FF_TRY(ff_launch_status());
    } else {
      FF_TRY(launch_w16_fmt<0>(shared->format, q, smf, std::min<unsigned>(blocks, (q.total_units + 7u) & ~7u), stream));
    }
  }
  if (stage_mask & 2) {
    q.a = (const uint16_t*)act;
    q.w0_codes = shared->slot[4]; q.w0_scales = shared->slot[5]; q.w1_codes = 0; q.w1_scales = 0;
    q.g0 = shared->global_scales[2]; q.g1 = q.g0;
    q.total_units = sgroups * uint32_t((H + 255) / 256);
    q.out = (uint16_t*)shared_out; q.K = SI; q.N = H;
    if (may_narrow && q.total_units < (unsigned)num_cus_p()) {
      q.total_units = sgroups * uint32_t((H + 63) / 64);
      launch_w16_narrow<2>(shared->format, q, smf, std::min<unsigned>(nblocks, (q.total_units + 7u) & ~7u), stream);
      FF_TRY(ff_launch_status());
    } else {
      FF_TRY(launch_w16_fmt<2>(shared->format, q, smf, std::min<unsigned>(blocks, (q.total_units + 7u) & ~7u), stream));
    }
  }
  return 0;
}
}
extern "C" __attribute__((visibility("default"))) int ffmoe_prefill_contribute(const ffmoe_expert_table* table, const ffmoe_prefill* args, void* stream) {
  return prefill_impl(table, args, 15, stream);
}
extern "C" __attribute__((visibility("default"))) int ffmoe_prefill_contribute_stage(const ffmoe_expert_table* table, const ffmoe_prefill* args, int stage, void* stream) {
  FF_REQUIRE(stage >= 0 && stage <= 3, FFMOE_ERR_SHAPE, "prefill stage %d (0 plan, 1 gate/up, 2 re-quantize, 3 down)", stage);
  return prefill_impl(table, args, 1 << stage, stream);
}
namespace ffmoe {
int prefill_impl(const ffmoe_expert_table* table, const ffmoe_prefill* args, int stages, void* stream_) {
  hipStream_t stream = (hipStream_t)stream_;
  FF_REQUIRE(table != nullptr && args != nullptr, FFMOE_ERR_NULL, "table or args is NULL");
  // FFMOE_ACT_FP8_BLOCK128: W8A8 on the FP8 matrix cores (block-FP8 experts); FFMOE_ACT_BF16: the decode path's W*A16
  // arithmetic on the BF16 matrix cores, any expert format
  const bool a16 = args->act_mode == FFMOE_ACT_BF16;
  // FFMOE_FMT_E2M1_E8M0 experts with FFMOE_ACT_E4M3_E8M0_32: the W4A8 contract on the MX matrix cores
  const bool mx = table->format == FFMOE_FMT_E2M1_E8M0;
  if (mx) {
    FF_REQUIRE(args->act_mode == FFMOE_ACT_E4M3_E8M0_32, FFMOE_ERR_UNSUPPORTED, "E2M1/E8M0 experts take FFMOE_ACT_E4M3_E8M0_32 activations (act_mode %d)", args->act_mode);
    FF_REQUIRE(args->routed_weight == FFMOE_WEIGHT_BEFORE_DOWN_F32 && args->weights_f32 == 1, FFMOE_ERR_UNSUPPORTED,
               "the routed weight is an f32 applied before the down projection (FFMOE_WEIGHT_BEFORE_DOWN_F32)");
    FF_REQUIRE(args->swiglu_limit > 0.0f && args->swiglu_limit < INFINITY, FFMOE_ERR_SHAPE, "the contract clamps the SwiGLU inputs: limit %g", (double)args->swiglu_limit);
    FF_REQUIRE(!args->shared || args->shared->format == FFMOE_FMT_E4M3_E8M0_32, FFMOE_ERR_UNSUPPORTED, "the shared expert must be FFMOE_FMT_E4M3_E8M0_32 (format %d)",
               args->shared ? args->shared->format : -1);
    FF_REQUIRE((long long)args->rows * args->top_k <= 65535, FFMOE_ERR_SHAPE, "the activation quantizer takes at most 65535 assignments per call (rows=%d top_k=%d)", args->rows, args->top_k);
  } else {
  FF_REQUIRE(a16 || args->act_mode == FFMOE_ACT_FP8_BLOCK128, FFMOE_ERR_UNSUPPORTED, "prefill act_mode %d (FFMOE_ACT_FP8_BLOCK128 or FFMOE_ACT_BF16)", args->act_mode);
  if (a16)
    FF_REQUIRE(table->format == FFMOE_FMT_FP8_BLOCK128 || table->format == FFMOE_FMT_NVFP4 || table->format == FFMOE_FMT_BF16 || table->format == FFMOE_FMT_FP8_CHANNEL,
               FFMOE_ERR_UNSUPPORTED, "unknown expert format %d", table->format);
  else
    FF_REQUIRE(table->format == FFMOE_FMT_FP8_BLOCK128 || table->format == FFMOE_FMT_NVFP4, FFMOE_ERR_UNSUPPORTED,
               "FP8 activations on the FP8 matrix cores take FFMOE_FMT_FP8_BLOCK128 experts (W8A8) or FFMOE_FMT_NVFP4 experts (W4A8) (format %d)", table->format);
  }
  // W4A8: NVFP4 experts with FP8 activations. Each weight becomes E4M3 inside the kernel (E2M1 value x E4M3 scale / 8,
  // rounded to nearest even), the matrix's global scale x 8 takes the place of the block scales
  const bool nv = !mx && !a16 && table->format == FFMOE_FMT_NVFP4;
  if (nv) FF_PTR4(table->global_scales);
  const int E = table->experts, H = table->hidden, I = table->inter, R = args->rows, K = args->top_k;
  FF_REQUIRE(E >= 1 && E <= FFMOE_MAX_EXPERTS, FFMOE_ERR_SHAPE, "experts=%d out of range", E);
  FF_REQUIRE(R >= 1 && K >= 1 && K <= FFMOE_MAX_TOP_K && (long long)R * K <= 0x3fffffffLL, FFMOE_ERR_SHAPE, "rows=%d top_k=%d out of range", R, K);
  if (a16 && table->format != FFMOE_FMT_FP8_BLOCK128)
    FF_REQUIRE(H >= 64 && H % 64 == 0 && I >= 64 && I % 64 == 0, FFMOE_ERR_SHAPE, "hidden=%d and inter=%d must be multiples of 64", H, I);
  else
    FF_REQUIRE(H >= 128 && H % 128 == 0 && I >= 128 && I % 128 == 0, FFMOE_ERR_SHAPE, "hidden=%d and inter=%d must be multiples of 128", H, I);
  if (a16 && table->format == FFMOE_FMT_NVFP4) FF_PTR4(table->global_scales);
  FF_REQUIRE(args->swiglu >= 0 && args->swiglu <= FFMOE_SWIGLU_GELU_TWICE, FFMOE_ERR_UNSUPPORTED, "unknown SwiGLU mode %d", args->swiglu);
  FF_REQUIRE(args->swiglu != FFMOE_SWIGLU_GELU_TWICE || a16, FFMOE_ERR_UNSUPPORTED,
             "FFMOE_SWIGLU_GELU_TWICE needs act_mode FFMOE_ACT_BF16 (the FP8-activation kernels implement the SiLU forms only)");
  if (args->swiglu == FFMOE_SWIGLU_CLAMPED_TWICE || args->swiglu == FFMOE_SWIGLU_CLAMPED_ONCE) FF_REQUIRE(args->swiglu_limit > 0.0f && args->swiglu_limit < INFINITY, FFMOE_ERR_SHAPE, "invalid SwiGLU limit %g", (double)args->swiglu_limit);
  if (!mx)
    FF_REQUIRE(args->routed_weight == FFMOE_WEIGHT_AFTER_DOWN_BF16 || args->routed_weight == FFMOE_WEIGHT_BEFORE_CONTRIBUTION_BF16,
               FFMOE_ERR_UNSUPPORTED, "unknown routed_weight %d", args->routed_weight);
  FF_PTR16(table->slots); FF_PTR16(args->x); FF_PTR4(args->ids); FF_PTR16(args->contributions);
  if (args->weights_f32) FF_PTR4(args->weights); else FF_PTR2(args->weights);
  const ffmoe_shared_expert* shared = args->shared;
  int SI = 0;
  if (shared) {
    SI = shared->inter;
    if (mx) {
      FF_REQUIRE(SI >= 128 && SI % 128 == 0, FFMOE_ERR_SHAPE, "shared inter=%d must be a positive multiple of 128", SI);
    } else if (a16) {
      FF_REQUIRE(shared->format == FFMOE_FMT_FP8_BLOCK128 || shared->format == FFMOE_FMT_NVFP4 || shared->format == FFMOE_FMT_BF16 || shared->format == FFMOE_FMT_FP8_CHANNEL,
                 FFMOE_ERR_UNSUPPORTED, "unknown shared expert format %d", shared->format);
      const int gran = shared->format == FFMOE_FMT_FP8_BLOCK128 ? 128 : 64;
      FF_REQUIRE(SI >= gran && SI % gran == 0 && H % gran == 0, FFMOE_ERR_SHAPE, "shared inter=%d and hidden=%d must be multiples of %d", SI, H, gran);
    } else {
      FF_REQUIRE(shared->format == FFMOE_FMT_FP8_BLOCK128 || (nv && shared->format == FFMOE_FMT_NVFP4), FFMOE_ERR_UNSUPPORTED,
                 "with FP8 activations the shared expert is FFMOE_FMT_FP8_BLOCK128, or FFMOE_FMT_NVFP4 next to NVFP4 experts (format %d)", shared->format);
      FF_REQUIRE(SI >= 128 && SI % 128 == 0, FFMOE_ERR_SHAPE, "shared inter=%d must be a positive multiple of 128", SI);
    }
    FF_PTR16(args->shared_out);
    for (int i = 0; i < 6; ++i) {
      const bool scale_entry = i % 2 == 1;
      if (scale_entry && shared->format == FFMOE_FMT_BF16) continue;  // BF16 weights carry no scales
      FF_REQUIRE(shared->slot[i] != 0 && shared->slot[i] % (scale_entry ? (shared->format == FFMOE_FMT_FP8_BLOCK128 || shared->format == FFMOE_FMT_NVFP4 ? 4 : (mx ? 1 : 2)) : 16) == 0, FFMOE_ERR_ALIGN,
                 "shared expert slot[%d] is NULL or misaligned", i);
    }
  }
  const PrefillLayout l = prefill_layout(R, K, E, H, I, SI);
  FF_PTR_ALIGNED(args->scratch, 256);
  FF_REQUIRE(args->scratch_bytes >= l.total, FFMOE_ERR_SCRATCH, "prefill scratch holds %llu bytes, %llu needed",
             (unsigned long long)args->scratch_bytes, (unsigned long long)l.total);
  const size_t A = size_t(R) * K;
  FF_NO_OVERLAP(args->contributions, A * H * 2, args->x, size_t(R) * H * 2);
  FF_NO_OVERLAP(args->contributions, A * H * 2, args->scratch, l.total);
  FF_NO_OVERLAP(args->scratch, l.total, args->x, size_t(R) * H * 2);
  FF_NO_OVERLAP(args->scratch, l.total, args->ids, A * 4);
  if (args->done) { FF_PTR4(args->done); FF_NO_OVERLAP(args->done, A * 4, args->scratch, l.total); }
  if (shared) {
    FF_NO_OVERLAP(args->shared_out, size_t(R) * H * 2, args->scratch, l.total);
    FF_NO_OVERLAP(args->shared_out, size_t(R) * H * 2, args->x, size_t(R) * H * 2);
    FF_NO_OVERLAP(args->shared_out, size_t(R) * H * 2, args->contributions, A * H * 2);
  }

  uint8_t* s = (uint8_t*)args->scratch;
  PrefillBook b{(uint32_t*)(s + l.counts), (uint32_t*)(s + l.offsets), (uint32_t*)(s + l.gbase), (uint32_t*)(s + l.totals),
                (int*)(s + l.perm), (GemmGroup*)(s + l.groups), (u32x2*)(s + l.units0), (u32x2*)(s + l.units1)};
  const int mf = nv ? 4 : pick_mf(double(A) / E, (mx || a16) ? 4 : 8, !mx && !a16);
  const int tm = 16 * mf;
  // W8A8, W*A16 and MX cohorts in 64-row groups: eight waves per block share a token tile (FFMOE_PREFILL_WIDE=0: four, two blocks per CU)
  bool wide = mf == 4;
  if (const char* f = getenv("FFMOE_PREFILL_WIDE")) wide = (wide && atoi(f) != 0) || nv;
  const int tiles0 = wide ? (I + 255) / 256 : (I + 127) / 128, tiles1 = wide ? (H + 511) / 512 : (H + 255) / 256;
  // A shared expert of the routed experts' format and width rides in the routed launches as further row groups (W*A16
  // cohorts): on its own it is a few dozen blocks per launch, which at small cohorts take longer than the routed experts'
  // thousands. FFMOE_PREFILL_SHARED_RIDE=0 keeps it in launches of its own (the results are the same bits either way).
  bool ride = a16 && shared && shared->format == table->format && SI == I;
  if (const char* f = getenv("FFMOE_PREFILL_SHARED_RIDE")) ride = ride && atoi(f) != 0;

  if (stages & 1) {
    const LiveTest lt{args->ids, args->active, table->valid, table->generation, args->assignment_gen, E};
    // up to this many assignments one launch does the bookkeeping (measured at 256 experts: 64 assignments 10 us against
    // 21 us for the four launches, 512 assignments 31 against 29 us); FFMOE_PREFILL_BOOK_SMALL overrides the limit
    // (0: the four launches at any size, at most FFMOE_BOOK_SMALL_MAX)
    int small_max = 256;
    if (const char* f = getenv("FFMOE_PREFILL_BOOK_SMALL")) small_max = std::max(0, std::min(atoi(f), FFMOE_BOOK_SMALL_MAX));
    const bool small = A <= size_t(small_max);
    if (small) {
      // The unit lists are one entry per (row group, column tile): thousands of entries even for a few hundred assignments
      // (32 rows, top-8 of 256 at hidden 7168: 7260), too many for the one block - from 2048 possible units on they are
      // written by a launch of their own over as many blocks as they need (FFMOE_PREFILL_BOOK_UNITS overrides the bound)
      const uint64_t max_units = l.max_groups * uint64_t(tiles0 + tiles1);
      uint64_t own_launch_from = 2048;
      if (const char* f = getenv("FFMOE_PREFILL_BOOK_UNITS")) own_launch_from = uint64_t(std::max(0, atoi(f)));
      const bool split_units = max_units >= own_launch_from;
      hipLaunchKernelGGL(k_prefill_book_small, dim3(1), dim3(1024), 0, stream, lt, b, int(A), E, tm, tiles0, tiles1, pick_rgb(), pick_tgb(), ride ? R : 0,
                         split_units ? 0 : 1);
      if (split_units)
        hipLaunchKernelGGL(k_prefill_units, dim3((unsigned)((max_units + 255) / 256)), dim3(256), 0, stream, b, E, tm, tiles0, tiles1, pick_rgb(), pick_tgb(), ride ? R : 0);
    } else {
      hipLaunchKernelGGL(k_prefill_zero, dim3((E + 255) / 256), dim3(256), 0, stream, b.counts, E, b.totals);
      hipLaunchKernelGGL(k_prefill_count, dim3((unsigned)((A + FFMOE_COUNT_PER_BLOCK - 1) / FFMOE_COUNT_PER_BLOCK)), dim3(256), 0, stream, lt, b.counts, (long long)A);
      hipLaunchKernelGGL(k_prefill_plan, dim3(1), dim3(1024), 0, stream, b, E, tm, tiles0, tiles1, pick_rgb(), pick_tgb(), ride ? R : 0);
      const uint64_t max_units = l.max_groups * uint64_t(tiles0 + tiles1);
      hipLaunchKernelGGL(k_prefill_units, dim3((unsigned)((max_units + 255) / 256)), dim3(256), 0, stream, b, E, tm, tiles0, tiles1, pick_rgb(), pick_tgb(), ride ? R : 0);
      hipLaunchKernelGGL(k_prefill_fill, dim3(E), dim3(256), 0, stream, lt, b, (long long)A);
    }
    FF_TRY(ff_launch_status());
    // activations -> E4M3 + per-128 scales
    if (mx) FF_TRY(ffmoe_act_quant_e8m0(args->x, s + l.xq, s + l.sx, R, H, stream_));  // E4M3 codes + one E8M0 byte per 32
    else if (!a16) FF_TRY(ffmoe_quant_fp8_f32_128(args->x, s + l.xq, (float*)(s + l.sx), R, H, stream_));
  }
  const unsigned blocks = ((unsigned)num_cus_p() * 2u) & ~7u;
  if (mx) {
    MxParams p{};
    p.slots = table->slots; p.groups = b.groups; p.perm = b.perm; p.top_k = K; p.limit = args->swiglu_limit;
    if (stages & 2) {
      p.a_codes = s + l.xq; p.a_scales = s + l.sx; p.units = b.units0; p.unit_total = b.totals + 0;
      p.weights = (const float*)args->weights; p.out = (uint16_t*)(s + l.act); p.K = H; p.N = I;
      FF_TRY((launch_mx<0, 1>(p, mf, wide ? blocks / 2 : blocks, stream, wide)));
    }
    if (stages & 4) FF_TRY(ffmoe_act_quant_e8m0(s + l.act, s + l.aq, s + l.sa, int(A), I, stream_));
    if (stages & 8) {
      p.a_codes = s + l.aq; p.a_scales = s + l.sa; p.units = b.units1; p.unit_total = b.totals + 1;
      p.weights = nullptr; p.out = (uint16_t*)args->contributions; p.done = args->done; p.K = I; p.N = H;
      FF_TRY((launch_mx<1, 1>(p, mf, wide ? blocks / 2 : blocks, stream, wide)));
    }
    if (shared) {
      const int smf = R > 32 ? 4 : R > 16 ? 2 : 1;
      const int stm = 16 * smf;
      const uint32_t sgroups = uint32_t((R + stm - 1) / stm);
      MxParams q{};
      q.rows_total = R; q.top_k = 1; q.limit = args->swiglu_limit;
      if (stages & 2) {
        q.a_codes = s + l.xq; q.a_scales = s + l.sx;
        q.w0_codes = shared->slot[0]; q.w0_scales = shared->slot[1]; q.w1_codes = shared->slot[2]; q.w1_scales = shared->slot[3];
        q.total_units = sgroups * uint32_t((SI + 127) / 128);
        q.out = (uint16_t*)(s + l.sh_act); q.K = H; q.N = SI;
        FF_TRY((launch_mx<0, 0>(q, smf, std::min<unsigned>(blocks, (q.total_units + 7u) & ~7u), stream)));
      }
      if (stages & 4) FF_TRY(ffmoe_act_quant_e8m0(s + l.sh_act, s + l.sh_aq, s + l.sh_sa, R, SI, stream_));
      if (stages & 8) {
        q.a_codes = s + l.sh_aq; q.a_scales = s + l.sh_sa;
        q.w0_codes = shared->slot[4]; q.w0_scales = shared->slot[5]; q.w1_codes = 0; q.w1_scales = 0;
        q.total_units = sgroups * uint32_t((H + 255) / 256);
        q.out = (uint16_t*)args->shared_out; q.K = SI; q.N = H;
        FF_TRY((launch_mx<2, 0>(q, smf, std::min<unsigned>(blocks, (q.total_units + 7u) & ~7u), stream)));
      }
    }
    return 0;
  }
  if (a16) {
    // BF16 activations end to end: x -> (gate/up + SwiGLU) -> act -> (down x routing weight) -> contributions
    W16Params p{};
    p.slots = table->slots; p.global_scales = table->format == FFMOE_FMT_NVFP4 ? table->global_scales : nullptr;
    p.groups = b.groups; p.perm = b.perm; p.top_k = K;
    p.swiglu = args->swiglu; p.limit = args->swiglu_limit; p.routed_weight = args->routed_weight; p.weights_f32 = args->weights_f32;
    p.shared_expert = ride ? E : -1;
    if (ride) {
      for (int i = 0; i < 6; ++i) p.sh_w[i] = shared->slot[i];
      for (int i = 0; i < 3; ++i) p.sh_g[i] = shared->global_scales[i];
    }
    if (stages & 2) {
      p.a = (const uint16_t*)args->x; p.units = b.units0; p.unit_total = b.totals + 0;
      p.out = (uint16_t*)(s + l.act); p.K = H; p.N = I;
      p.a_sh = (const uint16_t*)args->x; p.out_sh = (uint16_t*)(s + l.sh_act);
      FF_TRY(launch_w16_fmt<0>(table->format, p, mf, wide ? blocks / 2 : blocks, stream, wide));
    }
    if (stages & 8) {
      p.a = (const uint16_t*)(s + l.act); p.units = b.units1; p.unit_total = b.totals + 1;
      p.out = (uint16_t*)args->contributions; p.done = args->done; p.weights = args->weights; p.K = I; p.N = H;
      p.a_sh = (const uint16_t*)(s + l.sh_act); p.out_sh = (uint16_t*)args->shared_out;
      FF_TRY(launch_w16_fmt<1>(table->format, p, mf, wide ? blocks / 2 : blocks, stream, wide));
    }
    if (shared && !ride)
      FF_TRY(shared_expert_w16(shared, args->x, R, H, args->swiglu, args->swiglu_limit, s + l.sh_act, args->shared_out,
                               (stages & 2 ? 1 : 0) | (stages & 8 ? 2 : 0), stream_));
    return 0;
  }
  GemmParams p{};
  p.slots = table->slots; p.groups = b.groups; p.perm = b.perm; p.top_k = K;
  p.global_scales = nv ? table->global_scales : nullptr;
  p.swiglu = args->swiglu; p.limit = args->swiglu_limit; p.routed_weight = args->routed_weight; p.weights_f32 = args->weights_f32;
  if (stages & 2) {  // gate/up + SwiGLU
    p.a_codes = s + l.xq; p.a_scales = (const float*)(s + l.sx); p.units = b.units0; p.unit_total = b.totals + 0;
    p.out = (uint16_t*)(s + l.act); p.K = H; p.N = I;
    FF_TRY(launch_gemm<0>(p, mf, wide ? blocks / 2 : blocks, stream, wide, nv));
  }
  if (stages & 4) {  // re-quantize the activations of the live rows
    const long long cells = (long long)A * (I / 128);
    hipLaunchKernelGGL(k_quant_live, dim3((unsigned)((cells + 15) / 16)), dim3(256), 0, stream, (const uint16_t*)(s + l.act), s + l.aq,
                       (float*)(s + l.sa), (const uint32_t*)(b.totals + 3), I);
    FF_TRY(ff_launch_status());
  }
  if (stages & 8) {  // down x routing weight, scattered to contributions[assignment]
    p.a_codes = s + l.aq; p.a_scales = (const float*)(s + l.sa); p.units = b.units1; p.unit_total = b.totals + 1;
    p.out = (uint16_t*)args->contributions; p.done = args->done; p.weights = args->weights; p.K = I; p.N = H;
    FF_TRY(launch_gemm<1>(p, mf, wide ? blocks / 2 : blocks, stream, wide, nv));
  }
  if (shared) {
    // the always-on expert: the same three steps over all rows in their own order (no grouping, no routing weight),
    // as the reference runs it on the block-FP8 path (src/backend/cuda/moe/decode.rs:1187-1297)
    const bool snv = shared->format == FFMOE_FMT_NVFP4;  // its weights through the same conversion: 64-row groups, eight waves
    const int smf = snv ? 4 : (R > 32 ? 4 : R > 16 ? 2 : 1);
    const int stm = 16 * smf;
    const uint32_t sgroups = uint32_t((R + stm - 1) / stm);
    GemmParams q{};
    q.w0_global = shared->global_scales[0]; q.w1_global = shared->global_scales[1];
    q.rows_total = R; q.top_k = 1;
    q.swiglu = args->swiglu; q.limit = args->swiglu_limit;
    if (stages & 2) {
      q.a_codes = s + l.xq; q.a_scales = (const float*)(s + l.sx);
      q.w0_codes = shared->slot[0]; q.w0_scales = shared->slot[1]; q.w1_codes = shared->slot[2]; q.w1_scales = shared->slot[3];
      q.total_units = sgroups * uint32_t(snv ? (SI + 255) / 256 : (SI + 127) / 128);
      q.out = (uint16_t*)(s + l.sh_act); q.K = H; q.N = SI;
      FF_TRY(launch_gemm<0>(q, smf, std::min<unsigned>(snv ? blocks / 2 : blocks, (q.total_units + 7u) & ~7u), stream, false, snv));
    }
    if (stages & 4)
      FF_TRY(ffmoe_quant_fp8_f32_128(s + l.sh_act, s + l.sh_aq, (float*)(s + l.sh_sa), R, SI, stream_));
    if (stages & 8) {
      q.a_codes = s + l.sh_aq; q.a_scales = (const float*)(s + l.sh_sa);
      q.w0_codes = shared->slot[4]; q.w0_scales = shared->slot[5]; q.w1_codes = 0; q.w1_scales = 0;
      q.w0_global = shared->global_scales[2];
      q.total_units = sgroups * uint32_t(snv ? (H + 511) / 512 : (H + 255) / 256);
      q.out = (uint16_t*)args->shared_out; q.K = SI; q.N = H;
      FF_TRY(launch_gemm<2>(q, smf, std::min<unsigned>(snv ? blocks / 2 : blocks, (q.total_units + 7u) & ~7u), stream, false, snv));
    }
  }
  return 0;
}
}  // namespace ffmoe
