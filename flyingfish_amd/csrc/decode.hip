// Decode expert FFN: weight-streaming grouped GEMV kernels for FP8-block, NVFP4 and BF16 experts.
//
// Work model. Assignments (row, choice) that hit the same expert are gathered into groups of at most
// RG rows, so one pass over an expert's weights serves all of them. A "unit" is one output row of
// one group (one gate row + one up row, or one down row). The unit space is split evenly over a
// fixed grid; every block walks a contiguous unit range, so each wave streams whole weight rows
// with 16-byte loads per lane (a wave covers 1 KiB of a row per load instruction), dequantizes in
// registers and keeps one FP32 accumulator per (row-of-group, matrix), reduced across the wave at
// the end of the unit. Activations of the group live in LDS. The loads of the next unit are issued
// before the arithmetic of the current one, so every wave always has a full weight row in flight.
//
// Arithmetic (FFMOE_ACT_BF16): effective weight = bf16(decode(code) * scale) as in the reference's
// CPU path (src/fp8.rs:138-145), FP32 accumulation, BF16 boundaries at gate, up, SiLU, product,
// down and weighted contribution (src/cpu/expert_ffn.rs:592-679; kernels/moe_ffn.cu:198-209,293-301).
#include "gemv.cuh"
#include "api.h"
#include "decode.h"

namespace ffmoe {

// ---------------------------------------------------------------------------------------------
// group descriptors
__device__ __forceinline__ void make_group(GroupDesc& gd, const DecodeParams& p, int g) {
  if (p.groups) { gd = p.groups[g]; return; }
  // ungrouped: one group per assignment, then one per shared row
  const int A = p.rows * p.top_k;
  gd.n = 1;
  if (g < A) {
    gd.expert = p.ids[g];
    gd.row[0] = g / p.top_k;
    gd.slot[0] = g;
    if (p.active && p.active[g] == 0u) gd.n = 0;
    if (p.valid && (unsigned)gd.expert < (unsigned)p.experts && p.valid[gd.expert] == 0u) gd.n = 0;
    if ((unsigned)gd.expert >= (unsigned)p.experts) gd.n = 0;  // out-of-range id: contribute nothing, done stays 0
  } else {
    gd.expert = -1;
    gd.row[0] = g - A;
    gd.slot[0] = g;
  }
}

__device__ __forceinline__ int uni(int v) { return __builtin_amdgcn_readfirstlane(v); }

// STAGE 0: gate/up + SwiGLU -> h[slot, j].   STAGE 1: down (+ routing weight) -> contributions / shared_out.
// A unit is NR consecutive output rows of one group: stage 0 streams NR gate rows and the NR matching up rows
// (2*NR weight rows sharing every activation read), stage 1 streams NR down rows.
//
// Every quantity that decides an address (group, expert, row index, slab) is held wave-uniform in scalar
// registers, so weight loads take a scalar base plus one per-lane offset. A wave owns a contiguous run of
// units of the segment; reduced sums of up to 64 units are parked one per lane and the epilogue (SwiGLU or
// weighting, BF16 rounding, store) runs once per 64 units with coalesced stores.
template <class F, int S, int STAGE, int RG, int NR>
__global__ __launch_bounds__(256) void k_decode_stage(const DecodeParams p) {
  constexpr int NROWS = STAGE == 0 ? 2 * NR : NR;
  constexpr int NW = 4;
  extern __shared__ __align__(16) uint8_t xs[];
  __shared__ GroupDesc s_gd;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = uni(tid >> 6);
  const int A = p.rows * p.top_k;
  const int n_routed = p.counters ? p.counters[0] : A;
  const int n_shared = p.counters ? p.counters[1] : (p.has_shared ? p.rows : 0);
  // units per group
  const int out_r = (STAGE == 0 ? p.inter : p.hidden) / NR;
  const int out_s = (STAGE == 0 ? p.shared_inter : p.hidden) / NR;
  const long long routed_units = (long long)n_routed * out_r;
  const long long total = routed_units + (long long)n_shared * out_s;
  const long long lo = total * blockIdx.x / gridDim.x, hi = total * (blockIdx.x + 1) / gridDim.x;
  long long u0 = lo;
  while (u0 < hi) {
    // group segment containing u0
    int g, j0, width;
    if (u0 < routed_units) { g = int(u0 / out_r); j0 = int(u0 % out_r); width = out_r; }
    else { const long long v = u0 - routed_units; g = n_routed + int(v / out_s); j0 = int(v % out_s); width = out_s; }
    const long long seg_end = u0 + (width - j0) < hi ? u0 + (width - j0) : hi;
    const int count = int(seg_end - u0);
    __syncthreads();  // previous segment's readers are done with xs and s_gd
    if (tid == 0) make_group(s_gd, p, g);
    __syncthreads();
    const int expert = uni(s_gd.expert);
    const int gn = uni(s_gd.n);
    int grow[RG], gslot[RG];
#pragma unroll
    for (int r = 0; r < RG; ++r) { grow[r] = uni(s_gd.row[r]); gslot[r] = uni(s_gd.slot[r]); }
    const bool shared = expert < 0;
    const int Kg = STAGE == 0 ? p.hidden : (shared ? p.shared_inter : p.inter);
    if (gn > 0) {
      // activations of the group -> LDS (row r at r*Kg*2)
      const uint16_t* src = STAGE == 0 ? p.x : p.h;
      const int row_words = Kg >> 3;  // 16-byte words per row
#pragma unroll
      for (int r = 0; r < RG; ++r) {
        if (r < gn) {
          const size_t base = STAGE == 0 ? size_t(grow[r]) * p.hidden : size_t(gslot[r]) * p.h_stride;
          u32x4* d4 = reinterpret_cast<u32x4*>(xs + size_t(r) * Kg * 2);
          for (int v = tid; v < row_words; v += 256) d4[v] = load16(src + base + size_t(v) * 8);
        }
      }
    }
    __syncthreads();
    if (gn > 0) {
      // weight row m of a unit comes from matrix m / NR (stage 0: gate, up; stage 1: down). The six addresses are
      // fetched through scalar-friendly paths (kernel argument or global table), never through a generic pointer.
      uint64_t sl[6];
      float gl3[3];
      if (shared) {
#pragma unroll
        for (int i = 0; i < 6; ++i) sl[i] = p.shared_slot[i];
#pragma unroll
        for (int i = 0; i < 3; ++i) gl3[i] = p.shared_global[i];
      } else {
#pragma unroll
        for (int i = 0; i < 6; ++i) sl[i] = load_global<uint64_t>(p.slots + size_t(expert) * 6 + i);
#pragma unroll
        for (int i = 0; i < 3; ++i) gl3[i] = p.global_scales ? load_global<float>(p.global_scales + size_t(expert) * 3 + i) : 1.0f;
      }
      uint64_t codes[2], scales[2];
      float global[2];
      if (STAGE == 0) {
        codes[0] = sl[0]; scales[0] = sl[1]; global[0] = gl3[0];
        codes[1] = sl[2]; scales[1] = sl[3]; global[1] = gl3[1];
      } else {
        codes[0] = codes[1] = sl[4]; scales[0] = scales[1] = sl[5]; global[0] = global[1] = gl3[2];
      }
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        codes[i] = (uint64_t(uint32_t(uni(int(codes[i] >> 32)))) << 32) | uint32_t(uni(int(codes[i])));
        scales[i] = (uint64_t(uint32_t(uni(int(scales[i] >> 32)))) << 32) | uint32_t(uni(int(scales[i])));
        global[i] = __builtin_bit_cast(float, uni(__builtin_bit_cast(int, global[i])));
      }
      const int nchunks = Kg / F::EPL;
      const int nslabs = (nchunks + S * 64 - 1) / (S * 64);
      // this wave's contiguous run of units inside the segment
      const int w_lo = count * wave / NW, w_hi = count * (wave + 1) / NW;
      const int my_units = w_hi - w_lo;
      const int items = my_units * nslabs;
      const int jw = j0 + w_lo;  // first unit of the run
      UnitBuf<F, S, NROWS> bufA, bufB;
      float acc[NROWS][RG];
      float park[NROWS][RG];  // lane L keeps the sums of unit (batch base + L)
#pragma unroll
      for (int m = 0; m < NROWS; ++m)
#pragma unroll
        for (int r = 0; r < RG; ++r) { acc[m][r] = 0.0f; park[m][r] = 0.0f; }
      auto issue = [&](UnitBuf<F, S, NROWS>& b, int t) {
        const int j = (jw + t / nslabs) * NR;  // first output row of the unit
        const int chunk0 = (t % nslabs) * (S * 64);
#pragma unroll
        for (int m = 0; m < NROWS; ++m) {
          const int mat = m / NR;
          const typename F::Row rw = F::row(codes[mat], scales[mat], global[mat], j + (m % NR), Kg);
#pragma unroll
          for (int s = 0; s < S; ++s) {
            const int chunk = chunk0 + s * 64 + lane;
            F::load(b.c[m][s], rw, chunk < nchunks ? chunk : nchunks - 1);
          }
        }
      };
      // epilogue for the units [ub, ub + nu) of the run, one unit per lane
      auto flush = [&](int ub, int nu) {
        if (lane < nu) {
          const int j = (jw + ub + lane) * NR;
#pragma unroll
          for (int r = 0; r < RG; ++r) {
            if (RG == 1 || r < gn) {
              if (STAGE == 0) {
                uint16_t outv[NR];
#pragma unroll
                for (int m = 0; m < NR; ++m)
                  outv[m] = swiglu_bf16(bround(park[m][r]), bround(park[NR + m][r]), p.swiglu, p.swiglu_limit);
                uint16_t* dst = p.h + size_t(gslot[r]) * p.h_stride + j;
#pragma unroll
                for (int m = 0; m < NR; ++m) dst[m] = outv[m];
              } else if (shared) {
                uint16_t* dst = p.shared_out + size_t(grow[r]) * p.hidden + j;
                if (NR == 4) {
                  u32x2 o = {pack_bf16x2(park[0][r], park[1][r]), pack_bf16x2(park[2 % NR][r], park[3 % NR][r])};
                  *reinterpret_cast<u32x2*>(dst) = o;
                } else {
#pragma unroll
                  for (int m = 0; m < NR; ++m) dst[m] = f32_to_bf16(park[m][r]);
                }
              } else {
                const int a = gslot[r];
                const float wk = p.weights_f32 ? reinterpret_cast<const float*>(p.weights)[a]
                                               : bf16_to_f32(reinterpret_cast<const uint16_t*>(p.weights)[a]);
                float v[NR];
#pragma unroll
                for (int m = 0; m < NR; ++m) {
                  const float d = p.routed_weight == FFMOE_WEIGHT_AFTER_DOWN_BF16 ? bround(park[m][r]) : park[m][r];
                  v[m] = __fmul_rn(d, wk);
                }
                uint16_t* dst = p.contributions + size_t(a) * p.hidden + j;
                if (NR == 4) {
                  u32x2 o = {pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2 % NR], v[3 % NR])};
                  *reinterpret_cast<u32x2*>(dst) = o;
                } else {
#pragma unroll
                  for (int m = 0; m < NR; ++m) dst[m] = f32_to_bf16(v[m]);
                }
                if (j == 0 && p.done) p.done[a] = 1u;
              }
            }
          }
        }
      };
      auto finish = [&](const UnitBuf<F, S, NROWS>& b, int t) {
        const int unit = t / nslabs, slab = t % nslabs;
        slab_compute<F, S, NROWS, RG>(b, xs, Kg, nchunks, slab * (S * 64), gn, lane, acc);
        if (slab != nslabs - 1) return;
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
      int t = 0;
      if (t < items) issue(bufA, t);
      while (t < items) {
        if (t + 1 < items) issue(bufB, t + 1);
        finish(bufA, t);
        if (++t >= items) break;
        if (t + 1 < items) issue(bufA, t + 1);
        finish(bufB, t);
        ++t;
      }
      if (my_units & 63) flush(my_units & ~63, my_units & 63);
    }
    u0 = seg_end;
  }
}

// ---------------------------------------------------------------------------------------------
// Gather assignments by expert into groups of at most RGMAX rows (single block; A <= FFMOE_DECODE_MAX_ASSIGN).
// Groups are ordered by expert id, rows inside a group by assignment index, so the result does not
// depend on scheduling. counters[0] = routed groups, counters[1] = shared groups.
__global__ __launch_bounds__(1024) void k_group_assignments(const int* __restrict__ ids, const uint32_t* __restrict__ active,
                                                            const uint32_t* __restrict__ valid,
                                                            GroupDesc* __restrict__ groups, int* __restrict__ counters,
                                                            int rows, int top_k, int experts, int has_shared, int rgmax) {
  extern __shared__ int s_ids[];  // [A] expert id or -1
  __shared__ int s_scan[FFMOE_MAX_EXPERTS];
  const int tid = threadIdx.x;
  const int A = rows * top_k;
  for (int a = tid; a < A; a += blockDim.x) {
    int e = (!active || active[a]) ? ids[a] : -1;
    if ((unsigned)e >= (unsigned)experts || (valid && valid[e] == 0u)) e = -1;
    s_ids[a] = e;
  }
  __syncthreads();
  int cnt = 0;
  if (tid < experts)
    for (int a = 0; a < A; ++a) cnt += s_ids[a] == tid;
  const int chunks = (cnt + rgmax - 1) / rgmax;
  // inclusive scan over experts (blockDim == 1024 >= experts)
  s_scan[tid] = tid < experts ? chunks : 0;
  __syncthreads();
  for (int off = 1; off < 1024; off <<= 1) {
    const int v = tid >= off ? s_scan[tid - off] : 0;
    __syncthreads();
    s_scan[tid] += v;
    __syncthreads();
  }
  const int base = s_scan[tid] - chunks;
  const int n_routed = s_scan[1023];
  if (tid < experts && cnt > 0) {
    int filled = 0, gi = base;
    for (int a = 0; a < A; ++a) {
      if (s_ids[a] != tid) continue;
      GroupDesc& gd = groups[gi];
      if (filled == 0) { gd.expert = tid; gd.n = cnt - (gi - base) * rgmax < rgmax ? cnt - (gi - base) * rgmax : rgmax; }
      gd.row[filled] = a / top_k;
      gd.slot[filled] = a;
      if (++filled == rgmax) { filled = 0; ++gi; }
    }
  }
  const int n_shared = has_shared ? (rows + rgmax - 1) / rgmax : 0;
  for (int t = tid; t < n_shared; t += blockDim.x) {
    GroupDesc& gd = groups[n_routed + t];
    gd.expert = -1;
    const int r0 = t * rgmax;
    gd.n = rows - r0 < rgmax ? rows - r0 : rgmax;
    for (int r = 0; r < gd.n; ++r) { gd.row[r] = r0 + r; gd.slot[r] = A + r0 + r; }
  }
  if (tid == 0) { counters[0] = n_routed; counters[1] = n_shared; }
}

}  // namespace ffmoe

using namespace ffmoe;

namespace {

int g_cus = 0;
int num_cus() {
  if (g_cus == 0) {
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) == hipSuccess && hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && n > 0)
      g_cus = n;
    else
      g_cus = 256;
  }
  return g_cus;
}

// Launch shapes. S = 16-byte loads per lane and weight row in flight per buffer (two buffers per wave): a row
// needs ceil(K / (64 * EPL)) steps; with one row of the group per pass (RG == 1) up to 8 steps go in one slab so
// a whole row is prefetched at once, with several rows per pass the slab is capped at 4 steps to bound registers.
// NR = output rows per unit: stage 0 streams 2*NR rows of `hidden` elements, stage 1 NR rows of `inter`.
template <class F, int STAGE, int RG, int NR, int S>
void launch_one(const DecodeParams& p, int blocks, size_t lds, hipStream_t st) {
  hipLaunchKernelGGL((k_decode_stage<F, S, STAGE, RG, NR>), dim3(blocks), dim3(256), lds, st, p);
}

template <class F, int STAGE>
int launch_stage(const DecodeParams& p, int rg, hipStream_t st) {
  const int kr = STAGE == 0 ? p.hidden : p.inter;
  const int ks = STAGE == 0 ? p.hidden : (p.has_shared ? p.shared_inter : p.inter);
  const int kmax = kr > ks ? kr : ks;
  const size_t lds = size_t(rg) * kmax * 2;
  const int blocks = num_cus() * 2;
  constexpr int NR = STAGE == 0 ? 1 : 4;
  const int steps = (kmax / F::EPL + 63) / 64;
  if (rg == 1) {
    const int nslabs = (steps + 7) / 8;
    const int S = (steps + nslabs - 1) / nslabs;
    switch (S) {
      case 1: launch_one<F, STAGE, 1, NR, 1>(p, blocks, lds, st); break;
      case 2: launch_one<F, STAGE, 1, NR, 2>(p, blocks, lds, st); break;
      case 3: launch_one<F, STAGE, 1, NR, 3>(p, blocks, lds, st); break;
      case 4: launch_one<F, STAGE, 1, NR, 4>(p, blocks, lds, st); break;
      case 5: launch_one<F, STAGE, 1, NR, 5>(p, blocks, lds, st); break;
      case 6: launch_one<F, STAGE, 1, NR, 6>(p, blocks, lds, st); break;
      case 7: launch_one<F, STAGE, 1, NR, 7>(p, blocks, lds, st); break;
      default: launch_one<F, STAGE, 1, NR, 8>(p, blocks, lds, st); break;
    }
  } else {
    if (steps == 1) launch_one<F, STAGE, FFMOE_DECODE_RG, NR, 1>(p, blocks, lds, st);
    else if (steps == 2) launch_one<F, STAGE, FFMOE_DECODE_RG, NR, 2>(p, blocks, lds, st);
    else launch_one<F, STAGE, FFMOE_DECODE_RG, NR, 4>(p, blocks, lds, st);
  }
  return ff_launch_status();
}

}  // namespace

extern "C" __attribute__((visibility("default"))) uint64_t ffmoe_decode_scratch_bytes(int rows, int top_k, int experts, int hidden, int inter, int shared_inter) {
  (void)hidden;
  if (rows < 1 || top_k < 1 || experts < 1 || inter < 1) return 0;
  const uint64_t A = uint64_t(rows) * top_k;
  const uint64_t imax = uint64_t(inter > shared_inter ? inter : shared_inter);
  const uint64_t h = ((A + rows) * imax * 2 + 255) & ~uint64_t(255);
  (void)experts;
  const uint64_t max_groups = A + rows + 2;  // worst case: one row per group
  const uint64_t groups = (max_groups * sizeof(GroupDesc) + 255) & ~uint64_t(255);
  return h + groups + 256;
}

static int decode_impl(const ffmoe_expert_table* table, const ffmoe_shared_expert* shared, const ffmoe_decode* args,
                       int stage_mask, void* stream) {
  FF_REQUIRE(table && args, FFMOE_ERR_NULL, "table/args is NULL");
  const int R = args->rows, K = args->top_k, E = table->experts, H = table->hidden, I = table->inter;
  FF_REQUIRE(R >= 1 && K >= 1 && K <= FFMOE_MAX_TOP_K && E >= 1 && E <= FFMOE_MAX_EXPERTS, FFMOE_ERR_SHAPE,
             "decode rows=%d top_k=%d experts=%d out of range", R, K, E);
  FF_REQUIRE((long long)R * K <= FFMOE_DECODE_MAX_ASSIGN, FFMOE_ERR_SHAPE,
             "decode handles at most %d assignments per call (got %lld); use ffmoe_prefill_contribute", FFMOE_DECODE_MAX_ASSIGN,
             (long long)R * K);
  const int fmt = table->format;
  FF_REQUIRE(fmt == FFMOE_FMT_FP8_BLOCK128 || fmt == FFMOE_FMT_NVFP4 || fmt == FFMOE_FMT_BF16, FFMOE_ERR_UNSUPPORTED,
             "unknown expert format %d", fmt);
  // every format's granule is a multiple of 4, the largest number of output rows a wave handles per unit
  const int gran = fmt == FFMOE_FMT_FP8_BLOCK128 ? 128 : (fmt == FFMOE_FMT_NVFP4 ? 32 : 8);
  FF_REQUIRE(H >= gran && I >= gran && H % gran == 0 && I % gran == 0, FFMOE_ERR_SHAPE,
             "hidden=%d inter=%d must be positive multiples of %d for this format", H, I, gran);
  FF_REQUIRE(args->act_mode == FFMOE_ACT_BF16, FFMOE_ERR_UNSUPPORTED,
             "decode act_mode %d is not implemented (only FFMOE_ACT_BF16)", args->act_mode);
  FF_REQUIRE(args->swiglu >= 0 && args->swiglu <= 3, FFMOE_ERR_UNSUPPORTED, "unknown SwiGLU mode %d", args->swiglu);
  if (args->swiglu >= 2)
    FF_REQUIRE(args->swiglu_limit > 0.0f && args->swiglu_limit < INFINITY, FFMOE_ERR_SHAPE, "invalid SwiGLU limit %g",
               (double)args->swiglu_limit);
  FF_REQUIRE(args->routed_weight == 0 || args->routed_weight == 1, FFMOE_ERR_UNSUPPORTED, "unknown routed-weight boundary %d",
             args->routed_weight);
  FF_PTR16(args->x); FF_PTR4(args->ids); FF_PTR16(args->contributions); FF_PTR16(table->slots);
  if (args->weights_f32) { FF_PTR4(args->weights); } else { FF_PTR2(args->weights); }
  if (fmt == FFMOE_FMT_NVFP4) FF_PTR4(table->global_scales);
  int SI = I;
  if (shared) {
    FF_REQUIRE(shared->format == fmt, FFMOE_ERR_UNSUPPORTED, "shared expert format %d differs from the table format %d",
               shared->format, fmt);
    SI = shared->inter;
    FF_REQUIRE(SI >= gran && SI % gran == 0, FFMOE_ERR_SHAPE, "shared inter=%d must be a positive multiple of %d", SI, gran);
    FF_PTR16(args->shared_out);
    for (int i = 0; i < 6; i += 2)
      FF_REQUIRE(shared->slot[i] != 0 && shared->slot[i] % 16 == 0, FFMOE_ERR_ALIGN, "shared expert slot[%d] is NULL or misaligned", i);
  }
  const uint64_t need = ffmoe_decode_scratch_bytes(R, K, E, H, I, shared ? SI : 0);
  FF_PTR_ALIGNED(args->scratch, 256);
  FF_REQUIRE(args->scratch_bytes >= need, FFMOE_ERR_SCRATCH, "decode scratch holds %llu bytes, %llu needed",
             (unsigned long long)args->scratch_bytes, (unsigned long long)need);
  const size_t A = size_t(R) * K;
  const size_t xb = size_t(R) * H * 2, cb = A * H * 2;
  FF_NO_OVERLAP(args->contributions, cb, args->x, xb);
  FF_NO_OVERLAP(args->contributions, cb, args->ids, A * 4);
  FF_NO_OVERLAP(args->contributions, cb, args->weights, A * (args->weights_f32 ? 4 : 2));
  FF_NO_OVERLAP(args->contributions, cb, args->scratch, args->scratch_bytes);
  FF_NO_OVERLAP(args->scratch, args->scratch_bytes, args->x, xb);
  if (shared) {
    FF_NO_OVERLAP(args->shared_out, xb, args->x, xb);
    FF_NO_OVERLAP(args->shared_out, xb, args->contributions, cb);
    FF_NO_OVERLAP(args->shared_out, xb, args->scratch, args->scratch_bytes);
  }
  if (args->done) {
    FF_PTR4(args->done);
    FF_NO_OVERLAP(args->done, A * 4, args->contributions, cb);
    FF_NO_OVERLAP(args->done, A * 4, args->scratch, args->scratch_bytes);
  }

  const int imax = I > SI ? I : SI;
  const int kmax_lds = H > imax ? H : imax;
  FF_REQUIRE(size_t(kmax_lds) * 2 <= 160 * 1024 / 2, FFMOE_ERR_SHAPE, "row of %d BF16 does not fit the LDS staging", kmax_lds);

  DecodeParams p;
  p.rows = R; p.top_k = K; p.experts = E; p.hidden = H; p.inter = I; p.shared_inter = SI;
  p.has_shared = shared ? 1 : 0;
  p.swiglu = args->swiglu; p.swiglu_limit = args->swiglu_limit; p.routed_weight = args->routed_weight;
  p.weights_f32 = args->weights_f32;
  p.x = (const uint16_t*)args->x; p.ids = args->ids; p.active = args->active; p.weights = args->weights;
  p.slots = table->slots; p.valid = table->valid; p.global_scales = table->global_scales;
  for (int i = 0; i < 6; ++i) p.shared_slot[i] = shared ? shared->slot[i] : 0;
  for (int i = 0; i < 3; ++i) p.shared_global[i] = shared ? shared->global_scales[i] : 1.0f;
  p.contributions = (uint16_t*)args->contributions; p.shared_out = (uint16_t*)args->shared_out; p.done = args->done;
  uint8_t* sc = (uint8_t*)args->scratch;
  p.h = (uint16_t*)sc;
  p.h_stride = imax;
  const uint64_t hbytes = ((uint64_t(A) + R) * imax * 2 + 255) & ~uint64_t(255);
  hipStream_t st = (hipStream_t)stream;
  int rg = 1;
  // LDS budget per block: rg rows of the widest contraction; two blocks per CU must fit in 160 KiB
  if (R > 1) {
    rg = FFMOE_DECODE_RG;
    while (rg > 1 && size_t(rg) * kmax_lds * 2 > 64 * 1024) rg >>= 1;
  }
  if (rg > 1) {
    p.groups = (GroupDesc*)(sc + hbytes);
    const uint64_t max_groups = uint64_t(A) + R + 2;
    p.counters = (int*)(sc + hbytes + ((max_groups * sizeof(GroupDesc) + 255) & ~uint64_t(255)));
    if (stage_mask & 1) hipLaunchKernelGGL(k_group_assignments, dim3(1), dim3(1024), A * sizeof(int), st, args->ids, args->active, table->valid, p.groups,
                       p.counters, R, K, E, p.has_shared, rg);
    FF_TRY(ff_launch_status());
  } else {
    p.groups = nullptr;
    p.counters = nullptr;
  }
  switch (fmt) {
    case FFMOE_FMT_FP8_BLOCK128:
      if (stage_mask & 1) FF_TRY((launch_stage<FmtFp8, 0>(p, rg, st)));
      if (stage_mask & 2) FF_TRY((launch_stage<FmtFp8, 1>(p, rg, st)));
      break;
    case FFMOE_FMT_NVFP4:
      if (stage_mask & 1) FF_TRY((launch_stage<FmtNvfp4, 0>(p, rg, st)));
      if (stage_mask & 2) FF_TRY((launch_stage<FmtNvfp4, 1>(p, rg, st)));
      break;
    default:
      if (stage_mask & 1) FF_TRY((launch_stage<FmtBf16, 0>(p, rg, st)));
      if (stage_mask & 2) FF_TRY((launch_stage<FmtBf16, 1>(p, rg, st)));
      break;
  }
  return 0;
}

extern "C" __attribute__((visibility("default"))) int ffmoe_decode_contribute(const ffmoe_expert_table* table, const ffmoe_shared_expert* shared,
                                       const ffmoe_decode* args, void* stream) {
  return decode_impl(table, shared, args, 3, stream);
}

extern "C" __attribute__((visibility("default"))) int ffmoe_decode_contribute_stage(const ffmoe_expert_table* table, const ffmoe_shared_expert* shared,
                                             const ffmoe_decode* args, int stage, void* stream) {
  FF_REQUIRE(stage == 0 || stage == 1, FFMOE_ERR_SHAPE, "decode stage %d is neither 0 (gate/up) nor 1 (down)", stage);
  return decode_impl(table, shared, args, 1 << stage, stream);
}
