// Standalone linears y[M,N] = x[M,K] W[N,K]^T for block-scaled FP8, NVFP4 and BF16 weights
// (W8A16 / W4A16 arithmetic: BF16-rounded effective weights, FP32 accumulation, BF16 output),
// the per-128 E4M3 activation quantizer and the elementwise SwiGLU.
#include "gemv.cuh"
#include "api.h"
#include <cstdlib>

namespace ffmoe {

struct LinearParams {
  const uint16_t* x;   // [m, k] BF16
  uint16_t* y;         // [m, n] BF16
  uint64_t codes, scales;
  const float* global; // device pointer (NVFP4) or NULL
  int m, n, k;
};

// Each block walks a contiguous range of output columns and each wave a contiguous run of it, streaming one
// weight row at a time against up to RG activation rows held in LDS; rows beyond RG are served by further
// passes. One register buffer of S steps per wave: step s of the next item is requested as soon as step s of
// the current one has been consumed.
// NR: weight rows per unit (they share every activation chunk read from LDS, and NR x S KiB per wave are in flight).
template <class F, int S, int RG, int NR = 1>
__global__ __launch_bounds__(256) void k_linear(const LinearParams p) {
  constexpr int NW = 4;
  extern __shared__ __align__(16) uint8_t xs[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int K = p.k;
  const long long lo = (long long)p.n * blockIdx.x / gridDim.x, hi = (long long)p.n * (blockIdx.x + 1) / gridDim.x;
  const int count = int(hi - lo);
  const float global = p.global ? load_global<float>(p.global) : 1.0f;
  const int nchunks = K / F::EPL;
  const int nslabs = (nchunks + S * 64 - 1) / (S * 64);
  const int w_lo = count * wave / NW, w_hi = count * (wave + 1) / NW;
  const int my_rows = w_hi - w_lo;
  const int my_units = (my_rows + NR - 1) / NR;
  const int items = my_units * nslabs;
  const int jw = int(lo) + w_lo;
  // NVFP4: the split dot's constants per scale code (one global scale per matrix); the first barrier below publishes it
  constexpr bool NV = std::is_same<F, FmtNvfp4>::value;
  __shared__ u32x2 s_lut[NV ? FmtNvfp4::LUT_ENTRIES : 1];
  if constexpr (NV) FmtNvfp4::build_lut(s_lut, global, tid, 256);
  for (int r0 = 0; r0 < p.m; r0 += RG) {
    const int n = p.m - r0 < RG ? p.m - r0 : RG;
    typename F::Chunk buf[NR][S];
    auto issue_step = [&](int t, int s) {
      const int chunk = (t % nslabs) * (S * 64) + s * 64 + lane;
#pragma unroll
      for (int w = 0; w < NR; ++w) {
        const int jr = (t / nslabs) * NR + w;  // a ragged last unit repeats the wave's last row
        F::load(buf[w][s], F::row(p.codes, p.scales, global, jw + (jr < my_rows ? jr : my_rows - 1), K), chunk < nchunks ? chunk : nchunks - 1);
      }
    };
    if (items > 0) {
#pragma unroll
      for (int s = 0; s < S; ++s) issue_step(0, s);
    }
    __syncthreads();
    {
      u32x4* d4 = reinterpret_cast<u32x4*>(xs);
      const int words = n * (K >> 3);
      for (int v = tid; v < words; v += 256) d4[v] = load16(p.x + size_t(r0) * K + size_t(v) * 8);
    }
    __syncthreads();
    if (items > 0) {
      float acc[NR][RG];
#pragma unroll
      for (int w = 0; w < NR; ++w)
#pragma unroll
        for (int r = 0; r < RG; ++r) acc[w][r] = 0.0f;
      auto compute_step = [&](int t, int s) {
        const int chunk = (t % nslabs) * (S * 64) + s * 64 + lane;
        step_compute<F, NR, RG, S, NV>(buf, s, xs, K, nchunks, chunk, n, acc, s_lut, s_lut, NR);
      };
      auto item_end = [&](int t) {
        if (t % nslabs != nslabs - 1) return;
#pragma unroll
        for (int w = 0; w < NR; ++w) {
          const int jr = (t / nslabs) * NR + w;
#pragma unroll
          for (int r = 0; r < RG; ++r) {
            if (RG == 1 || r < n) {
              const float total = wave_sum(acc[w][r]);
              if (lane == r && jr < my_rows) p.y[size_t(r0 + r) * p.n + jw + jr] = f32_to_bf16(total);
            }
            acc[w][r] = 0.0f;
          }
        }
      };
      for (int t = 0; t + 1 < items; ++t) {
#pragma unroll
        for (int s = 0; s < S; ++s) {
          compute_step(t, s);
          issue_step(t + 1, s);
        }
        item_end(t);
      }
#pragma unroll
      for (int s = 0; s < S; ++s) compute_step(items - 1, s);
      item_end(items - 1);
    }
  }
}

// Several independent skinny linears of one shape in ONE launch (the projections a decoder layer applies side by side):
// the rows of all items form one unit space that is split evenly over the grid, so a call's start-up and tail are paid
// once per batch instead of once per matrix; a 14.7 MB matrix alone streams for about 2.3 us against 2 - 3 us of
// start-up. Per row the arithmetic is k_linear's (same chunk -> lane mapping, step order and wave reduction), so every
// item's y is bit-identical to its own ffmoe_linear_* call.
struct LinearItem { uint64_t codes, scales, x, y; };  // device addresses of one item's operands

struct LinearBatchParams {
  const LinearItem* items;  // device [count]
  const float* global;      // NVFP4: device [count] global scales, else NULL
  int count, m, n, k;
};

// NR: weight rows per unit. With several activation rows a unit of two weight rows reads every activation chunk from LDS
// once for both (the LDS pipe, not the weight stream, is what four activation rows per weight row load).
template <class F, int S, int RG, int NR = 1>
__global__ __launch_bounds__(256) void k_linear_batch(const LinearBatchParams p) {
  constexpr int NW = 4;
  extern __shared__ __align__(16) uint8_t xs[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = uni(tid >> 6);
  const int K = p.k, N = p.n;
  const long long total = (long long)p.count * N;
  const long long lo = total * blockIdx.x / gridDim.x, hi = total * (blockIdx.x + 1) / gridDim.x;
  const int nchunks = K / F::EPL;
  const int nslabs = (nchunks + S * 64 - 1) / (S * 64);
  long long u0 = lo;
  while (u0 < hi) {
    const int item = int(u0 / N), j0 = int(u0 % N);
    const long long seg_end = u0 + (N - j0) < hi ? u0 + (N - j0) : hi;
    const int count = int(seg_end - u0);
    const uint64_t* it = reinterpret_cast<const uint64_t*>(p.items + item);
    const uint64_t codes = uni64(load_global<uint64_t>(it)), scales = uni64(load_global<uint64_t>(it + 1));
    const uint16_t* x = reinterpret_cast<const uint16_t*>(uni64(load_global<uint64_t>(it + 2)));
    uint16_t* y = reinterpret_cast<uint16_t*>(uni64(load_global<uint64_t>(it + 3)));
    const float global = p.global ? unif(load_global<float>(p.global + item)) : 1.0f;
    const int w_lo = count * wave / NW, w_hi = count * (wave + 1) / NW;
    const int my_rows = w_hi - w_lo;
    const int my_units = (my_rows + NR - 1) / NR;
    const int items_w = my_units * nslabs;
    const int jw = j0 + w_lo;
    typename F::Chunk buf[NR][S];
    auto issue_step = [&](int t, int s) {
      const int chunk = (t % nslabs) * (S * 64) + s * 64 + lane;
#pragma unroll
      for (int r = 0; r < NR; ++r) {
        const int jr = (t / nslabs) * NR + r;  // a ragged last unit repeats the wave's last row
        F::load(buf[r][s], F::row(codes, scales, global, jw + (jr < my_rows ? jr : my_rows - 1), K), chunk < nchunks ? chunk : nchunks - 1);
      }
    };
    if (items_w > 0) {
#pragma unroll
      for (int s = 0; s < S; ++s) issue_step(0, s);
    }
    __syncthreads();  // the previous segment's readers are done with xs
    {
      u32x4* d4 = reinterpret_cast<u32x4*>(xs);
      const int words = p.m * (K >> 3);
      for (int v = tid; v < words; v += 256) d4[v] = load16(x + size_t(v) * 8);
    }
    __syncthreads();
    if (items_w > 0) {
      float acc[NR][RG];
#pragma unroll
      for (int w = 0; w < NR; ++w)
#pragma unroll
        for (int r = 0; r < RG; ++r) acc[w][r] = 0.0f;
      auto compute_step = [&](int t, int s) {
        const int chunk = (t % nslabs) * (S * 64) + s * 64 + lane;
        step_compute<F, NR, RG, S>(buf, s, xs, K, nchunks, chunk, p.m, acc);
      };
      auto item_end = [&](int t) {
        if (t % nslabs != nslabs - 1) return;
#pragma unroll
        for (int w = 0; w < NR; ++w) {
          const int jr = (t / nslabs) * NR + w;
#pragma unroll
          for (int r = 0; r < RG; ++r) {
            if (RG == 1 || r < p.m) {
              const float sum = wave_sum(acc[w][r]);
              if (lane == r && jr < my_rows) y[size_t(r) * N + jw + jr] = f32_to_bf16(sum);
            }
            acc[w][r] = 0.0f;
          }
        }
      };
      for (int t = 0; t + 1 < items_w; ++t) {
#pragma unroll
        for (int s = 0; s < S; ++s) {
          compute_step(t, s);
          issue_step(t + 1, s);
        }
        item_end(t);
      }
#pragma unroll
      for (int s = 0; s < S; ++s) compute_step(items_w - 1, s);
      item_end(items_w - 1);
    }
    u0 = seg_end;
  }
}

// Skinny linear for up to 16 activation rows per pass on the BF16 matrix cores. The streaming kernel above pays one
// v_dot2 per weight pair and activation row and serves at most 4 (K > 4096) or 8 rows per pass over the weights; here
// the weights are dequantized once (the same BF16 effective weights, bit for bit) and a 16-row activation panel meets
// them in v_mfma_f32_16x16x32_bf16: products of BF16 values are exact in FP32, the sum is the matrix core's FP32
// accumulation, so the result differs from the FP32 fma chain only in summation order.
//
// Block = 8 waves on TR weight rows (8 rows when that is what it takes to have a block per CU; the upper half of the
// 16-row operand then repeats them and is dropped); the waves split the contraction. x goes through LDS in panels of
// at most 3584 columns x 16 rows (rows past m are zeros). A unit is 4 * EPL columns: lane (row i, group c) loads the
// 16-byte chunk 4 * unit + c of its weight row (EPL elements), which feeds EPL / 8 instructions of 8 elements each,
// and reads the matching activations of its token from LDS. The eight partial tiles are added in wave order.
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));

template <class F, int TR>
__global__ __launch_bounds__(512) void k_linear_mfma(const LinearParams p, int m0) {
  constexpr int NW = 8, PANEL = 3584, UC = 4 * F::EPL, UMAX = (PANEL / UC + NW - 1) / NW;
  extern __shared__ __align__(16) uint8_t lds[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = uni(tid >> 6);
  const int K = p.k, N = p.n;
  const int n0 = blockIdx.x * TR;
  const int mcount = p.m - m0 < 16 ? p.m - m0 : 16;
  const int i = lane & 15, c = lane >> 4;
  const float global = p.global ? load_global<float>(p.global) : 1.0f;
  const typename F::Row wrow = F::row(p.codes, p.scales, global, n0 + (i & (TR - 1)), K);
  const int panel = K < PANEL ? K : PANEL;
  const int stride = panel * 2 + 16;  // bytes per token row in LDS; the 16 spread the 16 tokens of a read over all banks
  f32x4 acc = {0.0f, 0.0f, 0.0f, 0.0f};
  typename F::Chunk wv[UMAX], wn[UMAX];
  // unconditional requests (clamped index), masked at use
  auto request = [&](int k_lo, typename F::Chunk (&wd)[UMAX]) {
    const int pk = K - k_lo < panel ? K - k_lo : panel;
    const int units = pk / UC;
    const int u_lo = units * wave / NW, u_hi = units * (wave + 1) / NW;  // at most UMAX units
#pragma unroll
    for (int u = 0; u < UMAX; ++u) {
      const int idx = u_lo + u < u_hi ? u_lo + u : (u_hi > u_lo ? u_hi - 1 : 0);
      F::load(wd[u], wrow, (k_lo + UC * idx) / F::EPL + c);
    }
  };
  request(0, wv);
  for (int k_lo = 0; k_lo < K; k_lo += panel) {
    const int pk = K - k_lo < panel ? K - k_lo : panel;
    const int units = pk / UC;
    const int u_lo = units * wave / NW, u_hi = units * (wave + 1) / NW;
    __syncthreads();  // the previous panel has been read
    {
      const int per_row = pk >> 3;
      for (int v = tid; v < 16 * per_row; v += 512) {
        const int j = v / per_row, q = v - j * per_row;
        u32x4 val = {0u, 0u, 0u, 0u};
        if (j < mcount) val = load16(p.x + size_t(m0 + j) * K + k_lo + q * 8);
        *reinterpret_cast<u32x4*>(lds + size_t(j) * stride + q * 16) = val;
      }
    }
    __syncthreads();
    const bool more = k_lo + panel < K;
    if (more) request(k_lo + panel, wn);  // the next panel's weights travel while this one is multiplied
#pragma unroll
    for (int u = 0; u < UMAX; ++u) {
      if (u_lo + u < u_hi) {
        uint32_t w[F::EPL / 2];
        F::dequant(wv[u], w, true);
        const uint8_t* xb = lds + size_t(i) * stride + size_t(UC * (u_lo + u) + F::EPL * c) * 2;
#pragma unroll
        for (int t = 0; t < F::EPL / 8; ++t) {
          const u32x4 b = *reinterpret_cast<const u32x4*>(xb + 16 * t);
          const u32x4 a = {w[4 * t], w[4 * t + 1], w[4 * t + 2], w[4 * t + 3]};
          acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), acc, 0, 0, 0);
        }
      }
    }
    if (more) {
#pragma unroll
      for (int u = 0; u < UMAX; ++u) wv[u] = wn[u];
    }
  }
  // lane (token i, group c) holds weight rows 4c .. 4c+3 of the tile; the waves' tiles are added in wave order
  __syncthreads();
  float* red = reinterpret_cast<float*>(lds);  // [wave][row 0..15][token 0..15]
#pragma unroll
  for (int r = 0; r < 4; ++r) red[(wave * 16 + 4 * c + r) * 16 + i] = acc[r];
  __syncthreads();
  if (tid < 16 * TR) {
    const int j = tid / TR, r = tid - j * TR;
    float v = red[r * 16 + j];
#pragma unroll
    for (int w = 1; w < NW; ++w) v = __fadd_rn(v, red[(w * 16 + r) * 16 + j]);
    if (j < mcount) p.y[size_t(m0 + j) * N + n0 + r] = f32_to_bf16(v);
  }
}

// Per (row, 128-group): scale = amax * (1/448), code = e4m3(clamp(x / max(scale, 1e-12), +-448))
// (kernels/fp8_linear.cu:12-48 of the reference). One wave per 4 cells, 16 lanes x 8 elements per cell.
__global__ __launch_bounds__(256) void k_quant_fp8_128(const uint16_t* __restrict__ x, uint8_t* __restrict__ codes,
                                                       float* __restrict__ scales, int m, int k) {
  const int groups = (k + 127) >> 7;
  const long long cell = (long long)blockIdx.x * 16 + (threadIdx.x >> 4);
  if (cell >= (long long)m * groups) return;  // whole 16-lane groups leave together
  const int sub = threadIdx.x & 15;
  const long long row = cell / groups;
  const int first = int(cell % groups) * 128 + sub * 8;
  float v[8];
  float amax = 0.0f;
  const uint16_t* src = x + row * k + first;
  if (first + 8 <= k) {
    const u32x4 w = load16(src);
#pragma unroll
    for (int q = 0; q < 4; ++q) { v[2 * q] = bf16lo(w[q]); v[2 * q + 1] = bf16hi(w[q]); }
  } else {
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] = first + i < k ? bf16_to_f32(src[i]) : 0.0f;
  }
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
  uint8_t* dst = codes + row * k + first;
  if (first + 8 <= k) {
    u32x2 o = {out[0], out[1]};
    *reinterpret_cast<u32x2*>(dst) = o;
  } else {
    for (int i = 0; i < 8; ++i)
      if (first + i < k) dst[i] = uint8_t(out[i >> 2] >> (8 * (i & 3)));
  }
}

// y = swiglu(gate, up), 8 elements per thread (kernels/act.cu:65-99, :125-159 of the reference).
__global__ __launch_bounds__(256) void k_swiglu(const uint16_t* __restrict__ gate, const uint16_t* __restrict__ up,
                                                uint16_t* __restrict__ y, long long vectors, int mode, float limit) {
  const long long v = (long long)blockIdx.x * 256 + threadIdx.x;
  if (v >= vectors) return;
  const u32x4 g = load16(gate + v * 8), u = load16(up + v * 8);
  u32x4 o;
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    const uint32_t lo = swiglu_bf16(bf16lo(g[q]), bf16lo(u[q]), mode, limit);
    const uint32_t hi = swiglu_bf16(bf16hi(g[q]), bf16hi(u[q]), mode, limit);
    o[q] = lo | (hi << 16);
  }
  *reinterpret_cast<u32x4*>(y + v * 8) = o;
}

}  // namespace ffmoe

using namespace ffmoe;

namespace {
int g_cus_l = 0;
int num_cus_l() {
  if (g_cus_l == 0) {
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) == hipSuccess && hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && n > 0)
      g_cus_l = n;
    else
      g_cus_l = 256;
  }
  return g_cus_l;
}

template <class F, int RG, int SMAX, int S = 1>
void launch_linear_steps(int want, const LinearParams& p, int blocks, size_t lds, hipStream_t st) {
  if constexpr (S <= SMAX) {
    if (want == S) hipLaunchKernelGGL((k_linear<F, S, RG, 1>), dim3(blocks), dim3(256), lds, st, p);
    else launch_linear_steps<F, RG, SMAX, S + 1>(want, p, blocks, lds, st);
  }
}

template <class F>
int launch_linear(const LinearParams& p, hipStream_t st) {
  // rows per pass bounded by 64 KiB of LDS
  int blocks = num_cus_l() * 2;
  if (blocks > (p.n + 3) / 4) blocks = (p.n + 3) / 4;
  const size_t row = size_t(p.k) * 2;
  // Steps of a weight row held in flight at once: slabs of at most four, the row cut into equal slabs (K 2048: two steps, no
  // masked ones). A single call is bound by its start-up - the whole row of seven steps in flight (FFMOE_LINEAR_SMAX=8; same
  // bits) measures 6.74 against 6.37 us at M = 1, K 7168, and more weight rows per unit, which pay in the batched entry, change
  // nothing or lose. NVFP4 rows hold their split-dot operands in registers and cannot take more than four.
  const int steps = (p.k / F::EPL + 63) / 64;
  constexpr int SMAX = std::is_same<F, FmtNvfp4>::value ? 4 : 8;
  int smax = 4;
  if (const char* e = getenv("FFMOE_LINEAR_SMAX")) { const int v = atoi(e); if (v >= 1 && v <= SMAX) smax = v; }
  auto steps_per_slab = [&](int cap) {  // the row in equal slabs of at most cap steps
    const int nslabs = (steps + cap - 1) / cap;
    return (steps + nslabs - 1) / nslabs;
  };
  const int S = steps_per_slab(smax);
  if (p.m > 4 && 8 * row <= 64 * 1024) launch_linear_steps<F, 8, 4>(steps_per_slab(smax < 4 ? smax : 4), p, blocks, 8 * row, st);
  else if (p.m > 1 && 4 * row <= 64 * 1024) launch_linear_steps<F, 4, SMAX>(S, p, blocks, 4 * row, st);
  else launch_linear_steps<F, 1, SMAX>(S, p, blocks, row, st);
  return ff_launch_status();
}

// the matrix-core kernel takes whole units of 4 * EPL columns
template <class F>
bool mfma_linear_fits(int k) { return k % (4 * F::EPL) == 0 && !getenv("FFMOE_LINEAR_NO_MFMA"); }

template <class F>
int launch_linear_mfma(const LinearParams& p, hipStream_t st) {
  const int panel = p.k < 3584 ? p.k : 3584;
  const size_t tile = size_t(16) * (panel * 2 + 16);
  const size_t lds = tile > 8 * 16 * 16 * 4 ? tile : 8 * 16 * 16 * 4;  // the x panel, later the eight partial tiles
  const bool wide = p.n / 16 >= num_cus_l();
  for (int m0 = 0; m0 < p.m; m0 += 16) {
    if (wide) hipLaunchKernelGGL((k_linear_mfma<F, 16>), dim3(p.n / 16), dim3(512), lds, st, p, m0);
    else hipLaunchKernelGGL((k_linear_mfma<F, 8>), dim3(p.n / 8), dim3(512), lds, st, p, m0);
  }
  return ff_launch_status();
}

int check_linear(const void* w, const void* x, const void* y, int m, int n, int k, int kgran) {
  FF_REQUIRE(m >= 1 && n >= 1 && k >= kgran && k % kgran == 0, FFMOE_ERR_SHAPE, "linear m=%d n=%d k=%d (k must be a positive multiple of %d)", m, n, k, kgran);
  FF_REQUIRE(size_t(k) * 2 <= 64 * 1024, FFMOE_ERR_SHAPE, "linear k=%d exceeds the LDS row staging (32768)", k);
  FF_PTR16(w); FF_PTR16(x); FF_PTR16(y);
  FF_NO_OVERLAP(y, size_t(m) * n * 2, x, size_t(m) * k * 2);
  return 0;
}
}  // namespace

extern "C" __attribute__((visibility("default"))) int ffmoe_quant_fp8_f32_128(const void* x, void* codes, float* scales, int m, int k, void* stream) {
  FF_REQUIRE(m >= 1 && k >= 1, FFMOE_ERR_SHAPE, "quant m=%d k=%d", m, k);
  FF_REQUIRE(k % 8 == 0, FFMOE_ERR_SHAPE, "quant k=%d must be a multiple of 8", k);
  FF_PTR16(x); FF_PTR16(codes); FF_PTR4(scales);
  const long long cells = (long long)m * ((k + 127) / 128);
  FF_NO_OVERLAP(codes, size_t(m) * k, x, size_t(m) * k * 2);
  FF_NO_OVERLAP(scales, size_t(cells) * 4, x, size_t(m) * k * 2);
  FF_NO_OVERLAP(scales, size_t(cells) * 4, codes, size_t(m) * k);
  hipLaunchKernelGGL(k_quant_fp8_128, dim3((unsigned)((cells + 15) / 16)), dim3(256), 0, (hipStream_t)stream,
                     (const uint16_t*)x, (uint8_t*)codes, scales, m, k);
  return ff_launch_status();
}

extern "C" __attribute__((visibility("default"))) int ffmoe_linear_fp8_block(const void* w_codes, const float* w_scales, const void* x, void* y, int m, int n, int k,
                                      int act_mode, void* scratch, uint64_t scratch_bytes, void* stream) {
  FF_TRY(check_linear(w_codes, x, y, m, n, k, 16));
  FF_PTR4(w_scales);
  if (act_mode == FFMOE_ACT_FP8_BLOCK128) {
    const uint64_t groups = uint64_t(k + 127) / 128;
    const uint64_t cb = (uint64_t(m) * k + 255) & ~uint64_t(255);
    FF_PTR_ALIGNED(scratch, 256);
    FF_REQUIRE(scratch_bytes >= cb + uint64_t(m) * groups * 4, FFMOE_ERR_SCRATCH, "linear scratch holds %llu bytes, %llu needed",
               (unsigned long long)scratch_bytes, (unsigned long long)(cb + uint64_t(m) * groups * 4));
    FF_TRY(ffmoe_quant_fp8_f32_128(x, scratch, (float*)((uint8_t*)scratch + cb), m, k, stream));
    return ffmoe_linear_fp8_block_w8a8(w_codes, w_scales, scratch, (const float*)((uint8_t*)scratch + cb), y, m, n, k, stream);
  }
  FF_REQUIRE(act_mode == FFMOE_ACT_BF16, FFMOE_ERR_UNSUPPORTED, "unknown act_mode %d", act_mode);
  LinearParams p{(const uint16_t*)x, (uint16_t*)y, (uint64_t)(uintptr_t)w_codes, (uint64_t)(uintptr_t)w_scales, nullptr, m, n, k};
  if (m > 4 && n % 16 == 0 && mfma_linear_fits<FmtFp8>(k)) return launch_linear_mfma<FmtFp8>(p, (hipStream_t)stream);
  return launch_linear<FmtFp8>(p, (hipStream_t)stream);
}

namespace {
template <class F, int RG, int SMAX, int NR, int S = 1>
void launch_batch_steps(int want, const LinearBatchParams& p, int blocks, size_t lds, hipStream_t st) {
  if constexpr (S <= SMAX) {
    if (want == S) hipLaunchKernelGGL((k_linear_batch<F, S, RG, NR>), dim3(blocks), dim3(256), lds, st, p);
    else launch_batch_steps<F, RG, SMAX, NR, S + 1>(want, p, blocks, lds, st);
  }
}
}  // namespace

extern "C" __attribute__((visibility("default"))) int ffmoe_linear_fp8_block_batch(const ffmoe_linear_item* items, int count, int m, int n, int k, void* stream) {
  FF_REQUIRE(count >= 1 && count <= 4096, FFMOE_ERR_SHAPE, "batch of %d linears (1 .. 4096)", count);
  FF_REQUIRE(m >= 1 && m <= 4, FFMOE_ERR_UNSUPPORTED, "batched linears take 1 .. 4 activation rows per item (m=%d): use ffmoe_linear_fp8_block", m);
  FF_REQUIRE(n >= 1 && k >= 16 && k % 16 == 0, FFMOE_ERR_SHAPE, "linear n=%d k=%d (k must be a positive multiple of 16)", n, k);
  FF_REQUIRE(size_t(m) * k * 2 <= 64 * 1024, FFMOE_ERR_SHAPE, "m=%d rows of k=%d exceed the LDS row staging", m, k);
  FF_PTR_ALIGNED(items, 8);
  static_assert(sizeof(ffmoe_linear_item) == sizeof(LinearItem), "item layout");
  LinearBatchParams p{reinterpret_cast<const LinearItem*>(items), nullptr, count, m, n, k};
  const long long total = (long long)count * n;
  int blocks = num_cus_l() * 2;
  if (blocks > (total + 3) / 4) blocks = int((total + 3) / 4);
  const int steps = (k / 16 + 63) / 64;
  int smax = 8;
  if (const char* e = getenv("FFMOE_LINEAR_BATCH_SMAX")) { const int v = atoi(e); if (v >= 1 && v <= 8) smax = v; }
  const int nslabs = (steps + smax - 1) / smax;
  const int S = (steps + nslabs - 1) / nslabs;
  const size_t lds = size_t(m) * k * 2;
  hipStream_t st = (hipStream_t)stream;
  // Weight rows per unit (bit-identical whatever it is: a row's dot product does not depend on its neighbours). One activation
  // row: what counts is bytes in flight per wave - two rows of seven steps (14 KB) at K 7168, four rows of two steps (8 KB) at
  // K 2048 (eight matrices per launch, us per matrix with 1 / 2 / 4 rows per unit: 3.00 / 2.83 / 3.43 and 4.03 / 3.11 / 2.95).
  // Several activation rows: four weight rows share every activation chunk read from LDS (M = 4: 6.61 / 4.74 / 4.31 and
  // 7.44 / 5.45 / 4.77 us; with rows of at most four steps per slab, as before, 7.51 and 7.42).
  int nr = m == 1 ? (steps >= 4 ? 2 : 4) : 4;
  if (const char* e = getenv("FFMOE_LINEAR_BATCH_NR")) { const int v = atoi(e); if (v == 1 || v == 2 || v == 4) nr = v; }
  if (m == 1 && nr == 4) launch_batch_steps<FmtFp8, 1, 8, 4>(S, p, blocks, lds, st);
  else if (m == 1 && nr == 2) launch_batch_steps<FmtFp8, 1, 8, 2>(S, p, blocks, lds, st);
  else if (m == 1) launch_batch_steps<FmtFp8, 1, 8, 1>(S, p, blocks, lds, st);
  else if (nr == 4) launch_batch_steps<FmtFp8, 4, 8, 4>(S, p, blocks, lds, st);
  else if (nr == 2) launch_batch_steps<FmtFp8, 4, 8, 2>(S, p, blocks, lds, st);
  else launch_batch_steps<FmtFp8, 4, 8, 1>(S, p, blocks, lds, st);
  return ff_launch_status();
}

extern "C" __attribute__((visibility("default"))) int ffmoe_linear_nvfp4(const void* w_codes, const void* w_scales, const float* global_scale, const void* x, void* y,
                                  int m, int n, int k, void* stream) {
  FF_TRY(check_linear(w_codes, x, y, m, n, k, 32));
  FF_PTR2(w_scales); FF_PTR4(global_scale);
  LinearParams p{(const uint16_t*)x, (uint16_t*)y, (uint64_t)(uintptr_t)w_codes, (uint64_t)(uintptr_t)w_scales, global_scale, m, n, k};
  // up to 16 rows: the direct kernel, bit-equal to the reference's host mirror; beyond, its matrix-core path (nvfp4_linear.cu:262-573)
  if (m > 16 && n % 16 == 0 && mfma_linear_fits<FmtNvfp4>(k)) return launch_linear_mfma<FmtNvfp4>(p, (hipStream_t)stream);
  return launch_linear<FmtNvfp4>(p, (hipStream_t)stream);
}

extern "C" __attribute__((visibility("default"))) int ffmoe_gemm_skinny_bf16(const void* w, const void* x, void* y, int m, int n, int k, void* stream) {
  FF_TRY(check_linear(w, x, y, m, n, k, 8));
  LinearParams p{(const uint16_t*)x, (uint16_t*)y, (uint64_t)(uintptr_t)w, 0, nullptr, m, n, k};
  if (m > 4 && n % 16 == 0 && mfma_linear_fits<FmtBf16>(k)) return launch_linear_mfma<FmtBf16>(p, (hipStream_t)stream);
  return launch_linear<FmtBf16>(p, (hipStream_t)stream);
}

extern "C" __attribute__((visibility("default"))) int ffmoe_swiglu(const void* gate, const void* up, void* y, int rows, int width, int mode, float limit, void* stream) {
  FF_REQUIRE(rows >= 1 && width >= 8 && width % 8 == 0, FFMOE_ERR_SHAPE, "swiglu rows=%d width=%d (width must be a positive multiple of 8)", rows, width);
  FF_REQUIRE(mode >= 0 && mode <= FFMOE_SWIGLU_GELU_TWICE, FFMOE_ERR_UNSUPPORTED, "unknown SwiGLU mode %d", mode);
  if (mode == FFMOE_SWIGLU_CLAMPED_TWICE || mode == FFMOE_SWIGLU_CLAMPED_ONCE) FF_REQUIRE(limit > 0.0f && limit < INFINITY, FFMOE_ERR_SHAPE, "invalid SwiGLU limit %g", (double)limit);
  FF_PTR16(gate); FF_PTR16(up); FF_PTR16(y);
  const size_t bytes = size_t(rows) * width * 2;
  FF_NO_OVERLAP(y, bytes, gate, bytes);
  FF_NO_OVERLAP(y, bytes, up, bytes);
  const long long vectors = (long long)rows * width / 8;
  hipLaunchKernelGGL(k_swiglu, dim3((unsigned)((vectors + 255) / 256)), dim3(256), 0, (hipStream_t)stream, (const uint16_t*)gate,
                     (const uint16_t*)up, (uint16_t*)y, vectors, mode, limit);
  return ff_launch_status();
}
