// Experts of the E8M0 block-32 contract in exact arithmetic: W4A8 routed experts (E2M1 weights, one E8M0 scale per 32
// elements of a row) and the W8A8 shared expert (E4M3 weights, one E8M0 scale per 32x32 block), activations quantized
// on the fly to E4M3 with one E8M0 scale per 32 elements (kernels/q38_contract.cuh:53-101,140-170 and
// kernels/moe_ffn.cu:398-700 of the reference: moe_act_quant_e4m0, moe_ffn_dispatch_{gate_up,down}_e2m1_e8m0_exact,
// moe_ffn_{gate_up,down}_e4m3_block32_exact).
//
// Contract. Every operand is an integer times a power of two (E4M3 = av * 2^-9, E2M1 = bv * 2^-1), so the dot of a
// 32-element group is an exact integer; the groups are accumulated in ascending order by
// total = fma(double(sum), 2^(sa + sb - bias), total) and the total takes one BF16 rounding with the FP32 double-rounding
// tie repaired. Gate clamps from above, up on both sides, FP32 SiLU * up * routed weight, one BF16 cast; that row is
// quantized again for the down projection.
//
// Mapping. The reference gives a 32-lane warp to an output row and a lane to an element of the group; here eight lanes
// share an output row, each owning a contiguous eighth of the groups: a lane computes whole group sums (exact integers,
// order-free; for E2M1 weights as packed-byte dot products) and its own FP64 chain, and the eight totals are added at
// the end (see k_e8m0_stage for why that is the reference's result).
#pragma once
#include "decode_kernel.cuh"

namespace ffmoe {

struct E8m0Params {
  DecodeParams d;          // rows, top_k, ids, active, slots, valid, weights (f32), h (BF16 down inputs), outputs
  const uint8_t* xq;       // [rows, hidden] E4M3 codes of the tokens
  const uint8_t* xs;       // [rows, hidden / 32] E8M0 scales
  uint8_t* hq;             // [(rows * top_k + rows), h_stride] E4M3 codes of the down inputs
  uint8_t* hs;             // [(rows * top_k + rows), h_stride / 32]
};

// E4M3 code -> signed integer multiple of 2^-9 (q38_contract.cuh:62-64)
__device__ __forceinline__ int e4m3_int(uint32_t a) {
  const uint32_t ae = (a >> 3) & 15u;
  const int av = ae ? int((8u + (a & 7u)) << (ae - 1u)) : int(a & 7u);
  return (a & 0x80u) ? -av : av;
}
// E2M1 nibble -> signed integer multiple of 2^-1: magnitudes 0, 1, 2, 3, 4, 6, 8, 12 (q38_contract.cuh:68-71)
__device__ __forceinline__ int e2m1_int(uint32_t nib) {
  const uint32_t mag = nib & 7u;
  const int bv = mag < 4u ? int(mag) : int((2u | (mag & 1u)) << ((mag >> 1) - 1u));
  return (nib & 8u) ? -bv : bv;
}
// 2^exponent as FP64 (q38_contract.cuh:84-85)
__device__ __forceinline__ double pow2_f64(int exponent) {
  return __longlong_as_double((long long)(uint64_t(exponent + 1023) << 52));
}
// FP64 -> BF16 through FP32 with the double-rounding tie repaired (q38_contract.cuh:92-98)
__device__ __forceinline__ uint16_t bf16_round_f64(double value) {
  float rounded = __double2float_rn(value);
  uint32_t bits = __float_as_uint(rounded);
  if ((bits & 65535u) == 32768u && double(rounded) != value) {
    // one FP32 step towards the value: the magnitude grows when the value lies further from zero
    const bool away = (value > double(rounded)) == (rounded > 0.0f);
    bits = away ? bits + 1u : bits - 1u;
    rounded = __uint_as_float(bits);
  }
  return f32_to_bf16(rounded);
}

// One 32-element activation-quant group per half wave, a lane per element (q38_contract.cuh:153-170):
// grid (ceil(groups / 64), rows_to_quantize), block 256: four lanes per group of 32, eight elements each (one 16-byte
// load, one 8-byte store). `live` (optional) marks the rows to quantize.
__global__ __launch_bounds__(256) void k_act_quant_e8m0(const uint16_t* __restrict__ x, int x_stride, uint8_t* __restrict__ codes,
                                                        int c_stride, uint8_t* __restrict__ scales, int s_stride, int k,
                                                        const uint32_t* __restrict__ live) {
  const int row = blockIdx.y;
  if (live && live[row] == 0u) return;
  const int groups = k >> 5;
  const int group = blockIdx.x * 64 + (threadIdx.x >> 2);
  if (group >= groups) return;  // the four lanes of a group leave together
  const int part = threadIdx.x & 3;
  const u32x4 w = load16(x + size_t(row) * x_stride + size_t(group) * 32 + part * 8);
  float v[8];
#pragma unroll
  for (int q = 0; q < 4; ++q) { v[2 * q] = bf16lo(w[q]); v[2 * q + 1] = bf16hi(w[q]); }
  float amax = 0.0f;
#pragma unroll
  for (int i = 0; i < 8; ++i) amax = fmaxf(amax, fabsf(v[i]));
  amax = fmaxf(amax, __shfl_xor(amax, 1, 4));
  amax = fmaxf(amax, __shfl_xor(amax, 2, 4));
  amax = fmaxf(amax, 1e-4f);
  const uint32_t qb = __float_as_uint(__fmul_rn(amax, 1.0f / 448.0f));
  int exponent = int((qb >> 23) & 0xffu) - 127 + ((qb & 0x7fffffu) != 0u ? 1 : 0);
  exponent = exponent < -127 ? -127 : (exponent > 127 ? 127 : exponent);  // the reference traps outside this range
  const float scale = __uint_as_float(uint32_t(exponent + 127) << 23);
  uint32_t out[2] = {0u, 0u};
#pragma unroll
  for (int i = 0; i < 8; ++i)
    out[i >> 2] |= uint32_t(e4m3_encode(fminf(448.0f, fmaxf(-448.0f, __fdiv_rn(v[i], scale))))) << (8 * (i & 3));
  const u32x2 o = {out[0], out[1]};
  *reinterpret_cast<u32x2*>(codes + size_t(row) * c_stride + size_t(group) * 32 + part * 8) = o;
  if (part == 0) scales[size_t(row) * s_stride + group] = uint8_t(exponent + 127);
}

// liveness of every activation slot (rows * top_k routed choices, then one per token row for the shared expert)
__global__ void k_e8m0_live(const DecodeParams p, uint32_t* __restrict__ live) {
  const int A = p.rows * p.top_k;
  const int s = blockIdx.x * blockDim.x + threadIdx.x;
  if (s >= A + p.rows) return;
  if (s >= A) { live[s] = p.has_shared ? 1u : 0u; return; }
  int expert, gn, grow[1], gslot[1];
  load_group<1>(p, s, expert, gn, grow, gslot);
  live[s] = gn > 0 ? 1u : 0u;
}

// One group of a routed (E2M1) weight row against the pre-split activations of the group: the exact integer
// sum of av * bv over 32 elements. act = 24 dwords: three planes of signed 7-bit pieces of av (av = p0 + (p1 << 7) +
// (p2 << 14)), first the 16 even elements, then the 16 odd ones, four elements per dword, so that the low nibbles of
// a weight dword (elements 8c, 8c+2, ...) and its high nibbles meet their activations as packed bytes in
// v_dot4_i32_i8. Weight magnitudes come from a byte permute over the table {0,1,2,3,4,6,8,12}.
__device__ __forceinline__ int e2m1_group_sum(const u32x4 w, const int* __restrict__ act) {
  int acc0 = 0, acc1 = 0, acc2 = 0;
#pragma unroll
  for (int c = 0; c < 4; ++c) {
    const uint32_t we = w[c], wo = w[c] >> 4;
    uint32_t be, bo;
    {
      const uint32_t mag = __builtin_amdgcn_perm(0x0C080604u, 0x03020100u, we & 0x07070707u);
      uint32_t sg = (we >> 3) & 0x01010101u;
      sg &= ((mag + 0x7f7f7f7fu) >> 7) & 0x01010101u;  // a negative zero stays zero (no carry into the next byte)
      be = (mag ^ ((sg << 8) - sg)) + sg;              // signed bytes
    }
    {
      const uint32_t mag = __builtin_amdgcn_perm(0x0C080604u, 0x03020100u, wo & 0x07070707u);
      uint32_t sg = (wo >> 3) & 0x01010101u;
      sg &= ((mag + 0x7f7f7f7fu) >> 7) & 0x01010101u;
      bo = (mag ^ ((sg << 8) - sg)) + sg;
    }
    acc0 = __builtin_amdgcn_sdot4(act[c], int(be), acc0, false);
    acc0 = __builtin_amdgcn_sdot4(act[4 + c], int(bo), acc0, false);
    acc1 = __builtin_amdgcn_sdot4(act[8 + c], int(be), acc1, false);
    acc1 = __builtin_amdgcn_sdot4(act[12 + c], int(bo), acc1, false);
    acc2 = __builtin_amdgcn_sdot4(act[16 + c], int(be), acc2, false);
    acc2 = __builtin_amdgcn_sdot4(act[20 + c], int(bo), acc2, false);
  }
  return acc0 + (acc1 << 7) + (acc2 << 14);  // |sum| < 2^27
}

// The same sum element by element from the raw codes (any operand layout): the slow path of a row whose groups span
// too many binades for an order-free FP64 sum, and the reference of the fast path in the tests.
__device__ __forceinline__ long long e8m0_group_sum_plain(bool packed, const uint8_t* __restrict__ wrow, const uint8_t* __restrict__ xcodes, int g) {
  long long sum = 0;
  for (int i = 0; i < 32; ++i) {
    const int inner = g * 32 + i;
    const int av = e4m3_int(xcodes[inner]);
    const int bv = packed ? e2m1_int((wrow[inner >> 1] >> (4 * (inner & 1))) & 15u) : e4m3_int(wrow[inner]);
    sum += (long long)av * bv;
  }
  return sum;
}

// grid (ceil(out / 8), rows, top_k + 1), block 256 = RPB output rows x SEG segments of the contraction (32 x 8 for a
// routed expert, whose blocks past ceil(out / 32) leave at once; 8 x 32 for the shared expert): lane (row, seg) sums the
// groups [G * seg / SEG, G * (seg + 1) / SEG) of its row in ascending order, the partial totals are then added. That equals the reference's one chain over all groups whenever no addition rounds, which is certain when
// sum |term| < 2^53 * (the smallest term's unit): every partial sum of the row, in any order, is then a multiple of
// that unit below 2^53 of them, i.e. exactly representable. The lanes carry sum |term| and the smallest unit and check
// it; a row that fails (block scales spanning ~26 binades or more) is recomputed by one lane in the reference's order.
// STAGE 0: gate/up exact dots -> clamped SwiGLU * routed weight -> h (BF16). STAGE 1: down exact dots -> BF16.
template <int STAGE>
__global__ __launch_bounds__(256) void k_e8m0_stage(const E8m0Params q) {
  const DecodeParams& p = q.d;
  extern __shared__ __align__(16) uint8_t lds[];
  const int tid = threadIdx.x;
  const int r = blockIdx.y, z = blockIdx.z;
  const bool is_shared = z == p.top_k;
  if (is_shared && !p.has_shared) return;
  const int A = p.rows * p.top_k;
  int expert, gn, grow[1], gslot[1];
  load_group<1>(p, is_shared ? A + r : r * p.top_k + z, expert, gn, grow, gslot);
  if (gn == 0) return;
  const bool packed = !is_shared;  // routed experts are E2M1, the shared expert E4M3 with 32x32 block scales
  const int Kg = STAGE == 0 ? p.hidden : (is_shared ? p.shared_inter : p.inter);
  const int out = STAGE == 0 ? (is_shared ? p.shared_inter : p.inter) : p.hidden;
  const int G = Kg >> 5;
  // lanes per output row: 8 for the packed-byte dot products of the routed experts, 32 for the shared expert, whose
  // E4M3 x E4M3 products need 64-bit arithmetic per element (four times the work per group)
  const int SEG = packed ? 8 : 32;
  const int RPB = 256 / SEG;  // output rows per block
  if (int(blockIdx.x) * RPB >= out) return;
  const uint8_t* xcodes = STAGE == 0 ? q.xq + size_t(r) * p.hidden : q.hq + size_t(gslot[0]) * p.h_stride;
  const uint8_t* xscales = STAGE == 0 ? q.xs + size_t(r) * (p.hidden >> 5) : q.hs + size_t(gslot[0]) * (p.h_stride >> 5);
  // activations of the token, per group: packed path 24 dwords of signed 7-bit pieces (see e2m1_group_sum), plain path
  // 32 signed integers; one more dword holds the group's scale code. The odd stride spreads the segments over banks.
  const int gstride = packed ? 25 : 33;
  int* act = reinterpret_cast<int*>(lds);
  if (packed) {
    for (int v = tid; v < G * 8; v += 256) {  // one dword of each plane per thread: four elements
      const int g = v >> 3, c = v & 7;        // c < 4: even elements 8c, 8c+2, ..; c >= 4: odd elements
      uint32_t w0 = 0, w1 = 0, w2 = 0;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int e = (c & 3) * 8 + 2 * i + (c >> 2);
        const int av = e4m3_int(xcodes[g * 32 + e]);
        const int mag = av < 0 ? -av : av;
        const int sg = av < 0 ? -1 : 1;
        w0 |= uint32_t((sg * (mag & 127)) & 0xff) << (8 * i);
        w1 |= uint32_t((sg * ((mag >> 7) & 127)) & 0xff) << (8 * i);
        w2 |= uint32_t((sg * (mag >> 14)) & 0xff) << (8 * i);
      }
      int* dst = act + size_t(g) * gstride;
      dst[c] = int(w0); dst[8 + c] = int(w1); dst[16 + c] = int(w2);
      if (c == 0) dst[24] = xscales[g];
    }
  } else {
    for (int v = tid; v < Kg; v += 256) act[size_t(v >> 5) * gstride + (v & 31)] = e4m3_int(xcodes[v]);
    for (int g = tid; g < G; g += 256) act[size_t(g) * gstride + 32] = xscales[g];
  }
  __syncthreads();
  const int j = blockIdx.x * RPB + tid / SEG;
  const int seg = tid % SEG;
  const bool row_ok = j < out;
  const int jr = row_ok ? j : out - 1;  // lanes past the end repeat the last row and store nothing
  uint64_t sl[6];
#pragma unroll
  for (int i = 0; i < 6; ++i) sl[i] = is_shared ? p.shared_slot[i] : p.slots[size_t(expert) * 6 + i];
  constexpr int NMAT = STAGE == 0 ? 2 : 1;
  const uint8_t* wrow[NMAT];
  const uint8_t* srow[NMAT];
#pragma unroll
  for (int m = 0; m < NMAT; ++m) {
    const int base = STAGE == 0 ? 2 * m : 4;
    wrow[m] = reinterpret_cast<const uint8_t*>(sl[base]) + size_t(jr) * (packed ? Kg >> 1 : Kg);
    srow[m] = reinterpret_cast<const uint8_t*>(sl[base + 1]) + size_t(packed ? jr : jr >> 5) * G;
  }
  const int bias = packed ? 264 : 272;
  const int g_lo = G * seg / SEG, g_hi = G * (seg + 1) / SEG;
  double total[NMAT], mass[NMAT];
  int emin[NMAT];
#pragma unroll
  for (int m = 0; m < NMAT; ++m) { total[m] = 0.0; mass[m] = 0.0; emin[m] = 4096; }
  auto add_group = [&](int m, int g, long long sum, int sa) {
    const int e = sa + int(srow[m][g]) - bias;
    const double scale = pow2_f64(e);
    total[m] = fma(double(sum), scale, total[m]);
    mass[m] += fabs(double(sum) * scale);
    if (sum != 0) emin[m] = e < emin[m] ? e : emin[m];
  };
  if (packed) {
    for (int g0 = g_lo; g0 < g_hi; g0 += 4) {  // four groups of weights requested together
      u32x4 w[NMAT][4];
#pragma unroll
      for (int b = 0; b < 4; ++b) {
        const int g = g0 + b < g_hi ? g0 + b : g_hi - 1;
#pragma unroll
        for (int m = 0; m < NMAT; ++m) w[m][b] = load16(wrow[m] + size_t(g) * 16);
      }
#pragma unroll
      for (int b = 0; b < 4; ++b) {
        const int g = g0 + b;
        if (g < g_hi) {
          const int* ag = act + size_t(g) * gstride;
#pragma unroll
          for (int m = 0; m < NMAT; ++m) add_group(m, g, e2m1_group_sum(w[m][b], ag), ag[24]);
        }
      }
    }
  } else {
    for (int g = g_lo; g < g_hi; ++g) {
      const int* ag = act + size_t(g) * gstride;
#pragma unroll
      for (int m = 0; m < NMAT; ++m) {
        const u32x4 w0 = load16(wrow[m] + size_t(g) * 32), w1 = load16(wrow[m] + size_t(g) * 32 + 16);
        long long sum = 0;
#pragma unroll
        for (int c = 0; c < 8; ++c) {
          const uint32_t w = c < 4 ? w0[c] : w1[c - 4];
          sum += (long long)ag[4 * c] * e4m3_int(w & 0xffu) + (long long)ag[4 * c + 1] * e4m3_int((w >> 8) & 0xffu) +
                 (long long)ag[4 * c + 2] * e4m3_int((w >> 16) & 0xffu) + (long long)ag[4 * c + 3] * e4m3_int(w >> 24);
        }
        add_group(m, g, sum, ag[32]);
      }
    }
  }
  // the eight segments of a row
#pragma unroll
  for (int m = 0; m < NMAT; ++m) {
    for (int off = 1; off < SEG; off <<= 1) {
      total[m] += __shfl_xor(total[m], off, SEG);
      mass[m] += __shfl_xor(mass[m], off, SEG);
      const int o = __shfl_xor(emin[m], off, SEG);
      emin[m] = o < emin[m] ? o : emin[m];
    }
    const bool exact = emin[m] == 4096 || mass[m] < pow2_f64(53 + emin[m]);
    if (!exact && seg == 0) {  // the reference's order, one group after the other
      double t = 0.0;
      for (int g = 0; g < G; ++g)
        t = fma(double(e8m0_group_sum_plain(packed, wrow[m], xcodes, g)), pow2_f64(int(xscales[g]) + int(srow[m][g]) - bias), t);
      total[m] = t;
    }
  }
  if (!row_ok || seg != 0) return;
  if (STAGE == 0) {
    const float g = fminf(bf16_to_f32(bf16_round_f64(total[0])), p.swiglu_limit);
    const float u = fmaxf(fminf(bf16_to_f32(bf16_round_f64(total[NMAT - 1])), p.swiglu_limit), -p.swiglu_limit);
    const float wk = is_shared ? 1.0f : reinterpret_cast<const float*>(p.weights)[gslot[0]];
    const float silu = __fdiv_rn(g, __fadd_rn(1.0f, det_expf(-g)));
    p.h[size_t(gslot[0]) * p.h_stride + j] = f32_to_bf16(__fmul_rn(__fmul_rn(silu, u), wk));
  } else {
    const uint16_t o = bf16_round_f64(total[0]);
    if (is_shared) p.shared_out[size_t(r) * p.hidden + j] = o;
    else {
      p.contributions[size_t(gslot[0]) * p.hidden + j] = o;
      if (j == 0 && p.done) p.done[gslot[0]] = 1u;
    }
  }
}

// ---------------------------------------------------------------------------------------------------------------
// The FP32-chain variant (kernels/moe_ffn.cu:469-576 W4A8, :764-865 W8A8 shared expert): the reference gives a 32-lane
// warp to an output row; here a half wave plays the warp, lane for lane, so chunk ownership, the fma chains and the
// xor-butterfly sum are the reference's and the result is bit-equal to it (up to its expf).

// E2M1 nibble -> FP32 (kernels/moe_ffn.cu:425-431)
__device__ __forceinline__ float e2m1_f32(uint32_t nibble) {
  const uint32_t u = nibble & 7u;
  uint32_t bits = 0x3F000000u + u * 0x400000u;
  bits = u == 0u ? 0u : (u == 1u ? 0x3F000000u : bits);
  return __uint_as_float(bits | ((nibble & 8u) << 28));
}
__device__ __forceinline__ float half_wave_sum(float v) {
#pragma unroll
  for (int off = 16; off > 0; off >>= 1) v = __fadd_rn(v, __shfl_xor(v, off, 32));
  return v;
}

// grid (ceil(out / 8), rows, top_k + 1), block 256 = 8 output rows x 32 lanes (the reference's launch shape).
template <int STAGE>
__global__ __launch_bounds__(256) void k_e8m0_stage_f32(const E8m0Params q) {
  const DecodeParams& p = q.d;
  extern __shared__ __align__(16) uint8_t lds[];
  const int tid = threadIdx.x;
  const int r = blockIdx.y, z = blockIdx.z;
  const bool is_shared = z == p.top_k;
  if (is_shared && !p.has_shared) return;
  const int A = p.rows * p.top_k;
  int expert, gn, grow[1], gslot[1];
  load_group<1>(p, is_shared ? A + r : r * p.top_k + z, expert, gn, grow, gslot);
  if (gn == 0) return;
  const bool packed = !is_shared;
  const int Kg = STAGE == 0 ? p.hidden : (is_shared ? p.shared_inter : p.inter);
  const int out = STAGE == 0 ? (is_shared ? p.shared_inter : p.inter) : p.hidden;
  const int G = Kg >> 5;
  if (int(blockIdx.x) * 8 >= out) return;
  // decoded activations and scales of the token
  float* xf = reinterpret_cast<float*>(lds);
  float* sxf = xf + Kg;
  {
    const uint8_t* codes = STAGE == 0 ? q.xq + size_t(r) * p.hidden : q.hq + size_t(gslot[0]) * p.h_stride;
    const uint8_t* scales = STAGE == 0 ? q.xs + size_t(r) * (p.hidden >> 5) : q.hs + size_t(gslot[0]) * (p.h_stride >> 5);
    for (int i = tid; i < Kg; i += 256) xf[i] = e4m3_to_f32(codes[i]);
    for (int i = tid; i < G; i += 256) sxf[i] = __uint_as_float(uint32_t(scales[i]) << 23);  // 2^(code - 127); code 0 is the denormal 2^-127
  }
  __syncthreads();
  const int j = blockIdx.x * 8 + (tid >> 5);
  const int lane = tid & 31;
  const bool row_ok = j < out;
  const int jr = row_ok ? j : out - 1;
  uint64_t sl[6];
#pragma unroll
  for (int i = 0; i < 6; ++i) sl[i] = is_shared ? p.shared_slot[i] : p.slots[size_t(expert) * 6 + i];
  constexpr int NMAT = STAGE == 0 ? 2 : 1;
  float acc[NMAT];
#pragma unroll
  for (int m = 0; m < NMAT; ++m) {
    const int base = STAGE == 0 ? 2 * m : 4;
    const uint8_t* wrow = reinterpret_cast<const uint8_t*>(sl[base]) + size_t(jr) * (packed ? Kg >> 1 : Kg);
    const uint8_t* srow = reinterpret_cast<const uint8_t*>(sl[base + 1]) + size_t(packed ? jr : jr >> 5) * G;
    float a = 0.0f;
    if (packed) {
      // lane L takes the 8-element chunks L, L + 32, ... (kernels/moe_ffn.cu:472-505)
      const int chunks = Kg >> 3;
      for (int chunk = lane; chunk < chunks; chunk += 32) {
        const uint32_t word = load_global<uint32_t>(wrow + size_t(chunk) * 4);
        const f32x4 x0 = *reinterpret_cast<const f32x4*>(xf + size_t(chunk) * 8), x1 = *reinterpret_cast<const f32x4*>(xf + size_t(chunk) * 8 + 4);
        const float xv[8] = {x0[0], x0[1], x0[2], x0[3], x1[0], x1[1], x1[2], x1[3]};
        float sum = 0.0f;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const uint32_t byte = (word >> (8 * i)) & 0xffu;
          sum = __fmaf_rn(e2m1_f32(byte & 0xfu), xv[2 * i], sum);
          sum = __fmaf_rn(e2m1_f32(byte >> 4), xv[2 * i + 1], sum);
        }
        const int group = chunk >> 2;
        const float sw = __uint_as_float(uint32_t(srow[group]) << 23);
        a = __fmaf_rn(sum, __fmul_rn(sxf[group], sw), a);
      }
    } else {
      // eight K blocks per pass, a block split over four lanes of eight elements (kernels/moe_ffn.cu:768-797)
      const int sub = lane & 3, stride = lane >> 2;
      for (int base_g = 0; base_g < G; base_g += 8) {
        const int block = base_g + stride;
        float sum = 0.0f;
        if (block < G) {
          const u32x2 w = load_global<u32x2>(wrow + size_t(block) * 32 + sub * 8);
          const float* xa = xf + size_t(block) * 32 + sub * 8;
#pragma unroll
          for (int i = 0; i < 8; ++i) sum = __fmaf_rn(e4m3_to_f32(uint8_t((w[i >> 2] >> (8 * (i & 3))) & 0xffu)), xa[i], sum);
        }
        sum = __fadd_rn(sum, __shfl_xor(sum, 1, 4));
        sum = __fadd_rn(sum, __shfl_xor(sum, 2, 4));
        if (sub == 0 && block < G) a = __fmaf_rn(sum, __fmul_rn(sxf[block], __uint_as_float(uint32_t(srow[block]) << 23)), a);
      }
    }
    acc[m] = half_wave_sum(a);
  }
  if (!row_ok || lane != 0) return;
  if (STAGE == 0) {
    const float g = fminf(bround(acc[0]), p.swiglu_limit);
    const float u = fmaxf(fminf(bround(acc[NMAT - 1]), p.swiglu_limit), -p.swiglu_limit);
    const float silu = __fdiv_rn(g, __fadd_rn(1.0f, det_expf(-g)));
    const float prod = __fmul_rn(silu, u);
    p.h[size_t(gslot[0]) * p.h_stride + j] = f32_to_bf16(is_shared ? prod : __fmul_rn(prod, reinterpret_cast<const float*>(p.weights)[gslot[0]]));
  } else {
    const uint16_t o = f32_to_bf16(acc[0]);
    if (is_shared) p.shared_out[size_t(r) * p.hidden + j] = o;
    else {
      p.contributions[size_t(gslot[0]) * p.hidden + j] = o;
      if (j == 0 && p.done) p.done[gslot[0]] = 1u;
    }
  }
}

}  // namespace ffmoe
