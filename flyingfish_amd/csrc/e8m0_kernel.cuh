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
// Mapping. The reference gives a 32-lane warp to an output row and a lane to an element of the group; here a LANE owns
// an output ROW: all 64 lanes walk the groups in step, the 32 activations of the group are the same for every lane (LDS
// broadcast reads of pre-decoded signed integers), the group sum and the FP64 chain live in the lane, and nothing is
// reduced across lanes. The result is the same by construction: integer sums are order-free, the FP64 chain is per row.
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
// grid (ceil(groups / 8), rows_to_quantize), block 256. `live` (optional) marks the rows to quantize.
__global__ __launch_bounds__(256) void k_act_quant_e8m0(const uint16_t* __restrict__ x, int x_stride, uint8_t* __restrict__ codes,
                                                        int c_stride, uint8_t* __restrict__ scales, int s_stride, int k,
                                                        const uint32_t* __restrict__ live) {
  const int row = blockIdx.y;
  if (live && live[row] == 0u) return;
  const int groups = k >> 5;
  const int group = blockIdx.x * 8 + (threadIdx.x >> 5);
  if (group >= groups) return;
  const int lane = threadIdx.x & 31;
  const float value = bf16_to_f32(x[size_t(row) * x_stride + size_t(group) * 32 + lane]);
  float amax = fabsf(value);
#pragma unroll
  for (int off = 16; off > 0; off >>= 1) amax = fmaxf(amax, __shfl_xor(amax, off, 32));
  amax = fmaxf(amax, 1e-4f);
  const uint32_t qb = __float_as_uint(__fmul_rn(amax, 1.0f / 448.0f));
  int exponent = int((qb >> 23) & 0xffu) - 127 + ((qb & 0x7fffffu) != 0u ? 1 : 0);
  exponent = exponent < -127 ? -127 : (exponent > 127 ? 127 : exponent);  // the reference traps outside this range
  const float scale = __uint_as_float(uint32_t(exponent + 127) << 23);
  codes[size_t(row) * c_stride + size_t(group) * 32 + lane] = e4m3_encode(fminf(448.0f, fmaxf(-448.0f, __fdiv_rn(value, scale))));
  if (lane == 0) scales[size_t(row) * s_stride + group] = uint8_t(exponent + 127);
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

// grid (ceil(out / 256), rows, top_k + 1), block 256: thread = output row of (token row y, choice z | shared expert).
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
  if (int(blockIdx.x) * 256 >= out) return;
  // activations of the row: signed integers (multiples of 2^-9) and scale codes, read by every lane alike
  int* avs = reinterpret_cast<int*>(lds);
  uint8_t* sxs = lds + size_t(Kg) * 4;
  {
    const uint8_t* codes = STAGE == 0 ? q.xq + size_t(r) * p.hidden : q.hq + size_t(gslot[0]) * p.h_stride;
    const uint8_t* scales = STAGE == 0 ? q.xs + size_t(r) * (p.hidden >> 5) : q.hs + size_t(gslot[0]) * (p.h_stride >> 5);
    for (int i = tid; i < Kg; i += 256) avs[i] = e4m3_int(codes[i]);
    for (int i = tid; i < G; i += 256) sxs[i] = scales[i];
  }
  __syncthreads();
  const int j = blockIdx.x * 256 + tid;
  if (j >= out) return;
  uint64_t sl[6];
#pragma unroll
  for (int i = 0; i < 6; ++i) sl[i] = is_shared ? p.shared_slot[i] : p.slots[size_t(expert) * 6 + i];
  constexpr int NMAT = STAGE == 0 ? 2 : 1;
  const uint8_t* wrow[NMAT];
  const uint8_t* srow[NMAT];
#pragma unroll
  for (int m = 0; m < NMAT; ++m) {
    const int base = STAGE == 0 ? 2 * m : 4;
    wrow[m] = reinterpret_cast<const uint8_t*>(sl[base]) + size_t(j) * (packed ? Kg >> 1 : Kg);
    srow[m] = reinterpret_cast<const uint8_t*>(sl[base + 1]) + size_t(packed ? j : j >> 5) * G;
  }
  const int bias = packed ? 264 : 272;
  double total[NMAT];
#pragma unroll
  for (int m = 0; m < NMAT; ++m) total[m] = 0.0;
  for (int g = 0; g < G; ++g) {
    const int sa = sxs[g];
    const int4* a4 = reinterpret_cast<const int4*>(avs + size_t(g) * 32);
#pragma unroll
    for (int m = 0; m < NMAT; ++m) {
      long long sum = 0;
      if (packed) {
        const u32x4 w = load16(wrow[m] + size_t(g) * 16);
        int isum = 0;  // |av * bv| < 2^22, 32 terms: fits 32 bits
#pragma unroll
        for (int c = 0; c < 4; ++c) {
          const int4 lo = a4[2 * c], hi = a4[2 * c + 1];
          const int av[8] = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
#pragma unroll
          for (int n = 0; n < 8; ++n) isum += av[n] * e2m1_int((w[c] >> (4 * n)) & 15u);
        }
        sum = isum;
      } else {
        const u32x4 w0 = load16(wrow[m] + size_t(g) * 32), w1 = load16(wrow[m] + size_t(g) * 32 + 16);
#pragma unroll
        for (int c = 0; c < 8; ++c) {
          const int4 a = a4[c];
          const uint32_t w = c < 4 ? w0[c] : w1[c - 4];
          sum += (long long)a.x * e4m3_int(w & 0xffu) + (long long)a.y * e4m3_int((w >> 8) & 0xffu) +
                 (long long)a.z * e4m3_int((w >> 16) & 0xffu) + (long long)a.w * e4m3_int(w >> 24);
        }
      }
      const int sb = srow[m][g];
      total[m] = fma(double(sum), pow2_f64(sa + sb - bias), total[m]);
    }
  }
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

}  // namespace ffmoe
