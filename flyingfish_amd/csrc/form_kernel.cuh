// Decode expert FFN in the reference's own reduction orders, bit for bit.
//
// The reference keeps two summation orders for an expert dot product and its CPU path reproduces both exactly
// (src/cpu/expert_ffn.rs:689-776, `Form::Lane16` and `Form::Lane8`), so that a layer may run some experts on the CPU and
// some on the GPU with identical results; on the GPU they are the "invariant" kernels moe_ffn_*_lane16
// (kernels/moe_ffn.cu:364-393) and the production kernels moe_gate_up / moe_down (kernels/moe_ffn.cu:98-302):
//
//   Lane16: 16 accumulators; element k goes to accumulator k % 16 by fused multiply-add in ascending k; the result is
//           ((l0+l1)+(l2+l3))+((l4+l5)+(l6+l7)) + the same of l8..l15  (expert_ffn.rs:681-687).
//   Lane8:  every vector of 8 consecutive elements is summed by a fused multiply-add chain starting from 0; vector v is
//           ADDED to accumulator v % 8; the result is ((l0+l4)+(l2+l6))+((l1+l5)+(l3+l7))  (expert_ffn.rs:37-41).
//
// The streaming kernels of decode_kernel.cuh use one 64-lane sum per row and match these only to tolerance. The
// kernels here keep the orders exactly: Lane16 gives two hardware lanes to a row, each holding 8 of the 16
// accumulators in registers (elements 16i .. 16i+7 and 16i+8 .. 16i+15 are contiguous, so each lane still loads whole
// words); Lane8 gives eight hardware lanes to a row, lane l taking the vectors v = l, l+8, ...; the final trees are
// lane-pair exchanges in the order above. Activation roundings are those of the streaming kernels. SiLU follows the
// reference per form: g / (1 + exp(-g)) for Lane8 and for Lane16 with one rounding, g * (1 / (1 + exp(-g))) for Lane16
// with two roundings (kernels/moe_ffn.cu:58, :201-203).
//
// Formats: BF16 and per-channel FP8 experts, the formats the reference's CPU path executes.
#pragma once
#include "decode_kernel.cuh"

namespace ffmoe {

#define FFMOE_FORM_LANE16_ 0
#define FFMOE_FORM_LANE8_ 1

// 8 consecutive effective weights of a row as FP32, from element k0 (a multiple of 8)
template <class F>
struct FormRow;

template <>
struct FormRow<FmtBf16> {
  const uint16_t* w;
  __device__ __forceinline__ FormRow(uint64_t codes, uint64_t, int j, int K) : w(reinterpret_cast<const uint16_t*>(codes) + size_t(j) * K) {}
  __device__ __forceinline__ void load8(int k0, float (&o)[8]) const {
    const u32x4 v = load16(w + k0);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      o[2 * i] = __uint_as_float(v[i] << 16);
      o[2 * i + 1] = __uint_as_float(v[i] & 0xffff0000u);
    }
  }
};

template <>
struct FormRow<FmtFp8Channel> {
  const uint8_t* w;
  float scale;
  __device__ __forceinline__ FormRow(uint64_t codes, uint64_t scales, int j, int K)
      : w(reinterpret_cast<const uint8_t*>(codes) + size_t(j) * K), scale(bf16_to_f32(reinterpret_cast<const uint16_t*>(scales)[j])) {}
  __device__ __forceinline__ void load8(int k0, float (&o)[8]) const {
    const u32x2 v = load_global<u32x2>(w + k0);
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      uint32_t w01, w23;
      dequant4_e4m3(v[i], scale, w01, w23);  // bf16(e4m3 * scale), src/fp8.rs:138-140
      o[4 * i] = __uint_as_float(w01 << 16);
      o[4 * i + 1] = __uint_as_float(w01 & 0xffff0000u);
      o[4 * i + 2] = __uint_as_float(w23 << 16);
      o[4 * i + 3] = __uint_as_float(w23 & 0xffff0000u);
    }
  }
};

// 8 consecutive BF16 activations from LDS as FP32
__device__ __forceinline__ void form_x8(const uint8_t* xs, int k0, float (&o)[8]) {
  const u32x4 v = *reinterpret_cast<const u32x4*>(xs + size_t(k0) * 2);
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    o[2 * i] = __uint_as_float(v[i] << 16);
    o[2 * i + 1] = __uint_as_float(v[i] & 0xffff0000u);
  }
}

__device__ __forceinline__ float lane_xor(float v, int mask) { return __shfl_xor(v, mask, 64); }

// Dot product of the LDS row xs[0..K) with one weight row in the given form. `sub` is this lane's index inside the
// row's lane group (Lane16: 0..1, Lane8: 0..7); every lane of the group returns the result.
template <class F, int FORM>
__device__ __forceinline__ float form_dot(const uint8_t* xs, const FormRow<F>& row, int K, int sub) {
  float x[8], w[8];
  if (FORM == FFMOE_FORM_LANE16_) {
    float acc[8] = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
    // this lane owns accumulators 8*sub .. 8*sub+7: elements 16i + 8*sub + t. A last half step (K % 16 == 8) belongs
    // to accumulators 0..7, i.e. to sub 0 only.
    for (int k0 = 8 * sub; k0 < K; k0 += 16) {
      form_x8(xs, k0, x);
      row.load8(k0, w);
#pragma unroll
      for (int t = 0; t < 8; ++t) acc[t] = __fmaf_rn(x[t], w[t], acc[t]);
    }
    const float half = __fadd_rn(__fadd_rn(__fadd_rn(acc[0], acc[1]), __fadd_rn(acc[2], acc[3])),
                                 __fadd_rn(__fadd_rn(acc[4], acc[5]), __fadd_rn(acc[6], acc[7])));
    const float other = lane_xor(half, 1);
    return sub == 0 ? __fadd_rn(half, other) : __fadd_rn(other, half);  // low + high
  }
  float acc = 0.0f;
  for (int k0 = 8 * sub; k0 < K; k0 += 64) {  // vectors sub, sub + 8, ...
    form_x8(xs, k0, x);
    row.load8(k0, w);
    float inner = 0.0f;
#pragma unroll
    for (int t = 0; t < 8; ++t) inner = __fmaf_rn(x[t], w[t], inner);
    acc = __fadd_rn(acc, inner);
  }
  // ((l0+l4)+(l2+l6)) + ((l1+l5)+(l3+l7)): partners 4, 2, 1; the lower lane index is the left operand
  float o = lane_xor(acc, 4);
  acc = (sub & 4) ? __fadd_rn(o, acc) : __fadd_rn(acc, o);
  o = lane_xor(acc, 2);
  acc = (sub & 2) ? __fadd_rn(o, acc) : __fadd_rn(acc, o);
  o = lane_xor(acc, 1);
  acc = (sub & 1) ? __fadd_rn(o, acc) : __fadd_rn(acc, o);
  return acc;
}

// SwiGLU with the reference's SiLU per form (see the file comment)
__device__ __forceinline__ uint16_t form_swiglu(float g, float u, int mode, float limit, bool reciprocal) {
  if (mode == FFMOE_SWIGLU_GELU_TWICE) return f32_to_bf16(__fmul_rn(bround(gelu_tanh(g)), u));
  if (mode >= 2) {
    g = fminf(g, limit);
    u = fminf(fmaxf(u, -limit), limit);
  }
  const float den = __fadd_rn(1.0f, det_expf(-g));
  const float act = reciprocal ? __fmul_rn(g, __fdiv_rn(1.0f, den)) : __fdiv_rn(g, den);
  const float prod = (mode == 0 || mode == 2) ? __fmul_rn(bround(act), u) : __fmul_rn(act, u);
  return f32_to_bf16(prod);
}

// grid (ceil(out / ROWS), rows, top_k + 1): block z < top_k is choice z of token row y, z == top_k the shared expert
// (the reference's launch shape, src/backend/cuda/moe/decode.rs:486-514). STAGE 0: gate/up + SwiGLU -> h,
// STAGE 1: down (+ routing weight) -> contributions / shared_out.
template <class F, int FORM, int STAGE>
__global__ __launch_bounds__(256) void k_decode_form(const DecodeParams p) {
  constexpr int LPR = FORM == FFMOE_FORM_LANE16_ ? 2 : 8;  // hardware lanes per output row
  constexpr int ROWS = 256 / LPR;
  extern __shared__ __align__(16) uint8_t xs[];
  const int tid = threadIdx.x;
  const int r = blockIdx.y, z = blockIdx.z;
  const bool is_shared = z == p.top_k;
  if (is_shared && !p.has_shared) return;
  const int A = p.rows * p.top_k;
  int expert, gn, grow[1], gslot[1];
  load_group<1>(p, is_shared ? A + r : r * p.top_k + z, expert, gn, grow, gslot);
  if (gn == 0) return;  // inactive, invalid or stale choice: nothing written, done stays 0
  const int Kg = STAGE == 0 ? p.hidden : (is_shared ? p.shared_inter : p.inter);
  const int out = STAGE == 0 ? (is_shared ? p.shared_inter : p.inter) : p.hidden;
  if (int(blockIdx.x) * ROWS >= out) return;
  {
    const uint16_t* src = STAGE == 0 ? p.x + size_t(r) * p.hidden : p.h + size_t(gslot[0]) * p.h_stride;
    u32x4* d4 = reinterpret_cast<u32x4*>(xs);
    for (int v = tid; v < (Kg >> 3); v += 256) d4[v] = load16(src + size_t(v) * 8);
  }
  __syncthreads();
  const int j = blockIdx.x * ROWS + tid / LPR;
  const int sub = tid % LPR;
  if (j >= out) return;
  uint64_t sl[6];
#pragma unroll
  for (int i = 0; i < 6; ++i) sl[i] = is_shared ? p.shared_slot[i] : p.slots[size_t(expert) * 6 + i];
  if (STAGE == 0) {
    const FormRow<F> gate(sl[0], sl[1], j, Kg), up(sl[2], sl[3], j, Kg);
    const float g = form_dot<F, FORM>(xs, gate, Kg, sub);
    const float u = form_dot<F, FORM>(xs, up, Kg, sub);
    const bool reciprocal = FORM == FFMOE_FORM_LANE16_ && (p.swiglu == FFMOE_SWIGLU_TWICE || p.swiglu == FFMOE_SWIGLU_CLAMPED_TWICE);
    if (sub == 0) p.h[size_t(gslot[0]) * p.h_stride + j] = form_swiglu(bround(g), bround(u), p.swiglu, p.swiglu_limit, reciprocal);
  } else {
    const FormRow<F> down(sl[4], sl[5], j, Kg);
    const float d = form_dot<F, FORM>(xs, down, Kg, sub);
    if (sub == 0) {
      if (is_shared) {
        p.shared_out[size_t(r) * p.hidden + j] = f32_to_bf16(d);
      } else {
        const float wk = p.weights_f32 ? reinterpret_cast<const float*>(p.weights)[gslot[0]]
                                       : bf16_to_f32(reinterpret_cast<const uint16_t*>(p.weights)[gslot[0]]);
        const float v = __fmul_rn(p.routed_weight == FFMOE_WEIGHT_AFTER_DOWN_BF16 ? bround(d) : d, wk);
        p.contributions[size_t(gslot[0]) * p.hidden + j] = f32_to_bf16(v);
        if (j == 0 && p.done) p.done[gslot[0]] = 1u;
      }
    }
  }
}

// The same dot product for up to RG activation rows at once: a weight word is loaded once and every row keeps its own
// accumulators, so each (row, column) result is the chain of form_dot bit for bit. n = live rows (uniform in the block).
template <class F, int FORM, int RG>
__device__ __forceinline__ void form_dot_rows(const uint8_t* xs, int xstride, int n, const FormRow<F>& row, int K, int sub, float (&out)[RG]) {
  float x[8], w[8];
  if (FORM == FFMOE_FORM_LANE16_) {
    float acc[RG][8];
#pragma unroll
    for (int r = 0; r < RG; ++r)
#pragma unroll
      for (int t = 0; t < 8; ++t) acc[r][t] = 0.0f;
    for (int k0 = 8 * sub; k0 < K; k0 += 16) {
      row.load8(k0, w);
#pragma unroll
      for (int r = 0; r < RG; ++r) {
        if (r < n) {
          form_x8(xs + size_t(r) * xstride, k0, x);
#pragma unroll
          for (int t = 0; t < 8; ++t) acc[r][t] = __fmaf_rn(x[t], w[t], acc[r][t]);
        }
      }
    }
#pragma unroll
    for (int r = 0; r < RG; ++r) {
      const float half = __fadd_rn(__fadd_rn(__fadd_rn(acc[r][0], acc[r][1]), __fadd_rn(acc[r][2], acc[r][3])),
                                   __fadd_rn(__fadd_rn(acc[r][4], acc[r][5]), __fadd_rn(acc[r][6], acc[r][7])));
      const float other = lane_xor(half, 1);
      out[r] = sub == 0 ? __fadd_rn(half, other) : __fadd_rn(other, half);
    }
    return;
  }
  float acc[RG];
#pragma unroll
  for (int r = 0; r < RG; ++r) acc[r] = 0.0f;
  for (int k0 = 8 * sub; k0 < K; k0 += 64) {
    row.load8(k0, w);
#pragma unroll
    for (int r = 0; r < RG; ++r) {
      if (r < n) {
        form_x8(xs + size_t(r) * xstride, k0, x);
        float inner = 0.0f;
#pragma unroll
        for (int t = 0; t < 8; ++t) inner = __fmaf_rn(x[t], w[t], inner);
        acc[r] = __fadd_rn(acc[r], inner);
      }
    }
  }
#pragma unroll
  for (int r = 0; r < RG; ++r) {
    float a = acc[r];
    float o = lane_xor(a, 4);
    a = (sub & 4) ? __fadd_rn(o, a) : __fadd_rn(a, o);
    o = lane_xor(a, 2);
    a = (sub & 2) ? __fadd_rn(o, a) : __fadd_rn(a, o);
    o = lane_xor(a, 1);
    a = (sub & 1) ? __fadd_rn(o, a) : __fadd_rn(a, o);
    out[r] = a;
  }
}

// Token-sorted form of k_decode_form: grid (ceil(out / ROWS), groups). A block takes one group of up to RG assignments of
// one expert (k_group_assignments; the shared expert's rows come as groups of their own), stages their activation rows
// in LDS and streams each weight row once for all of them. The reference's grouped kernels read a weight row once per
// (row, column) and leave the reuse to the cache (kernels/moe_prefill.cu:13-71); the results are the same bits.
template <class F, int FORM, int STAGE, int RG>
__global__ __launch_bounds__(256) void k_decode_form_grouped(const DecodeParams p) {
  constexpr int LPR = FORM == FFMOE_FORM_LANE16_ ? 2 : 8;
  constexpr int ROWS = 256 / LPR;
  extern __shared__ __align__(16) uint8_t xs[];
  const int tid = threadIdx.x;
  const int g = blockIdx.y;
  const int n_routed = uni(load_global<int>(p.counters)), n_shared = uni(load_global<int>(p.counters + 1));
  if (g >= n_routed + n_shared) return;
  int expert, gn, grow[RG], gslot[RG];
  load_group<RG>(p, g, expert, gn, grow, gslot);
  if (gn == 0) return;
  const bool is_shared = expert < 0;
  const int Kg = STAGE == 0 ? p.hidden : (is_shared ? p.shared_inter : p.inter);
  const int out = STAGE == 0 ? (is_shared ? p.shared_inter : p.inter) : p.hidden;
  if (int(blockIdx.x) * ROWS >= out) return;
  const int xstride = Kg * 2;
#pragma unroll
  for (int r = 0; r < RG; ++r) {
    if (r < gn) {
      const uint16_t* src = STAGE == 0 ? p.x + size_t(grow[r]) * p.hidden : p.h + size_t(gslot[r]) * p.h_stride;
      u32x4* d4 = reinterpret_cast<u32x4*>(xs + size_t(r) * xstride);
      for (int v = tid; v < (Kg >> 3); v += 256) d4[v] = load16(src + size_t(v) * 8);
    }
  }
  __syncthreads();
  const int j = blockIdx.x * ROWS + tid / LPR;
  const int sub = tid % LPR;
  if (j >= out) return;
  uint64_t sl[6];
#pragma unroll
  for (int i = 0; i < 6; ++i) sl[i] = is_shared ? p.shared_slot[i] : p.slots[size_t(expert) * 6 + i];
  if (STAGE == 0) {
    const FormRow<F> gate(sl[0], sl[1], j, Kg), up(sl[2], sl[3], j, Kg);
    float gv[RG], uv[RG];
    form_dot_rows<F, FORM, RG>(xs, xstride, gn, gate, Kg, sub, gv);
    form_dot_rows<F, FORM, RG>(xs, xstride, gn, up, Kg, sub, uv);
    const bool reciprocal = FORM == FFMOE_FORM_LANE16_ && (p.swiglu == FFMOE_SWIGLU_TWICE || p.swiglu == FFMOE_SWIGLU_CLAMPED_TWICE);
    if (sub == 0) {
#pragma unroll
      for (int r = 0; r < RG; ++r)
        if (r < gn) p.h[size_t(gslot[r]) * p.h_stride + j] = form_swiglu(bround(gv[r]), bround(uv[r]), p.swiglu, p.swiglu_limit, reciprocal);
    }
  } else {
    const FormRow<F> down(sl[4], sl[5], j, Kg);
    float dv[RG];
    form_dot_rows<F, FORM, RG>(xs, xstride, gn, down, Kg, sub, dv);
    if (sub == 0) {
#pragma unroll
      for (int r = 0; r < RG; ++r) {
        if (r < gn) {
          if (is_shared) {
            p.shared_out[size_t(grow[r]) * p.hidden + j] = f32_to_bf16(dv[r]);
          } else {
            const float wk = p.weights_f32 ? reinterpret_cast<const float*>(p.weights)[gslot[r]]
                                           : bf16_to_f32(reinterpret_cast<const uint16_t*>(p.weights)[gslot[r]]);
            const float v = __fmul_rn(p.routed_weight == FFMOE_WEIGHT_AFTER_DOWN_BF16 ? bround(dv[r]) : dv[r], wk);
            p.contributions[size_t(gslot[r]) * p.hidden + j] = f32_to_bf16(v);
            if (j == 0 && p.done) p.done[gslot[r]] = 1u;
          }
        }
      }
    }
  }
}

template <class F, int FORM, int RG>
int launch_form_grouped(const DecodeParams& p, unsigned max_groups, int stage_mask, hipStream_t st) {
  constexpr int ROWS = 256 / (FORM == FFMOE_FORM_LANE16_ ? 2 : 8);
  const int imax = p.inter > p.shared_inter ? p.inter : p.shared_inter;
  if (stage_mask & 1) {
    hipLaunchKernelGGL((k_decode_form_grouped<F, FORM, 0, RG>), dim3((imax + ROWS - 1) / ROWS, max_groups), dim3(256), size_t(RG) * p.hidden * 2, st, p);
    FF_TRY(ff_launch_status());
  }
  if (stage_mask & 2) {
    hipLaunchKernelGGL((k_decode_form_grouped<F, FORM, 1, RG>), dim3((p.hidden + ROWS - 1) / ROWS, max_groups), dim3(256), size_t(RG) * imax * 2, st, p);
    FF_TRY(ff_launch_status());
  }
  return 0;
}

template <class F, int FORM>
int launch_form(const DecodeParams& p, int stage_mask, hipStream_t st) {
  constexpr int ROWS = 256 / (FORM == FFMOE_FORM_LANE16_ ? 2 : 8);
  const int imax = p.inter > p.shared_inter ? p.inter : p.shared_inter;
  if (stage_mask & 1) {
    hipLaunchKernelGGL((k_decode_form<F, FORM, 0>), dim3((imax + ROWS - 1) / ROWS, p.rows, p.top_k + 1), dim3(256), size_t(p.hidden) * 2, st, p);
    FF_TRY(ff_launch_status());
  }
  if (stage_mask & 2) {
    hipLaunchKernelGGL((k_decode_form<F, FORM, 1>), dim3((p.hidden + ROWS - 1) / ROWS, p.rows, p.top_k + 1), dim3(256), size_t(imax) * 2, st, p);
    FF_TRY(ff_launch_status());
  }
  return 0;
}

}  // namespace ffmoe
