// Device-side helpers shared by every kernel of libffmoe (gfx950, wave64).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <type_traits>

namespace ffmoe {

typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

constexpr int WAVE = 64;

__device__ __forceinline__ float bf16_to_f32(uint16_t h) { return __uint_as_float(uint32_t(h) << 16); }
__device__ __forceinline__ float bf16lo(uint32_t pair) { return __uint_as_float(pair << 16); }
__device__ __forceinline__ float bf16hi(uint32_t pair) { return __uint_as_float(pair & 0xffff0000u); }

// FP32 -> BF16 round-to-nearest-even (v_cvt_pk_bf16_f32 on gfx950).
__device__ __forceinline__ uint16_t f32_to_bf16(float f) {
  const __bf16 b = static_cast<__bf16>(f);
  return __builtin_bit_cast(uint16_t, b);
}
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  f32x2 v = {lo, hi};
  const bf16x2 b = __builtin_convertvector(v, bf16x2);
  return __builtin_bit_cast(uint32_t, b);
}
__device__ __forceinline__ float bround(float f) { return bf16_to_f32(f32_to_bf16(f)); }

// acc + a.lo*b.lo + a.hi*b.hi over packed BF16 pairs (v_dot2c_f32_bf16).
__device__ __forceinline__ float dot2_bf16(uint32_t a, uint32_t b, float acc) {
  return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, a), __builtin_bit_cast(bf16x2, b), acc, false);
}

// Two OCP E4M3 codes -> two f32 (v_cvt_pk_f32_fp8); hi selects the upper 16 bits of the dword.
template <bool HI>
__device__ __forceinline__ f32x2 e4m3x2_to_f32(uint32_t packed) {
  return __builtin_amdgcn_cvt_pk_f32_fp8(packed, HI);
}
// Four codes of one dword scaled and rounded to BF16: two packed pairs (elements 0,1 and 2,3).
__device__ __forceinline__ void dequant4_e4m3(uint32_t codes, float scale, uint32_t& w01, uint32_t& w23) {
  const f32x2 lo = e4m3x2_to_f32<false>(codes);
  const f32x2 hi = e4m3x2_to_f32<true>(codes);
  w01 = pack_bf16x2(lo.x * scale, lo.y * scale);
  w23 = pack_bf16x2(hi.x * scale, hi.y * scale);
}
__device__ __forceinline__ float e4m3_to_f32(uint8_t code) { return e4m3x2_to_f32<false>(uint32_t(code)).x; }

// E4M3 code of a finite value already clamped to [-448, 448], round-to-nearest-even
// (same function as src/fp8.rs:85-121 of the reference).
// Four finite values inside +-448 to E4M3 by the hardware conversion (round to nearest even, OCP E4M3 on this GPU): the
// same codes as e4m3_encode for such values (-0 -> 0x80, subnormals on the m / 512 grid), two instructions instead of four
// software encodings. The quantizers clamp to +-448 first, so saturation and NaN handling never come into it.
__device__ __forceinline__ uint32_t e4m3x4_encode_finite(float a, float b, float c, float d) {
  int w = 0;
  w = __builtin_amdgcn_cvt_pk_fp8_f32(a, b, w, false);
  w = __builtin_amdgcn_cvt_pk_fp8_f32(c, d, w, true);
  return uint32_t(w);
}

__device__ __forceinline__ uint8_t e4m3_encode(float value) {
  const uint32_t bits = __float_as_uint(value);
  const uint32_t sign = (bits >> 24) & 0x80u;
  const uint32_t mag = bits & 0x7fffffffu;
  if (mag < 0x3c800000u) {  // |v| < 2^-6: subnormal grid m/512, ties to even
    const float scaled = __uint_as_float(mag) * 512.0f;
    const uint32_t m = uint32_t(__builtin_rintf(scaled));
    return uint8_t(sign | m);  // m == 8 is code 0x08 = 2^-6, the first normal
  }
  uint32_t rounded = mag >> 20;
  const uint32_t rest = mag & 0xfffffu;
  rounded += (rest > 0x80000u || (rest == 0x80000u && (rounded & 1u))) ? 1u : 0u;
  rounded -= 960u;  // (exponent 120) << 3
  return uint8_t(sign | (rounded > 126u ? 126u : rounded));
}

// E2M1 magnitude table; both zero codes give +0 (kernels/nvfp4_linear.cu:12-14 of the reference).
__device__ __forceinline__ float e2m1_to_f32(uint32_t nib) {
  const uint32_t m = nib & 7u;
  // {0, .5, 1, 1.5, 2, 3, 4, 6}: bits of the f32 value
  const uint32_t expo = m < 2u ? (m == 0u ? 0u : 0x3f000000u) : (0x3f800000u + (((m >> 1) - 1u) << 23));
  const uint32_t frac = (m >= 2u && (m & 1u)) ? 0x00400000u : 0u;
  const uint32_t bits = expo | frac;
  return __uint_as_float(m == 0u ? 0u : (bits | ((nib & 8u) << 28)));
}

// Deterministic expf: IEEE +,-,*,fma only, so the host restatement gives the same bits.
// x = n ln2 + r, Cephes polynomial for (e^r - 1 - r)/r^2, two-step scaling by 2^n.
__device__ __forceinline__ float det_expf(float x) {
  if (x != x) return x;
  if (!(x > -104.0f)) return 0.0f;
  if (x > 88.72283935546875f) return __uint_as_float(0x7f800000u);
  const float magic = 12582912.0f;
  const float t = __fmaf_rn(x, 1.44269502162933349609375f, magic);
  const float n = __fsub_rn(t, magic);
  float r = __fmaf_rn(n, -0.693145751953125f, x);
  r = __fmaf_rn(n, -1.428606765330187045037746429443359375e-06f, r);
  float p = 1.9875691500e-4f;
  p = __fmaf_rn(p, r, 1.3981999507e-3f);
  p = __fmaf_rn(p, r, 8.3334519073e-3f);
  p = __fmaf_rn(p, r, 4.1665795894e-2f);
  p = __fmaf_rn(p, r, 1.6666665459e-1f);
  p = __fmaf_rn(p, r, 5.0000001201e-1f);
  const float r2 = __fmul_rn(r, r);
  float y = __fmaf_rn(p, r2, r);
  y = __fadd_rn(y, 1.0f);
  const int ni = int(n);
  const int a = ni >> 1, b = ni - a;
  y = __fmul_rn(y, __uint_as_float(uint32_t(a + 127) << 23));
  y = __fmul_rn(y, __uint_as_float(uint32_t(b + 127) << 23));
  return y;
}

// log(1+u), 0 <= u <= 1.
__device__ __forceinline__ float det_log1pf_unit(float u) {
  const float w = __fadd_rn(1.0f, u);
  if (w == 1.0f) return u;
  float m = w;
  float e = 0.0f;
  if (m > 1.41421353816986083984375f) { m = __fmul_rn(m, 0.5f); e = 1.0f; }
  const float f = __fsub_rn(m, 1.0f);
  const float z = __fmul_rn(f, f);
  float p = 7.0376836292e-2f;
  p = __fmaf_rn(p, f, -1.1514610310e-1f);
  p = __fmaf_rn(p, f, 1.1676998740e-1f);
  p = __fmaf_rn(p, f, -1.2420140846e-1f);
  p = __fmaf_rn(p, f, 1.4249322787e-1f);
  p = __fmaf_rn(p, f, -1.6668057665e-1f);
  p = __fmaf_rn(p, f, 2.0000714765e-1f);
  p = __fmaf_rn(p, f, -2.4999993993e-1f);
  p = __fmaf_rn(p, f, 3.3333331174e-1f);
  float y = __fmul_rn(__fmul_rn(f, z), p);
  y = __fmaf_rn(-0.5f, z, y);
  float lg = __fadd_rn(f, y);
  lg = __fmaf_rn(e, 0.693147182464599609375f, lg);
  const float c = __fdiv_rn(__fsub_rn(u, __fsub_rn(w, 1.0f)), w);
  return __fadd_rn(lg, c);
}

__device__ __forceinline__ float sigmoid1(float l) {
  return __fdiv_rn(1.0f, __fadd_rn(1.0f, det_expf(-l)));
}

// tanhf from the same operations as det_expf: odd Taylor polynomial through x^11 below 0.3, 1 - 2 / (exp(2|x|) + 1)
// above, +-1 beyond 9; within 3 ulp of the exact function.
__device__ __forceinline__ float det_tanhf(float x) {
  const float a = fabsf(x);
  if (a < 0.3f) {
    const float z = __fmul_rn(x, x);
    float p = -8.8632355e-3f;
    p = __fmaf_rn(p, z, 2.1869488e-2f);
    p = __fmaf_rn(p, z, -5.3968254e-2f);
    p = __fmaf_rn(p, z, 1.3333334e-1f);
    p = __fmaf_rn(p, z, -3.3333334e-1f);
    return __fmaf_rn(__fmul_rn(x, z), p, x);
  }
  float t = 1.0f;
  if (!(a > 9.0f)) t = __fsub_rn(1.0f, __fdiv_rn(2.0f, __fadd_rn(det_expf(__fmul_rn(2.0f, a)), 1.0f)));
  return copysignf(t, x);
}
// tanh form of GELU with one rounding per operation (src/cpu/expert_ffn.rs:87-91 of the reference)
__device__ __forceinline__ float gelu_tanh(float g) {
  const float cube = __fmul_rn(__fmul_rn(g, g), g);
  const float inner = __fmul_rn(0.7978846f, __fadd_rn(g, __fmul_rn(0.044715f, cube)));
  return __fmul_rn(__fmul_rn(0.5f, g), __fadd_rn(1.0f, det_tanhf(inner)));
}

// SwiGLU with the BF16 rounding boundary selected by `mode` (FFMOE_SWIGLU_*): returns BF16 bits.
// SiLU = g / (1 + exp(-g)) as in the production decode kernels of the reference.
// SiLU as x * sigmoid(x) with the two-branch sigmoid of the reference's dense activation kernels
// (kernels/q38_contract.cuh:17-21, kernels/act.cu:152-156).
__device__ __forceinline__ float silu_two_branch(float g) {
  float s;
  if (g >= 0.0f) s = __fdiv_rn(1.0f, __fadd_rn(1.0f, det_expf(-g)));
  else { const float e = det_expf(g); s = __fdiv_rn(e, __fadd_rn(1.0f, e)); }
  return __fmul_rn(g, s);
}
__device__ __forceinline__ uint16_t swiglu_bf16_two_branch(float g, float u, int mode, float limit) {
  if (mode >= 2) {
    g = fminf(g, limit);
    u = fminf(fmaxf(u, -limit), limit);
  }
  const float act = silu_two_branch(g);
  const float prod = (mode == 0 || mode == 2) ? __fmul_rn(bround(act), u) : __fmul_rn(act, u);
  return f32_to_bf16(prod);
}

__device__ __forceinline__ uint16_t swiglu_bf16(float g, float u, int mode, float limit) {
  // mode 4 (FFMOE_SWIGLU_GELU_TWICE) is bf16(bf16(gelu_tanh(g)) * u) without a clamp; it is written out here so that it shares
  // the one expf of the SiLU forms
  const bool gelu = mode == 4;
  float inner = 0.0f, arg;
  if (gelu) {
    const float cube = __fmul_rn(__fmul_rn(g, g), g);
    inner = __fmul_rn(0.7978846f, __fadd_rn(g, __fmul_rn(0.044715f, cube)));
    arg = __fmul_rn(2.0f, fabsf(inner));
  } else {
    if (mode >= 2) {
      g = fminf(g, limit);
      u = fminf(fmaxf(u, -limit), limit);
    }
    arg = -g;
  }
  const float den = __fadd_rn(det_expf(arg), 1.0f);
  float act;
  if (gelu) {
    const float a = fabsf(inner);
    float t = a > 9.0f ? 1.0f : __fsub_rn(1.0f, __fdiv_rn(2.0f, den));
    t = copysignf(t, inner);
    if (a < 0.3f) {
      const float z = __fmul_rn(inner, inner);
      float q = -8.8632355e-3f;
      q = __fmaf_rn(q, z, 2.1869488e-2f);
      q = __fmaf_rn(q, z, -5.3968254e-2f);
      q = __fmaf_rn(q, z, 1.3333334e-1f);
      q = __fmaf_rn(q, z, -3.3333334e-1f);
      t = __fmaf_rn(__fmul_rn(inner, z), q, inner);
    }
    act = __fmul_rn(__fmul_rn(0.5f, g), __fadd_rn(1.0f, t));
  } else {
    act = __fdiv_rn(g, den);
  }
  const float prod = (mode == 0 || mode == 2 || gelu) ? __fmul_rn(bround(act), u) : __fmul_rn(act, u);
  return f32_to_bf16(prod);
}

// ---------------------------------------------------------------------------------------------
// Wave-wide reductions on the DPP data path (no LDS round trips). The sequence is the usual gfx9 one:
// quad swaps, half-row and row mirrors leave every lane of a 16-lane row with the row total; two
// row broadcasts then carry the totals up, so lane 63 ends with the wave total, which is read back
// as a wave-uniform value. The summation order is fixed, so results do not depend on scheduling.
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ float dpp_or(float old, float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, old), __builtin_bit_cast(int, v), CTRL,
                                                                ROW_MASK, 0xf, false));
}
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ int dpp_or(int old, int v) {
  return __builtin_amdgcn_update_dpp(old, v, CTRL, ROW_MASK, 0xf, false);
}
constexpr int DPP_QUAD_SWAP1 = 0xB1;    // quad_perm:[1,0,3,2]
constexpr int DPP_QUAD_SWAP2 = 0x4E;    // quad_perm:[2,3,0,1]
constexpr int DPP_ROW_HALF_MIRROR = 0x141;
constexpr int DPP_ROW_MIRROR = 0x140;
constexpr int DPP_ROW_BCAST15 = 0x142;
constexpr int DPP_ROW_BCAST31 = 0x143;

// Sum over the 64 lanes of a wave; every lane receives the total.
__device__ __forceinline__ float wave_sum(float v) {
  v += dpp_or<DPP_QUAD_SWAP1, 0xf>(0.0f, v);
  v += dpp_or<DPP_QUAD_SWAP2, 0xf>(0.0f, v);
  v += dpp_or<DPP_ROW_HALF_MIRROR, 0xf>(0.0f, v);
  v += dpp_or<DPP_ROW_MIRROR, 0xf>(0.0f, v);
  v += dpp_or<DPP_ROW_BCAST15, 0xa>(0.0f, v);
  v += dpp_or<DPP_ROW_BCAST31, 0xc>(0.0f, v);
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));
}
__device__ __forceinline__ float wave_max(float v) {
  v = fmaxf(v, dpp_or<DPP_QUAD_SWAP1, 0xf>(v, v));
  v = fmaxf(v, dpp_or<DPP_QUAD_SWAP2, 0xf>(v, v));
  v = fmaxf(v, dpp_or<DPP_ROW_HALF_MIRROR, 0xf>(v, v));
  v = fmaxf(v, dpp_or<DPP_ROW_MIRROR, 0xf>(v, v));
  v = fmaxf(v, dpp_or<DPP_ROW_BCAST15, 0xa>(v, v));
  v = fmaxf(v, dpp_or<DPP_ROW_BCAST31, 0xc>(v, v));
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));
}
// Arg-max under (value desc, id asc); the winner is returned wave-uniform.
__device__ __forceinline__ void wave_argmax(float& v, int& id) {
#define FF_ARGMAX_STEP(CTRL, MASK)                                  \
  {                                                                 \
    const float ov = dpp_or<CTRL, MASK>(v, v);                      \
    const int oi = dpp_or<CTRL, MASK>(id, id);                      \
    const bool take = ov > v || (ov == v && oi < id);               \
    v = take ? ov : v;                                              \
    id = take ? oi : id;                                            \
  }
  FF_ARGMAX_STEP(DPP_QUAD_SWAP1, 0xf)
  FF_ARGMAX_STEP(DPP_QUAD_SWAP2, 0xf)
  FF_ARGMAX_STEP(DPP_ROW_HALF_MIRROR, 0xf)
  FF_ARGMAX_STEP(DPP_ROW_MIRROR, 0xf)
  FF_ARGMAX_STEP(DPP_ROW_BCAST15, 0xa)
  FF_ARGMAX_STEP(DPP_ROW_BCAST31, 0xc)
#undef FF_ARGMAX_STEP
  v = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));
  id = __builtin_amdgcn_readlane(id, 63);
}

// 64 values per lane in, one value per lane out: lane L ends with the sum over the wave's 64 lanes of value
// bitrev6(L), added in the adjacent-pair tree (lanes 2i and 2i+1, then pairs of pairs, ...), i.e. bit for bit what
// wave_sum gives for that value. At every level the two partners split the values they still hold: each keeps one half,
// sends the other and adds what it receives, so level k moves 64 / 2^k values instead of 64 - about 200 instructions
// where 64 calls of wave_sum take 1600. Levels 1-4 exchange inside a row of 16 lanes on the DPP path, levels 5 and 6
// with the row and half-wave swaps of gfx950.
// v_permlane16_swap_b32 a, b: lanes 16-31 and 48-63 of a trade places with lanes 0-15 and 32-47 of b;
// v_permlane32_swap_b32 a, b: lanes 32-63 of a trade places with lanes 0-31 of b. Both operands are read and written,
// which is stated here operand by operand (the compiler's own builtins for the two instructions lost the second result in
// this toolchain: the sum of the two results came out as twice the first). The idle cycles in front and behind are
// the wait states the compiler would insert between vector ALU writes and these cross-lane reads.
__device__ __forceinline__ void swap_rows16(float& a, float& b) {
  asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
}
__device__ __forceinline__ void swap_halves32(float& a, float& b) {
  asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
}
constexpr int DPP_ROW_SHL4 = 0x104, DPP_ROW_SHR4 = 0x114, DPP_ROW_SHL8 = 0x108, DPP_ROW_SHR8 = 0x118;
__device__ __forceinline__ float wave_reduce_scatter64(float (&a)[64], int lane) {
  const bool b0 = lane & 1, b1 = lane & 2, b2 = lane & 4, b3 = lane & 8;
  float c[32];
#pragma unroll
  for (int j = 0; j < 32; ++j) {  // partner lane ^ 1; a lane with bit 0 set keeps the upper half
    const float send = b0 ? a[j] : a[j + 32], keep = b0 ? a[j + 32] : a[j];
    c[j] = __fadd_rn(keep, dpp_or<DPP_QUAD_SWAP1, 0xf>(0.0f, send));
  }
  float d[16];
#pragma unroll
  for (int j = 0; j < 16; ++j) {  // lane ^ 2
    const float send = b1 ? c[j] : c[j + 16], keep = b1 ? c[j + 16] : c[j];
    d[j] = __fadd_rn(keep, dpp_or<DPP_QUAD_SWAP2, 0xf>(0.0f, send));
  }
  float e[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) {  // lane ^ 4: banks 0 and 2 of a row read four lanes up, banks 1 and 3 four lanes down
    const float send = b2 ? d[j] : d[j + 8], keep = b2 ? d[j + 8] : d[j];
    float got = __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, send), DPP_ROW_SHL4, 0xf, 0x5, false));
    got = __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, got), __builtin_bit_cast(int, send), DPP_ROW_SHR4, 0xf, 0xa, false));
    e[j] = __fadd_rn(keep, got);
  }
  float f[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {  // lane ^ 8: banks 0 and 1 read eight lanes up, banks 2 and 3 eight lanes down
    const float send = b3 ? e[j] : e[j + 4], keep = b3 ? e[j + 4] : e[j];
    float got = __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, send), DPP_ROW_SHL8, 0xf, 0x3, false));
    got = __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, got), __builtin_bit_cast(int, send), DPP_ROW_SHR8, 0xf, 0xc, false));
    f[j] = __fadd_rn(keep, got);
  }
  // lane ^ 16: the odd rows of the first operand trade places with the even rows of the second, after which an even-row
  // lane holds both partners' copies of the first value and an odd-row lane both copies of the second
  float g[2];
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    float lo = f[j], hi = f[j + 2];
    swap_rows16(lo, hi);
    g[j] = __fadd_rn(lo, hi);
  }
  // lane ^ 32: the same with the two halves of the wave
  swap_halves32(g[0], g[1]);
  return __fadd_rn(g[0], g[1]);
}
__device__ __forceinline__ int bitrev6(int v) { return int(__builtin_bitreverse32(unsigned(v)) >> 26); }

// Wave-uniform copies of values every lane already agrees on: they move to scalar registers, so addresses built
// from them use a scalar base.
__device__ __forceinline__ int uni(int v) { return __builtin_amdgcn_readfirstlane(v); }
__device__ __forceinline__ float unif(float v) { return __builtin_bit_cast(float, uni(__builtin_bit_cast(int, v))); }
__device__ __forceinline__ uint64_t uni64(uint64_t v) {
  return (uint64_t(uint32_t(uni(int(v >> 32)))) << 32) | uint32_t(uni(int(uint32_t(v))));
}

// Loads through pointers known to be global memory. Weight and scale addresses arrive as integers in slot
// tables, so without the explicit address space the compiler would emit flat loads, which also count against
// the LDS counter and serialize with the activation reads.
#define FF_GLOBAL __attribute__((address_space(1)))
template <class T>
__device__ __forceinline__ T load_global(const void* p) {
  return *(const FF_GLOBAL T*)(p);
}
__device__ __forceinline__ u32x4 load16(const void* p) { return load_global<u32x4>(p); }
// A load of a value every lane of the wave wants from the same address (tables written by earlier launches): through the
// scalar data cache, so it neither queues with the wave's vector requests nor counts against their hand-counted waits.
#define FF_CONSTANT __attribute__((address_space(4)))
template <class T>
__device__ __forceinline__ T load_uniform(const void* p) {
  return *(const FF_CONSTANT T*)(p);
}
// A copy of a loaded value that is known to have arrived. The compiler waits for a load where its result is first
// read; inside a loop it repeats that wait in every iteration when the load was issued before the loop, and because
// loads retire in order such a wait also drains every younger load in flight. Reading the value once through this
// copy before the loop keeps the loop free of it.
// Loads whose waits are placed by hand. The compiler sees an ordinary instruction that defines its result at once, so
// it places no wait of its own; the caller counts the loads it has issued since (they retire in issue order) and names
// that count in wait_loads<N>() before the first read. The registers go through the wait as in/out operands, which
// keeps every read of them behind it. A register that still has such a load in flight must not be left dead (the
// compiler would reuse it): drain with wait_loads<0>() over all of them before they go out of use.
__device__ __forceinline__ void load16_async(u32x4& d, const void* p) {
  asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(d) : "v"(p));
}
// The same with a wave-uniform 64-bit base in scalar registers and a 32-bit byte offset per lane: no 64-bit address
// arithmetic and no address registers per load on the vector side.
__device__ __forceinline__ void load16_async(u32x4& d, uint64_t base, uint32_t offset) {
  asm volatile("global_load_dwordx4 %0, %1, %2" : "=v"(d) : "v"(offset), "s"(base));
}
__device__ __forceinline__ void load4_async(float& d, const void* p) {
  asm volatile("global_load_dword %0, %1, off" : "=v"(d) : "v"(p));
}
__device__ __forceinline__ void load4_async(float& d, uint64_t base, uint32_t offset) {
  asm volatile("global_load_dword %0, %1, %2" : "=v"(d) : "v"(offset), "s"(base));
}
template <int N>
__device__ __forceinline__ void wait_loads(u32x4& a, u32x4& b, u32x4& c, u32x4& d, u32x4& e, u32x4& f, u32x4& g, u32x4& h) {
  asm volatile("s_waitcnt vmcnt(%8)" : "+v"(a), "+v"(b), "+v"(c), "+v"(d), "+v"(e), "+v"(f), "+v"(g), "+v"(h) : "n"(N));
}
template <int N>
__device__ __forceinline__ void wait_loads(u32x4& a, u32x4& b, u32x4& c, u32x4& d, float& e, float& f, float& g, float& h) {
  asm volatile("s_waitcnt vmcnt(%8)" : "+v"(a), "+v"(b), "+v"(c), "+v"(d), "+v"(e), "+v"(f), "+v"(g), "+v"(h) : "n"(N));
}
template <int N>
__device__ __forceinline__ void wait_loads(u32x4& a) {
  asm volatile("s_waitcnt vmcnt(%1)" : "+v"(a) : "n"(N));
}
template <int N>
__device__ __forceinline__ void wait_loads(u32x4& a, u32x4& b) {
  asm volatile("s_waitcnt vmcnt(%2)" : "+v"(a), "+v"(b) : "n"(N));
}
template <int N>
__device__ __forceinline__ void wait_loads(u32x4& a, float& b) {
  asm volatile("s_waitcnt vmcnt(%2)" : "+v"(a), "+v"(b) : "n"(N));
}
template <int N>
__device__ __forceinline__ void wait_loads(u32x4& a, u32x4& b, float& c) {
  asm volatile("s_waitcnt vmcnt(%3)" : "+v"(a), "+v"(b), "+v"(c) : "n"(N));
}
template <int N>
__device__ __forceinline__ void wait_loads(u32x4& a, u32x4& b, u32x4& c, u32x4& d, float& e) {
  asm volatile("s_waitcnt vmcnt(%5)" : "+v"(a), "+v"(b), "+v"(c), "+v"(d), "+v"(e) : "n"(N));
}
__device__ __forceinline__ float landed(float v) {
  float r;
  asm volatile("v_mov_b32 %0, %1" : "=v"(r) : "v"(v));
  return r;
}
// f(std::integral_constant<int, 0>{}) ... f(std::integral_constant<int, N - 1>{}): a loop whose index is a constant
// expression in the body (register arrays indexed by it stay in registers)
template <int N, int I = 0, class Fn>
__device__ __forceinline__ void static_for(Fn&& f) {
  if constexpr (I < N) {
    f(std::integral_constant<int, I>{});
    static_for<N, I + 1>(f);
  }
}
// LDS hand-over between the lanes of ONE wave: earlier LDS writes of the wave are complete and later reads are not
// moved above this point (LDS operations of a wave execute in order; the fence also stops the compiler).
__device__ __forceinline__ void wave_lds_fence() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
}
// Device-coherent accesses (relaxed, agent scope): the store is written through to memory and the load is served from
// there, so blocks on different XCDs (each with its own L2) can hand data to each other inside one kernel without
// cache-wide write-back / invalidate operations. Ordering comes from a counter the consumer polls the same way.
__device__ __forceinline__ void store_agent(uint16_t* p, uint16_t v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ void store_agent(uint32_t* p, uint32_t v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ u32x4 load16_agent(const void* p) {
  const uint64_t* q = reinterpret_cast<const uint64_t*>(p);
  const uint64_t a = __hip_atomic_load(q, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  const uint64_t b = __hip_atomic_load(q + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  return u32x4{uint32_t(a), uint32_t(a >> 32), uint32_t(b), uint32_t(b >> 32)};
}
// Streaming 16-byte load for data read exactly once (weights): the non-temporal hint keeps it from
// displacing reusable lines.
__device__ __forceinline__ u32x4 load16_stream(const void* p) {
  return __builtin_nontemporal_load((const FF_GLOBAL u32x4*)(p));
}

}  // namespace ffmoe
