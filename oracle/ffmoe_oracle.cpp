// CPU oracle for the quantized MoE expert-FFN path.
//
// THIS FILE IS TEST INFRASTRUCTURE. It restates, in plain scalar C++, the arithmetic of the
// reference (GreatV/flyingfish) for the router, the expert SwiGLU FFN, the block-scaled linears
// and the combine, so that the HIP kernels can be checked against it. Nothing in the shipped
// library links, loads or calls it; only tests, the smoke check and the CPU-baseline leg of the
// benchmark do.
//
// Every function cites the reference lines it follows (paths relative to the reference root).
// Parity status per function group:
//   * codecs, BF16 rounding, effective weights ............ pinned (exhaustive closed forms, spot values)
//   * noaux / sigmoid / softmax top-k ...................... pinned (golden router vectors, brute force)
//   * SwiGLU boundaries ..................................... pinned (golden BF16 bit patterns)
//   * tanh-GELU with two roundings .......................... pinned up to the last bits of tanh (the same FP32 operation
//     chain with a correctly rounded tanh, every BF16 gate value; the reference pins no tanh and holds no vectors)
//   * expert FFN on BF16 / per-channel FP8 weights .......... pinned (FP64 boundary oracle at 0 BF16 steps)
//   * W8A8 quantizer + block dot ............................ pinned (FP64 gamma bound, wrong-cell mutant)
//   * NVFP4 / BF16-scale skinny linear orders ............... pinned (closed-form dequant table, FP64 bound)
//   * Lane16 / Lane8 summation orders ....................... pinned (hand-computed cancellation witnesses)
//   * E8M0 block-32 contract: activation quantizer, exact
//     integer dot, repaired BF16 rounding ................... pinned (closed forms, rational arithmetic, tie witness)
//   * combine variants ...................................... pinned (order-spread constants of the fixture)
//   * NVFP4 weights re-rounded to E4M3 (W4A8 mode) .......... pinned as a function (rational arithmetic + brute-force nearest
//     code); the mode itself is this build's definition, the reference has no FP8 form of NVFP4
//   * expert FFN composed over 128x128-f32 block scales or
//     NVFP4 weights, grouped routing with n_group > 1,
//     FP32-logit dot order, last-bit behaviour of expf / tanhf parity unpinned (no reference code or vectors)
#include <cmath>
#include <cstdint>
#include <cstring>
#include <algorithm>
#include <vector>

#define ORC_API extern "C" __attribute__((visibility("default")))

namespace {

inline uint32_t f2u(float f) { uint32_t u; std::memcpy(&u, &f, 4); return u; }
inline float u2f(uint32_t u) { float f; std::memcpy(&f, &u, 4); return f; }

// BF16 round-to-nearest-even; crate `half` 2.7.1 `bf16::from_f32`, restated by the reference in
// src/cpu/expert_ffn.rs:1072-1080. NaN keeps its sign and gains the quiet bit.
inline uint16_t bf16_rne(float f) {
  uint32_t b = f2u(f);
  if ((b & 0x7fffffffu) > 0x7f800000u) return uint16_t((b >> 16) | 0x40u);
  b += 0x7fffu + ((b >> 16) & 1u);
  return uint16_t(b >> 16);
}
inline float bf16_f32(uint16_t h) { return u2f(uint32_t(h) << 16); }
inline float bround(float f) { return bf16_f32(bf16_rne(f)); }

// src/fp8.rs:69-82
inline float decode_e4m3(uint8_t code) {
  const uint32_t sign = uint32_t(code & 0x80u) << 24;
  const uint32_t mag = code & 0x7fu;
  if (mag == 0x7fu) return u2f(sign | 0x7fc00000u);
  const uint32_t e = mag >> 3, m = mag & 7u;
  if (e == 0) return u2f(f2u(float(m) * (1.0f / 512.0f)) | sign);
  return u2f(sign | ((e + 120u) << 23) | (m << 20));
}

// src/fp8.rs:85-121 (value already clamped to [-448, 448]).
inline uint8_t encode_e4m3(float value) {
  const uint32_t bits = f2u(value);
  const uint8_t sign = uint8_t((bits >> 31) & 1u);
  const uint32_t magnitude = bits & 0x7fffffffu;
  if (magnitude == 0) return uint8_t(sign << 7);
  const int exponent = int((magnitude >> 23) & 0xffu) - 127;
  const uint32_t mantissa = magnitude & 0x7fffffu;
  if (exponent < -6) {
    const double scaled = double(std::fabs(value)) * 512.0;
    uint64_t m = uint64_t(std::floor(scaled));
    const double fraction = scaled - double(m);
    if (fraction > 0.5 || (fraction == 0.5 && (m & 1u) == 1u)) m += 1;
    if (m >= 8) return uint8_t((sign << 7) | 0x08u);
    return uint8_t((sign << 7) | uint8_t(m));
  }
  int e = exponent + 7;
  uint32_t m = mantissa >> 20;
  const uint32_t rest = mantissa & 0xfffffu;
  if (rest > 0x80000u || (rest == 0x80000u && (m & 1u) == 1u)) {
    m += 1;
    if (m == 8) { m = 0; e += 1; }
  }
  if (e > 15) return uint8_t((sign << 7) | 0x7eu);
  // exponent field 15 with mantissa 7 is the NaN code; the reference clamps its input to 448
  // (mantissa 6) before calling, so that pattern never forms.
  return uint8_t((sign << 7) | (uint8_t(e) << 3) | uint8_t(m));
}

// src/fp8.rs:124-136; kernels/q38_contract.cuh:172-178 keeps the sign of zero.
inline float decode_e2m1(uint8_t code) {
  static const float mags[8] = {0.0f, 0.5f, 1.0f, 1.5f, 2.0f, 3.0f, 4.0f, 6.0f};
  if ((code & 7u) == 0) return 0.0f;  // fp8.rs:126 returns +0 for both zero codes
  return u2f(f2u(mags[code & 7u]) | (uint32_t(code & 8u) << 28));
}

// kernels/q38_contract.cuh:180-187
inline uint8_t encode_e2m1(float value) {
  const float m = std::fabs(value);
  const uint8_t code = m <= 0.25f ? 0 : m < 0.75f ? 1 : m <= 1.25f ? 2 : m < 1.75f ? 3
                     : m <= 2.5f ? 4 : m < 3.5f ? 5 : m <= 5.0f ? 6 : 7;
  return uint8_t(code | uint8_t((f2u(value) >> 28) & 8u));
}

// ---------------------------------------------------------------------------------------------
// expf / log1pf built from IEEE +,-,*,/ and fused multiply-add only, so that host and device
// produce the same bits. The reference takes expf from libm (CPU) or the CUDA math library (GPU)
// and pins neither; this oracle therefore fixes one definition and checks it to <= 2 ulp of the
// exact function (see tests). Range reduction x = n ln2 + r, degree-5 polynomial in r for
// (e^r - 1 - r)/r^2 (Cephes expf coefficients), two-step scaling so subnormal results round once.
inline float det_expf(float x) {
  if (x != x) return x;
  if (!(x > -104.0f)) return 0.0f;
  if (x > 88.72283935546875f) return u2f(0x7f800000u);
  const float magic = 12582912.0f;  // 1.5 * 2^23: adding it rounds to the nearest integer
  const float t = std::fmaf(x, 1.44269502162933349609375f, magic);
  const float n = t - magic;
  float r = std::fmaf(n, -0.693145751953125f, x);
  r = std::fmaf(n, -1.428606765330187045037746429443359375e-06f, r);
  float p = 1.9875691500e-4f;
  p = std::fmaf(p, r, 1.3981999507e-3f);
  p = std::fmaf(p, r, 8.3334519073e-3f);
  p = std::fmaf(p, r, 4.1665795894e-2f);
  p = std::fmaf(p, r, 1.6666665459e-1f);
  p = std::fmaf(p, r, 5.0000001201e-1f);
  const float r2 = r * r;
  float y = std::fmaf(p, r2, r);
  y = y + 1.0f;
  const int ni = int(n);
  const int a = ni >> 1, b = ni - a;
  y = y * u2f(uint32_t(a + 127) << 23);
  y = y * u2f(uint32_t(b + 127) << 23);
  return y;
}

// log(1+u) for 0 <= u <= 1 (the only range sqrt-softplus needs): w = 1+u rounded, Cephes logf
// polynomial on the reduced argument, then the first-order correction for the rounding of w.
inline float det_log1pf_unit(float u) {
  const float w = 1.0f + u;
  if (w == 1.0f) return u;
  float m = w;
  float e = 0.0f;
  if (m > 1.41421353816986083984375f) { m = m * 0.5f; e = 1.0f; }
  const float f = m - 1.0f;
  const float z = f * f;
  float p = 7.0376836292e-2f;
  p = std::fmaf(p, f, -1.1514610310e-1f);
  p = std::fmaf(p, f, 1.1676998740e-1f);
  p = std::fmaf(p, f, -1.2420140846e-1f);
  p = std::fmaf(p, f, 1.4249322787e-1f);
  p = std::fmaf(p, f, -1.6668057665e-1f);
  p = std::fmaf(p, f, 2.0000714765e-1f);
  p = std::fmaf(p, f, -2.4999993993e-1f);
  p = std::fmaf(p, f, 3.3333331174e-1f);
  float y = (f * z) * p;
  y = std::fmaf(-0.5f, z, y);
  float lg = f + y;
  lg = std::fmaf(e, 0.693147182464599609375f, lg);
  // log1p(u) = log(w) + (u - (w - 1)) / w
  const float c = (u - (w - 1.0f)) / w;
  return lg + c;
}

inline float sigmoid1(float l) { return 1.0f / (1.0f + det_expf(-l)); }  // moe_route.cu:255,330

// tanhf from the same operations: the odd Taylor polynomial through x^11 below 0.3 (truncation < 2e-9 relative),
// 1 - 2 / (exp(2|x|) + 1) above, +-1 beyond 9. The reference takes tanh from libm (src/cpu/expert_ffn.rs:91) or the
// CUDA math library (kernels/act.cu:21) and pins neither; the tests hold this one to a few ulp of the exact function.
inline float det_tanhf(float x) {
  const float a = std::fabs(x);
  if (a < 0.3f) {
    const float z = x * x;
    float p = -8.8632355e-3f;             // -1382/155925
    p = std::fmaf(p, z, 2.1869488e-2f);   //  62/2835
    p = std::fmaf(p, z, -5.3968254e-2f);  // -17/315
    p = std::fmaf(p, z, 1.3333334e-1f);   //  2/15
    p = std::fmaf(p, z, -3.3333334e-1f);  // -1/3
    return std::fmaf(x * z, p, x);
  }
  float t = 1.0f;
  if (!(a > 9.0f)) t = 1.0f - 2.0f / (det_expf(2.0f * a) + 1.0f);
  return std::copysign(t, x);
}

// moe_route.cu:332-335 (non-literal form) / moe/reference.rs:73-76
inline float sqrt_softplus(float l) {
  const float softplus = std::fmax(l, 0.0f) + det_log1pf_unit(det_expf(-std::fabs(l)));
  return std::sqrt(softplus);
}

// ---------------------------------------------------------------------------------------------
// reductions of src/cpu/expert_ffn.rs
enum Form { LANE16 = 0, LANE8 = 1, F64 = 2 };

// expert_ffn.rs:681-687
inline float pairwise16(const float* l) {
  const float low = ((l[0] + l[1]) + (l[2] + l[3])) + ((l[4] + l[5]) + (l[6] + l[7]));
  const float high = ((l[8] + l[9]) + (l[10] + l[11])) + ((l[12] + l[13]) + (l[14] + l[15]));
  return low + high;
}
// expert_ffn.rs:37-41
inline float group_sum8(const float* l) {
  return ((l[0] + l[4]) + (l[2] + l[6])) + ((l[1] + l[5]) + (l[3] + l[7]));
}

// expert_ffn.rs:689-732 (scalar_dot); weights are already BF16-rounded effective weights, which
// makes scalar_dot_e4m3 (:734-776) the same function. F64 is the reference's test oracle
// accumulation (:3290-3299): double sum in index order, one cast to f32.
float dot_form(const float* x, const uint16_t* w, int n, int form) {
  if (form == F64) {
    double acc = 0.0;
    for (int k = 0; k < n; ++k) acc += double(x[k]) * double(bf16_f32(w[k]));
    return float(acc);
  }
  float lanes[16] = {0};
  if (form == LANE16) {
    int k = 0;
    for (; k + 16 <= n; k += 16)
      for (int l = 0; l < 16; ++l) lanes[l] = std::fmaf(x[k + l], bf16_f32(w[k + l]), lanes[l]);
    for (; k < n; ++k) lanes[k % 16] = std::fmaf(x[k], bf16_f32(w[k]), lanes[k % 16]);
    return pairwise16(lanes);
  }
  const int vectors = n / 8;
  for (int v = 0; v < vectors; ++v) {
    float inner = 0.0f;
    for (int s = 0; s < 8; ++s) inner = std::fmaf(x[v * 8 + s], bf16_f32(w[v * 8 + s]), inner);
    lanes[v % 8] += inner;
  }
  for (int k = vectors * 8; k < n; ++k) lanes[k % 8] = std::fmaf(x[k], bf16_f32(w[k]), lanes[k % 8]);
  return group_sum8(lanes);
}

enum Swiglu { TWICE = 0, ONCE = 1, CLAMPED_TWICE = 2, CLAMPED_ONCE = 3, GELU_TWICE = 4 };
enum Boundary { AFTER_DOWN_BF16 = 0, BEFORE_CONTRIBUTION_BF16 = 1 };

// expert_ffn.rs:58-100 (silu_mul_value) followed by the BF16 store of :103-114.
// silu_kind 0: g / (1 + exp(-g))      (Lane8, and Lane16 with Once; moe_ffn.cu:58)
//           1: g * (1 / (1 + exp(-g))) (Lane16 with Twice; moe_ffn.cu:201-203)
//           2: g * sigmoid2(g)         (two-branch sigmoid of q38_contract.cuh:17-21, act.cu:152-156)
inline float silu_kind(float g, int kind) {
  if (kind == 0) return g / (1.0f + det_expf(-g));
  if (kind == 1) return g * (1.0f / (1.0f + det_expf(-g)));
  float s;
  if (g >= 0.0f) s = 1.0f / (1.0f + det_expf(-g));
  else { const float e = det_expf(g); s = e / (1.0f + e); }
  return g * s;
}
// tanh form of GELU, every operation rounded on its own (expert_ffn.rs:87-91; kernels/act.cu:18-22)
inline float gelu_tanh(float g) {
  const float cube = (g * g) * g;
  const float inner = 0.7978846f * (g + 0.044715f * cube);
  return (0.5f * g) * (1.0f + det_tanhf(inner));
}
inline uint16_t silu_mul_bits(uint16_t gate, uint16_t up, int rounding, float limit, int kind) {
  float g = bf16_f32(gate), u = bf16_f32(up);
  if (rounding == GELU_TWICE) return bf16_rne(bround(gelu_tanh(g)) * u);  // expert_ffn.rs:110-113: no clamp, any form
  if (rounding == CLAMPED_TWICE || rounding == CLAMPED_ONCE) {
    g = std::fmin(g, limit);
    u = std::fmin(std::fmax(u, -limit), limit);
  }
  const float act = silu_kind(g, kind);
  const float prod = (rounding == TWICE || rounding == CLAMPED_TWICE) ? bround(act) * u : act * u;
  return bf16_rne(prod);
}

// 32-lane shuffle-down tree (offsets 16,8,4,2,1): lane 0 ends with the full pairwise sum.
inline float warp_tree32(float* v) {
  for (int off = 16; off > 0; off >>= 1)
    for (int l = 0; l + off < 32; ++l) v[l] = v[l] + v[l + off];  // ascending l reads unmodified v[l+off]
  return v[0];
}

}  // namespace

// =============================================================================================
// codecs
ORC_API float orc_decode_e4m3(uint8_t c) { return decode_e4m3(c); }
ORC_API uint8_t orc_encode_e4m3(float v) { return encode_e4m3(v); }
ORC_API float orc_decode_e2m1(uint8_t c) { return decode_e2m1(c); }
ORC_API uint8_t orc_encode_e2m1(float v) { return encode_e2m1(v); }
ORC_API uint16_t orc_bf16_rne(float v) { return bf16_rne(v); }
ORC_API float orc_expf(float v) { return det_expf(v); }
ORC_API float orc_log1pf_unit(float v) { return det_log1pf_unit(v); }
ORC_API void orc_expf_array(const float* x, float* y, long n) { for (long i = 0; i < n; ++i) y[i] = det_expf(x[i]); }
ORC_API void orc_tanhf_array(const float* x, float* y, long n) { for (long i = 0; i < n; ++i) y[i] = det_tanhf(x[i]); }
ORC_API void orc_gelu_tanh_array(const float* x, float* y, long n) { for (long i = 0; i < n; ++i) y[i] = gelu_tanh(x[i]); }
ORC_API void orc_bf16_rne_array(const float* x, uint16_t* y, long n) { for (long i = 0; i < n; ++i) y[i] = bf16_rne(x[i]); }

// src/fp8.rs:138-140 with an f32 scale: bf16(decode(code) * scale).
ORC_API uint16_t orc_effective_weight(uint8_t code, float scale) { return bf16_rne(decode_e4m3(code) * scale); }
// src/fp8.rs:143-145: bf16(e2m1 * (e4m3(scale) * global)); kernels/nvfp4_linear.cu:12-14 zero rule.
ORC_API uint16_t orc_nvfp4_effective_weight(uint8_t code, uint8_t scale_code, float global) {
  return bf16_rne(decode_e2m1(code & 15u) * (decode_e4m3(scale_code) * global));
}

// Materialise BF16 effective weights of an [n,k] FP8 matrix with [ceil(n/bn), ceil(k/bk)] f32 scales
// (scale geometry: src/fp8.rs:31-36).
ORC_API void orc_dequant_fp8_block(const uint8_t* codes, const float* scales, int n, int k, int bn, int bk,
                                   uint16_t* out) {
  const int gk = (k + bk - 1) / bk;
  for (int r = 0; r < n; ++r)
    for (int c = 0; c < k; ++c)
      out[size_t(r) * k + c] = bf16_rne(decode_e4m3(codes[size_t(r) * k + c]) * scales[size_t(r / bn) * gk + c / bk]);
}
// per-output-channel BF16 scales (src/cpu/expert_ffn.rs:542-545,734-737)
ORC_API void orc_dequant_fp8_channel(const uint8_t* codes, const uint16_t* scales, int n, int k, uint16_t* out) {
  for (int r = 0; r < n; ++r)
    for (int c = 0; c < k; ++c)
      out[size_t(r) * k + c] = bf16_rne(decode_e4m3(codes[size_t(r) * k + c]) * bf16_f32(scales[r]));
}
// kernels/nvfp4_linear.cu:17-47: low nibble = even column.
ORC_API void orc_dequant_nvfp4(const uint8_t* codes, const uint8_t* scales, float global, int n, int k, uint16_t* out) {
  for (int r = 0; r < n; ++r)
    for (int c = 0; c < k; ++c) {
      const uint8_t b = codes[size_t(r) * (k / 2) + c / 2];
      const uint8_t nib = (c & 1) ? uint8_t(b >> 4) : uint8_t(b & 15u);
      const float s = decode_e4m3(scales[size_t(r) * (k / 16) + c / 16]) * global;
      out[size_t(r) * k + c] = bf16_rne(decode_e2m1(nib) * s);
    }
}

// NVFP4 weights as the FP8 matrix cores take them in the W4A8 mode (FP8 activations on NVFP4 experts; the reference's
// MMA path for NVFP4 dequantizes to BF16 instead, kernels/nvfp4_linear.cu:262-573, and has no FP8 form): each weight is
// rounded to E4M3 once more, code value x group scale / 8 (6 x 448 / 8 = 336 stays inside E4M3's 448), nearest even by
// the reference's own encoder (src/fp8.rs:85-121), and 8 x the matrix's global scale is every 128 x 128 block's scale.
// Defined by this build; the derived codes then go through the block-FP8 W8A8 arithmetic above the reference defines.
ORC_API void orc_nvfp4_to_e4m3(const uint8_t* codes, const uint8_t* scales, int n, int k, uint8_t* out) {
  for (int r = 0; r < n; ++r)
    for (int c = 0; c < k; ++c) {
      const uint8_t b = codes[size_t(r) * (k / 2) + c / 2];
      const uint8_t nib = (c & 1) ? uint8_t(b >> 4) : uint8_t(b & 15u);
      out[size_t(r) * k + c] = encode_e4m3(decode_e2m1(nib) * decode_e4m3(scales[size_t(r) * (k / 16) + c / 16]) * 0.125f);
    }
}

// =============================================================================================
// quantizers for synthetic weights (absmax block scales; the layout rules are the reference's,
// the recipe is the benchmark's: s = amax/448 per 128x128 block, code = encode(clamp(w/s))).
ORC_API void orc_quant_weight_fp8_block(const float* w, int n, int k, int bn, int bk, uint8_t* codes, float* scales) {
  const int gn = (n + bn - 1) / bn, gk = (k + bk - 1) / bk;
  for (int br = 0; br < gn; ++br)
    for (int bc = 0; bc < gk; ++bc) {
      float amax = 0.0f;
      for (int r = br * bn; r < std::min(n, (br + 1) * bn); ++r)
        for (int c = bc * bk; c < std::min(k, (bc + 1) * bk); ++c) amax = std::fmax(amax, std::fabs(w[size_t(r) * k + c]));
      const float s = amax * (1.0f / 448.0f);
      scales[size_t(br) * gk + bc] = s;
      const float d = std::fmax(s, 1.0e-12f);
      for (int r = br * bn; r < std::min(n, (br + 1) * bn); ++r)
        for (int c = bc * bk; c < std::min(k, (bc + 1) * bk); ++c)
          codes[size_t(r) * k + c] = encode_e4m3(std::fmin(448.0f, std::fmax(-448.0f, w[size_t(r) * k + c] / d)));
    }
}

// NVFP4: s16 = amax16/6, global = max(s16)/448, stored scale = e4m3(s16/global) floored at code 1
// (kernels/q38_contract.cuh:207-209), code = e2m1(w / (e4m3(scale) * global)) (:180-187).
ORC_API void orc_quant_weight_nvfp4(const float* w, int n, int k, uint8_t* codes, uint8_t* scales, float* global_out) {
  float smax = 0.0f;
  const int g = k / 16;
  std::vector<float> s16(size_t(n) * g);
  for (int r = 0; r < n; ++r)
    for (int j = 0; j < g; ++j) {
      float amax = 0.0f;
      for (int c = 0; c < 16; ++c) amax = std::fmax(amax, std::fabs(w[size_t(r) * k + j * 16 + c]));
      s16[size_t(r) * g + j] = amax / 6.0f;
      smax = std::fmax(smax, amax / 6.0f);
    }
  float global = smax / 448.0f;
  if (!(global > 0.0f)) global = 1.0f;
  *global_out = global;
  for (int r = 0; r < n; ++r)
    for (int j = 0; j < g; ++j) {
      uint8_t sc = encode_e4m3(std::fmin(448.0f, s16[size_t(r) * g + j] / global));
      if (sc == 0) sc = 1;
      scales[size_t(r) * g + j] = sc;
      const float s = decode_e4m3(sc) * global;
      for (int c = 0; c < 16; c += 2) {
        const uint8_t lo = encode_e2m1(w[size_t(r) * k + j * 16 + c] / s);
        const uint8_t hi = encode_e2m1(w[size_t(r) * k + j * 16 + c + 1] / s);
        codes[size_t(r) * (k / 2) + (j * 16 + c) / 2] = uint8_t(lo | (hi << 4));
      }
    }
}

// kernels/fp8_linear.cu:12-48 (fp8_quant_f32_128): per (row, 128-group) scale = amax * (1/448) as
// an f32 multiply, divisor max(scale, 1e-12), code = encode(clamp(x / divisor, +-448)).
ORC_API void orc_quant_act_fp8_128(const uint16_t* x, int m, int k, uint8_t* codes, float* scales) {
  const int groups = (k + 127) / 128;
  for (int r = 0; r < m; ++r)
    for (int g = 0; g < groups; ++g) {
      float amax = 0.0f;
      const int end = std::min(k, (g + 1) * 128);
      for (int c = g * 128; c < end; ++c) amax = std::fmax(amax, std::fabs(bf16_f32(x[size_t(r) * k + c])));
      const float scale = amax * (1.0f / 448.0f);
      scales[size_t(r) * groups + g] = scale;
      const float divisor = std::fmax(scale, 1.0e-12f);
      for (int c = g * 128; c < end; ++c)
        codes[size_t(r) * k + c] = encode_e4m3(std::fmin(448.0f, std::fmax(-448.0f, bf16_f32(x[size_t(r) * k + c]) / divisor)));
    }
}

// =============================================================================================
// router
// kernels/moe_route.cu:392-403,496-560: one ascending FP32 fma chain per (row, expert), BF16 store.
ORC_API void orc_route_logits_bf16(const uint16_t* x, const uint16_t* w, uint16_t* logits, int rows, int experts, int hidden) {
  for (int r = 0; r < rows; ++r)
    for (int e = 0; e < experts; ++e) {
      float acc = 0.0f;
      for (int k = 0; k < hidden; ++k) acc = std::fmaf(bf16_f32(x[size_t(r) * hidden + k]), bf16_f32(w[size_t(e) * hidden + k]), acc);
      logits[size_t(r) * experts + e] = bf16_rne(acc);
    }
}

// FP32 logits. The reference takes these from a BLAS GEMM whose summation order is undefined
// (src/backend/cuda/moe/route.rs:505-562), so any order is within its contract; the order fixed
// here is the one the HIP kernel uses, so ids can be compared bit for bit: 256 partial chains,
// partial p owning the 8-element vectors v = p, p+256, ... with fma in ascending order; the 256
// partials are summed by a balanced pairwise tree in natural order (adjacent pairs, then pairs of
// pairs, ...). PARITY UNPINNED at bit level (tolerance-checked against float64 in the tests, as
// the reference's own tests do).
ORC_API void orc_route_logits_f32(const uint16_t* x, const uint16_t* w, float* logits, int rows, int experts, int hidden) {
  const int vectors = hidden / 8;
  for (int r = 0; r < rows; ++r)
    for (int e = 0; e < experts; ++e) {
      float part[256];
      for (int p = 0; p < 256; ++p) {
        float acc = 0.0f;
        for (int v = p; v < vectors; v += 256)
          for (int s = 0; s < 8; ++s)
            acc = std::fmaf(bf16_f32(x[size_t(r) * hidden + v * 8 + s]), bf16_f32(w[size_t(e) * hidden + v * 8 + s]), acc);
        part[p] = acc;
      }
      for (int width = 1; width < 256; width <<= 1)
        for (int p = 0; p < 256; p += 2 * width) part[p] = part[p] + part[p + width];
      logits[size_t(r) * experts + e] = part[0];
    }
}

namespace {
// K rounds of arg-max under (score desc, id asc) over not-yet-taken experts
// (kernels/moe_route.cu:205-235); returns ids in selection order.
void select_topk(const float* score, const bool* allowed, int experts, int top_k, int* out) {
  std::vector<char> taken(experts, 0);
  for (int r = 0; r < top_k; ++r) {
    int best = -1;
    for (int e = 0; e < experts; ++e) {
      if (taken[e] || (allowed && !allowed[e])) continue;
      if (best < 0 || score[e] > score[best]) best = e;  // strict > keeps the lower id on ties
    }
    out[r] = best;
    if (best >= 0) taken[best] = 1;
  }
}
}  // namespace

// kernels/moe_route.cu:154-242 (moe_route_select): FP32 softmax over BF16 logits with the max and
// the sum taken by 32-lane shuffle-down trees per warp and again over the per-warp partials;
// weights = p / (sum of selected p in selection order), BF16 store.
ORC_API void orc_route_topk_softmax(const uint16_t* logits, int* ids, uint16_t* weights, int rows, int experts, int top_k) {
  const int nthr = (experts + 31) & ~31, nw = nthr / 32;
  std::vector<float> ev(nthr), prob(experts);
  for (int r = 0; r < rows; ++r) {
    float mx = -INFINITY;
    for (int e = 0; e < experts; ++e) mx = std::fmax(mx, bf16_f32(logits[size_t(r) * experts + e]));
    for (int e = 0; e < nthr; ++e) ev[e] = e < experts ? det_expf(bf16_f32(logits[size_t(r) * experts + e]) - mx) : 0.0f;
    float partial[32];
    for (int w = 0; w < 32; ++w) partial[w] = 0.0f;
    for (int w = 0; w < nw; ++w) {
      float lanes[32];
      for (int l = 0; l < 32; ++l) lanes[l] = ev[w * 32 + l];
      partial[w] = warp_tree32(lanes);
    }
    const float sum = warp_tree32(partial);
    for (int e = 0; e < experts; ++e) prob[e] = ev[e] / sum;
    std::vector<int> sel(top_k);
    select_topk(prob.data(), nullptr, experts, top_k, sel.data());
    float tsum = 0.0f;
    for (int j = 0; j < top_k; ++j) tsum += prob[sel[j]];
    for (int j = 0; j < top_k; ++j) {
      ids[size_t(r) * top_k + j] = sel[j];
      weights[size_t(r) * top_k + j] = bf16_rne(prob[sel[j]] / tsum);
    }
  }
}

// kernels/moe_route.cu:244-301 (moe_route_select_sigmoid)
ORC_API void orc_route_topk_sigmoid(const uint16_t* logits, int* ids, uint16_t* weights, int rows, int experts, int top_k) {
  std::vector<float> score(experts);
  std::vector<int> sel(top_k);
  for (int r = 0; r < rows; ++r) {
    for (int e = 0; e < experts; ++e) score[e] = sigmoid1(bf16_f32(logits[size_t(r) * experts + e]));
    select_topk(score.data(), nullptr, experts, top_k, sel.data());
    float tsum = 0.0f;
    for (int j = 0; j < top_k; ++j) tsum += score[sel[j]];
    for (int j = 0; j < top_k; ++j) {
      ids[size_t(r) * top_k + j] = sel[j];
      weights[size_t(r) * top_k + j] = bf16_rne(score[sel[j]] / (tsum + 1.0e-20f));
    }
  }
}

// kernels/moe_route.cu:315-390 (moe_route_select_noaux) and its host twin
// src/backend/cuda/moe/reference.rs:79-131: select on score+bias, weight = score / (sum + 1e-20) *
// routed_scaling with the sum accumulated in selection order. score_mode 0 sigmoid, 1 sqrt-softplus.
// n_group > 1 adds the DeepSeek-V3 group filter, which the reference does not implement
// (src/model_spec.rs:3832-3841 requires n_group == topk_group == 1): group score = sum of the two
// largest score+bias values of the group, keep the topk_group best groups under (score desc,
// group id asc), drop the other experts. PARITY UNPINNED for n_group > 1; n_group == 1 is the
// reference path exactly.
ORC_API void orc_route_topk_noaux(const float* logits, const float* bias, int* ids, float* weights, int rows, int experts,
                                  int top_k, int score_mode, float routed_scaling, int n_group, int topk_group) {
  std::vector<float> score(experts), sel_score(experts);
  std::vector<int> sel(top_k);
  std::vector<char> allowed_c(experts);
  for (int r = 0; r < rows; ++r) {
    for (int e = 0; e < experts; ++e) {
      const float l = logits[size_t(r) * experts + e];
      score[e] = score_mode == 0 ? sigmoid1(l) : sqrt_softplus(l);
      sel_score[e] = score[e] + (bias ? bias[size_t(r) * experts + e] : 0.0f);
    }
    const bool* allowed = nullptr;
    std::vector<char> keep;
    if (n_group > 1) {
      const int per = experts / n_group;
      std::vector<float> gscore(n_group);
      for (int g = 0; g < n_group; ++g) {
        float a = -INFINITY, b = -INFINITY;  // largest, second largest
        for (int e = g * per; e < (g + 1) * per; ++e) {
          const float v = sel_score[e];
          if (v > a) { b = a; a = v; } else if (v > b) { b = v; }
        }
        gscore[g] = a + b;
      }
      std::vector<int> gsel(topk_group);
      select_topk(gscore.data(), nullptr, n_group, topk_group, gsel.data());
      std::fill(allowed_c.begin(), allowed_c.end(), 0);
      for (int j = 0; j < topk_group; ++j)
        for (int e = gsel[j] * per; e < (gsel[j] + 1) * per; ++e) allowed_c[e] = 1;
      allowed = reinterpret_cast<const bool*>(allowed_c.data());
    }
    select_topk(sel_score.data(), allowed, experts, top_k, sel.data());
    float tsum = 0.0f;
    for (int j = 0; j < top_k; ++j) tsum += score[sel[j]];
    for (int j = 0; j < top_k; ++j) {
      ids[size_t(r) * top_k + j] = sel[j];
      weights[size_t(r) * top_k + j] = (score[sel[j]] / (tsum + 1.0e-20f)) * routed_scaling;
    }
  }
}

// Plain descending top-k with lower-id tie break (src/backend/cuda/moe/reference.rs:35-71).
ORC_API void orc_topk_ids(const float* scores, int n, int k, int* ids) { select_topk(scores, nullptr, n, k, ids); }

// =============================================================================================
// SwiGLU boundary (expert_ffn.rs:58-114; act.cu:24-159)
ORC_API uint16_t orc_silu_mul(uint16_t gate, uint16_t up, int rounding, float limit, int kind) {
  return silu_mul_bits(gate, up, rounding, limit, kind);
}
ORC_API void orc_silu_mul_array(const uint16_t* gate, const uint16_t* up, uint16_t* out, long n, int rounding, float limit, int kind) {
  for (long i = 0; i < n; ++i) out[i] = silu_mul_bits(gate[i], up[i], rounding, limit, kind);
}

ORC_API float orc_dot(const float* x, const uint16_t* w, int n, int form) { return dot_form(x, w, n, form); }

// One (row, choice) contribution over BF16 effective weights: src/cpu/expert_ffn.rs:431-497
// (compute) and :592-679 (compute_fp8, identical once weights are BF16-rounded effective weights).
// form F64 restates the reference's own test oracle (:3281-3320, :3725-3790): FP64 accumulation,
// SiLU in FP64 as g * (1/(1+exp(-g))), the same BF16 boundaries.
// gate/up [I,H], down [H,I] row-major BF16; act_out (optional) receives the BF16 activation [I];
// apply_weight 0 leaves the down output as bf16(d) (shared expert, moe_ffn.cu:300).
ORC_API void orc_expert_ffn(const uint16_t* x, const uint16_t* gate, const uint16_t* up, const uint16_t* down, int H, int I,
                            float routing, int rounding, float limit, int boundary, int form, int silu_k, int apply_weight,
                            uint16_t* out, uint16_t* act_out) {
  std::vector<float> xf(H), af(I);
  for (int k = 0; k < H; ++k) xf[k] = bf16_f32(x[k]);
  for (int j = 0; j < I; ++j) {
    const uint16_t g = bf16_rne(dot_form(xf.data(), gate + size_t(j) * H, H, form));
    const uint16_t u = bf16_rne(dot_form(xf.data(), up + size_t(j) * H, H, form));
    uint16_t a;
    if (form == F64) {
      const double gd = double(bf16_f32(g)), ud = double(bf16_f32(u));
      const double silu = double(bround(float(gd * (1.0 / (1.0 + std::exp(-gd))))));
      a = bf16_rne(float(silu * ud));
    } else {
      a = silu_mul_bits(g, u, rounding, limit, silu_k);
    }
    af[j] = bf16_f32(a);
    if (act_out) act_out[j] = a;
  }
  for (int d = 0; d < H; ++d) {
    const float lin = dot_form(af.data(), down + size_t(d) * I, I, form);
    float v;
    if (!apply_weight) v = bround(lin);
    else if (boundary == AFTER_DOWN_BF16) v = bround(lin) * routing;
    else v = lin * routing;
    out[d] = bf16_rne(v);
  }
}

// The second half of orc_expert_ffn from a given BF16 activation [I] (src/cpu/expert_ffn.rs:470-497): lets a test
// judge the down stage on the activations the device itself produced. Equal to orc_expert_ffn bit for bit when fed
// its act_out (tests/test_oracle_golden.py).
ORC_API void orc_expert_down(const uint16_t* act, const uint16_t* down, int H, int I, float routing, int boundary, int form,
                             int apply_weight, uint16_t* out) {
  std::vector<float> af(I);
  for (int j = 0; j < I; ++j) af[j] = bf16_f32(act[j]);
  for (int d = 0; d < H; ++d) {
    const float lin = dot_form(af.data(), down + size_t(d) * I, I, form);
    float v;
    if (!apply_weight) v = bround(lin);
    else if (boundary == AFTER_DOWN_BF16) v = bround(lin) * routing;
    else v = lin * routing;
    out[d] = bf16_rne(v);
  }
}

// =============================================================================================
// W8A8 block linear: kernels/q38_contract.cuh:239-279 (fp8_block_decode<float,128>): per output
// and per 128-group, lane L of 32 chains fma over elements L, L+32, L+64, L+96, a shuffle-down
// tree 16..1 gives the group sum, then total = fma(sum, sw*sx, total); BF16 store.
// order 1 = FP64 reference (src/backend/cuda/linear.rs:2105-2142) rounded f64 -> f32 -> bf16.
ORC_API void orc_linear_fp8_block_w8a8(const uint8_t* w, const float* sw, const uint8_t* xq, const float* sx, int m, int n,
                                       int k, int order, uint16_t* y, float* y_f32) {
  const int groups = (k + 127) / 128;
  for (int r = 0; r < m; ++r)
    for (int c = 0; c < n; ++c) {
      float result;
      if (order == 1) {
        double sum = 0.0;
        for (int i = 0; i < k; ++i)
          sum += (double(decode_e4m3(w[size_t(c) * k + i])) * double(sw[size_t(c / 128) * groups + i / 128])) *
                 (double(decode_e4m3(xq[size_t(r) * k + i])) * double(sx[size_t(r) * groups + i / 128]));
        result = float(sum);
      } else {
        float total = 0.0f;
        for (int g = 0; g < groups; ++g) {
          float lanes[32];
          for (int l = 0; l < 32; ++l) {
            float s = 0.0f;
            for (int off = l; off < 128; off += 32) {
              const int i = g * 128 + off;
              if (i < k) s = std::fmaf(decode_e4m3(w[size_t(c) * k + i]), decode_e4m3(xq[size_t(r) * k + i]), s);
            }
            lanes[l] = s;
          }
          const float sum = warp_tree32(lanes);
          const float scale = sw[size_t(c / 128) * groups + g] * sx[size_t(r) * groups + g];
          total = std::fmaf(sum, scale, total);
        }
        result = total;
      }
      if (y) y[size_t(r) * n + c] = bf16_rne(result);
      if (y_f32) y_f32[size_t(r) * n + c] = result;
    }
}

// One (row, choice) contribution on the block-F32 W8A8 path, the composition the reference runs for block-FP8 models
// (NativeMoe::run, src/backend/cuda/moe/decode.rs:1187-1297): fp8_quant_f32_128 on x (kernels/fp8_linear.cu:12-48),
// gate and up through fp8_block_decode to BF16 (kernels/moe_ffn.cu:870-891), SwiGLU on the BF16 pair
// (kernels/act.cu:125-159), fp8_quant_f32_128 on the activation, down to BF16, then the routing weight
// (kernels/moe_ffn.cu:894-908: bf16(float(bf16 down) * w); BeforeContributionBf16 multiplies the FP32 sum instead).
// gate/up codes [I,H] + scales [ceil(I/128), H/128]; down codes [H,I] + scales [ceil(H/128), I/128].
ORC_API void orc_expert_ffn_w8a8(const uint16_t* x, const uint8_t* gate, const float* sgate, const uint8_t* up, const float* sup,
                                 const uint8_t* down, const float* sdown, int H, int I, float routing, int rounding, float limit,
                                 int boundary, int order, int silu_k, int apply_weight, uint16_t* out, uint16_t* act_out) {
  std::vector<uint8_t> xq(H), aq(I);
  std::vector<float> sx((H + 127) / 128), sa((I + 127) / 128), lin(H);
  std::vector<uint16_t> g(I), u(I), act(I), d(H);
  orc_quant_act_fp8_128(x, 1, H, xq.data(), sx.data());
  orc_linear_fp8_block_w8a8(gate, sgate, xq.data(), sx.data(), 1, I, H, order, g.data(), nullptr);
  orc_linear_fp8_block_w8a8(up, sup, xq.data(), sx.data(), 1, I, H, order, u.data(), nullptr);
  for (int j = 0; j < I; ++j) act[j] = silu_mul_bits(g[j], u[j], rounding, limit, silu_k);
  if (act_out) std::memcpy(act_out, act.data(), size_t(I) * 2);
  orc_quant_act_fp8_128(act.data(), 1, I, aq.data(), sa.data());
  orc_linear_fp8_block_w8a8(down, sdown, aq.data(), sa.data(), 1, H, I, order, d.data(), lin.data());
  for (int c = 0; c < H; ++c) {
    float v;
    if (!apply_weight) v = bf16_f32(d[c]);
    else if (boundary == AFTER_DOWN_BF16) v = bf16_f32(d[c]) * routing;
    else v = lin[c] * routing;
    out[c] = bf16_rne(v);
  }
}

// W8A16 skinny linear with the reduction of src/fp8.rs:245-287 (host mirror of
// kernels/fp8_linear.cu:407-487) over BF16 effective weights [n,k]; the NVFP4 twin is
// src/fp8.rs:290-340 (kernels/nvfp4_linear.cu:50-229). kind 0 = FP8 order, 1 = NVFP4 order,
// 2 = FP64 accumulate.
ORC_API void orc_linear_skinny(const uint16_t* weight, const uint16_t* x, int m, int n, int k, int kind, uint16_t* y) {
  for (int r = 0; r < m; ++r) {
    const uint16_t* in = x + size_t(r) * k;
    for (int c = 0; c < n; ++c) {
      const uint16_t* row = weight + size_t(c) * k;
      if (kind == 2) {
        double acc = 0.0;
        for (int i = 0; i < k; ++i) acc += double(bf16_f32(row[i])) * double(bf16_f32(in[i]));
        y[size_t(r) * n + c] = bf16_rne(float(acc));
        continue;
      }
      float lanes[32];
      for (int lane = 0; lane < 32; ++lane) {
        float sums[4] = {0, 0, 0, 0};
        if (k % 1024 == 0) {
          for (int base = 0; base < k; base += 1024) {
            if (kind == 0) {
              for (int word = 0; word < 4; ++word)
                for (int byte = 0; byte < 4; ++byte) {
                  int col = base + lane * 16 + word * 4 + byte;
                  sums[byte] = std::fmaf(bf16_f32(row[col]), bf16_f32(in[col]), sums[byte]);
                  col += 512;
                  const int idx = (byte + 2) & 3;
                  sums[idx] = std::fmaf(bf16_f32(row[col]), bf16_f32(in[col]), sums[idx]);
                }
            } else {
              const int col = base + lane * 32;
              for (int word = 0; word < 4; ++word)
                for (int byte = 0; byte < 4; ++byte) {
                  const int lo = col + 8 * word + 2 * byte, hi = lo + 1;
                  const float acc = std::fmaf(bf16_f32(row[lo]), bf16_f32(in[lo]), sums[byte]);
                  sums[byte] = std::fmaf(bf16_f32(row[hi]), bf16_f32(in[hi]), acc);
                }
            }
          }
        } else if (kind == 0) {
          for (int col = lane; col < k; col += 32) sums[0] = std::fmaf(bf16_f32(row[col]), bf16_f32(in[col]), sums[0]);
        } else {
          for (int pair = lane; pair < k / 2; pair += 32) {
            const int lo = 2 * pair, hi = lo + 1;
            const float acc = std::fmaf(bf16_f32(row[lo]), bf16_f32(in[lo]), sums[0]);
            sums[0] = std::fmaf(bf16_f32(row[hi]), bf16_f32(in[hi]), acc);
          }
        }
        lanes[lane] = (sums[0] + sums[1]) + (sums[2] + sums[3]);
      }
      y[size_t(r) * n + c] = bf16_rne(warp_tree32(lanes));
    }
  }
}

// =============================================================================================
// combine (kernels/moe_combine.cu)
namespace {
// moe_combine.cu:51-69: stable insertion sort of the active choices by ascending expert id.
int order_row(const int* ids, const uint32_t* active, int a0, int top_k, int* order) {
  int live = 0;
  for (int c = 0; c < top_k; ++c) {
    if (active && active[a0 + c] == 0u) continue;
    int p = live;
    while (p > 0 && ids[a0 + order[p - 1]] > ids[a0 + c]) { order[p] = order[p - 1]; --p; }
    order[p] = c;
    ++live;
  }
  return live;
}
}  // namespace

// moe_combine.cu:21-49: scale[r] = bf16(sigmoid(bf16(dot))) with the dot strided over 256 threads,
// products added (not fused), 32-lane trees per warp then over the 8 warp partials.
ORC_API void orc_shared_scale(const uint16_t* x, const uint16_t* seg, uint16_t* scale, int rows, int hidden) {
  for (int r = 0; r < rows; ++r) {
    float part[256];
    for (int t = 0; t < 256; ++t) {
      float p = 0.0f;
      for (int c = t; c < hidden; c += 256) p += bf16_f32(x[size_t(r) * hidden + c]) * bf16_f32(seg[c]);
      part[t] = p;
    }
    float red[32];
    for (int w = 0; w < 32; ++w) red[w] = 0.0f;
    for (int w = 0; w < 8; ++w) red[w] = warp_tree32(part + w * 32);
    const float v = warp_tree32(red);
    scale[r] = bf16_rne(1.0f / (1.0f + det_expf(-bround(v))));
  }
}

// mode 0: moe_combine (:71-93) FP32 sum ascending id -> bf16, + bf16(scale*shared) in BF16
// mode 1: moe_combine_ungated (:95-116) same, + shared in BF16
// mode 2: moe_combine_bf16 (:592-613) BF16 running sum ascending id, + shared in BF16
// mode 3: moe_combine_accum fp32_accum=1 (:541-591) choice order, shared added in FP32, one round
// mode 4: moe_combine_accum fp32_accum=0: choice order FP32 -> bf16, + shared -> bf16
// mode 5: moe_combine_routed (:176-196) FP32 sum ascending id -> bf16, no shared
// mode 6: descending-id BF16 running sum + gated shared (reference.rs:559-573, order-noise control)
// mode 7: ascending-id BF16 running sum + gated shared (reference.rs:559-573 AscendingBf16)
ORC_API void orc_combine(const uint16_t* contributions, const uint16_t* shared, const uint16_t* scale, const int* ids,
                         const uint32_t* active, uint16_t* y, int rows, int top_k, int hidden, int mode) {
  std::vector<int> order(top_k);
  for (int r = 0; r < rows; ++r) {
    const int a0 = r * top_k;
    int live;
    if (mode == 3 || mode == 4) { live = top_k; for (int c = 0; c < top_k; ++c) order[c] = c; }
    else live = order_row(ids, active, a0, top_k, order.data());
    if (mode == 6) std::reverse(order.begin(), order.begin() + live);
    for (int d = 0; d < hidden; ++d) {
      const float sh = shared ? bf16_f32(shared[size_t(r) * hidden + d]) : 0.0f;
      auto c = [&](int k) { return bf16_f32(contributions[(size_t(a0) + order[k]) * hidden + d]); };
      float out;
      if (mode == 2 || mode == 6 || mode == 7) {
        float acc = 0.0f;
        for (int k = 0; k < live; ++k) acc = bround(acc + c(k));
        const float add = mode == 2 ? sh : bround(bf16_f32(scale[r]) * sh);
        out = bround(acc + add);
      } else {
        float acc = 0.0f;
        for (int k = 0; k < live; ++k) acc += c(k);
        if (mode == 0) out = bround(bround(acc) + bround(bf16_f32(scale[r]) * sh));
        else if (mode == 1 || mode == 4) out = bround(bround(acc) + sh);
        else if (mode == 3) out = bround(acc + sh);
        else out = bround(acc);
      }
      y[size_t(r) * hidden + d] = bf16_rne(out);
    }
  }
}

// kernels/moe_ffn.cu:894-908 (moe_ffn_weight_f32): contrib = bf16(float(down_bf16) * w_f32)
ORC_API void orc_weight_f32(const uint16_t* down, const float* w, uint16_t* contrib, int assignments, int hidden) {
  for (int a = 0; a < assignments; ++a)
    for (int d = 0; d < hidden; ++d) contrib[size_t(a) * hidden + d] = bf16_rne(bf16_f32(down[size_t(a) * hidden + d]) * w[a]);
}

// =============================================================================================
// reference fixture generator (src/backend/cuda/moe/reference.rs:204-224)
namespace {
uint64_t mix(uint64_t salt, uint64_t a, uint64_t b, uint64_t c) {
  uint64_t z = salt + a * 0x9E3779B1ull + b * 0x85EBCA77ull + c * 0xC2B2AE3Dull;
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}
}  // namespace
ORC_API float orc_fixture_unit(uint64_t salt, uint64_t a, uint64_t b, uint64_t c) {
  return float(mix(salt, a, b, c) >> 40) / 8388608.0f - 1.0f;
}
ORC_API uint64_t orc_fixture_seed(uint32_t variant, uint64_t slot) {
  return uint64_t(variant) * 0x9E3779B97F4A7C15ull ^ slot * 0xC2B2AE3D27D4EB4Full;
}
// out[i0*n1*n2 + i1*n2 + i2] = bf16(unit(salt, a0+i0, i1, i2) * scale)
ORC_API void orc_fixture_fill(uint64_t salt, uint64_t a0, int n0, int n1, int n2, float scale, uint16_t* out) {
  for (int i0 = 0; i0 < n0; ++i0)
    for (int i1 = 0; i1 < n1; ++i1)
      for (int i2 = 0; i2 < n2; ++i2)
        out[(size_t(i0) * n1 + i1) * n2 + i2] = bf16_rne(orc_fixture_unit(salt, a0 + i0, i1, i2) * scale);
}
// sine fixture of src/cpu/expert_ffn.rs:3077-3079
ORC_API void orc_pattern_fill(uint64_t seed0, double phase, long n, uint16_t* out) {
  for (long i = 0; i < n; ++i) out[i] = bf16_rne(float(std::sin(double(seed0 + uint64_t(i)) * 0.6180339887498949 + phase) * 0.75));
}

// =============================================================================================
// E8M0 block-32 experts of the DeepSeek-V4.1 contract: W4A8 routed experts (E2M1 weights, one E8M0 scale per 32
// elements of a row) and the W8A8 shared expert (E4M3 weights, one E8M0 scale per 32x32 block), activations quantized
// to E4M3 with one E8M0 scale per 32 elements, dots as exact integers (kernels/q38_contract.cuh:53-101,140-170;
// kernels/moe_ffn.cu:601-700).
namespace {
// q38_contract.cuh:132-137
inline int act_quant_log2_ceil(float v) {
  uint32_t bits;
  std::memcpy(&bits, &v, 4);
  const int exponent = int((bits >> 23) & 0xffu) - 127;
  return exponent + ((bits & 0x7fffffu) != 0u ? 1 : 0);
}
// q38_contract.cuh:53-90: per 32 elements the integer sum of av * bv (E4M3 activation as an integer multiple of 2^-9,
// E2M1 weight as a multiple of 2^-1 or E4M3 weight as a multiple of 2^-9), then total = fma(sum, 2^(sa + sb - bias),
// total) in FP64, groups in ascending order. Returns false on a NaN code or a 0xff scale (the reference traps).
bool scaled_dot_exact(bool packed, const uint8_t* w, const uint8_t* sw, const uint8_t* x, const uint8_t* sx, int k, double* out) {
  static const uint32_t e2m1_int[8] = {0, 1, 2, 3, 4, 6, 8, 12};
  double total = 0.0;
  for (int group = 0; group < k / 32; ++group) {
    long long sum = 0;
    for (int lane = 0; lane < 32; ++lane) {
      const int inner = group * 32 + lane;
      const uint8_t a = x[inner];
      if ((a & 127) == 127) return false;
      const uint32_t ae = (a >> 3) & 15;
      const uint32_t av = ae ? (8u + (a & 7u)) << (ae - 1) : (a & 7u);
      uint32_t bv, sign;
      if (packed) {
        const uint8_t b = (w[inner / 2] >> (4 * (inner & 1))) & 15;
        bv = e2m1_int[b & 7];
        sign = (a >> 7) ^ (b >> 3);
      } else {
        const uint8_t b = w[inner];
        if ((b & 127) == 127) return false;
        const uint32_t be = (b >> 3) & 15;
        bv = be ? (8u + (b & 7u)) << (be - 1) : (b & 7u);
        sign = uint32_t(a ^ b) >> 7;
      }
      const long long prod = (long long)(uint64_t(av) * bv);
      sum += sign ? -prod : prod;
    }
    const uint8_t sa = sx[group], sb = sw[group];
    if (sa == 255 || sb == 255) return false;
    const int exponent = int(sa) + int(sb) - (packed ? 264 : 272);
    total = std::fma(double(sum), std::ldexp(1.0, exponent), total);
  }
  *out = total;
  return true;
}
// q38_contract.cuh:92-98: FP64 -> BF16 through FP32 with the double-rounding tie repaired
inline uint16_t bf16_round_f64(double value) {
  float rounded = float(value);
  uint32_t bits;
  std::memcpy(&bits, &rounded, 4);
  if ((bits & 65535u) == 32768u && double(rounded) != value)
    rounded = std::nextafterf(rounded, value < double(rounded) ? -INFINITY : INFINITY);
  return bf16_rne(rounded);
}
}  // namespace

// q38_contract.cuh:153-170 (act_quant32) over rows of k BF16 values, k a multiple of 32: amax floored at 1e-4, scale
// 2^ceil(log2(amax / 448)) as an E8M0 code, codes = E4M3 RNE of value / scale clamped to +-448. Returns 0, or -1 when
// an exponent leaves [-127, 127] (the reference traps).
ORC_API int orc_act_quant_e8m0(const uint16_t* x, int rows, int k, uint8_t* codes, uint8_t* scales) {
  for (int r = 0; r < rows; ++r)
    for (int g = 0; g < k / 32; ++g) {
      const uint16_t* src = x + size_t(r) * k + size_t(g) * 32;
      float amax = 0.0f;
      for (int i = 0; i < 32; ++i) amax = std::fmax(amax, std::fabs(bf16_f32(src[i])));
      amax = std::fmax(amax, 1e-4f);
      const int exponent = act_quant_log2_ceil(amax * (1.0f / 448.0f));
      if (exponent < -127 || exponent > 127) return -1;
      const float scale = std::ldexp(1.0f, exponent);
      for (int i = 0; i < 32; ++i)
        codes[size_t(r) * k + size_t(g) * 32 + i] = encode_e4m3(std::fmin(448.0f, std::fmax(-448.0f, bf16_f32(src[i]) / scale)));
      scales[size_t(r) * (k / 32) + g] = uint8_t(exponent + 127);
    }
  return 0;
}

// One exact dot, exposed for the tests: packed = 1 E2M1 weights (two per byte, low nibble first), 0 E4M3 weights.
ORC_API int orc_scaled_dot_exact(int packed, const uint8_t* w, const uint8_t* sw, const uint8_t* x, const uint8_t* sx, int k,
                                 double* total, uint16_t* rounded) {
  double t;
  if (!scaled_dot_exact(packed != 0, w, sw, x, sx, k, &t)) return -1;
  *total = t;
  *rounded = bf16_round_f64(t);
  return 0;
}

// One expert on one token in the exact contract (kernels/moe_ffn.cu:601-657; host sequence
// src/backend/cuda/moe/w4a8.rs:268-360): quantize x, gate/up exact dots -> BF16 each, gate clamped from above, up on
// both sides, FP32 SiLU times up times the routed weight, one BF16 cast; quantize that row; down exact dots -> BF16.
// packed = 1: E2M1 codes [N, K/2] with scales [N, K/32]; packed = 0: E4M3 codes [N, K] with scales [ceil(N/32), K/32].
// act_out (optional) receives the BF16 down-input row [I].
ORC_API int orc_expert_ffn_e8m0(int packed, const uint16_t* x, const uint8_t* gate, const uint8_t* sgate, const uint8_t* up,
                                const uint8_t* sup, const uint8_t* down, const uint8_t* sdown, int H, int I, float limit,
                                float route_weight, uint16_t* out, uint16_t* act_out) {
  if (H % 32 || I % 32 || !(limit > 0.0f)) return -2;
  std::vector<uint8_t> xc(H), xs(H / 32), hc(I), hs(I / 32);
  std::vector<uint16_t> h(I);
  if (orc_act_quant_e8m0(x, 1, H, xc.data(), xs.data())) return -1;
  const int stride_gu = packed ? H / 2 : H, stride_d = packed ? I / 2 : I;
  for (int j = 0; j < I; ++j) {
    const int sr = packed ? j : j / 32;
    double g64, u64;
    if (!scaled_dot_exact(packed, gate + size_t(j) * stride_gu, sgate + size_t(sr) * (H / 32), xc.data(), xs.data(), H, &g64)) return -1;
    if (!scaled_dot_exact(packed, up + size_t(j) * stride_gu, sup + size_t(sr) * (H / 32), xc.data(), xs.data(), H, &u64)) return -1;
    const float g = std::fmin(bf16_f32(bf16_round_f64(g64)), limit);
    const float u = std::fmax(std::fmin(bf16_f32(bf16_round_f64(u64)), limit), -limit);
    h[j] = bf16_rne(((g / (1.0f + det_expf(-g))) * u) * route_weight);
  }
  if (act_out) std::memcpy(act_out, h.data(), size_t(I) * 2);
  if (orc_act_quant_e8m0(h.data(), 1, I, hc.data(), hs.data())) return -1;
  for (int d = 0; d < H; ++d) {
    const int sr = packed ? d : d / 32;
    double t;
    if (!scaled_dot_exact(packed, down + size_t(d) * stride_d, sdown + size_t(sr) * (I / 32), hc.data(), hs.data(), I, &t)) return -1;
    out[d] = bf16_round_f64(t);
  }
  return 0;
}

// ---------------------------------------------------------------------------------------------
// The FP32-chain variant of the same formats (kernels/moe_ffn.cu:469-576 W4A8, :764-865 W8A8 shared expert): one
// 32-lane warp per output row, FP32 fma chains, the block scales multiply chunk sums in FP32, xor-butterfly warp sum.
namespace {
// q38_contract.cuh:36-42
inline float e8m0_decode_f32(uint8_t code) {
  if (code == 0xffu) return NAN;
  return std::ldexp(1.0f, int(code) - 127);
}
// kernels/moe_ffn.cu:425-431
inline float e2m1_f32(unsigned nibble) {
  const unsigned u = nibble & 7u;
  uint32_t bits = 0x3F000000u + u * 0x400000u;
  if (u == 0u) bits = 0u;
  else if (u == 1u) bits = 0x3F000000u;
  bits |= (nibble & 8u) << 28;
  float f;
  std::memcpy(&f, &bits, 4);
  return f;
}
// kernels/moe_ffn.cu:437-442: every lane receives the total
inline float warp_sum_xor32(float* v) {
  for (int off = 16; off > 0; off >>= 1) {
    float n[32];
    for (int l = 0; l < 32; ++l) n[l] = v[l] + v[l ^ off];
    std::memcpy(v, n, sizeof(n));
  }
  return v[0];
}
// kernels/moe_ffn.cu:472-505: lane L takes the 8-element chunks L, L+32, ...
float w4a8_dot_f32(const uint8_t* w, const uint8_t* sw, const uint8_t* x, const uint8_t* sx, int k) {
  float lanes[32];
  const int chunks = k / 8;
  for (int lane = 0; lane < 32; ++lane) {
    float acc = 0.0f;
    for (int chunk = lane; chunk < chunks; chunk += 32) {
      float sum = 0.0f;
      for (int i = 0; i < 4; ++i) {
        const unsigned byte = w[size_t(chunk) * 4 + i];
        sum = std::fmaf(e2m1_f32(byte & 0xfu), decode_e4m3(x[size_t(chunk) * 8 + 2 * i]), sum);
        sum = std::fmaf(e2m1_f32(byte >> 4), decode_e4m3(x[size_t(chunk) * 8 + 2 * i + 1]), sum);
      }
      const int group = chunk / 4;
      acc = std::fmaf(sum, e8m0_decode_f32(sx[group]) * e8m0_decode_f32(sw[group]), acc);
    }
    lanes[lane] = acc;
  }
  return warp_sum_xor32(lanes);
}
// kernels/moe_ffn.cu:768-797: lane = (block slot lane >> 2, quarter lane & 3); eight K blocks per pass
float w8a8_dot_f32(const uint8_t* w, const uint8_t* sw, const uint8_t* x, const uint8_t* sx, int k) {
  float lanes[32];
  const int groups = k / 32;
  for (int l = 0; l < 32; ++l) lanes[l] = 0.0f;
  for (int base = 0; base < groups; base += 8) {
    for (int stride = 0; stride < 8; ++stride) {
      const int block = base + stride;
      if (block >= groups) continue;
      float part[4];
      for (int sub = 0; sub < 4; ++sub) {
        float sum = 0.0f;
        for (int i = 0; i < 8; ++i) {
          const size_t at = size_t(block) * 32 + sub * 8 + i;
          sum = std::fmaf(decode_e4m3(w[at]), decode_e4m3(x[at]), sum);
        }
        part[sub] = sum;
      }
      // xor 1 then xor 2 inside the quad; quarter 0 keeps (p0 + p1) + (p2 + p3)
      const float s = (part[0] + part[1]) + (part[2] + part[3]);
      lanes[stride * 4] = std::fmaf(s, e8m0_decode_f32(sx[block]) * e8m0_decode_f32(sw[block]), lanes[stride * 4]);
    }
  }
  return warp_sum_xor32(lanes);
}
}  // namespace

// packed = 1: W4A8 dot of one row; 0: W8A8 dot of one row (sw = the scale row of its 32-row block).
ORC_API float orc_e8m0_dot_f32(int packed, const uint8_t* w, const uint8_t* sw, const uint8_t* x, const uint8_t* sx, int k) {
  return packed ? w4a8_dot_f32(w, sw, x, sx, k) : w8a8_dot_f32(w, sw, x, sx, k);
}

// One expert on one token, FP32-chain variant (kernels/moe_ffn.cu:507-576, :799-865); same layouts as
// orc_expert_ffn_e8m0. The shared expert (packed = 0) carries no routed weight.
ORC_API int orc_expert_ffn_e8m0_f32(int packed, const uint16_t* x, const uint8_t* gate, const uint8_t* sgate, const uint8_t* up,
                                    const uint8_t* sup, const uint8_t* down, const uint8_t* sdown, int H, int I, float limit,
                                    float route_weight, uint16_t* out, uint16_t* act_out) {
  if (H % 32 || I % 32 || !(limit > 0.0f)) return -2;
  std::vector<uint8_t> xc(H), xs(H / 32), hc(I), hs(I / 32);
  std::vector<uint16_t> h(I);
  if (orc_act_quant_e8m0(x, 1, H, xc.data(), xs.data())) return -1;
  const int stride_gu = packed ? H / 2 : H, stride_d = packed ? I / 2 : I;
  for (int j = 0; j < I; ++j) {
    const int sr = packed ? j : j / 32;
    const float gate_v = orc_e8m0_dot_f32(packed, gate + size_t(j) * stride_gu, sgate + size_t(sr) * (H / 32), xc.data(), xs.data(), H);
    const float up_v = orc_e8m0_dot_f32(packed, up + size_t(j) * stride_gu, sup + size_t(sr) * (H / 32), xc.data(), xs.data(), H);
    const float g = std::fmin(bround(gate_v), limit);
    const float u = std::fmax(std::fmin(bround(up_v), limit), -limit);
    const float silu = g / (1.0f + det_expf(-g));
    h[j] = packed ? bf16_rne((silu * u) * route_weight) : bf16_rne(silu * u);
  }
  if (act_out) std::memcpy(act_out, h.data(), size_t(I) * 2);
  if (orc_act_quant_e8m0(h.data(), 1, I, hc.data(), hs.data())) return -1;
  for (int d = 0; d < H; ++d) {
    const int sr = packed ? d : d / 32;
    out[d] = bf16_rne(orc_e8m0_dot_f32(packed, down + size_t(d) * stride_d, sdown + size_t(sr) * (I / 32), hc.data(), hs.data(), I));
  }
  return 0;
}
