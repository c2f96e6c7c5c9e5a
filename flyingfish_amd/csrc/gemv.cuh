// Weight-streaming GEMV building blocks shared by the decode and the standalone linear kernels:
// the three weight formats (16-byte lane chunks, in-register dequantization to packed BF16 pairs)
// and the slab inner loop (weights in registers x activations in LDS, v_dot2 accumulation).
#pragma once
#include "common.cuh"
#include <type_traits>

namespace ffmoe {

// ---------------------------------------------------------------------------------------------
// weight formats
struct FmtFp8 {
  static constexpr int EPL = 16;  // elements per 16-byte lane chunk
  struct Chunk { u32x4 codes; float scale; };
  struct Row { const uint8_t* codes; const float* scales; };
  // slot entries: codes [N,K] u8, scales [ceil(N/128), ceil(K/128)] f32
  static __device__ __forceinline__ Row row(uint64_t codes, uint64_t scales, float, int j, int K) {
    Row r;
    r.codes = reinterpret_cast<const uint8_t*>(codes) + size_t(j) * K;
    r.scales = reinterpret_cast<const float*>(scales) + size_t(j >> 7) * ((K + 127) >> 7);
    return r;
  }
  // Loads are unconditional and nothing consumes them here (the caller clamps `chunk` into the row), so no
  // branch or wait sits between the prefetch and its use; masking happens at dequantization time.
  // Offsets are unsigned 32-bit so the loads can take the row base from scalar registers.
  static __device__ __forceinline__ void load(Chunk& c, const Row& r, int chunk) {
    c.codes = load16_stream(r.codes + uint32_t(chunk) * 16u);
    c.scale = load_global<float>(r.scales + (uint32_t(chunk) >> 3));
  }
  static __device__ __forceinline__ void dequant(const Chunk& c, uint32_t* w, bool valid) {
    const float s = valid ? c.scale : 0.0f;  // masked lane: zero scale, zero weights
#pragma unroll
    for (int q = 0; q < 4; ++q) dequant4_e4m3(c.codes[q], s, w[2 * q], w[2 * q + 1]);
  }
};

// E4M3 codes [N,K] with one BF16 scale per output row (the reference's per-channel W8A16 experts,
// src/experts/catalogue.rs:31-39; effective weight bf16(e4m3(code) * f32(scale)), src/fp8.rs:138-140)
struct FmtFp8Channel {
  static constexpr int EPL = 16;
  struct Chunk { u32x4 codes; uint32_t scale; };  // scale: BF16 bits of the row's scale
  struct Row { const uint8_t* codes; const uint16_t* scale; };
  // slot entries: codes [N,K] u8, scales [N] bf16
  static __device__ __forceinline__ Row row(uint64_t codes, uint64_t scales, float, int j, int K) {
    Row r;
    r.codes = reinterpret_cast<const uint8_t*>(codes) + size_t(j) * K;
    r.scale = reinterpret_cast<const uint16_t*>(scales) + j;
    return r;
  }
  // the scale travels with every chunk (one 2-byte word, the same for all lanes) so that nothing waits for it before
  // the weights themselves are used
  static __device__ __forceinline__ void load(Chunk& c, const Row& r, int chunk) {
    c.codes = load16_stream(r.codes + uint32_t(chunk) * 16u);
    c.scale = uint32_t(load_global<uint16_t>(r.scale));
  }
  static __device__ __forceinline__ void dequant(const Chunk& c, uint32_t* w, bool valid) {
    const float s = valid ? bf16_to_f32(uint16_t(c.scale)) : 0.0f;  // masked lane: zero scale, zero weights
#pragma unroll
    for (int q = 0; q < 4; ++q) dequant4_e4m3(c.codes[q], s, w[2 * q], w[2 * q + 1]);
  }
};

struct FmtNvfp4 {
  static constexpr int EPL = 32;
  struct Chunk { u32x4 codes; uint32_t scales; float global; };
  struct Row { const uint8_t* codes; const uint8_t* scales; float global; };
  // slot entries: codes [N,K/2] u8 (low nibble = even k), scales [N,K/16] e4m3; global f32
  static __device__ __forceinline__ Row row(uint64_t codes, uint64_t scales, float global, int j, int K) {
    Row r;
    r.codes = reinterpret_cast<const uint8_t*>(codes) + size_t(j) * (K >> 1);
    r.scales = reinterpret_cast<const uint8_t*>(scales) + size_t(j) * (K >> 4);
    r.global = global;
    return r;
  }
  static __device__ __forceinline__ void load(Chunk& c, const Row& r, int chunk) {
    c.codes = load16_stream(r.codes + uint32_t(chunk) * 16u);
    c.scales = uint32_t(load_global<uint16_t>(r.scales + uint32_t(chunk) * 2u));
    c.global = r.global;
  }
  static __device__ __forceinline__ void dequant(const Chunk& c, uint32_t* w, bool valid) {
    // s = e4m3(scale) * global first, then e2m1 * s (kernels/nvfp4_linear.cu:83-98 of the reference)
    const f32x2 sc = e4m3x2_to_f32<false>(c.scales);
    const float gl = valid ? c.global : 0.0f;  // masked lane: zero scale, zero weights
    const float s0 = __fmul_rn(sc.x, gl), s1 = __fmul_rn(sc.y, gl);
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const float s = q < 2 ? s0 : s1;
      const uint32_t d = c.codes[q];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const uint32_t byte = (d >> (8 * i)) & 0xffu;
        w[4 * q + i] = pack_bf16x2(__fmul_rn(e2m1_to_f32(byte & 15u), s), __fmul_rn(e2m1_to_f32(byte >> 4), s));
      }
    }
  }
  // Split form of the same weights. An E2M1 magnitude is 2^j or 1.5 * 2^j, and scaling by a power of two commutes
  // with both roundings, so bf16(e2m1 * s) is exactly 2^j * b1 or 2^j * b15 with b1 = bf16(s), b15 = bf16(f32(1.5 s)).
  // With m = the raw E2M1 value and u = m with its mantissa bit cleared (2^j for both classes),
  //     sum x * w  =  c1 * sum x*u  +  c2 * sum x*m,     c1 = 3 b1 - 2 b15,   c2 = 2 (b15 - b1)
  // (a 2^j element contributes x u (c1 + c2) = x u b1, a 1.5 * 2^j element x u (c1 + 1.5 c2) = x u b15). c1 and c2
  // are exact in FP32, m and u are exact BF16 values straight from the hardware FP4 conversion, so per element
  // this costs one conversion, one AND and two dot2 lanes instead of a multiply and a rounding per weight.
  struct Split { uint32_t m[16], u[16]; float c1[2], c2[2]; };
  static __device__ __forceinline__ void split(const Chunk& c, Split& o, bool valid) {
    const f32x2 sc = e4m3x2_to_f32<false>(c.scales);
    const float gl = valid ? c.global : 0.0f;
#pragma unroll
    for (int g = 0; g < 2; ++g) {
      const float s = __fmul_rn(g == 0 ? sc.x : sc.y, gl);
      const float b1 = bround(s), b15 = bround(__fmul_rn(1.5f, s));
      o.c1[g] = __fsub_rn(__fmul_rn(3.0f, b1), __fmul_rn(2.0f, b15));
      o.c2[g] = __fmul_rn(2.0f, __fsub_rn(b15, b1));
    }
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const uint32_t d = c.codes[q];
      // byte i of the dword: low nibble = even k -> low half of the pair
      const bf16x2 p0 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(d, 1.0f, 0);
      const bf16x2 p1 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(d, 1.0f, 1);
      const bf16x2 p2 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(d, 1.0f, 2);
      const bf16x2 p3 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(d, 1.0f, 3);
      o.m[4 * q + 0] = __builtin_bit_cast(uint32_t, p0);
      o.m[4 * q + 1] = __builtin_bit_cast(uint32_t, p1);
      o.m[4 * q + 2] = __builtin_bit_cast(uint32_t, p2);
      o.m[4 * q + 3] = __builtin_bit_cast(uint32_t, p3);
#pragma unroll
      for (int i = 0; i < 4; ++i) o.u[4 * q + i] = o.m[4 * q + i] & 0xffbfffbfu;
    }
  }
  // The pair (c1, c2) depends on the scale code and the matrix's global scale alone: a table of the 256 codes per
  // matrix in LDS (entry 256 = zeros, for a masked lane) replaces the dozen instructions per group of 16 by one
  // 8-byte LDS read. Same formulas, same values.
  static constexpr int LUT_ENTRIES = 257;
  static __device__ __forceinline__ void build_lut(u32x2* lut, float global, int tid, int nthreads) {
    for (int i = tid; i < LUT_ENTRIES; i += nthreads) {
      const float s = __fmul_rn(e4m3x2_to_f32<false>(uint32_t(i & 255)).x, i < 256 ? global : 0.0f);
      const float b1 = bround(s), b15 = bround(__fmul_rn(1.5f, s));
      u32x2 e;
      e.x = __float_as_uint(__fsub_rn(__fmul_rn(3.0f, b1), __fmul_rn(2.0f, b15)));
      e.y = __float_as_uint(__fmul_rn(2.0f, __fsub_rn(b15, b1)));
      lut[i] = e;
    }
  }
  static __device__ __forceinline__ void split_lut(const Chunk& c, Split& o, bool valid, const u32x2* lut) {
#pragma unroll
    for (int g = 0; g < 2; ++g) {
      const uint32_t code = (c.scales >> (8 * g)) & 0xffu;
      const u32x2 e = lut[valid ? code : 256u];
      o.c1[g] = __uint_as_float(e.x);
      o.c2[g] = __uint_as_float(e.y);
    }
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const uint32_t d = c.codes[q];
      o.m[4 * q + 0] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(d, 1.0f, 0));
      o.m[4 * q + 1] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(d, 1.0f, 1));
      o.m[4 * q + 2] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(d, 1.0f, 2));
      o.m[4 * q + 3] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(d, 1.0f, 3));
#pragma unroll
      for (int i = 0; i < 4; ++i) o.u[4 * q + i] = o.m[4 * q + i] & 0xffbfffbfu;
    }
  }
};

struct FmtBf16 {
  static constexpr int EPL = 8;
  struct Chunk { u32x4 codes; };
  struct Row { const uint8_t* codes; };
  static __device__ __forceinline__ Row row(uint64_t codes, uint64_t, float, int j, int K) {
    Row r;
    r.codes = reinterpret_cast<const uint8_t*>(codes) + size_t(j) * K * 2;
    return r;
  }
  static __device__ __forceinline__ void load(Chunk& c, const Row& r, int chunk) {
    c.codes = load16_stream(r.codes + uint32_t(chunk) * 16u);
  }
  static __device__ __forceinline__ void dequant(const Chunk& c, uint32_t* w, bool valid) {
    const uint32_t keep = valid ? 0xffffffffu : 0u;
#pragma unroll
    for (int q = 0; q < 4; ++q) w[q] = c.codes[q] & keep;
  }
};

// One step: this lane's 16-byte chunk of NROWS weight rows against the n activation rows in LDS. The activation
// chunk is read once and used for every weight row. Straight-line code: a chunk past the end of the row is
// masked (zero weights), never branched around, so the waits on the prefetched registers stay precise.
// NVFP4 with scale tables in LDS (FmtNvfp4::build_lut): weight rows 0 .. lut_rows-1 use lut0, the rest lut1.
template <class F, int NROWS, int RG, int S, bool LUT = false>
__device__ __forceinline__ void step_compute(const typename F::Chunk (&c)[NROWS][S], int s, const uint8_t* xs, int K, int nchunks,
                                             int chunk, int n, float (&acc)[NROWS][RG], const u32x2* lut0 = nullptr,
                                             const u32x2* lut1 = nullptr, int lut_rows = NROWS) {
  const bool valid = chunk < nchunks;
  const int cl = valid ? chunk : 0;  // keep the LDS read in range
  if constexpr (std::is_same<F, FmtNvfp4>::value) {
    // two groups of 16 per chunk, each with its own pair of constants (see FmtNvfp4::split)
    FmtNvfp4::Split w[NROWS];
    if constexpr (LUT) {
#pragma unroll
      for (int m = 0; m < NROWS; ++m) FmtNvfp4::split_lut(c[m][s], w[m], valid, m < lut_rows ? lut0 : lut1);
    } else {
#pragma unroll
      for (int m = 0; m < NROWS; ++m) FmtNvfp4::split(c[m][s], w[m], valid);
    }
#pragma unroll
    for (int r = 0; r < RG; ++r) {
      if (RG == 1 || r < n) {
        const u32x4* xp = reinterpret_cast<const u32x4*>(xs + size_t(r) * K * 2 + size_t(cl) * 64);
#pragma unroll
        for (int g = 0; g < 2; ++g) {
          const u32x4 xa = xp[2 * g], xb = xp[2 * g + 1];
#pragma unroll
          for (int m = 0; m < NROWS; ++m) {
            float sm = 0.0f, su = 0.0f;
#pragma unroll
            for (int q = 0; q < 4; ++q) {
              sm = dot2_bf16(w[m].m[8 * g + q], xa[q], sm);
              su = dot2_bf16(w[m].u[8 * g + q], xa[q], su);
            }
#pragma unroll
            for (int q = 0; q < 4; ++q) {
              sm = dot2_bf16(w[m].m[8 * g + 4 + q], xb[q], sm);
              su = dot2_bf16(w[m].u[8 * g + 4 + q], xb[q], su);
            }
            acc[m][r] = __fmaf_rn(su, w[m].c1[g], __fmaf_rn(sm, w[m].c2[g], acc[m][r]));
          }
        }
      }
    }
    return;
  }
  uint32_t w[NROWS][F::EPL / 2];
#pragma unroll
  for (int m = 0; m < NROWS; ++m) F::dequant(c[m][s], w[m], valid);
#pragma unroll
  for (int r = 0; r < RG; ++r) {
    if (RG == 1 || r < n) {
      const u32x4* xp = reinterpret_cast<const u32x4*>(xs + size_t(r) * K * 2 + size_t(cl) * (F::EPL * 2));
#pragma unroll
      for (int v = 0; v < F::EPL / 8; ++v) {
        const u32x4 xv = xp[v];
#pragma unroll
        for (int q = 0; q < 4; ++q)
#pragma unroll
          for (int m = 0; m < NROWS; ++m) acc[m][r] = dot2_bf16(w[m][4 * v + q], xv[q], acc[m][r]);
      }
    }
  }
}

}  // namespace ffmoe
