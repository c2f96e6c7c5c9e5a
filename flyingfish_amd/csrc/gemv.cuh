// Weight-streaming GEMV building blocks shared by the decode and the standalone linear kernels:
// the three weight formats (16-byte lane chunks, in-register dequantization to packed BF16 pairs)
// and the slab inner loop (weights in registers x activations in LDS, v_dot2 accumulation).
#pragma once
#include "common.cuh"

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
template <class F, int NROWS, int RG, int S>
__device__ __forceinline__ void step_compute(const typename F::Chunk (&c)[NROWS][S], int s, const uint8_t* xs, int K, int nchunks,
                                             int chunk, int n, float (&acc)[NROWS][RG]) {
  const bool valid = chunk < nchunks;
  const int cl = valid ? chunk : 0;  // keep the LDS read in range
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
