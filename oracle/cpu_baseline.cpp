// CPU baseline for the benchmark: a multithreaded port of the reference's CPU expert path
// (src/cpu/expert_ffn.rs), extended to 128x128-f32 block scales by the rule
// w = bf16(decode_e4m3(code) * scale) (src/fp8.rs:138-140).
//
// TEST / BENCHMARK INFRASTRUCTURE ONLY: timed next to the GPU by bench.py, checked against the scalar
// oracle by the tests. The shipped library never links or calls it.
//
// Arithmetic = the reference's Lane16 form (expert_ffn.rs:689-706, :739-752): 16 FP32 partial sums,
// lane L owning elements k = L (mod 16), pairwise 1/2/4/8 tree (:681-687), BF16 boundaries at gate,
// up, SiLU, product, down and weighted contribution (:592-679). A 16-wide vector accumulator is that
// form exactly; products of two BF16 values are exact in FP32, so fused and unfused multiply-adds agree.
// Work split = the reference's two-phase pool (:2623-2898): phase 1 partitions the (assignment, gate/up
// row) space evenly over the threads, barrier, phase 2 partitions the (assignment, down row) space.
#include <cmath>
#include <cstdint>
#include <cstring>
#include <omp.h>

#define BASE_API extern "C" __attribute__((visibility("default")))
#define CLONES __attribute__((target_clones("avx512f", "avx2", "default")))

namespace {
typedef float v16f __attribute__((vector_size(64)));
typedef int32_t v16i __attribute__((vector_size(64)));
typedef uint8_t v16b __attribute__((vector_size(16)));
typedef uint16_t v16h __attribute__((vector_size(32)));

inline uint32_t f2u(float f) { uint32_t u; std::memcpy(&u, &f, 4); return u; }
inline float u2f(uint32_t u) { float f; std::memcpy(&f, &u, 4); return f; }
inline uint16_t bf16_rne(float f) {
  uint32_t b = f2u(f);
  if ((b & 0x7fffffffu) > 0x7f800000u) return uint16_t((b >> 16) | 0x40u);
  b += 0x7fffu + ((b >> 16) & 1u);
  return uint16_t(b >> 16);
}
inline float bround(float f) { return u2f(uint32_t(bf16_rne(f)) << 16); }

// same deterministic expf as the oracle (ffmoe_oracle.cpp)
inline float det_expf(float x) {
  if (x != x) return x;
  if (!(x > -104.0f)) return 0.0f;
  if (x > 88.72283935546875f) return u2f(0x7f800000u);
  const float magic = 12582912.0f;
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

// 16 E4M3 codes -> BF16-rounded effective weights as f32. (mag << 20) read as a float is
// decode(mag) * 2^-120 for every finite code, subnormals included, so one multiply decodes.
inline v16f effective16(const uint8_t* codes, float scale) {
  v16b raw;
  std::memcpy(&raw, codes, 16);
  const v16i c = __builtin_convertvector(raw, v16i);
  const v16i mag = c & 0x7f;
  const v16i sign = (c & 0x80) << 24;
  const v16f dec = (v16f)((mag << 20) | sign) * 0x1p120f;
  const v16f prod = dec * scale;
  v16i b = (v16i)prod;
  b = (b + 0x7fff + ((b >> 16) & 1)) & (int32_t)0xffff0000;
  return (v16f)b;
}

inline float pairwise16(const v16f& l) {
  const float low = ((l[0] + l[1]) + (l[2] + l[3])) + ((l[4] + l[5]) + (l[6] + l[7]));
  const float high = ((l[8] + l[9]) + (l[10] + l[11])) + ((l[12] + l[13]) + (l[14] + l[15]));
  return low + high;
}

// dot of an f32 activation row with one FP8 weight row under 128-wide scale blocks
inline float dot_row(const float* x, const uint8_t* codes, const float* scales, int k) {
  v16f acc = {0};
  for (int b = 0; b < k; b += 128) {
    const float s = scales[b >> 7];
    const int end = b + 128 < k ? b + 128 : k;
    for (int i = b; i < end; i += 16) {
      v16f xv;
      std::memcpy(&xv, x + i, 64);
      acc += xv * effective16(codes + i, s);
    }
  }
  return pairwise16(acc);
}

struct Expert {
  const uint8_t* gate; const float* gate_s;
  const uint8_t* up; const float* up_s;
  const uint8_t* down; const float* down_s;
};
}  // namespace

// One decode batch: n assignments, assignment a uses expert table entry ex[a] (six host pointers),
// token row rows[a] of x [*, H] (BF16 bits) and routing weight w[a]; apply_w[a] == 0 leaves bf16(d)
// (shared expert). act [n, I] is scratch. out [n, H] BF16 bits. Twice rounding, SiLU as g*(1/(1+e^-g))
// (Lane16/Twice, expert_ffn.rs:81-86), boundary 0 = AfterDownBf16, 1 = BeforeContributionBf16.
CLONES BASE_API int cpubase_moe_decode(const uint16_t* x, const int* rows, const uint64_t* ex, const float* w, const int* apply_w,
                                       int n, int H, int I, int boundary, int threads, float* xf, uint16_t* act, uint16_t* out) {
  if (H % 16 || I % 16 || I > 16384) return -1;
  const int kbh = (H + 127) / 128, kbi = (I + 127) / 128;
#pragma omp parallel num_threads(threads)
  {
    const int t = omp_get_thread_num(), nt = omp_get_num_threads();
    // activations to f32 once (scratch.hidden, expert_ffn.rs:603-605)
#pragma omp for schedule(static)
    for (int a = 0; a < n; ++a)
      for (int k = 0; k < H; ++k) xf[size_t(a) * H + k] = u2f(uint32_t(x[size_t(rows[a]) * H + k]) << 16);
    // phase 1: (assignment, j) rows, contiguous block per thread (expert_ffn.rs:1984-1989)
    const long long total1 = (long long)n * I;
    for (long long u = total1 * t / nt; u < total1 * (t + 1) / nt; ++u) {
      const int a = int(u / I), j = int(u % I);
      const Expert* e = reinterpret_cast<const Expert*>(ex + size_t(a) * 6);
      const float* xa = xf + size_t(a) * H;
      const float g = bround(dot_row(xa, e->gate + size_t(j) * H, e->gate_s + size_t(j >> 7) * kbh, H));
      const float uu = bround(dot_row(xa, e->up + size_t(j) * H, e->up_s + size_t(j >> 7) * kbh, H));
      const float silu = g * (1.0f / (1.0f + det_expf(-g)));
      act[size_t(a) * I + j] = bf16_rne(bround(silu) * uu);
    }
#pragma omp barrier
    // phase 2: (assignment, d) rows
    const long long total2 = (long long)n * H;
    float af[16384];
    int loaded = -1;
    for (long long u = total2 * t / nt; u < total2 * (t + 1) / nt; ++u) {
      const int a = int(u / H), d = int(u % H);
      if (a != loaded) {
        for (int j = 0; j < I; ++j) af[j] = u2f(uint32_t(act[size_t(a) * I + j]) << 16);
        loaded = a;
      }
      const Expert* e = reinterpret_cast<const Expert*>(ex + size_t(a) * 6);
      const float lin = dot_row(af, e->down + size_t(d) * I, e->down_s + size_t(d >> 7) * kbi, I);
      float v;
      if (!apply_w[a]) v = bround(lin);
      else if (boundary == 0) v = bround(lin) * w[a];
      else v = lin * w[a];
      out[size_t(a) * H + d] = bf16_rne(v);
    }
  }
  return 0;
}

BASE_API int cpubase_max_threads() { return omp_get_max_threads(); }
BASE_API const char* cpubase_isa() {
  __builtin_cpu_init();
  if (__builtin_cpu_supports("avx512f")) return "avx512f";
  if (__builtin_cpu_supports("avx2")) return "avx2";
  return "scalar";
}
