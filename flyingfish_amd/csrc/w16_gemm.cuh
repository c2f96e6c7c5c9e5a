// Grouped W*A16 GEMM on the BF16 matrix cores: the prefill form of the decode path's arithmetic. Weights of any expert
// format are dequantized in registers to the very BF16 effective weights the decode kernels use
// (bf16(e4m3 * scale), bf16(e2m1 * (e4m3(scale) * global)), src/fp8.rs:138-145), activations stay BF16, and
// v_mfma_f32_16x16x32_bf16 accumulates the exact products in FP32 over the whole contraction. This is what the reference's
// prefill computes for its per-channel FP8 and BF16 experts (moe_gemm_w8a16 and the BF16 grouped GEMM,
// kernels/moe_prefill.cu:157-350, src/backend/cuda/moe/prefill.rs:1053-1408), whose summation order its own tests bound
// by tolerance only; NVFP4 and block-FP8 experts get the same treatment.
//
// Work model, unit list and token staging are those of k_w8a8_grouped (w8a8_gemm.cuh): a unit is one group of at most
// 16 * MF token rows of an expert x one tile of output columns, a K block is 64 columns = 128 bytes of a BF16 token row
// (staged through LDS, XOR-swizzled, shared by the four waves), each wave owns four 16-row weight fragments and streams
// them global -> registers P K blocks ahead. Per K block a lane holds 16 columns of one weight row: after dequantization
// two operands of 8 columns, i.e. two instructions per (weight fragment, token fragment).
//
// MODE 0: gate/up + SwiGLU with the decode path's roundings (kernels/moe_ffn.cu:98-302) -> act[pos, j]
// MODE 1: down, then the routing weight at the configured boundary -> contributions[assignment, d], done = 1
// MODE 2: plain product -> y[row, n] (the shared expert's down projection)
#pragma once
#include "gemv.cuh"
#include "w8a8_gemm.cuh"

namespace ffmoe {

typedef __bf16 w16_bf16x8 __attribute__((ext_vector_type(8)));

// 16 consecutive columns of one weight row -> 8 packed BF16 pairs of effective weights
template <class F>
struct W16;

template <>
struct W16<FmtFp8> {
  struct Frag { u32x4 codes; float scale; };
  struct Row { const uint8_t* codes; const float* scales; };
  static __device__ __forceinline__ Row row(uint64_t codes, uint64_t scales, float, int j, int K) {
    return Row{reinterpret_cast<const uint8_t*>(codes) + size_t(j) * K, reinterpret_cast<const float*>(scales) + size_t(j >> 7) * ((K + 127) >> 7)};
  }
  static constexpr int LOADS = 2;  // loads one fragment issues per K block
  static __device__ __forceinline__ void load(Frag& f, const Row& r, uint32_t col) {
    load16_async(f.codes, r.codes + col);
    load4_async(f.scale, r.scales + (col >> 7));
  }
  static __device__ __forceinline__ void pin(Frag& f) { asm volatile("" : "+v"(f.codes), "+v"(f.scale)); }
  static __device__ __forceinline__ void dequant(const Frag& f, uint32_t (&w)[8]) {
#pragma unroll
    for (int q = 0; q < 4; ++q) dequant4_e4m3(f.codes[q], f.scale, w[2 * q], w[2 * q + 1]);
  }
};

template <>
struct W16<FmtFp8Channel> {
  struct Frag { u32x4 codes; };
  struct Row { const uint8_t* codes; float scale; };
  static __device__ __forceinline__ Row row(uint64_t codes, uint64_t scales, float, int j, int K) {
    // the row scale must have arrived before the K loop: a wait of the compiler's inside it would drain the prefetch queue
    return Row{reinterpret_cast<const uint8_t*>(codes) + size_t(j) * K, landed(bf16_to_f32(load_global<uint16_t>(reinterpret_cast<const uint16_t*>(scales) + j)))};
  }
  static constexpr int LOADS = 1;
  static __device__ __forceinline__ void load(Frag& f, const Row& r, uint32_t col) { load16_async(f.codes, r.codes + col); }
  static __device__ __forceinline__ void pin(Frag& f) { asm volatile("" : "+v"(f.codes)); }
  static __device__ __forceinline__ void dequant(const Frag& f, const Row& r, uint32_t (&w)[8]) {
#pragma unroll
    for (int q = 0; q < 4; ++q) dequant4_e4m3(f.codes[q], r.scale, w[2 * q], w[2 * q + 1]);
  }
};

template <>
struct W16<FmtBf16> {
  struct Frag { u32x4 lo, hi; };
  struct Row { const uint8_t* codes; };
  static __device__ __forceinline__ Row row(uint64_t codes, uint64_t, float, int j, int K) {
    return Row{reinterpret_cast<const uint8_t*>(codes) + size_t(j) * K * 2};
  }
  static constexpr int LOADS = 2;
  static __device__ __forceinline__ void load(Frag& f, const Row& r, uint32_t col) {
    load16_async(f.lo, r.codes + col * 2u);
    load16_async(f.hi, r.codes + col * 2u + 16u);
  }
  static __device__ __forceinline__ void pin(Frag& f) { asm volatile("" : "+v"(f.lo), "+v"(f.hi)); }
  static __device__ __forceinline__ void dequant(const Frag& f, uint32_t (&w)[8]) {
#pragma unroll
    for (int q = 0; q < 4; ++q) { w[q] = f.lo[q]; w[4 + q] = f.hi[q]; }
  }
};

template <>
struct W16<FmtNvfp4> {
  struct Frag { u32x2 codes; uint32_t scale; };
  struct Row { const uint8_t* codes; const uint8_t* scales; float global; };
  static __device__ __forceinline__ Row row(uint64_t codes, uint64_t scales, float global, int j, int K) {
    return Row{reinterpret_cast<const uint8_t*>(codes) + size_t(j) * (K >> 1), reinterpret_cast<const uint8_t*>(scales) + size_t(j) * (K >> 4), global};
  }
  static constexpr int LOADS = 0;  // requested row-contiguously by the kernel itself (two loads per pair of fragments)
  static __device__ __forceinline__ void load(Frag&, const Row&, uint32_t) {}
  static __device__ __forceinline__ void pin(Frag&) {}
  // s = e4m3(scale) * global first, then bf16(e2m1 * s) (kernels/nvfp4_linear.cu:83-98); the E2M1 values come from the
  // hardware conversion as exact FP32 pairs, low nibble = even column
  static __device__ __forceinline__ void dequant(const Frag& f, const Row& r, uint32_t (&w)[8]) {
    typedef float w16_f32x2 __attribute__((ext_vector_type(2)));
    const float s = __fmul_rn(e4m3x2_to_f32<false>(f.scale).x, r.global);
#pragma unroll
    for (int q = 0; q < 2; ++q) {
      const uint32_t d = f.codes[q];
      w16_f32x2 pr[4];
      pr[0] = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(d, 1.0f, 0);
      pr[1] = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(d, 1.0f, 1);
      pr[2] = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(d, 1.0f, 2);
      pr[3] = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(d, 1.0f, 3);
#pragma unroll
      for (int i = 0; i < 4; ++i) w[4 * q + i] = pack_bf16x2(__fmul_rn(pr[i].x, s), __fmul_rn(pr[i].y, s));
    }
  }
};

// A load whose wait the kernel places by hand (see load16_async): one word
__device__ __forceinline__ void load4_async(uint32_t& d, const void* p) {
  asm volatile("global_load_dword %0, %1, off" : "=v"(d) : "v"(p));
}
// load16_async with the streaming hint: the line is the first the L2 gives up again
__device__ __forceinline__ void load16_async_nt(u32x4& d, uint64_t base, uint32_t offset) {
  asm volatile("global_load_dwordx4 %0, %1, %2 nt" : "=v"(d) : "v"(offset), "s"(base));
}
// At most N of the loads issued so far may still be in flight behind this point. A register is read only after it went
// through a pin() behind the wait that covers its load (volatile statements keep their order).
template <int N>
__device__ __forceinline__ void wait_vm() {
  static_assert(N >= 0 && N < 64, "vmcnt is a six-bit count");
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N));
}
__device__ __forceinline__ void pin(u32x4& v) { asm volatile("" : "+v"(v)); }
__device__ __forceinline__ void pin(uint32_t& v) { asm volatile("" : "+v"(v)); }
__device__ __forceinline__ void pin(float& v) { asm volatile("" : "+v"(v)); }

// formats whose dequantization needs the row (a per-row scale or the global scale)
template <class F> struct W16NeedsRow { static constexpr bool value = false; };
template <> struct W16NeedsRow<FmtFp8Channel> { static constexpr bool value = true; };
template <> struct W16NeedsRow<FmtNvfp4> { static constexpr bool value = true; };

// Formats whose 16 columns are 16 bytes (64 bytes of a row per K block): their weights are requested row-contiguously
// (4 lanes per row, 16 rows per instruction, whole 64-byte segments) and turned into the operand's lane order through
// a wave-private LDS buffer. Requested directly in operand order, a lane owns 16 bytes of ONE row, the 16 consecutive
// lanes of a quarter wave touch 16 different lines, and the vector L1 spends one look-up per 16 bytes.
template <class F> struct W16Transpose { static constexpr bool value = false; };
template <> struct W16Transpose<FmtFp8> { static constexpr bool value = true; };
template <> struct W16Transpose<FmtFp8Channel> { static constexpr bool value = true; };

struct W16Params {
  const uint16_t* a;         // activations [*, K] BF16
  const uint64_t* slots;     // [E, 6] expert table, or NULL: the four addresses below
  uint64_t w0_codes, w0_scales, w1_codes, w1_scales;  // MODE 0: gate, up; MODE 1/2: w0 only
  const float* global_scales;  // [E, 3] (NVFP4 table) or NULL
  float g0, g1;              // global scales when slots == NULL
  const GemmGroup* groups;   // NULL: rows split arithmetically into groups of TM
  const u32x2* units;
  const uint32_t* unit_total;
  uint32_t total_units;
  const int* perm;           // permuted position -> assignment index (NULL: identity)
  const void* weights;       // routing weights per assignment (MODE 1)
  uint16_t* out;
  uint32_t* done;
  int rows_total;
  int K, N, top_k, weights_f32, swiglu, routed_weight;
  float limit;
  // Groups whose expert id is shared_expert (>= 0) are the always-on expert riding in the routed launch: weights from
  // sh_w / sh_g (gate, up, down: codes and scales; NVFP4 global scales), token rows are the rows themselves (no
  // permutation) read from a_sh, results go to out_sh[row] as plain BF16 (no routing weight, no done flag).
  int shared_expert;
  uint64_t sh_w[6];
  float sh_g[3];
  const uint16_t* a_sh;
  uint16_t* out_sh;
};

// One entry of the unit list: the group's expert and rows, the column tile, and where the expert's matrices are
struct W16Unit {
  int expert, start, n, t;
  bool ride;
  uint64_t wc[2], ws[2];
  float gl[2];
};
template <int MODE>
__device__ __forceinline__ W16Unit w16_unit(const W16Params& p, uint32_t u, int ntiles, int TM) {
  int expert, start, n, t;
  if (p.groups) {
    const u32x2 un = load_uniform<u32x2>(p.units + u);
    const int g = int(un.x);
    t = int(un.y);
    const int* gd = reinterpret_cast<const int*>(p.groups + g);
    expert = load_uniform<int>(gd);
    start = load_uniform<int>(gd + 1);
    n = load_uniform<int>(gd + 2);
  } else {
    const int g = int(u) / ntiles;
    t = int(u) - g * ntiles;
    expert = 0;
    start = g * TM;
    n = min(TM, p.rows_total - start);
  }
  uint64_t wc[2], ws[2];
  float gl[2] = {p.g0, p.g1};
  const bool ride = p.groups && expert == p.shared_expert;  // wave-uniform
  if (ride) {
    wc[0] = MODE == 0 ? p.sh_w[0] : p.sh_w[4]; ws[0] = MODE == 0 ? p.sh_w[1] : p.sh_w[5];
    wc[1] = MODE == 0 ? p.sh_w[2] : p.sh_w[4]; ws[1] = MODE == 0 ? p.sh_w[3] : p.sh_w[5];
    gl[0] = MODE == 0 ? p.sh_g[0] : p.sh_g[2];
    gl[1] = MODE == 0 ? p.sh_g[1] : p.sh_g[2];
  } else if (p.slots) {
    const uint64_t* sl = p.slots + size_t(expert) * 6;
    if (MODE == 0) {
      wc[0] = load_uniform<uint64_t>(sl + 0); ws[0] = load_uniform<uint64_t>(sl + 1);
      wc[1] = load_uniform<uint64_t>(sl + 2); ws[1] = load_uniform<uint64_t>(sl + 3);
    } else {
      wc[0] = wc[1] = load_uniform<uint64_t>(sl + 4); ws[0] = ws[1] = load_uniform<uint64_t>(sl + 5);
    }
    if (p.global_scales) {
      const float* g3 = p.global_scales + size_t(expert) * 3;
      gl[0] = load_uniform<float>(g3 + (MODE == 0 ? 0 : 2));
      gl[1] = MODE == 0 ? load_uniform<float>(g3 + 1) : gl[0];
    }
  } else {
    wc[0] = p.w0_codes; ws[0] = p.w0_scales;
    wc[1] = MODE == 0 ? p.w1_codes : p.w0_codes; ws[1] = MODE == 0 ? p.w1_scales : p.w0_scales;
    if (MODE != 0) gl[1] = gl[0];
  }
  W16Unit r;
  r.expert = expert; r.start = start; r.n = n; r.t = t; r.ride = ride;
  r.wc[0] = wc[0]; r.wc[1] = wc[1]; r.ws[0] = ws[0]; r.ws[1] = ws[1]; r.gl[0] = gl[0]; r.gl[1] = gl[1];
  return r;
}

// Epilogue of the grouped W*A16 kernels: a lane holds token (lane % 16) of each row fragment and output columns
// 4 (lane / 16) .. + 3 of each weight fragment.
template <int MF, int MODE>
__device__ __forceinline__ void w16_store(const v4f (&acc)[MF][4], const W16Params& p, bool ride, int start, int n, int t, const int (&col0)[4], int wave,
                                          int lane) {
  const int N = p.N;
  const int tk = lane & 15, sub = (lane >> 4) * 4;
#pragma unroll
  for (int m = 0; m < MF; ++m) {
    const int token = 16 * m + tk;
    if (token < n) {
      const int pos = start + token;
      if (MODE == 0) {
#pragma unroll
        for (int f = 0; f < 2; ++f) {
          const int col = col0[f] + sub;
          if (col0[f] + 16 <= N) {
            uint32_t o[2];
#pragma unroll
            for (int h = 0; h < 2; ++h) {
              const uint32_t lo = swiglu_bf16(bround(acc[m][f][2 * h]), bround(acc[m][f + 2][2 * h]), p.swiglu, p.limit);
              const uint32_t hi = swiglu_bf16(bround(acc[m][f][2 * h + 1]), bround(acc[m][f + 2][2 * h + 1]), p.swiglu, p.limit);
              o[h] = lo | (hi << 16);
            }
            const u32x2 v = {o[0], o[1]};
            *reinterpret_cast<u32x2*>((ride ? p.out_sh : p.out) + size_t(pos) * N + col) = v;
          }
        }
      } else {
        const int a = (MODE == 1 && p.perm && !ride) ? load_global<int>(p.perm + pos) : pos;
        const bool weighted = MODE == 1 && p.weights && !ride;
        float rw = 1.0f;
        if (weighted)
          rw = p.weights_f32 ? load_global<float>(reinterpret_cast<const float*>(p.weights) + a)
                             : bf16_to_f32(load_global<uint16_t>(reinterpret_cast<const uint16_t*>(p.weights) + a));
#pragma unroll
        for (int f = 0; f < 4; ++f) {
          const int col = col0[f] + sub;
          if (col0[f] + 16 <= N) {
            float v[4];
#pragma unroll
            for (int r = 0; r < 4; ++r) {
              if (weighted)
                v[r] = p.routed_weight == FFMOE_WEIGHT_AFTER_DOWN_BF16 ? __fmul_rn(bround(acc[m][f][r]), rw) : __fmul_rn(acc[m][f][r], rw);
              else
                v[r] = acc[m][f][r];
            }
            const u32x2 o = {pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3])};
            *reinterpret_cast<u32x2*>((ride ? p.out_sh : p.out) + size_t(a) * N + col) = o;
          }
        }
        if (MODE == 1 && p.done && !ride && t == 0 && wave == 0 && lane < 16) p.done[a] = 1u;
      }
    }
  }
}

// One unit of the grouped W*A16 GEMM, run by the NW waves of a block: a group of at most 16 MF token rows of one expert x
// one tile of output columns, over the whole contraction. The LDS buffers are the function's own.
template <class F, int MF, int MODE, int P, int NW>
__device__ __forceinline__ void w16_unit_run(const W16Params& p, const W16Unit& un_) {
  constexpr int NT = 64 * NW;
  constexpr int TM = 16 * MF;
  constexpr int CHUNKS = TM * 8;             // 16-byte token chunks per K block (64 BF16 columns = 128 bytes per row)
  constexpr int CPT = (CHUNKS + NT - 1) / NT;
  constexpr int TILE = TM * 128;
  constexpr bool TR = W16Transpose<F>::value;
  // NVFP4: a row's K block is 32 code bytes and 4 scale bytes. Two lanes request one row's codes (32 rows = two
  // fragments per instruction), the scale bytes of a row come as one word, and both are turned into operand order
  // (8 code bytes and one scale byte per lane) through wave-private LDS, like the FP8 formats below.
  constexpr bool NVT = std::is_same<F, FmtNvfp4>::value;
  __shared__ __attribute__((aligned(16))) uint8_t nstage[NVT ? NW : 1][NVT ? 2 : 1][NVT ? 1024 : 16];  // [wave][row pair of fragments][32 rows x 32 B]
  __shared__ uint32_t nscale[NVT ? NW : 1][NVT ? 2 : 1][NVT ? 32 : 1];
  __shared__ __attribute__((aligned(16))) uint8_t tile[2][TILE];
  __shared__ __attribute__((aligned(16))) uint8_t wstage[TR ? NW : 1][TR ? 4 : 1][TR ? 1024 : 16];  // [wave][fragment][16 rows x 64 B]
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = uni(tid >> 6);
  const int K = p.K, N = p.N, KB = K >> 6;
  // wave-private transposition buffer: written as (row lane / 4, 16-byte piece lane % 4), read as (row lane % 16, piece
  // lane / 16); pieces are XOR-swizzled by (row / 4) % 4 so that the 16 rows of a read fall into distinct banks
  const int wr_off = (lane >> 2) * 64 + (((lane & 3) ^ ((lane >> 4) & 3)) << 4);
  const int rd_off = (lane & 15) * 64 + (((lane >> 4) ^ ((lane >> 2) & 3)) << 4);
  const int expert = un_.expert, start = un_.start, n = un_.n, t = un_.t;
  const bool ride = un_.ride;  // wave-uniform
  const uint64_t wc[2] = {un_.wc[0], un_.wc[1]}, ws[2] = {un_.ws[0], un_.ws[1]};
  const float gl[2] = {un_.gl[0], un_.gl[1]};
  (void)expert;
  // weight rows of this lane's four fragments; fragments past N are clamped onto the last 16 rows and dropped at the store
  int col0[4];
  typename W16<F>::Row wrow[4];
#pragma unroll
  for (int f = 0; f < 4; ++f) {
    col0[f] = MODE == 0 ? t * (32 * NW) + wave * 32 + (f & 1) * 16 : t * (64 * NW) + wave * 64 + f * 16;
    const int base = min(col0[f], N - 16);
    const int which = MODE == 0 ? f >> 1 : 0;
    wrow[f] = W16<F>::row(wc[which], ws[which], gl[which], base + (lane & 15), K);
  }
  const uint32_t wcol = TR ? 0u : uint32_t(lane >> 4) * 16u;  // this lane's 16 columns inside a K block
  typename W16<F>::Row lrow[4];  // what the loads address: the operand's row, or the row-contiguous pattern
#pragma unroll
  for (int f = 0; f < 4; ++f) {
    if constexpr (TR) {
      const int which = MODE == 0 ? f >> 1 : 0;
      lrow[f] = W16<F>::row(wc[which], ws[which], gl[which], min(col0[f], N - 16) + (lane >> 2), K);
      lrow[f].codes += (lane & 3) * 16;
    } else {
      lrow[f] = wrow[f];
    }
  }

  const uint8_t* ncod[2] = {nullptr, nullptr};
  const uint8_t* nscl[2] = {nullptr, nullptr};
  if constexpr (NVT) {
#pragma unroll
    for (int j = 0; j < 2; ++j) {  // fragments 2j and 2j + 1 are 32 consecutive rows of one matrix
      const int which = MODE == 0 ? j : 0;
      const int row = min(col0[2 * j], N - 32) + (lane >> 1);
      ncod[j] = reinterpret_cast<const uint8_t*>(wc[which]) + size_t(row) * (K >> 1) + (lane & 1) * 16;
      nscl[j] = reinterpret_cast<const uint8_t*>(ws[which]) + size_t(row) * (K >> 4);
    }
  }
  u32x4 nvc[NVT ? P : 1][2];
  uint32_t nvs[NVT ? P : 1][2];  // the four scale bytes of a row's K block (K is a multiple of 64: a whole aligned word)

  // token rows this thread stages
  const uint8_t* tsrc[CPT];
  int tdst[CPT];
#pragma unroll
  for (int i = 0; i < CPT; ++i) {
    const int q = min(tid + NT * i, CHUNKS - 1);
    const int m = q >> 3, c = q & 7;
    const int pos = start + min(m, n - 1);
    const int row = MODE == 0 && p.perm && !ride ? load_global<int>(p.perm + pos) / p.top_k : pos;
    tsrc[i] = reinterpret_cast<const uint8_t*>(ride ? p.a_sh : p.a) + size_t(row) * K * 2 + c * 16;
    tdst[i] = m * 128 + ((c ^ (m & 7)) << 4);
  }
  const bool stage_chunk = CHUNKS >= NT || tid < CHUNKS;

  v4f acc[MF][4];
#pragma unroll
  for (int m = 0; m < MF; ++m)
#pragma unroll
    for (int f = 0; f < 4; ++f) acc[m][f] = v4f{0.0f, 0.0f, 0.0f, 0.0f};

  // Loads inside the K loop are issued and awaited by hand (load16_async / wait_vm / pin, see k_w8a8_grouped): the
  // compiler's own waits drain the queue at the top of every stage, which leaves one stage of lead whatever P is. A
  // thread issues its loads in a fixed order - per stage the token chunks of tile kb+2, then the weights of K block kb+P
  // into the slot just consumed - so the weights of a stage have the P-1 later stages' loads behind them and a token
  // tile the weight loads of its own stage.
  constexpr int WL = NVT ? 4 : 4 * W16<F>::LOADS;  // weight loads per stage
  constexpr int LPS = CPT + WL;
  typename W16<F>::Frag w[P][4];
#define FF_W16_REQUEST(s_, kb_)                                                              \
  do {                                                                                        \
  if constexpr (NVT) {                                                                      \
    _Pragma("unroll") for (int j_ = 0; j_ < 2; ++j_) {                                      \
      load16_async(nvc[s_][j_], ncod[j_] + (kb_) * 32u);                                    \
      load4_async(nvs[s_][j_], nscl[j_] + (kb_) * 4u);                                      \
    }                                                                                       \
  } else {                                                                                  \
    _Pragma("unroll") for (int f_ = 0; f_ < 4; ++f_) W16<F>::load(w[s_][f_], lrow[f_], (kb_) * 64u + wcol); \
  }                                                                                         \
  } while (0)
#define FF_W16_PIN(s_)                                                                        \
  do {                                                                                        \
  if constexpr (NVT) {                                                                      \
    _Pragma("unroll") for (int j_ = 0; j_ < 2; ++j_) { pin(nvc[s_][j_]); pin(nvs[s_][j_]); } \
  } else {                                                                                  \
    _Pragma("unroll") for (int f_ = 0; f_ < 4; ++f_) W16<F>::pin(w[s_][f_]);                \
  }                                                                                         \
  } while (0)
  // prologue: weights of the first P K blocks, token tile 0 into LDS, everything landed; then token tile 1 and the
  // last weight stage once more, so that tile 1 too has a stage's weight loads behind it
#pragma unroll
  for (int s = 0; s < P; ++s) FF_W16_REQUEST(s, uint32_t(min(s, KB - 1)));
  u32x4 tv[CPT];
  {
#pragma unroll
    for (int i = 0; i < CPT; ++i) {
      const u32x4 v = load16(tsrc[i]);
      if (stage_chunk) *reinterpret_cast<u32x4*>(&tile[0][tdst[i]]) = v;
    }
    wait_vm<0>();
#pragma unroll
    for (int s = 0; s < P; ++s) FF_W16_PIN(s);
    const uint32_t k1 = uint32_t(min(1, KB - 1));
#pragma unroll
    for (int i = 0; i < CPT; ++i) load16_async(tv[i], tsrc[i] + k1 * 128u);
    FF_W16_REQUEST(P - 1, uint32_t(min(P - 1, KB - 1)));
  }
  __syncthreads();

  // LDS addresses of this lane's token operands: row (16 m + lane % 16), columns 16 (lane / 16) .. + 15 = chunks 2q, 2q + 1
  int tlo[MF], thi[MF];
#pragma unroll
  for (int m = 0; m < MF; ++m) {
    const int trow = 16 * m + (lane & 15);
    const int q2 = (lane >> 4) * 2;
    tlo[m] = trow * 128 + (((q2) ^ (trow & 7)) << 4);
    thi[m] = trow * 128 + (((q2 + 1) ^ (trow & 7)) << 4);
  }

  for (int kbo = 0; kbo < KB; kbo += P) {
#pragma unroll
    for (int s = 0; s < P; ++s) {
      const int kb = kbo + s;
      if (kb < KB) {
        const uint8_t* tb = tile[kb & 1];
        w16_bf16x8 a0[4], a1[4];
        typename W16<F>::Frag wm[4];
        wait_vm<(P - 1) * LPS>();
        FF_W16_PIN(s);
#pragma unroll
        for (int f = 0; f < 4; ++f) wm[f] = w[s][f];
        if constexpr (NVT) {
          uint8_t* nl = &nstage[wave][0][0];
          uint32_t* ns = &nscale[wave][0][0];
#pragma unroll
          for (int j = 0; j < 2; ++j) {
            *reinterpret_cast<u32x4*>(nl + j * 1024 + (lane >> 1) * 32 + (lane & 1) * 16) = nvc[s][j];
            if ((lane & 1) == 0) ns[j * 32 + (lane >> 1)] = nvs[s][j];
          }
          __builtin_amdgcn_wave_barrier();
#pragma unroll
          for (int f = 0; f < 4; ++f) {
            const int r32 = (f & 1) * 16 + (lane & 15);
            wm[f].codes = *reinterpret_cast<const u32x2*>(nl + (f >> 1) * 1024 + r32 * 32 + (lane >> 4) * 8);
            wm[f].scale = (ns[(f >> 1) * 32 + r32] >> (8 * (lane >> 4))) & 0xffu;
          }
          __builtin_amdgcn_wave_barrier();
        }
        if constexpr (TR) {  // LDS operations of one wave execute in order: no wait between the writes and the reads
          uint8_t* wl = &wstage[wave][0][0];
#pragma unroll
          for (int f = 0; f < 4; ++f) *reinterpret_cast<u32x4*>(wl + f * 1024 + wr_off) = w[s][f].codes;
          __builtin_amdgcn_wave_barrier();
#pragma unroll
          for (int f = 0; f < 4; ++f) wm[f].codes = *reinterpret_cast<const u32x4*>(wl + f * 1024 + rd_off);
          __builtin_amdgcn_wave_barrier();
        }
#pragma unroll
        for (int f = 0; f < 4; ++f) {
          uint32_t wd[8];
          if constexpr (W16NeedsRow<F>::value) W16<F>::dequant(wm[f], wrow[f], wd);
          else W16<F>::dequant(wm[f], wd);
          const u32x4 x0 = {wd[0], wd[1], wd[2], wd[3]}, x1 = {wd[4], wd[5], wd[6], wd[7]};
          a0[f] = __builtin_bit_cast(w16_bf16x8, x0);
          a1[f] = __builtin_bit_cast(w16_bf16x8, x1);
        }
#pragma unroll
        for (int m = 0; m < MF; ++m) {
          const u32x4 lo = *reinterpret_cast<const u32x4*>(tb + tlo[m]);
          const u32x4 hi = *reinterpret_cast<const u32x4*>(tb + thi[m]);
          const w16_bf16x8 b0 = __builtin_bit_cast(w16_bf16x8, lo), b1 = __builtin_bit_cast(w16_bf16x8, hi);
#pragma unroll
          for (int f = 0; f < 4; ++f) {
            acc[m][f] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a0[f], b0, acc[m][f], 0, 0, 0);
            acc[m][f] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a1[f], b1, acc[m][f], 0, 0, 0);
          }
        }
        // publish token tile kb+1 (requested one stage ago, the weight loads of that stage behind it)
        wait_vm<WL>();
#pragma unroll
        for (int i = 0; i < CPT; ++i) {
          pin(tv[i]);
          if (stage_chunk) *reinterpret_cast<u32x4*>(&tile[(kb & 1) ^ 1][tdst[i]]) = tv[i];
        }
        __syncthreads();
      } else {
        // a stage past the last K block: its registers still have (clamped) loads in flight and are about to be
        // requested into again; a register with a load in flight is never left unread
        wait_vm<0>();
        FF_W16_PIN(s);
#pragma unroll
        for (int i = 0; i < CPT; ++i) pin(tv[i]);
      }
      // request token tile kb+2, then K block kb+P of the weights into the slot just consumed; also past the last K
      // block (clamped addresses), so that the number of loads per stage does not depend on the path
      {
        const uint32_t kn = uint32_t(min(kb + 2, KB - 1));
#pragma unroll
        for (int i = 0; i < CPT; ++i) load16_async(tv[i], tsrc[i] + kn * 128u);
        FF_W16_REQUEST(s, uint32_t(min(kb + P, KB - 1)));
      }
    }
  }
  // the last stages have requested (clamped) data nobody reads: let it land before the registers are reused
  wait_vm<0>();
#pragma unroll
  for (int s = 0; s < P; ++s) FF_W16_PIN(s);
#pragma unroll
  for (int i = 0; i < CPT; ++i) pin(tv[i]);
#undef FF_W16_REQUEST
#undef FF_W16_PIN

  w16_store<MF, MODE>(acc, p, ride, start, n, t, col0, wave, lane);
}

// NW waves per block share one token tile (see k_w8a8_grouped): eight for 64-row groups of a cohort, one block per CU.
template <class F, int MF, int MODE, int P, int NW = 4>
__global__ __launch_bounds__(64 * NW, NW == 4 ? 2 : 1) void k_w16_grouped(const W16Params p) {
  constexpr int TM = 16 * MF;
  const uint32_t total = p.unit_total ? uint32_t(uni(int(load_global<uint32_t>(p.unit_total)))) : p.total_units;
  const int ntiles = (p.N + gemm_tile_cols<MODE, NW>() - 1) / gemm_tile_cols<MODE, NW>();

  // one contiguous span of the unit list per XCD (see k_w8a8_grouped)
  const uint32_t xcd = blockIdx.x & 7u, slot = blockIdx.x >> 3, per_xcd = gridDim.x >> 3;
  const uint32_t span = (total + 7u) >> 3;
  const uint32_t span_end = min(total, (xcd + 1u) * span);
  for (uint32_t u = xcd * span + slot; u < span_end; u += per_xcd) {
    const W16Unit un_ = w16_unit<MODE>(p, u, ntiles, TM);
    w16_unit_run<F, MF, MODE, P, NW>(p, un_);
  }
}

// NVFP4 experts with K a multiple of 256: the codes of 256 columns are one 128-byte line of a weight row, and the kernel
// above asks for a quarter of it per K block (two lanes per row, 32 lines per request, and as many again for the four
// scale bytes) - the vector L1's look-ups, not HBM, bound it. Here a wave moves whole lines: per four K blocks eight
// requests of 8 rows x 128 bytes for its 64 weight rows and one request of 16 scale bytes per row, P such sets ahead,
// into a wave-private LDS image (pieces XOR-swizzled by row / 2 so that the 8-byte operand reads of 16 rows fall into
// distinct banks) that the four K blocks read their operand order from. Arithmetic, token path and epilogue are those of
// k_w16_grouped<FmtNvfp4>, results equal bit for bit.
// Loads per thread and stage, in issue order: the token chunks of tile kb+3 (two tiles are in flight, in two register
// sets), then, in the first K block of a set, the nine weight loads of the set P ahead.
// OCC: blocks per CU the kernel is compiled for. With one set of lines ahead (P = 1) the 16-row kernel holds 143 registers and
// three blocks fit a CU: the conversion work (two VALU instructions per weight) is what bounds NVFP4 cohorts, and a third wave
// per SIMD keeps the vector ALUs busier than a second set of lines in flight does (C4 layer, 32 tokens: 1022 -> 943 us; 8
// tokens: 405 -> 362 us). Four blocks would need 128 registers, which spills.
template <int MF, int MODE, int P, int NW = 4, int OCC = (NW == 4 ? 2 : 1)>
__global__ __launch_bounds__(64 * NW, OCC) void k_w16_nvfp4_lines(const W16Params p) {
  using F = FmtNvfp4;
  constexpr int NT = 64 * NW;
  constexpr int TM = 16 * MF;
  constexpr int CHUNKS = TM * 8;
  constexpr int CPT = (CHUNKS + NT - 1) / NT;
  constexpr int TILE = TM * 128;
  constexpr int WL = 9;                      // weight loads per set of four K blocks
  // Short groups (the cohorts of a decode batch) see an expert's codes once: they are requested with the streaming hint,
  // so that the 128-byte lines of scale bytes, which a row comes back to for eight sets, outlive them in L2 (FETCH_SIZE
  // 1.28 -> 1.08 x the algorithmic bytes in gate/up, C4 batch 32: 1107 -> 1065 us per layer). It takes whole-line
  // requests: on the per-K-block kernels, whose requests leave half a line or more for the next K block, the same hint
  // doubles the traffic (block FP8, batch 64: 1861 -> 2622 us). The 64-row groups of a prefill cohort share an expert's
  // codes through L2 and keep the plain requests.
  constexpr bool STREAM = MF <= 2;
  constexpr int U = 4 * P;                   // stages per trip of the K loop
  __shared__ __attribute__((aligned(16))) uint8_t cstage[NW][2][4096];  // [wave][pair of fragments][32 rows x 128 B]
  __shared__ __attribute__((aligned(16))) uint8_t sstage[NW][1024];     // [wave][64 rows x 16 scale bytes]
  __shared__ __attribute__((aligned(16))) uint8_t tile[2][TILE];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = uni(tid >> 6);
  const int K = p.K, N = p.N, KB = K >> 6, SB = K >> 8;
  const uint32_t total = p.unit_total ? uint32_t(uni(int(load_global<uint32_t>(p.unit_total)))) : p.total_units;
  const int ntiles = (N + gemm_tile_cols<MODE, NW>() - 1) / gemm_tile_cols<MODE, NW>();
  // LDS image: a request i of a pair holds rows 8 i + lane / 8, piece lane % 8; an operand read of K block q takes the
  // 8 bytes of row (16 (f % 2) + lane % 16) at 32 q + 8 (lane / 16)
  const int wr_off = (lane >> 3) * 128 + (((lane & 7) ^ ((lane >> 4) & 3)) << 4);   // + 1024 i, swizzle key (4 i + lane / 16) % 8
  const int rd_row = lane & 15, rd_key = rd_row >> 1;  // the swizzle key (row / 2) % 8 is the same for both fragments of a pair

  const uint32_t xcd = blockIdx.x & 7u, slot = blockIdx.x >> 3, per_xcd = gridDim.x >> 3;
  const uint32_t span = (total + 7u) >> 3;
  const uint32_t span_end = min(total, (xcd + 1u) * span);
  for (uint32_t u = xcd * span + slot; u < span_end; u += per_xcd) {
    const W16Unit un_ = w16_unit<MODE>(p, u, ntiles, TM);
    const int start = un_.start, n = un_.n, t = un_.t;
    const bool ride = un_.ride;  // wave-uniform
    int col0[4];
    typename W16<F>::Row wrow[4];
#pragma unroll
    for (int f = 0; f < 4; ++f) {
      col0[f] = MODE == 0 ? t * (32 * NW) + wave * 32 + (f & 1) * 16 : t * (64 * NW) + wave * 64 + f * 16;
      const int which = MODE == 0 ? f >> 1 : 0;
      wrow[f] = W16<F>::row(un_.wc[which], un_.ws[which], un_.gl[which], min(col0[f], N - 16) + (lane & 15), K);
    }
    // fragments 2 j and 2 j + 1 are 32 consecutive rows of one matrix
    // code addresses: a wave-uniform base per pair (scalar registers) and one byte offset per lane
    uint64_t ncod[2];
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int which = MODE == 0 ? j : 0;
      ncod[j] = uni64(un_.wc[which] + uint64_t(min(col0[2 * j], N - 32)) * uint64_t(K >> 1));
    }
    const uint32_t coff = uint32_t(lane >> 3) * uint32_t(K >> 1) + uint32_t(lane & 7) * 16u;
    const uint32_t rstep = uint32_t(K) * 4u;  // eight rows of codes
    const uint8_t* nscl;
    {
      const bool second = lane >= 32;
      const int row = min(second ? col0[2] : col0[0], N - 32) + (lane & 31);
      nscl = reinterpret_cast<const uint8_t*>(MODE == 0 && second ? un_.ws[1] : un_.ws[0]) + size_t(row) * (K >> 4);
    }
    const uint8_t* nscl_first = reinterpret_cast<const uint8_t*>(un_.ws[0]);  // one valid line for requests past the last set
    u32x4 nvc[P][2][4], nvs[P];

    const uint8_t* tsrc[CPT];
    int tdst[CPT];
#pragma unroll
    for (int i = 0; i < CPT; ++i) {
      const int q = min(tid + NT * i, CHUNKS - 1);
      const int m = q >> 3, c = q & 7;
      const int pos = start + min(m, n - 1);
      const int row = MODE == 0 && p.perm && !ride ? load_global<int>(p.perm + pos) / p.top_k : pos;
      tsrc[i] = reinterpret_cast<const uint8_t*>(ride ? p.a_sh : p.a) + size_t(row) * K * 2 + c * 16;
      tdst[i] = m * 128 + ((c ^ (m & 7)) << 4);
    }
    const bool stage_chunk = CHUNKS >= NT || tid < CHUNKS;

    v4f acc[MF][4];
#pragma unroll
    for (int m = 0; m < MF; ++m)
#pragma unroll
      for (int f = 0; f < 4; ++f) acc[m][f] = v4f{0.0f, 0.0f, 0.0f, 0.0f};

    // nx_: the set asked for. Past the last set the requests only keep the hand-counted number of loads per stage constant
    // and nothing reads them: every one of them then asks for the same line (the first row's last set) instead of the last
    // set's 64 rows once more - with the streaming hint those lines have left L2 by then and came from HBM a second time,
    // 32 KB per block and unit (an eighth of a down unit's bytes).
#define FF_NV_REQUEST(s_, nx_)                                                                          \
  do {                                                                                                   \
    const bool past_ = P == 1 && int(nx_) >= SB; /* two sets ahead: the last set once more, as before */ \
    const uint32_t sb_ = uint32_t(min(int(nx_), SB - 1));                                                \
    const uint32_t rs_ = past_ ? 0u : rstep;                                                             \
    const uint32_t co_ = past_ ? uint32_t(lane & 7) * 16u : coff;                                        \
    _Pragma("unroll") for (int j_ = 0; j_ < 2; ++j_)                                                     \
      _Pragma("unroll") for (int i_ = 0; i_ < 4; ++i_) {                                                 \
        if constexpr (STREAM) load16_async_nt(nvc[s_][j_][i_], ncod[j_] + uint32_t(i_) * rs_ + sb_ * 128u, co_); \
        else load16_async(nvc[s_][j_][i_], ncod[j_] + uint32_t(i_) * rs_ + sb_ * 128u, co_);             \
      }                                                                                                  \
    load16_async(nvs[s_], past_ ? nscl_first : nscl + sb_ * 16u);                                         \
  } while (0)
#define FF_NV_PIN(s_)                                                                                    \
  do {                                                                                                   \
    _Pragma("unroll") for (int j_ = 0; j_ < 2; ++j_)                                                     \
      _Pragma("unroll") for (int i_ = 0; i_ < 4; ++i_) pin(nvc[s_][j_][i_]);                             \
    pin(nvs[s_]);                                                                                        \
  } while (0)
    // prologue: the first P weight sets and token tile 0, everything landed; then token tiles 1 and 2
#pragma unroll
    for (int s = 0; s < P; ++s) FF_NV_REQUEST(s, s);
    u32x4 tv[2][CPT];
    {
#pragma unroll
      for (int i = 0; i < CPT; ++i) {
        const u32x4 v = load16(tsrc[i]);
        if (stage_chunk) *reinterpret_cast<u32x4*>(&tile[0][tdst[i]]) = v;
      }
      wait_vm<0>();
#pragma unroll
      for (int s = 0; s < P; ++s) FF_NV_PIN(s);
#pragma unroll
      for (int tl = 1; tl <= 2; ++tl) {
        const uint32_t kt = uint32_t(min(tl, KB - 1));
#pragma unroll
        for (int i = 0; i < CPT; ++i) load16_async(tv[tl & 1][i], tsrc[i] + kt * 128u);
      }
    }
    __syncthreads();

    int tlo[MF], thi[MF];
#pragma unroll
    for (int m = 0; m < MF; ++m) {
      const int trow = 16 * m + (lane & 15);
      const int q2 = (lane >> 4) * 2;
      tlo[m] = trow * 128 + (((q2) ^ (trow & 7)) << 4);
      thi[m] = trow * 128 + (((q2 + 1) ^ (trow & 7)) << 4);
    }
    uint8_t* cl = &cstage[wave][0][0];
    uint8_t* sl = &sstage[wave][0];

    for (int kbo = 0; kbo < KB; kbo += U) {
      static_for<U>([&](auto st_) {
        constexpr int st = decltype(st_)::value;
        const int kb = kbo + st;
        constexpr int q = st & 3, s = st >> 2;  // K block inside its set, register slot of the set
        if (kb < KB) {
          if (q == 0) {
            // the set was requested 4 P stages ago: behind it the token loads of 4 P - 1 stages and P - 1 later sets
            wait_vm<(4 * P - 1) * CPT + (P - 1) * WL>();
            FF_NV_PIN(s);
#pragma unroll
            for (int j = 0; j < 2; ++j)
#pragma unroll
              for (int i = 0; i < 4; ++i) *reinterpret_cast<u32x4*>(cl + j * 4096 + i * 1024 + (wr_off ^ ((i & 1) << 6))) = nvc[s][j][i];
            *reinterpret_cast<u32x4*>(sl + lane * 16) = nvs[s];
          }
          const uint8_t* tb = tile[st & 1];
          w16_bf16x8 a0[4], a1[4];
#pragma unroll
          for (int f = 0; f < 4; ++f) {
            typename W16<F>::Frag wm;
            const int row = (f & 1) * 16 + rd_row;
            const int piece = 2 * q + (lane >> 5);
            wm.codes = *reinterpret_cast<const u32x2*>(cl + (f >> 1) * 4096 + row * 128 + ((piece ^ rd_key) << 4) + ((lane >> 4) & 1) * 8);
            wm.scale = (*reinterpret_cast<const uint32_t*>(sl + ((f >> 1) * 32 + row) * 16 + q * 4) >> (8 * (lane >> 4))) & 0xffu;
            uint32_t wd[8];
            W16<F>::dequant(wm, wrow[f], wd);
            const u32x4 x0 = {wd[0], wd[1], wd[2], wd[3]}, x1 = {wd[4], wd[5], wd[6], wd[7]};
            a0[f] = __builtin_bit_cast(w16_bf16x8, x0);
            a1[f] = __builtin_bit_cast(w16_bf16x8, x1);
          }
#pragma unroll
          for (int m = 0; m < MF; ++m) {
            const u32x4 lo = *reinterpret_cast<const u32x4*>(tb + tlo[m]);
            const u32x4 hi = *reinterpret_cast<const u32x4*>(tb + thi[m]);
            const w16_bf16x8 b0 = __builtin_bit_cast(w16_bf16x8, lo), b1 = __builtin_bit_cast(w16_bf16x8, hi);
#pragma unroll
            for (int f = 0; f < 4; ++f) {
              acc[m][f] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a0[f], b0, acc[m][f], 0, 0, 0);
              acc[m][f] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a1[f], b1, acc[m][f], 0, 0, 0);
            }
          }
          // publish token tile kb+1: requested two stages ago, behind it tile kb+2 and the set a first K block requests
          wait_vm<CPT + ((q == 1 || q == 2) ? WL : 0)>();
#pragma unroll
          for (int i = 0; i < CPT; ++i) {
            pin(tv[(st + 1) & 1][i]);
            if (stage_chunk) *reinterpret_cast<u32x4*>(&tile[(st + 1) & 1][tdst[i]]) = tv[(st + 1) & 1][i];
          }
          __syncthreads();
        } else {
          // past the last K block: registers with (clamped) loads in flight are about to be requested into again
          wait_vm<0>();
#pragma unroll
          for (int ss = 0; ss < P; ++ss) FF_NV_PIN(ss);
#pragma unroll
          for (int i = 0; i < CPT; ++i) { pin(tv[0][i]); pin(tv[1][i]); }
        }
        {
          const uint32_t kt = uint32_t(min(kb + 3, KB - 1));
#pragma unroll
          for (int i = 0; i < CPT; ++i) load16_async(tv[(st + 1) & 1][i], tsrc[i] + kt * 128u);
          if (q == 0) FF_NV_REQUEST(s, (kb >> 2) + P);
        }
      });
    }
    wait_vm<0>();
#pragma unroll
    for (int s = 0; s < P; ++s) FF_NV_PIN(s);
#pragma unroll
    for (int i = 0; i < CPT; ++i) { pin(tv[0][i]); pin(tv[1][i]); }
#undef FF_NV_REQUEST
#undef FF_NV_PIN

    w16_store<MF, MODE>(acc, p, ride, start, n, t, col0, wave, lane);
  }
}

// Block-FP8 experts the same way: 128 columns of a row are one 128-byte line, a set is two K blocks, and the block scale of a
// pair of fragments and a set is one float (a pair's 32 rows lie inside one 128-row block). Bit-identical to
// k_w16_grouped<FmtFp8>, whose requests take half a line per K block and rely on L2 for the other half.
template <int MF, int MODE, int P, int NW = 4, int OCC = (NW == 4 ? 2 : 1)>
__global__ __launch_bounds__(64 * NW, OCC) void k_w16_fp8_lines(const W16Params p) {
  using F = FmtFp8;
  // One set of lines ahead (P = 1): 118 - 123 registers instead of 183 - 187, so three or four blocks fit a CU (OCC; 36 KB of LDS
  // per block), and more waves per SIMD beat a second set of lines in flight here too (C3 layer, 64 tokens: 1736 -> 1647 us; 8
  // tokens: 481 -> 461 us). Its K loop covers TWO sets per trip: with one set per trip (two stages) the register allocator
  // split the token registers' live ranges at the back edge and restored them with v_mov_b64 while their loads were in flight
  // (flagged by the check of the generated assembly; wrong bits on the GPU, with the loads' destinations as outputs and as
  // in/out operands alike); with four stages per trip it does not.
  constexpr int NT = 64 * NW;
  constexpr int TM = 16 * MF;
  constexpr int CHUNKS = TM * 8;
  constexpr int CPT = (CHUNKS + NT - 1) / NT;
  constexpr int TILE = TM * 128;
  constexpr int WL = 10;                     // weight loads per set of two K blocks: eight of codes, two block scales
  // 16-row groups (the cohorts of a decode batch) see an expert's codes once: streaming hint on their whole-line requests
  constexpr bool STREAM = MF == 1;
  constexpr int U = P == 1 ? 4 : 2 * P;      // stages per trip of the K loop (one set ahead: two sets per trip)
  __shared__ __attribute__((aligned(16))) uint8_t cstage[NW][2][4096];  // [wave][pair of fragments][32 rows x 128 B]
  __shared__ __attribute__((aligned(16))) uint8_t tile[2][TILE];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = uni(tid >> 6);
  const int K = p.K, N = p.N, KB = K >> 6, SB = K >> 7;
  const uint32_t total = p.unit_total ? uint32_t(uni(int(load_global<uint32_t>(p.unit_total)))) : p.total_units;
  const int ntiles = (N + gemm_tile_cols<MODE, NW>() - 1) / gemm_tile_cols<MODE, NW>();
  // LDS image: a request i of a pair holds rows 8 i + lane / 8, piece lane % 8; an operand read of K block q takes the
  // 16 bytes of row (16 (f % 2) + lane % 16) at 64 q + 16 (lane / 16)
  const int wr_off = (lane >> 3) * 128 + (((lane & 7) ^ ((lane >> 4) & 3)) << 4);   // + 1024 i, swizzle key (4 i + lane / 16) % 8
  const int rd_row = lane & 15, rd_key = rd_row >> 1;  // the swizzle key (row / 2) % 8 is the same for both fragments of a pair

  const uint32_t xcd = blockIdx.x & 7u, slot = blockIdx.x >> 3, per_xcd = gridDim.x >> 3;
  const uint32_t span = (total + 7u) >> 3;
  const uint32_t span_end = min(total, (xcd + 1u) * span);
  for (uint32_t u = xcd * span + slot; u < span_end; u += per_xcd) {
    const W16Unit un_ = w16_unit<MODE>(p, u, ntiles, TM);
    const int start = un_.start, n = un_.n, t = un_.t;
    const bool ride = un_.ride;  // wave-uniform
    int col0[4];
#pragma unroll
    for (int f = 0; f < 4; ++f) col0[f] = MODE == 0 ? t * (32 * NW) + wave * 32 + (f & 1) * 16 : t * (64 * NW) + wave * 64 + f * 16;
    // fragments 2 j and 2 j + 1 are 32 consecutive rows of one matrix
    // code addresses: a wave-uniform base per pair (scalar registers) and one byte offset per lane
    uint64_t ncod[2];
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int which = MODE == 0 ? j : 0;
      ncod[j] = uni64(un_.wc[which] + uint64_t(min(col0[2 * j], N - 32)) * uint64_t(K));
    }
    const uint32_t coff = uint32_t(lane >> 3) * uint32_t(K) + uint32_t(lane & 7) * 16u;
    const uint32_t rstep = uint32_t(K) * 8u;  // eight rows of codes
    // block scales: one per pair of fragments (32 rows inside one 128-row block) and set (128 columns)
    const float* nscl[2];
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int which = MODE == 0 ? j : 0;
      nscl[j] = reinterpret_cast<const float*>(un_.ws[which]) + size_t(min(col0[2 * j], N - 32) >> 7) * size_t(SB);
    }
    u32x4 nvc[P][2][4];
    float nvs[P][2];

    const uint8_t* tsrc[CPT];
    int tdst[CPT];
#pragma unroll
    for (int i = 0; i < CPT; ++i) {
      const int q = min(tid + NT * i, CHUNKS - 1);
      const int m = q >> 3, c = q & 7;
      const int pos = start + min(m, n - 1);
      const int row = MODE == 0 && p.perm && !ride ? load_global<int>(p.perm + pos) / p.top_k : pos;
      tsrc[i] = reinterpret_cast<const uint8_t*>(ride ? p.a_sh : p.a) + size_t(row) * K * 2 + c * 16;
      tdst[i] = m * 128 + ((c ^ (m & 7)) << 4);
    }
    const bool stage_chunk = CHUNKS >= NT || tid < CHUNKS;

    v4f acc[MF][4];
#pragma unroll
    for (int m = 0; m < MF; ++m)
#pragma unroll
      for (int f = 0; f < 4; ++f) acc[m][f] = v4f{0.0f, 0.0f, 0.0f, 0.0f};

    // nx_: the set asked for; past the last set every request asks for one and the same line (see k_w16_nvfp4_lines)
#define FF_NV_REQUEST(s_, nx_)                                                                          \
  do {                                                                                                   \
    const bool past_ = P == 1 && int(nx_) >= SB; /* two sets ahead: the last set once more, as before */ \
    const uint32_t sb_ = uint32_t(min(int(nx_), SB - 1));                                                \
    const uint32_t rs_ = past_ ? 0u : rstep;                                                             \
    const uint32_t co_ = past_ ? uint32_t(lane & 7) * 16u : coff;                                        \
    _Pragma("unroll") for (int j_ = 0; j_ < 2; ++j_)                                                     \
      _Pragma("unroll") for (int i_ = 0; i_ < 4; ++i_) {                                                 \
        if constexpr (STREAM) load16_async_nt(nvc[s_][j_][i_], ncod[j_] + uint32_t(i_) * rs_ + sb_ * 128u, co_); \
        else load16_async(nvc[s_][j_][i_], ncod[j_] + uint32_t(i_) * rs_ + sb_ * 128u, co_);             \
      }                                                                                                  \
    _Pragma("unroll") for (int j_ = 0; j_ < 2; ++j_) load4_async(nvs[s_][j_], nscl[j_] + sb_);             \
  } while (0)
#define FF_NV_PIN(s_)                                                                                    \
  do {                                                                                                   \
    _Pragma("unroll") for (int j_ = 0; j_ < 2; ++j_)                                                     \
      _Pragma("unroll") for (int i_ = 0; i_ < 4; ++i_) pin(nvc[s_][j_][i_]);                             \
    _Pragma("unroll") for (int j_ = 0; j_ < 2; ++j_) pin(nvs[s_][j_]);                                     \
  } while (0)
    // prologue: the first P - 1 weight sets and token tile 0, everything landed; then token tile 1, set P - 1 (a tile has
    // one set's loads and the next tile behind it when it is published) and token tile 2
#pragma unroll
    for (int s = 0; s + 1 < P; ++s) FF_NV_REQUEST(s, s);
    u32x4 tv[2][CPT];
    {
#pragma unroll
      for (int i = 0; i < CPT; ++i) {
        const u32x4 v = load16(tsrc[i]);
        if (stage_chunk) *reinterpret_cast<u32x4*>(&tile[0][tdst[i]]) = v;
      }
      wait_vm<0>();
#pragma unroll
      for (int s = 0; s + 1 < P; ++s) FF_NV_PIN(s);
      const uint32_t k1 = uint32_t(min(1, KB - 1)), k2 = uint32_t(min(2, KB - 1));
#pragma unroll
      for (int i = 0; i < CPT; ++i) load16_async(tv[1][i], tsrc[i] + k1 * 128u);
      FF_NV_REQUEST(P - 1, P - 1);
#pragma unroll
      for (int i = 0; i < CPT; ++i) load16_async(tv[0][i], tsrc[i] + k2 * 128u);
    }
    __syncthreads();

    int tlo[MF], thi[MF];
#pragma unroll
    for (int m = 0; m < MF; ++m) {
      const int trow = 16 * m + (lane & 15);
      const int q2 = (lane >> 4) * 2;
      tlo[m] = trow * 128 + (((q2) ^ (trow & 7)) << 4);
      thi[m] = trow * 128 + (((q2 + 1) ^ (trow & 7)) << 4);
    }
    uint8_t* cl = &cstage[wave][0][0];
    float sc_set[2] = {0.0f, 0.0f};  // block scales of the set at work (its register slot is requested into again after the set's first K block)

    for (int kbo = 0; kbo < KB; kbo += U) {
      static_for<U>([&](auto st_) {
        constexpr int st = decltype(st_)::value;
        const int kb = kbo + st;
        constexpr int q = st & 1, s = (st >> 1) % P;  // K block inside its set, register slot of the set
        if (kb < KB) {
          if (q == 0) {
            // the set was requested 2 P stages ago: behind it the token loads of 2 P - 1 stages and P - 1 later sets
            wait_vm<(2 * P - 1) * CPT + (P - 1) * WL>();
            FF_NV_PIN(s);
#pragma unroll
            for (int j = 0; j < 2; ++j)
#pragma unroll
              for (int i = 0; i < 4; ++i) *reinterpret_cast<u32x4*>(cl + j * 4096 + i * 1024 + (wr_off ^ ((i & 1) << 6))) = nvc[s][j][i];
            sc_set[0] = nvs[s][0];
            sc_set[1] = nvs[s][1];
          }
          const uint8_t* tb = tile[st & 1];
          w16_bf16x8 a0[4], a1[4];
#pragma unroll
          for (int f = 0; f < 4; ++f) {
            typename W16<F>::Frag wm;
            const int row = (f & 1) * 16 + rd_row;
            const int piece = 4 * q + (lane >> 4);
            wm.codes = *reinterpret_cast<const u32x4*>(cl + (f >> 1) * 4096 + row * 128 + ((piece ^ rd_key) << 4));
            wm.scale = sc_set[f >> 1];
            uint32_t wd[8];
            W16<F>::dequant(wm, wd);
            const u32x4 x0 = {wd[0], wd[1], wd[2], wd[3]}, x1 = {wd[4], wd[5], wd[6], wd[7]};
            a0[f] = __builtin_bit_cast(w16_bf16x8, x0);
            a1[f] = __builtin_bit_cast(w16_bf16x8, x1);
          }
#pragma unroll
          for (int m = 0; m < MF; ++m) {
            const u32x4 lo = *reinterpret_cast<const u32x4*>(tb + tlo[m]);
            const u32x4 hi = *reinterpret_cast<const u32x4*>(tb + thi[m]);
            const w16_bf16x8 b0 = __builtin_bit_cast(w16_bf16x8, lo), b1 = __builtin_bit_cast(w16_bf16x8, hi);
#pragma unroll
            for (int f = 0; f < 4; ++f) {
              acc[m][f] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a0[f], b0, acc[m][f], 0, 0, 0);
              acc[m][f] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a1[f], b1, acc[m][f], 0, 0, 0);
            }
          }
          // publish token tile kb+1: requested two stages ago, behind it tile kb+2 and the one set the two stages requested
          wait_vm<CPT + WL>();
#pragma unroll
          for (int i = 0; i < CPT; ++i) {
            pin(tv[(st + 1) & 1][i]);
            if (stage_chunk) *reinterpret_cast<u32x4*>(&tile[(st + 1) & 1][tdst[i]]) = tv[(st + 1) & 1][i];
          }
          __syncthreads();
        } else {
          // past the last K block: registers with (clamped) loads in flight are about to be requested into again
          wait_vm<0>();
#pragma unroll
          for (int ss = 0; ss < P; ++ss) FF_NV_PIN(ss);
#pragma unroll
          for (int i = 0; i < CPT; ++i) { pin(tv[0][i]); pin(tv[1][i]); }
        }
        {
          const uint32_t kt = uint32_t(min(kb + 3, KB - 1));
#pragma unroll
          for (int i = 0; i < CPT; ++i) load16_async(tv[(st + 1) & 1][i], tsrc[i] + kt * 128u);
          if (q == 0) FF_NV_REQUEST(s, (kb >> 1) + P);
        }
      });
    }
    wait_vm<0>();
#pragma unroll
    for (int s = 0; s < P; ++s) FF_NV_PIN(s);
#pragma unroll
    for (int i = 0; i < CPT; ++i) { pin(tv[0][i]); pin(tv[1][i]); }
#undef FF_NV_REQUEST
#undef FF_NV_PIN

    w16_store<MF, MODE>(acc, p, ride, start, n, t, col0, wave, lane);
  }
}

}  // namespace ffmoe
