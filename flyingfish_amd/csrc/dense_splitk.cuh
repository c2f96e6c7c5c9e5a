// A dense BF16 expert (the shared expert next to experts of another format) over a few dozen token rows, the contraction
// split over the eight waves of a block. The grouped kernels give such an expert a few dozen one-wave tiles, each
// walking the whole contraction behind a token tile with one stage of lead: 62 + 19 us for 32 rows at hidden 7168 /
// intermediate 2048, 1.1 TB/s. Here a block owns 16 weight rows (MODE 0: 8 gate rows and the 8 matching up rows in one
// fragment; MODE 2: 16 output columns) and its waves an eighth of K each, every operand is
// requested straight from memory in the matrix instruction's lane order (a lane's 8 consecutive K elements of one weight
// row or token row are 16 contiguous bytes), a chunk of K steps ahead, and the eight partial tiles meet in LDS and are
// added in wave order.
//
// Arithmetic: BF16 weights as they are, BF16 activations, v_mfma_f32_16x16x32_bf16, FP32 partial sums; BF16 boundaries at
// gate, up (before SwiGLU), the SwiGLU product and the down output, as in w16_gemm.cuh and the streaming kernels - the
// summation order (matrix instruction, then eight partials) is this kernel's own, so it is a tolerance-checked variant
// like the other matrix-core paths.
//
// MODE 0: act[row, j] = SwiGLU(gate_j . x_row, up_j . x_row)      MODE 2: y[row, n] = w_n . act_row
#pragma once
#include "w16_gemm.cuh"

namespace ffmoe {

struct DenseParams {
  const uint16_t* x;   // [rows, K] BF16
  const uint16_t* w0;  // [N, K] BF16 (gate, or down)
  const uint16_t* w1;  // [N, K] BF16 (up; MODE 0)
  uint16_t* out;       // [rows, N] BF16
  int rows, K, N, swiglu;
  float limit;
};

// MFT token fragments of 16 rows per block; blockIdx.x = column tile of 16, blockIdx.y = row block of 16 * MFT
// TC output columns per block: MODE 0: 8 (gate rows 0-7, up rows 8-15 of the fragment); MODE 2: 16. (Half of that, the
// fragment's upper rows repeating the lower ones, also works and is slower: every block reads the whole token panel.)
// XL: the token panel goes through LDS. Requested in the instruction's lane order a token load touches 64 lines for 16 bytes
// each (the 16 lanes of a quarter wave are 16 token rows), and with two or four token fragments per weight fragment those
// loads, not the weights, were the kernel's time: 31.6 us for the gate/up launch of 32 rows at hidden 7168, 16.6 us with
// every lane reading one row's bytes (wrong results). A round is one chunk of every wave = 1024 contiguous columns; the
// block moves the round's 16 MFT x 2 KB of token rows with row-contiguous requests (128 threads per row) into one of two
// LDS buffers a round ahead, and a lane reads its fragment pieces from there (rows padded by 16 bytes). Same operands into
// the same instructions in the same order: bit-identical. Needs the dealt chunk order (steps per wave a multiple of CH).
template <int MODE, int MFT, int TC, int NA = 1, bool XL = false>
__global__ __launch_bounds__(512, 1) void k_dense_bf16_splitk(const DenseParams p) {
  constexpr int NWV = 8;               // waves = parts of the contraction
  constexpr int CH = 4;                // K steps (of 32) per chunk in flight
  // NA weight fragments per block: one of 8 gate + 8 up rows (MODE 0), NA of 16 down rows (MODE 2: TC * NA columns)
  static_assert(MODE != 0 || NA == 1, "gate/up blocks hold one fragment");
  constexpr int RR = MODE == 0 ? 2 * TC : TC;  // distinct weight rows of the fragment
  static_assert(RR == 16 || RR == 8, "fragment rows");
  constexpr int XROWS = 16 * MFT, XRS = 2048 + 16, XBUF = XROWS * XRS;  // XL: token rows, bytes per row and per buffer
  extern __shared__ __attribute__((aligned(16))) uint8_t xl_lds[];        // XL: two token buffers, then the partial tiles
  __shared__ __attribute__((aligned(16))) float red_s[XL ? 4 : NWV * NA * MFT * 64 * 4];
  float* red = XL ? reinterpret_cast<float*>(xl_lds) : red_s;             // [wave][fragment][lane][4]
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = uni(tid >> 6);
  const int K = p.K, N = p.N;
  const int n0 = blockIdx.x * (TC * NA), m0 = blockIdx.y * (16 * MFT);
  const int i = lane & 15, c = lane >> 4;
  const int steps = K / (32 * NWV);  // per wave; K is a multiple of 256
  // Which steps a wave takes: chunks of CH steps dealt round-robin to the waves, so that the block reads 8 * CH * 64 bytes =
  // 2 KB of a weight row side by side (one DRAM page's worth) instead of eight runs 1/8 of the row apart; rows whose
  // steps per wave are no multiple of CH fall back to one contiguous eighth per wave.
  const bool dealt = steps % CH == 0;
  auto step_k = [&](int s) { return (dealt ? ((s / CH) * NWV + wave) * CH + (s % CH) : wave * steps + s) * 32; };
  // operand rows of this lane: weight row n0 + i, token rows m0 + 16 m + i (clamped into the cohort, dropped at the store)
  const uint16_t* wr[NA];
#pragma unroll
  for (int a = 0; a < NA; ++a) {
    const int ir = i & (RR - 1);  // rows past RR repeat the fragment's first rows
    wr[a] = (MODE == 0 && ir >= TC ? p.w1 + size_t(n0 + ir - TC) * K : p.w0 + size_t(n0 + TC * a + ir) * K) + 8 * c;
  }
  const uint16_t* xr[MFT];
#pragma unroll
  for (int m = 0; m < MFT; ++m) xr[m] = p.x + size_t(min(m0 + 16 * m + i, p.rows - 1)) * K + 8 * c;

  v4f acc[NA][MFT];
#pragma unroll
  for (int a = 0; a < NA; ++a)
#pragma unroll
    for (int m = 0; m < MFT; ++m) acc[a][m] = v4f{0.0f, 0.0f, 0.0f, 0.0f};
  // a ring of NBUF chunk buffers: chunk q sits in buffer q % NBUF and is requested NBUF - 1 chunks before it is multiplied
  // (four buffers where the registers allow them measured slower than two: 36.7 against 31.9 us for the gate/up launch of
  // 32 rows at hidden 7168)
  constexpr int NBUF = 2;
  u32x4 wa[NBUF][CH][NA], xb[NBUF][CH][MFT];
  auto request = [&](auto slot_, int s0) {  // steps s0 .. s0 + CH - 1, clamped to the wave's last step
    constexpr int s_ = decltype(slot_)::value;
#pragma unroll
    for (int j = 0; j < CH; ++j) {
      const int st = step_k(min(s0 + j, steps - 1));
#pragma unroll
      // no streaming hint: a request covers half of each 128-byte line it touches, the next step's request the other half,
      // and a hinted line may be gone from the L2 in between
      for (int a = 0; a < NA; ++a) wa[s_][j][a] = load16(wr[a] + st);
#pragma unroll
      for (int m = 0; m < MFT; ++m) xb[s_][j][m] = load16(xr[m] + st);
    }
  };
  auto multiply = [&](auto slot_, int s0) {
    constexpr int s_ = decltype(slot_)::value;
#pragma unroll
    for (int j = 0; j < CH; ++j) {
      if (s0 + j < steps) {
#pragma unroll
        for (int a = 0; a < NA; ++a)
#pragma unroll
          for (int m = 0; m < MFT; ++m)
            acc[a][m] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(w16_bf16x8, wa[s_][j][a]), __builtin_bit_cast(w16_bf16x8, xb[s_][j][m]),
                                                               acc[a][m], 0, 0, 0);
      }
    }
  };
  if constexpr (XL) {
    // token rows of a round: thread (piece tid % 128, row tid / 128 + 4 k)
    constexpr int TP = XROWS / 4;
    u32x4 tv[TP];
    const int piece = tid & 127, rsub = tid >> 7;
    auto load_tokens = [&](int r) {
#pragma unroll
      for (int k = 0; k < TP; ++k)
        tv[k] = load16(p.x + size_t(min(m0 + 4 * k + rsub, p.rows - 1)) * K + size_t(r) * 1024 + piece * 8);
    };
    auto store_tokens = [&](int r) {
#pragma unroll
      for (int k = 0; k < TP; ++k) *reinterpret_cast<u32x4*>(xl_lds + (r & 1) * XBUF + (4 * k + rsub) * XRS + piece * 16) = tv[k];
    };
    auto request_w = [&](auto slot_, int s0) {
      constexpr int s_ = decltype(slot_)::value;
#pragma unroll
      for (int j = 0; j < CH; ++j) {
        const int st = step_k(min(s0 + j, steps - 1));
#pragma unroll
        for (int a = 0; a < NA; ++a) wa[s_][j][a] = load16(wr[a] + st);
      }
    };
    auto multiply_l = [&](auto slot_, int r) {
      constexpr int s_ = decltype(slot_)::value;
      const uint8_t* tok = xl_lds + (r & 1) * XBUF + i * XRS + (wave * CH) * 64 + 16 * c;
#pragma unroll
      for (int j = 0; j < CH; ++j) {
#pragma unroll
        for (int m = 0; m < MFT; ++m) {
          const u32x4 xv = *reinterpret_cast<const u32x4*>(tok + 16 * m * XRS + j * 64);
#pragma unroll
          for (int a = 0; a < NA; ++a)
            acc[a][m] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(w16_bf16x8, wa[s_][j][a]), __builtin_bit_cast(w16_bf16x8, xv),
                                                               acc[a][m], 0, 0, 0);
        }
      }
    };
    const int rounds = steps / CH;
    load_tokens(0);
    request_w(std::integral_constant<int, 0>{}, 0);
    store_tokens(0);
    if (rounds > 1) load_tokens(1);
    __syncthreads();
    auto round = [&](auto slot_, int r) {
      constexpr int s_ = decltype(slot_)::value;
      if (r + 1 < rounds) request_w(std::integral_constant<int, s_ ^ 1>{}, (r + 1) * CH);
      multiply_l(slot_, r);
      if (r + 1 < rounds) store_tokens(r + 1);
      if (r + 2 < rounds) load_tokens(r + 2);
      __syncthreads();
    };
    for (int r = 0; r < rounds; r += 2) {
      round(std::integral_constant<int, 0>{}, r);
      if (r + 1 < rounds) round(std::integral_constant<int, 1>{}, r + 1);
    }
  } else {
  static_for<NBUF - 1>([&](auto ib) { request(ib, decltype(ib)::value * CH); });
  for (int s0 = 0; s0 < steps; s0 += NBUF * CH) {
    static_for<NBUF>([&](auto ib) {
      constexpr int b = decltype(ib)::value;
      request(std::integral_constant<int, (b + NBUF - 1) % NBUF>{}, s0 + (b + NBUF - 1) * CH);
      multiply(ib, s0 + b * CH);
    });
  }
  }

  // the eight partial tiles, added in wave order
#pragma unroll
  for (int a = 0; a < NA; ++a)
#pragma unroll
    for (int m = 0; m < MFT; ++m) *reinterpret_cast<v4f*>(red + ((wave * (NA * MFT) + a * MFT + m) * 64 + lane) * 4) = acc[a][m];
  __syncthreads();
  // wave m < MFT finishes token fragment m: lane (token i, group c) holds weight rows 4c .. 4c+3 of the fragment. MODE 0:
  // the first TC / 4 groups are gate columns n0 .. n0 + TC - 1 and the next TC / 4 the same columns of up, so a lane of the
  // first groups also reads the partials of the lane 4 TC further on.
  if (wave < MFT && c < TC / 4) {
    const int m = wave;
    const int row = m0 + 16 * m + i;
#pragma unroll
    for (int f = 0; f < NA; ++f) {
      float v[2][4];
#pragma unroll
      for (int a = 0; a < (MODE == 0 ? 2 : 1); ++a) {
        const int src = lane + 4 * TC * a;  // the up rows sit TC rows = TC / 4 lane groups further on
        const v4f first = *reinterpret_cast<const v4f*>(red + ((f * MFT + m) * 64 + src) * 4);
#pragma unroll
        for (int r = 0; r < 4; ++r) v[a][r] = first[r];
#pragma unroll
        for (int w = 1; w < NWV; ++w) {
          const v4f part = *reinterpret_cast<const v4f*>(red + ((w * (NA * MFT) + f * MFT + m) * 64 + src) * 4);
#pragma unroll
          for (int r = 0; r < 4; ++r) v[a][r] = __fadd_rn(v[a][r], part[r]);
        }
      }
      if (row < p.rows) {
        u32x2 o;
        if (MODE == 0) {
          uint32_t h[4];
#pragma unroll
          for (int r = 0; r < 4; ++r) h[r] = swiglu_bf16(bround(v[0][r]), bround(v[1][r]), p.swiglu, p.limit);
          o = u32x2{h[0] | (h[1] << 16), h[2] | (h[3] << 16)};
        } else {
          o = u32x2{pack_bf16x2(v[0][0], v[0][1]), pack_bf16x2(v[0][2], v[0][3])};
        }
        *reinterpret_cast<u32x2*>(p.out + size_t(row) * N + n0 + TC * f + 4 * c) = o;
      }
    }
  }
}

}  // namespace ffmoe
