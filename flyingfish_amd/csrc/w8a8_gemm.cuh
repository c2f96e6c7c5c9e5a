// Grouped W8A8 GEMM on the FP8 matrix cores: E4M3 weights with 128x128 f32 block scales against E4M3 activations
// with one f32 scale per (row, 128 columns), as the reference's block-F32 path defines it
// (kernels/q38_contract.cuh:239-279): for every output and every K block of 128
//     total = fma(sum_128(w * x), sw[n/128][kb] * sx[row][kb], total),   BF16 store.
// One v_mfma_f32_16x16x128_f8f6f4 is exactly one K block for a 16x16 tile, so the block sum comes out of the
// matrix core with a zero accumulator and the scale product is applied by one VALU fma per output.
//
// Work model. Token rows that hit the same expert are gathered into groups of at most TM = 16*MF rows. A unit is
// one group x one tile of output columns; blocks take units round-robin, so blocks running side by side work on
// neighbouring units (same expert, same column tile, different row groups) and share the weight lines in cache. Each wave
// owns four 16-row weight fragments of the tile and streams them straight from global memory into registers
// (a lane loads 32 contiguous bytes of one weight row, P K-blocks ahead); the token tile of a K block is staged
// through LDS once per block and shared by the four waves. Weights are the A operand, tokens the B operand, so a
// lane ends up with four consecutive output columns of one token: one 8-byte store per fragment.
//
// MODE 0: gate/up + SwiGLU (two-branch sigmoid, kernels/act.cu:125-159) -> act[pos, j]
// MODE 1: down, BF16, x routing weight (kernels/moe_ffn.cu:894-908) -> contributions[assignment, d], done = 1
// MODE 2: plain linear -> y[row, n]
#pragma once
#include "common.cuh"
#include "../../include/ffmoe.h"

namespace ffmoe {

typedef int v8i __attribute__((ext_vector_type(8)));
typedef float v4f __attribute__((ext_vector_type(4)));

struct GemmGroup { int expert, start, n, pad; };  // rows [start, start + n) of the permuted order

struct GemmParams {
  const uint8_t* a_codes;    // activation codes [*, K]
  const float* a_scales;     // activation scales [*, K/128]
  const uint64_t* slots;     // [E, 6] expert table, or NULL: the four addresses below
  uint64_t w0_codes, w0_scales, w1_codes, w1_scales;  // MODE 0: gate, up; MODE 1/2: w0 only
  const GemmGroup* groups;   // NULL: rows split arithmetically into groups of TM (single matrix)
  const u32x2* units;       // (group, tile) per unit, or NULL with groups == NULL
  const uint32_t* unit_total;  // device word: number of units (NULL: total_units)
  uint32_t total_units;
  const int* perm;           // permuted position -> assignment index (NULL: identity)
  const void* weights;       // routing weights per assignment (MODE 1; NULL: 1)
  uint16_t* out;
  uint32_t* done;
  int rows_total;            // identity mode: number of rows
  int K, N, top_k, weights_f32, swiglu, routed_weight;
  float limit;
};

template <int MODE>
__device__ __forceinline__ constexpr int gemm_tile_cols() { return MODE == 0 ? 128 : 256; }

template <int MF, int MODE, int P>
__global__ __launch_bounds__(256, MF <= 4 ? 2 : 1) void k_w8a8_grouped(const GemmParams p) {
  constexpr int TM = 16 * MF;
  constexpr int CHUNKS = TM * 8;                    // 16-byte token chunks per K block
  constexpr int CPT = (CHUNKS + 255) / 256;         // chunks a thread moves per K block
  constexpr int TILE = TM * 128 + TM * 4;           // codes + scales
  __shared__ __attribute__((aligned(16))) uint8_t tile[2][TILE];
  // Weight fragments are requested row-contiguously (8 lanes per 128-byte row segment, 8 rows per instruction) and
  // turned into the operand's lane order (row lane % 16, bytes 32 (lane / 16) .. + 31) through this wave-private
  // buffer: requested in operand order, the 16 consecutive lanes of a quarter wave touch 16 different lines for 16
  // bytes each and the vector L1 spends one look-up per 16 bytes (929 -> 1295 TFLOP/s in the cache-resident case when
  // only the addresses are changed). Pieces are XOR-swizzled by the row; LDS operations of one wave execute in order,
  // so no wait sits between the writes and the reads.
  // Short groups (MF < 4) are bound by HBM, not by the L1: they keep the direct requests and skip the LDS round trip.
  constexpr bool TW = MF >= 4;
  __shared__ __attribute__((aligned(16))) uint8_t wstage[TW ? 4 : 1][TW ? 4 : 1][TW ? 2048 : 16];  // [wave][fragment][16 rows x 128 B]
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = uni(tid >> 6);
  const int K = p.K, N = p.N, KB = K >> 7;
  const int wr_off = (lane >> 3) * 128 + (((lane & 7) ^ ((lane >> 3) & 7)) << 4);                 // rows 0..7; rows 8..15 at + 1024
  const int rd_lo = (lane & 15) * 128 + (((2 * (lane >> 4)) ^ (lane & 7)) << 4);
  const int rd_hi = (lane & 15) * 128 + (((2 * (lane >> 4) + 1) ^ (lane & 7)) << 4);
  const uint32_t total = p.unit_total ? uint32_t(uni(int(load_global<uint32_t>(p.unit_total)))) : p.total_units;
  const int ntiles = (N + gemm_tile_cols<MODE>() - 1) / gemm_tile_cols<MODE>();

  // Blocks are dealt to the 8 XCDs round-robin, and each XCD has its own L2. The unit list is cut into 8 contiguous
  // spans, one per XCD, and the blocks of an XCD walk their span side by side, so the row groups of one (expert,
  // column tile) meet in the same L2 and its weights leave HBM once.
  const uint32_t xcd = blockIdx.x & 7u, slot = blockIdx.x >> 3, per_xcd = gridDim.x >> 3;
  const uint32_t span = (total + 7u) >> 3;
  const uint32_t span_end = min(total, (xcd + 1u) * span);
  for (uint32_t u = xcd * span + slot; u < span_end; u += per_xcd) {

    int expert, start, n, t;
    if (p.groups) {
      const u32x2 un = load_global<u32x2>(p.units + u);
      const int g = uni(int(un.x));
      t = uni(int(un.y));
      const int* gd = reinterpret_cast<const int*>(p.groups + g);
      expert = uni(load_global<int>(gd));
      start = uni(load_global<int>(gd + 1));
      n = uni(load_global<int>(gd + 2));
    } else {
      const int g = int(u) / ntiles;
      t = int(u) - g * ntiles;
      expert = 0;
      start = g * TM;
      n = min(TM, p.rows_total - start);
    }

    // weight fragments of this wave
    uint64_t wc[2], ws[2];
    if (p.slots) {
      const uint64_t* sl = p.slots + size_t(expert) * 6;
      if (MODE == 0) {
        wc[0] = uni64(load_global<uint64_t>(sl + 0)); ws[0] = uni64(load_global<uint64_t>(sl + 1));
        wc[1] = uni64(load_global<uint64_t>(sl + 2)); ws[1] = uni64(load_global<uint64_t>(sl + 3));
      } else {
        wc[0] = wc[1] = uni64(load_global<uint64_t>(sl + 4)); ws[0] = ws[1] = uni64(load_global<uint64_t>(sl + 5));
      }
    } else {
      wc[0] = p.w0_codes; ws[0] = p.w0_scales;
      wc[1] = MODE == 0 ? p.w1_codes : p.w0_codes; ws[1] = MODE == 0 ? p.w1_scales : p.w0_scales;
    }
    // first output column of fragment f; fragments past N are clamped onto the last 16 rows and dropped at the store
    int col0[4];
    const uint8_t* wrow[4];
#pragma unroll
    for (int f = 0; f < 4; ++f) {
      col0[f] = MODE == 0 ? t * 128 + wave * 32 + (f & 1) * 16 : t * 256 + wave * 64 + f * 16;
      const int base = min(col0[f], N - 16);
      const uint64_t codes = MODE == 0 ? wc[f >> 1] : wc[0];
      wrow[f] = TW ? reinterpret_cast<const uint8_t*>(codes) + size_t(base + (lane >> 3)) * K + (lane & 7) * 16  // rows 0..7 of the fragment
                   : reinterpret_cast<const uint8_t*>(codes) + size_t(base + (lane & 15)) * K + (lane >> 4) * 32;
    }
    const uint32_t wsecond = TW ? 8u * uint32_t(K) : 16u;  // second request of a fragment: rows 8..15, or the lane's next 16 bytes
    // block-scale rows: one per wave (its fragments sit inside one 128-row block), lane l keeps K block l (+64)
    const int srow = min(MODE == 0 ? t * 128 + wave * 32 : t * 256 + wave * 64, N - 16) >> 7;
    const float* sw0 = reinterpret_cast<const float*>(ws[0]) + size_t(srow) * KB;
    const float* sw1 = reinterpret_cast<const float*>(ws[1]) + size_t(srow) * KB;

    // token rows this thread stages
    const uint8_t* tsrc[CPT];
    int tdst[CPT];
#pragma unroll
    for (int i = 0; i < CPT; ++i) {
      const int q = min(tid + 256 * i, CHUNKS - 1);
      const int m = q >> 3, c = q & 7;
      const int pos = start + min(m, n - 1);
      const int row = MODE == 0 && p.perm ? load_global<int>(p.perm + pos) / p.top_k : pos;
      tsrc[i] = p.a_codes + size_t(row) * K + c * 16;
      tdst[i] = m * 128 + ((c ^ (m & 7)) << 4);
    }
    const bool stage_chunk = CHUNKS >= 256 || tid < CHUNKS;
    const float* ssrc;
    {
      const int pos = start + min(min(tid, TM - 1), n - 1);
      const int row = MODE == 0 && p.perm ? load_global<int>(p.perm + pos) / p.top_k : pos;
      ssrc = p.a_scales + size_t(row) * KB;
    }

    float acc[MF][4][4];
#pragma unroll
    for (int m = 0; m < MF; ++m)
#pragma unroll
      for (int f = 0; f < 4; ++f)
#pragma unroll
        for (int r = 0; r < 4; ++r) acc[m][f][r] = 0.0f;

    // prologue: weight fragments of the first P K blocks, token tile 0 into LDS, token tile 1 into registers.
    // Loads retire in issue order, so anything consumed early must be requested before anything consumed late: in
    // steady state an iteration first requests token tile kb+2 (written to LDS one iteration later) and then the
    // weight fragments of K block kb+P, so waiting for the tokens never forces the younger weight loads to land.
    u32x4 w[P][4][2];
#pragma unroll
    for (int s = 0; s < P; ++s) {
      const uint32_t kb = uint32_t(min(s, KB - 1));
#pragma unroll
      for (int f = 0; f < 4; ++f) {
        w[s][f][0] = load16(wrow[f] + kb * 128u);
        w[s][f][1] = load16(wrow[f] + kb * 128u + wsecond);
      }
    }
    u32x4 tv[CPT];
    float tsv;
    {
#pragma unroll
      for (int i = 0; i < CPT; ++i) {
        const u32x4 v = load16(tsrc[i]);
        if (stage_chunk) *reinterpret_cast<u32x4*>(&tile[0][tdst[i]]) = v;
      }
      if (tid < TM) *reinterpret_cast<float*>(&tile[0][TM * 128 + tid * 4]) = load_global<float>(ssrc);
      const uint32_t k1 = uint32_t(min(1, KB - 1));
#pragma unroll
      for (int i = 0; i < CPT; ++i) tv[i] = load16(tsrc[i] + k1 * 128u);
      tsv = load_global<float>(ssrc + k1);
    }
    __syncthreads();

    // LDS addresses of this lane's token fragment pieces (buffer 0)
    int tlo[MF], thi[MF], tsx[MF];
#pragma unroll
    for (int m = 0; m < MF; ++m) {
      const int trow = 16 * m + (lane & 15);
      const int q2 = (lane >> 4) * 2;
      tlo[m] = trow * 128 + (((q2) ^ (trow & 7)) << 4);
      thi[m] = trow * 128 + (((q2 + 1) ^ (trow & 7)) << 4);
      tsx[m] = TM * 128 + trow * 4;
    }

    for (int kb0 = 0; kb0 < KB; kb0 += 64) {
      // block scales of K blocks kb0 .. kb0+63, one per lane
      const int kl = min(kb0 + lane, KB - 1);
      const float swl0 = load_global<float>(sw0 + kl);
      const float swl1 = MODE == 0 ? load_global<float>(sw1 + kl) : 0.0f;
      const int kend = min(KB, kb0 + 64);
      for (int kbo = kb0; kbo < kend; kbo += P) {
#pragma unroll
        for (int s = 0; s < P; ++s) {
          const int kb = kbo + s;
          if (kb < kend) {
            const uint8_t* tb = tile[kb & 1];
            const float s0 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, swl0), kb - kb0));
            const float s1 = MODE == 0 ? __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, swl1), kb - kb0)) : s0;
            // every row fragment is computed, also the padding of a short group: straight-line code lets the matrix
            // core overlap with the scale fmas, and short groups are bandwidth-bound anyway
            u32x4 wt[4][2];  // the four fragments in operand order
            if constexpr (!TW) {
#pragma unroll
              for (int f = 0; f < 4; ++f) { wt[f][0] = w[s][f][0]; wt[f][1] = w[s][f][1]; }
            } else {
              uint8_t* wl = &wstage[wave][0][0];
#pragma unroll
              for (int f = 0; f < 4; ++f) {
                *reinterpret_cast<u32x4*>(wl + f * 2048 + wr_off) = w[s][f][0];
                *reinterpret_cast<u32x4*>(wl + f * 2048 + 1024 + wr_off) = w[s][f][1];
              }
              __builtin_amdgcn_wave_barrier();
#pragma unroll
              for (int f = 0; f < 4; ++f) {
                wt[f][0] = *reinterpret_cast<const u32x4*>(wl + f * 2048 + rd_lo);
                wt[f][1] = *reinterpret_cast<const u32x4*>(wl + f * 2048 + rd_hi);
              }
              __builtin_amdgcn_wave_barrier();
            }
            v4f pr[MF][4];
            float sc[MF][2];
#pragma unroll
            for (int m = 0; m < MF; ++m) {
              const u32x4 lo = *reinterpret_cast<const u32x4*>(tb + tlo[m]);
              const u32x4 hi = *reinterpret_cast<const u32x4*>(tb + thi[m]);
              const float sx = *reinterpret_cast<const float*>(tb + tsx[m]);
              const v8i tok = {int(lo[0]), int(lo[1]), int(lo[2]), int(lo[3]), int(hi[0]), int(hi[1]), int(hi[2]), int(hi[3])};
              sc[m][0] = __fmul_rn(s0, sx);
              sc[m][1] = __fmul_rn(s1, sx);
#pragma unroll
              for (int f = 0; f < 4; ++f) {
                const v8i wf = {int(wt[f][0][0]), int(wt[f][0][1]), int(wt[f][0][2]), int(wt[f][0][3]),
                                int(wt[f][1][0]), int(wt[f][1][1]), int(wt[f][1][2]), int(wt[f][1][3])};
                const v4f z = {0.0f, 0.0f, 0.0f, 0.0f};
                pr[m][f] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(wf, tok, z, 0, 0, 0, 0, 0, 0);
              }
            }
#pragma unroll
            for (int m = 0; m < MF; ++m)
#pragma unroll
              for (int f = 0; f < 4; ++f)
#pragma unroll
                for (int r = 0; r < 4; ++r) acc[m][f][r] = __fmaf_rn(pr[m][f][r], sc[m][(MODE == 0 && f >= 2) ? 1 : 0], acc[m][f][r]);
            // publish token tile kb+1 (requested one iteration ago)
#pragma unroll
            for (int i = 0; i < CPT; ++i)
              if (stage_chunk) *reinterpret_cast<u32x4*>(&tile[(kb & 1) ^ 1][tdst[i]]) = tv[i];
            if (tid < TM) *reinterpret_cast<float*>(&tile[(kb & 1) ^ 1][TM * 128 + tid * 4]) = tsv;
            __syncthreads();
            // request token tile kb+2, then K block kb+P of the weights into the slot just consumed
            {
              const uint32_t kn = uint32_t(min(kb + 2, KB - 1));
#pragma unroll
              for (int i = 0; i < CPT; ++i) tv[i] = load16(tsrc[i] + kn * 128u);
              tsv = load_global<float>(ssrc + kn);
              const uint32_t kw = uint32_t(min(kb + P, KB - 1));
#pragma unroll
              for (int f = 0; f < 4; ++f) {
                w[s][f][0] = load16(wrow[f] + kw * 128u);
                w[s][f][1] = load16(wrow[f] + kw * 128u + wsecond);
              }
            }
          }
        }
      }
    }

    // epilogue
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
                const uint32_t lo = swiglu_bf16_two_branch(bround(acc[m][f][2 * h]), bround(acc[m][f + 2][2 * h]), p.swiglu, p.limit);
                const uint32_t hi = swiglu_bf16_two_branch(bround(acc[m][f][2 * h + 1]), bround(acc[m][f + 2][2 * h + 1]), p.swiglu, p.limit);
                o[h] = lo | (hi << 16);
              }
              const u32x2 v = {o[0], o[1]};
              *reinterpret_cast<u32x2*>(p.out + size_t(pos) * N + col) = v;
            }
          }
        } else {
          const int a = (MODE == 1 && p.perm) ? load_global<int>(p.perm + pos) : pos;
          float rw = 1.0f;
          if (MODE == 1 && p.weights)
            rw = p.weights_f32 ? load_global<float>(reinterpret_cast<const float*>(p.weights) + a)
                               : bf16_to_f32(load_global<uint16_t>(reinterpret_cast<const uint16_t*>(p.weights) + a));
#pragma unroll
          for (int f = 0; f < 4; ++f) {
            const int col = col0[f] + sub;
            if (col0[f] + 16 <= N) {
              float v[4];
#pragma unroll
              for (int r = 0; r < 4; ++r) {
                if (MODE == 1 && p.weights)
                  v[r] = p.routed_weight == FFMOE_WEIGHT_AFTER_DOWN_BF16 ? __fmul_rn(bround(acc[m][f][r]), rw) : __fmul_rn(acc[m][f][r], rw);
                else
                  v[r] = acc[m][f][r];
              }
              const u32x2 o = {pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3])};
              *reinterpret_cast<u32x2*>(p.out + size_t(a) * N + col) = o;
            }
          }
          if (MODE == 1 && p.done && t == 0 && wave == 0 && lane < 16) p.done[a] = 1u;
        }
      }
    }
  }
}

}  // namespace ffmoe
