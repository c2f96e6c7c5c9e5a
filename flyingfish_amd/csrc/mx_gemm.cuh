// Grouped GEMM for the E8M0 block-32 formats on the MX matrix cores: E2M1 (or E4M3) weights with one E8M0 scale per 32
// columns against E4M3 activations with one E8M0 scale per 32 columns are exactly the operand form of
// v_mfma_scale_f32_16x16x128_f8f6f4 - a lane's 32 K elements are one scale block - so a K block of 128 columns is one
// instruction per (weight fragment, token fragment), the block scales are applied by the matrix core, and the sum over
// the whole contraction stays in its accumulator: no dequantization and no per-block VALU work at all.
//
// This is the cohort (prefill) form of the W4A8 / W8A8 contract of kernels/moe_ffn.cu:398-867 and
// src/backend/cuda/moe/w4a8.rs. The decode entry (e8m0_kernel.cuh) reproduces the contract's exact integer arithmetic
// bit for bit; the matrix core adds the 128 products of an instruction in its own FP32 tree, so this path is the
// tolerance-checked variant (same quantized operands, same roundings between the stages).
//
// Work model, unit list and token staging are those of k_w8a8_grouped (w8a8_gemm.cuh); the token tile carries 128 code
// bytes and the 4 scale bytes of the K block per row. Operand layout of the instruction, measured on the device with
// one-hot operands (the two element widths do NOT share it): with c = lane / 16,
//   * a 4-bit operand holds columns 32 c .. 32 c + 31 of the K block in its 16 bytes (low nibble = even column);
//   * an 8-bit operand holds columns 16 c .. 16 c + 15 in bytes 0-15 and columns 64 + 16 c .. 64 + 16 c + 15 in bytes 16-31;
//   * the scale of columns 32 b .. 32 b + 31 is taken from lane group b of the scale register, for both operands,
//     wherever the operand's data for those columns sit.
//
// MODE 0: gate/up -> BF16 -> clamped SwiGLU x routing weight (f32, before the down projection) -> act[pos, j]
// MODE 1: down -> contributions[assignment, d] = BF16, done = 1
// MODE 2: down of the shared expert -> y[row, d]
#pragma once
#include "w8a8_gemm.cuh"

namespace ffmoe {

struct MxParams {
  const uint8_t* a_codes;    // activation E4M3 codes [*, K]
  const uint8_t* a_scales;   // activation E8M0 scales [*, K / 32]
  const uint64_t* slots;     // [E, 6] expert table, or NULL: the four addresses below
  uint64_t w0_codes, w0_scales, w1_codes, w1_scales;  // MODE 0: gate, up; MODE 1/2: w0 only
  const GemmGroup* groups;   // NULL: rows split arithmetically into groups of TM
  const u32x2* units;
  const uint32_t* unit_total;
  uint32_t total_units;
  const int* perm;           // permuted position -> assignment index (NULL: identity)
  const float* weights;      // routing weights per assignment (MODE 0 with perm; NULL: 1)
  uint16_t* out;
  uint32_t* done;
  int rows_total;
  int K, N, top_k;
  float limit;
};

// PACKED 1: E2M1 codes [N, K / 2] (low nibble = even column), E8M0 scales [N, K / 32]
// PACKED 0: E4M3 codes [N, K], E8M0 scales [N / 32, K / 32]
// NW waves per block share one token tile (see k_w8a8_grouped): eight for 64-row groups of a cohort, one block per CU.
template <int MF, int MODE, int PACKED, int P, int NW = 4>
__global__ __launch_bounds__(64 * NW, NW == 4 ? 2 : 1) void k_mx_grouped(const MxParams p) {
  constexpr int TM = 16 * MF;
  constexpr int NT = 64 * NW;
  constexpr int CHUNKS = TM * 8;
  constexpr int CPT = (CHUNKS + NT - 1) / NT;
  constexpr int TILE = TM * 128 + TM * 4;  // codes + the K block's four scale bytes per row
  constexpr int WL = PACKED ? 1 : 2;        // 16-byte loads per lane, fragment and K block
  __shared__ __attribute__((aligned(16))) uint8_t tile[2][TILE];
  // E2M1 experts request their weights row-contiguously (4 lanes per 64-byte row segment, the four
  // scale bytes of the row as one word) and turn them into operand order through a wave-private LDS buffer, as
  // k_w16_grouped does: requested in operand order, every lane touches a line of its own for 16 bytes, and once more
  // for one scale byte. LDS operations of one wave execute in order, so no wait sits between the writes and the reads.
  constexpr bool TW = PACKED != 0;
  __shared__ __attribute__((aligned(16))) uint8_t wstage[TW ? NW : 1][TW ? 4 : 1][TW ? 1024 : 16];
  __shared__ uint32_t sstage[TW ? NW : 1][TW ? 4 : 1][TW ? 16 : 1];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = uni(tid >> 6);
  const int K = p.K, N = p.N, KB = K >> 7, SB = K >> 5;
  const int wr_off = (lane >> 2) * 64 + (((lane & 3) ^ ((lane >> 4) & 3)) << 4);
  const int rd_off = (lane & 15) * 64 + (((lane >> 4) ^ ((lane >> 2) & 3)) << 4);
  const uint32_t total = p.unit_total ? uint32_t(uni(int(load_global<uint32_t>(p.unit_total)))) : p.total_units;
  const int ntiles = (N + gemm_tile_cols<MODE, NW>() - 1) / gemm_tile_cols<MODE, NW>();
  const int q4 = lane >> 4;  // this lane's scale block inside a K block

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
    int col0[4];
    const uint8_t* wrow[4];   // this lane's codes of K block 0
    const uint8_t* srow[4];   // this lane's scale byte of K block 0
#pragma unroll
    for (int f = 0; f < 4; ++f) {
      col0[f] = MODE == 0 ? t * (32 * NW) + wave * 32 + (f & 1) * 16 : t * (64 * NW) + wave * 64 + f * 16;
      const int which = MODE == 0 ? f >> 1 : 0;
      if (TW) {  // row lane / 4 of the fragment, 16-byte piece lane % 4; the row's scale word
        const int row = min(col0[f], N - 16) + (lane >> 2);
        wrow[f] = reinterpret_cast<const uint8_t*>(wc[which]) + size_t(row) * (K >> 1) + (lane & 3) * 16;
        srow[f] = reinterpret_cast<const uint8_t*>(ws[which]) + size_t(row) * SB;
      } else {
        const int row = min(col0[f], N - 16) + (lane & 15);
        wrow[f] = reinterpret_cast<const uint8_t*>(wc[which]) + (PACKED ? size_t(row) * (K >> 1) + q4 * 16 : size_t(row) * K + q4 * 16);
        srow[f] = reinterpret_cast<const uint8_t*>(ws[which]) + size_t(PACKED ? row : row >> 5) * SB + q4;
      }
    }

    const uint8_t* tsrc[CPT];
    int tdst[CPT];
#pragma unroll
    for (int i = 0; i < CPT; ++i) {
      const int q = min(tid + NT * i, CHUNKS - 1);
      const int m = q >> 3, c = q & 7;
      const int pos = start + min(m, n - 1);
      const int row = MODE == 0 && p.perm ? load_global<int>(p.perm + pos) / p.top_k : pos;
      tsrc[i] = p.a_codes + size_t(row) * K + c * 16;
      tdst[i] = m * 128 + ((c ^ (m & 7)) << 4);
    }
    const bool stage_chunk = CHUNKS >= NT || tid < CHUNKS;
    const uint8_t* ssrc;
    {
      const int pos = start + min(min(tid, TM - 1), n - 1);
      const int row = MODE == 0 && p.perm ? load_global<int>(p.perm + pos) / p.top_k : pos;
      ssrc = p.a_scales + size_t(row) * SB;
    }

    v4f acc[MF][4];
#pragma unroll
    for (int m = 0; m < MF; ++m)
#pragma unroll
      for (int f = 0; f < 4; ++f) acc[m][f] = v4f{0.0f, 0.0f, 0.0f, 0.0f};

    u32x4 w[P][4][WL];
    uint32_t wsc[P][4];
#pragma unroll
    for (int s = 0; s < P; ++s) {
      const uint32_t kb = uint32_t(min(s, KB - 1));
#pragma unroll
      for (int f = 0; f < 4; ++f) {
#pragma unroll
        for (int l = 0; l < WL; ++l) w[s][f][l] = load16(wrow[f] + kb * (PACKED ? 64u : 128u) + 64u * l);
        wsc[s][f] = TW ? load_global<uint32_t>(srow[f] + kb * 4u) : uint32_t(load_global<uint8_t>(srow[f] + kb * 4u));
      }
    }
    u32x4 tv[CPT];
    uint32_t tsv;
    {
#pragma unroll
      for (int i = 0; i < CPT; ++i) {
        const u32x4 v = load16(tsrc[i]);
        if (stage_chunk) *reinterpret_cast<u32x4*>(&tile[0][tdst[i]]) = v;
      }
      if (tid < TM) *reinterpret_cast<uint32_t*>(&tile[0][TM * 128 + tid * 4]) = load_global<uint32_t>(ssrc);
      const uint32_t k1 = uint32_t(min(1, KB - 1));
#pragma unroll
      for (int i = 0; i < CPT; ++i) tv[i] = load16(tsrc[i] + k1 * 128u);
      tsv = load_global<uint32_t>(ssrc + k1 * 4u);
    }
    __syncthreads();

    int tlo[MF], thi[MF], tsx[MF];
#pragma unroll
    for (int m = 0; m < MF; ++m) {
      const int trow = 16 * m + (lane & 15);
      tlo[m] = trow * 128 + (((q4) ^ (trow & 7)) << 4);      // columns 16 c .. 16 c + 15
      thi[m] = trow * 128 + (((q4 + 4) ^ (trow & 7)) << 4);  // columns 64 + 16 c .. 64 + 16 c + 15
      tsx[m] = TM * 128 + trow * 4;
    }

    for (int kbo = 0; kbo < KB; kbo += P) {
#pragma unroll
      for (int s = 0; s < P; ++s) {
        const int kb = kbo + s;
        if (kb < KB) {
          const uint8_t* tb = tile[kb & 1];
          u32x4 wt[4];       // first 16 bytes of the four fragments in operand order
          uint32_t st[4];    // this lane's weight scale byte
#pragma unroll
          for (int f = 0; f < 4; ++f) { wt[f] = w[s][f][0]; st[f] = wsc[s][f]; }
          if constexpr (TW) {
            uint8_t* wl = &wstage[wave][0][0];
            uint32_t* sl = &sstage[wave][0][0];
#pragma unroll
            for (int f = 0; f < 4; ++f) {
              *reinterpret_cast<u32x4*>(wl + f * 1024 + wr_off) = w[s][f][0];
              if ((lane & 3) == 0) sl[f * 16 + (lane >> 2)] = wsc[s][f];
            }
            __builtin_amdgcn_wave_barrier();
#pragma unroll
            for (int f = 0; f < 4; ++f) {
              wt[f] = *reinterpret_cast<const u32x4*>(wl + f * 1024 + rd_off);
              st[f] = (sl[f * 16 + (lane & 15)] >> (8 * q4)) & 0xffu;
            }
            __builtin_amdgcn_wave_barrier();
          }
#pragma unroll
          for (int m = 0; m < MF; ++m) {
            const u32x4 lo = *reinterpret_cast<const u32x4*>(tb + tlo[m]);
            const u32x4 hi = *reinterpret_cast<const u32x4*>(tb + thi[m]);
            const uint32_t sx4 = *reinterpret_cast<const uint32_t*>(tb + tsx[m]);
            const int sx = int((sx4 >> (8 * q4)) & 0xffu);  // the scale of this lane's 32 columns
            const v8i tok = {int(lo[0]), int(lo[1]), int(lo[2]), int(lo[3]), int(hi[0]), int(hi[1]), int(hi[2]), int(hi[3])};
#pragma unroll
            for (int f = 0; f < 4; ++f) {
              v8i wf;
              if (PACKED) wf = v8i{int(wt[f][0]), int(wt[f][1]), int(wt[f][2]), int(wt[f][3]), 0, 0, 0, 0};
              else wf = v8i{int(wt[f][0]), int(wt[f][1]), int(wt[f][2]), int(wt[f][3]),
                            int(w[s][f][WL - 1][0]), int(w[s][f][WL - 1][1]), int(w[s][f][WL - 1][2]), int(w[s][f][WL - 1][3])};
              acc[m][f] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(wf, tok, acc[m][f], PACKED ? 4 : 0, 0, 0, int(st[f]), 0, sx);
            }
          }
#pragma unroll
          for (int i = 0; i < CPT; ++i)
            if (stage_chunk) *reinterpret_cast<u32x4*>(&tile[(kb & 1) ^ 1][tdst[i]]) = tv[i];
          if (tid < TM) *reinterpret_cast<uint32_t*>(&tile[(kb & 1) ^ 1][TM * 128 + tid * 4]) = tsv;
          __syncthreads();
          {
            const uint32_t kn = uint32_t(min(kb + 2, KB - 1));
#pragma unroll
            for (int i = 0; i < CPT; ++i) tv[i] = load16(tsrc[i] + kn * 128u);
            tsv = load_global<uint32_t>(ssrc + kn * 4u);
            const uint32_t kw = uint32_t(min(kb + P, KB - 1));
#pragma unroll
            for (int f = 0; f < 4; ++f) {
#pragma unroll
              for (int l = 0; l < WL; ++l) w[s][f][l] = load16(wrow[f] + kw * (PACKED ? 64u : 128u) + 64u * l);
              wsc[s][f] = TW ? load_global<uint32_t>(srow[f] + kw * 4u) : uint32_t(load_global<uint8_t>(srow[f] + kw * 4u));
            }
          }
        }
      }
    }

    const int tk = lane & 15, sub = q4 * 4;
#pragma unroll
    for (int m = 0; m < MF; ++m) {
      const int token = 16 * m + tk;
      if (token < n) {
        const int pos = start + token;
        if (MODE == 0) {
          float wk = 1.0f;
          if (p.perm && p.weights) wk = load_global<float>(p.weights + load_global<int>(p.perm + pos));
#pragma unroll
          for (int f = 0; f < 2; ++f) {
            const int col = col0[f] + sub;
            if (col0[f] + 16 <= N) {
              uint32_t o[4];
#pragma unroll
              for (int r = 0; r < 4; ++r) {
                // the contract's epilogue (kernels/moe_ffn.cu:601-700): BF16 dots, clamp, SiLU by division, x up x weight
                const float g = fminf(bround(acc[m][f][r]), p.limit);
                const float uu = fmaxf(fminf(bround(acc[m][f + 2][r]), p.limit), -p.limit);
                const float silu = __fdiv_rn(g, __fadd_rn(1.0f, det_expf(-g)));
                o[r] = f32_to_bf16(__fmul_rn(__fmul_rn(silu, uu), wk));
              }
              const u32x2 v = {o[0] | (o[1] << 16), o[2] | (o[3] << 16)};
              *reinterpret_cast<u32x2*>(p.out + size_t(pos) * N + col) = v;
            }
          }
        } else {
          const int a = (MODE == 1 && p.perm) ? load_global<int>(p.perm + pos) : pos;
#pragma unroll
          for (int f = 0; f < 4; ++f) {
            const int col = col0[f] + sub;
            if (col0[f] + 16 <= N) {
              const u32x2 o = {pack_bf16x2(acc[m][f][0], acc[m][f][1]), pack_bf16x2(acc[m][f][2], acc[m][f][3])};
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
