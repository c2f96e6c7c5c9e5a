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
  const float* global_scales;  // NVFP4 experts: [E, 3] f32 (gate, up, down), with slots
  float w0_global, w1_global;  // NVFP4 experts without a table: the global scales of w0 / w1
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

// output columns per unit: every wave owns 32 activation columns (gate and up rows) or 64 down columns
template <int MODE, int NW = 4>
__device__ __forceinline__ constexpr int gemm_tile_cols() { return (MODE == 0 ? 32 : 64) * NW; }

// NW waves per block share one token tile in LDS. Blocks drift apart by more than a line lives in an XCD's L2 under the
// weight stream, so a token tile that two blocks need is fetched twice (the fetch counters show every token read of a
// cohort as an L2 miss, whatever the unit order); with NW = 8 one block per CU covers twice the columns per token tile
// and the token traffic halves, at the same number of waves per CU as two blocks of four.
//
// NV: the weights are NVFP4 (two E2M1 codes per byte, one E4M3 scale per 16 columns, an f32 per matrix). A fragment's
// 16 rows x 128 columns are requested as 64 bytes of codes per row (four lanes) and the row's eight scale bytes, turned
// into E4M3 on the way into the wave's transposition buffer - code value x scale / 8, rounded to nearest even, which
// 6 x 448 / 8 = 336 keeps inside E4M3 - and from there on the kernel is the block-FP8 one with 8 x global as every
// block's scale. That rounding is the arithmetic of this mode (a weight rounded twice, where the BF16-activation paths
// round it once): its CPU restatement derives the same E4M3 codes and runs the block-FP8 W8A8 oracle on them.
template <int MF, int MODE, int P, int NW = 4, bool NV = false>
__global__ __launch_bounds__(64 * NW, (NW == 4 && MF <= 4) ? 2 : 1) void k_w8a8_grouped(const GemmParams p) {
  constexpr int TM = 16 * MF;
  constexpr int NT = 64 * NW;                       // threads per block
  constexpr int CHUNKS = TM * 8;                    // 16-byte token chunks per K block
  constexpr int CPT = (CHUNKS + NT - 1) / NT;       // chunks a thread moves per K block
  constexpr int TILE = TM * 128 + TM * 4;           // codes + scales
  constexpr int LPS = CPT + 1 + 8;                  // loads a thread issues per stage: token chunks, token scale, weights
  static_assert(CPT == 1 || CPT == 2 || CPT == 4, "token chunks per thread");
  __shared__ __attribute__((aligned(16))) uint8_t tile[2][TILE];
  // Weight fragments are requested row-contiguously (8 lanes per 128-byte row segment, 8 rows per instruction) and
  // turned into the operand's lane order (row lane % 16, bytes 32 (lane / 16) .. + 31) through this wave-private
  // buffer: requested in operand order, the 16 consecutive lanes of a quarter wave touch 16 different lines for 16
  // bytes each and the vector L1 spends one look-up per 16 bytes (929 -> 1295 TFLOP/s in the cache-resident case when
  // only the addresses are changed). Pieces are XOR-swizzled by the row; LDS operations of one wave execute in order,
  // so no wait sits between the writes and the reads.
  // Short groups (MF < 4) are bound by HBM, not by the L1: they keep the direct requests and skip the LDS round trip.
  constexpr bool TW = MF >= 4;
  static_assert(!TW || P == 2, "the hand-counted waits of the long-group path assume two weight stages");
  static_assert(!NV || MF == 4, "NVFP4 weights take the 64-row path, whose weights pass through LDS");
  __shared__ __attribute__((aligned(16))) uint8_t wstage[TW ? NW : 1][TW ? 4 : 1][TW ? 2048 : 16];  // [wave][fragment][16 rows x 128 B]
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = uni(tid >> 6);
  const int K = p.K, N = p.N, KB = K >> 7;
  const int wr_off = (lane >> 3) * 128 + (((lane & 7) ^ ((lane >> 3) & 7)) << 4);                 // rows 0..7; rows 8..15 at + 1024
  const int rd_lo = (lane & 15) * 128 + (((2 * (lane >> 4)) ^ (lane & 7)) << 4);
  const int rd_hi = (lane & 15) * 128 + (((2 * (lane >> 4) + 1) ^ (lane & 7)) << 4);
  const uint32_t total = p.unit_total ? uint32_t(uni(int(load_global<uint32_t>(p.unit_total)))) : p.total_units;
  const int ntiles = (N + gemm_tile_cols<MODE, NW>() - 1) / gemm_tile_cols<MODE, NW>();

  // Blocks are dealt to the 8 XCDs round-robin, and each XCD has its own L2. The unit list is cut into 8 contiguous
  // spans, one per XCD, and the blocks of an XCD walk their span side by side, so the row groups of one (expert,
  // column tile) meet in the same L2 and its weights leave HBM once.
  const uint32_t xcd = blockIdx.x & 7u, slot = blockIdx.x >> 3, per_xcd = gridDim.x >> 3;
  const uint32_t span = (total + 7u) >> 3;
  const uint32_t span_end = min(total, (xcd + 1u) * span);
  // What a unit is and where its expert's matrices are: unit list -> group record -> slot table, three loads that depend on
  // each other. They are wave-uniform and go through the scalar cache, and the next unit's chain is walked while this unit's
  // first weights are on their way (one block of this kernel fills a CU, so nothing else would hide the three round trips
  // in front of every unit's first weight request).
  struct UnitDesc { int expert, start, n, t; uint64_t wc[2], ws[2]; float nvg[2]; };
  auto fetch_unit = [&](uint32_t u) {
    UnitDesc d;
    if (p.groups) {
      const u32x2 un = load_uniform<u32x2>(p.units + u);
      const int g = int(un.x);
      d.t = int(un.y);
      const int* gd = reinterpret_cast<const int*>(p.groups + g);
      d.expert = load_uniform<int>(gd);
      d.start = load_uniform<int>(gd + 1);
      d.n = load_uniform<int>(gd + 2);
    } else {
      const int g = int(u) / ntiles;
      d.t = int(u) - g * ntiles;
      d.expert = 0;
      d.start = g * TM;
      d.n = min(TM, p.rows_total - d.start);
    }
    if (p.slots) {
      const uint64_t* sl = p.slots + size_t(d.expert) * 6;
      if (MODE == 0) {
        d.wc[0] = load_uniform<uint64_t>(sl + 0); d.ws[0] = load_uniform<uint64_t>(sl + 1);
        d.wc[1] = load_uniform<uint64_t>(sl + 2); d.ws[1] = load_uniform<uint64_t>(sl + 3);
      } else {
        d.wc[0] = d.wc[1] = load_uniform<uint64_t>(sl + 4); d.ws[0] = d.ws[1] = load_uniform<uint64_t>(sl + 5);
      }
    } else {
      d.wc[0] = p.w0_codes; d.ws[0] = p.w0_scales;
      d.wc[1] = MODE == 0 ? p.w1_codes : p.w0_codes; d.ws[1] = MODE == 0 ? p.w1_scales : p.w0_scales;
    }
    d.nvg[0] = d.nvg[1] = 1.0f;  // NV: 8 x the matrix's global scale stands in for every block scale
    if constexpr (NV) {
      if (p.slots) {
        const float* gl = p.global_scales + size_t(d.expert) * 3;
        d.nvg[0] = load_uniform<float>(gl + (MODE == 0 ? 0 : 2));
        d.nvg[1] = MODE == 0 ? load_uniform<float>(gl + 1) : d.nvg[0];
      } else {
        d.nvg[0] = p.w0_global; d.nvg[1] = MODE == 0 ? p.w1_global : p.w0_global;
      }
      d.nvg[0] = __fmul_rn(d.nvg[0], 8.0f); d.nvg[1] = __fmul_rn(d.nvg[1], 8.0f);
    }
    return d;
  };
  constexpr bool AHEAD = !NV;  // (next to the NVFP4 conversion the chain walked ahead costs scalar registers it does not have: measured slower)
  const uint32_t u_first = xcd * span + slot;
  UnitDesc next_unit = {};
  if (AHEAD && u_first < span_end) next_unit = fetch_unit(u_first);
  for (uint32_t u = u_first; u < span_end; u += per_xcd) {
    if (!AHEAD) next_unit = fetch_unit(u);
    const UnitDesc unit = next_unit;
    const int expert = unit.expert, start = unit.start, n = unit.n, t = unit.t;
    (void)expert;
    const uint64_t wc[2] = {unit.wc[0], unit.wc[1]}, ws[2] = {unit.ws[0], unit.ws[1]};
    const float nvg[2] = {unit.nvg[0], unit.nvg[1]};
    // first output column of fragment f; fragments past N are clamped onto the last 16 rows and dropped at the store
    int col0[4];
    // weight addresses: a wave-uniform base per fragment (scalar registers) and one byte offset per lane
    uint64_t wfrag[4];
#pragma unroll
    for (int f = 0; f < 4; ++f) {
      col0[f] = MODE == 0 ? t * (32 * NW) + wave * 32 + (f & 1) * 16 : t * (64 * NW) + wave * 64 + f * 16;
      const int base = min(col0[f], N - 16);
      const uint64_t codes = MODE == 0 ? wc[f >> 1] : wc[0];
      wfrag[f] = uni64(codes + uint64_t(base) * uint64_t(NV ? K >> 1 : K));
    }
    // NV: the scale bytes of the fragment's rows, [N, K / 16]
    uint64_t sfrag[4] = {0, 0, 0, 0};
    if constexpr (NV) {
#pragma unroll
      for (int f = 0; f < 4; ++f) sfrag[f] = uni64((MODE == 0 ? ws[f >> 1] : ws[0]) + uint64_t(min(col0[f], N - 16)) * uint64_t(K >> 4));
    }
    // long groups: 8 lanes per 128-byte row segment, rows 0..7 of the fragment (rows 8..15 with the second request);
    // short groups: operand order, 32 bytes of row lane % 16 as two requests
    // NV: four lanes per row of 64 code bytes, 16 rows per request; a lane's two scale bytes sit in the dword its pair shares
    const uint32_t woff0 = NV ? uint32_t(lane >> 2) * uint32_t(K >> 1) + uint32_t(lane & 3) * 16u
                              : TW ? uint32_t(lane >> 3) * uint32_t(K) + uint32_t(lane & 7) * 16u : uint32_t(lane & 15) * uint32_t(K) + uint32_t(lane >> 4) * 32u;
    const uint32_t woff1 = NV ? uint32_t(lane >> 2) * uint32_t(K >> 4) + uint32_t((lane & 3) >> 1) * 4u : woff0 + (TW ? 8u * uint32_t(K) : 16u);
    const int nv_wr = ((lane >> 2) & 7) * 128 + (lane >> 5) * 1024;  // NV: this lane's row of the fragment in the buffer
    const int nv_key = (lane >> 2) & 7, nv_piece = (lane & 3) * 2;
    // block-scale rows: one per wave (its fragments sit inside one 128-row block), lane l keeps K block l (+64)
    const int srow = min(MODE == 0 ? t * (32 * NW) + wave * 32 : t * (64 * NW) + wave * 64, N - 16) >> 7;
    const float* sw0 = reinterpret_cast<const float*>(NV ? uint64_t(p.a_scales) : ws[0]) + (NV ? 0 : size_t(srow) * KB);  // NV: any readable floats, never used
    const float* sw1 = reinterpret_cast<const float*>(NV ? uint64_t(p.a_scales) : ws[1]) + (NV ? 0 : size_t(srow) * KB);

    // token rows this thread stages
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

    // block scales of K blocks 0 .. 63, one per lane. They are requested before everything else and made to land
    // (landed()) outside the K loop: a value still counted as in flight when the loop is entered makes the compiler
    // wait for it in every iteration, and since loads retire in order that wait drains the whole prefetch queue.
    float swn0 = load_global<float>(sw0 + min(lane, KB - 1));
    float swn1 = MODE == 0 ? load_global<float>(sw1 + min(lane, KB - 1)) : 0.0f;

    // Loads inside the K loop are issued and awaited by hand (load16_async / wait_loads): the compiler's own waits are
    // placed for the path with the fewest loads in flight and drain the queue in every iteration. Per stage a thread
    // issues LPS loads in a fixed order, so "how many younger loads may still be in flight" is a constant:
    //   64-row groups and longer (TW), stage kb with register slot s = kb % 2: the operand-order fragments of K block
    //     kb are read from the wave's transposition buffer; then, spread over the matrix instructions of the row
    //     fragments (an issue that finds the memory or LDS pipeline full stalls under matrix work of the same
    //     wave): token tile kb+1 (published at the end of this stage), the weights of K block kb+2 into slot s,
    //     and slot s^1 (K block kb+1, requested one stage ago) written row-contiguously into the transposition
    //     buffer for the next stage;
    //   shorter groups: after the barrier token tile kb+2, then the weights of K block kb+P.
    // Either way the token tile published in a stage has exactly the eight weight loads issued after it behind it.
    constexpr int WAIT_W = (P - 1) * LPS;  // short groups: younger loads behind a stage's weights
    // prologue: weight fragments of the first P K blocks, token tile 0 into LDS, everything landed, then token tile 1
    // (and for short groups the last weight stage once more, so that tile 1 too has eight loads behind it).
    u32x4 w[P][4][2];
    float wsc[P][4];  // NV: the dword with the lane's scale bytes (w[..][1] stays unused)
#define FF_REQUEST_WEIGHTS(s_, kb_, f_)                                   \
  do {                                                                     \
    if constexpr (NV) {                                                    \
      load16_async(w[s_][f_][0], wfrag[f_] + (kb_) * 64u, woff0);          \
      load4_async(wsc[s_][f_], sfrag[f_] + (kb_) * 8u, woff1);             \
    } else {                                                               \
      load16_async(w[s_][f_][0], wfrag[f_] + (kb_) * 128u, woff0);         \
      load16_async(w[s_][f_][1], wfrag[f_] + (kb_) * 128u, woff1);         \
    }                                                                      \
  } while (0)
#define FF_DRAIN_WEIGHTS()                                                                                                  \
  _Pragma("unroll") for (int s_ = 0; s_ < P; ++s_) {                                                                        \
    if constexpr (NV) wait_loads<0>(w[s_][0][0], w[s_][1][0], w[s_][2][0], w[s_][3][0], wsc[s_][0], wsc[s_][1], wsc[s_][2], wsc[s_][3]); \
    else wait_loads<0>(w[s_][0][0], w[s_][0][1], w[s_][1][0], w[s_][1][1], w[s_][2][0], w[s_][2][1], w[s_][3][0], w[s_][3][1]); \
  }
    // NV: a landed fragment piece (32 codes and their two scale bytes) as 32 E4M3 bytes into the transposition buffer
    auto nv_store = [&](uint8_t* frag_base, const u32x4& codes, float scale_word) {
      const uint32_t sb = __float_as_uint(scale_word) >> (16 * (lane & 1));
      const f32x2 sc = e4m3x2_to_f32<false>(sb);
      const float s2[2] = {__fmul_rn(sc.x, 0.125f), __fmul_rn(sc.y, 0.125f)};
      uint32_t o[8];
#pragma unroll
      for (int d = 0; d < 4; ++d) {
        const float sg = s2[d >> 1];
        int lo = 0, hi = 0;
        const f32x2 v0 = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(codes[d], 1.0f, 0), v1 = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(codes[d], 1.0f, 1);
        const f32x2 v2 = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(codes[d], 1.0f, 2), v3 = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(codes[d], 1.0f, 3);
        lo = __builtin_amdgcn_cvt_pk_fp8_f32(__fmul_rn(v0.x, sg), __fmul_rn(v0.y, sg), lo, false);
        lo = __builtin_amdgcn_cvt_pk_fp8_f32(__fmul_rn(v1.x, sg), __fmul_rn(v1.y, sg), lo, true);
        hi = __builtin_amdgcn_cvt_pk_fp8_f32(__fmul_rn(v2.x, sg), __fmul_rn(v2.y, sg), hi, false);
        hi = __builtin_amdgcn_cvt_pk_fp8_f32(__fmul_rn(v3.x, sg), __fmul_rn(v3.y, sg), hi, true);
        o[2 * d] = uint32_t(lo); o[2 * d + 1] = uint32_t(hi);
      }
      *reinterpret_cast<u32x4*>(frag_base + nv_wr + ((nv_piece ^ nv_key) << 4)) = u32x4{o[0], o[1], o[2], o[3]};
      *reinterpret_cast<u32x4*>(frag_base + nv_wr + (((nv_piece + 1) ^ nv_key) << 4)) = u32x4{o[4], o[5], o[6], o[7]};
    };
#pragma unroll
    for (int s = 0; s < P; ++s) {
      const uint32_t kb = uint32_t(min(s, KB - 1));
#pragma unroll
      for (int f = 0; f < 4; ++f) FF_REQUEST_WEIGHTS(s, kb, f);
    }
    u32x4 tv[CPT];
    float tsv;
#define FF_WAIT_TOKENS(n_)                                                    \
  do {                                                                         \
    if constexpr (CPT == 1) wait_loads<n_>(tv[0], tsv);                        \
    else if constexpr (CPT == 2) wait_loads<n_>(tv[0], tv[1], tsv);            \
    else wait_loads<n_>(tv[0], tv[1], tv[2], tv[3], tsv);                      \
  } while (0)
    {
#pragma unroll
      for (int i = 0; i < CPT; ++i) {
        const u32x4 v = load16(tsrc[i]);
        if (stage_chunk) *reinterpret_cast<u32x4*>(&tile[0][tdst[i]]) = v;
      }
      if (tid < TM) *reinterpret_cast<float*>(&tile[0][TM * 128 + tid * 4]) = load_global<float>(ssrc);
      // the next unit's descriptor chain, under the round trip of this unit's first weights
      if (AHEAD && u + per_xcd < span_end) next_unit = fetch_unit(u + per_xcd);
      FF_DRAIN_WEIGHTS();
      if constexpr (TW) {
        // K block 0 goes into the wave's transposition buffer; stage 0 requests token tile 1 itself
        uint8_t* wl = &wstage[wave][0][0];
#pragma unroll
        for (int f = 0; f < 4; ++f) {
          if constexpr (NV) {
            nv_store(wl + f * 2048, w[0][f][0], wsc[0][f]);
          } else {
            *reinterpret_cast<u32x4*>(wl + f * 2048 + wr_off) = w[0][f][0];
            *reinterpret_cast<u32x4*>(wl + f * 2048 + 1024 + wr_off) = w[0][f][1];
          }
        }
#pragma unroll
        for (int i = 0; i < CPT; ++i) tv[i] = u32x4{0u, 0u, 0u, 0u};
        tsv = 0.0f;
      } else {
        const uint32_t k1 = uint32_t(min(1, KB - 1));
#pragma unroll
        for (int i = 0; i < CPT; ++i) load16_async(tv[i], tsrc[i] + k1 * 128u);
        load4_async(tsv, ssrc + k1);
        const uint32_t kb = uint32_t(min(P - 1, KB - 1));
#pragma unroll
        for (int f = 0; f < 4; ++f) FF_REQUEST_WEIGHTS(P - 1, kb, f);
      }
    }
    __syncthreads();

    // LDS addresses of this lane's token fragment pieces (buffer 0)
    // Row fragment m sits 2048 bytes (scales: 64 bytes) behind fragment 0 and keeps its swizzle key (16 m leaves the low
    // row bits alone), and K block kb sits in buffer kb % 2 = stage % 2 (P is even and the loop advances by P): every
    // token address is one of three lane values plus a compile-time constant.
    static_assert(P % 2 == 0, "token buffer = stage parity");
    const int trow0 = lane & 15, q2 = (lane >> 4) * 2;
    const int tlo0 = trow0 * 128 + (((q2) ^ (trow0 & 7)) << 4);
    const int thi0 = trow0 * 128 + (((q2 + 1) ^ (trow0 & 7)) << 4);
    const int tsx0 = TM * 128 + trow0 * 4;

    // 64-row groups keep LDS latency off the matrix core's path: the operand-order weight fragments of a stage are read at
    // the end of the stage before (behind the token publication and the barrier), and the token fragment of row fragment
    // m + 1 is read before the matrix instructions of fragment m are issued.
    constexpr bool PF = TW && MF == 4;
    u32x4 wt[4][2];  // the four weight fragments in operand order
    if constexpr (PF) {
      const uint8_t* wl0 = &wstage[wave][0][0];
#pragma unroll
      for (int f = 0; f < 4; ++f) {
        wt[f][0] = *reinterpret_cast<const u32x4*>(wl0 + f * 2048 + rd_lo);
        wt[f][1] = *reinterpret_cast<const u32x4*>(wl0 + f * 2048 + rd_hi);
      }
      __builtin_amdgcn_wave_barrier();
    }
    for (int kb0 = 0; kb0 < KB; kb0 += 64) {
      // block scales of K blocks kb0 .. kb0+63, one per lane; the next 64 are requested right away
      const float swl0 = NV ? nvg[0] : landed(swn0);
      const float swl1 = NV ? nvg[1] : (MODE == 0 ? landed(swn1) : 0.0f);
      if (kb0 + 64 < KB) {
        const int kl = min(kb0 + 64 + lane, KB - 1);
        swn0 = load_global<float>(sw0 + kl);
        if (MODE == 0) swn1 = load_global<float>(sw1 + kl);
      }
      const int kend = min(KB, kb0 + 64);
      for (int kbo = kb0; kbo < kend; kbo += P) {
#pragma unroll
        for (int s = 0; s < P; ++s) {
          const int kb = kbo + s;
          if (kb < kend) {
            const uint8_t* tb = tile[s & 1];
            const float s0 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, swl0), kb - kb0));
            const float s1 = MODE == 0 ? __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, swl1), kb - kb0)) : s0;
            // every row fragment is computed, also the padding of a short group: straight-line code lets the matrix
            // core overlap with the scale fmas, and short groups are bandwidth-bound anyway
            uint8_t* wl = &wstage[TW ? wave : 0][0][0];
            if constexpr (!TW) {
              wait_loads<WAIT_W>(w[s][0][0], w[s][0][1], w[s][1][0], w[s][1][1], w[s][2][0], w[s][2][1], w[s][3][0], w[s][3][1]);
#pragma unroll
              for (int f = 0; f < 4; ++f) { wt[f][0] = w[s][f][0]; wt[f][1] = w[s][f][1]; }
            } else if constexpr (!PF) {
#pragma unroll
              for (int f = 0; f < 4; ++f) {
                wt[f][0] = *reinterpret_cast<const u32x4*>(wl + f * 2048 + rd_lo);
                wt[f][1] = *reinterpret_cast<const u32x4*>(wl + f * 2048 + rd_hi);
              }
              __builtin_amdgcn_wave_barrier();
            }
            // Row fragment m's products are folded into the totals while fragment m + 1 is in the matrix core, so two
            // fragments' worth of product registers are live instead of MF (the scheduling fences keep that order).
            v4f pr[2][4];
            float sc[2][2];
            u32x4 tfl[2], tfh[2];  // token fragment pieces, two row fragments in rotation
            float tfs[2];
            if constexpr (PF) {
              tfl[0] = *reinterpret_cast<const u32x4*>(tb + tlo0);
              tfh[0] = *reinterpret_cast<const u32x4*>(tb + thi0);
              tfs[0] = *reinterpret_cast<const float*>(tb + tsx0);
            }
#pragma unroll
            for (int m = 0; m <= MF; ++m) {
              if (m < MF) {
                constexpr int ahead = PF ? 1 : 0;
                if (!PF || m + 1 < MF) {
                  tfl[(m + ahead) & 1] = *reinterpret_cast<const u32x4*>(tb + tlo0 + (m + ahead) * 2048);
                  tfh[(m + ahead) & 1] = *reinterpret_cast<const u32x4*>(tb + thi0 + (m + ahead) * 2048);
                  tfs[(m + ahead) & 1] = *reinterpret_cast<const float*>(tb + tsx0 + (m + ahead) * 64);
                }
                const u32x4 lo = tfl[m & 1], hi = tfh[m & 1];
                const float sx = tfs[m & 1];
                const v8i tok = {int(lo[0]), int(lo[1]), int(lo[2]), int(lo[3]), int(hi[0]), int(hi[1]), int(hi[2]), int(hi[3])};
                sc[m & 1][0] = __fmul_rn(s0, sx);
                sc[m & 1][1] = __fmul_rn(s1, sx);
#pragma unroll
                for (int f = 0; f < 4; ++f) {
                  const v8i wf = {int(wt[f][0][0]), int(wt[f][0][1]), int(wt[f][0][2]), int(wt[f][0][3]),
                                  int(wt[f][1][0]), int(wt[f][1][1]), int(wt[f][1][2]), int(wt[f][1][3])};
                  const v4f z = {0.0f, 0.0f, 0.0f, 0.0f};
                  pr[m & 1][f] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(wf, tok, z, 0, 0, 0, 0, 0, 0);
                }
                if constexpr (TW) {
                  const int o = s ^ 1;
                  if (m == 0) {  // token tile kb+1
                    const uint32_t kn = uint32_t(min(kb + 1, KB - 1));
#pragma unroll
                    for (int i = 0; i < CPT; ++i) load16_async(tv[i], tsrc[i] + kn * 128u);
                    load4_async(tsv, ssrc + kn);
                  }
                  // slot s went into the transposition buffer one stage ago: request K block kb+2 into it. A piece
                  // of slot s^1 (K block kb+1) has the rest of its own stage's weight loads, this stage's token
                  // loads and this stage's weight loads so far behind it: CPT + 1 + 8 whichever piece it is
                  const uint32_t kw = uint32_t(min(kb + 2, KB - 1));
                  if constexpr (MF == 4 && NV) {
                    FF_REQUEST_WEIGHTS(s, kw, m);
                    wait_loads<CPT + 1 + 8>(w[o][m][0], wsc[o][m]);
                    nv_store(wl + m * 2048, w[o][m][0], wsc[o][m]);
                  } else if constexpr (MF == 4) {
                    FF_REQUEST_WEIGHTS(s, kw, m);
                    wait_loads<CPT + 1 + 8>(w[o][m][0], w[o][m][1]);
                    *reinterpret_cast<u32x4*>(wl + m * 2048 + wr_off) = w[o][m][0];
                    *reinterpret_cast<u32x4*>(wl + m * 2048 + 1024 + wr_off) = w[o][m][1];
                  } else {
                    if (m & 1) load16_async(w[s][m >> 1][1], wfrag[m >> 1] + kw * 128u, woff1);
                    else load16_async(w[s][m >> 1][0], wfrag[m >> 1] + kw * 128u, woff0);
                    wait_loads<CPT + 1 + 8>(w[o][m >> 1][m & 1]);
                    *reinterpret_cast<u32x4*>(wl + (m >> 1) * 2048 + (m & 1) * 1024 + wr_off) = w[o][m >> 1][m & 1];
                  }
                }
              }
              if (m > 0) {
#pragma unroll
                for (int f = 0; f < 4; ++f)
#pragma unroll
                  for (int r = 0; r < 4; ++r)
                    acc[m - 1][f][r] = __fmaf_rn(pr[(m - 1) & 1][f][r], sc[(m - 1) & 1][(MODE == 0 && f >= 2) ? 1 : 0], acc[m - 1][f][r]);
                // The fmas have no ordering edge of their own, and instruction selection would emit all of them behind the
                // last fence of the K block (64 product registers live, the VALU work after the matrix work instead of
                // under it): an empty statement that reads the totals pins them in front of this fragment's fence.
                if constexpr (TW) {
#pragma unroll
                  for (int f = 0; f < 4; ++f)
#pragma unroll
                    for (int r = 0; r < 4; ++r) asm volatile("" ::"v"(acc[m - 1][f][r]));
                }
              }
              if constexpr (TW) __builtin_amdgcn_sched_barrier(0);
            }
            if constexpr (PF) {  // K block kb+1 sits in the transposition buffer by now: its fragments for the next stage
#pragma unroll
              for (int f = 0; f < 4; ++f) {
                wt[f][0] = *reinterpret_cast<const u32x4*>(wl + f * 2048 + rd_lo);
                wt[f][1] = *reinterpret_cast<const u32x4*>(wl + f * 2048 + rd_hi);
              }
              __builtin_amdgcn_wave_barrier();
            }
            // publish token tile kb+1
            FF_WAIT_TOKENS(8);
#pragma unroll
            for (int i = 0; i < CPT; ++i)
              if (stage_chunk) *reinterpret_cast<u32x4*>(&tile[(s & 1) ^ 1][tdst[i]]) = tv[i];
            if (tid < TM) *reinterpret_cast<float*>(&tile[(s & 1) ^ 1][TM * 128 + tid * 4]) = tsv;
            __syncthreads();
          } else {
            // a stage past the last K block: its registers still have (clamped) loads in flight and are about to be
            // requested into again; a register with a load in flight is never left unread
            if constexpr (NV) wait_loads<0>(w[s][0][0], w[s][1][0], w[s][2][0], w[s][3][0], wsc[s][0], wsc[s][1], wsc[s][2], wsc[s][3]);
            else wait_loads<0>(w[s][0][0], w[s][0][1], w[s][1][0], w[s][1][1], w[s][2][0], w[s][2][1], w[s][3][0], w[s][3][1]);
            FF_WAIT_TOKENS(0);
          }
          // Short groups: request token tile kb+2 and K block kb+P of the weights into the slot just consumed. The
          // requests are made also when the stage itself is past the last K block (clamped addresses), so that the
          // number of loads per stage does not depend on the path.
          if constexpr (!TW) {
            const uint32_t kn = uint32_t(min(kb + 2, KB - 1));
#pragma unroll
            for (int i = 0; i < CPT; ++i) load16_async(tv[i], tsrc[i] + kn * 128u);
            load4_async(tsv, ssrc + kn);
            const uint32_t kw = uint32_t(min(kb + P, KB - 1));
#pragma unroll
            for (int f = 0; f < 4; ++f) FF_REQUEST_WEIGHTS(s, kw, f);
          }
        }
      }
    }

    // The last stages have requested (clamped) data nobody reads: let it land before the registers are reused.
    FF_DRAIN_WEIGHTS();
    FF_WAIT_TOKENS(0);

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

#undef FF_REQUEST_WEIGHTS
#undef FF_DRAIN_WEIGHTS
#undef FF_WAIT_TOKENS

}  // namespace ffmoe
