// Ordered weighted combine of per-(row, choice) BF16 contributions with the shared expert.
// Orders and rounding boundaries follow kernels/moe_combine.cu of the reference.
#include "common.cuh"
#include "api.h"

namespace ffmoe {

// scale[r] = bf16(sigmoid(bf16(dot))): thread-strided partial products (mul then add, not fused),
// 32-lane shuffle-down trees, then the tree over the 8 group partials (kernels/moe_combine.cu:21-49).
// scale = BF16(sigmoid(BF16(dot(x_row, seg)))): thread-strided FP32 products, 32-lane shuffle-down trees, then one tree
// over the 8 partials (kernels/moe_combine.cu:21-49 and moe_row_scale, :126-151). Every thread of the block gets it.
__device__ __forceinline__ float block_row_scale(const uint16_t* __restrict__ xr, const uint16_t* __restrict__ seg, int hidden) {
  __shared__ float red[32];
  __shared__ float s_scale;
  const int tid = threadIdx.x;
  float part = 0.0f;
  for (int c = tid; c < hidden; c += 256) part = __fadd_rn(part, __fmul_rn(bf16_to_f32(xr[c]), bf16_to_f32(seg[c])));
#pragma unroll
  for (int off = 16; off > 0; off >>= 1) {
    const float o = __shfl_down(part, off, 32);
    part = __fadd_rn(part, ((tid & 31) + off < 32) ? o : 0.0f);
  }
  if (tid < 32) red[tid] = 0.0f;
  __syncthreads();
  if ((tid & 31) == 0) red[tid >> 5] = part;
  __syncthreads();
  if (tid < 32) {
    float v = red[tid];
#pragma unroll
    for (int off = 16; off > 0; off >>= 1) {
      const float o = __shfl_down(v, off, 32);
      v = __fadd_rn(v, (tid + off < 32) ? o : 0.0f);
    }
    if (tid == 0) s_scale = bround(sigmoid1(bround(v)));
  }
  __syncthreads();
  return s_scale;
}

__global__ __launch_bounds__(256) void k_shared_scale(const uint16_t* __restrict__ x, const uint16_t* __restrict__ seg,
                                                      uint16_t* __restrict__ scale, int hidden) {
  const int row = blockIdx.x;
  const float v = block_row_scale(x + size_t(row) * hidden, seg, hidden);
  if (threadIdx.x == 0) scale[row] = f32_to_bf16(v);
}

// grid (ceil(hidden / 2048), rows): one 16-byte vector of 8 BF16 per thread. The first top_k threads rank the
// active choices by ascending expert id (stable), which is the order of the reference's insertion sort
// (kernels/moe_combine.cu:51-69); the ranks go through LDS so the accumulation loop indexes no private array.
__global__ __launch_bounds__(256) void k_combine(const uint16_t* __restrict__ contributions, const uint16_t* __restrict__ shared_out,
                                                 const uint16_t* __restrict__ scale, const int* __restrict__ ids,
                                                 const uint32_t* __restrict__ done, const uint32_t* __restrict__ final_active,
                                                 uint16_t* __restrict__ y, uint32_t* __restrict__ status, int top_k, int hidden,
                                                 int mode) {
  __shared__ int s_order[FFMOE_MAX_TOP_K];
  __shared__ int s_live;
  const int tid = threadIdx.x, row = blockIdx.y;
  const int a0 = row * top_k;
  const bool ordered = !(mode == FFMOE_COMBINE_ACCUM_FP32 || mode == FFMOE_COMBINE_ACCUM_BF16);
  if (tid < top_k) {
    if (!ordered) {
      s_order[tid] = tid;
    } else {
      const uint32_t want = final_active ? final_active[a0 + tid] : 1u;
      if (done && done[a0 + tid] != want && status && blockIdx.x == 0) atomicOr(status, 1u);
      if (want != 0u) {
        const int mine = ids[a0 + tid];
        int rank = 0;
        for (int c = 0; c < top_k; ++c) {
          const bool act = final_active ? final_active[a0 + c] != 0u : true;
          const int other = ids[a0 + c];
          rank += (act && (other < mine || (other == mine && c < tid))) ? 1 : 0;
        }
        s_order[rank] = tid;
      }
    }
  }
  if (tid == 0) {
    int live = top_k;
    if (ordered && final_active) {
      live = 0;
      for (int c = 0; c < top_k; ++c) live += final_active[a0 + c] != 0u ? 1 : 0;
    }
    s_live = live;
  }
  __syncthreads();
  const int live = s_live;
  const int d0 = (blockIdx.x * 256 + tid) * 8;
  if (d0 >= hidden) return;
  const float sc = (mode == FFMOE_COMBINE_GATED) ? bf16_to_f32(scale[row]) : 0.0f;
  float acc[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) acc[j] = 0.0f;
  u32x4 sh = {0, 0, 0, 0};
  if (mode != FFMOE_COMBINE_ROUTED) sh = load16(shared_out + size_t(row) * hidden + d0);
  for (int k0 = 0; k0 < live; k0 += 8) {
    u32x4 c[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int k = k0 + i < live ? k0 + i : live - 1;  // all eight loads go out before the first add
      c[i] = load16(contributions + (size_t(a0) + s_order[k]) * hidden + d0);
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      if (k0 + i < live) {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          if (mode == FFMOE_COMBINE_BF16) {
            acc[2 * q] = bround(__fadd_rn(acc[2 * q], bf16lo(c[i][q])));
            acc[2 * q + 1] = bround(__fadd_rn(acc[2 * q + 1], bf16hi(c[i][q])));
          } else {
            acc[2 * q] = __fadd_rn(acc[2 * q], bf16lo(c[i][q]));
            acc[2 * q + 1] = __fadd_rn(acc[2 * q + 1], bf16hi(c[i][q]));
          }
        }
      }
    }
  }
  u32x4 out;
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    float r[2];
#pragma unroll
    for (int hsel = 0; hsel < 2; ++hsel) {
      const float s = hsel ? bf16hi(sh[q]) : bf16lo(sh[q]);
      const float a = acc[2 * q + hsel];
      float v;
      switch (mode) {
        case FFMOE_COMBINE_GATED: v = __fadd_rn(bround(a), bround(__fmul_rn(sc, s))); break;
        case FFMOE_COMBINE_UNGATED:
        case FFMOE_COMBINE_ACCUM_BF16: v = __fadd_rn(bround(a), s); break;
        case FFMOE_COMBINE_BF16:
        case FFMOE_COMBINE_ACCUM_FP32: v = __fadd_rn(a, s); break;
        default: v = a; break;
      }
      r[hsel] = v;
    }
    out[q] = pack_bf16x2(r[0], r[1]);
  }
  *reinterpret_cast<u32x4*>(y + size_t(row) * hidden + d0) = out;
}

// Combine group with the residual add (kernels/moe_combine.cu:246-533): ff = BF16(BF16(routed) + gated) with
// routed = the ordered FP32 sum of the row's live contributions (or a routed sum handed in, the peer-join form) and
// gated = BF16(scale_row * shared) when seg is given, shared otherwise; then y_out = ff, or residual += ff in BF16.
// grid (ceil(hidden / 2048), rows); the row scale is recomputed by every block of the row (one pass over x_row).
__global__ __launch_bounds__(256) void k_combine_residual(const uint16_t* __restrict__ contributions, const uint16_t* __restrict__ routed_in,
                                                          const uint16_t* __restrict__ shared_out, const uint16_t* __restrict__ seg,
                                                          const uint16_t* __restrict__ x, long long x_stride, const int* __restrict__ ids,
                                                          const uint32_t* __restrict__ done, const uint32_t* __restrict__ final_active,
                                                          uint16_t* __restrict__ residual, uint16_t* __restrict__ y_out,
                                                          uint32_t* __restrict__ status, int top_k, int hidden) {
  __shared__ int s_order[FFMOE_MAX_TOP_K];
  __shared__ int s_live;
  const int tid = threadIdx.x, row = blockIdx.y;
  const int a0 = row * top_k;
  if (contributions) {
    if (tid < top_k) {
      const uint32_t want = final_active ? final_active[a0 + tid] : 1u;
      if (done && done[a0 + tid] != want && status && blockIdx.x == 0) atomicOr(status, 1u);
      if (want != 0u) {
        const int mine = ids[a0 + tid];
        int rank = 0;
        for (int c = 0; c < top_k; ++c) {
          const bool act = final_active ? final_active[a0 + c] != 0u : true;
          const int other = ids[a0 + c];
          rank += (act && (other < mine || (other == mine && c < tid))) ? 1 : 0;
        }
        s_order[rank] = tid;
      }
    }
    if (tid == 0) {
      int live = top_k;
      if (final_active) {
        live = 0;
        for (int c = 0; c < top_k; ++c) live += final_active[a0 + c] != 0u ? 1 : 0;
      }
      s_live = live;
    }
  }
  const float sc = seg ? block_row_scale(x + (long long)row * x_stride, seg, hidden) : 0.0f;  // ends with a block barrier
  if (!seg) __syncthreads();
  const int d0 = (blockIdx.x * 256 + tid) * 8;
  if (d0 >= hidden) return;
  float routed[8];
  if (contributions) {
    const int live = s_live;
#pragma unroll
    for (int j = 0; j < 8; ++j) routed[j] = 0.0f;
    for (int k = 0; k < live; ++k) {
      const u32x4 c = load16(contributions + (size_t(a0) + s_order[k]) * hidden + d0);
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        routed[2 * q] = __fadd_rn(routed[2 * q], bf16lo(c[q]));
        routed[2 * q + 1] = __fadd_rn(routed[2 * q + 1], bf16hi(c[q]));
      }
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) routed[j] = bround(routed[j]);
  } else {
    const u32x4 r = load16(routed_in + size_t(row) * hidden + d0);
#pragma unroll
    for (int q = 0; q < 4; ++q) { routed[2 * q] = bf16lo(r[q]); routed[2 * q + 1] = bf16hi(r[q]); }
  }
  const u32x4 sh = load16(shared_out + size_t(row) * hidden + d0);
  u32x4 res = {0, 0, 0, 0};
  if (!y_out) res = load16(residual + size_t(row) * hidden + d0);
  u32x4 out;
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    float v[2];
#pragma unroll
    for (int hsel = 0; hsel < 2; ++hsel) {
      const float s = hsel ? bf16hi(sh[q]) : bf16lo(sh[q]);
      const float gated = seg ? bround(__fmul_rn(sc, s)) : s;
      const float ff = bround(__fadd_rn(routed[2 * q + hsel], gated));
      v[hsel] = y_out ? ff : __fadd_rn(hsel ? bf16hi(res[q]) : bf16lo(res[q]), ff);
    }
    out[q] = pack_bf16x2(v[0], v[1]);
  }
  *reinterpret_cast<u32x4*>((y_out ? y_out : residual) + size_t(row) * hidden + d0) = out;
}

}  // namespace ffmoe

using namespace ffmoe;

extern "C" __attribute__((visibility("default"))) int ffmoe_shared_scale(const void* x, const void* seg, void* scale, int rows, int hidden, void* stream) {
  FF_REQUIRE(rows >= 1 && hidden >= 1, FFMOE_ERR_SHAPE, "shared_scale rows=%d hidden=%d", rows, hidden);
  FF_PTR16(x); FF_PTR16(seg); FF_PTR2(scale);
  FF_NO_OVERLAP(scale, size_t(rows) * 2, x, size_t(rows) * hidden * 2);
  FF_NO_OVERLAP(scale, size_t(rows) * 2, seg, size_t(hidden) * 2);
  hipLaunchKernelGGL(k_shared_scale, dim3(rows), dim3(256), 0, (hipStream_t)stream, (const uint16_t*)x, (const uint16_t*)seg,
                     (uint16_t*)scale, hidden);
  return ff_launch_status();
}

extern "C" __attribute__((visibility("default"))) int ffmoe_combine(const void* contributions, const void* shared_out, const void* scale, const int* ids,
                             const uint32_t* done, const uint32_t* final_active, void* y, uint32_t* status, int rows,
                             int top_k, int hidden, int mode, void* stream) {
  FF_REQUIRE(rows >= 1 && top_k >= 1 && top_k <= FFMOE_MAX_TOP_K, FFMOE_ERR_SHAPE, "combine rows=%d top_k=%d out of range", rows, top_k);
  FF_REQUIRE(hidden >= 8 && hidden % 8 == 0, FFMOE_ERR_SHAPE, "combine hidden=%d must be a positive multiple of 8", hidden);
  FF_REQUIRE(mode >= 0 && mode <= FFMOE_COMBINE_ROUTED, FFMOE_ERR_UNSUPPORTED, "unknown combine mode %d", mode);
  FF_PTR16(contributions); FF_PTR16(y);
  const bool ordered = !(mode == FFMOE_COMBINE_ACCUM_FP32 || mode == FFMOE_COMBINE_ACCUM_BF16);
  if (ordered) FF_PTR4(ids);
  if (mode != FFMOE_COMBINE_ROUTED) FF_PTR16(shared_out);
  if (mode == FFMOE_COMBINE_GATED) FF_PTR2(scale);
  if (done) FF_PTR4(done);
  if (final_active) FF_PTR4(final_active);
  if (status) FF_PTR4(status);
  const size_t yb = size_t(rows) * hidden * 2, cb = size_t(rows) * top_k * hidden * 2;
  FF_NO_OVERLAP(y, yb, contributions, cb);
  if (mode != FFMOE_COMBINE_ROUTED) FF_NO_OVERLAP(y, yb, shared_out, yb);
  if (ordered) FF_NO_OVERLAP(y, yb, ids, size_t(rows) * top_k * 4);
  hipLaunchKernelGGL(k_combine, dim3((hidden / 8 + 255) / 256, rows), dim3(256), 0, (hipStream_t)stream, (const uint16_t*)contributions,
                     (const uint16_t*)shared_out, (const uint16_t*)scale, ids, done, final_active, (uint16_t*)y, status, top_k,
                     hidden, mode);
  return ff_launch_status();
}

extern "C" __attribute__((visibility("default"))) int ffmoe_combine_residual(const void* contributions, const void* routed_in, const void* shared_out,
                                                                            const void* seg, const void* x, long long x_stride, const int* ids,
                                                                            const uint32_t* done, const uint32_t* final_active, void* residual,
                                                                            void* y_out, uint32_t* status, int rows, int top_k, int hidden, void* stream) {
  FF_REQUIRE(rows >= 1 && hidden >= 8 && hidden % 8 == 0, FFMOE_ERR_SHAPE, "combine_residual rows=%d hidden=%d (hidden must be a positive multiple of 8)", rows, hidden);
  FF_REQUIRE((contributions != nullptr) != (routed_in != nullptr), FFMOE_ERR_NULL, "give either contributions or routed_in");
  if (contributions) {
    FF_REQUIRE(top_k >= 1 && top_k <= FFMOE_MAX_TOP_K, FFMOE_ERR_SHAPE, "combine_residual top_k=%d out of range", top_k);
    FF_PTR16(contributions); FF_PTR4(ids);
  } else {
    FF_PTR16(routed_in);
  }
  FF_PTR16(shared_out);
  if (seg) { FF_PTR2(seg); FF_PTR2(x); FF_REQUIRE(x_stride >= hidden, FFMOE_ERR_SHAPE, "x_stride=%lld is shorter than a row", x_stride); }
  FF_REQUIRE(residual != nullptr || y_out != nullptr, FFMOE_ERR_NULL, "give residual (updated in place) or y_out");
  void* target = y_out ? y_out : residual;
  FF_PTR16(target);
  if (done) FF_PTR4(done);
  if (final_active) FF_PTR4(final_active);
  if (status) FF_PTR4(status);
  const size_t yb = size_t(rows) * hidden * 2;
  if (contributions) FF_NO_OVERLAP(target, yb, contributions, size_t(rows) * top_k * hidden * 2);
  if (routed_in) FF_NO_OVERLAP(target, yb, routed_in, yb);
  FF_NO_OVERLAP(target, yb, shared_out, yb);
  hipLaunchKernelGGL(k_combine_residual, dim3((hidden / 8 + 255) / 256, rows), dim3(256), 0, (hipStream_t)stream, (const uint16_t*)contributions,
                     (const uint16_t*)routed_in, (const uint16_t*)shared_out, (const uint16_t*)seg, (const uint16_t*)x, x_stride, ids, done,
                     final_active, (uint16_t*)residual, (uint16_t*)y_out, status, top_k, hidden);
  return ff_launch_status();
}
