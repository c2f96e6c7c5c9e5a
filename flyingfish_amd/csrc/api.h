// Host-side contract checks shared by the entry points of libffmoe.
// The checks mirror the reference's operator validators (non-null, aligned, dense, non-overlapping
// views: src/backend/cuda/contracts.rs:80-137 and the `no_overlap` calls of each op).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stddef.h>
#include "../../include/ffmoe.h"

namespace ffmoe {
int ff_fail(int code, const char* fmt, ...) __attribute__((format(printf, 2, 3)));
int ff_launch_status();
inline bool ff_overlap(const void* a, size_t na, const void* b, size_t nb) {
  const uintptr_t pa = reinterpret_cast<uintptr_t>(a), pb = reinterpret_cast<uintptr_t>(b);
  return na != 0 && nb != 0 && pa < pb + nb && pb < pa + na;
}
}  // namespace ffmoe

#define FF_REQUIRE(cond, code, ...) \
  do { if (!(cond)) return ::ffmoe::ff_fail((code), __VA_ARGS__); } while (0)
#define FF_TRY(expr) \
  do { const int ff_rc_ = (expr); if (ff_rc_) return ff_rc_; } while (0)
#define FF_PTR_ALIGNED(p, align)                                                                   \
  do {                                                                                             \
    if ((p) == nullptr) return ::ffmoe::ff_fail(FFMOE_ERR_NULL, "%s is NULL", #p);                 \
    if (reinterpret_cast<uintptr_t>(p) % (align))                                                  \
      return ::ffmoe::ff_fail(FFMOE_ERR_ALIGN, "%s is not %d-byte aligned", #p, int(align));       \
  } while (0)
#define FF_PTR16(p) FF_PTR_ALIGNED(p, 16)
#define FF_PTR4(p) FF_PTR_ALIGNED(p, 4)
#define FF_PTR2(p) FF_PTR_ALIGNED(p, 2)
#define FF_NO_OVERLAP(out, nout, in, nin)                                                          \
  do {                                                                                             \
    if (::ffmoe::ff_overlap((out), (nout), (in), (nin)))                                           \
      return ::ffmoe::ff_fail(FFMOE_ERR_OVERLAP, "%s overlaps %s", #out, #in);                     \
  } while (0)
