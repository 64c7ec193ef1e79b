// Shared declarations of the tpuhip library: context, error reporting and the
// device-side requantisation arithmetic every kernel epilogue uses.
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <string>

#include "tpuhip.h"

struct tpuhip_ctx {
  int device = 0;
  hipStream_t stream = nullptr;
  bool owns_stream = false;
  int num_cu = 0;
  bool autotune = true;  // time the conv tile variants on a layer's first use
  // when set, every kernel launch carries these events: they bracket the dispatch
  // itself (begin / end of execution), not the gaps around it
  hipEvent_t prof_start = nullptr, prof_stop = nullptr;
  // device memory kernels use beyond their operands (split-K partial sums): allocated on first need, grown when a larger layer comes, freed with the context
  void *workspace = nullptr;
  size_t workspace_bytes = 0;
};

// conv.hip: looks up this device's copy of the library's static scratch array (the one the
// allocation-free entry point works in); called once per context with the device current
extern "C" int tpuhip_static_scratch_init(int device);
// conv.hip: a context being destroyed stops being the static scratch's last user
extern "C" void tpuhip_static_scratch_forget(const tpuhip_ctx *ctx);

namespace tpuhip {

int set_error(int status, const char *fmt, ...) __attribute__((format(printf, 2, 3)));

#define TPUHIP_CHECK_HIP(expr)                                                          \
  do {                                                                                  \
    hipError_t e__ = (expr);                                                            \
    if (e__ != hipSuccess)                                                              \
      return ::tpuhip::set_error(TPUHIP_ERR_HIP, "%s failed: %s (%s:%d)", #expr,        \
                                 hipGetErrorString(e__), __FILE__, __LINE__);           \
  } while (0)

#define TPUHIP_REQUIRE(cond, ...)                                                       \
  do {                                                                                  \
    if (!(cond)) return ::tpuhip::set_error(TPUHIP_ERR_INVALID, __VA_ARGS__);           \
  } while (0)

// Launches on the context's stream; with profiling events set the dispatch records
// its own begin / end timestamps into them.
template <typename F, typename... Args>
inline void launch(tpuhip_ctx *ctx, F kernel, dim3 grid, dim3 block, Args... args) {
  if (ctx->prof_start)
    hipExtLaunchKernelGGL(kernel, grid, block, 0, ctx->stream, ctx->prof_start, ctx->prof_stop, 0,
                          args...);
  else
    hipLaunchKernelGGL(kernel, grid, block, 0, ctx->stream, args...);
}

inline int round_up(int v, int m) { return (v + m - 1) / m * m; }
inline int64_t ceil_div64(int64_t a, int64_t b) { return (a + b - 1) / b; }

// 256-entry int8 table passed to kernels by value (lives in the kernel-argument
// segment, so no device allocation or copy is needed and launches stay capturable).
struct Table256 {
  uint32_t w[64];
};

// ---------------------------------------------------------------------------
// Requantisation arithmetic (QuantizationArithmetic.cpp:487-539), device side.
// ---------------------------------------------------------------------------

// SaturatingRoundingDoublingHighMul (:501-509).  The reference adds a
// sign-dependent nudge and divides by 2^31 truncating toward zero; for every
// pair of int32 that equals floor((a*b + 2^30) / 2^31), i.e. one 64-bit
// multiply-add and an arithmetic shift.  The cast keeps the low 32 bits like
// the reference's static_cast.
__device__ __forceinline__ int32_t srdhm(int32_t a, int32_t b) {
  const int64_t ab = (int64_t)a * (int64_t)b;
  return (int32_t)((ab + (1ll << 30)) >> 31);
}

// RoundingDivideByPOT (:487-499) with mask = 2^e - 1 and half = mask >> 1
// precomputed per channel; exact for e in [0,31] (e == 0 gives mask 0, so the
// value passes through) and for x == 0.
__device__ __forceinline__ int32_t rdbp(int32_t x, int32_t e, int32_t mask, int32_t half) {
  const int32_t rem = x & mask;
  const int32_t thr = half - (x >> 31);  // + 1 when x < 0
  return (x >> e) + (rem > thr ? 1 : 0);
}

__device__ __forceinline__ int32_t clamp_i32(int32_t v, int32_t lo, int32_t hi) {
  return min(max(v, lo), hi);
}

// applyMultiplierAndRShiftAndSaturateInt8(int32, rshift, multiplier, qdm=true) (:530-539)
// followed by the optional ReLU of :866-868, folded into the lower clamp bound.
__device__ __forceinline__ int32_t requant_qdm(int32_t v, int32_t mult, int32_t e, int32_t mask,
                                               int32_t half, int32_t lo) {
  return clamp_i32(rdbp(srdhm(v, mult), e, mask, half), lo, 127);
}

// saturateInt8 (:301-334) of a float that holds v * m / 2^r computed the
// reference's way (float product, float quotient): floor(f + 0.5) evaluated
// exactly, then the clamp.
__device__ __forceinline__ int32_t saturate_int8_f(float f) {
  f = fminf(fmaxf(f, -1024.0f), 1024.0f);   // the clamp makes the range harmless
  const float fl = floorf(f);
  const float frac = f - fl;                // exact
  int32_t q = (int32_t)fl + (frac >= 0.5f ? 1 : 0);
  return clamp_i32(q, -128, 127);
}

}  // namespace tpuhip
