// Device-side pieces shared by the convolution kernels: MFMA register layout helpers, the
// saturating pack, the 64-bit-constant requantisation of a row block, the fused EltwiseAdd on 16
// requantised channels, and buffer-descriptor loads.
#pragma once

#include "common.hpp"

#include <type_traits>
#include <utility>

namespace tpuhip {}
using namespace tpuhip;

// f(integral_constant<int, 0>) ... f(integral_constant<int, N - 1>), in order: a loop whose index is a
// compile-time constant in every trip
template <typename F, int... I>
__device__ __forceinline__ void static_for_impl(F &&f, std::integer_sequence<int, I...>) {
  (f(std::integral_constant<int, I>{}), ...);
}
template <int N, typename F>
__device__ __forceinline__ void static_for(F &&f) {
  static_for_impl(f, std::make_integer_sequence<int, N>{});
}

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef unsigned int v4u __attribute__((ext_vector_type(4)));

// tile-local weight row (as the MFMA sees it) -> tile-local output channel
__host__ __device__ inline int mfma_row_to_oc(int row, int tm) {
  const int wave_rows = tm * 32;
  const int wrow = row % wave_rows, wbase = row - wrow;
  const int i = wrow / 32, ri = wrow % 32;
  const int fk = (ri >> 2) & 1;
  const int r = (ri >> 3) * 4 + (ri & 3);
  return wbase + fk * 16 * tm + i * 16 + r;
}

typedef short v2s __attribute__((ext_vector_type(2)));
typedef unsigned short v2us __attribute__((ext_vector_type(2)));

// four int32 -> four saturated int8 in one dword; lo is -128 or 0 (fused ReLU)
__device__ __forceinline__ uint32_t pack_sat4(int32_t a, int32_t b, int32_t c, int32_t d, int lo) {
  v2s p0 = __builtin_amdgcn_cvt_pk_i16(a, b);
  v2s p1 = __builtin_amdgcn_cvt_pk_i16(c, d);
  const v2s vlo = {(short)lo, (short)lo}, vhi = {127, 127};
  p0 = __builtin_elementwise_min(__builtin_elementwise_max(p0, vlo), vhi);
  p1 = __builtin_elementwise_min(__builtin_elementwise_max(p1, vlo), vhi);
  return __builtin_amdgcn_perm(__builtin_bit_cast(uint32_t, p1), __builtin_bit_cast(uint32_t, p0),
                               0x06040200u);
}

// 16-byte load through a buffer descriptor: an offset at or beyond the
// descriptor's size yields zeros, which is how padding taps, pixels past the end
// of the tensor and K steps past the end of the filter are fed to the MFMAs
// without a branch.
__device__ __forceinline__ v4i buffer_load16(__amdgpu_buffer_rsrc_t rsrc, uint32_t offset) {
  return (v4i)__builtin_amdgcn_raw_buffer_load_b128(rsrc, offset, 0, 0);
}
constexpr uint32_t kOobOffset = 0x7fffffffu;

// Requantisation of accumulators that started at zero, for layers whose overflow-free form the
// host has proved: the bias rides in the addend of the 64-bit multiply-add,
//   (acc + b) * m + 2^30 == acc * m + c,   c = b * m + 2^30   (pc64: (low, high) pairs per channel).
// RELU (the layer clamps at 0 after saturation): pc64 holds c + 2^(r-1) * 2^31, pshift r - 1, and the
// result is hi32(acc * m + c') >> (r - 1); otherwise x = (acc * m + c) >> 31 and the rounding shift
// (x + 2^(r-1) - (x < 0)) >> r with pshift = r, phpot = 2^(r-1).
template <int TN, bool RELU>
__device__ __forceinline__ void requant_rows_c64(const v16i (&acc)[TN], int lo, const int32_t *pc64,
                                                 const int32_t *pmult, const int32_t *pshift,
                                                 const int32_t *phpot, uint32_t (&outw)[TN][4]) {
#pragma unroll
  for (int qd = 0; qd < 4; ++qd) {
    const v4i c01 = *reinterpret_cast<const v4i *>(pc64 + qd * 8);
    const v4i c23 = *reinterpret_cast<const v4i *>(pc64 + qd * 8 + 4);
    const v4i m4 = *reinterpret_cast<const v4i *>(pmult + qd * 4);
    const v4i r4 = *reinterpret_cast<const v4i *>(pshift + qd * 4);
    v4i h4 = {0, 0, 0, 0};
    if (!RELU) h4 = *reinterpret_cast<const v4i *>(phpot + qd * 4);
    const int64_t c[4] = {(int64_t)(((uint64_t)(uint32_t)c01[1] << 32) | (uint32_t)c01[0]),
                          (int64_t)(((uint64_t)(uint32_t)c01[3] << 32) | (uint32_t)c01[2]),
                          (int64_t)(((uint64_t)(uint32_t)c23[1] << 32) | (uint32_t)c23[0]),
                          (int64_t)(((uint64_t)(uint32_t)c23[3] << 32) | (uint32_t)c23[2])};
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      int32_t y[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int64_t p = (int64_t)acc[j][qd * 4 + e] * (int64_t)m4[e] + c[e];
        if (RELU) {
          y[e] = (int32_t)(p >> 32) >> r4[e];
        } else {
          const int32_t x = (int32_t)(p >> 31);
          y[e] = (x + h4[e] + (x >> 31)) >> r4[e];
        }
      }
      outw[j][qd] = pack_sat4(y[0], y[1], y[2], y[3], lo);
    }
    __builtin_amdgcn_sched_barrier(0);
  }
}


// EltwiseAdd (core/eltwise.cpp:52-85, integer form) of 16 freshly requantised channels o with
// the other operand's 16 bytes sv:  sat8(floor(relu?(sv * m_src + o * m_conv) / 2^rshift + 0.5)).
// pk: |multipliers| <= 127 and rshift <= 8, so the sum fits packed int16 arithmetic.
__device__ __forceinline__ v4i fused_add_chunk(const v4i &o, const v4i &sv, int m_src, int m_conv, int rshift,
                                               int relu, int pk) {
  v4i z;
  if (pk) {
    // two outputs per instruction: the bytes of both operands widen to packed int16 (even and
    // odd bytes apart), src * m_src + y * m_conv + 2^(r-1) stays inside int16, and ReLU / lower
    // saturation (a floor before the shift), shift and upper saturation are packed ops too
    const int r = rshift;
    const short rnd = (short)(r > 0 ? (1 << (r - 1)) : 0);
    const short fl = (short)(relu ? 0 : -(128 << r));
    const v2s msrc = {(short)m_src, (short)m_src}, mconv = {(short)m_conv, (short)m_conv};
    const v2s rnd2 = {rnd, rnd}, fl2 = {fl, fl}, top = {127, 127}, sh = {(short)r, (short)r}, eight = {8, 8};
    const v2us ueight = {8, 8};
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int32_t ow = o[q], sw_ = sv[q];   // plain copies: a vector element is no object to bit_cast
      const v2s o16 = __builtin_bit_cast(v2s, ow), s16 = __builtin_bit_cast(v2s, sw_);
      // even bytes: up by 8 as unsigned halves (a signed shift may be assumed not to overflow), down arithmetically
      const v2s olo = __builtin_bit_cast(v2s, __builtin_bit_cast(v2us, ow) << ueight) >> eight, ohi = o16 >> eight;
      const v2s slo = __builtin_bit_cast(v2s, __builtin_bit_cast(v2us, sw_) << ueight) >> eight, shi = s16 >> eight;
      v2s tlo = olo * mconv + (slo * msrc + rnd2);
      v2s thi = ohi * mconv + (shi * msrc + rnd2);
      tlo = __builtin_elementwise_min(__builtin_elementwise_max(tlo, fl2) >> sh, top);
      thi = __builtin_elementwise_min(__builtin_elementwise_max(thi, fl2) >> sh, top);
      z[q] = (int)__builtin_amdgcn_perm(__builtin_bit_cast(uint32_t, thi), __builtin_bit_cast(uint32_t, tlo),
                                        0x06020400u);
    }
    return z;
  }
  // sum = src * m_src + y * m_conv as one 4 x int8 dot product per output (the two unused byte
  // lanes are zero), with the rounding term as its addend: adding 2^(r-1) before the ReLU gives
  // the same quotient as after it.
  int32_t rnd = rshift > 0 ? (1 << (rshift - 1)) : 0;
  int32_t mpair = (m_src & 0xff) | ((m_conv & 0xff) << 8);
  int32_t floor_ = relu ? 0 : (int32_t)0x80000000;
  // one scalar and one vector copy of the uniform operands, made once
  asm volatile("" : "+s"(rnd), "+v"(mpair), "+s"(floor_));
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    int32_t t[4];
#pragma unroll
    for (int b = 0; b < 4; ++b) {
      const uint32_t pair = __builtin_amdgcn_perm((uint32_t)o[q], (uint32_t)sv[q],
                                                  0x0c0c0000u | ((4u + b) << 8) | (uint32_t)b);
      int32_t sum;   // the three-operand form: no copy of the addend into the result first
      asm("v_dot4_i32_i8 %0, %1, %2, %3" : "=v"(sum) : "v"(pair), "v"(mpair), "s"(rnd));
      t[b] = max(sum, floor_) >> rshift;
    }
    z[q] = (int)pack_sat4(t[0], t[1], t[2], t[3], -128);
  }
  return z;
}
