// RoPE arithmetic shared by the kernels that rotate keys (gfx950 only): an
// 8-element slice of a head row as four interleaved (even, odd) pairs, the
// table fetch for a lane's four pairs and the rotation itself.
#ifndef SDV2KV_ROPE_DEVICE_H
#define SDV2KV_ROPE_DEVICE_H

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "sdv2kv_internal.h"

namespace sdv2 {

template <typename T>
struct Vec8;

template <>
struct Vec8<uint16_t> {                     // bf16 bit patterns
  uint4 raw;
  __device__ static Vec8 load(const uint16_t* p) {
    Vec8 v;
    v.raw = *reinterpret_cast<const uint4*>(p);
    return v;
  }
  __device__ void store(uint16_t* p) const { *reinterpret_cast<uint4*>(p) = raw; }
  __device__ double get(int i) const {
    const uint32_t w = (&raw.x)[i >> 1];
    const uint32_t bits = (i & 1) ? (w & 0xffff0000u) : (w << 16);
    return static_cast<double>(__uint_as_float(bits));
  }
  __device__ void set_pair(int p, double re, double im) {
    (&raw.x)[p] = pack_bf16_rne(static_cast<float>(re), static_cast<float>(im));
  }
  __device__ float getf(int i) const {
    const uint32_t w = (&raw.x)[i >> 1];
    return __uint_as_float((i & 1) ? (w & 0xffff0000u) : (w << 16));
  }
  // element i = x rounded to the storage type (bf16, nearest-even)
  __device__ void setf_pair(int p, float lo, float hi) {
    (&raw.x)[p] = pack_bf16_rne(lo, hi);
  }
};

template <>
struct Vec8<float> {
  float4 lo, hi;
  __device__ static Vec8 load(const float* p) {
    Vec8 v;
    v.lo = *reinterpret_cast<const float4*>(p);
    v.hi = *reinterpret_cast<const float4*>(p + 4);
    return v;
  }
  __device__ void store(float* p) const {
    *reinterpret_cast<float4*>(p) = lo;
    *reinterpret_cast<float4*>(p + 4) = hi;
  }
  __device__ double get(int i) const {
    return static_cast<double>(i < 4 ? (&lo.x)[i] : (&hi.x)[i - 4]);
  }
  __device__ void set_pair(int p, double re, double im) {
    float* dst = p < 2 ? &lo.x + 2 * p : &hi.x + 2 * (p - 2);
    dst[0] = static_cast<float>(re);
    dst[1] = static_cast<float>(im);
  }
  __device__ float getf(int i) const { return i < 4 ? (&lo.x)[i] : (&hi.x)[i - 4]; }
  __device__ void setf_pair(int p, float a, float b) {
    float* dst = p < 2 ? &lo.x + 2 * p : &hi.x + 2 * (p - 2);
    dst[0] = a;
    dst[1] = b;
  }
};

// (a + bi)(c + di) with every product and sum rounded separately, as the
// reference's complex128 multiply on the CPU does.
template <typename T>
__device__ __forceinline__ Vec8<T> rotate(const Vec8<T>& x, const double2 (&cs)[4]) {
#pragma clang fp contract(off)
  Vec8<T> y;
#pragma unroll
  for (int p = 0; p < 4; ++p) {
    const double a = x.get(2 * p), b = x.get(2 * p + 1);
    const double ac = a * cs[p].x;
    const double bd = b * cs[p].y;
    const double ad = a * cs[p].y;
    const double bc = b * cs[p].x;
    y.set_pair(p, ac - bd, ad + bc);
  }
  return y;
}

// Table entries of the four pairs a lane owns (pairs 4*lane .. 4*lane+3):
// pair p uses table row `frame` for p < split_t, `hi` for p < split_h, else
// `wi`, at column p (causal_model.py:64-68, 77-78).
__device__ __forceinline__ void load_rotation(const double2* freqs, int pairs, int split_t, int split_h, int lane,
                                              int64_t frame, int hi, int wi, double2 (&cs)[4]) {
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int p = lane * 4 + j;
    const int64_t pos = p < split_t ? frame : (p < split_h ? hi : wi);
    cs[j] = freqs[pos * pairs + p];
  }
}

}  // namespace sdv2

#endif  // SDV2KV_ROPE_DEVICE_H
