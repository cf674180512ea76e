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
  __device__ static Vec8 zero() {
    Vec8 v;
    v.raw = make_uint4(0u, 0u, 0u, 0u);
    return v;
  }
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
  __device__ static Vec8 zero() {
    Vec8 v;
    v.lo = make_float4(0.f, 0.f, 0.f, 0.f);
    v.hi = v.lo;
    return v;
  }
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

// WanRMSNorm of an 8-element slice once the token's 1 / rms is known
// (wan_base/modules/model.py:77-86): x * r rounded to the storage type, times
// the weight, rounded to the storage type again.
template <typename T>
__device__ __forceinline__ Vec8<T> normalise(const Vec8<T>& x, float r, const Vec8<T>& w) {
  Vec8<T> y;
  Vec8<T> n;                           // x * r in the storage type
#pragma unroll
  for (int p = 0; p < 4; ++p) n.setf_pair(p, x.getf(2 * p) * r, x.getf(2 * p + 1) * r);
#pragma unroll
  for (int p = 0; p < 4; ++p) y.setf_pair(p, n.getf(2 * p) * w.getf(2 * p), n.getf(2 * p + 1) * w.getf(2 * p + 1));
  return y;
}

// Sum of squares of a token's full heads * 128 vector, for two vectors at once
// (k and q), by one wave, in the order of PyTorch's CPU sum kernel (ATen
// cascade_sum / vectorized_inner_sum with 8-float vectors, which the AVX2 and
// AVX512 builds share): element e of the row belongs to accumulator (e / 8 % 4,
// e % 8); an accumulator adds its elements in blocks of 16, each block summed
// in order from zero, the block sums added up in order; a trailing partial
// block goes first; then the four accumulators of a vector lane are added in
// order, then the eight lanes in order, starting from zero.  The caller has
// checked this against torch bit for bit on the CPU.
//
// Lane l of the wave holds, per step j, the slice l % 16 of head 4 j + l / 16
// (zeros past the last head).  With e = 128 head + 8 slice + t the 16 lanes
// l % 4 == c of a step hold exactly one block of accumulator (c, t), in lane
// order.  Per step every lane parks its 8 + 8 squares in `scratch` (2 x 512
// floats of this wave) and lanes 0-31 (k) / 32-63 (q) each walk one
// accumulator's block; LDS operations of a wave complete in order, so no
// barrier is needed.
template <typename T, int kSteps>
__device__ __forceinline__ void wave_sum_squares(const Vec8<T> (&k)[kSteps], const Vec8<T> (&q)[kSteps], int heads,
                                                 float (&scratch)[2][64 * 8], int lane, float& sum_k, float& sum_q) {
#pragma clang fp contract(off)
  const int which = lane >> 5;               // lanes 0-31 add up k, lanes 32-63 q
  const int chain = lane & 31;               // accumulator (c, t) = (chain % 4, chain / 4)
  const int c = chain & 3, t = chain >> 2;
  const int full = heads >> 2;               // steps whose four heads all exist: whole blocks of 16
  const int tail = 4 * (heads & 3);          // elements of the trailing partial block
  float blocks = 0.f;                        // the whole blocks' sums, added up in order
  float trailing = 0.f;
#pragma unroll
  for (int j = 0; j < kSteps; ++j) {
    if (4 * j < heads) {
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        scratch[0][lane * 8 + i] = k[j].getf(i) * k[j].getf(i);
        scratch[1][lane * 8 + i] = q[j].getf(i) * q[j].getf(i);
      }
      const int count = j < full ? 16 : tail;
      float block = 0.f;
#pragma unroll
      for (int m = 0; m < 16; ++m)
        if (m < count) block += scratch[which][(c + 4 * m) * 8 + t];
      if (j < full) blocks += block;
      else trailing = block;
    }
  }
  const float mine = tail ? trailing + blocks : blocks;
  // the four accumulators of vector lane t, in order (they sit in neighbouring lanes)
  const int quad = lane & ~3;
  float lane_sum = __shfl(mine, quad, 64);
  lane_sum += __shfl(mine, quad + 1, 64);
  lane_sum += __shfl(mine, quad + 2, 64);
  lane_sum += __shfl(mine, quad + 3, 64);
  // the eight vector lanes, in order, from zero
  float total = 0.f;
#pragma unroll
  for (int v = 0; v < 8; ++v) total += __shfl(lane_sum, (lane & 32) + 4 * v, 64);
  sum_k = __shfl(total, 0, 64);
  sum_q = __shfl(total, 32, 64);
}

}  // namespace sdv2

#endif  // SDV2KV_ROPE_DEVICE_H
