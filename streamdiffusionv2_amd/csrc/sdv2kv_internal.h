// Device helpers shared by the sdv2kv kernels (gfx950 only).
#ifndef SDV2KV_INTERNAL_H
#define SDV2KV_INTERNAL_H

#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>
#include <stdint.h>

struct sdv2_attn_params;

namespace sdv2 {

// sdv2_swa_attn_fwd for fp32 tensors (swa_attn_fwd_f32.hip): fp32 arithmetic throughout, unsplit
int attn_fwd_f32(const sdv2_attn_params* p);

// Measurement hooks (sdv2kv_profile.h), kept per calling thread in
// sdv2kv_api.hip: the event pair armed for the next launch of a kernel (taken
// = disarmed).
struct TimingPair {
  void* start;
  void* stop;
};
TimingPair take_timing(int kernel);

// Launch kernel `which` (an sdv2_profile_kernel); when the calling thread has
// armed timing events for it they are attached to the kernel's own dispatch.
template <typename Kernel, typename Args>
inline void launch_timed(int which, Kernel kernel, dim3 grid, dim3 block, uint32_t lds_bytes, hipStream_t stream,
                         const Args& args) {
  const TimingPair t = take_timing(which);
  if (t.start && t.stop)
    hipExtLaunchKernelGGL(kernel, grid, block, lds_bytes, stream, static_cast<hipEvent_t>(t.start),
                          static_cast<hipEvent_t>(t.stop), 0, args);
  else
    hipLaunchKernelGGL(kernel, grid, block, lds_bytes, stream, args);
}

// float -> bfloat16 bit pattern, round-to-nearest-even, NaN -> 0x7FC0: the
// rounding PyTorch applies when a float (or a double already narrowed to
// float) is stored as bfloat16.
__device__ __forceinline__ uint32_t f32_to_bf16_rne(float f) {
  const uint32_t u = __float_as_uint(f);
  if (f != f) return 0x7fc0u;
  return (u + 0x7fffu + ((u >> 16) & 1u)) >> 16;
}

__device__ __forceinline__ float bf16_bits_to_f32(uint32_t b) { return __uint_as_float(b << 16); }

// Two floats -> packed bfloat16 pair (lo in the low half), nearest-even: the
// hardware conversion v_cvt_pk_bf16_f32.  Same bits as f32_to_bf16_rne for every
// number; a NaN stays a NaN but keeps its sign and payload bits (PyTorch itself
// encodes a NaN result differently on its scalar, vectorised and GPU paths:
// 0x7FC0, 0xFFFF, 0x7FFF).
__device__ __forceinline__ uint32_t pack_bf16_rne(float lo, float hi) {
  typedef __attribute__((ext_vector_type(2))) float f32x2_t;
  typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2_t;
  const f32x2_t x = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(x, bf16x2_t));
}

}  // namespace sdv2

#endif  // SDV2KV_INTERNAL_H
