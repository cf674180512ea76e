// WanRMSNorm over the full model width for gfx950.
//
// Stands in for WanRMSNorm.forward (models/wan/wan_base/modules/model.py:77-86)
// where it runs as a module of its own - the query norm of the text
// cross-attention (model.py:181) and the q / k norms of the self-attention when
// they are not folded into the append:
//   y = type_as(float(x) * rsqrt(mean(float(x)^2) + eps)) * weight
// One launch instead of the seven elementwise and reduction kernels the torch
// expression turns into.  One wave per token: the token's row stays in
// registers between the sum of squares and the write.  The fp32 sum of squares
// is taken in the order of PyTorch's CPU sum kernel (sdv2::wave_sum_squares), so
// the result is bit for bit what the torch module gives on the CPU, and what
// the append kernel with the norm folded in computes for the same row.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

#include "sdv2kv.h"
#include "sdv2kv_profile.h"
#include "sdv2kv_internal.h"
#include "rope_device.h"

namespace {

constexpr int kWavesPerGroup = 4;
constexpr int kMaxSteps = 16;               // 4 heads of 128 per step: widths up to 64 * 128

struct NormKernelArgs {
  const void* x;
  void* out;
  const void* weight;
  int64_t x_stride, out_stride;             // elements between tokens
  int64_t tokens;
  int32_t heads;                            // width / 128
  float eps;
};

// grid (ceil(tokens / 4)), 256 threads: wave w of a workgroup takes token 4 * blockIdx.x + w.
// Lane l holds, per step j, the 8-element slice l % 16 of the 128-element group 4 j + l / 16.
template <typename T, int kSteps>
__global__ __launch_bounds__(kWavesPerGroup * 64)
void rms_norm_kernel(const NormKernelArgs a) {
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int64_t tok = static_cast<int64_t>(blockIdx.x) * kWavesPerGroup + wave;
  __shared__ float squares[kWavesPerGroup][2][64 * 8];
  if (tok >= a.tokens) return;
  const T* xi = static_cast<const T*>(a.x) + tok * a.x_stride + (lane & 15) * 8;
  sdv2::Vec8<T> x[kSteps];
#pragma unroll
  for (int j = 0; j < kSteps; ++j) {
    const int h = 4 * j + (lane >> 4);
    x[j] = 4 * j < a.heads && h < a.heads ? sdv2::Vec8<T>::load(xi + h * 128) : sdv2::Vec8<T>::zero();
  }
  // (the weight's slices ride along with the row: they are needed only after the sum)
  sdv2::Vec8<T> w[kSteps];
  const T* wi = static_cast<const T*>(a.weight) + (lane & 15) * 8;
#pragma unroll
  for (int j = 0; j < kSteps; ++j) {
    const int h = 4 * j + (lane >> 4);
    w[j] = 4 * j < a.heads && h < a.heads ? sdv2::Vec8<T>::load(wi + h * 128) : sdv2::Vec8<T>::zero();
  }
  float ssq, same;
  sdv2::wave_sum_squares<T, kSteps>(x, x, a.heads, squares[wave], lane, ssq, same);
  const float r = 1.0f / sqrtf(ssq / static_cast<float>(a.heads * 128) + a.eps);
  T* oi = static_cast<T*>(a.out) + tok * a.out_stride + (lane & 15) * 8;
#pragma unroll
  for (int j = 0; j < kSteps; ++j) {
    const int h = 4 * j + (lane >> 4);
    if (4 * j < a.heads && h < a.heads) sdv2::normalise(x[j], r, w[j]).store(oi + h * 128);
  }
}

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

}  // namespace

extern "C" int sdv2_rms_norm(const sdv2_rms_norm_params* p) {
  if (!p) return SDV2_ERR_INVALID_ARG;
  if (p->dtype != SDV2_BF16 && p->dtype != SDV2_F32) return SDV2_ERR_UNSUPPORTED;
  if (p->tokens < 0 || p->width <= 0) return SDV2_ERR_INVALID_ARG;
  if (p->width % SDV2_HEAD_DIM != 0 || p->width / SDV2_HEAD_DIM > 4 * kMaxSteps) return SDV2_ERR_UNSUPPORTED;
  if (p->tokens == 0) return SDV2_OK;
  if (p->tokens > (static_cast<int64_t>(1) << 31) - 8) return SDV2_ERR_UNSUPPORTED;
  if (!p->x || !p->out || !p->weight) return SDV2_ERR_INVALID_ARG;
  if (!(p->eps >= 0.f)) return SDV2_ERR_INVALID_ARG;
  // 16-byte vector access: 8 bf16 or 4 floats per transaction
  const int vec = p->dtype == SDV2_BF16 ? 8 : 4;
  if (!aligned16(p->x) || !aligned16(p->out) || !aligned16(p->weight)) return SDV2_ERR_INVALID_ARG;
  if (p->x_token_stride < p->width || p->out_token_stride < p->width) return SDV2_ERR_INVALID_ARG;
  if (p->x_token_stride % vec != 0 || p->out_token_stride % vec != 0) return SDV2_ERR_INVALID_ARG;

  NormKernelArgs a{};
  a.x = p->x; a.out = p->out; a.weight = p->weight;
  a.x_stride = p->x_token_stride; a.out_stride = p->out_token_stride;
  a.tokens = p->tokens;
  a.heads = p->width / SDV2_HEAD_DIM;
  a.eps = p->eps;
  hipStream_t stream = static_cast<hipStream_t>(p->stream);
  const dim3 grid(static_cast<uint32_t>((p->tokens + kWavesPerGroup - 1) / kWavesPerGroup));
  const dim3 block(kWavesPerGroup * 64);
  const int steps = (a.heads + 3) / 4;
  auto launch = [&](auto steps_c) {
    constexpr int kS = decltype(steps_c)::value;
    if (p->dtype == SDV2_BF16) sdv2::launch_timed(SDV2_KERNEL_NORM, rms_norm_kernel<uint16_t, kS>, grid, block, 0, stream, a);
    else sdv2::launch_timed(SDV2_KERNEL_NORM, rms_norm_kernel<float, kS>, grid, block, 0, stream, a);
  };
  if (steps <= 3) launch(std::integral_constant<int, 3>{});
  else if (steps <= 10) launch(std::integral_constant<int, 10>{});
  else launch(std::integral_constant<int, kMaxSteps>{});
  return hipGetLastError() == hipSuccess ? SDV2_OK : SDV2_ERR_LAUNCH;
}
