// Small entry points of the sdv2kv C ABI that are not kernels of the path
// itself: version, status strings, timing events and the counter-calibration copy.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "sdv2kv.h"
#include "sdv2kv_profile.h"
#include "sdv2kv_internal.h"

namespace {

thread_local sdv2::TimingPair armed[SDV2_KERNEL_COUNT];

struct CopyArgs {
  uint4* dst;
  const uint4* src;
  size_t n16;
};

__global__ __launch_bounds__(256) void copy16_kernel(const CopyArgs a) {
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < a.n16; i += stride) a.dst[i] = a.src[i];
}

}  // namespace

sdv2::TimingPair sdv2::take_timing(int kernel) {
  if (kernel < 0 || kernel >= SDV2_KERNEL_COUNT) return {nullptr, nullptr};
  const TimingPair t = armed[kernel];
  armed[kernel] = {nullptr, nullptr};
  return t;
}

extern "C" int sdv2_profile_time_next(int kernel, void* start, void* stop) {
  if (kernel < 0 || kernel >= SDV2_KERNEL_COUNT) return SDV2_ERR_INVALID_ARG;
  if ((start == nullptr) != (stop == nullptr)) return SDV2_ERR_INVALID_ARG;
  armed[kernel] = {start, stop};
  return SDV2_OK;
}

extern "C" int sdv2_abi_version(void) { return SDV2KV_ABI_VERSION; }

extern "C" const char* sdv2_status_string(int status) {
  switch (status) {
    case SDV2_OK: return "ok";
    case SDV2_ERR_INVALID_ARG: return "invalid argument (null pointer, bad shape, misaligned pointer or stride)";
    case SDV2_ERR_UNSUPPORTED: return "unsupported head_dim or dtype";
    case SDV2_ERR_OUT_OF_RANGE: return "write range outside the cache or RoPE position beyond the table";
    case SDV2_ERR_WORKSPACE: return "split-KV workspace missing or too small";
    case SDV2_ERR_LAUNCH: return "kernel launch failed";
    case SDV2_ERR_SCRATCH_LIMIT: return "the call needs more split-KV scratch than the library's static buffer holds";
    default: return "unknown status";
  }
}

extern "C" int sdv2_event_create(void** event) {
  if (!event) return SDV2_ERR_INVALID_ARG;
  hipEvent_t e = nullptr;
  if (hipEventCreate(&e) != hipSuccess) return SDV2_ERR_LAUNCH;
  *event = e;
  return SDV2_OK;
}

extern "C" int sdv2_event_destroy(void* event) {
  if (!event) return SDV2_OK;
  return hipEventDestroy(static_cast<hipEvent_t>(event)) == hipSuccess ? SDV2_OK : SDV2_ERR_INVALID_ARG;
}

extern "C" int sdv2_event_elapsed_ms(void* start, void* stop, float* ms) {
  if (!start || !stop || !ms) return SDV2_ERR_INVALID_ARG;
  if (hipEventSynchronize(static_cast<hipEvent_t>(stop)) != hipSuccess) return SDV2_ERR_LAUNCH;
  return hipEventElapsedTime(ms, static_cast<hipEvent_t>(start), static_cast<hipEvent_t>(stop)) == hipSuccess
             ? SDV2_OK
             : SDV2_ERR_INVALID_ARG;
}

extern "C" int sdv2_copy_bytes(void* dst, const void* src, size_t bytes, void* stream) {
  if (bytes == 0) return SDV2_OK;
  if (!dst || !src) return SDV2_ERR_INVALID_ARG;
  if ((reinterpret_cast<uintptr_t>(dst) | reinterpret_cast<uintptr_t>(src) | bytes) & 15) return SDV2_ERR_INVALID_ARG;
  const size_t n16 = bytes / 16;
  size_t blocks = (n16 + 255) / 256;
  if (blocks > 256 * 32) blocks = 256 * 32;
  const CopyArgs args{static_cast<uint4*>(dst), static_cast<const uint4*>(src), n16};
  sdv2::launch_timed(SDV2_KERNEL_COPY, copy16_kernel, dim3((unsigned)blocks), dim3(256), 0,
                     static_cast<hipStream_t>(stream), args);
  return hipGetLastError() == hipSuccess ? SDV2_OK : SDV2_ERR_LAUNCH;
}
