// Layout-changing copy of one layer's cache block, for the hand-off of a
// block between owners.
//
// The reference moves a block by broadcasting kv_cache1[i]["k"], ["v"] and the
// two index tensors from the donor and then shifting the receiver's
// global_end_index (streamv2v/communication/kv_cache_manager.py:66-82).  Its
// tensors are token-major [B, cap, H, 128]; this library keeps a cache
// head-major in HBM.  The wire format stays the reference's, so a block goes
// through this kernel once on either side: head-major -> token-major
// contiguous before it is sent, back after it was received, with the index
// update folded into the second copy (no host round trip for the indices).
//
// HBM-bound: every byte is read once and written once.  A thread moves 16
// bytes; the 16 (bf16) or 32 (fp32) threads of one (token, head) cover its 128
// elements, so either side is touched in whole 256 / 512-byte runs whatever
// the two stride sets are.  Four independent vectors per thread are in flight.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "sdv2kv.h"
#include "sdv2kv_profile.h"
#include "sdv2kv_internal.h"

namespace {

constexpr int kThreads = 256;
constexpr int kVecsPerThread = 4;

struct RelayoutArgs {
  const char* src;
  char* dst;
  int64_t src_row, src_token, src_head;     // byte strides
  int64_t dst_row, dst_token, dst_head;
  int64_t tokens;
  int32_t heads;
  int32_t vec_shift;                         // log2(16-byte vectors per (token, head)): 4 bf16, 5 fp32
  const int64_t* src_global;
  const int64_t* src_local;
  int64_t* dst_global;
  int64_t* dst_local;
  int64_t global_shift;
};

__global__ __launch_bounds__(kThreads) void cache_relayout_kernel(const RelayoutArgs a) {
  const int row = blockIdx.y;
  if (blockIdx.x == 0 && threadIdx.x == 0) {
    if (a.dst_global) a.dst_global[row] = a.src_global[row] + a.global_shift;
    if (a.dst_local) a.dst_local[row] = a.src_local[row];
  }
  const int64_t per_token = (int64_t)a.heads << a.vec_shift;
  const int64_t total = a.tokens * per_token;
  const int64_t base = (int64_t)blockIdx.x * (kThreads * kVecsPerThread) + threadIdx.x;
  uint4 val[kVecsPerThread];
  int64_t dst_off[kVecsPerThread];
#pragma unroll
  for (int j = 0; j < kVecsPerThread; ++j) {
    const int64_t i = base + j * kThreads;
    if (i < total) {
      const int64_t tok = i / per_token;
      const int rem = (int)(i - tok * per_token);
      const int head = rem >> a.vec_shift;
      const int c = rem & ((1 << a.vec_shift) - 1);
      val[j] = *reinterpret_cast<const uint4*>(a.src + row * a.src_row + tok * a.src_token + head * a.src_head + c * 16);
      dst_off[j] = row * a.dst_row + tok * a.dst_token + head * a.dst_head + c * 16;
    }
  }
#pragma unroll
  for (int j = 0; j < kVecsPerThread; ++j)
    if (base + j * kThreads < total) *reinterpret_cast<uint4*>(a.dst + dst_off[j]) = val[j];
}

bool stride_ok(const sdv2_stride3& s, int64_t elem) {
  // 16-byte vectors: every stride a multiple of 16 bytes
  return ((s.row * elem) % 16 == 0) && ((s.token * elem) % 16 == 0) && ((s.head * elem) % 16 == 0) && s.row >= 0 &&
         s.token >= 0 && s.head >= 0;
}

}  // namespace

extern "C" int sdv2_cache_relayout(const sdv2_relayout_params* p) {
  if (!p) return SDV2_ERR_INVALID_ARG;
  if (p->head_dim != SDV2_HEAD_DIM) return SDV2_ERR_UNSUPPORTED;
  if (p->dtype != SDV2_BF16 && p->dtype != SDV2_F32) return SDV2_ERR_UNSUPPORTED;
  if (p->rows < 0 || p->tokens < 0 || p->heads < 0 || p->rows > 65535) return SDV2_ERR_INVALID_ARG;
  const bool with_idx = p->dst_global_end_index || p->dst_local_end_index;
  if ((p->dst_global_end_index && !p->src_global_end_index) || (p->dst_local_end_index && !p->src_local_end_index))
    return SDV2_ERR_INVALID_ARG;
  if (p->rows == 0) return SDV2_OK;
  const int64_t elem = p->dtype == SDV2_BF16 ? 2 : 4;
  const bool with_data = p->tokens > 0 && p->heads > 0;
  if (with_data) {
    if (!p->src || !p->dst) return SDV2_ERR_INVALID_ARG;
    if ((reinterpret_cast<uintptr_t>(p->src) | reinterpret_cast<uintptr_t>(p->dst)) & 15) return SDV2_ERR_INVALID_ARG;
    if (!stride_ok(p->src_stride, elem) || !stride_ok(p->dst_stride, elem)) return SDV2_ERR_INVALID_ARG;
    // distinct (token, head) elements of the destination must not overlap
    if (p->dst_stride.token < SDV2_HEAD_DIM && p->tokens > 1) return SDV2_ERR_INVALID_ARG;
    if (p->dst_stride.head < SDV2_HEAD_DIM && p->heads > 1) return SDV2_ERR_INVALID_ARG;
    if (p->dst_stride.row == 0 && p->rows > 1) return SDV2_ERR_INVALID_ARG;
  } else if (!with_idx) {
    return SDV2_OK;
  }
  RelayoutArgs a;
  a.src = static_cast<const char*>(p->src);
  a.dst = static_cast<char*>(p->dst);
  a.src_row = p->src_stride.row * elem;
  a.src_token = p->src_stride.token * elem;
  a.src_head = p->src_stride.head * elem;
  a.dst_row = p->dst_stride.row * elem;
  a.dst_token = p->dst_stride.token * elem;
  a.dst_head = p->dst_stride.head * elem;
  a.tokens = with_data ? p->tokens : 0;
  a.heads = p->heads;
  a.vec_shift = p->dtype == SDV2_BF16 ? 4 : 5;
  a.src_global = p->src_global_end_index;
  a.src_local = p->src_local_end_index;
  a.dst_global = p->dst_global_end_index;
  a.dst_local = p->dst_local_end_index;
  a.global_shift = p->global_end_shift;
  const int64_t total = a.tokens * ((int64_t)a.heads << a.vec_shift);
  int64_t blocks = (total + kThreads * kVecsPerThread - 1) / (kThreads * kVecsPerThread);
  if (blocks < 1) blocks = 1;
  if (blocks > 0x7fffffff) return SDV2_ERR_INVALID_ARG;
  sdv2::launch_timed(SDV2_KERNEL_RELAYOUT, cache_relayout_kernel, dim3((unsigned)blocks, (unsigned)p->rows),
                     dim3(kThreads), 0, static_cast<hipStream_t>(p->stream), a);
  return hipGetLastError() == hipSuccess ? SDV2_OK : SDV2_ERR_LAUNCH;
}
