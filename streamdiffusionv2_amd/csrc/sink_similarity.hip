// Adaptive sink refresh decision for gfx950.
//
// Stands in for models/wan/causal_model.py:284-299: per cache row, the mean
// over the tokens of every sink frame of the cached K and V is compared (cosine
// similarity over the flattened heads x 128 vector) with the mean of the
// incoming one-frame chunk's roped K and its V; the two similarities are
// averaged and, when the smallest falls below the threshold, that sink frame
// is to be overwritten next.  The reference does this with four reductions and
// two host round trips per row; here one reduction kernel produces every frame
// mean (rotating the new keys on the fly with the append kernel's arithmetic,
// so they never have to be staged) and a second, tiny kernel turns the means
// into similarities and the decision.  The caller reads back one int per row.
//
// Rounding follows the storage dtype: with bf16 tensors the frame means, the
// two cosine similarities and their sum are each rounded to bf16 (they are
// bf16 tensors in the reference); sums inside a reduction are fp32 in a fixed
// order, so results are deterministic.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "sdv2kv.h"
#include "sdv2kv_internal.h"
#include "rope_device.h"

namespace {

constexpr int kLanesPerRow = 16;            // 16 lanes x 8 elements = 128
constexpr int kTokenLanes = 16;             // 256 threads

struct SinkSimKernelArgs {
  const void* k_in;
  const void* v_in;
  const void* k_cache;
  const void* v_cache;
  sdv2_stride3 k_in_st, v_in_st, k_st, v_st;
  const double2* freqs;
  float* means;                             // [rows][2*sink+2][heads*128]
  float* similarity;                        // [rows][sink]
  int32_t* refresh;                         // [rows]
  int32_t tokens, heads, grid_w, sink_frames;
  int32_t split_t, split_h, pairs;
  float threshold;
  int64_t start_frame[SDV2_MAX_ROWS];
};

template <typename T>
__device__ __forceinline__ float round_to_storage(float x);
template <>
__device__ __forceinline__ float round_to_storage<uint16_t>(float x) {
  return sdv2::bf16_bits_to_f32(sdv2::f32_to_bf16_rne(x));
}
template <>
__device__ __forceinline__ float round_to_storage<float>(float x) { return x; }

// grid (heads, 2*sink+2, rows): one workgroup reduces one head's 128 columns
// of one frame over its tokens.
template <typename T>
__global__ __launch_bounds__(kLanesPerRow * kTokenLanes)
void sink_frame_mean_kernel(const SinkSimKernelArgs a) {
  __shared__ float part[kTokenLanes][kLanesPerRow * 8];
  const int lane = threadIdx.x & (kLanesPerRow - 1);
  const int tl = threadIdx.x >> 4;
  const int head = blockIdx.x;
  const int m = blockIdx.y;
  const int row = blockIdx.z;
  const int sink = a.sink_frames;

  const bool is_new = m >= 2 * sink;
  const bool is_k = is_new ? (m == 2 * sink) : (m < sink);
  const int frame = is_new ? 0 : (m < sink ? m : m - sink);
  const sdv2_stride3 st = is_new ? (is_k ? a.k_in_st : a.v_in_st) : (is_k ? a.k_st : a.v_st);
  const T* base = static_cast<const T*>(is_new ? (is_k ? a.k_in : a.v_in) : (is_k ? a.k_cache : a.v_cache));
  base += row * st.row + static_cast<int64_t>(frame) * a.tokens * st.token + head * st.head + lane * 8;

  float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  for (int t = tl; t < a.tokens; t += kTokenLanes) {
    sdv2::Vec8<T> x = sdv2::Vec8<T>::load(base + t * st.token);
    if (is_new && is_k) {
      const int hi = t / a.grid_w;
      const int wi = t - hi * a.grid_w;
      double2 cs[4];
      sdv2::load_rotation(a.freqs, a.pairs, a.split_t, a.split_h, lane, a.start_frame[row], hi, wi, cs);
      x = sdv2::rotate(x, cs);
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[i] += static_cast<float>(x.get(i));
  }
#pragma unroll
  for (int i = 0; i < 8; ++i) part[tl][lane * 8 + i] = acc[i];
  __syncthreads();
  if (threadIdx.x < kLanesPerRow * 8) {
    float s = 0.f;
#pragma unroll
    for (int j = 0; j < kTokenLanes; ++j) s += part[j][threadIdx.x];
    const float mean = round_to_storage<T>(s * (1.0f / static_cast<float>(a.tokens)));
    const int64_t width = static_cast<int64_t>(a.heads) * 128;
    a.means[(static_cast<int64_t>(row) * (2 * sink + 2) + m) * width + head * 128 + threadIdx.x] = mean;
  }
}

// sum over the workgroup in a fixed order; result valid in every thread
__device__ __forceinline__ float block_sum(float x, float* scratch) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) x += __shfl_xor(x, off, 64);
  __syncthreads();
  if ((threadIdx.x & 63) == 0) scratch[threadIdx.x >> 6] = x;
  __syncthreads();
  return (scratch[0] + scratch[1]) + (scratch[2] + scratch[3]);
}

// grid (rows): cosine similarities, their average, the decision.
template <typename T>
__global__ __launch_bounds__(256)
void sink_decide_kernel(const SinkSimKernelArgs a) {
  __shared__ float scratch[4];
  const int row = blockIdx.x;
  const int sink = a.sink_frames;
  const int width = a.heads * 128;
  const float* means = a.means + static_cast<int64_t>(row) * (2 * sink + 2) * width;
  const float* k_new = means + static_cast<int64_t>(2 * sink) * width;
  const float* v_new = k_new + width;
  constexpr float kEps = 1e-8f;             // torch.cosine_similarity default

  float kk = 0.f, vv = 0.f;
  for (int c = threadIdx.x; c < width; c += 256) {
    kk += k_new[c] * k_new[c];
    vv += v_new[c] * v_new[c];
  }
  const float k_new_norm = fmaxf(sqrtf(block_sum(kk, scratch)), kEps);
  const float v_new_norm = fmaxf(sqrtf(block_sum(vv, scratch)), kEps);

  float best = 0.f;
  int best_frame = -1;
  for (int j = 0; j < sink; ++j) {
    const float* ks = means + static_cast<int64_t>(j) * width;
    const float* vs = means + static_cast<int64_t>(sink + j) * width;
    float dk = 0.f, nk = 0.f, dv = 0.f, nv = 0.f;
    for (int c = threadIdx.x; c < width; c += 256) {
      dk += ks[c] * k_new[c];
      nk += ks[c] * ks[c];
      dv += vs[c] * v_new[c];
      nv += vs[c] * vs[c];
    }
    dk = block_sum(dk, scratch);
    nk = block_sum(nk, scratch);
    dv = block_sum(dv, scratch);
    nv = block_sum(nv, scratch);
    const float cos_k = round_to_storage<T>(dk / (fmaxf(sqrtf(nk), kEps) * k_new_norm));
    const float cos_v = round_to_storage<T>(dv / (fmaxf(sqrtf(nv), kEps) * v_new_norm));
    const float sim = round_to_storage<T>(cos_k + cos_v) * 0.5f;
    if (threadIdx.x == 0) a.similarity[row * sink + j] = sim;
    if (best_frame < 0 || sim < best) {       // first minimum, as torch.argmin
      best = sim;
      best_frame = j;
    }
  }
  if (threadIdx.x == 0) a.refresh[row] = best < round_to_storage<T>(a.threshold) ? best_frame : -1;
}

bool stride_ok(const sdv2_stride3& s, int vec) {
  return s.row % vec == 0 && s.token % vec == 0 && s.head % vec == 0;
}

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

}  // namespace

extern "C" size_t sdv2_sink_similarity_workspace_bytes(int32_t rows, int32_t heads, int32_t sink_frames) {
  if (rows <= 0 || heads <= 0 || sink_frames <= 0) return 0;
  return static_cast<size_t>(rows) * (2 * static_cast<size_t>(sink_frames) + 2) * heads * SDV2_HEAD_DIM * sizeof(float);
}

extern "C" int sdv2_sink_similarity(const sdv2_sink_sim_params* p) {
  if (!p) return SDV2_ERR_INVALID_ARG;
  if (p->head_dim != SDV2_HEAD_DIM) return SDV2_ERR_UNSUPPORTED;
  if (p->dtype != SDV2_BF16 && p->dtype != SDV2_F32) return SDV2_ERR_UNSUPPORTED;
  if (p->rows <= 0 || p->rows > SDV2_MAX_ROWS || p->heads <= 0) return SDV2_ERR_INVALID_ARG;
  if (p->sink_frames <= 0 || p->sink_frames > SDV2_MAX_SINK_FRAMES) return SDV2_ERR_INVALID_ARG;
  if (p->grid_h <= 0 || p->grid_w <= 0) return SDV2_ERR_INVALID_ARG;
  // the reference's reshape(1, frame_seqlen, -1) only holds for a one-frame chunk
  if (p->tokens != p->grid_h * p->grid_w) return SDV2_ERR_INVALID_ARG;
  if (!p->k_in || !p->v_in || !p->k_cache || !p->v_cache || !p->freqs || !p->start_frame)
    return SDV2_ERR_INVALID_ARG;
  if (!p->similarity || !p->refresh) return SDV2_ERR_INVALID_ARG;
  if (static_cast<int64_t>(p->sink_frames) * p->tokens > p->cache_tokens) return SDV2_ERR_OUT_OF_RANGE;
  const int vec = p->dtype == SDV2_BF16 ? 8 : 4;
  const void* ptrs[] = {p->k_in, p->v_in, p->k_cache, p->v_cache};
  for (const void* ptr : ptrs)
    if (!aligned16(ptr)) return SDV2_ERR_INVALID_ARG;
  if (!stride_ok(p->k_in_stride, vec) || !stride_ok(p->v_in_stride, vec) ||
      !stride_ok(p->k_cache_stride, vec) || !stride_ok(p->v_cache_stride, vec))
    return SDV2_ERR_INVALID_ARG;
  if (p->grid_h > p->freq_rows || p->grid_w > p->freq_rows) return SDV2_ERR_OUT_OF_RANGE;
  for (int i = 0; i < p->rows; ++i)
    if (p->start_frame[i] < 0 || p->start_frame[i] >= p->freq_rows) return SDV2_ERR_OUT_OF_RANGE;
  const size_t need = sdv2_sink_similarity_workspace_bytes(p->rows, p->heads, p->sink_frames);
  if (!p->workspace || p->workspace_bytes < need || (reinterpret_cast<uintptr_t>(p->workspace) & 15))
    return SDV2_ERR_WORKSPACE;

  SinkSimKernelArgs a{};
  a.k_in = p->k_in; a.v_in = p->v_in; a.k_cache = p->k_cache; a.v_cache = p->v_cache;
  a.k_in_st = p->k_in_stride; a.v_in_st = p->v_in_stride; a.k_st = p->k_cache_stride; a.v_st = p->v_cache_stride;
  a.freqs = reinterpret_cast<const double2*>(p->freqs);
  a.means = static_cast<float*>(p->workspace);
  a.similarity = p->similarity;
  a.refresh = p->refresh;
  a.tokens = p->tokens; a.heads = p->heads; a.grid_w = p->grid_w; a.sink_frames = p->sink_frames;
  a.pairs = p->head_dim / 2;
  const int third = a.pairs / 3;
  a.split_t = a.pairs - 2 * third;
  a.split_h = a.split_t + third;
  a.threshold = p->threshold;
  for (int i = 0; i < p->rows; ++i) a.start_frame[i] = p->start_frame[i];

  hipStream_t stream = static_cast<hipStream_t>(p->stream);
  const dim3 block(kLanesPerRow * kTokenLanes);
  const dim3 grid_mean(p->heads, 2 * p->sink_frames + 2, p->rows);
  const dim3 grid_decide(p->rows);
  if (p->dtype == SDV2_BF16) {
    hipLaunchKernelGGL(sink_frame_mean_kernel<uint16_t>, grid_mean, block, 0, stream, a);
    hipLaunchKernelGGL(sink_decide_kernel<uint16_t>, grid_decide, dim3(256), 0, stream, a);
  } else {
    hipLaunchKernelGGL(sink_frame_mean_kernel<float>, grid_mean, block, 0, stream, a);
    hipLaunchKernelGGL(sink_decide_kernel<float>, grid_decide, dim3(256), 0, stream, a);
  }
  return hipGetLastError() == hipSuccess ? SDV2_OK : SDV2_ERR_LAUNCH;
}
