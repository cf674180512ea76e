// Attention of a chunk's queries against an fp32 ring KV cache, computed in
// fp32 throughout, for gfx950 (MI355X).
//
// Stands in for what the reference computes on fp32 tensors at
// models/wan/causal_model.py:111-157 (attention_with_kvcache_fallback: scaled
// dot product attention of q against k_cache[:, :seq_len], no mask inside the
// chunk) - the configuration the reference itself can run on a CPU.  This is a
// plumbing mode, not the performance path: the bf16 kernel in swa_attn_fwd.hip
// is the one that runs on the matrix cores.  Here products and sums are plain
// fp32 fused multiply-adds, the softmax keeps a running maximum per query row,
// and nothing is rounded below fp32 anywhere.
//
// Work decomposition: workgroup = 256 threads = 64 query rows of one (row,
// head); keys stream through LDS 32 at a time.  Thread (ty, tx) = (tid / 16,
// tid % 16) owns query rows 4 ty .. 4 ty + 3; of a key tile's scores it
// computes keys tx and tx + 16 for those rows, of the output the eight dims
// 8 tx .. 8 tx + 7.  The sixteen threads that share a query row are sixteen
// neighbouring lanes of one wave, so row maxima and row sums are wave shuffles.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>

#include "sdv2kv.h"
#include "sdv2kv_profile.h"
#include "sdv2kv_internal.h"

namespace {

constexpr int kD = SDV2_HEAD_DIM;     // 128
constexpr int kRows = 64;             // query rows per workgroup
constexpr int kKeys = 32;             // keys per tile
constexpr int kThreads = 256;
constexpr int kQStride = kD + 4;      // floats per Q / K row in LDS: rows stay 16-byte aligned and start 4 banks apart
constexpr int kPStride = kKeys + 4;
constexpr int kLdsFloats = kRows * kQStride + kKeys * kQStride + kKeys * kD + kRows * kPStride;
constexpr int kMaxDevices = 64;

struct AttnF32Args {
  const float* q;
  const float* k;
  const float* v;
  float* out;
  const int32_t* seq_lens;
  sdv2_stride3 q_st, k_st, v_st, o_st;
  int32_t rows, q_tokens, heads, max_seq_len;
  float scale;
  int32_t mask_block_tokens;
  const int32_t* chunk_start;
};

__device__ __forceinline__ float dot4(const float4& a, const float4& b, float acc) {
  acc = __builtin_fmaf(a.x, b.x, acc);
  acc = __builtin_fmaf(a.y, b.y, acc);
  acc = __builtin_fmaf(a.z, b.z, acc);
  return __builtin_fmaf(a.w, b.w, acc);
}

// over the sixteen lanes that share a query row
__device__ __forceinline__ float row_max(float x) {
#pragma unroll
  for (int off = 8; off > 0; off >>= 1) x = fmaxf(x, __shfl_xor(x, off, 16));
  return x;
}
__device__ __forceinline__ float row_sum(float x) {
#pragma unroll
  for (int off = 8; off > 0; off >>= 1) x += __shfl_xor(x, off, 16);
  return x;
}

__global__ __launch_bounds__(kThreads)
void swa_attn_fwd_f32_kernel(const AttnF32Args a) {
  extern __shared__ __attribute__((aligned(16))) float lds_f32[];
  float* q_s = lds_f32;                         // [kRows][kQStride]
  float* k_s = q_s + kRows * kQStride;          // [kKeys][kQStride]
  float* v_s = k_s + kKeys * kQStride;          // [kKeys][kD]
  float* p_s = v_s + kKeys * kD;                // [kRows][kPStride]

  const int tid = threadIdx.x;
  const int ty = tid >> 4, tx = tid & 15;
  const int q0 = blockIdx.x * kRows;
  const int head = blockIdx.y;
  const int row = blockIdx.z;

  int seq = a.seq_lens ? a.seq_lens[row] : a.max_seq_len;
  seq = seq < a.max_seq_len ? seq : a.max_seq_len;
  seq = seq < 0 ? 0 : seq;

  // the chunk's own later blocks, hidden from a query when the mask inside the chunk is on
  int m_lo[4], m_hi = 0;
#pragma unroll
  for (int i = 0; i < 4; ++i) m_lo[i] = 0x7fffffff;
  if (a.mask_block_tokens > 0) {
    const int first = a.chunk_start[row];
    m_hi = first + a.q_tokens;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int t = q0 + 4 * ty + i;
      m_lo[i] = first + (t / a.mask_block_tokens + 1) * a.mask_block_tokens;
    }
  }

  // the query tile (rows past the last query repeat it; their results are not stored)
  {
    const float* qp = a.q + row * a.q_st.row + head * a.q_st.head;
#pragma unroll
    for (int n = 0; n < kRows * (kD / 4) / kThreads; ++n) {
      const int idx = tid + n * kThreads;
      const int r = idx >> 5, c4 = idx & 31;
      int t = q0 + r;
      t = t < a.q_tokens ? t : a.q_tokens - 1;
      *reinterpret_cast<float4*>(q_s + r * kQStride + 4 * c4) =
          *reinterpret_cast<const float4*>(qp + (int64_t)t * a.q_st.token + 4 * c4);
    }
  }

  float o[4][8];
  float m_run[4], l_run[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    m_run[i] = -INFINITY;
    l_run[i] = 0.f;           // this thread's share of the row sum
#pragma unroll
    for (int e = 0; e < 8; ++e) o[i][e] = 0.f;
  }

  const float* kp = a.k + row * a.k_st.row + head * a.k_st.head;
  const float* vp = a.v + row * a.v_st.row + head * a.v_st.head;
  for (int key0 = 0; key0 < seq; key0 += kKeys) {
    __syncthreads();          // the previous tile has been read by everyone (and the query tile written)
#pragma unroll
    for (int n = 0; n < kKeys * (kD / 4) / kThreads; ++n) {
      const int idx = tid + n * kThreads;
      const int r = idx >> 5, c4 = idx & 31;
      int key = key0 + r;
      key = key < seq ? key : seq - 1;        // rows past the valid length repeat the last valid key; their scores are masked
      *reinterpret_cast<float4*>(k_s + r * kQStride + 4 * c4) =
          *reinterpret_cast<const float4*>(kp + (int64_t)key * a.k_st.token + 4 * c4);
      *reinterpret_cast<float4*>(v_s + r * kD + 4 * c4) =
          *reinterpret_cast<const float4*>(vp + (int64_t)key * a.v_st.token + 4 * c4);
    }
    __syncthreads();

    float s[4][2];
#pragma unroll
    for (int i = 0; i < 4; ++i) s[i][0] = s[i][1] = 0.f;
#pragma unroll 4
    for (int d4 = 0; d4 < kD / 4; ++d4) {
      float4 qv[4], kv[2];
#pragma unroll
      for (int i = 0; i < 4; ++i) qv[i] = *reinterpret_cast<const float4*>(q_s + (4 * ty + i) * kQStride + 4 * d4);
#pragma unroll
      for (int j = 0; j < 2; ++j) kv[j] = *reinterpret_cast<const float4*>(k_s + (tx + 16 * j) * kQStride + 4 * d4);
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) s[i][j] = dot4(qv[i], kv[j], s[i][j]);
    }

#pragma unroll
    for (int i = 0; i < 4; ++i) {
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        const int key = key0 + tx + 16 * j;
        const bool hidden = key >= seq || (key >= m_lo[i] && key < m_hi);
        s[i][j] = hidden ? -INFINITY : s[i][j] * a.scale;
      }
      const float m_tile = row_max(fmaxf(s[i][0], s[i][1]));
      const float m_new = fmaxf(m_run[i], m_tile);
      // -inf only while every key so far was hidden from this query: nothing has been summed yet
      const float alpha = m_new == -INFINITY ? 1.0f : expf(m_run[i] - m_new);
      const float p0 = m_new == -INFINITY ? 0.f : expf(s[i][0] - m_new);
      const float p1 = m_new == -INFINITY ? 0.f : expf(s[i][1] - m_new);
      m_run[i] = m_new;
      l_run[i] = l_run[i] * alpha + (p0 + p1);
#pragma unroll
      for (int e = 0; e < 8; ++e) o[i][e] *= alpha;
      p_s[(4 * ty + i) * kPStride + tx] = p0;
      p_s[(4 * ty + i) * kPStride + tx + 16] = p1;
    }
    __syncthreads();

#pragma unroll 2
    for (int k4 = 0; k4 < kKeys / 4; ++k4) {
      float4 pv[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) pv[i] = *reinterpret_cast<const float4*>(p_s + (4 * ty + i) * kPStride + 4 * k4);
#pragma unroll
      for (int kk = 0; kk < 4; ++kk) {
        const float4 v0 = *reinterpret_cast<const float4*>(v_s + (4 * k4 + kk) * kD + 8 * tx);
        const float4 v1 = *reinterpret_cast<const float4*>(v_s + (4 * k4 + kk) * kD + 8 * tx + 4);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const float p = kk == 0 ? pv[i].x : (kk == 1 ? pv[i].y : (kk == 2 ? pv[i].z : pv[i].w));
          o[i][0] = __builtin_fmaf(p, v0.x, o[i][0]);
          o[i][1] = __builtin_fmaf(p, v0.y, o[i][1]);
          o[i][2] = __builtin_fmaf(p, v0.z, o[i][2]);
          o[i][3] = __builtin_fmaf(p, v0.w, o[i][3]);
          o[i][4] = __builtin_fmaf(p, v1.x, o[i][4]);
          o[i][5] = __builtin_fmaf(p, v1.y, o[i][5]);
          o[i][6] = __builtin_fmaf(p, v1.z, o[i][6]);
          o[i][7] = __builtin_fmaf(p, v1.w, o[i][7]);
        }
      }
    }
  }

  float* op = a.out + row * a.o_st.row + head * a.o_st.head + 8 * tx;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int t = q0 + 4 * ty + i;
    const float l = row_sum(l_run[i]);
    const float inv = l > 0.f ? 1.0f / l : 0.f;       // no visible key: zeros, as the bf16 kernel writes
    if (t < a.q_tokens) {
      float4 w0 = {o[i][0] * inv, o[i][1] * inv, o[i][2] * inv, o[i][3] * inv};
      float4 w1 = {o[i][4] * inv, o[i][5] * inv, o[i][6] * inv, o[i][7] * inv};
      *reinterpret_cast<float4*>(op + (int64_t)t * a.o_st.token) = w0;
      *reinterpret_cast<float4*>(op + (int64_t)t * a.o_st.token + 4) = w1;
    }
  }
}

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }
bool stride_ok(const sdv2_stride3& s) { return s.row % 4 == 0 && s.token % 4 == 0 && s.head % 4 == 0; }

}  // namespace

int sdv2::attn_fwd_f32(const sdv2_attn_params* p) {
  if (p->head_dim != kD) return SDV2_ERR_UNSUPPORTED;
  if (p->rows < 0 || p->q_tokens < 0 || p->heads <= 0 || p->max_seq_len < 0) return SDV2_ERR_INVALID_ARG;
  if (p->rows == 0 || p->q_tokens == 0) return SDV2_OK;
  if (!p->q || !p->k_cache || !p->v_cache || !p->out) return SDV2_ERR_INVALID_ARG;
  if (!aligned16(p->q) || !aligned16(p->k_cache) || !aligned16(p->v_cache) || !aligned16(p->out))
    return SDV2_ERR_INVALID_ARG;
  if (!stride_ok(p->q_stride) || !stride_ok(p->k_stride) || !stride_ok(p->v_stride) || !stride_ok(p->out_stride))
    return SDV2_ERR_INVALID_ARG;
  if (p->rows > 65535 || p->heads > 65535) return SDV2_ERR_INVALID_ARG;
  if (p->rope_freqs || p->q_norm_weight || p->q_inv_rms)
    return SDV2_ERR_UNSUPPORTED;                        // fp32 queries arrive normalised and rotated (the append returns them)
  if (p->mask_block_tokens < 0) return SDV2_ERR_INVALID_ARG;

  AttnF32Args a{};
  a.q = static_cast<const float*>(p->q);
  a.k = static_cast<const float*>(p->k_cache);
  a.v = static_cast<const float*>(p->v_cache);
  a.out = static_cast<float*>(p->out);
  a.seq_lens = p->seq_lens;
  a.q_st = p->q_stride; a.k_st = p->k_stride; a.v_st = p->v_stride; a.o_st = p->out_stride;
  a.rows = p->rows; a.q_tokens = p->q_tokens; a.heads = p->heads; a.max_seq_len = p->max_seq_len;
  a.scale = p->softmax_scale > 0.f ? p->softmax_scale : 0.08838834764831845f;  // 1/sqrt(128)
  if (p->mask_block_tokens > 0 && p->mask_block_tokens < p->q_tokens) {
    if (!p->chunk_key_start) return SDV2_ERR_INVALID_ARG;
    a.chunk_start = p->chunk_key_start;
    a.mask_block_tokens = p->mask_block_tokens;
  }

  static std::atomic<bool> lds_ready[kMaxDevices];
  int device = 0;
  if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= kMaxDevices) return SDV2_ERR_LAUNCH;
  constexpr uint32_t lds_bytes = kLdsFloats * sizeof(float);
  if (!lds_ready[device].load(std::memory_order_acquire)) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(swa_attn_fwd_f32_kernel),
                            hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes) != hipSuccess)
      return SDV2_ERR_LAUNCH;
    lds_ready[device].store(true, std::memory_order_release);
  }
  const dim3 grid((unsigned)((p->q_tokens + kRows - 1) / kRows), (unsigned)p->heads, (unsigned)p->rows);
  sdv2::launch_timed(SDV2_KERNEL_ATTENTION, swa_attn_fwd_f32_kernel, grid, dim3(kThreads), lds_bytes,
                     static_cast<hipStream_t>(p->stream), a);
  if (hipGetLastError() != hipSuccess) return SDV2_ERR_LAUNCH;
  return SDV2_OK;
}
