// Fused RoPE-on-write chunk append for gfx950.
//
// One launch per transformer layer rotates the chunk's Q and K in IEEE double
// (no fused multiply-add), rounds double -> float (-> bf16 nearest-even),
// scatters K' and V into the ring slot chosen by the host state machine and
// stores the two int64 end indices.  It stands in for causal_rope_apply x2
// plus the per-row slice writes and index fills of
// models/wan/causal_model.py:253-266, 321-322, 336-342.
//
// The kernel is a pure stream: 16-byte loads and stores, 16 lanes per
// 256-byte head row, two heads per thread so the four table entries a
// lane needs are fetched once and reused.  Algorithmic traffic per launch is
// 6*B*S*H*128*sizeof(T) bytes (read q,k,v; write q', k', v).
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

#include "sdv2kv.h"
#include "sdv2kv_profile.h"
#include "sdv2kv_internal.h"
#include "rope_device.h"

namespace {

constexpr int kLanesPerRow = 16;            // 16 lanes x 8 elements = 128
constexpr int kTokensPerBlock = 16;         // 256 threads
constexpr int kHeadsPerThread = 2;        // measured best of 1 / 2 / 4 at every workload size

struct AppendKernelArgs {
  const void* q_in;
  const void* k_in;
  const void* v_in;
  void* q_out;
  void* k_cache;
  void* v_cache;
  sdv2_stride3 q_in_st, k_in_st, v_in_st, q_out_st, k_st, v_st;
  const double2* freqs;
  const void* q_norm_w;                     // RMSNorm weights over heads * 128, or null
  const void* k_norm_w;
  float norm_eps;
  int64_t* global_end;
  int64_t* local_end;
  const int64_t* dst_override;              // device [rows] or null; a value >= 0 replaces dst_start[row]
  float* q_inv_rms;                         // device [rows][tokens] or null: 1 / rms of every q token (fused norm)
  int64_t cache_tokens;
  int32_t tokens, heads, grid_w, frame_tokens;
  int32_t split_t, split_h;                 // pair index bounds: [0,split_t) temporal, [split_t,split_h) height
  int32_t pairs;                            // 64
  int64_t start_frame[SDV2_MAX_ROWS];
  int64_t dst_start[SDV2_MAX_ROWS];
  int64_t new_global[SDV2_MAX_ROWS];
  int64_t new_local[SDV2_MAX_ROWS];
};

// First cache token of the row's write: the host's choice unless a kernel
// earlier on the stream (the adaptive sink decision) has put a slot into
// dst_override.  A value that would not fit the cache is ignored.
__device__ __forceinline__ int64_t row_dst_start(const AppendKernelArgs& a, int row) {
  int64_t dst = a.dst_start[row];
  if (a.dst_override) {
    const int64_t o = a.dst_override[row];
    if (o >= 0 && o + a.tokens <= a.cache_tokens) dst = o;
  }
  return dst;
}

// kWithKV = false: rotation of q alone (the stand-alone causal_rope_apply,
// causal_model.py:94-108), no cache and no index is touched.
template <typename T, bool kWithQ, bool kWithKV>
__global__ __launch_bounds__(kLanesPerRow * kTokensPerBlock)
void kv_append_rope_kernel(const AppendKernelArgs a) {
  const int lane = threadIdx.x & (kLanesPerRow - 1);
  const int tok = blockIdx.x * kTokensPerBlock + (threadIdx.x >> 4);
  const int row = blockIdx.z;
  const int head0 = blockIdx.y * kHeadsPerThread;

  if (kWithKV && blockIdx.x == 0 && blockIdx.y == 0 && threadIdx.x == 0) {
    if (a.global_end) a.global_end[row] = a.new_global[row];
    if (a.local_end) a.local_end[row] = a.new_local[row];
  }
  if (tok >= a.tokens) return;

  const int fi = tok / a.frame_tokens;
  const int rem = tok - fi * a.frame_tokens;
  const int hi = rem / a.grid_w;
  const int wi = rem - hi * a.grid_w;
  const int64_t frame = a.start_frame[row] + fi;

  double2 cs[4];
  sdv2::load_rotation(a.freqs, a.pairs, a.split_t, a.split_h, lane, frame, hi, wi, cs);

  const int64_t e0 = lane * 8;
  const int64_t dst_tok = kWithKV ? row_dst_start(a, row) + tok : 0;
  const T* qi = static_cast<const T*>(a.q_in) + row * a.q_in_st.row + tok * a.q_in_st.token + e0;
  const T* ki = static_cast<const T*>(a.k_in) + row * a.k_in_st.row + tok * a.k_in_st.token + e0;
  const T* vi = static_cast<const T*>(a.v_in) + row * a.v_in_st.row + tok * a.v_in_st.token + e0;
  T* qo = static_cast<T*>(a.q_out) + row * a.q_out_st.row + tok * a.q_out_st.token + e0;
  T* kc = static_cast<T*>(a.k_cache) + row * a.k_st.row + dst_tok * a.k_st.token + e0;
  T* vc = static_cast<T*>(a.v_cache) + row * a.v_st.row + dst_tok * a.v_st.token + e0;

  sdv2::Vec8<T> q[kHeadsPerThread], k[kHeadsPerThread], v[kHeadsPerThread];
#pragma unroll
  for (int j = 0; j < kHeadsPerThread; ++j) {
    const int h = head0 + j;
    if (h < a.heads) {
      if (kWithKV) {
        k[j] = sdv2::Vec8<T>::load(ki + h * a.k_in_st.head);
        v[j] = sdv2::Vec8<T>::load(vi + h * a.v_in_st.head);
      }
      if (kWithQ) q[j] = sdv2::Vec8<T>::load(qi + h * a.q_in_st.head);
    }
  }
#pragma unroll
  for (int j = 0; j < kHeadsPerThread; ++j) {
    const int h = head0 + j;
    if (h < a.heads) {
      if (kWithKV) {
        v[j].store(vc + h * a.v_st.head);
        sdv2::rotate(k[j], cs).store(kc + h * a.k_st.head);
      }
      if (kWithQ) sdv2::rotate(q[j], cs).store(qo + h * a.q_out_st.head);
    }
  }
}

// ---------------------------------------------------------------------------
// Append with the q / k RMSNorm of the projection outputs folded in
// (WanRMSNorm, wan_base/modules/model.py:70-86, as applied in qkv_fn,
// causal_model.py:212-218): y = type_as(x.float() * rsqrt(mean(x^2) + eps)) *
// weight over the full heads * 128 vector of a token, then RoPE and the
// scatter as above.  Rounding steps are the reference's: normalised value to
// the storage type, times weight to the storage type, rotation in double to
// float to the storage type.
//
// One workgroup of four waves per token.  Heads go in steps of four (lane l
// of a wave owns the 8-element slice l % 16 of head 4 j + l / 16 of its step
// j); wave w takes the steps w, w + 4, ... and keeps their q / k slices in
// registers between the sum of squares and the write.  The sum of squares is
// taken in the order of PyTorch's CPU sum kernel (ATen cascade_sum /
// vectorized_inner_sum with 8-float vectors, which the AVX2 and AVX512 builds
// share), so that mean, rsqrt and everything after them come out bit for bit
// as on the reference's CPU path: element e of the row belongs to accumulator
// (e / 8 % 4, e % 8); an accumulator adds its elements in blocks of 16, each
// block summed in order from zero, the block sums added up in order; a
// trailing partial block goes first; then the four accumulators of a vector
// lane are added in order, then the eight lanes in order, starting from zero.
// With e = 128 head + 8 slice + t the 16 lanes l % 4 == c of a step hold
// exactly one block of accumulator (c, t), in lane order: every wave parks its
// step's squares in LDS, lanes 0-31 (k) / 32-63 (q) each walk one accumulator's
// block, and the block sums meet in LDS, where every wave adds them up in
// step order.  The caller has checked this order against torch on the CPU.
//
// The query is needed for its sum of squares only when q_inv_rms is given:
// the attention kernel then normalises and rotates the raw query itself
// (sdv2_attn_params.q_norm_weight / q_inv_rms) and no rotated copy is written.
// ---------------------------------------------------------------------------
constexpr int kNormMaxSteps = 16;           // heads <= 64
constexpr int kNormWaves = 4;

template <typename T, int kStepsPerWave, bool kWriteQ>
__global__ __launch_bounds__(64 * kNormWaves)
void kv_append_norm_rope_kernel(const AppendKernelArgs a) {
#pragma clang fp contract(off)
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int sub = lane & (kLanesPerRow - 1);            // 8-element slice of a head row
  const int head_in_step = lane >> 4;                   // 0..3
  const int tok = blockIdx.x;
  const int row = blockIdx.z;

  if (blockIdx.x == 0 && threadIdx.x == 0) {
    if (a.global_end) a.global_end[row] = a.new_global[row];
    if (a.local_end) a.local_end[row] = a.new_local[row];
  }

  const int64_t e0 = sub * 8;
  const int64_t dst_tok = row_dst_start(a, row) + tok;
  const T* qi = static_cast<const T*>(a.q_in) + row * a.q_in_st.row + tok * a.q_in_st.token + e0;
  const T* ki = static_cast<const T*>(a.k_in) + row * a.k_in_st.row + tok * a.k_in_st.token + e0;
  const T* vi = static_cast<const T*>(a.v_in) + row * a.v_in_st.row + tok * a.v_in_st.token + e0;
  T* kc = static_cast<T*>(a.k_cache) + row * a.k_st.row + dst_tok * a.k_st.token + e0;
  T* vc = static_cast<T*>(a.v_cache) + row * a.v_st.row + dst_tok * a.v_st.token + e0;
  const int steps = (a.heads + 3) >> 2;

  sdv2::Vec8<T> q[kStepsPerWave], k[kStepsPerWave];
#pragma unroll
  for (int i = 0; i < kStepsPerWave; ++i) {
    const int j = wave + kNormWaves * i;
    const int h = 4 * j + head_in_step;
    if (j < steps && h < a.heads) {
      q[i] = sdv2::Vec8<T>::load(qi + h * a.q_in_st.head);
      k[i] = sdv2::Vec8<T>::load(ki + h * a.k_in_st.head);
      sdv2::Vec8<T>::load(vi + h * a.v_in_st.head).store(vc + h * a.v_st.head);
    } else {
      q[i] = sdv2::Vec8<T>::zero();
      k[i] = sdv2::Vec8<T>::zero();
    }
  }

  const int fi = tok / a.frame_tokens;
  const int rem = tok - fi * a.frame_tokens;
  const int hi = rem / a.grid_w;
  const int wi = rem - hi * a.grid_w;
  double2 cs[4];
  sdv2::load_rotation(a.freqs, a.pairs, a.split_t, a.split_h, sub, a.start_frame[row] + fi, hi, wi, cs);

  __shared__ float squares[kNormWaves][2][64 * 8];     // per wave: one step's squares of k and of q
  __shared__ float block_sums[2][kNormMaxSteps][32];   // k / q, step, accumulator
  const int which = lane >> 5;               // lanes 0-31 add up k, lanes 32-63 q
  const int chain = lane & 31;               // accumulator (c, t) = (chain % 4, chain / 4)
  const int c = chain & 3, t = chain >> 2;
  const int full = a.heads >> 2;             // steps whose four heads all exist: whole blocks of 16
  const int tail = 4 * (a.heads & 3);        // elements of the trailing partial block
#pragma unroll
  for (int i = 0; i < kStepsPerWave; ++i) {
    const int j = wave + kNormWaves * i;
    if (j < steps) {                         // (wave-uniform)
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        squares[wave][0][lane * 8 + e] = k[i].getf(e) * k[i].getf(e);
        squares[wave][1][lane * 8 + e] = q[i].getf(e) * q[i].getf(e);
      }
      // (LDS operations of one wave complete in order: no barrier between the stores and the loads)
      const int count = j < full ? 16 : tail;
      float block = 0.f;
#pragma unroll
      for (int m = 0; m < 16; ++m)
        if (m < count) block += squares[wave][which][(c + 4 * m) * 8 + t];
      block_sums[which][j][chain] = block;
    }
  }
  __syncthreads();
  float blocks = 0.f;                        // the whole blocks' sums, added up in order
  for (int j = 0; j < full; ++j) blocks += block_sums[which][j][chain];
  const float mine = tail ? block_sums[which][full][chain] + blocks : blocks;
  // the four accumulators of vector lane t, in order: they sit in the four lanes of a quad, whose values
  // every lane of the quad can take without a trip through LDS
  auto quad_lane = [](float x, auto which_c) {
    constexpr int i = decltype(which_c)::value;
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), i | (i << 2) | (i << 4) | (i << 6), 0xf, 0xf, false));
  };
  float lane_sum = quad_lane(mine, std::integral_constant<int, 0>{});
  lane_sum += quad_lane(mine, std::integral_constant<int, 1>{});
  lane_sum += quad_lane(mine, std::integral_constant<int, 2>{});
  lane_sum += quad_lane(mine, std::integral_constant<int, 3>{});
  // the eight vector lanes, in order, from zero: k's in lanes 0, 4, ... 28, q's 32 lanes further up
  float ssq_k = 0.f, ssq_q = 0.f;
#pragma unroll
  for (int v = 0; v < 8; ++v) {
    ssq_k += __int_as_float(__builtin_amdgcn_readlane(__float_as_int(lane_sum), 4 * v));
    ssq_q += __int_as_float(__builtin_amdgcn_readlane(__float_as_int(lane_sum), 32 + 4 * v));
  }

  const float width = static_cast<float>(a.heads * 128);
  const float rq = 1.0f / sqrtf(ssq_q / width + a.norm_eps);
  const float rk = 1.0f / sqrtf(ssq_k / width + a.norm_eps);
  if (a.q_inv_rms && threadIdx.x == 0) a.q_inv_rms[(int64_t)row * a.tokens + tok] = rq;
  const T* wq = static_cast<const T*>(a.q_norm_w) + e0;
  const T* wk = static_cast<const T*>(a.k_norm_w) + e0;
#pragma unroll
  for (int i = 0; i < kStepsPerWave; ++i) {
    const int j = wave + kNormWaves * i;
    const int h = 4 * j + head_in_step;
    if (j < steps && h < a.heads) {
      const sdv2::Vec8<T> kn = sdv2::normalise(k[i], rk, sdv2::Vec8<T>::load(wk + h * 128));
      sdv2::rotate(kn, cs).store(kc + h * a.k_st.head);
      if constexpr (kWriteQ) {
        T* qo = static_cast<T*>(a.q_out) + row * a.q_out_st.row + tok * a.q_out_st.token + e0;
        const sdv2::Vec8<T> qn = sdv2::normalise(q[i], rq, sdv2::Vec8<T>::load(wq + h * 128));
        sdv2::rotate(qn, cs).store(qo + h * a.q_out_st.head);
      }
    }
  }
}

bool stride_ok(const sdv2_stride3& s, int vec) {
  return s.row % vec == 0 && s.token % vec == 0 && s.head % vec == 0;
}

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

}  // namespace

extern "C" int sdv2_kv_append_rope(const sdv2_append_params* p) {
  if (!p) return SDV2_ERR_INVALID_ARG;
  if (p->head_dim != SDV2_HEAD_DIM) return SDV2_ERR_UNSUPPORTED;
  if (p->dtype != SDV2_BF16 && p->dtype != SDV2_F32) return SDV2_ERR_UNSUPPORTED;
  if (p->rows < 0 || p->tokens < 0 || p->heads <= 0) return SDV2_ERR_INVALID_ARG;
  if (p->rows > SDV2_MAX_ROWS) return SDV2_ERR_INVALID_ARG;
  if (p->rows == 0 || p->tokens == 0) return SDV2_OK;
  if (p->grid_f <= 0 || p->grid_h <= 0 || p->grid_w <= 0) return SDV2_ERR_INVALID_ARG;
  if (static_cast<int64_t>(p->grid_f) * p->grid_h * p->grid_w != p->tokens) return SDV2_ERR_INVALID_ARG;
  if (!p->freqs) return SDV2_ERR_INVALID_ARG;
  const bool with_norm = p->q_norm_weight != nullptr || p->k_norm_weight != nullptr;
  // q comes with the tensor its rotation goes to - or, with the norm folded in, with the place for its 1 / rms
  if (p->q_inv_rms && !with_norm) return SDV2_ERR_INVALID_ARG;
  if (p->q_in == nullptr ? (p->q_out != nullptr || p->q_inv_rms != nullptr) : (p->q_out == nullptr && p->q_inv_rms == nullptr))
    return SDV2_ERR_INVALID_ARG;
  const bool with_q = p->q_in != nullptr;
  // k, v and the two caches come together or not at all; without them the call
  // only rotates q (and then has nothing to do with a cache or its indices)
  const bool with_kv = p->k_in != nullptr;
  if ((p->v_in != nullptr) != with_kv || (p->k_cache != nullptr) != with_kv || (p->v_cache != nullptr) != with_kv)
    return SDV2_ERR_INVALID_ARG;
  if (!with_kv && (!with_q || p->global_end_index || p->local_end_index || p->dst_start_override ||
                   p->q_norm_weight || p->k_norm_weight))
    return SDV2_ERR_INVALID_ARG;
  if (!p->start_frame || (with_kv && !p->dst_start)) return SDV2_ERR_INVALID_ARG;
  if ((p->global_end_index || p->local_end_index) && (!p->new_global_end || !p->new_local_end))
    return SDV2_ERR_INVALID_ARG;
  if (with_norm) {
    // the fused norm covers q and k together, as qkv_fn applies it
    if (!p->q_norm_weight || !p->k_norm_weight || !with_q) return SDV2_ERR_INVALID_ARG;
    if (p->heads > 4 * kNormMaxSteps) return SDV2_ERR_UNSUPPORTED;
    if (!(p->norm_eps >= 0.f)) return SDV2_ERR_INVALID_ARG;
    if (!aligned16(p->q_norm_weight) || !aligned16(p->k_norm_weight)) return SDV2_ERR_INVALID_ARG;
    if (p->q_inv_rms && (reinterpret_cast<uintptr_t>(p->q_inv_rms) & 3)) return SDV2_ERR_INVALID_ARG;
  }

  // 16-byte vector access: 8 bf16 or 4 floats per transaction.
  const int vec = p->dtype == SDV2_BF16 ? 8 : 4;
  const void* ptrs[] = {p->q_in, p->k_in, p->v_in, p->q_out, p->k_cache, p->v_cache};
  for (const void* ptr : ptrs)
    if (ptr && !aligned16(ptr)) return SDV2_ERR_INVALID_ARG;
  if (with_kv && (!stride_ok(p->k_in_stride, vec) || !stride_ok(p->v_in_stride, vec) ||
                  !stride_ok(p->k_cache_stride, vec) || !stride_ok(p->v_cache_stride, vec)))
    return SDV2_ERR_INVALID_ARG;
  if (with_q && (!stride_ok(p->q_in_stride, vec) || (p->q_out && !stride_ok(p->q_out_stride, vec))))
    return SDV2_ERR_INVALID_ARG;

  if (p->grid_h > p->freq_rows || p->grid_w > p->freq_rows) return SDV2_ERR_OUT_OF_RANGE;
  for (int i = 0; i < p->rows; ++i) {
    if (p->start_frame[i] < 0 || p->start_frame[i] + p->grid_f > p->freq_rows) return SDV2_ERR_OUT_OF_RANGE;
    if (with_kv && (p->dst_start[i] < 0 || p->dst_start[i] + p->tokens > p->cache_tokens))
      return SDV2_ERR_OUT_OF_RANGE;
  }

  AppendKernelArgs a{};
  a.q_in = p->q_in; a.k_in = p->k_in; a.v_in = p->v_in;
  a.q_out = p->q_out; a.k_cache = p->k_cache; a.v_cache = p->v_cache;
  a.q_in_st = p->q_in_stride; a.k_in_st = p->k_in_stride; a.v_in_st = p->v_in_stride;
  a.q_out_st = p->q_out_stride; a.k_st = p->k_cache_stride; a.v_st = p->v_cache_stride;
  a.freqs = reinterpret_cast<const double2*>(p->freqs);
  a.q_norm_w = p->q_norm_weight; a.k_norm_w = p->k_norm_weight; a.norm_eps = p->norm_eps;
  a.global_end = p->global_end_index;
  a.local_end = p->local_end_index;
  a.dst_override = p->dst_start_override;
  a.q_inv_rms = p->q_inv_rms;
  a.cache_tokens = p->cache_tokens;
  a.tokens = p->tokens; a.heads = p->heads; a.grid_w = p->grid_w;
  a.frame_tokens = p->grid_h * p->grid_w;
  a.pairs = p->head_dim / 2;
  // column split of the table: c - 2*(c/3) | c/3 | c/3  (causal_model.py:77-78)
  const int third = a.pairs / 3;
  a.split_t = a.pairs - 2 * third;
  a.split_h = a.split_t + third;
  for (int i = 0; i < p->rows; ++i) {
    a.start_frame[i] = p->start_frame[i];
    a.dst_start[i] = with_kv ? p->dst_start[i] : 0;
    a.new_global[i] = p->new_global_end ? p->new_global_end[i] : 0;
    a.new_local[i] = p->new_local_end ? p->new_local_end[i] : 0;
  }

  dim3 block(kLanesPerRow * kTokensPerBlock);
  dim3 grid((p->tokens + kTokensPerBlock - 1) / kTokensPerBlock,
            (p->heads + kHeadsPerThread - 1) / kHeadsPerThread, p->rows);
  hipStream_t stream = static_cast<hipStream_t>(p->stream);
  if (with_norm) {
    const dim3 norm_grid(p->tokens, 1, p->rows);
    const dim3 norm_block(64 * kNormWaves);
    // the q / k slices of a wave's steps stay in registers: the variant fixes how many steps a wave takes
    auto launch = [&](auto steps_c) {
      constexpr int kS = decltype(steps_c)::value;
      const bool write_q = p->q_out != nullptr;
      if (p->dtype == SDV2_BF16) {
        if (write_q) sdv2::launch_timed(SDV2_KERNEL_APPEND, kv_append_norm_rope_kernel<uint16_t, kS, true>, norm_grid, norm_block, 0, stream, a);
        else sdv2::launch_timed(SDV2_KERNEL_APPEND, kv_append_norm_rope_kernel<uint16_t, kS, false>, norm_grid, norm_block, 0, stream, a);
      } else {
        if (write_q) sdv2::launch_timed(SDV2_KERNEL_APPEND, kv_append_norm_rope_kernel<float, kS, true>, norm_grid, norm_block, 0, stream, a);
        else sdv2::launch_timed(SDV2_KERNEL_APPEND, kv_append_norm_rope_kernel<float, kS, false>, norm_grid, norm_block, 0, stream, a);
      }
    };
    const int per_wave = ((p->heads + 3) / 4 + kNormWaves - 1) / kNormWaves;
    if (per_wave <= 1) launch(std::integral_constant<int, 1>{});
    else if (per_wave <= 3) launch(std::integral_constant<int, 3>{});
    else launch(std::integral_constant<int, kNormMaxSteps / kNormWaves>{});
    return hipGetLastError() == hipSuccess ? SDV2_OK : SDV2_ERR_LAUNCH;
  }
  auto launch = [&](auto kernel) {
    sdv2::launch_timed(SDV2_KERNEL_APPEND, kernel, grid, block, 0, stream, a);
  };
  if (p->dtype == SDV2_BF16) {
    if (!with_kv) launch(kv_append_rope_kernel<uint16_t, true, false>);
    else if (with_q) launch(kv_append_rope_kernel<uint16_t, true, true>);
    else launch(kv_append_rope_kernel<uint16_t, false, true>);
  } else {
    if (!with_kv) launch(kv_append_rope_kernel<float, true, false>);
    else if (with_q) launch(kv_append_rope_kernel<float, true, true>);
    else launch(kv_append_rope_kernel<float, false, true>);
  }
  return hipGetLastError() == hipSuccess ? SDV2_OK : SDV2_ERR_LAUNCH;
}
