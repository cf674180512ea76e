// Adaptive sink refresh decision for gfx950.
//
// Stands in for models/wan/causal_model.py:284-299: per cache row, the mean
// over the tokens of every sink frame of the cached K and V is compared (cosine
// similarity over the flattened heads x 128 vector) with the mean of the
// incoming one-frame chunk's roped K and its V; the two similarities are
// averaged and, when the smallest falls below the threshold, that sink frame
// is to be overwritten next.  The reference does this with four reductions and
// two host round trips per row; here ONE launch does it: workgroups sum the
// frames over their tokens, eight token ranges per (frame, head) side by side
// (rotating the new keys on the fly with the append kernel's arithmetic, so
// they never have to be staged), and the workgroup that finishes last for a
// row turns the sums into means, similarities and the decision.  The caller
// reads back one int per row - not necessarily at once: the decision can also
// hand the slot a refresh selects straight to the append kernel that follows
// on the stream (dst_start_override), so the host may pick the decision up a
// whole model pass later, when it plans this layer's next call.
//
// Rounding follows the storage dtype: with bf16 tensors the frame means, the
// two cosine similarities and their sum are each rounded to bf16 (they are
// bf16 tensors in the reference); sums inside a reduction are fp32 in a fixed
// order, so results are deterministic.
//
// The means of the cached sink frames only change when a sink frame is written.
// A caller that keeps them between calls (frame_sums) has the reduction read
// the new chunk alone: the deciding workgroup files the new chunk's means under
// the sink frame the append that follows will overwrite, and only frames the
// caller marks stale are summed from the cache again.
//
// When the q / k RMSNorm is folded into the append the keys arrive raw: a
// first small kernel then takes every token's 1 / rms (in the append's
// arithmetic) and the reduction normalises before it rotates.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

#include "sdv2kv.h"
#include "sdv2kv_profile.h"
#include "sdv2kv_internal.h"
#include "rope_device.h"

namespace {

constexpr int kLanesPerRow = 16;            // 16 lanes x 8 elements = 128
constexpr int kTokenLanes = 16;             // 256 threads
constexpr int kTokenSplits = 8;             // workgroups per (frame, head): token ranges summed apart
constexpr int kMaxHeads = 64;
constexpr int kThreads = kLanesPerRow * kTokenLanes;
constexpr int kTicketBytes = 256;           // one ticket word per row at the head of the workspace
static_assert(SDV2_MAX_ROWS * sizeof(int32_t) <= kTicketBytes, "ticket words");

struct SinkSimKernelArgs {
  const void* k_in;
  const void* v_in;
  const void* k_cache;
  const void* v_cache;
  sdv2_stride3 k_in_st, v_in_st, k_st, v_st;
  const double2* freqs;
  int32_t* tickets;                         // [rows], zero between calls
  float* sums;                              // [rows][2*sink+2][heads][kTokenSplits][128]: token sums of this call
  float* kept;                              // [rows][2*sink][heads*128] frame means kept between calls, or null
  const void* k_norm_w;                     // RMSNorm weight of k over heads * 128, or null
  float* inv_rms;                           // [rows][tokens]: 1 / rms of every new key token (with k_norm_w)
  float norm_eps;
  uint32_t stale[SDV2_MAX_ROWS];            // bit j: sink frame j of the row is summed from the cache in this call
  int32_t planned_frame[SDV2_MAX_ROWS];     // sink frame the host's plan writes this call's chunk to, or -1
  float* similarity;                        // [rows][sink]
  int32_t* refresh;                         // [rows]
  int64_t* dst_override;                    // [rows] or null: slot start for the append that follows
  uint32_t override_rows;                   // bit i: row i is about to evict, so a refresh moves its write
  int32_t tokens, heads, grid_w, sink_frames;
  int32_t first_matrix;                     // matrices below this one are not summed in this call: the grid leaves them out
  int32_t split_t, split_h, pairs;
  float threshold;
  int64_t start_frame[SDV2_MAX_ROWS];
};

// Token sums travel from the workgroups that form them to the one that
// decides, which may sit behind another XCD's L2: both sides use relaxed
// device-scope accesses (the store writes through, the load does not hit in a
// stale line), ordered by the ticket the deciding workgroup draws last.
__device__ __forceinline__ void store_coherent(float* p, float x) {
  __hip_atomic_store(reinterpret_cast<uint32_t*>(p), __float_as_uint(x), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ float load_coherent(const float* p) {
  return __uint_as_float(
      __hip_atomic_load(reinterpret_cast<const uint32_t*>(p), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
}

// The token sums of four neighbouring columns, all kTokenSplits ranges (512
// bytes apart): 16-byte device-coherent loads, which have no spelling in the
// language.  Issue and wait are ONE asm statement: between a load's issue and
// its return the compiler believes the destination registers hold the value and
// is free to copy or reuse them.
typedef __attribute__((ext_vector_type(4))) float f32x4;
__device__ __forceinline__ void load_coherent_ranges(const float* base, f32x4 (&w)[8]) {
  static_assert(kTokenSplits == 8, "eight ranges per statement");
  asm volatile(
      "global_load_dwordx4 %0, %8, off sc1\n\t"
      "global_load_dwordx4 %1, %8, off offset:512 sc1\n\t"
      "global_load_dwordx4 %2, %8, off offset:1024 sc1\n\t"
      "global_load_dwordx4 %3, %8, off offset:1536 sc1\n\t"
      "global_load_dwordx4 %4, %8, off offset:2048 sc1\n\t"
      "global_load_dwordx4 %5, %8, off offset:2560 sc1\n\t"
      "global_load_dwordx4 %6, %8, off offset:3072 sc1\n\t"
      "global_load_dwordx4 %7, %8, off offset:3584 sc1\n\t"
      "s_waitcnt vmcnt(0)"
      : "=&v"(w[0]), "=&v"(w[1]), "=&v"(w[2]), "=&v"(w[3]), "=&v"(w[4]), "=&v"(w[5]), "=&v"(w[6]), "=&v"(w[7])
      : "v"(base)
      : "memory");
}
// the same for two groups of four columns in one trip
__device__ __forceinline__ void load_coherent_ranges2(const float* base0, const float* base1, f32x4 (&w0)[8], f32x4 (&w1)[8]) {
  asm volatile(
      "global_load_dwordx4 %0, %16, off sc1\n\t"
      "global_load_dwordx4 %1, %16, off offset:512 sc1\n\t"
      "global_load_dwordx4 %2, %16, off offset:1024 sc1\n\t"
      "global_load_dwordx4 %3, %16, off offset:1536 sc1\n\t"
      "global_load_dwordx4 %4, %16, off offset:2048 sc1\n\t"
      "global_load_dwordx4 %5, %16, off offset:2560 sc1\n\t"
      "global_load_dwordx4 %6, %16, off offset:3072 sc1\n\t"
      "global_load_dwordx4 %7, %16, off offset:3584 sc1\n\t"
      "global_load_dwordx4 %8, %17, off sc1\n\t"
      "global_load_dwordx4 %9, %17, off offset:512 sc1\n\t"
      "global_load_dwordx4 %10, %17, off offset:1024 sc1\n\t"
      "global_load_dwordx4 %11, %17, off offset:1536 sc1\n\t"
      "global_load_dwordx4 %12, %17, off offset:2048 sc1\n\t"
      "global_load_dwordx4 %13, %17, off offset:2560 sc1\n\t"
      "global_load_dwordx4 %14, %17, off offset:3072 sc1\n\t"
      "global_load_dwordx4 %15, %17, off offset:3584 sc1\n\t"
      "s_waitcnt vmcnt(0)"
      : "=&v"(w0[0]), "=&v"(w0[1]), "=&v"(w0[2]), "=&v"(w0[3]), "=&v"(w0[4]), "=&v"(w0[5]), "=&v"(w0[6]), "=&v"(w0[7]),
        "=&v"(w1[0]), "=&v"(w1[1]), "=&v"(w1[2]), "=&v"(w1[3]), "=&v"(w1[4]), "=&v"(w1[5]), "=&v"(w1[6]), "=&v"(w1[7])
      : "v"(base0), "v"(base1)
      : "memory");
}

// Sum over the 64 lanes of a wave without a trip through LDS per step: within
// quads, rows of 16 lanes, then across the rows (the wave-wide broadcasts of
// the data-parallel-primitive operand modes); lane 63 ends up with the total.
__device__ __forceinline__ float wave_sum(float x) {
  auto dpp = [](float v, auto ctrl_c, auto rows_c) {
    constexpr int ctrl = decltype(ctrl_c)::value, rows = decltype(rows_c)::value;
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), ctrl, rows, 0xf, false));
  };
  using All = std::integral_constant<int, 0xf>;
  x += dpp(x, std::integral_constant<int, 0xb1>{}, All{});      // quad_perm [1, 0, 3, 2]
  x += dpp(x, std::integral_constant<int, 0x4e>{}, All{});      // quad_perm [2, 3, 0, 1]
  x += dpp(x, std::integral_constant<int, 0x141>{}, All{});     // row_half_mirror
  x += dpp(x, std::integral_constant<int, 0x140>{}, All{});     // row_mirror
  x += dpp(x, std::integral_constant<int, 0x142>{}, std::integral_constant<int, 0xa>{});   // row_bcast15 into rows 1, 3
  x += dpp(x, std::integral_constant<int, 0x143>{}, std::integral_constant<int, 0xc>{});   // row_bcast31 into rows 2, 3
  return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(x), 63));
}

// matrices of a row: sink K frames, sink V frames, new K, new V
__device__ __forceinline__ float* sums_of(const SinkSimKernelArgs& a, int row, int m) {
  return a.sums + (static_cast<int64_t>(row) * (2 * a.sink_frames + 2) + m) * a.heads * (kTokenSplits * 128);
}
__device__ __forceinline__ float* kept_of(const SinkSimKernelArgs& a, int row, int m) {
  return a.kept + (static_cast<int64_t>(row) * 2 * a.sink_frames + m) * a.heads * 128;
}
// is matrix m summed over its tokens in this call?  (The new chunk always; a
// sink frame unless its mean is kept and the caller vouches for it.)
__device__ __forceinline__ bool summed_now(const SinkSimKernelArgs& a, int row, int m) {
  const int sink = a.sink_frames;
  if (m >= 2 * sink || !a.kept) return true;
  return (a.stale[row] >> (m < sink ? m : m - sink)) & 1u;
}

template <typename T>
__device__ __forceinline__ float round_to_storage(float x);
template <>
__device__ __forceinline__ float round_to_storage<uint16_t>(float x) {
  return sdv2::bf16_bits_to_f32(sdv2::f32_to_bf16_rne(x));
}
template <>
__device__ __forceinline__ float round_to_storage<float>(float x) { return x; }

// Frame means from the token sums, cosine similarities, their average, the
// decision: run by the one workgroup of a row that finished its sums last.  A
// thread owns kCols columns (columns past the width are clamped and weighted
// with zero instead of branched around, so all loads of a frame are issued
// together).  Every dot product is reduced inside its wave as soon as it is
// formed and the per-wave results wait in LDS, so nothing but loads and
// arithmetic sits between two frames; the workgroup synchronises once, before
// the tail.
template <typename T, int kCols>
__device__ __forceinline__ void decide(const SinkSimKernelArgs& a, int row) {
  constexpr int kWaves = kThreads / 64;
  __shared__ float wave_part[SDV2_MAX_SINK_FRAMES + 1][kWaves][4];
  __shared__ float sims[SDV2_MAX_SINK_FRAMES];
  const int sink = a.sink_frames;
  const int width = a.heads * 128;
  const float inv_tokens = 1.0f / static_cast<float>(a.tokens);
  constexpr float kEps = 1e-8f;             // torch.cosine_similarity default
  // Column i of this thread, and its weight (0 past the width).  Columns come
  // in groups of four neighbours (4 * thread .. 4 * thread + 3, then 4 * kThreads
  // further on), so that the token sums of a group arrive in 16-byte accesses;
  // a group past the width is clamped to the last group and weighted with zero.
  static_assert(kCols % 4 == 0, "columns are owned in groups of four");
  auto raw_col = [&](int i) { return 4 * static_cast<int>(threadIdx.x) + (i & 3) + (i >> 2) * 4 * kThreads; };
  auto col = [&](int i) {
    const int c = raw_col(i);
    return c < width ? c : width - 4 + (i & 3);
  };
  // where the eight ranges' sums of the column group that starts at column i of this thread begin
  auto ranges_of = [&](const float* p, int i) { return p + (col(i) >> 7) * (kTokenSplits * 128) + (col(i) & 127); };
  auto live = [&](int i) { return raw_col(i) < width ? 1.f : 0.f; };
  // means of matrix m at this thread's columns: the token ranges in order and
  // the rounding of a stored mean, or the mean kept from an earlier call.  The
  // token sums are fetched for eight columns at a time (64 loads in flight).
  auto means = [&](int m, float (&out)[kCols]) {
    if (summed_now(a, row, m)) {
      const float* p = sums_of(a, row, m);
#pragma unroll
      for (int i0 = 0; i0 < kCols; i0 += 4) {
        f32x4 part[kTokenSplits];
        load_coherent_ranges(ranges_of(p, i0), part);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          float sum = 0.f;
#pragma unroll
          for (int j = 0; j < kTokenSplits; ++j) sum += part[j][e];
          out[i0 + e] = round_to_storage<T>(sum * inv_tokens);
        }
      }
      if (a.kept && m < 2 * sink) {
        float* keep = kept_of(a, row, m);
#pragma unroll
        for (int i = 0; i < kCols; ++i) keep[col(i)] = out[i];      // (clamped columns repeat the last one's value)
      }
    } else {
      const float* keep = kept_of(a, row, m);
#pragma unroll
      for (int i = 0; i < kCols; ++i) out[i] = keep[col(i)];
    }
  };
  // this wave's share of four sums, in a fixed order, parked in LDS
  auto park = [&](int slot, float (&x)[4]) {
#pragma unroll
    for (int i = 0; i < 4; ++i) x[i] = wave_sum(x[i]);
    if ((threadIdx.x & 63) == 0)
#pragma unroll
      for (int i = 0; i < 4; ++i) wave_part[slot][threadIdx.x >> 6][i] = x[i];
  };
  auto total = [&](int slot, int i) {
    float sum = 0.f;
#pragma unroll
    for (int w = 0; w < kWaves; ++w) sum += wave_part[slot][w][i];
    return sum;
  };

  // Sink frames are taken kBatch at a time, and the first batch is requested
  // ahead of the new chunk's sums: loads return in order, so nothing the dot
  // products need is still on its way when the sums have arrived.  (A batch that
  // reaches past the last frame repeats it; its results are dropped.)
  constexpr int kBatch = kCols <= 8 ? 4 : (kCols <= 20 ? 2 : 1);
  float ks[kBatch][kCols], vs[kBatch][kCols];
  auto fetch_frames = [&](int j0) {
#pragma unroll
    for (int b = 0; b < kBatch; ++b) {
      const int j = j0 + b < sink ? j0 + b : sink - 1;
      means(j, ks[b]);
      means(sink + j, vs[b]);
    }
  };
  fetch_frames(0);
  float k_new[kCols], v_new[kCols];
  if constexpr (kCols <= 8) {
    // two column groups per thread: all the token sums of a new matrix come in one trip to memory
    static_assert(kCols == 8, "two column groups per thread");
    f32x4 part[2][2][kTokenSplits];          // matrix, column group, token range
#pragma unroll
    for (int m = 0; m < 2; ++m) {
      const float* p = sums_of(a, row, 2 * sink + m);
      load_coherent_ranges2(ranges_of(p, 0), ranges_of(p, 4), part[m][0], part[m][1]);
    }
#pragma unroll
    for (int i = 0; i < kCols; ++i) {
      float sum_k = 0.f, sum_v = 0.f;
#pragma unroll
      for (int j = 0; j < kTokenSplits; ++j) {
        sum_k += part[0][i >> 2][j][i & 3];
        sum_v += part[1][i >> 2][j][i & 3];
      }
      k_new[i] = round_to_storage<T>(sum_k * inv_tokens);
      v_new[i] = round_to_storage<T>(sum_v * inv_tokens);
    }
  } else {
    means(2 * sink, k_new);
    means(2 * sink + 1, v_new);
  }
  float n[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int i = 0; i < kCols; ++i) {
    n[0] += k_new[i] * k_new[i] * live(i);
    n[1] += v_new[i] * v_new[i] * live(i);
  }
  park(sink, n);
  for (int j0 = 0; j0 < sink; j0 += kBatch) {
    if (j0 > 0) fetch_frames(j0);
#pragma unroll
    for (int b = 0; b < kBatch; ++b) {
      float d[4] = {0.f, 0.f, 0.f, 0.f};    // k.k_new, |k|^2, v.v_new, |v|^2
#pragma unroll
      for (int i = 0; i < kCols; ++i) {
        d[0] += ks[b][i] * k_new[i] * live(i);
        d[1] += ks[b][i] * ks[b][i] * live(i);
        d[2] += vs[b][i] * v_new[i] * live(i);
        d[3] += vs[b][i] * vs[b][i] * live(i);
      }
      if (j0 + b < sink) park(j0 + b, d);
    }
  }
  __syncthreads();
  if (threadIdx.x < sink) {
    const int j = threadIdx.x;
    const float k_new_norm = fmaxf(sqrtf(total(sink, 0)), kEps);
    const float v_new_norm = fmaxf(sqrtf(total(sink, 1)), kEps);
    const float cos_k = round_to_storage<T>(total(j, 0) / (fmaxf(sqrtf(total(j, 1)), kEps) * k_new_norm));
    const float cos_v = round_to_storage<T>(total(j, 2) / (fmaxf(sqrtf(total(j, 3)), kEps) * v_new_norm));
    const float sim = round_to_storage<T>(cos_k + cos_v) * 0.5f;
    a.similarity[row * sink + j] = sim;
    sims[j] = sim;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    float best = sims[0];
    int best_frame = 0;
    for (int j = 1; j < sink; ++j)
      if (sims[j] < best) {                   // first minimum, as torch.argmin
        best = sims[j];
        best_frame = j;
      }
    const int frame = best < round_to_storage<T>(a.threshold) ? best_frame : -1;
    a.refresh[row] = frame;
    sims[0] = __int_as_float(frame);          // (for the hand-over of the kept means below)
    // The refreshed sink frame goes to the head of the row's eviction queue
    // (causal_model.py:297-299); a call on the evict branch then writes its
    // one-frame chunk at [(frame + 1) * tokens - tokens, (frame + 1) * tokens).
    if (a.dst_override)
      a.dst_override[row] = frame >= 0 && ((a.override_rows >> row) & 1u) ? static_cast<int64_t>(frame) * a.tokens : -1;
  }
  if (a.kept) {
    // The append that follows overwrites a sink frame when the row evicts into
    // the frame just chosen, or when the host's plan (a filling call) lands
    // there: the new chunk's means become that frame's kept means.
    __syncthreads();
    const int chosen = __float_as_int(sims[0]);
    const bool evicting = (a.override_rows >> row) & 1u;
    const int target = evicting && a.dst_override && chosen >= 0 ? chosen : a.planned_frame[row];
    if (target >= 0 && target < sink) {
      float* keep_k = kept_of(a, row, target);
      float* keep_v = kept_of(a, row, sink + target);
#pragma unroll
      for (int i = 0; i < kCols; ++i) {
        keep_k[col(i)] = k_new[i];
        keep_v[col(i)] = v_new[i];
      }
    }
  }
}

// grid (heads, matrices summed in this call, rows * kTokenSplits): one workgroup sums one head's
// 128 columns of one frame over one eighth of its tokens.  (With every sink
// frame's mean kept, the matrices are the new K and V alone: first_matrix.)  (One workgroup per
// frame and head would leave most of the chip idle: 96 workgroups for three
// sink frames of twelve heads.)  Then it draws its row's ticket, after its
// sums have been acknowledged by memory; the workgroup that draws the last one
// finds every sum of the row in memory, decides, and leaves the ticket at zero
// for the next call.
template <typename T, int kCols>
__global__ __launch_bounds__(kThreads)
void sink_similarity_kernel(const SinkSimKernelArgs a) {
  __shared__ float part[kTokenLanes][kLanesPerRow * 8];
  __shared__ int is_last;
  const int lane = threadIdx.x & (kLanesPerRow - 1);
  const int tl = threadIdx.x >> 4;
  const int head = blockIdx.x;
  const int m = blockIdx.y + a.first_matrix;
  const int row = blockIdx.z / kTokenSplits;
  const int split = blockIdx.z - row * kTokenSplits;
  const int sink = a.sink_frames;

  const bool is_new = m >= 2 * sink;
  const bool is_k = is_new ? (m == 2 * sink) : (m < sink);
  const int frame = is_new ? 0 : (m < sink ? m : m - sink);
  // a kept frame mean stands until the caller calls it stale
  if (!summed_now(a, row, m)) return;
  const sdv2_stride3 st = is_new ? (is_k ? a.k_in_st : a.v_in_st) : (is_k ? a.k_st : a.v_st);
  const T* base = static_cast<const T*>(is_new ? (is_k ? a.k_in : a.v_in) : (is_k ? a.k_cache : a.v_cache));
  base += row * st.row + static_cast<int64_t>(frame) * a.tokens * st.token + head * st.head + lane * 8;

  const int per = (a.tokens + kTokenSplits - 1) / kTokenSplits;
  const int t_end = (split + 1) * per < a.tokens ? (split + 1) * per : a.tokens;
  float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  // A token lane walks every sixteenth token of the range.  The range is short
  // (195 tokens of a 1560-token frame: 12 or 13 per lane) and every trip to
  // memory costs the same few microseconds whatever it carries, so a lane asks
  // for up to kFlight of its tokens at once; past the end of the range it asks
  // for the last token again and leaves it out of the sum.  The order of the
  // adds is the token order.
  constexpr int kFlight = 16;
  if (is_new && is_k) {
    // the new keys are rotated on the way in; their table entries (four per lane and token) are fetched for
    // half a flight at a time, which is what the registers hold beside the tokens themselves
    constexpr int kHalf = kFlight / 2;
    auto rotation = [&](int t, double2 (&cs)[4]) {
      const int hi = t / a.grid_w;
      sdv2::load_rotation(a.freqs, a.pairs, a.split_t, a.split_h, lane, a.start_frame[row], hi, t - hi * a.grid_w, cs);
    };
    // with the norm folded in: the key as the append will normalise it (same two roundings)
    sdv2::Vec8<T> weight;
    if (a.k_norm_w) weight = sdv2::Vec8<T>::load(static_cast<const T*>(a.k_norm_w) + head * 128 + lane * 8);
    for (int t0 = split * per + tl; t0 < t_end; t0 += kFlight * kTokenLanes) {
      sdv2::Vec8<T> x[kFlight];
      float r[kFlight];
#pragma unroll
      for (int u = 0; u < kFlight; ++u) {
        const int t = t0 + u * kTokenLanes < t_end ? t0 + u * kTokenLanes : t_end - 1;
        x[u] = sdv2::Vec8<T>::load(base + t * st.token);
        r[u] = a.k_norm_w ? a.inv_rms[static_cast<int64_t>(row) * a.tokens + t] : 1.0f;
      }
#pragma unroll
      for (int half = 0; half < 2; ++half) {
        if (t0 + half * kHalf * kTokenLanes >= t_end) break;
        double2 cs[kHalf][4];
#pragma unroll
        for (int u = 0; u < kHalf; ++u) {
          const int t = t0 + (half * kHalf + u) * kTokenLanes;
          rotation(t < t_end ? t : t_end - 1, cs[u]);
        }
#pragma unroll
        for (int u = 0; u < kHalf; ++u) {
          if (t0 + (half * kHalf + u) * kTokenLanes < t_end) {
            sdv2::Vec8<T> xx = x[half * kHalf + u];
            if (a.k_norm_w) xx = sdv2::normalise(xx, r[half * kHalf + u], weight);
            const sdv2::Vec8<T> y = sdv2::rotate(xx, cs[u]);
#pragma unroll
            for (int i = 0; i < 8; ++i) acc[i] += static_cast<float>(y.get(i));
          }
        }
      }
    }
  } else {
    for (int t0 = split * per + tl; t0 < t_end; t0 += kFlight * kTokenLanes) {
      sdv2::Vec8<T> x[kFlight];
#pragma unroll
      for (int u = 0; u < kFlight; ++u) {
        const int t = t0 + u * kTokenLanes < t_end ? t0 + u * kTokenLanes : t_end - 1;
        x[u] = sdv2::Vec8<T>::load(base + t * st.token);
      }
#pragma unroll
      for (int u = 0; u < kFlight; ++u)
        if (t0 + u * kTokenLanes < t_end)
#pragma unroll
          for (int i = 0; i < 8; ++i) acc[i] += static_cast<float>(x[u].get(i));
    }
  }
#pragma unroll
  for (int i = 0; i < 8; ++i) part[tl][lane * 8 + i] = acc[i];
  __syncthreads();
  if (threadIdx.x < kLanesPerRow * 8) {
    float sum = 0.f;
#pragma unroll
    for (int j = 0; j < kTokenLanes; ++j) sum += part[j][threadIdx.x];
    store_coherent(sums_of(a, row, m) + (head * kTokenSplits + split) * 128 + threadIdx.x, sum);
  }
  __builtin_amdgcn_s_waitcnt(0x0F70);       // vmcnt(0): the stores have been acknowledged
  __syncthreads();
  if (threadIdx.x == 0) {
    // workgroups of this row that sum anything in this call
    int matrices = 2;
    for (int f = 0; f < sink; ++f) matrices += summed_now(a, row, f) ? 2 : 0;
    const int expected = matrices * a.heads * kTokenSplits;
    const int drawn = __hip_atomic_fetch_add(a.tickets + row, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    const int last = drawn == expected - 1;
    if (last) __hip_atomic_store(a.tickets + row, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    is_last = last;
  }
  __syncthreads();
  if (!is_last) return;
  decide<T, kCols>(a, row);
}

// grid (tokens / 4, 1, rows): one wave per new key token takes 1 / sqrt(mean(k^2) + eps)
// over the token's heads * 128 values, exactly as the append kernel with the
// norm folded in does (same order of additions, same operations).
template <typename T, int kSteps>
__global__ __launch_bounds__(256)
void key_inv_rms_kernel(const SinkSimKernelArgs a) {
  const int lane = threadIdx.x & 63;
  const int tok = blockIdx.x * 4 + (threadIdx.x >> 6);
  const int row = blockIdx.z;
  if (tok >= a.tokens) return;
  const T* ki = static_cast<const T*>(a.k_in) + row * a.k_in_st.row + tok * a.k_in_st.token + (lane & 15) * 8;
  sdv2::Vec8<T> k[kSteps];
#pragma unroll
  for (int j = 0; j < kSteps; ++j) {
    const int h = 4 * j + (lane >> 4);
    k[j] = 4 * j < a.heads && h < a.heads ? sdv2::Vec8<T>::load(ki + h * a.k_in_st.head) : sdv2::Vec8<T>::zero();
  }
  __shared__ float squares[4][2][64 * 8];
  float ssq_k, unused;
  sdv2::wave_sum_squares<T, kSteps>(k, k, a.heads, squares[threadIdx.x >> 6], lane, ssq_k, unused);
  if (lane == 0)
    a.inv_rms[static_cast<int64_t>(row) * a.tokens + tok] =
        1.0f / sqrtf(ssq_k / static_cast<float>(a.heads * 128) + a.norm_eps);
}

bool stride_ok(const sdv2_stride3& s, int vec) {
  return s.row % vec == 0 && s.token % vec == 0 && s.head % vec == 0;
}

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

size_t sums_bytes(int32_t rows, int32_t heads, int32_t sink_frames) {
  return static_cast<size_t>(rows) * (2 * static_cast<size_t>(sink_frames) + 2) * kTokenSplits * heads * SDV2_HEAD_DIM *
         sizeof(float);
}

}  // namespace

extern "C" size_t sdv2_sink_similarity_workspace_bytes(int32_t rows, int32_t tokens, int32_t heads,
                                                        int32_t sink_frames) {
  if (rows <= 0 || tokens <= 0 || heads <= 0 || sink_frames <= 0) return 0;
  // ticket words, token sums of every matrix of the call, then 1 / rms per new
  // key token (used with the norm folded in)
  return kTicketBytes + sums_bytes(rows, heads, sink_frames) + static_cast<size_t>(rows) * tokens * sizeof(float);
}

extern "C" size_t sdv2_sink_frame_sums_bytes(int32_t rows, int32_t heads, int32_t sink_frames) {
  if (rows <= 0 || heads <= 0 || sink_frames <= 0) return 0;
  return static_cast<size_t>(rows) * 2 * sink_frames * heads * SDV2_HEAD_DIM * sizeof(float);
}

extern "C" int sdv2_sink_similarity(const sdv2_sink_sim_params* p) {
  if (!p) return SDV2_ERR_INVALID_ARG;
  if (p->head_dim != SDV2_HEAD_DIM) return SDV2_ERR_UNSUPPORTED;
  if (p->dtype != SDV2_BF16 && p->dtype != SDV2_F32) return SDV2_ERR_UNSUPPORTED;
  if (p->rows <= 0 || p->rows > SDV2_MAX_ROWS || p->heads <= 0) return SDV2_ERR_INVALID_ARG;
  if (p->heads > kMaxHeads) return SDV2_ERR_UNSUPPORTED;
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
  const size_t need = sdv2_sink_similarity_workspace_bytes(p->rows, p->tokens, p->heads, p->sink_frames);
  if (!p->workspace || p->workspace_bytes < need || (reinterpret_cast<uintptr_t>(p->workspace) & 15))
    return SDV2_ERR_WORKSPACE;
  if (p->k_norm_weight && (!aligned16(p->k_norm_weight) || !(p->norm_eps >= 0.f))) return SDV2_ERR_INVALID_ARG;
  if (p->frame_sums) {
    if (reinterpret_cast<uintptr_t>(p->frame_sums) & 15) return SDV2_ERR_INVALID_ARG;
    if (!p->stale_frames || !p->planned_frame) return SDV2_ERR_INVALID_ARG;
    for (int i = 0; i < p->rows; ++i)
      if (p->planned_frame[i] < -1 || p->planned_frame[i] >= p->sink_frames) return SDV2_ERR_OUT_OF_RANGE;
  }

  SinkSimKernelArgs a{};
  a.k_in = p->k_in; a.v_in = p->v_in; a.k_cache = p->k_cache; a.v_cache = p->v_cache;
  a.k_in_st = p->k_in_stride; a.v_in_st = p->v_in_stride; a.k_st = p->k_cache_stride; a.v_st = p->v_cache_stride;
  a.freqs = reinterpret_cast<const double2*>(p->freqs);
  a.tickets = static_cast<int32_t*>(p->workspace);
  a.sums = reinterpret_cast<float*>(static_cast<char*>(p->workspace) + kTicketBytes);
  a.inv_rms = reinterpret_cast<float*>(static_cast<char*>(p->workspace) + kTicketBytes +
                                       sums_bytes(p->rows, p->heads, p->sink_frames));
  a.kept = p->frame_sums;
  a.k_norm_w = p->k_norm_weight;
  a.norm_eps = p->norm_eps;
  a.similarity = p->similarity;
  a.refresh = p->refresh;
  a.dst_override = p->dst_start_override;
  a.override_rows = p->override_rows;
  a.tokens = p->tokens; a.heads = p->heads; a.grid_w = p->grid_w; a.sink_frames = p->sink_frames;
  a.pairs = p->head_dim / 2;
  const int third = a.pairs / 3;
  a.split_t = a.pairs - 2 * third;
  a.split_h = a.split_t + third;
  a.threshold = p->threshold;
  for (int i = 0; i < p->rows; ++i) {
    a.start_frame[i] = p->start_frame[i];
    a.stale[i] = p->frame_sums ? p->stale_frames[i] : 0xffffffffu;
    a.planned_frame[i] = p->frame_sums ? p->planned_frame[i] : -1;
  }

  hipStream_t stream = static_cast<hipStream_t>(p->stream);
  const dim3 block(kThreads);
  // no frame of any row stale: the grid holds the new chunk's two matrices only (workgroups that
  // would find nothing to sum still cost their dispatch, and the ones that work start behind them)
  bool any_stale = false;
  for (int i = 0; i < p->rows; ++i) any_stale |= (a.stale[i] & ((1u << p->sink_frames) - 1u)) != 0;
  a.first_matrix = any_stale ? 0 : 2 * p->sink_frames;
  const dim3 grid(p->heads, 2 * p->sink_frames + 2 - a.first_matrix, p->rows * kTokenSplits);
  if (p->k_norm_weight) {
    const dim3 grid_rms((p->tokens + 3) / 4, 1, p->rows);
    const int steps = (p->heads + 3) / 4;
    auto launch = [&](auto steps_c) {
      constexpr int kS = decltype(steps_c)::value;
      if (p->dtype == SDV2_BF16) hipLaunchKernelGGL((key_inv_rms_kernel<uint16_t, kS>), grid_rms, dim3(256), 0, stream, a);
      else hipLaunchKernelGGL((key_inv_rms_kernel<float, kS>), grid_rms, dim3(256), 0, stream, a);
    };
    if (steps <= 4) launch(std::integral_constant<int, 4>{});
    else if (steps <= 10) launch(std::integral_constant<int, 10>{});
    else launch(std::integral_constant<int, 16>{});
  }
  // columns per thread of the deciding workgroup: 8 up to 16 heads, 20 up to 40, 32 up to 64
  auto launch = [&](auto cols_c) {
    constexpr int kCols = decltype(cols_c)::value;
    if (p->dtype == SDV2_BF16)
      sdv2::launch_timed(SDV2_KERNEL_SINK, sink_similarity_kernel<uint16_t, kCols>, grid, block, 0, stream, a);
    else
      sdv2::launch_timed(SDV2_KERNEL_SINK, sink_similarity_kernel<float, kCols>, grid, block, 0, stream, a);
  };
  const int width = p->heads * SDV2_HEAD_DIM;
  if (width <= 8 * kThreads) launch(std::integral_constant<int, 8>{});
  else if (width <= 20 * kThreads) launch(std::integral_constant<int, 20>{});
  else launch(std::integral_constant<int, 32>{});
  return hipGetLastError() == hipSuccess ? SDV2_OK : SDV2_ERR_LAUNCH;
}
