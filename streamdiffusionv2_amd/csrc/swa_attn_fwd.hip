// Sliding-window (sink + window) flash attention of a chunk's queries against
// the ring KV cache, for gfx950 (MI355X).
//
// Stands in for flash_attn_with_kvcache(q, k_cache, v_cache, cache_seqlens)
// as called at models/wan/causal_model.py:353-358: no mask inside the chunk,
// keys >= seq_lens[row] ignored.  The cache is read in place, in physical slot
// order — softmax attention does not depend on key order, so the ring never
// has to be unrolled.
//
// Work decomposition
//   workgroup = 4 waves, 128 query rows of one (row, head); wave w owns rows
//   32w..32w+31.  Keys stream through LDS in tiles of 64 (K 16 KB + V 16 KB,
//   double buffered, 64 KB per workgroup, two workgroups per CU).
//
// Matrix layout (v_mfma_f32_32x32x16_bf16, D = A(32x16) * B(16x32) + C):
//   S^T = K Q^T   A = K tile rows (16 B per lane straight from LDS),
//                 B = Q, held in registers for the whole kernel.
//   O^T = V^T P^T A = V^T read with ds_read_b64_tr_b16 (LDS transpose load),
//                 B = P^T, which is exactly the S^T accumulator layout after
//                 packing to bf16 — no cross-lane movement between the GEMMs.
//   In both products a lane owns ONE query (column lane%32), so the online
//   softmax statistics are per-lane scalars; the only cross-lane step is one
//   exchange between lane halves (v_permlane32_swap).
//
// LDS tile layout: row r (key) holds sixteen 16-byte chunks; chunk c is stored
// at position c ^ g(r), g(r) = ((r & 3) << 2) | ((r >> 2) & 3).  That makes the
// ds_read_b128 K reads (16 keys, one chunk) and the transposing V reads
// (4 keys x 64 bytes per half-wave) both bank-conflict free without padding.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <utility>

#include "sdv2kv.h"
#include "sdv2kv_internal.h"

namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) short s16x4;
typedef __attribute__((ext_vector_type(8))) short s16x8;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(2))) float f32x2;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;
typedef __attribute__((address_space(3))) char lds_char;

constexpr int kD = SDV2_HEAD_DIM;           // 128
constexpr int kWaves = 4;
constexpr int kThreads = kWaves * 64;
constexpr int kQRowsPerWave = 32;
constexpr int kQTile = kWaves * kQRowsPerWave;   // 128
constexpr int kKTile = 64;
constexpr int kTileBytes = kKTile * kD * 2;      // 16 KB per matrix
constexpr int kStageBytes = 2 * kTileBytes;      // K + V
constexpr float kLog2e = 1.4426950408889634f;

struct AttnKernelArgs {
  const uint16_t* q;
  const uint16_t* k;
  const uint16_t* v;
  uint16_t* out;
  const int32_t* seq_lens;
  sdv2_stride3 q_st, k_st, v_st, o_st;
  int32_t rows, q_tokens, heads, max_seq_len, num_splits;
  float scale_log2;            // softmax_scale * log2(e)
  float* part_o;               // [split][row][head][q][128] fp32, normalised
  float* part_lse;             // [split][row][head][q]      log2 sum exp
};

__device__ __forceinline__ int swz(int r) { return ((r & 3) << 2) | ((r >> 2) & 3); }

// max over the two lanes that share a query column (lane and lane ^ 32)
__device__ __forceinline__ float half_max(float x) {
  auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float half_sum(float x) {
  auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  // fptrunc <2 x float> -> <2 x bfloat> selects v_cvt_pk_bf16_f32 (nearest-even)
  const f32x2 x = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(x, bf16x2));
}

// ---------------------------------------------------------------------------
// Tile loader: global -> LDS without passing through registers
// (global_load_lds_dwordx4).  One wave-wide instruction deposits 64 x 16 bytes
// at consecutive LDS addresses, i.e. four 256-byte key rows.  Instruction i
// (0..15, four per wave) fills rows 4i..4i+3; lane l lands on row 4i + l/16,
// physical chunk l%16, so it must fetch logical chunk (l%16) ^ g(row).
// ---------------------------------------------------------------------------
// ---------------------------------------------------------------------------
// LDS reads with hand-placed waits.  The compiler treats every LDS access as
// possibly aliasing an in-flight global->LDS transfer and would drain all
// counters before each dependent MFMA; issuing the reads as asm and tying an
// explicit s_waitcnt to the fragment about to be consumed keeps several reads
// in flight behind the matrix pipe.  LDS returns data in issue order, so
// lgkmcnt(N) means "all but the newest N reads have landed".
// ---------------------------------------------------------------------------
template <int... I, typename F>
__device__ __forceinline__ void static_for_impl(std::integer_sequence<int, I...>, F&& f) {
  (f(std::integral_constant<int, I>{}), ...);
}
template <int N, typename F>
__device__ __forceinline__ void static_for(F&& f) {
  static_for_impl(std::make_integer_sequence<int, N>{}, f);
}

template <int kOffset>
__device__ __forceinline__ u32x4 lds_read_b128(uint32_t addr) {
  u32x4 r;
  asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(r) : "v"(addr), "n"(kOffset));
  return r;
}
template <int kOffset>
__device__ __forceinline__ u32x2 lds_read_tr16_b64(uint32_t addr) {
  u32x2 r;
  asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(r) : "v"(addr), "n"(kOffset));
  return r;
}
template <int kPending>
__device__ __forceinline__ void wait_lds(u32x4& frag) {
  asm volatile("s_waitcnt lgkmcnt(%1)" : "+v"(frag) : "n"(kPending));
}

struct LoaderOffsets {
  uint32_t k[4];   // byte offsets from the tile's first key row, per instruction
  uint32_t v[4];
};

__device__ __forceinline__ void dma16(const char* g, lds_char* l) {
  __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)g,
                                   (__attribute__((address_space(3))) void*)l, 16, 0, 0);
}

// full tile: every row is valid, addresses are tile base + precomputed offsets
__device__ __forceinline__ void load_tile_dma(const LoaderOffsets& o, const char* ktile, const char* vtile,
                                              lds_char* stage, int wave_u) {
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    dma16(ktile + o.k[j], stage + (wave_u * 4 + j) * 1024);
    dma16(vtile + o.v[j], stage + kTileBytes + (wave_u * 4 + j) * 1024);
  }
}

// last, partial tile: rows at or past the valid length are redirected to the
// last valid key (their scores are masked), so nothing outside the rows the
// caller declared valid is read.
__device__ __forceinline__ void load_tile_dma_tail(const char* kbase, const char* vbase, int64_t k_tok_bytes,
                                                   int64_t v_tok_bytes, int key0, int last_key,
                                                   lds_char* stage, int wave_u, int lane) {
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int r = 4 * (wave_u * 4 + j) + (lane >> 4);
    int key = key0 + r;
    key = key < last_key ? key : last_key;
    const int chunk = (lane & 15) ^ swz(r);
    dma16(kbase + key * k_tok_bytes + chunk * 16, stage + (wave_u * 4 + j) * 1024);
    dma16(vbase + key * v_tok_bytes + chunk * 16, stage + kTileBytes + (wave_u * 4 + j) * 1024);
  }
}

__device__ __forceinline__ void wait_vmem_and_sync() {
  __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0): this wave's DMA has landed
  __syncthreads();
}

struct SoftmaxState {
  float m;   // running max of the raw scores of this lane's query
  float l;   // this lane's share of the running sum
};

// One 64-key tile from LDS stage `kBuf` (compile-time, so every LDS address is
// register + immediate).
template <int kBuf>
__device__ __forceinline__ void process_tile(const uint32_t (&k_addr)[8], const uint32_t (&v_addr)[4][2],
                                             const bf16x8 (&qf)[8], f32x16 (&oacc)[4], SoftmaxState& st,
                                             float c2, int key0, int seq, int hf) {
  constexpr int kBase = kBuf * kStageBytes;
  constexpr int vBase = kBuf * kStageBytes + kTileBytes;

  // ---- S^T = K Q^T : two 32-key blocks --------------------------------
  // 16 MFMAs, the two accumulators alternating; K fragments are fetched from
  // LDS kAhead MFMAs ahead.  Step s covers d-step s/2 of key block s%2.
  f32x16 sacc[2];
#pragma unroll
  for (int kb = 0; kb < 2; ++kb)
#pragma unroll
    for (int i = 0; i < 16; ++i) sacc[kb][i] = 0.f;
  constexpr int kAhead = 4;
  u32x4 kf[16];
  static_for<kAhead>([&](auto ic) {
    constexpr int s = decltype(ic)::value;
    kf[s] = lds_read_b128<kBase + (s & 1) * 32 * 256>(k_addr[s >> 1]);
  });
  static_for<16>([&](auto ic) {
    constexpr int s = decltype(ic)::value;
    if constexpr (s + kAhead < 16)
      kf[s + kAhead] = lds_read_b128<kBase + ((s + kAhead) & 1) * 32 * 256>(k_addr[(s + kAhead) >> 1]);
    wait_lds<(s + kAhead < 16) ? kAhead : 15 - s>(kf[s]);
    sacc[s & 1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, kf[s]), qf[s >> 1],
                                                          sacc[s & 1], 0, 0, 0);
    __builtin_amdgcn_sched_barrier(0);
  });

  // first V^T fragments: issued now, they land while the softmax runs.
  // Step s covers key step s/4 (16 keys) and d block s%4.
  constexpr int vAhead = 4;
  u32x4 vf[16];
  auto v_frag = [&](auto ic) {
    constexpr int s = decltype(ic)::value;
    constexpr int kk = s >> 2, db = s & 3;
    const u32x2 lo = lds_read_tr16_b64<vBase + kk * 16 * 256>(v_addr[db][0]);
    const u32x2 hi = lds_read_tr16_b64<vBase + kk * 16 * 256>(v_addr[db][1]);
    vf[s] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3);
  };
  static_for<vAhead>(v_frag);
  __builtin_amdgcn_sched_barrier(0);

  // ---- mask the tail of the last tile ---------------------------------
  if (key0 + kKTile > seq) {
#pragma unroll
    for (int kb = 0; kb < 2; ++kb)
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int key = key0 + kb * 32 + 8 * (i >> 2) + 4 * hf + (i & 3);
        if (key >= seq) sacc[kb][i] = -INFINITY;
      }
  }

  // ---- online softmax, one query per lane ------------------------------
  float mloc = sacc[0][0];
#pragma unroll
  for (int kb = 0; kb < 2; ++kb)
#pragma unroll
    for (int i = 0; i < 16; ++i) mloc = fmaxf(mloc, sacc[kb][i]);
  mloc = half_max(mloc);
  const float m_new = fmaxf(st.m, mloc);
  const float alpha = __builtin_amdgcn_exp2f((st.m - m_new) * c2);
  const float mc = m_new * c2;
  st.m = m_new;
  float psum = 0.f;
#pragma unroll
  for (int kb = 0; kb < 2; ++kb)
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const float p = __builtin_amdgcn_exp2f(__builtin_fmaf(sacc[kb][i], c2, -mc));
      sacc[kb][i] = p;
      psum += p;
    }
  st.l = st.l * alpha + psum;
  if (__builtin_amdgcn_ballot_w64(alpha != 1.0f) != 0) {
#pragma unroll
    for (int db = 0; db < 4; ++db)
#pragma unroll
      for (int i = 0; i < 16; ++i) oacc[db][i] *= alpha;
  }

  // ---- P^T as the B operand: accumulator registers 8*step..8*step+7 ----
  bf16x8 pf[2][2];
#pragma unroll
  for (int kb = 0; kb < 2; ++kb)
#pragma unroll
    for (int s2 = 0; s2 < 2; ++s2) {
      union { uint32_t u[4]; bf16x8 v; } pk;
#pragma unroll
      for (int j = 0; j < 4; ++j)
        pk.u[j] = pack_bf16x2(sacc[kb][8 * s2 + 2 * j], sacc[kb][8 * s2 + 2 * j + 1]);
      pf[kb][s2] = pk.v;
    }

  // ---- O^T += V^T P^T ----------------------------------------------------
  __builtin_amdgcn_sched_barrier(0);
  static_for<16>([&](auto ic) {
    constexpr int s = decltype(ic)::value;
    if constexpr (s + vAhead < 16) v_frag(std::integral_constant<int, s + vAhead>{});
    wait_lds<(s + vAhead < 16) ? 2 * vAhead : 2 * (15 - s)>(vf[s]);
    constexpr int kk = s >> 2, db = s & 3;
    oacc[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, vf[s]), pf[kk >> 1][kk & 1],
                                                       oacc[db], 0, 0, 0);
    __builtin_amdgcn_sched_barrier(0);
  });
}

__global__ __launch_bounds__(kThreads, 2)
void swa_attn_fwd_kernel(const AttnKernelArgs a) {
  __shared__ __attribute__((aligned(1024))) char smem[2 * kStageBytes];
  lds_char* lds = (lds_char*)smem;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wave_u = __builtin_amdgcn_readfirstlane(wave);
  const int hf = lane >> 5;                 // which half of the wave
  const int qtile = blockIdx.x;
  const int head = blockIdx.y;
  const int row = blockIdx.z / a.num_splits;
  const int split = blockIdx.z - row * a.num_splits;

  int seq = a.seq_lens ? a.seq_lens[row] : a.max_seq_len;
  seq = seq < a.max_seq_len ? seq : a.max_seq_len;
  seq = seq < 0 ? 0 : seq;
  const int ntiles = (seq + kKTile - 1) / kKTile;
  const int per_split = (ntiles + a.num_splits - 1) / a.num_splits;
  const int tile_begin = split * per_split;
  int tile_end = tile_begin + per_split;
  tile_end = tile_end < ntiles ? tile_end : ntiles;

  const char* kbase = reinterpret_cast<const char*>(a.k + row * a.k_st.row + head * a.k_st.head);
  const char* vbase = reinterpret_cast<const char*>(a.v + row * a.v_st.row + head * a.v_st.head);
  const int64_t k_tok_bytes = a.k_st.token * 2;
  const int64_t v_tok_bytes = a.v_st.token * 2;

  LoaderOffsets lo;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int r = 4 * (wave * 4 + j) + (lane >> 4);
    const int chunk = (lane & 15) ^ swz(r);
    lo.k[j] = (uint32_t)(r * k_tok_bytes + chunk * 16);
    lo.v[j] = (uint32_t)(r * v_tok_bytes + chunk * 16);
  }

  auto issue_tile = [&](int t, int buf) {
    const int key0 = t * kKTile;
    lds_char* stage = lds + buf * kStageBytes;
    if (key0 + kKTile <= seq)
      load_tile_dma(lo, kbase + key0 * k_tok_bytes, vbase + key0 * v_tok_bytes, stage, wave_u);
    else
      load_tile_dma_tail(kbase, vbase, k_tok_bytes, v_tok_bytes, key0, seq - 1, stage, wave_u, lane);
  };

  if (tile_begin < tile_end) issue_tile(tile_begin, 0);

  // ---- this lane's query row, as the B operand of S^T = K Q^T -------------
  const int q_row = qtile * kQTile + wave * kQRowsPerWave + (lane & 31);
  const int q_row_c = q_row < a.q_tokens ? q_row : a.q_tokens - 1;
  const uint16_t* qp = a.q + row * a.q_st.row + (int64_t)q_row_c * a.q_st.token + head * a.q_st.head + 8 * hf;
  bf16x8 qf[8];
#pragma unroll
  for (int ks = 0; ks < 8; ++ks) qf[ks] = *reinterpret_cast<const bf16x8*>(qp + 16 * ks);

  // ---- per-lane LDS read offsets -------------------------------------------
  // K (A operand): key = kb*32 + lane%32, chunk = 2*ks + hf
  const uint32_t lds_addr0 = (uint32_t)(uintptr_t)lds;
  uint32_t k_addr[8];
  {
    const int r = lane & 31;
    const int base = r * 256 + ((hf ^ swz(r)) << 4);
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) k_addr[ks] = lds_addr0 + (uint32_t)(base ^ (ks << 5));
  }
  // V^T (A operand) through the transposing read: in each group of 16 lanes,
  // lane i supplies the address of key (i / 4), 8 bytes at d-offset 4 * (i % 4);
  // it receives d = i, keys 0..3.  Group = (hf, dhalf).
  uint32_t v_addr[4][2];
  {
    const int i16 = lane & 15;
    const int dhalf = (lane >> 4) & 1;
    const int krow = i16 >> 2;
#pragma unroll
    for (int db = 0; db < 4; ++db)
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        const int r = 8 * j + 4 * hf + krow;                 // + 16 * kk added as an immediate
        const int c = db * 4 + dhalf * 2 + ((i16 & 3) >> 1);
        v_addr[db][j] = lds_addr0 + (uint32_t)(r * 256 + ((c ^ swz(r)) << 4) + (i16 & 1) * 8);
      }
  }

  f32x16 oacc[4];
#pragma unroll
  for (int db = 0; db < 4; ++db)
#pragma unroll
    for (int i = 0; i < 16; ++i) oacc[db][i] = 0.f;
  SoftmaxState st{-INFINITY, 0.f};
  const float c2 = a.scale_log2;

  wait_vmem_and_sync();   // first tile and the Q fragments have arrived

  // Two tiles per trip so the LDS stage is a compile-time constant.
  for (int t = tile_begin; t < tile_end; t += 2) {
    if (t + 1 < tile_end) issue_tile(t + 1, 1);
    process_tile<0>(k_addr, v_addr, qf, oacc, st, c2, t * kKTile, seq, hf);
    wait_vmem_and_sync();
    if (t + 1 >= tile_end) break;
    if (t + 2 < tile_end) issue_tile(t + 2, 0);
    process_tile<1>(k_addr, v_addr, qf, oacc, st, c2, (t + 1) * kKTile, seq, hf);
    wait_vmem_and_sync();
  }

  float m_run = st.m;
  float l_run = st.l;

  // ---- epilogue ---------------------------------------------------------------
  const float l_tot = half_sum(l_run);
  const float inv = l_tot > 0.f ? 1.0f / l_tot : 0.f;
  if (q_row >= a.q_tokens) return;

  if (a.num_splits == 1) {
    uint16_t* op = a.out + row * a.o_st.row + (int64_t)q_row * a.o_st.token + head * a.o_st.head;
#pragma unroll
    for (int db = 0; db < 4; ++db)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        uint2 w;
        w.x = pack_bf16x2(oacc[db][4 * g] * inv, oacc[db][4 * g + 1] * inv);
        w.y = pack_bf16x2(oacc[db][4 * g + 2] * inv, oacc[db][4 * g + 3] * inv);
        *reinterpret_cast<uint2*>(op + db * 32 + 8 * g + 4 * hf) = w;
      }
  } else {
    const int64_t prow = (((int64_t)split * a.rows + row) * a.heads + head) * a.q_tokens + q_row;
    float* po = a.part_o + prow * kD;
#pragma unroll
    for (int db = 0; db < 4; ++db)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        float4 w;
        w.x = oacc[db][4 * g] * inv;
        w.y = oacc[db][4 * g + 1] * inv;
        w.z = oacc[db][4 * g + 2] * inv;
        w.w = oacc[db][4 * g + 3] * inv;
        *reinterpret_cast<float4*>(po + db * 32 + 8 * g + 4 * hf) = w;
      }
    if (hf == 0)
      a.part_lse[prow] = l_tot > 0.f ? m_run * c2 + __builtin_amdgcn_logf(l_tot) : -INFINITY;
  }
}

// Combine the per-split partial results: out = sum_s 2^(lse_s - LSE) O_s.
// One 16-lane group per (row, head, query); each lane owns 8 of the 128 dims.
__global__ __launch_bounds__(256)
void swa_attn_merge_kernel(const AttnKernelArgs a) {
  const int64_t nq = (int64_t)a.rows * a.heads * a.q_tokens;
  const int64_t idx = (int64_t)blockIdx.x * 16 + (threadIdx.x >> 4);
  if (idx >= nq) return;
  const int lane = threadIdx.x & 15;
  const int q_row = (int)(idx % a.q_tokens);
  const int head = (int)((idx / a.q_tokens) % a.heads);
  const int row = (int)(idx / ((int64_t)a.q_tokens * a.heads));

  float lse_max = -INFINITY;
  for (int s = 0; s < a.num_splits; ++s) lse_max = fmaxf(lse_max, a.part_lse[s * nq + idx]);
  float acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
  float wsum = 0.f;
  for (int s = 0; s < a.num_splits; ++s) {
    const float lse = a.part_lse[s * nq + idx];
    const float w = lse == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(lse - lse_max);
    wsum += w;
    const float4* po = reinterpret_cast<const float4*>(a.part_o + (s * nq + idx) * kD + lane * 8);
    const float4 x = po[0], y = po[1];
    acc[0] += w * x.x; acc[1] += w * x.y; acc[2] += w * x.z; acc[3] += w * x.w;
    acc[4] += w * y.x; acc[5] += w * y.y; acc[6] += w * y.z; acc[7] += w * y.w;
  }
  const float inv = wsum > 0.f ? 1.0f / wsum : 0.f;
  uint4 o;
  o.x = pack_bf16x2(acc[0] * inv, acc[1] * inv);
  o.y = pack_bf16x2(acc[2] * inv, acc[3] * inv);
  o.z = pack_bf16x2(acc[4] * inv, acc[5] * inv);
  o.w = pack_bf16x2(acc[6] * inv, acc[7] * inv);
  uint16_t* op = a.out + row * a.o_st.row + (int64_t)q_row * a.o_st.token + head * a.o_st.head + lane * 8;
  *reinterpret_cast<uint4*>(op) = o;
}

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }
bool stride_ok(const sdv2_stride3& s) { return s.row % 8 == 0 && s.token % 8 == 0 && s.head % 8 == 0; }

size_t align_up(size_t x, size_t a) { return (x + a - 1) / a * a; }

}  // namespace

extern "C" int sdv2_swa_attn_default_splits(int32_t rows, int32_t q_tokens, int32_t heads, int32_t max_seq_len) {
  if (rows <= 0 || q_tokens <= 0 || heads <= 0 || max_seq_len <= 0) return 1;
  // 256 CUs x 2 resident workgroups
  const int64_t slots = 512;
  const int64_t qwork = (int64_t)rows * heads * ((q_tokens + kQTile - 1) / kQTile);
  const int ntiles = (max_seq_len + kKTile - 1) / kKTile;
  int64_t splits = slots / qwork;
  if (splits < 1) splits = 1;
  if (splits > 8) splits = 8;
  if (splits > ntiles / 8) splits = ntiles / 8 > 0 ? ntiles / 8 : 1;
  return (int)splits;
}

extern "C" size_t sdv2_swa_attn_workspace_bytes(int32_t rows, int32_t q_tokens, int32_t heads,
                                                 int32_t max_seq_len, int32_t num_splits) {
  if (num_splits <= 0) num_splits = sdv2_swa_attn_default_splits(rows, q_tokens, heads, max_seq_len);
  if (num_splits <= 1) return 0;
  const size_t nq = (size_t)rows * heads * q_tokens;
  return align_up((size_t)num_splits * nq * kD * sizeof(float), 256) +
         align_up((size_t)num_splits * nq * sizeof(float), 256);
}

extern "C" int sdv2_swa_attn_fwd(const sdv2_attn_params* p) {
  if (!p) return SDV2_ERR_INVALID_ARG;
  if (p->head_dim != kD) return SDV2_ERR_UNSUPPORTED;
  if (p->rows < 0 || p->q_tokens < 0 || p->heads <= 0 || p->max_seq_len < 0) return SDV2_ERR_INVALID_ARG;
  if (p->rows == 0 || p->q_tokens == 0) return SDV2_OK;
  if (!p->q || !p->k_cache || !p->v_cache || !p->out) return SDV2_ERR_INVALID_ARG;
  if (!aligned16(p->q) || !aligned16(p->k_cache) || !aligned16(p->v_cache) || !aligned16(p->out))
    return SDV2_ERR_INVALID_ARG;
  if (!stride_ok(p->q_stride) || !stride_ok(p->k_stride) || !stride_ok(p->v_stride) || !stride_ok(p->out_stride))
    return SDV2_ERR_INVALID_ARG;
  if (p->rows > 65535 / 8 || p->heads > 65535) return SDV2_ERR_INVALID_ARG;

  int splits = p->num_splits > 0 ? p->num_splits
                                 : sdv2_swa_attn_default_splits(p->rows, p->q_tokens, p->heads, p->max_seq_len);
  if (splits > 64) return SDV2_ERR_INVALID_ARG;
  if (p->stages < SDV2_STAGE_ALL || p->stages > SDV2_STAGE_MERGE) return SDV2_ERR_INVALID_ARG;
  if (p->stages != SDV2_STAGE_ALL && splits == 1) return SDV2_ERR_INVALID_ARG;
  if ((int64_t)p->rows * splits > 65535) return SDV2_ERR_INVALID_ARG;

  AttnKernelArgs a{};
  a.q = static_cast<const uint16_t*>(p->q);
  a.k = static_cast<const uint16_t*>(p->k_cache);
  a.v = static_cast<const uint16_t*>(p->v_cache);
  a.out = static_cast<uint16_t*>(p->out);
  a.seq_lens = p->seq_lens;
  a.q_st = p->q_stride; a.k_st = p->k_stride; a.v_st = p->v_stride; a.o_st = p->out_stride;
  a.rows = p->rows; a.q_tokens = p->q_tokens; a.heads = p->heads; a.max_seq_len = p->max_seq_len;
  a.num_splits = splits;
  const float scale = p->softmax_scale > 0.f ? p->softmax_scale : 0.08838834764831845f;  // 1/sqrt(128)
  a.scale_log2 = scale * kLog2e;

  if (splits > 1) {
    const size_t need = sdv2_swa_attn_workspace_bytes(p->rows, p->q_tokens, p->heads, p->max_seq_len, splits);
    if (!p->workspace || p->workspace_bytes < need) return SDV2_ERR_WORKSPACE;
    if (reinterpret_cast<uintptr_t>(p->workspace) & 255) return SDV2_ERR_INVALID_ARG;
    const size_t nq = (size_t)p->rows * p->heads * p->q_tokens;
    a.part_o = static_cast<float*>(p->workspace);
    a.part_lse = reinterpret_cast<float*>(static_cast<char*>(p->workspace) +
                                          align_up((size_t)splits * nq * kD * sizeof(float), 256));
  }

  hipStream_t stream = static_cast<hipStream_t>(p->stream);
  dim3 grid((p->q_tokens + kQTile - 1) / kQTile, p->heads, p->rows * splits);
  if (p->stages != SDV2_STAGE_MERGE) {
    hipLaunchKernelGGL(swa_attn_fwd_kernel, grid, dim3(kThreads), 0, stream, a);
    if (hipGetLastError() != hipSuccess) return SDV2_ERR_LAUNCH;
  }
  if (splits > 1 && p->stages != SDV2_STAGE_PARTIAL) {
    const int64_t nq = (int64_t)p->rows * p->heads * p->q_tokens;
    hipLaunchKernelGGL(swa_attn_merge_kernel, dim3((unsigned)((nq + 15) / 16)), dim3(256), 0, stream, a);
    if (hipGetLastError() != hipSuccess) return SDV2_ERR_LAUNCH;
  }
  return SDV2_OK;
}
