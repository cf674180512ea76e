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

struct TileRegs {
  u32x4 k[4];
  u32x4 v[4];
};

// Each thread moves four 16-byte chunks of K and of V per tile: rows
// tid/16 + 16 i, chunk tid % 16.  Rows past the valid length are clamped to
// the last valid key (their scores are masked later), so nothing is read
// outside the rows the caller declared valid.
__device__ __forceinline__ void load_tile(TileRegs& t, const uint16_t* kbase, const uint16_t* vbase,
                                          int64_t k_tok_stride, int64_t v_tok_stride,
                                          int key0, int last_key, int tid) {
  const int c = tid & 15;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    int key = key0 + (tid >> 4) + 16 * i;
    key = key < last_key ? key : last_key;
    t.k[i] = *reinterpret_cast<const u32x4*>(kbase + key * k_tok_stride + c * 8);
    t.v[i] = *reinterpret_cast<const u32x4*>(vbase + key * v_tok_stride + c * 8);
  }
}

__device__ __forceinline__ void store_tile(const TileRegs& t, lds_char* stage, int tid) {
  const int c = tid & 15;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = (tid >> 4) + 16 * i;
    const int off = r * 256 + ((c ^ swz(r)) << 4);
    *reinterpret_cast<__attribute__((address_space(3))) u32x4*>(stage + off) = t.k[i];
    *reinterpret_cast<__attribute__((address_space(3))) u32x4*>(stage + kTileBytes + off) = t.v[i];
  }
}

__global__ __launch_bounds__(kThreads, 2)
void swa_attn_fwd_kernel(const AttnKernelArgs a) {
  __shared__ __attribute__((aligned(1024))) char smem[2 * kStageBytes];
  lds_char* lds = (lds_char*)smem;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
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

  // ---- this lane's query row, as the B operand of S^T = K Q^T -------------
  const int q_row = qtile * kQTile + wave * kQRowsPerWave + (lane & 31);
  const int q_row_c = q_row < a.q_tokens ? q_row : a.q_tokens - 1;
  const uint16_t* qp = a.q + row * a.q_st.row + (int64_t)q_row_c * a.q_st.token + head * a.q_st.head + 8 * hf;
  bf16x8 qf[8];
#pragma unroll
  for (int ks = 0; ks < 8; ++ks) qf[ks] = *reinterpret_cast<const bf16x8*>(qp + 16 * ks);

  const uint16_t* kbase = a.k + row * a.k_st.row + head * a.k_st.head;
  const uint16_t* vbase = a.v + row * a.v_st.row + head * a.v_st.head;

  // ---- per-lane LDS read offsets -------------------------------------------
  // K (A operand): key = kb*32 + lane%32, chunk = 2*ks + hf
  int k_off[8];
  {
    const int r = lane & 31;
    const int base = r * 256 + ((hf ^ swz(r)) << 4);
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) k_off[ks] = base ^ (ks << 5);
  }
  // V^T (A operand) through the transposing read: in each group of 16 lanes,
  // lane i supplies the address of key (i / 4), 8 bytes at d-offset 4 * (i % 4);
  // it receives d = i, keys 0..3.  Group = (hf, dhalf).
  int v_off[4][2];
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
        v_off[db][j] = kTileBytes + r * 256 + ((c ^ swz(r)) << 4) + (i16 & 1) * 8;
      }
  }

  f32x16 oacc[4];
#pragma unroll
  for (int db = 0; db < 4; ++db)
#pragma unroll
    for (int i = 0; i < 16; ++i) oacc[db][i] = 0.f;
  float m_run = -INFINITY;    // running max of raw scores (this lane's query)
  float l_run = 0.f;          // this lane's share of the running sum

  const float c2 = a.scale_log2;

  if (tile_begin < tile_end) {
    TileRegs stage_regs;
    load_tile(stage_regs, kbase, vbase, a.k_st.token, a.v_st.token, tile_begin * kKTile, seq - 1, tid);
    store_tile(stage_regs, lds, tid);
    __syncthreads();

    for (int t = tile_begin; t < tile_end; ++t) {
      const int buf = (t - tile_begin) & 1;
      lds_char* cur = lds + buf * kStageBytes;
      const bool has_next = t + 1 < tile_end;
      if (has_next)
        load_tile(stage_regs, kbase, vbase, a.k_st.token, a.v_st.token, (t + 1) * kKTile, seq - 1, tid);

      // ---- S^T = K Q^T : two 32-key blocks --------------------------------
      f32x16 sacc[2];
#pragma unroll
      for (int kb = 0; kb < 2; ++kb) {
#pragma unroll
        for (int i = 0; i < 16; ++i) sacc[kb][i] = 0.f;
#pragma unroll
        for (int ks = 0; ks < 8; ++ks) {
          const bf16x8 kf = *reinterpret_cast<__attribute__((address_space(3))) const bf16x8*>(
              cur + k_off[ks] + kb * 32 * 256);
          sacc[kb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf, qf[ks], sacc[kb], 0, 0, 0);
        }
      }

      // ---- mask the tail of the last tile ---------------------------------
      const int key0 = t * kKTile;
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
      const float m_new = fmaxf(m_run, mloc);
      const float alpha = __builtin_amdgcn_exp2f((m_run - m_new) * c2);
      const float mc = m_new * c2;
      m_run = m_new;
      float psum = 0.f;
#pragma unroll
      for (int kb = 0; kb < 2; ++kb)
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          const float p = __builtin_amdgcn_exp2f(__builtin_fmaf(sacc[kb][i], c2, -mc));
          sacc[kb][i] = p;
          psum += p;
        }
      l_run = l_run * alpha + psum;
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
        for (int st = 0; st < 2; ++st) {
          union { uint32_t u[4]; bf16x8 v; } pk;
#pragma unroll
          for (int j = 0; j < 4; ++j)
            pk.u[j] = pack_bf16x2(sacc[kb][8 * st + 2 * j], sacc[kb][8 * st + 2 * j + 1]);
          pf[kb][st] = pk.v;
        }

      // ---- O^T += V^T P^T ----------------------------------------------------
#pragma unroll
      for (int kk = 0; kk < 4; ++kk) {
#pragma unroll
        for (int db = 0; db < 4; ++db) {
          const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
              (__attribute__((address_space(3))) s16x4*)(cur + v_off[db][0] + kk * 16 * 256));
          const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
              (__attribute__((address_space(3))) s16x4*)(cur + v_off[db][1] + kk * 16 * 256));
          const s16x8 both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
          oacc[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
              __builtin_bit_cast(bf16x8, both), pf[kk >> 1][kk & 1], oacc[db], 0, 0, 0);
        }
      }

      if (has_next) store_tile(stage_regs, lds + (buf ^ 1) * kStageBytes, tid);
      __syncthreads();
    }
  }

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
