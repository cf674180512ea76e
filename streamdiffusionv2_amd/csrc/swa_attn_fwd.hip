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
//   workgroup = 8 waves = 256 query rows of one (row, head), one workgroup per
//   CU, two waves per SIMD with 256 registers each; wave w owns the 32-row
//   block 32w..32w+31.  While one wave of a SIMD is held up (issuing its
//   global->LDS transfers, at the barrier, waiting for an LDS fragment) the
//   other keeps the matrix pipe fed.  Keys stream through LDS in tiles of
//   64 (K 16 KB + V 16 KB), three buffers each, filled two tiles ahead by
//   global->LDS transfers that never touch registers.
//
//   Long caches are split over key ranges so that the grid fills the chip.
//   Every workgroup of a split call leaves its (normalised output, log-sum-exp)
//   in the workspace and takes a ticket; the workgroup that draws the last
//   ticket of a (row, head, query tile) combines all ranges and writes the
//   result, so a split call is still one launch.
//
// Matrix layout (v_mfma_f32_32x32x16_bf16, D = A(32x16) * B(16x32) + C):
//   S^T = K Q^T   A = K tile rows (ds_read_b128), B = Q, in registers for the
//                 whole kernel.
//   O^T = V^T P^T A = V^T read with ds_read_b64_tr_b16 (LDS transpose load),
//                 B = P^T, which is exactly the S^T accumulator layout after
//                 packing to bf16 — no cross-lane movement between the GEMMs.
//   In both products a lane owns ONE query per block (column lane%32), so the
//   softmax statistics are per-lane scalars.
//
// Softmax.  exp2 of the scaled scores is taken against a FIXED reference per
// query row, the largest score among the first 32 keys of the workgroup's
// range, instead of a running maximum: nothing is ever rescaled, and the
// weights stay in fp32 / bf16 range as long as no later score exceeds that
// reference by about 100 in log2 units (69 in natural units).  Each wave checks
// its row sums after its last tile; a wave that finds one outside [2^-100,
// 2^100] (or NaN) throws its block away and recomputes it with the
// conventional running-maximum recurrence (slower, exact for any finite
// input) while the other waves only keep the tiles coming.
//
// LDS tile layout: row r (key) holds sixteen 16-byte chunks; chunk c is stored
// at position c ^ g(r), g(r) = ((r & 3) << 2) | ((r >> 2) & 3).  That makes the
// ds_read_b128 K reads (16 keys, one chunk) and the transposing V reads
// (4 keys x 64 bytes per half-wave) both bank-conflict free without padding.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>
#include <mutex>
#include <utility>

#include "sdv2kv.h"
#include "sdv2kv_profile.h"
#include "sdv2kv_internal.h"
#include "rope_device.h"

namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(4))) short s16x4;
typedef __attribute__((ext_vector_type(8))) short s16x8;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(2))) float f32x2;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;
typedef __attribute__((ext_vector_type(2))) _Float16 f16x2;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8;
typedef __attribute__((address_space(3))) char lds_char;
typedef __attribute__((address_space(3))) int lds_int;

constexpr int kD = SDV2_HEAD_DIM;           // 128
constexpr int kWaves = 8;                   // two waves per SIMD, one 32-row query block each
constexpr int kThreads = kWaves * 64;
// The global->LDS transfers of a tile are issued by the first wave of every
// SIMD only (waves 0-3).  A wave is held while its transfers queue up; with all
// eight issuing, both waves of a SIMD are held at the same moment right after
// the barrier, with four the other one keeps the matrix pipe fed (measured
// 0.5-1.5 % faster; two or one issuing waves fall far behind the rest).
constexpr int kIssuers = 4;
constexpr int kPieces = 16 / kIssuers;      // global->LDS instructions per issuing wave and matrix tile
constexpr int kQBlock = 32;                 // query rows per wave
constexpr int kQTile = kWaves * kQBlock;    // 256
constexpr int kKTile = 64;
constexpr int kTileBytes = kKTile * kD * 2; // 16 KB per matrix
constexpr int kStages = 3;
constexpr int kStageBytes = 16384;          // epilogue staging per wave: 32 rows x 512 B
// Two flag words of the workgroup sit behind the tile buffers and the staging
// areas, so that setting and reading them needs no barrier of its own.
constexpr int kLdsFlags = 2 * kStages * kTileBytes > kWaves * kStageBytes ? 2 * kStages * kTileBytes
                                                                         : kWaves * kStageBytes;
constexpr int kLdsBytes = kLdsFlags + 256;
constexpr float kLog2e = 1.4426950408889634f;
constexpr int kCuSlots = 256;               // one workgroup per CU
constexpr int kMaxDevices = 64;
constexpr int kPartBlockHalves = kQBlock * kD;   // one block's partial output: 32 x 128 fp16 = 8 KB
// The ticket words of a split call sit in a region of FIXED size at the head of
// the workspace, whatever the shape: a region that grew with the shape would
// overlap, for a larger call, what an earlier smaller call left of its partial
// results, and tickets must be zero when a call starts.
constexpr int kMaxTickets = 16384;               // (row, head, query tile) groups of a split call

// LDS map: kStages K tile buffers, then kStages V tile buffers.  The DS
// instructions carry a 16-bit offset, so V fragment addresses are kept
// relative to the first V buffer (kLdsVRel) with the base folded into the
// per-lane address register.
constexpr int kLdsK(int buf) { return buf * kTileBytes; }
constexpr int kLdsVBase = kStages * kTileBytes;
constexpr int kLdsVRel(int buf) { return buf * kTileBytes; }
constexpr int kLdsV(int buf) { return kLdsVBase + kLdsVRel(buf); }

struct AttnKernelArgs {
  const uint16_t* q;
  const uint16_t* k;
  const uint16_t* v;
  uint16_t* out;
  const int32_t* seq_lens;
  sdv2_stride3 q_st, k_st, v_st, o_st;
  int32_t rows, q_tokens, heads, max_seq_len;
  // Key ranges per (row, head): num_splits, except that of every group_pairs
  // consecutive (row, head) pairs the last more_pairs take num_splits + 1.
  // (Uniform: group_pairs = rows * heads, more_pairs = 0.)
  int32_t num_splits, group_pairs, more_pairs;
  float scale_log2;            // softmax_scale * log2(e)
  int32_t mask_block_tokens;   // 0 = no mask inside the chunk
  const int32_t* chunk_start;  // device [rows]: cache position of the chunk's own first key
  // Split calls.  Partial results are kept per 32-row query block in the order
  // the registers hold them (see store_partial), q_blocks = ceil(q_tokens / 32).
  int32_t q_blocks;
  int32_t* tickets;            // [row][head][query tile], zero between calls
  uint16_t* part_o;            // [split][row][head][block][8 KB] fp16: normalised output / row scale
  float* part_lse;             // [split][row][head][block][32]   log2 sum exp
  float* part_scale;           // [split][row][head][block][32]   largest magnitude of the normalised row
  // Rotation of the queries inside the kernel (q is then the chunk's query
  // BEFORE RoPE): the complex128 table, or null when q arrives rotated.
  const double2* freqs;
  int32_t grid_w, frame_tokens, split_t, split_h;
  int64_t start_frame[SDV2_MAX_ROWS];
  // RMSNorm of the queries inside the kernel (q is then the raw projection):
  // the norm weight [heads * 128] and 1 / rms per (row, token), or null
  const uint16_t* q_norm_w;
  const float* q_inv_rms;
};

__device__ __forceinline__ int swz(int r) { return ((r & 3) << 2) | ((r >> 2) & 3); }

// v_max without the NaN-quieting canonicalisation fmaxf() drags in.
__device__ __forceinline__ float vmax(float a, float b) {
  float r;
  asm("v_max_f32 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
  return r;
}

// exchange between the two lanes that share a query column (lane and lane ^ 32)
__device__ __forceinline__ float half_max(float x) {
  auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return vmax(__uint_as_float(r[0]), __uint_as_float(r[1]));
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

// two floats -> packed fp16 pair (lo in the low half), nearest-even
__device__ __forceinline__ uint32_t pack_f16x2(float lo, float hi) {
  const f32x2 x = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(x, f16x2));
}

// acc + lo + hi of a packed bf16 pair (v_dot2c_f32_bf16 against (1, 1))
__device__ __forceinline__ float add_bf16_pair(uint32_t packed, float acc) {
  const bf16x2 ones = {(__bf16)1.0f, (__bf16)1.0f};
  return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, packed), ones, acc, false);
}

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
// The same reads for the exact pass, which is not pipelined: the value is
// waited for inside the statement and handed to compiler-generated MFMAs.
// (Absolute per-lane addresses as in the fast pass: taking them relative to
// the LDS base would keep a second copy of all sixteen alive across the
// streaming loop.)
__device__ __forceinline__ bf16x8 lds_read_b128_now(uint32_t addr) {
  u32x4 r;
  asm volatile("ds_read_b128 %0, %1\n\ts_waitcnt lgkmcnt(0)" : "=v"(r) : "v"(addr) : "memory");
  return __builtin_bit_cast(bf16x8, r);
}
__device__ __forceinline__ bf16x8 lds_read_tr16_b64x2_now(uint32_t addr_lo, uint32_t addr_hi) {
  u32x2 lo, hi;
  asm volatile("ds_read_b64_tr_b16 %0, %2\n\tds_read_b64_tr_b16 %1, %3\n\ts_waitcnt lgkmcnt(0)"
               : "=&v"(lo), "=&v"(hi) : "v"(addr_lo), "v"(addr_hi) : "memory");
  return __builtin_bit_cast(bf16x8, __builtin_shufflevector(lo, hi, 0, 1, 2, 3));
}
// Optimisation passes may sink pure arithmetic down to its first use, which
// here is a whole pipeline slot later.  Passing a value through an empty
// volatile asm fixes the point by which it has to be computed.
__device__ __forceinline__ void pin(float& x) { asm volatile("" : "+v"(x)); }
__device__ __forceinline__ void pin(uint32_t& x) { asm volatile("" : "+v"(x)); }

// The MFMAs of the fast pass are asm as well.  Left to itself the
// compiler keeps every MFMA accumulator in the accumulation registers, but the
// scores feed the vector ALU (which cannot read those) while the output tile
// never does until the epilogue; naming the register class per product puts S
// in VGPRs and O (with the Q fragments beside it: at 256 registers per wave at
// most 128 are VGPRs) in AGPRs.  `kPending` is the s_waitcnt that makes the A
// fragment valid (reads issued after it that may still be in flight); -1 = the
// fragment was already waited for.  Nothing here is covered by the compiler's
// hazard tracking: S is read by the vector ALU a full slot after its last
// MFMA, P is written a full slot before the MFMA that reads it, and O is only
// read after the final barrier, all far beyond the required wait states.
template <int kPending>
__device__ __forceinline__ void mfma_s_first(f32x16& d, const u32x4& a, const bf16x8& b) {
  if constexpr (kPending >= 0)
    asm volatile("s_waitcnt lgkmcnt(%3)\n\tv_mfma_f32_32x32x16_bf16 %0, %1, %2, 0"
                 : "=&v"(d) : "v"(a), "a"(b), "n"(kPending));
  else
    asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, 0" : "=&v"(d) : "v"(a), "a"(b));
}
template <int kPending>
__device__ __forceinline__ void mfma_s(f32x16& d, const u32x4& a, const bf16x8& b) {
  if constexpr (kPending >= 0)
    asm volatile("s_waitcnt lgkmcnt(%3)\n\tv_mfma_f32_32x32x16_bf16 %0, %1, %2, %0"
                 : "+v"(d) : "v"(a), "a"(b), "n"(kPending));
  else
    asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(d) : "v"(a), "a"(b));
}
template <int kPending>
__device__ __forceinline__ void mfma_o(f32x16& d, const u32x4& a, const u32x4& b) {
  if constexpr (kPending >= 0)
    asm volatile("s_waitcnt lgkmcnt(%3)\n\tv_mfma_f32_32x32x16_bf16 %0, %1, %2, %0"
                 : "+a"(d) : "v"(a), "v"(b), "n"(kPending));
  else
    asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+a"(d) : "v"(a), "v"(b));
}

// ---------------------------------------------------------------------------
// Tile loader: global -> LDS without passing through registers
// (global_load_lds_dwordx4).  One wave-wide instruction deposits 64 x 16 bytes
// at consecutive LDS addresses, i.e. four 256-byte key rows.  Instruction i
// (0..15, kPieces per issuing wave) fills rows 4i..4i+3; lane l lands on row 4i + l/16,
// physical chunk l%16, so it must fetch logical chunk (l%16) ^ g(row).
// ---------------------------------------------------------------------------
// 16 bytes per lane from (wave-uniform base + this lane's 32-bit offset) to
// (wave-uniform LDS address + 16 * lane).  Written as asm so that the address
// stays "SGPR pair + one VGPR" instead of a 64-bit pointer per lane.
__device__ __forceinline__ void dma16(const char* uniform_base, uint32_t lane_off, uint32_t lds_dst) {
  asm volatile(
      "s_mov_b32 m0, %2\n\t"
      "s_nop 0\n\t"
      "global_load_lds_dwordx4 %0, %1"
      :
      : "v"(lane_off), "s"(uniform_base), "s"(lds_dst)
      : "memory");
}

// One 64-key tile of K or of V.  `off` holds this lane's four byte offsets
// from the tile's first key row.  The last, partial tile redirects rows at or
// past the valid length to the last valid key (their scores are masked), so
// nothing outside the rows the caller declared valid is read.
__device__ __forceinline__ void issue_matrix_tile(const char* base, uint32_t tok_bytes, const uint32_t (&off)[kPieces],
                                                  int key0, int seq, uint32_t lds_dst, int wave_u, int lane) {
  if (wave_u >= kIssuers) return;
  const char* tile = base + (int64_t)key0 * tok_bytes;      // wave-uniform
  if (key0 + kKTile <= seq) {
#pragma unroll
    for (int j = 0; j < kPieces; ++j) dma16(tile, off[j], lds_dst + (wave_u * kPieces + j) * 1024);
  } else {
    const int last_rel = seq - 1 - key0;
#pragma unroll
    for (int j = 0; j < kPieces; ++j) {
      const int r = 4 * (wave_u * kPieces + j) + (lane >> 4);
      const int rr = r < last_rel ? r : last_rel;
      const uint32_t o = (uint32_t)rr * tok_bytes + (uint32_t)(((lane & 15) ^ swz(r)) << 4);
      dma16(tile, o, lds_dst + (wave_u * kPieces + j) * 1024);
    }
  }
}

// ---------------------------------------------------------------------------
// Partial results travel between workgroups that may sit on different XCDs,
// each behind its own L2.  Fences would make that safe by writing back and
// invalidating a whole L2 per workgroup (measured: 13 us per workgroup, and the
// K / V lines the neighbours are streaming go with it).  Instead every access
// to a partial result is itself device-coherent, as a relaxed atomic access of
// agent scope is (the sc1 scope bit: the store writes through to memory, the
// load does not hit in a stale line), and the ticket orders them: a workgroup
// draws its ticket only after its stores have been acknowledged (vmcnt(0),
// barrier), and the last one reads only after it has drawn.  The 16-byte
// accesses have no atomic spelling in the language, so they are asm (8-byte
// atomics were measured 4 % of the whole kernel slower).
// ---------------------------------------------------------------------------
__device__ __forceinline__ void store_coherent_x4(void* base, const u32x4& w0, const u32x4& w1, const u32x4& w2,
                                                  const u32x4& w3) {
  asm volatile(
      "global_store_dwordx4 %0, %1, off sc1\n\t"
      "global_store_dwordx4 %0, %2, off offset:1024 sc1\n\t"
      "global_store_dwordx4 %0, %3, off offset:2048 sc1\n\t"
      "global_store_dwordx4 %0, %4, off offset:3072 sc1"
      :
      : "v"(base), "v"(w0), "v"(w1), "v"(w2), "v"(w3)
      : "memory");
}
// One block's partial output as this lane holds it: eight 16-byte pieces 1 KB
// apart.  Issue and wait are ONE asm statement: between a load's issue and its
// return the compiler believes the destination registers hold the value, and
// is free to copy them elsewhere and reuse them - as an address, say - for the
// load to overwrite when it lands.
__device__ __forceinline__ void load_coherent_x8(const char* base, u32x4 (&w)[8]) {
  asm volatile(
      "global_load_dwordx4 %0, %8, off sc1\n\t"
      "global_load_dwordx4 %1, %8, off offset:1024 sc1\n\t"
      "global_load_dwordx4 %2, %8, off offset:2048 sc1\n\t"
      "global_load_dwordx4 %3, %8, off offset:3072 sc1\n\t"
      "global_load_dwordx4 %4, %9, off sc1\n\t"
      "global_load_dwordx4 %5, %9, off offset:1024 sc1\n\t"
      "global_load_dwordx4 %6, %9, off offset:2048 sc1\n\t"
      "global_load_dwordx4 %7, %9, off offset:3072 sc1\n\t"
      "s_waitcnt vmcnt(0)"
      : "=&v"(w[0]), "=&v"(w[1]), "=&v"(w[2]), "=&v"(w[3]), "=&v"(w[4]), "=&v"(w[5]), "=&v"(w[6]), "=&v"(w[7])
      : "v"(base), "v"(base + 4096)
      : "memory");
}
__device__ __forceinline__ void store_coherent(float* p, float x) {
  __hip_atomic_store(reinterpret_cast<uint32_t*>(p), __float_as_uint(x), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ float load_coherent(const float* p) {
  return __uint_as_float(
      __hip_atomic_load(reinterpret_cast<const uint32_t*>(p), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
}

// The compiler does not know that the asm MFMAs are still in flight when the
// asm statement retires, so wherever code it generates may touch S or O right
// after a slot (register moves at control-flow joins, the epilogue) the matrix
// pipe is drained first: an 8-pass MFMA needs 18 wait states before its result
// may be read.  The tag makes every use textually distinct, otherwise identical
// drains at the ends of sibling branches are merged into one AFTER the join,
// behind the very moves they are meant to precede.
template <int kTag>
__device__ __forceinline__ void mfma_drain(f32x16 (&oacc)[4], f32x16 (&s)[2]) {
  asm volatile("s_nop 15\n\ts_nop 15 ; matrix pipe drained, site %6"
               : "+a"(oacc[0]), "+a"(oacc[1]), "+a"(oacc[2]), "+a"(oacc[3]), "+v"(s[0]), "+v"(s[1])
               : "n"(kTag));
}

struct LaneConst {
  uint32_t k_addr[8];     // K fragment of d-step ks: key row lane%32 of a 32-key block
  uint32_t v_addr[4][2];  // V^T fragment of d block db, key sub-quad j, within a 16-key step
  float c2;               // softmax scale * log2(e)
  float neg_ref;          // minus the row's exponent reference, in log2 units (0 until it is chosen)
  int hf;                 // lane / 32
  // block-causal mask inside the chunk: keys [m_lo, m_hi) are the chunk's own
  // later blocks, hidden from this lane's query; [wg_m_lo, m_hi) is the union
  // over the workgroup's queries (wave-uniform).  Empty when the mask is off.
  int m_lo;
  int m_hi;
  int wg_m_lo;
};

__device__ __forceinline__ void mask_block(f32x16& s, int key0, int seq, int hf, int m_lo, int m_hi) {
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const int key = key0 + 8 * (i >> 2) + 4 * hf + (i & 3);
    if (key >= seq || (key >= m_lo && key < m_hi)) s[i] = -INFINITY;
  }
}

// ---------------------------------------------------------------------------
// One pipeline slot of the fast pass.  Keys advance in blocks of 32; block j
// goes through
//   S(j)  = K_j Q^T            8 K fragments, one MFMA each
//   SM(j) = exp2(scale * S - reference)   VALU only, 16 scores per lane
//   PV(j) = O^T += V_j^T P_j^T 8 V fragments, one MFMA each
// and slot j runs S(j+1), SM(j) and PV(j-1) together: MFMAs of the two
// products alternate (consecutive MFMAs never share an accumulator) and the
// softmax instructions of block j are dealt out between them, so the matrix
// pipe and the vector ALU of the wave work at the same time.  S(j) lives in
// s[j&1], P(j) in p[j&1]; with the slot parity a template argument this is
// pure register naming.
// ---------------------------------------------------------------------------
template <bool kMask, int kPar, int kKOff, int kVOff, bool kDoS, bool kDoPV, bool kDoSM>
__device__ __forceinline__ void slot(const LaneConst& c, const bf16x8 (&qf)[8], f32x16 (&s)[2], u32x4 (&p)[2][2],
                                     f32x16 (&oacc)[4], float& l, int key0, int key_end) {
  // Fragment pairs are requested one group early: with a second wave on the
  // SIMD to cover the wait that is enough and measured 2-3 % faster than two
  // (fewer fragments in flight); none ahead is 4 % slower.
  constexpr int kAhead = 1;
  u32x4 kfrag[8], vfrag[8];
  f32x16& s_cur = s[kPar];
  f32x16& s_nxt = s[kPar ^ 1];

  auto request = [&](auto ic) {
    constexpr int g = decltype(ic)::value;
    if constexpr (kDoS) kfrag[g] = lds_read_b128<kKOff>(c.k_addr[g]);
    if constexpr (kDoPV) {
      constexpr int kk = g >> 2, db = g & 3;
      const u32x2 lo = lds_read_tr16_b64<kVOff + kk * 16 * 256>(c.v_addr[db][0]);
      const u32x2 hi = lds_read_tr16_b64<kVOff + kk * 16 * 256>(c.v_addr[db][1]);
      vfrag[g] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3);
    }
  };
  // reads issued after the K (resp. V) fragment of group g, when group g runs
  constexpr int kPerGroup = (kDoS ? 1 : 0) + (kDoPV ? 2 : 0);

  static_for<kAhead>(request);

  if constexpr (kDoSM) {
    // the last, partial tile, and blocks that hold the chunk's own later
    // frames when a mask inside the chunk is asked for.  The test value
    // goes through an empty asm so that the compiler cannot fold this uniform,
    // rarely taken branch into the per-lane compares and hoist those.
    // > 0 when the block reaches past key_end or (with the mask inside the chunk
    // compiled in) overlaps [wg_m_lo, m_hi); integer min / max keep the test in
    // scalar registers
    int masked = key0 + 32 - key_end;
    if constexpr (kMask) {
      const int into_hidden = key0 + 32 - c.wg_m_lo < c.m_hi - key0 ? key0 + 32 - c.wg_m_lo : c.m_hi - key0;
      masked = masked > into_hidden ? masked : into_hidden;
    }
    asm volatile("" : "+s"(masked));
    if (masked > 0) mask_block(s_cur, key0, key_end, c.hf, kMask ? c.m_lo : 0x7fffffff, kMask ? c.m_hi : 0);
  }
  __builtin_amdgcn_sched_barrier(0);

  // A wave issues in order: a vector instruction only overlaps an MFMA if it
  // follows it in the stream, and it stalls the stream if it needs the result
  // of the instruction just before it.  So every MFMA is followed by a few
  // softmax instructions that are independent of each other: the 16 scores
  // of block j flow through scale -> exp2 -> pack + row sum one step apart.
  // Step t runs the S MFMA (t even) or the PV MFMA (t odd) of fragment group
  // t / 2 and handles score t = accumulator register t.
  constexpr int kSteps = 16;
  float scaled[kSteps + 1], weight[kSteps + 1];
  auto softmax_step = [&](auto tc) {
    constexpr int t = decltype(tc)::value;      // 0..17: stage 1 of score t, stage 2 of t-1, stage 3 of t-2
    if constexpr (kDoSM) {
      if constexpr (t < kSteps) {
        scaled[t] = __builtin_fmaf(s_cur[t], c.c2, c.neg_ref);
        pin(scaled[t]);
      }
      if constexpr (t >= 1 && t - 1 < kSteps) {
        weight[t - 1] = __builtin_amdgcn_exp2f(scaled[t - 1]);
        pin(weight[t - 1]);
      }
      if constexpr (t >= 2 && t - 2 < kSteps && ((t - 2) & 1) == 1) {
        constexpr int u = t - 2, g = u / 2;
        uint32_t packed = pack_bf16x2(weight[u - 1], weight[u]);
        l = add_bf16_pair(packed, l);
        pin(packed);
        pin(l);
        p[kPar][g >> 2][g & 3] = packed;
      }
    }
  };

  static_for<kSteps>([&](auto tc) {
    constexpr int t = decltype(tc)::value;
    constexpr int g = t / 2, i = t % 2;
    constexpr int later = (g + kAhead < 8 ? kAhead : 7 - g) * kPerGroup;   // reads of later groups in flight
    constexpr int kk = g >> 2, db = g & 3;
    if constexpr (i == 0 && g + kAhead < 8) request(std::integral_constant<int, g + kAhead>{});

    if constexpr (i == 0 && kDoS) {
      // the K fragment is followed by this group's two V reads
      constexpr int pending = later + (kDoPV ? 2 : 0);
      if constexpr (g == 0) mfma_s_first<pending>(s_nxt, kfrag[g], qf[g]);
      else mfma_s<pending>(s_nxt, kfrag[g], qf[g]);
    }
    if constexpr (i == 1 && kDoPV) mfma_o<later>(oacc[db], vfrag[g], p[kPar ^ 1][kk]);

    softmax_step(tc);
    __builtin_amdgcn_sched_barrier(0);
  });
  softmax_step(std::integral_constant<int, kSteps>{});
  softmax_step(std::integral_constant<int, kSteps + 1>{});
}

// ---------------------------------------------------------------------------
// Exact pass: conventional online softmax with a running maximum over the
// workgroup's key range, tiles double-buffered.  Every wave keeps the tiles
// coming and meets the barriers; only the waves whose fast result was unsafe
// (`compute`) redo their block.
// ---------------------------------------------------------------------------
__device__ __forceinline__ void exact_pass(const LaneConst& c, const bf16x8 (&qf)[8], f32x16 (&oacc)[4], float& m_run,
                                           float& l_run, bool compute, const char* kbase, const char* vbase,
                                           uint32_t k_tok_bytes, uint32_t v_tok_bytes, const uint32_t (&k_ld)[kPieces],
                                           const uint32_t (&v_ld)[kPieces], int tile_begin, int n, int seq,
                                           uint32_t lds_addr0, lds_char* lds, int wave_u, int lane) {
  if (compute) {
    m_run = -INFINITY;
    l_run = 0.f;
#pragma unroll
    for (int db = 0; db < 4; ++db)
#pragma unroll
      for (int i = 0; i < 16; ++i) oacc[db][i] = 0.f;
  }
  auto issue = [&](int T) {
    const int key0 = (tile_begin + T) * kKTile;
    issue_matrix_tile(kbase, k_tok_bytes, k_ld, key0, seq, lds_addr0 + kLdsK(T & 1), wave_u, lane);
    issue_matrix_tile(vbase, v_tok_bytes, v_ld, key0, seq, lds_addr0 + kLdsV(T & 1), wave_u, lane);
  };
  __syncthreads();       // everyone is done with the buffers of the fast pass
  issue(0);
  for (int T = 0; T < n; ++T) {
    const int key0 = (tile_begin + T) * kKTile;
    const int kb_off = kLdsK(T & 1), vb_off = kLdsVRel(T & 1);
    if (T + 1 < n) {
      issue(T + 1);      // into the buffer tile T - 1 left at the barrier that ended the last trip
      __builtin_amdgcn_s_waitcnt(0x0F70 | (2 * kPieces));
    } else {
      __builtin_amdgcn_s_waitcnt(0x0F70);
    }
    __syncthreads();     // tile T has landed for every wave
    if (compute) {
      f32x16 sacc[2];
#pragma unroll
      for (int kb = 0; kb < 2; ++kb) {
#pragma unroll
        for (int i = 0; i < 16; ++i) sacc[kb][i] = 0.f;
#pragma unroll
        for (int ks = 0; ks < 8; ++ks) {
          const bf16x8 kf = lds_read_b128_now(c.k_addr[ks] + (uint32_t)(kb_off + kb * 32 * 256));
          sacc[kb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf, qf[ks], sacc[kb], 0, 0, 0);
        }
        if (key0 + kb * 32 + 32 > seq || (key0 + kb * 32 + 32 > c.wg_m_lo && key0 + kb * 32 < c.m_hi))
          mask_block(sacc[kb], key0 + kb * 32, seq, c.hf, c.m_lo, c.m_hi);
      }
      float mloc = sacc[0][0];
#pragma unroll
      for (int kb = 0; kb < 2; ++kb)
#pragma unroll
        for (int i = 0; i < 16; ++i) mloc = fmaxf(mloc, sacc[kb][i]);
      mloc = half_max(mloc);
      const float m_new = fmaxf(m_run, mloc);
      // -inf only while every key so far was masked for this query: then nothing has been summed yet
      const float alpha = m_new == -INFINITY ? 1.0f : __builtin_amdgcn_exp2f((m_run - m_new) * c.c2);
      const float mc = m_new == -INFINITY ? 0.0f : m_new * c.c2;
      m_run = m_new;
      float psum = 0.f;
      bf16x8 pf[2][2];
#pragma unroll
      for (int kb = 0; kb < 2; ++kb)
#pragma unroll
        for (int st = 0; st < 2; ++st) {
          union { uint32_t u[4]; bf16x8 v; } pk;
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const float p0 = __builtin_amdgcn_exp2f(__builtin_fmaf(sacc[kb][8 * st + 2 * j], c.c2, -mc));
            const float p1 = __builtin_amdgcn_exp2f(__builtin_fmaf(sacc[kb][8 * st + 2 * j + 1], c.c2, -mc));
            psum += p0 + p1;
            pk.u[j] = pack_bf16x2(p0, p1);
          }
          pf[kb][st] = pk.v;
        }
      l_run = l_run * alpha + psum;
#pragma unroll
      for (int db = 0; db < 4; ++db) {
#pragma unroll
        for (int i = 0; i < 16; ++i) oacc[db][i] *= alpha;
#pragma unroll
        for (int kk = 0; kk < 4; ++kk) {
          const bf16x8 vf = lds_read_tr16_b64x2_now(c.v_addr[db][0] + (uint32_t)(vb_off + kk * 16 * 256),
                                                    c.v_addr[db][1] + (uint32_t)(vb_off + kk * 16 * 256));
          oacc[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf, pf[kk >> 1][kk & 1], oacc[db], 0, 0, 0);
        }
      }
    }
    __syncthreads();     // tile T's buffer is free for tile T + 2
  }
}

// This lane's query row as the B operand of S^T = K Q^T: d-step ks takes the
// 8 elements 16 ks + 8 (lane / 32) of the row.  With a RoPE table the row is
// the query before rotation and is rotated here, in the arithmetic of the
// append kernel (IEEE double, no fused multiply-add, double -> float -> bf16),
// so the kernel sees bit for bit the Q' the append would have stored.
struct QueryRope {
  const double2* freqs;        // null: the query arrives rotated
  int64_t start_frame;         // of this cache row
  int32_t grid_w, frame_tokens, split_t, split_h;
  // With norm_w (this head's 128 norm weights, offset like qp) the row is the
  // raw q projection: every slice is normalised with the token's 1 / rms as
  // the append kernel's fused norm would have done it (sdv2::normalise: two
  // roundings to bf16), then rotated.
  const uint16_t* norm_w;
  float inv_rms;
};

__device__ __forceinline__ void load_query(const QueryRope& rope, const uint16_t* qp, int token, int hf,
                                           bf16x8 (&qf)[8]) {
  if (rope.freqs == nullptr) {
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) qf[ks] = *reinterpret_cast<const bf16x8*>(qp + 16 * ks);
  } else {
    const int fi = token / rope.frame_tokens;
    const int rem = token - fi * rope.frame_tokens;
    const int hi = rem / rope.grid_w;
    const int wi = rem - hi * rope.grid_w;
    const int64_t frame = rope.start_frame + fi;
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) {
      double2 cs[4];
      sdv2::load_rotation(rope.freqs, kD / 2, rope.split_t, rope.split_h, 2 * ks + hf, frame, hi, wi, cs);
      sdv2::Vec8<uint16_t> x = sdv2::Vec8<uint16_t>::load(qp + 16 * ks);
      if (rope.norm_w) x = sdv2::normalise(x, rope.inv_rms, sdv2::Vec8<uint16_t>::load(rope.norm_w + 16 * ks));
      const sdv2::Vec8<uint16_t> y = sdv2::rotate(x, cs);
      qf[ks] = __builtin_bit_cast(bf16x8, y.raw);
    }
  }
  // the value is (re)defined in the register class every later use names, so it is never copied back and forth
#pragma unroll
  for (int ks = 0; ks < 8; ++ks) asm volatile("" : "+a"(qf[ks]));
}

template <bool kMask>
__global__ __launch_bounds__(kThreads, 1)
void swa_attn_fwd_kernel(const AttnKernelArgs a) {
  extern __shared__ __attribute__((aligned(1024))) char smem[];
  lds_char* lds = (lds_char*)smem;

  lds_int* flags = reinterpret_cast<lds_int*>(lds + kLdsFlags);

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wave_u = __builtin_amdgcn_readfirstlane(wave);
  const int hf = lane >> 5;                 // which half of the wave
  // Workgroups are dealt to the eight XCDs round robin by id, and each XCD has
  // its own L2.  Work items are ordered so that the query tiles of one (row,
  // head, key split) are neighbours, and XCD x takes the x-th eighth of that
  // list: the workgroups that stream the same K / V run on the same XCD at the
  // same time and all but the first fetch of a tile hit in L2.
  //
  // With a mixed split count a group of (row, head) pairs is one XCD's share:
  // its pairs with fewer, longer key ranges come first, so that the workgroups
  // the dispatcher hands out last are the short ones (longest first is what
  // packs unequal pieces best onto the CUs).
  int qtile, head, row, split, nsplits;
  const int nq = (a.q_tokens + kQTile - 1) / kQTile;
  {
    const int per_lo = nq * a.num_splits, per_hi = per_lo + nq;
    const int lo_pairs = a.group_pairs - a.more_pairs;
    const int per_group = lo_pairs * per_lo + a.more_pairs * per_hi;
    const int total = (a.heads * a.rows / a.group_pairs) * per_group;
    const int xcd = blockIdx.x & 7;
    const int first = (int)(((int64_t)xcd * total) >> 3);
    const int end = (int)(((int64_t)(xcd + 1) * total) >> 3);
    const int item = first + (blockIdx.x >> 3);
    if (item >= end) return;
    const int group = item / per_group;
    int r = item - group * per_group;
    int pair = group * a.group_pairs;
    if (r < lo_pairs * per_lo) {
      nsplits = a.num_splits;
      pair += r / per_lo;
      r %= per_lo;
    } else {
      nsplits = a.num_splits + 1;
      r -= lo_pairs * per_lo;
      pair += lo_pairs + r / per_hi;
      r %= per_hi;
    }
    qtile = r % nq;
    split = r / nq;
    head = pair % a.heads;
    row = pair / a.heads;
  }

  int seq = a.seq_lens ? a.seq_lens[row] : a.max_seq_len;
  seq = seq < a.max_seq_len ? seq : a.max_seq_len;
  seq = seq < 0 ? 0 : seq;
  const int ntiles = (seq + kKTile - 1) / kKTile;
  const int per_split = (ntiles + nsplits - 1) / nsplits;
  const int tile_begin = split * per_split;
  int tile_end = tile_begin + per_split;
  tile_end = tile_end < ntiles ? tile_end : ntiles;
  const int n = tile_end - tile_begin;       // tiles this workgroup streams

  // (the transfers take their base addresses from scalar registers: say so to the compiler)
  auto uniform = [](const void* ptr) {
    const uint64_t x = reinterpret_cast<uint64_t>(ptr);
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)x), hi = __builtin_amdgcn_readfirstlane((uint32_t)(x >> 32));
    return reinterpret_cast<const char*>(((uint64_t)hi << 32) | lo);
  };
  const uint32_t lds_addr0 = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)lds);
  const char* kbase = uniform(a.k + row * a.k_st.row + head * a.k_st.head);
  const char* vbase = uniform(a.v + row * a.v_st.row + head * a.v_st.head);
  const uint32_t k_tok_bytes = (uint32_t)(a.k_st.token * 2);
  const uint32_t v_tok_bytes = (uint32_t)(a.v_st.token * 2);

  uint32_t k_ld[kPieces], v_ld[kPieces];
#pragma unroll
  for (int j = 0; j < kPieces; ++j) {
    const int r = 4 * ((wave % kIssuers) * kPieces + j) + (lane >> 4);
    const int chunk = (lane & 15) ^ swz(r);
    k_ld[j] = (uint32_t)(r * k_tok_bytes + chunk * 16);
    v_ld[j] = (uint32_t)(r * v_tok_bytes + chunk * 16);
  }
  // T is the tile index inside this workgroup's range
  auto issue_k = [&](int T, int buf) {
    issue_matrix_tile(kbase, k_tok_bytes, k_ld, (tile_begin + T) * kKTile, seq, lds_addr0 + kLdsK(buf), wave_u, lane);
  };
  auto issue_v = [&](int T, int buf) {
    issue_matrix_tile(vbase, v_tok_bytes, v_ld, (tile_begin + T) * kKTile, seq, lds_addr0 + kLdsV(buf), wave_u, lane);
  };

  // The transfers the first two slots need go out first; the query rows are
  // fetched (and rotated) behind them, the rest of the look-ahead after that:
  // ordinary loads return in order with the transfers, so whatever is issued
  // ahead of the query rows is what the first wait for them also waits for.
  if (n > 0) {
    issue_k(0, 0);
    issue_v(0, 0);
    issue_k(n > 1 ? 1 : n - 1, 1);
    // V buffer 2 stands in for "V tile -1" in the first slot, where it meets the
    // all-zero P(-1): any finite values do, so it is cleared (two 16-byte stores per lane)
    {
      const u32x4 zero = {0u, 0u, 0u, 0u};
      *reinterpret_cast<__attribute__((address_space(3))) u32x4*>(lds + kLdsV(2) + tid * 16) = zero;
      *reinterpret_cast<__attribute__((address_space(3))) u32x4*>(lds + kLdsV(2) + (kThreads + tid) * 16) = zero;
    }
    if (tid == 0) flags[0] = 0;       // "a wave found an unsafe row sum": read behind the barrier that ends the loop
  }

  // ---- this lane's query row -------------------------------------------------
  const int q_row = qtile * kQTile + wave * kQBlock + (lane & 31);
  bf16x8 qf[8];
  {
    const int q_row_c = q_row < a.q_tokens ? q_row : a.q_tokens - 1;
    QueryRope rope;
    rope.freqs = a.freqs;
    rope.grid_w = a.grid_w; rope.frame_tokens = a.frame_tokens; rope.split_t = a.split_t; rope.split_h = a.split_h;
    // (constant indices and selects: indexing the by-value argument block with a run-time
    // row would move the whole block, its pointers included, out of scalar registers)
    rope.start_frame = a.start_frame[0];
    static_for<SDV2_MAX_ROWS - 1>([&](auto ic) {
      constexpr int i = decltype(ic)::value + 1;
      rope.start_frame = row == i ? a.start_frame[i] : rope.start_frame;
    });
    rope.norm_w = a.q_norm_w ? a.q_norm_w + head * kD + 8 * hf : nullptr;
    rope.inv_rms = a.q_norm_w ? a.q_inv_rms[(int64_t)row * a.q_tokens + q_row_c] : 1.0f;
    load_query(rope, a.q + row * a.q_st.row + (int64_t)q_row_c * a.q_st.token + head * a.q_st.head + 8 * hf, q_row_c,
               hf, qf);
  }
  if (n > 0) {
    // every buffer a slot may read starts with real (finite) data, also where the tile does not exist
    issue_v(n > 1 ? 1 : n - 1, 1);
    issue_k(n > 2 ? 2 : n - 1, 2);
  }

  // ---- per-lane LDS read addresses ------------------------------------------
  LaneConst c;
  c.c2 = a.scale_log2;
  c.neg_ref = 0.f;
  c.hf = hf;
  if (kMask && a.mask_block_tokens > 0) {
    const int bt = a.mask_block_tokens;
    const int first = a.chunk_start[row];
    c.m_hi = __builtin_amdgcn_readfirstlane(first + a.q_tokens);
    c.wg_m_lo = __builtin_amdgcn_readfirstlane(first + ((qtile * kQTile) / bt + 1) * bt);
    c.m_lo = first + (q_row / bt + 1) * bt;
  } else {
    c.m_hi = 0;
    c.wg_m_lo = 0x7fffffff;
    c.m_lo = 0x7fffffff;
  }
  {
    // K (A operand): key = lane%32 of the block, chunk = 2*ks + hf
    const int r = lane & 31;
    const int base = r * 256 + ((hf ^ swz(r)) << 4);
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) c.k_addr[ks] = lds_addr0 + (uint32_t)(base ^ (ks << 5));
  }
  {
    // V^T (A operand) through the transposing read: in each group of 16 lanes,
    // lane i supplies the address of key (i / 4), 8 bytes at d-offset 4 * (i % 4);
    // it receives d = i, keys 0..3.  Group = (hf, dhalf).  Relative to V buffer 0.
    const int i16 = lane & 15;
    const int dhalf = (lane >> 4) & 1;
    const int krow = i16 >> 2;
#pragma unroll
    for (int db = 0; db < 4; ++db)
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        const int r = 8 * j + 4 * hf + krow;                 // + 16 * kk added as an immediate
        const int ch = db * 4 + dhalf * 2 + ((i16 & 3) >> 1);
        c.v_addr[db][j] = lds_addr0 + kLdsVBase + (uint32_t)(r * 256 + ((ch ^ swz(r)) << 4) + (i16 & 1) * 8);
      }
  }

  f32x16 oacc[4];
#pragma unroll
  for (int db = 0; db < 4; ++db)
#pragma unroll
    for (int i = 0; i < 16; ++i) oacc[db][i] = 0.f;
  f32x16 s[2];
  u32x4 p[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) p[i][j] = u32x4{0u, 0u, 0u, 0u};
  float l_run = 0.f;                 // this lane's share of the row sum
  float m_run = 0.f;                 // the row's exponent reference, in score units
  bool unsafe = false;

  // Tile T (64 keys) = blocks 2T, 2T+1, in K / V buffers T % 3.  Slot 2T needs
  // K tile T (second half) and V tile T-1 (second half); slot 2T+1 needs K tile
  // T+1 (first half) and V tile T (first half).  After slot 2T the buffers of
  // K tile T and V tile T-1 are free: that is where the one barrier per tile
  // sits, followed by the requests for K tile T+3 and V tile T+2.  What the
  // next two slots read was requested two barriers earlier, so the wait before
  // the barrier leaves the newest 2 * kPieces transfers of an issuing wave (one
  // K and one V tile's worth) in flight.
  //
  // Every tile runs the same code and the loop body is three whole tiles with
  // a single way in and out, so the accumulators keep their registers from trip
  // to trip (the compiler must never be given a reason to move them while asm
  // MFMAs are in flight).  Scores of keys at or beyond the end of the range (the
  // tail of a partial tile, the look-ahead block of a tile that does not
  // exist) are masked to -inf, so their weights are exact zeros against
  // whatever finite data the buffers still hold.  In the first slot P(-1) is
  // zero likewise.
  const int key_end = seq < tile_end * kKTile ? seq : tile_end * kKTile;
  auto do_tile = [&](auto buf_c, int T) {
    constexpr int kB = decltype(buf_c)::value;              // T % 3
    constexpr int kBNext = (kB + 1) % kStages, kBPrev = (kB + 2) % kStages;
    const int key0 = (tile_begin + T) * kKTile;
    slot<kMask, 0, kLdsK(kB) + 32 * 256, kLdsVRel(kBPrev) + 32 * 256, true, true, true>(c, qf, s, p, oacc, l_run, key0,
                                                                                        key_end);
    if (T + 3 < n) {
      __builtin_amdgcn_s_waitcnt(0x0F70 | (2 * kPieces));   // vmcnt: one K and one V tile's worth per wave
    } else {
      __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0)
    }
    __syncthreads();
    if (T + 3 < n) issue_k(T + 3, kB);
    if (T + 2 < n) issue_v(T + 2, kBPrev);
    slot<kMask, 1, kLdsK(kBNext), kLdsVRel(kB), true, true, true>(c, qf, s, p, oacc, l_run, key0 + 32, key_end);
  };
  using B0 = std::integral_constant<int, 0>;
  using B1 = std::integral_constant<int, 1>;
  using B2 = std::integral_constant<int, 2>;

  const bool idle = __builtin_amdgcn_readfirstlane(qtile * kQTile + wave * kQBlock >= a.q_tokens);
  if (n > 0) {
    // K tile 0 (and, for the first slot of the loop, V tile 0 and K tile 1) have
    // landed once at most the last two transfers of an issuing wave are in flight
    if (wave_u < kIssuers) {
      __builtin_amdgcn_s_waitcnt(0x0070 | (2 * kPieces));   // vmcnt, and lgkmcnt(0) for the LDS clear
    } else {
      __builtin_amdgcn_s_waitcnt(0x0070);
    }
    __syncthreads();
    if (idle) {
      // No query row of this wave exists (the last query tile of a call is
      // rarely full).  The wave still moves its share of every K / V tile and
      // meets the others at every barrier, but issues no LDS read, MFMA or
      // softmax instruction: on a chip that runs this kernel against its power
      // limit, work on rows nobody reads would only lower the clock for the rest.
      for (int T = 0; T < n; ++T) {
        if (T + 3 < n) {
          __builtin_amdgcn_s_waitcnt(0x0F70 | (2 * kPieces));
        } else {
          __builtin_amdgcn_s_waitcnt(0x0F70);
        }
        __syncthreads();
        if (T + 3 < n) issue_k(T + 3, T % kStages);
        if (T + 2 < n) issue_v(T + 2, (T + 2) % kStages);
      }
    } else {
      // S(0) alone fills the pipeline, and its largest score becomes the row's exponent reference
      slot<kMask, 1, kLdsK(0), 0, true, false, false>(c, qf, s, p, oacc, l_run, 0, key_end);
      mfma_drain<1>(oacc, s);
      {
        float ref = s[0][0];
#pragma unroll
        for (int i = 1; i < 16; ++i) ref = vmax(ref, s[0][i]);
        ref = half_max(ref);
        ref = (ref > -0x1p120f && ref < 0x1p120f) ? ref : 0.f;      // also false for NaN
        m_run = ref;
        c.neg_ref = -ref * c.c2;
      }
      // Three tiles per trip, one per buffer; the last trip stops after the last
      // real tile.  The skipped tiles sit behind uniform branches that no value
      // is changed on, so the accumulators stay where they are on either way.
      for (int T = 0; T < n; T += 3) {
        do_tile(B0{}, T);
        if (T + 1 < n) {
          do_tile(B1{}, T + 1);
          if (T + 2 < n) do_tile(B2{}, T + 2);
        }
      }
      // PV of the last block (odd -> p[1], second half of the last tile's V
      // buffer) empties the pipeline.  The code addresses V buffer 2; the lane
      // addresses are moved when the last tile sits in another buffer.
      {
        LaneConst cf = c;
        const uint32_t shift = (uint32_t)(((n - 1) % kStages - 2) * kTileBytes);
#pragma unroll
        for (int db = 0; db < 4; ++db)
#pragma unroll
          for (int j = 0; j < 2; ++j) cf.v_addr[db][j] = c.v_addr[db][j] + shift;
        slot<kMask, 0, 0, kLdsVRel(2) + 32 * 256, false, true, false>(cf, qf, s, p, oacc, l_run, 0, key_end);
      }
      mfma_drain<0>(oacc, s);
      // Checked once, after the last tile: a sum that overflowed stays inf or NaN, one
      // that underflowed stays tiny.  With the mask inside the chunk a sum of exactly
      // zero is legitimate when every key of this workgroup's range is hidden from
      // the lane's query (its split then contributes nothing).
      {
        const float l_tot = half_sum(l_run);
        bool ok = l_tot >= 0x1p-100f && l_tot <= 0x1p100f;
        if constexpr (kMask) ok |= l_tot == 0.f && tile_begin * kKTile >= c.m_lo && key_end <= c.m_hi;
        unsafe = __builtin_amdgcn_ballot_w64(!ok) != 0;
      }
    }

    // Did any wave of the workgroup see an unsafe row sum?  One barrier: behind it every wave is done
    // with the K / V buffers (the epilogue stages its output there) and the flag, cleared before the
    // loop, holds every wave's word.
    if (unsafe && lane == 0) flags[0] = 1;
    __syncthreads();
    const int redo = flags[0];
    if (redo)
      exact_pass(c, qf, oacc, m_run, l_run, unsafe, kbase, vbase, k_tok_bytes, v_tok_bytes, k_ld, v_ld, tile_begin, n,
                 seq, lds_addr0, lds, wave_u, lane);
  }

  // ---- epilogue ---------------------------------------------------------------
  // (every wave is done with the K / V buffers: the barrier above, or the last one of the exact pass)
  const int block = qtile * kWaves + wave;              // this wave's 32-row block within the (row, head)
  float l_tot = half_sum(l_run);
  float inv = l_tot > 0.f ? 1.0f / l_tot : 0.f;

  if (nsplits > 1) {
    // Partial result of a key range: the normalised row divided by its largest
    // magnitude, as fp16 (values in [-1, 1]: 11 bits against the row's scale,
    // sixteen times finer than the bf16 of the final result), plus that scale
    // and the log-sum-exp.  Stored in register order - 16-byte piece j of a lane
    // holds its accumulator registers 8 j .. 8 j + 7 - so that every store and,
    // later, every load of the combining workgroup is one contiguous kilobyte
    // per wave and the values come back to the registers they left.
    const int64_t slab = (int64_t)a.rows * a.heads * a.q_blocks;
    const int64_t blk0 = ((int64_t)row * a.heads + head) * a.q_blocks + block;
    if (!idle) {
      float amax = 0.f;
#pragma unroll
      for (int db = 0; db < 4; ++db)
#pragma unroll
        for (int i = 0; i < 16; ++i) amax = vmax(amax, __builtin_fabsf(oacc[db][i]));
      amax = half_max(amax) * inv;
      const float row_scale = amax > 0.f && amax < INFINITY ? amax : 1.0f;
      const float to_unit = inv / row_scale;
      const int64_t blk = split * slab + blk0;
      // piece j of the lane (its accumulator registers 8 j .. 8 j + 7 as fp16) lies j KB into the block
      char* dst = reinterpret_cast<char*>(a.part_o + blk * kPartBlockHalves + lane * 8);
#pragma unroll
      for (int half = 0; half < 2; ++half) {
        u32x4 w[4];
#pragma unroll
        for (int jj = 0; jj < 4; ++jj) {
          const int j = 4 * half + jj, db = j >> 1, i0 = 8 * (j & 1);
#pragma unroll
          for (int e = 0; e < 4; ++e)
            w[jj][e] = pack_f16x2(oacc[db][i0 + 2 * e] * to_unit, oacc[db][i0 + 2 * e + 1] * to_unit);
        }
        store_coherent_x4(dst + half * 4096, w[0], w[1], w[2], w[3]);
      }
      if (hf == 0) {
        store_coherent(a.part_lse + blk * kQBlock + lane,
                       l_tot > 0.f ? m_run * c.c2 + __builtin_amdgcn_logf(l_tot) : -INFINITY);
        store_coherent(a.part_scale + blk * kQBlock + lane, row_scale);
      }
    }
    // Ticket.  Every wave has waited for its stores to be acknowledged before the
    // barrier; then one lane draws.  The workgroup that draws the last ticket of
    // its (row, head, query tile) finds every other range's results in memory,
    // and leaves the ticket at zero for the next call.
    __builtin_amdgcn_s_waitcnt(0x0F70);       // vmcnt(0)
    __syncthreads();
    if (tid == 0) {
      int32_t* ticket = a.tickets + ((int64_t)row * a.heads + head) * nq + qtile;
      const int drawn = __hip_atomic_fetch_add(ticket, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      const int last = drawn == nsplits - 1;
      if (last) __hip_atomic_store(ticket, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      flags[1] = last;
    }
    __syncthreads();
    if (flags[1] == 0 || idle) return;

    // combine: out = sum_s 2^(lse_s - LSE) O_s over the ranges in their fixed
    // order (every range, this workgroup's own included, as it lies in memory:
    // the sum does not depend on which workgroup happens to be last)
    const int r32 = lane & 31;
    constexpr int kBatch = 8;         // ranges whose statistics are fetched together
    float wsum = 0.f;
    float lse[kBatch], scale[kBatch], ws[kBatch];
    // log-sum-exp and row scale of the ranges of a batch; the loads go out together
    auto fetch = [&](int s0) {
#pragma unroll
      for (int u = 0; u < kBatch; ++u) {
        const int sp = s0 + u < nsplits ? s0 + u : nsplits - 1;
        lse[u] = load_coherent(a.part_lse + (sp * slab + blk0) * kQBlock + r32);
        scale[u] = load_coherent(a.part_scale + (sp * slab + blk0) * kQBlock + r32);
      }
    };
    fetch(0);
    float lse_max = lse[0];
#pragma unroll
    for (int u = 1; u < kBatch; ++u) lse_max = fmaxf(lse_max, lse[u]);         // (entries past the last range repeat it)
    for (int sp = kBatch; sp < nsplits; ++sp)
      lse_max = fmaxf(lse_max, load_coherent(a.part_lse + (sp * slab + blk0) * kQBlock + r32));
#pragma unroll
    for (int db = 0; db < 4; ++db)
#pragma unroll
      for (int i = 0; i < 16; ++i) oacc[db][i] = 0.f;
    for (int s0 = 0; s0 < nsplits; s0 += kBatch) {
      if (s0 > 0) fetch(s0);
#pragma unroll
      for (int u = 0; u < kBatch; ++u) {
        const float w = (s0 + u >= nsplits || lse[u] == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(lse[u] - lse_max);
        wsum += w;
        ws[u] = w * scale[u];         // weight times the row's fp16 scale
      }
#pragma unroll
      for (int u = 0; u < kBatch; ++u) {
        if (s0 + u >= nsplits) break;
        u32x4 x[8];
        load_coherent_x8(
            reinterpret_cast<const char*>(a.part_o + ((s0 + u) * slab + blk0) * kPartBlockHalves + lane * 8), x);
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const int db = j >> 1, i0 = 8 * (j & 1);
          const f16x8 h = __builtin_bit_cast(f16x8, x[j]);
#pragma unroll
          for (int e = 0; e < 8; ++e) oacc[db][i0 + e] += ws[u] * static_cast<float>(h[e]);
        }
      }
    }
    inv = wsum > 0.f ? 1.0f / wsum : 0.f;
  } else if (idle) {
    return;
  }

  // A lane holds one query row's values scattered over the 128 dims, so direct
  // stores would touch 32 rows with 16 or 32 bytes each.  Instead every wave
  // stages its 32-row block in its own 16 KB of the (now idle) LDS, 16-byte
  // chunks XOR-swizzled by row, and writes whole rows of 256 bytes.  LDS
  // operations of one wave complete in order, so the block needs no barrier of
  // its own.
  lds_char* stage = lds + wave * kStageBytes;
  const int q0 = qtile * kQTile + wave * kQBlock;
  const int r = lane & 31;
#pragma unroll
  for (int db = 0; db < 4; ++db)
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      u32x2 w;
      w[0] = pack_bf16x2(oacc[db][4 * g] * inv, oacc[db][4 * g + 1] * inv);
      w[1] = pack_bf16x2(oacc[db][4 * g + 2] * inv, oacc[db][4 * g + 3] * inv);
      const int chunk = db * 4 + g;
      *reinterpret_cast<__attribute__((address_space(3))) u32x2*>(stage + r * 256 + ((chunk ^ (r & 15)) << 4) + hf * 8) =
          w;
    }
  uint16_t* dst = a.out + row * a.o_st.row + head * a.o_st.head + (int64_t)q0 * a.o_st.token;
  const int j = lane & 15;
#pragma unroll
  for (int it = 0; it < 8; ++it) {
    const int rr = 4 * it + (lane >> 4);
    const u32x4 w = *reinterpret_cast<__attribute__((address_space(3))) const u32x4*>(
        stage + rr * 256 + ((j ^ (rr & 15)) << 4));
    if (q0 + rr < a.q_tokens) *reinterpret_cast<u32x4*>(dst + rr * a.o_st.token + j * 8) = w;
  }
}

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }
bool stride_ok(const sdv2_stride3& s) { return s.row % 8 == 0 && s.token % 8 == 0 && s.head % 8 == 0; }

size_t align_up(size_t x, size_t a) { return (x + a - 1) / a * a; }

// layout of the split-KV workspace: tickets, partial outputs, log-sum-exps, row scales
struct WorkspaceLayout {
  size_t tickets, part_o, part_lse, part_scale, total;
};
WorkspaceLayout workspace_layout(int32_t rows, int32_t q_tokens, int32_t heads, int32_t num_splits) {
  const size_t nq = (size_t)(q_tokens + kQTile - 1) / kQTile;
  const size_t blocks = (size_t)rows * heads * ((q_tokens + kQBlock - 1) / kQBlock);
  WorkspaceLayout w;
  (void)nq;
  w.tickets = 0;
  w.part_o = (size_t)kMaxTickets * sizeof(int32_t);
  w.part_lse = w.part_o + (size_t)num_splits * blocks * kPartBlockHalves * sizeof(uint16_t);
  w.part_scale = w.part_lse + align_up((size_t)num_splits * blocks * kQBlock * sizeof(float), 256);
  w.total = w.part_scale + align_up((size_t)num_splits * blocks * kQBlock * sizeof(float), 256);
  return w;
}

}  // namespace

// Device memory the library owns, for sdv2_swa_attn_fwd_static: the partial
// results of a split call when the caller cannot bring a workspace.  One copy
// per GPU, at an address of its own on each, held until the process ends.  In
// host code `scratch` is only a handle for hipGetSymbolAddress; kernels get the
// address that call returns.
static __device__ __align__(256) unsigned char scratch[SDV2_STATIC_SCRATCH_BYTES];

namespace {

// Address of `scratch` on the current device, looked up once per device with
// that device current; nullptr when the runtime refuses.
void* static_scratch_address() {
  static std::mutex lock;
  static void* address[kMaxDevices];
  int device = 0;
  if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= kMaxDevices) return nullptr;
  std::lock_guard<std::mutex> guard(lock);
  if (!address[device]) {
    void* ptr = nullptr;
    if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)) != hipSuccess) {
      (void)hipGetLastError();
      return nullptr;
    }
    address[device] = ptr;
  }
  return address[device];
}

int attn_fwd(const sdv2_attn_params* p, void* workspace, size_t workspace_bytes);

// How a call's key ranges are cut, as num_splits carries it: bits 0-7 the
// count s every (row, head) pair gets at least, bits 8-15 how many of the
// pairs of each eighth of the (row, head) list (one XCD's share) get s + 1.
struct SplitPlan {
  int base, more, group;
  int most() const { return base + (more > 0 ? 1 : 0); }
};
bool decode_splits(int32_t encoded, int32_t rows, int32_t heads, SplitPlan* plan) {
  if (encoded <= 0 || (encoded >> 16) != 0) return false;
  plan->base = encoded & 0xff;
  plan->more = (encoded >> 8) & 0xff;
  const int64_t pairs = (int64_t)rows * heads;
  plan->group = (int)pairs;
  if (plan->base < 1) return false;
  if (plan->more > 0) {
    if (pairs % 8 != 0 || plan->more >= pairs / 8) return false;
    plan->group = (int)(pairs / 8);
  }
  return plan->most() <= 64;
}

}  // namespace

extern "C" int sdv2_swa_attn_default_splits(int32_t rows, int32_t q_tokens, int32_t heads, int32_t max_seq_len) {
  if (rows <= 0 || q_tokens <= 0 || heads <= 0 || max_seq_len <= 0) return 1;
  // One workgroup per CU.  With s key-range splits there are qwork * s
  // workgroups; they run in ceil(qwork * s / 256) rounds, each as long as one
  // workgroup's tile count plus a fixed start / end cost of about three tile
  // times.  Writing and combining the partial results
  // costs roughly one tile time per 3.5 MB of them per split.  Constants fitted
  // to measurements on the five benchmark shapes.
  const int nq = (q_tokens + kQTile - 1) / kQTile;
  const int64_t pairs = (int64_t)rows * heads;
  const int64_t qwork = pairs * nq;
  if (qwork > kMaxTickets) return 1;
  // (the answer depends on the shape alone and costs a small simulation: the last one is remembered)
  static std::mutex lock;
  static int32_t last_shape[4] = {0, 0, 0, 0};
  static int last_answer = 0;
  {
    std::lock_guard<std::mutex> guard(lock);
    if (last_answer && last_shape[0] == rows && last_shape[1] == q_tokens && last_shape[2] == heads &&
        last_shape[3] == max_seq_len)
      return last_answer;
  }
  const int ntiles = (max_seq_len + kKTile - 1) / kKTile;
  const double partial_tiles = (double)rows * heads * q_tokens * kD * 4 / 7.0e6;
  int best = 1;
  double best_cost = 1e300;
  for (int sp = 1; sp <= 8; ++sp) {
    const int per = (ntiles + sp - 1) / sp;
    if (sp > 1 && per < 6) break;
    const int64_t rounds = (qwork * sp + kCuSlots - 1) / kCuSlots;
    const double cost = (double)rounds * (per + 3) + (sp > 1 ? sp * partial_tiles : 0.0);
    if (cost < best_cost - 1e-9) { best_cost = cost; best = sp; }
  }
  // A uniform count can leave the last round of workgroups mostly empty (1120
  // workgroups are 4.4 rounds of 256).  When the (row, head) pairs divide over
  // the eight XCDs, some pairs of each XCD's share may take one range more:
  // workgroups of two lengths, the long ones dispatched first, fill the 32 CUs
  // of an XCD more evenly.  Simulated as the dispatcher works (next workgroup
  // to the CU that is free first); taken when it beats the best uniform count
  // by 3 %.
  if (pairs % 8 == 0 && pairs / 8 >= 2 && pairs / 8 <= 255) {
    const int group = (int)(pairs / 8);
    constexpr int kCusPerXcd = kCuSlots / 8;
    double mixed_cost = 1e300;
    int mixed = 0;
    for (int sp = 1; sp <= 7; ++sp) {
      const int per_lo = (ntiles + sp - 1) / sp, per_hi = (ntiles + sp) / (sp + 1);
      if (per_hi < 6) break;
      for (int more = 1; more < group; ++more) {
        double busy[kCusPerXcd] = {};
        auto hand_out = [&](int count, double length) {
          for (int i = 0; i < count; ++i) {
            int cu = 0;
            for (int c = 1; c < kCusPerXcd; ++c)
              if (busy[c] < busy[cu]) cu = c;
            busy[cu] += length;
          }
        };
        hand_out((group - more) * nq * sp, per_lo + 3);
        hand_out(more * nq * (sp + 1), per_hi + 3);
        double span = 0;
        for (double b : busy) span = b > span ? b : span;
        const double ranges = ((double)(group - more) * sp + (double)more * (sp + 1)) / group;
        const double cost = span + ranges * partial_tiles;
        if (cost < mixed_cost - 1e-9) { mixed_cost = cost; mixed = sp | (more << 8); }
      }
    }
    if (mixed_cost < 0.97 * best_cost) best = mixed;
  }
  std::lock_guard<std::mutex> guard(lock);
  last_shape[0] = rows; last_shape[1] = q_tokens; last_shape[2] = heads; last_shape[3] = max_seq_len;
  last_answer = best;
  return best;
}

extern "C" size_t sdv2_swa_attn_workspace_bytes(int32_t rows, int32_t q_tokens, int32_t heads,
                                                 int32_t max_seq_len, int32_t num_splits) {
  if (rows <= 0 || q_tokens <= 0 || heads <= 0) return 0;
  if (num_splits <= 0) num_splits = sdv2_swa_attn_default_splits(rows, q_tokens, heads, max_seq_len);
  SplitPlan plan;
  if (!decode_splits(num_splits, rows, heads, &plan) || plan.most() <= 1) return 0;
  return workspace_layout(rows, q_tokens, heads, plan.most()).total;
}

extern "C" int sdv2_swa_attn_fwd(const sdv2_attn_params* p) {
  if (!p) return SDV2_ERR_INVALID_ARG;
  return attn_fwd(p, p->workspace, p->workspace_bytes);
}

extern "C" int sdv2_swa_attn_fwd_static(const sdv2_attn_params* p) {
  if (!p) return SDV2_ERR_INVALID_ARG;
  if (p->rows <= 0 || p->q_tokens <= 0 || p->heads <= 0 || p->max_seq_len < 0)
    return attn_fwd(p, nullptr, 0);                       // nothing to split: same answers as the plain entry point
  if (p->dtype == SDV2_F32) return attn_fwd(p, nullptr, 0);   // fp32 walks one key range: no scratch, whatever num_splits says
  const int splits = p->num_splits > 0 ? p->num_splits
                                       : sdv2_swa_attn_default_splits(p->rows, p->q_tokens, p->heads, p->max_seq_len);
  SplitPlan plan;
  if (!decode_splits(splits, p->rows, p->heads, &plan)) return SDV2_ERR_INVALID_ARG;   // as the plain entry point answers
  if (plan.most() <= 1) return attn_fwd(p, nullptr, 0);
  if (sdv2_swa_attn_workspace_bytes(p->rows, p->q_tokens, p->heads, p->max_seq_len, splits) >
      (size_t)SDV2_STATIC_SCRATCH_BYTES)
    return SDV2_ERR_SCRATCH_LIMIT;
  void* ptr = static_scratch_address();
  if (!ptr) return SDV2_ERR_LAUNCH;
  return attn_fwd(p, ptr, SDV2_STATIC_SCRATCH_BYTES);
}

namespace {

int attn_fwd(const sdv2_attn_params* p, void* workspace, size_t workspace_bytes) {
  if (p->dtype == SDV2_F32) return sdv2::attn_fwd_f32(p);        // fp32 arithmetic, one key range: no workspace
  if (p->dtype != SDV2_BF16) return SDV2_ERR_UNSUPPORTED;
  if (p->head_dim != kD) return SDV2_ERR_UNSUPPORTED;
  if (p->rows < 0 || p->q_tokens < 0 || p->heads <= 0 || p->max_seq_len < 0) return SDV2_ERR_INVALID_ARG;
  if (p->rows == 0 || p->q_tokens == 0) return SDV2_OK;
  if (!p->q || !p->k_cache || !p->v_cache || !p->out) return SDV2_ERR_INVALID_ARG;
  if (!aligned16(p->q) || !aligned16(p->k_cache) || !aligned16(p->v_cache) || !aligned16(p->out))
    return SDV2_ERR_INVALID_ARG;
  if (!stride_ok(p->q_stride) || !stride_ok(p->k_stride) || !stride_ok(p->v_stride) || !stride_ok(p->out_stride))
    return SDV2_ERR_INVALID_ARG;
  if (p->rows > 65535 / 8 || p->heads > 65535) return SDV2_ERR_INVALID_ARG;

  SplitPlan plan;
  if (!decode_splits(p->num_splits > 0 ? p->num_splits
                                       : sdv2_swa_attn_default_splits(p->rows, p->q_tokens, p->heads, p->max_seq_len),
                     p->rows, p->heads, &plan))
    return SDV2_ERR_INVALID_ARG;
  const int splits = plan.most();
  if ((int64_t)p->rows * splits > 65535) return SDV2_ERR_INVALID_ARG;
  // more (row, head, query tile) groups than there are ticket words: such a grid fills the chip unsplit
  if (splits > 1 && (int64_t)p->rows * p->heads * ((p->q_tokens + kQTile - 1) / kQTile) > kMaxTickets)
    return SDV2_ERR_UNSUPPORTED;

  AttnKernelArgs a{};
  a.q = static_cast<const uint16_t*>(p->q);
  a.k = static_cast<const uint16_t*>(p->k_cache);
  a.v = static_cast<const uint16_t*>(p->v_cache);
  a.out = static_cast<uint16_t*>(p->out);
  a.seq_lens = p->seq_lens;
  a.q_st = p->q_stride; a.k_st = p->k_stride; a.v_st = p->v_stride; a.o_st = p->out_stride;
  a.rows = p->rows; a.q_tokens = p->q_tokens; a.heads = p->heads; a.max_seq_len = p->max_seq_len;
  a.num_splits = plan.base;
  a.group_pairs = plan.group;
  a.more_pairs = plan.more;
  const float scale = p->softmax_scale > 0.f ? p->softmax_scale : 0.08838834764831845f;  // 1/sqrt(128)
  a.scale_log2 = scale * kLog2e;
  if (p->mask_block_tokens < 0) return SDV2_ERR_INVALID_ARG;
  if (p->mask_block_tokens > 0 && p->mask_block_tokens < p->q_tokens) {
    // a block as long as the chunk hides nothing: only shorter blocks switch the mask on
    if (!p->chunk_key_start) return SDV2_ERR_INVALID_ARG;
    a.chunk_start = p->chunk_key_start;
    a.mask_block_tokens = p->mask_block_tokens;
  }

  if (p->rope_freqs) {
    // q arrives before RoPE and is rotated as it is loaded; the chunk is grid_f whole frames of grid_h x grid_w
    if (p->rows > SDV2_MAX_ROWS || !p->rope_start_frame) return SDV2_ERR_INVALID_ARG;
    if (p->rope_grid_h <= 0 || p->rope_grid_w <= 0) return SDV2_ERR_INVALID_ARG;
    const int64_t frame_tokens = (int64_t)p->rope_grid_h * p->rope_grid_w;
    if (p->q_tokens % frame_tokens != 0) return SDV2_ERR_INVALID_ARG;
    const int64_t grid_f = p->q_tokens / frame_tokens;
    if (p->rope_grid_h > p->rope_freq_rows || p->rope_grid_w > p->rope_freq_rows) return SDV2_ERR_OUT_OF_RANGE;
    for (int i = 0; i < p->rows; ++i) {
      if (p->rope_start_frame[i] < 0 || p->rope_start_frame[i] + grid_f > p->rope_freq_rows)
        return SDV2_ERR_OUT_OF_RANGE;
      a.start_frame[i] = p->rope_start_frame[i];
    }
    a.freqs = reinterpret_cast<const double2*>(p->rope_freqs);
    a.grid_w = p->rope_grid_w;
    a.frame_tokens = (int32_t)frame_tokens;
    // column split of the table: c - 2*(c/3) | c/3 | c/3  (causal_model.py:77-78)
    const int third = (kD / 2) / 3;
    a.split_t = kD / 2 - 2 * third;
    a.split_h = a.split_t + third;
  }

  if (p->q_norm_weight || p->q_inv_rms) {
    // the raw q projection: normalised, then rotated, as it is loaded
    if (!p->q_norm_weight || !p->q_inv_rms || !p->rope_freqs) return SDV2_ERR_INVALID_ARG;
    if (!aligned16(p->q_norm_weight) || (reinterpret_cast<uintptr_t>(p->q_inv_rms) & 3)) return SDV2_ERR_INVALID_ARG;
    a.q_norm_w = static_cast<const uint16_t*>(p->q_norm_weight);
    a.q_inv_rms = p->q_inv_rms;
  }

  a.q_blocks = (p->q_tokens + kQBlock - 1) / kQBlock;
  if (splits > 1) {
    const WorkspaceLayout w = workspace_layout(p->rows, p->q_tokens, p->heads, splits);
    if (!workspace || workspace_bytes < w.total) return SDV2_ERR_WORKSPACE;
    if (reinterpret_cast<uintptr_t>(workspace) & 255) return SDV2_ERR_INVALID_ARG;
    char* ws = static_cast<char*>(workspace);
    a.tickets = reinterpret_cast<int32_t*>(ws + w.tickets);
    a.part_o = reinterpret_cast<uint16_t*>(ws + w.part_o);
    a.part_lse = reinterpret_cast<float*>(ws + w.part_lse);
    a.part_scale = reinterpret_cast<float*>(ws + w.part_scale);
  }

  hipStream_t stream = static_cast<hipStream_t>(p->stream);
  const int64_t nq_tiles = (p->q_tokens + kQTile - 1) / kQTile;
  const int64_t items = ((int64_t)p->rows * p->heads / plan.group) *
                        (nq_tiles * ((int64_t)(plan.group - plan.more) * plan.base + (int64_t)plan.more * (plan.base + 1)));
  if (items > (1 << 28)) return SDV2_ERR_INVALID_ARG;
  dim3 grid((unsigned)(8 * ((items + 7) / 8)));
  // The tile buffers (96 KB) or the epilogue staging (16 KB per wave) exceed the static limit:
  // ask for the dynamic size once per device.
  // The kernel exists twice: the mask inside the chunk costs the plain
  // variant about 2 % even when it is off, so it gets its own code.
  static std::atomic<bool> lds_ready[kMaxDevices];
  int device = 0;
  if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= kMaxDevices) return SDV2_ERR_LAUNCH;
  if (!lds_ready[device].load(std::memory_order_acquire)) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(swa_attn_fwd_kernel<false>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, kLdsBytes) != hipSuccess ||
        hipFuncSetAttribute(reinterpret_cast<const void*>(swa_attn_fwd_kernel<true>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, kLdsBytes) != hipSuccess)
      return SDV2_ERR_LAUNCH;
    lds_ready[device].store(true, std::memory_order_release);
  }
  if (a.mask_block_tokens > 0)
    sdv2::launch_timed(SDV2_KERNEL_ATTENTION, swa_attn_fwd_kernel<true>, grid, dim3(kThreads), kLdsBytes, stream, a);
  else
    sdv2::launch_timed(SDV2_KERNEL_ATTENTION, swa_attn_fwd_kernel<false>, grid, dim3(kThreads), kLdsBytes, stream, a);
  if (hipGetLastError() != hipSuccess) return SDV2_ERR_LAUNCH;
  return SDV2_OK;
}

}  // namespace
