// What this GPU sustains on the attention kernel's own instruction streams: a
// measurement hook (include/sdv2kv_profile.h), not part of the path.
//
// The attention kernel is priced against the dense bf16 matrix peak, but a
// chip under matrix load runs against its power limit, and how far below the
// peak that leaves it depends on what else the instruction stream does per
// matrix instruction.  These kernels run the loop of swa_attn_fwd.hip with
// parts taken away - same instructions (v_mfma_f32_32x32x16_bf16, ds_read_b128,
// ds_read_b64_tr_b16, global_load_lds_dwordx4), same LDS layout and fragment
// addresses, same software pipeline - on random operands, one workgroup per
// CU, and compute nothing anybody reads:
//
//   registers     the matrix instructions alone, operands resident in registers
//   lds 32 rows   + every A operand read from LDS as the attention kernel reads
//                 it (8 waves x 32 query rows: 1.5 LDS reads per MFMA)
//   lds 64 rows   the same with 64 query rows per wave (4 waves, 512 registers
//                 each): every fragment read feeds two MFMAs (0.75 reads per MFMA)
//   attention mix lds 32 rows + the softmax instructions of a key block
//                 between the MFMAs (fma, exp2, pack, row sum; the weights they
//                 produce are the B operands of the following block) + the
//                 global->LDS tile transfers and the barrier per 64-key tile
//   mix, 64 rows  the same additions on the 64-rows-per-wave stream: what a
//                 re-blocking of the attention kernel to two query blocks per
//                 wave could reach in its loop
//
// The distance between "attention mix" and the attention kernel's own rate is
// what the kernel loses outside its loop (prologue, partial results, combine,
// idle tail); the distance between the modes is what each ingredient costs.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>
#include <utility>

#include "sdv2kv.h"
#include "sdv2kv_profile.h"
#include "sdv2kv_internal.h"

namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(2))) float f32x2;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;
typedef __attribute__((address_space(3))) char lds_char;

constexpr int kTileBytes = 16384;               // 64 keys x 128 dims, bf16
constexpr int kLdsBytes = 6 * kTileBytes;       // three K and three V tile buffers
constexpr int kCus = 256;
constexpr int kMaxDevices = 64;

// Layout of the operand buffer (random bf16 supplied by the caller), in bytes.
constexpr size_t kImages = 64;                                   // distinct initial LDS contents
constexpr size_t kImagesBytes = kImages * kLdsBytes;
constexpr size_t kQBytes = 512 * 16 * 16;                        // per thread: up to 16 fragments of 16 bytes
constexpr size_t kPBytes = 512 * 8 * 16;
constexpr size_t kRBytes = 512 * 8 * 16;
constexpr size_t kQOff = kImagesBytes;
constexpr size_t kPOff = kQOff + kQBytes;
constexpr size_t kROff = kPOff + kPBytes;
constexpr size_t kStreamOff = kROff + kRBytes;
constexpr int kRegionTiles = 48;                                 // K/V tile pairs a workgroup cycles through
constexpr size_t kRegionBytes = (size_t)kRegionTiles * 2 * kTileBytes;
constexpr int kRegions = 32;
constexpr size_t kOperandBytes = kStreamOff + kRegions * kRegionBytes;

template <int... I, typename F>
__device__ __forceinline__ void static_for_impl(std::integer_sequence<int, I...>, F&& f) {
  (f(std::integral_constant<int, I>{}), ...);
}
template <int N, typename F>
__device__ __forceinline__ void static_for(F&& f) {
  static_for_impl(std::make_integer_sequence<int, N>{}, f);
}

__device__ __forceinline__ int swz(int r) { return ((r & 3) << 2) | ((r >> 2) & 3); }

// Fragment reads into accumulation registers, waits tied to the consuming MFMA
// (as in swa_attn_fwd.hip, where the fragments land in vector registers).
template <int kOffset>
__device__ __forceinline__ u32x4 lds_read_b128(uint32_t addr) {
  u32x4 r;
  asm volatile("ds_read_b128 %0, %1 offset:%2" : "=a"(r) : "v"(addr), "n"(kOffset));
  return r;
}
// Two transposing reads into the halves of one register quadruple: inline asm
// cannot name half of an operand, so the halves are pinned to physical
// registers (three quadruples in rotation, first register kFirst) and joined.
template <int kOffset, int kSet, int kFirst>
__device__ __forceinline__ u32x4 lds_read_tr16_b64x2(uint32_t addr_lo, uint32_t addr_hi) {
  u32x2 lo, hi;
#define SDV2_TR_PAIR(LO, HI)                                                                            \
  asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "={" LO "}"(lo) : "v"(addr_lo), "n"(kOffset));    \
  asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "={" HI "}"(hi) : "v"(addr_hi), "n"(kOffset));
  static_assert(kFirst == 112 || kFirst == 240, "register sets exist for 128 and 256 accumulation registers");
  if constexpr (kFirst == 112) {
    if constexpr (kSet == 0) { SDV2_TR_PAIR("a[112:113]", "a[114:115]") }
    else if constexpr (kSet == 1) { SDV2_TR_PAIR("a[116:117]", "a[118:119]") }
    else { SDV2_TR_PAIR("a[120:121]", "a[122:123]") }
  } else {
    if constexpr (kSet == 0) { SDV2_TR_PAIR("a[240:241]", "a[242:243]") }
    else if constexpr (kSet == 1) { SDV2_TR_PAIR("a[244:245]", "a[246:247]") }
    else { SDV2_TR_PAIR("a[248:249]", "a[250:251]") }
  }
#undef SDV2_TR_PAIR
  return __builtin_shufflevector(lo, hi, 0, 1, 2, 3);
}

// kPending: LDS reads issued after the fragment that may still be in flight (-1: operand already in registers)
template <int kPending>
__device__ __forceinline__ void mfma_s_first(f32x16& d, const u32x4& a, const bf16x8& b) {
  if constexpr (kPending >= 0)
    asm volatile("s_waitcnt lgkmcnt(%3)\n\tv_mfma_f32_32x32x16_bf16 %0, %1, %2, 0" : "=&v"(d) : "a"(a), "a"(b), "n"(kPending));
  else
    asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, 0" : "=&v"(d) : "a"(a), "a"(b));
}
template <int kPending>
__device__ __forceinline__ void mfma_s(f32x16& d, const u32x4& a, const bf16x8& b) {
  if constexpr (kPending >= 0)
    asm volatile("s_waitcnt lgkmcnt(%3)\n\tv_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(d) : "a"(a), "a"(b), "n"(kPending));
  else
    asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(d) : "a"(a), "a"(b));
}
template <int kPending>
__device__ __forceinline__ void mfma_o(f32x16& d, const u32x4& a, const u32x4& b) {
  if constexpr (kPending >= 0)
    asm volatile("s_waitcnt lgkmcnt(%3)\n\tv_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+a"(d) : "a"(a), "v"(b), "n"(kPending));
  else
    asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+a"(d) : "a"(a), "v"(b));
}

__device__ __forceinline__ void dma16(const char* uniform_base, uint32_t lane_off, uint32_t lds_dst) {
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
               :
               : "v"(lane_off), "s"(uniform_base), "s"(lds_dst)
               : "memory");
}
__device__ __forceinline__ void pin(float& x) { asm volatile("" : "+v"(x)); }
__device__ __forceinline__ void pin(uint32_t& x) { asm volatile("" : "+v"(x)); }
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  const f32x2 x = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(x, bf16x2));
}
__device__ __forceinline__ float add_bf16_pair(uint32_t packed, float acc) {
  const bf16x2 ones = {(__bf16)1.0f, (__bf16)1.0f};
  return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, packed), ones, acc, false);
}

// Per-lane fragment addresses, as the attention kernel forms them: K rows read
// with ds_read_b128, V^T with the transposing read, tiles XOR-swizzled by row.
struct LaneAddr {
  uint32_t k[8];
  uint32_t v[4][2];     // relative to the first V buffer
};
__device__ __forceinline__ LaneAddr lane_addresses(int lane) {
  LaneAddr c;
  const int hf = lane >> 5;
  {
    const int r = lane & 31;
    const int base = r * 256 + ((hf ^ swz(r)) << 4);
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) c.k[ks] = (uint32_t)(base ^ (ks << 5));
  }
  {
    const int i16 = lane & 15, dhalf = (lane >> 4) & 1, krow = i16 >> 2;
#pragma unroll
    for (int db = 0; db < 4; ++db)
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        const int r = 8 * j + 4 * hf + krow;
        const int ch = db * 4 + dhalf * 2 + ((i16 & 3) >> 1);
        c.v[db][j] = 3 * kTileBytes + (uint32_t)(r * 256 + ((ch ^ swz(r)) << 4) + (i16 & 1) * 8);
      }
  }
  return c;
}

struct StreamArgs {
  const char* operands;     // kOperandBytes of random bf16
  float* sink;              // never written (the condition that guards the store cannot hold)
  int32_t iterations;       // three 64-key tiles each
};

template <int kThreads>
__device__ __forceinline__ void fill_lds(lds_char* lds, const char* operands, int tid) {
  const char* image = operands + (size_t)(blockIdx.x % kImages) * kLdsBytes;
  for (int i = tid; i < kLdsBytes / 16; i += kThreads)
    *reinterpret_cast<__attribute__((address_space(3))) u32x4*>(lds + i * 16) = *reinterpret_cast<const u32x4*>(image + i * 16);
  __syncthreads();
}

// 8 waves x 32 query rows.  kLds: fragments come from LDS; kSoftmax: the
// softmax instructions of the previous key block run between the MFMAs and
// produce the next block's B operands; kDma: tile transfers and the per-tile
// barrier of the attention loop.
template <bool kLds, bool kSoftmax, bool kDma>
__global__ __launch_bounds__(512, 1)
void mfma_stream32_kernel(const StreamArgs a) {
  extern __shared__ __attribute__((aligned(1024))) char smem[];
  lds_char* lds = (lds_char*)smem;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave_u = __builtin_amdgcn_readfirstlane(tid >> 6);
  fill_lds<512>(lds, a.operands, tid);
  const LaneAddr c = lane_addresses(lane);
  bf16x8 qf[8];
  u32x4 p[2][2];
#pragma unroll
  for (int ks = 0; ks < 8; ++ks) {
    qf[ks] = *reinterpret_cast<const bf16x8*>(a.operands + kQOff + (size_t)(tid * 8 + ks) * 16);
    asm volatile("" : "+a"(qf[ks]));
  }
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) p[i][j] = *reinterpret_cast<const u32x4*>(a.operands + kPOff + (size_t)(tid * 4 + i * 2 + j) * 16);
  u32x4 rk[4], rv[4];
  if constexpr (!kLds) {
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      rk[g] = *reinterpret_cast<const u32x4*>(a.operands + kROff + (size_t)(tid * 8 + g) * 16);
      rv[g] = *reinterpret_cast<const u32x4*>(a.operands + kROff + (size_t)(tid * 8 + 4 + g) * 16);
      asm volatile("" : "+a"(rk[g]), "+a"(rv[g]));
    }
  }
  f32x16 oacc[4], s[2];
#pragma unroll
  for (int db = 0; db < 4; ++db)
#pragma unroll
    for (int i = 0; i < 16; ++i) oacc[db][i] = 0.f;
#pragma unroll
  for (int i = 0; i < 16; ++i) { s[0][i] = 0.f; s[1][i] = 0.f; }
  float l = 0.f;
  // scores of the random operands have a standard deviation near 1: scaled like natural-unit scores of that
  // spread and shifted below a typical row maximum, so the weights cover several octaves as real ones do
  float c2 = 1.4427f, neg_ref = -4.0f;
  pin(c2);
  pin(neg_ref);

  const char* region = a.operands + kStreamOff + (size_t)(blockIdx.x % kRegions) * kRegionBytes;
  {
    const uint64_t x = reinterpret_cast<uint64_t>(region);
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)x), hi = __builtin_amdgcn_readfirstlane((uint32_t)(x >> 32));
    region = reinterpret_cast<const char*>(((uint64_t)hi << 32) | lo);
  }
  uint32_t ld[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) ld[j] = (uint32_t)(((wave_u & 3) * 4 + j) * 1024 + lane * 16);
  // K tile T of the stream at region + (T % kRegionTiles) * 32 KB, its V tile 16 KB behind it; four issuing waves
  auto issue = [&](int T, int buf, int is_v) {
    if (wave_u >= 4) return;
    const char* tile = region + (size_t)(T % kRegionTiles) * (2 * kTileBytes) + is_v * kTileBytes;
    const uint32_t dst = (uint32_t)((is_v ? 3 : 0) * kTileBytes + buf * kTileBytes);
#pragma unroll
    for (int j = 0; j < 4; ++j) dma16(tile, ld[j], dst + (wave_u * 4 + j) * 1024);
  };

  // One pipeline slot: S of the next key block and PV of the previous one, MFMAs alternating, with the
  // softmax of the current block dealt out between them (see slot() in swa_attn_fwd.hip).
  auto slot = [&](auto par_c, auto koff_c, auto voff_c) {
    constexpr int kPar = decltype(par_c)::value, kKOff = decltype(koff_c)::value, kVOff = decltype(voff_c)::value;
    u32x4 kfrag[8], vfrag[8];
    f32x16& s_cur = s[kPar];
    f32x16& s_nxt = s[kPar ^ 1];
    auto request = [&](auto ic) {
      constexpr int g = decltype(ic)::value;
      if constexpr (kLds) {
        kfrag[g] = lds_read_b128<kKOff>(c.k[g]);
        constexpr int kk = g >> 2, db = g & 3;
        vfrag[g] = lds_read_tr16_b64x2<kVOff + kk * 16 * 256 - 3 * kTileBytes, g % 3, 112>(c.v[db][0], c.v[db][1]);
      }
    };
    request(std::integral_constant<int, 0>{});
    __builtin_amdgcn_sched_barrier(0);
    float scaled[17], weight[17];
    auto softmax_step = [&](auto tc) {
      constexpr int t = decltype(tc)::value;
      if constexpr (kSoftmax) {
        if constexpr (t < 16) {
          scaled[t] = __builtin_fmaf(s_cur[t], c2, neg_ref);
          pin(scaled[t]);
        }
        if constexpr (t >= 1 && t - 1 < 16) {
          weight[t - 1] = __builtin_amdgcn_exp2f(scaled[t - 1]);
          pin(weight[t - 1]);
        }
        if constexpr (t >= 2 && t - 2 < 16 && ((t - 2) & 1) == 1) {
          constexpr int u = t - 2, g = u / 2;
          uint32_t packed = pack_bf16x2(weight[u - 1], weight[u]);
          l = add_bf16_pair(packed, l);
          pin(packed);
          pin(l);
          p[kPar][g >> 2][g & 3] = packed;
        }
      }
    };
    static_for<16>([&](auto tc) {
      constexpr int t = decltype(tc)::value;
      constexpr int g = t / 2, i = t % 2;
      constexpr int later = (g + 1 < 8 ? 1 : 0) * 3;
      if constexpr (i == 0 && g + 1 < 8) request(std::integral_constant<int, g + 1>{});
      if constexpr (kLds) {
        if constexpr (i == 0) {
          if constexpr (g == 0) mfma_s_first<later + 2>(s_nxt, kfrag[g], qf[g]);
          else mfma_s<later + 2>(s_nxt, kfrag[g], qf[g]);
        } else {
          mfma_o<later>(oacc[g & 3], vfrag[g], p[kPar ^ 1][g >> 2]);
        }
      } else {
        if constexpr (i == 0) {
          if constexpr (g == 0) mfma_s_first<-1>(s_nxt, rk[g & 3], qf[g]);
          else mfma_s<-1>(s_nxt, rk[g & 3], qf[g]);
        } else {
          mfma_o<-1>(oacc[g & 3], rv[(g + kPar) & 3], p[kPar ^ 1][g >> 2]);
        }
      }
      softmax_step(tc);
      __builtin_amdgcn_sched_barrier(0);
    });
    softmax_step(std::integral_constant<int, 16>{});
    softmax_step(std::integral_constant<int, 17>{});
  };
  using I0 = std::integral_constant<int, 0>;
  using I1 = std::integral_constant<int, 1>;
  using I2 = std::integral_constant<int, 2>;
  auto do_tile = [&](auto buf_c, int T) {
    constexpr int kB = decltype(buf_c)::value;
    constexpr int kBNext = (kB + 1) % 3, kBPrev = (kB + 2) % 3;
    slot(I0{}, std::integral_constant<int, kB * kTileBytes + 8192>{},
         std::integral_constant<int, (3 + kBPrev) * kTileBytes + 8192>{});
    if constexpr (kDma) {
      __builtin_amdgcn_s_waitcnt(0x0F70 | 8);      // vmcnt: one K and one V tile's worth per issuing wave stay in flight
      __syncthreads();
      issue(T + 3, kB, 0);
      issue(T + 2, kBPrev, 1);
    }
    slot(I1{}, std::integral_constant<int, kBNext * kTileBytes>{}, std::integral_constant<int, (3 + kB) * kTileBytes>{});
  };
  if constexpr (kDma) {
    issue(0, 0, 0);
    issue(0, 0, 1);
    issue(1, 1, 0);
    issue(1, 1, 1);
    issue(2, 2, 0);
    __builtin_amdgcn_s_waitcnt(0x0F70 | 8);
    __syncthreads();
  }
  for (int it = 0; it < a.iterations; ++it) {
    do_tile(I0{}, 3 * it);
    do_tile(I1{}, 3 * it + 1);
    do_tile(I2{}, 3 * it + 2);
  }
  __builtin_amdgcn_s_waitcnt(0x0F70);              // every transfer has landed before the wave ends
  asm volatile("s_nop 15\n\ts_nop 15" : "+a"(oacc[0]), "+a"(oacc[1]), "+a"(oacc[2]), "+a"(oacc[3]), "+v"(s[0]), "+v"(s[1]));
  float acc = l;
#pragma unroll
  for (int i = 0; i < 16; ++i) acc += s[0][i] + s[1][i] + oacc[0][i] + oacc[1][i] + oacc[2][i] + oacc[3][i];
  if (acc == 12345.678f) a.sink[blockIdx.x * 512 + tid] = acc;      // keeps the work alive; does not happen
}

// 4 waves x 64 query rows (one wave per SIMD, 512 registers): two query blocks
// per wave, every K and V^T fragment feeds one MFMA of each.  kSoftmax / kDma
// add what they add to the 32-row kernel: the softmax instructions of both
// blocks between the MFMAs, the tile transfers (all four waves issue) and the
// barrier per tile.
template <bool kSoftmax, bool kDma>
__global__ __launch_bounds__(256, 1)
void mfma_stream64_kernel(const StreamArgs a) {
  extern __shared__ __attribute__((aligned(1024))) char smem[];
  lds_char* lds = (lds_char*)smem;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave_u = __builtin_amdgcn_readfirstlane(tid >> 6);
  fill_lds<256>(lds, a.operands, tid);
  const LaneAddr c = lane_addresses(lane);
  bf16x8 qf[2][8];
  u32x4 p[2][2][2];
#pragma unroll
  for (int b = 0; b < 2; ++b)
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) {
      qf[b][ks] = *reinterpret_cast<const bf16x8*>(a.operands + kQOff + (size_t)((tid * 2 + b) * 8 + ks) * 16);
      asm volatile("" : "+a"(qf[b][ks]));
    }
#pragma unroll
  for (int b = 0; b < 2; ++b)
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j)
        p[b][i][j] = *reinterpret_cast<const u32x4*>(a.operands + kPOff + (size_t)((tid * 2 + b) * 4 + i * 2 + j) * 16);
  f32x16 oacc[2][4], s[2][2];
#pragma unroll
  for (int b = 0; b < 2; ++b) {
#pragma unroll
    for (int db = 0; db < 4; ++db)
#pragma unroll
      for (int i = 0; i < 16; ++i) oacc[b][db][i] = 0.f;
#pragma unroll
    for (int i = 0; i < 16; ++i) { s[b][0][i] = 0.f; s[b][1][i] = 0.f; }
  }
  float l[2] = {0.f, 0.f};
  float c2 = 1.4427f, neg_ref = -4.0f;
  pin(c2);
  pin(neg_ref);

  const char* region = a.operands + kStreamOff + (size_t)(blockIdx.x % kRegions) * kRegionBytes;
  {
    const uint64_t x = reinterpret_cast<uint64_t>(region);
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)x), hi = __builtin_amdgcn_readfirstlane((uint32_t)(x >> 32));
    region = reinterpret_cast<const char*>(((uint64_t)hi << 32) | lo);
  }
  uint32_t ld[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) ld[j] = (uint32_t)((wave_u * 4 + j) * 1024 + lane * 16);
  auto issue = [&](int T, int buf, int is_v) {
    const char* tile = region + (size_t)(T % kRegionTiles) * (2 * kTileBytes) + is_v * kTileBytes;
    const uint32_t dst = (uint32_t)((is_v ? 3 : 0) * kTileBytes + buf * kTileBytes);
#pragma unroll
    for (int j = 0; j < 4; ++j) dma16(tile, ld[j], dst + (wave_u * 4 + j) * 1024);
  };

  auto slot = [&](auto par_c, auto koff_c, auto voff_c) {
    constexpr int kPar = decltype(par_c)::value, kKOff = decltype(koff_c)::value, kVOff = decltype(voff_c)::value;
    u32x4 kfrag[8], vfrag[8];
    auto request = [&](auto ic) {
      constexpr int g = decltype(ic)::value;
      kfrag[g] = lds_read_b128<kKOff>(c.k[g]);
      constexpr int kk = g >> 2, db = g & 3;
      vfrag[g] = lds_read_tr16_b64x2<kVOff + kk * 16 * 256 - 3 * kTileBytes, g % 3, 240>(c.v[db][0], c.v[db][1]);
    };
    request(std::integral_constant<int, 0>{});
    __builtin_amdgcn_sched_barrier(0);
    // 32 steps, one MFMA each: group g = t / 4 runs S of block 0, S of block 1, PV of block 0, PV of block 1;
    // score u = t (block u / 16, accumulator register u % 16) goes through fma -> exp2 -> pack + row sum one step apart
    float scaled[33], weight[33];
    auto softmax_step = [&](auto tc) {
      constexpr int t = decltype(tc)::value;
      if constexpr (kSoftmax) {
        if constexpr (t < 32) {
          scaled[t] = __builtin_fmaf(s[t >> 4][kPar][t & 15], c2, neg_ref);
          pin(scaled[t]);
        }
        if constexpr (t >= 1 && t - 1 < 32) {
          weight[t - 1] = __builtin_amdgcn_exp2f(scaled[t - 1]);
          pin(weight[t - 1]);
        }
        if constexpr (t >= 2 && t - 2 < 32 && ((t - 2) & 1) == 1) {
          constexpr int u = t - 2, b = u >> 4, g = (u & 15) / 2;
          uint32_t packed = pack_bf16x2(weight[u - 1], weight[u]);
          l[b] = add_bf16_pair(packed, l[b]);
          pin(packed);
          pin(l[b]);
          p[b][kPar][g >> 2][g & 3] = packed;
        }
      }
    };
    static_for<32>([&](auto tc) {
      constexpr int t = decltype(tc)::value;
      constexpr int g = t / 4, i = t % 4;
      constexpr int later = (g + 1 < 8 ? 1 : 0) * 3;
      if constexpr (i == 0 && g + 1 < 8) request(std::integral_constant<int, g + 1>{});
      if constexpr (i < 2) {
        if constexpr (g == 0) mfma_s_first<later + 2>(s[i][kPar ^ 1], kfrag[g], qf[i][g]);
        else mfma_s<later + 2>(s[i][kPar ^ 1], kfrag[g], qf[i][g]);
      } else {
        mfma_o<later>(oacc[i - 2][g & 3], vfrag[g], p[i - 2][kPar ^ 1][g >> 2]);
      }
      softmax_step(tc);
      __builtin_amdgcn_sched_barrier(0);
    });
    softmax_step(std::integral_constant<int, 32>{});
    softmax_step(std::integral_constant<int, 33>{});
  };
  using I0 = std::integral_constant<int, 0>;
  using I1 = std::integral_constant<int, 1>;
  using I2 = std::integral_constant<int, 2>;
  auto do_tile = [&](auto buf_c, int T) {
    constexpr int kB = decltype(buf_c)::value;
    constexpr int kBNext = (kB + 1) % 3, kBPrev = (kB + 2) % 3;
    slot(I0{}, std::integral_constant<int, kB * kTileBytes + 8192>{},
         std::integral_constant<int, (3 + kBPrev) * kTileBytes + 8192>{});
    if constexpr (kDma) {
      __builtin_amdgcn_s_waitcnt(0x0F70 | 8);
      __syncthreads();
      issue(T + 3, kB, 0);
      issue(T + 2, kBPrev, 1);
    }
    slot(I1{}, std::integral_constant<int, kBNext * kTileBytes>{}, std::integral_constant<int, (3 + kB) * kTileBytes>{});
  };
  if constexpr (kDma) {
    issue(0, 0, 0);
    issue(0, 0, 1);
    issue(1, 1, 0);
    issue(1, 1, 1);
    issue(2, 2, 0);
    __builtin_amdgcn_s_waitcnt(0x0F70 | 8);
    __syncthreads();
  }
  for (int it = 0; it < a.iterations; ++it) {
    do_tile(I0{}, 3 * it);
    do_tile(I1{}, 3 * it + 1);
    do_tile(I2{}, 3 * it + 2);
  }
  __builtin_amdgcn_s_waitcnt(0x0F70);
  asm volatile("s_nop 15\n\ts_nop 15"
               : "+a"(oacc[0][0]), "+a"(oacc[0][1]), "+a"(oacc[0][2]), "+a"(oacc[0][3]), "+a"(oacc[1][0]), "+a"(oacc[1][1]),
                 "+a"(oacc[1][2]), "+a"(oacc[1][3]));
  asm volatile("" : "+v"(s[0][0]), "+v"(s[0][1]), "+v"(s[1][0]), "+v"(s[1][1]));
  float acc = l[0] + l[1];
#pragma unroll
  for (int b = 0; b < 2; ++b)
#pragma unroll
    for (int i = 0; i < 16; ++i)
      acc += s[b][0][i] + s[b][1][i] + oacc[b][0][i] + oacc[b][1][i] + oacc[b][2][i] + oacc[b][3][i];
  if (acc == 12345.678f) a.sink[blockIdx.x * 256 + tid] = acc;
}

template <typename Kernel>
bool allow_lds(Kernel kernel, std::atomic<bool>& done) {
  if (done.load(std::memory_order_acquire)) return true;
  if (hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, kLdsBytes) !=
      hipSuccess)
    return false;
  done.store(true, std::memory_order_release);
  return true;
}

}  // namespace

extern "C" size_t sdv2_profile_mfma_stream_bytes(void) { return kOperandBytes + (size_t)kCus * 512 * sizeof(float); }

extern "C" int sdv2_profile_mfma_stream(int mode, const void* operands, size_t operand_bytes, int32_t iterations,
                                        void* stream, double* flops) {
  if (!operands || !flops || iterations <= 0 || iterations > (1 << 20)) return SDV2_ERR_INVALID_ARG;
  if (operand_bytes < sdv2_profile_mfma_stream_bytes()) return SDV2_ERR_WORKSPACE;
  if (reinterpret_cast<uintptr_t>(operands) & 255) return SDV2_ERR_INVALID_ARG;
  int device = 0;
  if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= kMaxDevices) return SDV2_ERR_LAUNCH;
  static std::atomic<bool> ready[5][kMaxDevices];
  StreamArgs a;
  a.operands = static_cast<const char*>(operands);
  a.sink = reinterpret_cast<float*>(const_cast<char*>(a.operands) + kOperandBytes);
  a.iterations = iterations;
  hipStream_t s = static_cast<hipStream_t>(stream);
  // per iteration and wave: six slots of 16 MFMAs (32 with two query blocks per wave)
  double mfma_per_launch = 0;
  switch (mode) {
    case SDV2_STREAM_REGISTERS:
      // (the tile buffers are filled in this mode too, so that all modes start alike)
      if (!allow_lds(mfma_stream32_kernel<false, false, false>, ready[0][device])) return SDV2_ERR_LAUNCH;
      hipLaunchKernelGGL((mfma_stream32_kernel<false, false, false>), dim3(kCus), dim3(512), kLdsBytes, s, a);
      mfma_per_launch = (double)kCus * 8 * 96 * iterations;
      break;
    case SDV2_STREAM_LDS_32_ROWS:
      if (!allow_lds(mfma_stream32_kernel<true, false, false>, ready[1][device])) return SDV2_ERR_LAUNCH;
      hipLaunchKernelGGL((mfma_stream32_kernel<true, false, false>), dim3(kCus), dim3(512), kLdsBytes, s, a);
      mfma_per_launch = (double)kCus * 8 * 96 * iterations;
      break;
    case SDV2_STREAM_LDS_64_ROWS:
      if (!allow_lds(mfma_stream64_kernel<false, false>, ready[2][device])) return SDV2_ERR_LAUNCH;
      hipLaunchKernelGGL((mfma_stream64_kernel<false, false>), dim3(kCus), dim3(256), kLdsBytes, s, a);
      mfma_per_launch = (double)kCus * 4 * 192 * iterations;
      break;
    case SDV2_STREAM_ATTENTION_MIX_64_ROWS:
      if (!allow_lds(mfma_stream64_kernel<true, true>, ready[4][device])) return SDV2_ERR_LAUNCH;
      hipLaunchKernelGGL((mfma_stream64_kernel<true, true>), dim3(kCus), dim3(256), kLdsBytes, s, a);
      mfma_per_launch = (double)kCus * 4 * 192 * iterations;
      break;
    case SDV2_STREAM_ATTENTION_MIX:
      if (!allow_lds(mfma_stream32_kernel<true, true, true>, ready[3][device])) return SDV2_ERR_LAUNCH;
      hipLaunchKernelGGL((mfma_stream32_kernel<true, true, true>), dim3(kCus), dim3(512), kLdsBytes, s, a);
      mfma_per_launch = (double)kCus * 8 * 96 * iterations;
      break;
    default:
      return SDV2_ERR_INVALID_ARG;
  }
  if (hipGetLastError() != hipSuccess) return SDV2_ERR_LAUNCH;
  *flops = mfma_per_launch * 32768.0;
  return SDV2_OK;
}
