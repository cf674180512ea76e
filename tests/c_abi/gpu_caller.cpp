// A caller of the sdv2kv C ABI that knows nothing of Python or PyTorch: plain
// HIP runtime calls for memory and the stream, then one layer call (append with
// RoPE, attention) per chunk through include/sdv2kv.h.
//
// usage: gpu_caller <in.bin> <out.bin>
// in.bin  : int32 header {chunks, tokens, heads, grid_f, grid_h, grid_w, cap, freq_rows, splits},
//           double table[freq_rows * 64 * 2], then per chunk:
//           int64 {start_frame, dst_start, new_global_end, new_local_end},
//           bf16 q, k, v [tokens * heads * 128] each (token-major)
// out.bin : per chunk bf16 roped q and bf16 attention output [tokens * heads * 128] each;
//           at the end the K cache and the V cache, bf16 [cap * heads * 128] in memory
//           order (head-major: [heads][cap][128]), and the two int64 indices.
#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <vector>

#include "sdv2kv.h"

#define HIP_OK(x)                                                                    \
  do {                                                                               \
    hipError_t e_ = (x);                                                             \
    if (e_ != hipSuccess) {                                                          \
      std::fprintf(stderr, "%s failed: %s\n", #x, hipGetErrorString(e_));            \
      return 3;                                                                      \
    }                                                                                \
  } while (0)

#define SDV2_OK_OR_DIE(x)                                                            \
  do {                                                                               \
    int s_ = (x);                                                                    \
    if (s_ != SDV2_OK) {                                                             \
      std::fprintf(stderr, "%s failed: %s\n", #x, sdv2_status_string(s_));           \
      return 4;                                                                      \
    }                                                                                \
  } while (0)

template <typename T>
static bool read_n(std::FILE* f, T* dst, size_t n) { return std::fread(dst, sizeof(T), n, f) == n; }

int main(int argc, char** argv) {
  if (argc != 3) { std::fprintf(stderr, "usage: %s in.bin out.bin\n", argv[0]); return 2; }
  if (sdv2_abi_version() != SDV2KV_ABI_VERSION) { std::fprintf(stderr, "ABI mismatch\n"); return 2; }
  std::FILE* in = std::fopen(argv[1], "rb");
  std::FILE* out = std::fopen(argv[2], "wb");
  if (!in || !out) { std::fprintf(stderr, "cannot open files\n"); return 2; }
  int32_t hdr[9];
  if (!read_n(in, hdr, 9)) return 2;
  const int chunks = hdr[0], tokens = hdr[1], heads = hdr[2], cap = hdr[6], freq_rows = hdr[7], splits = hdr[8];
  const size_t n_chunk = (size_t)tokens * heads * 128, n_cache = (size_t)cap * heads * 128;
  std::vector<double> table((size_t)freq_rows * 64 * 2);
  if (!read_n(in, table.data(), table.size())) return 2;

  hipStream_t stream;
  HIP_OK(hipStreamCreate(&stream));
  double* d_table;
  uint16_t *d_q, *d_k, *d_v, *d_rq, *d_o, *d_kc, *d_vc;
  int64_t* d_idx;
  int32_t* d_len;
  HIP_OK(hipMalloc(&d_table, table.size() * sizeof(double)));
  HIP_OK(hipMemcpy(d_table, table.data(), table.size() * sizeof(double), hipMemcpyHostToDevice));
  for (uint16_t** p : {&d_q, &d_k, &d_v, &d_rq, &d_o}) HIP_OK(hipMalloc(p, n_chunk * 2));
  HIP_OK(hipMalloc(&d_kc, n_cache * 2));
  HIP_OK(hipMalloc(&d_vc, n_cache * 2));
  HIP_OK(hipMemset(d_kc, 0, n_cache * 2));
  HIP_OK(hipMemset(d_vc, 0, n_cache * 2));
  HIP_OK(hipMalloc(&d_idx, 2 * sizeof(int64_t)));
  HIP_OK(hipMemset(d_idx, 0, 2 * sizeof(int64_t)));
  HIP_OK(hipMalloc(&d_len, sizeof(int32_t)));
  const size_t ws_bytes = sdv2_swa_attn_workspace_bytes(1, tokens, heads, cap, splits);
  void* d_ws = nullptr;
  if (ws_bytes) {
    HIP_OK(hipMalloc(&d_ws, ws_bytes));
    HIP_OK(hipMemset(d_ws, 0, ws_bytes));      // the ticket words start at zero, once
  }

  const sdv2_stride3 token_major = {(int64_t)n_chunk, (int64_t)heads * 128, 128};
  const sdv2_stride3 head_major = {(int64_t)n_cache, 128, (int64_t)cap * 128};   // [heads][cap][128] in memory
  std::vector<uint16_t> host(n_chunk);
  for (int c = 0; c < chunks; ++c) {
    int64_t sched[4];
    if (!read_n(in, sched, 4)) return 2;
    for (uint16_t* dst : {d_q, d_k, d_v}) {
      if (!read_n(in, host.data(), n_chunk)) return 2;
      HIP_OK(hipMemcpyAsync(dst, host.data(), n_chunk * 2, hipMemcpyHostToDevice, stream));
      HIP_OK(hipStreamSynchronize(stream));
    }
    sdv2_append_params ap = {};
    ap.q_in = d_q; ap.k_in = d_k; ap.v_in = d_v; ap.q_out = d_rq; ap.k_cache = d_kc; ap.v_cache = d_vc;
    ap.q_in_stride = ap.k_in_stride = ap.v_in_stride = ap.q_out_stride = token_major;
    ap.k_cache_stride = ap.v_cache_stride = head_major;
    ap.freqs = d_table; ap.freq_rows = freq_rows; ap.dtype = SDV2_BF16;
    ap.rows = 1; ap.tokens = tokens; ap.heads = heads; ap.head_dim = SDV2_HEAD_DIM;
    ap.grid_f = hdr[3]; ap.grid_h = hdr[4]; ap.grid_w = hdr[5];
    ap.cache_tokens = cap;
    ap.start_frame = &sched[0]; ap.dst_start = &sched[1];
    ap.global_end_index = d_idx; ap.local_end_index = d_idx + 1;
    ap.new_global_end = &sched[2]; ap.new_local_end = &sched[3];
    ap.stream = stream;
    SDV2_OK_OR_DIE(sdv2_kv_append_rope(&ap));

    const int32_t len = (int32_t)sched[3];
    HIP_OK(hipMemcpyAsync(d_len, &len, sizeof len, hipMemcpyHostToDevice, stream));
    sdv2_attn_params at = {};
    at.q = d_rq; at.k_cache = d_kc; at.v_cache = d_vc; at.out = d_o; at.seq_lens = d_len;
    at.q_stride = at.out_stride = token_major;
    at.k_stride = at.v_stride = head_major;
    at.rows = 1; at.q_tokens = tokens; at.heads = heads; at.head_dim = SDV2_HEAD_DIM;
    at.max_seq_len = cap; at.num_splits = splits;
    at.workspace = d_ws; at.workspace_bytes = ws_bytes; at.stream = stream;
    SDV2_OK_OR_DIE(sdv2_swa_attn_fwd(&at));
    HIP_OK(hipStreamSynchronize(stream));
    for (uint16_t* src : {d_rq, d_o}) {
      HIP_OK(hipMemcpy(host.data(), src, n_chunk * 2, hipMemcpyDeviceToHost));
      std::fwrite(host.data(), 2, n_chunk, out);
    }
  }
  std::vector<uint16_t> cache(n_cache);
  for (uint16_t* src : {d_kc, d_vc}) {
    HIP_OK(hipMemcpy(cache.data(), src, n_cache * 2, hipMemcpyDeviceToHost));
    std::fwrite(cache.data(), 2, n_cache, out);
  }
  int64_t idx[2];
  HIP_OK(hipMemcpy(idx, d_idx, sizeof idx, hipMemcpyDeviceToHost));
  std::fwrite(idx, sizeof(int64_t), 2, out);
  std::fclose(out);
  std::fclose(in);
  std::printf("gpu_caller: %d chunks done\n", chunks);
  return 0;
}
