/* A plain C caller of the sdv2kv C ABI: proves that include/sdv2kv.h is C
 * (not C++), that the library links from C, and that argument validation
 * answers with status codes before anything touches a GPU.  Built and run by
 * tests/test_capi_symbols.py; prints one line per check. */
#include <stddef.h>
#include <stdio.h>
#include <string.h>

#include "sdv2kv.h"
#include "sdv2kv_profile.h"

static int failures = 0;

static void expect(const char* what, int got, int want) {
  printf("%s: %d (%s)%s\n", what, got, sdv2_status_string(got), got == want ? "" : "  <-- UNEXPECTED");
  if (got != want) ++failures;
}

int main(void) {
  if (sdv2_abi_version() != SDV2KV_ABI_VERSION) {
    printf("ABI version %d, header says %d\n", sdv2_abi_version(), SDV2KV_ABI_VERSION);
    return 2;
  }
  expect("append(NULL)", sdv2_kv_append_rope(NULL), SDV2_ERR_INVALID_ARG);
  expect("attention(NULL)", sdv2_swa_attn_fwd(NULL), SDV2_ERR_INVALID_ARG);
  expect("sink_similarity(NULL)", sdv2_sink_similarity(NULL), SDV2_ERR_INVALID_ARG);

  sdv2_append_params ap;
  memset(&ap, 0, sizeof ap);
  ap.head_dim = 64;
  expect("append head_dim 64", sdv2_kv_append_rope(&ap), SDV2_ERR_UNSUPPORTED);
  ap.head_dim = SDV2_HEAD_DIM;
  ap.dtype = 7;
  expect("append unknown dtype", sdv2_kv_append_rope(&ap), SDV2_ERR_UNSUPPORTED);
  ap.dtype = SDV2_BF16;
  ap.heads = 12;
  ap.rows = SDV2_MAX_ROWS + 1;
  expect("append too many rows", sdv2_kv_append_rope(&ap), SDV2_ERR_INVALID_ARG);
  ap.rows = 0;
  expect("append of nothing", sdv2_kv_append_rope(&ap), SDV2_OK);
  ap.rows = 1;
  ap.tokens = 6;
  ap.grid_f = 1; ap.grid_h = 2; ap.grid_w = 2;     /* 4 != 6 tokens */
  expect("append grid/tokens mismatch", sdv2_kv_append_rope(&ap), SDV2_ERR_INVALID_ARG);

  sdv2_attn_params at;
  memset(&at, 0, sizeof at);
  at.head_dim = 96;
  expect("attention head_dim 96", sdv2_swa_attn_fwd(&at), SDV2_ERR_UNSUPPORTED);
  at.head_dim = SDV2_HEAD_DIM;
  at.heads = 12;
  at.rows = 0;
  expect("attention of nothing", sdv2_swa_attn_fwd(&at), SDV2_OK);
  at.rows = 1; at.q_tokens = 8; at.max_seq_len = 8;
  expect("attention null tensors", sdv2_swa_attn_fwd(&at), SDV2_ERR_INVALID_ARG);

  sdv2_relayout_params rl;
  expect("relayout(NULL)", sdv2_cache_relayout(NULL), SDV2_ERR_INVALID_ARG);
  memset(&rl, 0, sizeof rl);
  rl.head_dim = 64;
  expect("relayout head_dim 64", sdv2_cache_relayout(&rl), SDV2_ERR_UNSUPPORTED);
  rl.head_dim = SDV2_HEAD_DIM;
  expect("relayout of nothing", sdv2_cache_relayout(&rl), SDV2_OK);
  rl.rows = 1; rl.tokens = 4; rl.heads = 2;
  expect("relayout null tensors", sdv2_cache_relayout(&rl), SDV2_ERR_INVALID_ARG);
  rl.tokens = 0;
  rl.dst_global_end_index = (int64_t*)&rl;          /* destination index without a source */
  expect("relayout index without source", sdv2_cache_relayout(&rl), SDV2_ERR_INVALID_ARG);

  sdv2_rms_norm_params rn;
  expect("rms_norm(NULL)", sdv2_rms_norm(NULL), SDV2_ERR_INVALID_ARG);
  memset(&rn, 0, sizeof rn);
  rn.width = 100;
  expect("rms_norm width 100", sdv2_rms_norm(&rn), SDV2_ERR_UNSUPPORTED);
  rn.width = 65 * SDV2_HEAD_DIM;
  expect("rms_norm width 65 * 128", sdv2_rms_norm(&rn), SDV2_ERR_UNSUPPORTED);
  rn.width = 12 * SDV2_HEAD_DIM;
  expect("rms_norm of nothing", sdv2_rms_norm(&rn), SDV2_OK);
  rn.tokens = 4;
  expect("rms_norm null tensors", sdv2_rms_norm(&rn), SDV2_ERR_INVALID_ARG);
  rn.x = &rn; rn.out = &rn; rn.weight = &rn;                    /* (never launched: the stride below is refused) */
  rn.x_token_stride = 8;
  rn.out_token_stride = rn.width;
  expect("rms_norm rows that overlap", sdv2_rms_norm(&rn), SDV2_ERR_INVALID_ARG);

  /* struct layouts, for the bindings to compare themselves with */
  printf("layout sdv2_append_params size=%zu stream=%zu q_inv_rms=%zu\n", sizeof(sdv2_append_params),
         offsetof(sdv2_append_params, stream), offsetof(sdv2_append_params, q_inv_rms));
  printf("layout sdv2_attn_params size=%zu stream=%zu q_inv_rms=%zu\n", sizeof(sdv2_attn_params),
         offsetof(sdv2_attn_params, stream), offsetof(sdv2_attn_params, q_inv_rms));
  printf("layout sdv2_sink_sim_params size=%zu stream=%zu planned_frame=%zu\n", sizeof(sdv2_sink_sim_params),
         offsetof(sdv2_sink_sim_params, stream), offsetof(sdv2_sink_sim_params, planned_frame));
  printf("layout sdv2_rms_norm_params size=%zu stream=%zu eps=%zu\n", sizeof(sdv2_rms_norm_params),
         offsetof(sdv2_rms_norm_params, stream), offsetof(sdv2_rms_norm_params, eps));
  printf("layout sdv2_relayout_params size=%zu stream=%zu global_end_shift=%zu\n", sizeof(sdv2_relayout_params),
         offsetof(sdv2_relayout_params, stream), offsetof(sdv2_relayout_params, global_end_shift));

  printf("splits for 1x1560 tokens, 12 heads, 9360 keys: %d\n", sdv2_swa_attn_default_splits(1, 1560, 12, 9360));
  printf("workspace for that call: %zu bytes\n", sdv2_swa_attn_workspace_bytes(1, 1560, 12, 9360, 0));
  printf("sink-similarity workspace, 1 row, 12 heads, 3 sink frames: %zu bytes\n",
         sdv2_sink_similarity_workspace_bytes(1, 1560, 12, 3));
  expect("attention_static(NULL)", sdv2_swa_attn_fwd_static(NULL), SDV2_ERR_INVALID_ARG);
  expect("event_create(NULL)", sdv2_event_create(NULL), SDV2_ERR_INVALID_ARG);
  expect("time_next(unknown kernel)", sdv2_profile_time_next(SDV2_KERNEL_COUNT, NULL, NULL), SDV2_ERR_INVALID_ARG);
  expect("time_next(start only)", sdv2_profile_time_next(SDV2_KERNEL_APPEND, &failures, NULL), SDV2_ERR_INVALID_ARG);
  expect("time_next(disarm)", sdv2_profile_time_next(SDV2_KERNEL_APPEND, NULL, NULL), SDV2_OK);
  expect("copy of nothing", sdv2_copy_bytes(NULL, NULL, 0, NULL), SDV2_OK);
  printf(failures ? "FAILED: %d\n" : "all checks passed\n", failures);
  return failures ? 1 : 0;
}
