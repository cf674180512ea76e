/*
 * sdv2kv — C ABI of the MI355X (gfx950) ring-buffer KV-cache path for the
 * causal Wan DiT of StreamDiffusionV2.
 *
 * Four operators, all enqueued on a caller-supplied HIP stream, all working
 * on caller-owned device memory (the library keeps no state between calls; the
 * one entry point that brings its own scratch memory says so):
 *
 *   sdv2_kv_append_rope   fused RoPE-on-write chunk append
 *   sdv2_swa_attn_fwd     chunk-Q x (sink + window) K/V flash attention
 *   sdv2_sink_similarity  adaptive sink refresh decision
 *   sdv2_cache_relayout   cache block <-> token-major wire format (owner change)
 *
 * Tensors are addressed as [rows, tokens, heads, 128] with explicit element
 * strides for the first three dimensions; the last dimension is contiguous.
 * This lets one binary serve the reference's token-major cache
 * ([B, cap, H, 128], models/wan/causal_stream_inference.py:98-100) and the
 * head-major physical layout ([B, H, cap, 128] exposed as a permuted view)
 * that the kernels prefer.
 *
 * All functions return SDV2_OK (0) or a negative sdv2_status; they never
 * throw, never synchronise the device and never allocate device memory.
 */
#ifndef SDV2KV_H
#define SDV2KV_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define SDV2KV_ABI_VERSION 12
#define SDV2_HEAD_DIM 128      /* causal_stream_inference.py:99-100 fixes 128 */
#define SDV2_MAX_ROWS 16       /* rows (B) per sdv2_kv_append_rope call       */
#define SDV2_MAX_SINK_FRAMES 16 /* sink frames per sdv2_sink_similarity call  */

typedef enum sdv2_status {
  SDV2_OK = 0,
  SDV2_ERR_INVALID_ARG = -1,   /* null pointer, bad shape, misaligned stride  */
  SDV2_ERR_UNSUPPORTED = -2,   /* head_dim != 128, unknown dtype              */
  SDV2_ERR_OUT_OF_RANGE = -3,  /* write range outside the cache, RoPE row     */
                               /* beyond the table                            */
  SDV2_ERR_WORKSPACE = -4,     /* split-KV workspace missing or too small     */
  SDV2_ERR_LAUNCH = -5,        /* hipLaunchKernel reported an error           */
  SDV2_ERR_SCRATCH_LIMIT = -6  /* sdv2_swa_attn_fwd_static: the call needs    */
                               /* more than SDV2_STATIC_SCRATCH_BYTES         */
} sdv2_status;

typedef enum sdv2_dtype {
  SDV2_BF16 = 0,
  SDV2_F32 = 1                 /* the reference's CPU-runnable configuration: */
                               /* same operators, fp32 storage and arithmetic */
} sdv2_dtype;

/* element strides of a [rows, tokens, heads, 128] tensor */
typedef struct sdv2_stride3 {
  int64_t row;
  int64_t token;
  int64_t head;
} sdv2_stride3;

int sdv2_abi_version(void);
const char* sdv2_status_string(int status);

/* ------------------------------------------------------------------------
 * Fused RoPE-on-write chunk append.
 *
 * Replaces, for one transformer layer, the reference's
 *   causal_rope_apply(q), causal_rope_apply(k)   models/wan/causal_model.py:253-266 (-> :94-108)
 *   kv_cache["k"|"v"][i, a:b] = ...              models/wan/causal_model.py:321-322, 336-337
 *   kv_cache["global_end_index"|"local_end_index"][i].fill_(...)   :339-342
 *
 * For every row i and chunk token t (grid position (f,h,w) row-major,
 * absolute frame start_frame[i] + f):
 *   q_out[i,t]              = rope(q_in[i,t])
 *   k_cache[i,dst_start[i]+t] = rope(k_in[i,t])
 *   v_cache[i,dst_start[i]+t] = v_in[i,t]
 * rope() multiplies the 64 interleaved (even, odd) pairs of each head by the
 * complex128 table entry in IEEE double without fused multiply-add and rounds
 * double -> float (-> bfloat16, nearest-even), which is what the reference's
 * float64 complex multiply followed by .type_as() produces.  Pair p uses
 * table row `frame` for p < 22, `h` for 22 <= p < 43 and `w` for p >= 43, at
 * column p (causal_model.py:64-68, 77-78).
 *
 * Which slot a chunk lands in (dst_start) and the new index values are
 * decided by the caller's ring state machine (causal_model.py:302-342); the
 * kernel only performs the scatter and stores the two int64 indices, so
 * eviction costs nothing beyond the write of the new chunk.
 *
 * With k_in, v_in, k_cache and v_cache all NULL the call is the reference's
 * causal_rope_apply on its own (causal_model.py:94-108): q_out = rope(q_in),
 * no cache, index or dst_start is read or written.
 * ---------------------------------------------------------------------- */
typedef struct sdv2_append_params {
  const void* q_in;            /* [B,S,H,128]; may be NULL together with q_out */
  const void* k_in;            /* k_in, v_in and the caches: all or none       */
  const void* v_in;
  void* q_out;                 /* [B,S,H,128] roped query                      */
  void* k_cache;               /* [B,cap,H,128]                                */
  void* v_cache;
  sdv2_stride3 q_in_stride, k_in_stride, v_in_stride;
  sdv2_stride3 q_out_stride, k_cache_stride, v_cache_stride;
  const double* freqs;         /* device, complex128 [freq_rows, 64] as (re,im) */
  int32_t freq_rows;
  int32_t dtype;               /* sdv2_dtype of all six tensors                */
  int32_t rows, tokens, heads, head_dim;          /* B, S, H, 128              */
  int32_t grid_f, grid_h, grid_w;                 /* tokens == f*h*w           */
  int64_t cache_tokens;                           /* cap                       */
  const int64_t* start_frame;  /* host [B]: current_start // (h*w)             */
  const int64_t* dst_start;    /* host [B]: first cache token written          */
  int64_t* global_end_index;   /* device int64 [B], may be NULL                */
  int64_t* local_end_index;    /* device int64 [B], may be NULL                */
  const int64_t* new_global_end;  /* host [B] values stored by the kernel      */
  const int64_t* new_local_end;   /* host [B]                                  */
  void* stream;                /* hipStream_t                                  */
  /* Optional: fold the q / k RMSNorm of the projection outputs in (WanRMSNorm,
   * wan_base/modules/model.py:70-86, applied in qkv_fn, causal_model.py:212-218).
   * With both weights given, q_in and k_in are the raw projection outputs and
   *   x' = type_as(float(x) * rsqrt(mean_over_heads*128(float(x)^2) + norm_eps)) * weight
   * is what gets roped.  Weights have the tensors' dtype, heads * 128 elements.
   * The fp32 sum of squares is taken in the order of PyTorch's CPU sum kernel
   * (vectors of 8 floats, 4 accumulators, blocks of 16), so the result is bit
   * for bit what the two torch modules followed by the plain append store.     */
  const void* q_norm_weight;   /* device, or NULL (together with k_norm_weight) */
  const void* k_norm_weight;
  float norm_eps;
  /* Optional slot chosen on the device: device int64 [B] or NULL.  A value
   * >= 0 (and fitting the cache) replaces dst_start[i]; sdv2_sink_similarity
   * writes it, so that an adaptive sink refresh needs no host round trip
   * between the decision and the append.                                      */
  const int64_t* dst_start_override;
  /* Optional, with the norm weights: device float [B * S] that receives
   * rsqrt(mean(q^2) + norm_eps) of every query token.  q_out may then be NULL:
   * no rotated query is written, and sdv2_swa_attn_fwd normalises and rotates
   * the raw q itself (its q_norm_weight / q_inv_rms), to the same bits.       */
  float* q_inv_rms;
} sdv2_append_params;

int sdv2_kv_append_rope(const sdv2_append_params* p);

/* ------------------------------------------------------------------------
 * Sliding-window (sink + window) attention of the chunk's queries against
 * the cache, read in place in physical slot order.
 *
 * Replaces flash_attn_interface.flash_attn_with_kvcache(q=, k_cache=,
 * v_cache=, cache_seqlens=) as called at models/wan/causal_model.py:353-358
 * and its SDPA fallback attention_with_kvcache_fallback (:111-157):
 *   out[i] = softmax(q[i] k_cache[i,:seq_lens[i]]^T / sqrt(128)) v_cache[i,:seq_lens[i]]
 * with no mask inside the chunk (causal=False) unless one is asked for (see
 * mask_block_tokens) and keys at or beyond seq_lens[i] ignored.  bf16 in, fp32
 * accumulation, bf16 out - or, with dtype = SDV2_F32, fp32 tensors and fp32
 * arithmetic throughout (what the fallback computes on the reference's CPU-
 * runnable fp32 configuration).
 *
 * Long caches are split over key ranges to fill the 256 CUs; partial results
 * go through `workspace` (size from sdv2_swa_attn_workspace_bytes) and the
 * workgroup that finishes a query tile's last range combines them, in the same
 * launch.  The workspace begins with one ticket word per (row, head, query
 * tile): it must be ZERO-FILLED ONCE after allocation (hipMemset, or any fill)
 * before its first use; every call leaves the tickets at zero again, whatever
 * shape it had, so the same workspace can serve any sequence of calls that do
 * not overlap in time.
 *
 * The query may arrive before RoPE (rope_freqs != NULL): it is then rotated
 * while it is loaded, with the arithmetic of sdv2_kv_append_rope, so the
 * append that precedes the call need not write a rotated copy of q
 * (causal_model.py:253-266 rotates q only to feed it to this operator).
 * ---------------------------------------------------------------------- */
typedef struct sdv2_attn_params {
  const void* q;               /* [B,S,H,128] bf16 or fp32, see dtype (roped)  */
  const void* k_cache;         /* [B,L,H,128] view of the cache, same dtype    */
  const void* v_cache;
  void* out;                   /* [B,S,H,128], same dtype                      */
  const int32_t* seq_lens;     /* device int32 [B]; NULL = every row uses L    */
  sdv2_stride3 q_stride, k_stride, v_stride, out_stride;
  int32_t rows, q_tokens, heads, head_dim;        /* B, S, H, 128              */
  int32_t max_seq_len;                            /* L = k_cache.shape[1]      */
  int32_t num_splits;          /* key ranges per (row, head); 0 = choose from the
                                * shape.  Bits 0-7: the count s (<= 64).  Bits 8-15
                                * (optional, needs rows * heads divisible by 8): of
                                * every eighth of the (row, head) list - one XCD's
                                * share - that many pairs take s + 1 ranges instead,
                                * which fills the last round of workgroups better.
                                * sdv2_swa_attn_default_splits returns this form.  */
  float softmax_scale;         /* <= 0 selects 1/sqrt(head_dim)                */
  void* workspace;             /* device scratch, 256-byte aligned             */
  size_t workspace_bytes;
  void* stream;                /* hipStream_t                                  */
  /* Optional block-causal mask INSIDE the chunk.  The reference's cache path
   * applies none (the chunk is one block); its cache-less path masks with
   * kv_idx < ends[q_idx] (causal_model.py:670-686).  With mask_block_tokens =
   * b in (0, S) and the chunk's own keys at cache positions
   * [chunk_key_start[i], chunk_key_start[i] + S), query token t of row i does
   * not see the chunk's later blocks, i.e. cache positions
   * [chunk_key_start[i] + (t / b + 1) * b, chunk_key_start[i] + S); everything
   * else in the cache is older and stays visible.  0 (or b >= S) = no mask.  */
  int32_t mask_block_tokens;
  const int32_t* chunk_key_start;  /* device int32 [B], each in [0, L - S]; may be */
                                   /* NULL when the mask is off                    */
  /* Optional RoPE of q inside the call.  rope_freqs = the device table of
   * sdv2_kv_append_rope (complex128 [rope_freq_rows, 64] as (re, im)), or NULL
   * when q is already rotated.  The chunk's S tokens are S / (grid_h * grid_w)
   * whole frames in (f, h, w) row-major order, the first at absolute frame
   * rope_start_frame[i]; at most SDV2_MAX_ROWS rows.                         */
  const double* rope_freqs;
  int32_t rope_freq_rows;
  int32_t rope_grid_h, rope_grid_w;
  const int64_t* rope_start_frame; /* host [B]                                     */
  /* sdv2_dtype of q, both caches and out.  SDV2_BF16 (0): the matrix-core
   * kernel.  SDV2_F32: what the reference's fallback operator computes on fp32
   * tensors (causal_model.py:111-157) - products, sums and softmax in fp32,
   * one key range (num_splits, workspace and rope_freqs must be unset: fp32
   * queries arrive rotated), strides in multiples of 4 elements.             */
  int32_t dtype;
  /* Optional q RMSNorm inside the call (needs rope_freqs and SDV2_BF16): q is
   * the raw q projection, q_norm_weight the norm's weight (device, bf16,
   * heads * 128 elements, 16-byte aligned) and q_inv_rms what
   * sdv2_kv_append_rope stored (device float [B * S]).  Every element is
   * normalised (x * inv_rms rounded to bf16, times weight rounded to bf16, as
   * WanRMSNorm rounds, wan_base/modules/model.py:77-86) and then rotated.      */
  const void* q_norm_weight;
  const float* q_inv_rms;
} sdv2_attn_params;

/* the key-range split plan the library would pick for this shape, as num_splits carries it */
int sdv2_swa_attn_default_splits(int32_t rows, int32_t q_tokens, int32_t heads, int32_t max_seq_len);
/* bytes of workspace needed for `num_splits` (0 = default); 0 when unsplit */
size_t sdv2_swa_attn_workspace_bytes(int32_t rows, int32_t q_tokens, int32_t heads,
                                     int32_t max_seq_len, int32_t num_splits);
int sdv2_swa_attn_fwd(const sdv2_attn_params* p);

/* ------------------------------------------------------------------------
 * sdv2_swa_attn_fwd for callers that cannot allocate.  No counterpart in the
 * reference: it is for code under HIP graph capture, tight serving loops and
 * harnesses that forbid hipMalloc, which cannot size and bring the workspace
 * a split call needs.  Same arguments, kernels and results as
 * sdv2_swa_attn_fwd, except that `workspace` / `workspace_bytes` are ignored:
 * the partial results of a split call go to SDV2_STATIC_SCRATCH_BYTES of
 * device memory that the library itself holds on every GPU it runs on, from
 * load to process exit.  A call whose sdv2_swa_attn_workspace_bytes() exceeds
 * that returns SDV2_ERR_SCRATCH_LIMIT and launches nothing (64 MiB covers the
 * Wan 1.3B and 14B shapes at 480p: one row of a 1560-token chunk against six
 * frames).  The call allocates and frees nothing and does not synchronise.
 * The scratch starts out zeroed and every call leaves its ticket words at zero
 * again, so nothing has to be cleared between calls, but all calls on one GPU
 * share it: two calls that overlap in time on one GPU - different streams,
 * threads or graphs replayed concurrently - race.
 * ---------------------------------------------------------------------- */
#define SDV2_STATIC_SCRATCH_BYTES (64u << 20)
int sdv2_swa_attn_fwd_static(const sdv2_attn_params* p);

/* ------------------------------------------------------------------------
 * Adaptive sink refresh decision.
 *
 * Replaces models/wan/causal_model.py:284-299, which runs before the ring
 * placement of a one-frame chunk when sink_size > 0 and adapt_sink_thr > -1:
 *   k_sink_mean[j] = mean over tokens of cached K frame j   (j < sink_frames)
 *   k_new_mean     = mean over tokens of rope(k_in)
 *   sim[j] = (cos(k_sink_mean[j], k_new_mean) + cos(v_sink_mean[j], v_new_mean)) / 2
 *   refresh = argmin_j sim[j] if min_j sim[j] < threshold else -1
 * with the cosine taken over the flattened heads x 128 vector.  The caller
 * reads `refresh` back and, for a row with refresh >= 0, puts
 * (refresh + 1) * tokens at the head of that row's eviction queue (:297-299).
 * k_in is the chunk's key BEFORE RoPE (the kernel rotates it exactly as
 * sdv2_kv_append_rope does); the cache is read as it is before this call's
 * append.  With bf16 tensors the means, both cosines and their sum are rounded
 * to bf16, as the reference's bf16 tensors are.
 * ---------------------------------------------------------------------- */
typedef struct sdv2_sink_sim_params {
  const void* k_in;            /* [B,S,H,128] new keys, not yet roped          */
  const void* v_in;            /* [B,S,H,128] new values                       */
  const void* k_cache;         /* [B,cap,H,128]                                */
  const void* v_cache;
  sdv2_stride3 k_in_stride, v_in_stride, k_cache_stride, v_cache_stride;
  const double* freqs;         /* device, complex128 [freq_rows, 64] as (re,im) */
  int32_t freq_rows;
  int32_t dtype;               /* sdv2_dtype of the four tensors               */
  int32_t rows, tokens, heads, head_dim;          /* B, S, H, 128              */
  int32_t grid_h, grid_w;      /* tokens == grid_h * grid_w: exactly one frame */
  int32_t sink_frames;         /* sink_size                                    */
  float threshold;             /* adapt_sink_thr                               */
  int64_t cache_tokens;        /* cap                                          */
  const int64_t* start_frame;  /* host [B]: current_start // tokens            */
  float* similarity;           /* device float [B, sink_frames]                */
  int32_t* refresh;            /* device int32 [B]                             */
  void* workspace;             /* device scratch, sdv2_sink_similarity_workspace_bytes():
                                * its first 256 bytes are ticket words that must be ZERO
                                * when the buffer is first used (every call leaves them at
                                * zero); calls that overlap in time need a buffer each      */
  size_t workspace_bytes;
  void* stream;                /* hipStream_t                                  */
  /* Optional hand-over to the append that follows on the stream: device int64
   * [B] or NULL.  Row i gets refresh[i] * tokens (the start of the refreshed
   * sink frame: the slot (refresh + 1) * tokens at the head of the queue is
   * where an evicting call writes, causal_model.py:297-306, 321-322) when it
   * refreshes AND bit i of override_rows is set (= the caller's ring state
   * says the row is on the evict branch; a row still filling writes at its
   * fill position whatever the queue head is, :326-337), else -1.            */
  int64_t* dst_start_override;
  uint32_t override_rows;
  /* Optional: k_in is the raw k projection and its RMSNorm (WanRMSNorm,
   * wan_base/modules/model.py:70-86) is folded in, as in sdv2_kv_append_rope:
   * the weight (heads * 128 elements of the tensors' dtype) and eps.          */
  const void* k_norm_weight;
  float norm_eps;
  /* Optional: the means of the cached sink frames kept between calls (device,
   * sdv2_sink_frame_sums_bytes(), any initial contents, opaque to the caller).
   * The mean of a sink frame only changes when the frame is written, so a
   * caller that brings this buffer has the call read the new chunk alone:
   *   - stale_frames[i] (host [B]): bit j set = sink frame j of row i was
   *     written by something other than the appends this call was told about
   *     since its mean was last taken (or never summed): it is summed from the
   *     cache in this call;
   *   - planned_frame[i] (host [B]): the sink frame the append that follows
   *     writes row i's chunk to by the caller's plan (a cache still filling,
   *     or a queue headed by an earlier refresh), or -1.  The new chunk's means
   *     are then filed as that frame's; for a row flagged in override_rows
   *     that refreshes in this call, as the refreshed frame's instead.
   * All three NULL: every sink frame is summed from the cache, every call.    */
  float* frame_sums;
  const uint32_t* stale_frames;
  const int32_t* planned_frame;
} sdv2_sink_sim_params;

size_t sdv2_sink_similarity_workspace_bytes(int32_t rows, int32_t tokens, int32_t heads, int32_t sink_frames);
size_t sdv2_sink_frame_sums_bytes(int32_t rows, int32_t heads, int32_t sink_frames);
int sdv2_sink_similarity(const sdv2_sink_sim_params* p);

/* ------------------------------------------------------------------------
 * Layout-changing copy of one layer's cache block, with the index hand-over.
 *
 * Serves the owner change of a block in the reference's pipeline-parallel
 * mode, KVCacheManager.broadcast_kv_blocks
 * (streamv2v/communication/kv_cache_manager.py:48-84): the donor's
 * kv_cache1[i]["k"], ["v"], ["global_end_index"], ["local_end_index"] replace
 * the receiver's (:70-78) and a receiver of lower rank then adds
 * frame_seq_length * (donor - rank) * num_steps to global_end_index (:81-82).
 * The transport itself (dist.broadcast) is the caller's; what travels is the
 * reference's tensor, token-major contiguous [B, cap, H, 128].  This call
 * produces that buffer from a cache in any stride order (src = cache, dst =
 * wire) and absorbs it on the other side (src = wire, dst = cache):
 *   dst[i, t, h, :] = src[i, t, h, :]
 *   dst_global_end_index[i] = src_global_end_index[i] + global_end_shift
 *   dst_local_end_index[i]  = src_local_end_index[i]
 * The index part is skipped for a NULL dst pointer; tokens == 0 moves the
 * indices only.  src and dst must not overlap.
 * ---------------------------------------------------------------------- */
typedef struct sdv2_relayout_params {
  const void* src;             /* [B,cap,H,128]                                */
  void* dst;
  sdv2_stride3 src_stride, dst_stride;
  int32_t dtype;               /* sdv2_dtype of both tensors                   */
  int32_t rows, heads, head_dim;                  /* B, H, 128                 */
  int64_t tokens;                                 /* cap                       */
  const int64_t* src_global_end_index;            /* device int64 [B] or NULL  */
  const int64_t* src_local_end_index;
  int64_t* dst_global_end_index;                  /* device int64 [B] or NULL  */
  int64_t* dst_local_end_index;
  int64_t global_end_shift;
  void* stream;                /* hipStream_t                                  */
} sdv2_relayout_params;

int sdv2_cache_relayout(const sdv2_relayout_params* p);

/* ------------------------------------------------------------------------
 * RMS norm over the model width, as a call of its own.
 *
 * Replaces WanRMSNorm.forward (models/wan/wan_base/modules/model.py:77-86)
 * where the norm is not folded into sdv2_kv_append_rope: norm_q of the text
 * cross-attention (model.py:181), and norm_q / norm_k of the self-attention
 * when a caller applies them apart (causal_model.py:212-218):
 *   out[t, :] = type_as(float(x[t, :]) * rsqrt(mean(float(x[t, :])^2) + eps)) * weight
 * for every token t, with the three roundings of the torch expression.  The
 * fp32 sum of squares is taken in the order of PyTorch's CPU sum kernel, as in
 * sdv2_kv_append_rope, so the result is bit for bit the torch module's on the
 * CPU.  width must be a multiple of 128, at most 64 * 128; rows are `width`
 * contiguous elements, x_token_stride / out_token_stride elements apart (a
 * slice of a wider projection output works); out may be x.
 * ---------------------------------------------------------------------- */
typedef struct sdv2_rms_norm_params {
  const void* x;               /* [tokens, width]                              */
  void* out;                   /* [tokens, width]                              */
  const void* weight;          /* [width], the tensors' dtype                  */
  int64_t x_token_stride;      /* elements                                     */
  int64_t out_token_stride;
  int64_t tokens;
  int32_t width;
  int32_t dtype;               /* sdv2_dtype of x, out and weight              */
  float eps;
  void* stream;                /* hipStream_t                                  */
} sdv2_rms_norm_params;

int sdv2_rms_norm(const sdv2_rms_norm_params* p);

#ifdef __cplusplus
}
#endif
#endif /* SDV2KV_H */
