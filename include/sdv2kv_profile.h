/*
 * sdv2kv_profile — measurement hooks of libsdv2kv.so.
 *
 * Nothing here has a counterpart in the reference and no binding of the path
 * needs it: these calls exist so that a benchmark can time each kernel of the
 * path on its own and scale hardware counters.  The operator interface is
 * include/sdv2kv.h.
 */
#ifndef SDV2KV_PROFILE_H
#define SDV2KV_PROFILE_H

#include "sdv2kv.h"

#ifdef __cplusplus
extern "C" {
#endif

/* kernels a timing request can name */
typedef enum sdv2_profile_kernel {
  SDV2_KERNEL_APPEND = 0,      /* sdv2_kv_append_rope                          */
  SDV2_KERNEL_ATTENTION = 1,   /* sdv2_swa_attn_fwd                            */
  SDV2_KERNEL_RELAYOUT = 2,    /* sdv2_cache_relayout                          */
  SDV2_KERNEL_SINK = 3,        /* sdv2_sink_similarity                         */
  SDV2_KERNEL_COPY = 4,        /* sdv2_copy_bytes                              */
  SDV2_KERNEL_NORM = 5,        /* sdv2_rms_norm                                */
  SDV2_KERNEL_COUNT = 6
} sdv2_profile_kernel;

/* ------------------------------------------------------------------------
 * Timing events.  An event pair armed with sdv2_profile_time_next is recorded
 * in the dispatch of the NEXT launch of that kernel made by the calling thread
 * (start when the kernel begins to execute, stop when it has finished) and
 * then disarmed, so the interval is the kernel's own duration as a profiler
 * reports it, without the gap that separate event records on the stream would
 * add.  NULL, NULL disarms.  sdv2_event_elapsed_ms waits for the stop event.
 * ---------------------------------------------------------------------- */
int sdv2_event_create(void** event);
int sdv2_event_destroy(void* event);
int sdv2_event_elapsed_ms(void* start, void* stop, float* ms);
int sdv2_profile_time_next(int kernel, void* start, void* stop);

/* ------------------------------------------------------------------------
 * Plain device-to-device copy of `bytes` bytes with the library's own 16-byte
 * vector kernel, so that hardware counters (bytes fetched / written per
 * dispatch) can be scaled against a kernel whose traffic is known exactly.
 * ---------------------------------------------------------------------- */
int sdv2_copy_bytes(void* dst, const void* src, size_t bytes, void* stream);

/* ------------------------------------------------------------------------
 * What the GPU sustains on the attention kernel's own instruction streams.
 * One launch of a kernel that runs the attention loop's matrix instructions
 * on the caller's random operands, one workgroup per CU, `iterations` times
 * three 64-key tiles, with parts of the loop taken away by `mode`; *flops
 * receives the floating-point operations of the launch (32768 per MFMA).
 * The caller times the launch (events on `stream`).  `operands` is device
 * memory of at least sdv2_profile_mfma_stream_bytes() bytes, 256-byte aligned,
 * filled with bf16 values (random for the realistic case: the rate a chip
 * holds under matrix load depends on how much the operands toggle); only its
 * last 512 KB are written, if ever.  Nothing is computed that anybody reads.
 * ---------------------------------------------------------------------- */
typedef enum sdv2_stream_mode {
  SDV2_STREAM_REGISTERS = 0,      /* MFMAs alone, operands resident in registers               */
  SDV2_STREAM_LDS_32_ROWS = 1,    /* + LDS fragment reads as the attention kernel makes them:
                                     8 waves x 32 query rows, 1.5 reads per MFMA               */
  SDV2_STREAM_LDS_64_ROWS = 2,    /* the same with 4 waves x 64 query rows: 0.75 reads per MFMA */
  SDV2_STREAM_ATTENTION_MIX = 3,  /* mode 1 + the softmax instructions between the MFMAs + the
                                     global->LDS tile transfers and the barrier per tile       */
  SDV2_STREAM_ATTENTION_MIX_64_ROWS = 4   /* mode 2 + the same additions                        */
} sdv2_stream_mode;
size_t sdv2_profile_mfma_stream_bytes(void);
int sdv2_profile_mfma_stream(int mode, const void* operands, size_t operand_bytes, int32_t iterations,
                             void* stream, double* flops);

#ifdef __cplusplus
}
#endif
#endif /* SDV2KV_PROFILE_H */
