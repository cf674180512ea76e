/*
 * TEST INFRASTRUCTURE ONLY.  A second, independent restatement in plain C of
 * the two bit-exact pieces of the reference's KV-cache path, used by the CPU
 * tests to pin the PyTorch oracle (oracle/sdv2_oracle.py) from another side.
 * Nothing in the shipped package links or loads it.
 *
 *   sdv2_ref_rope      causal_rope_apply, models/wan/causal_model.py:94-108
 *                      with the table expansion of :57-91
 *   sdv2_ref_ring_step the placement state machine of
 *                      CausalWanSelfAttention.forward, :279-342
 *
 * Build with -ffp-contract=off: the reference multiplies complex128 numbers
 * on the CPU, every product and sum rounded once.
 */
#include <stdint.h>
#include <string.h>

static float bf16_to_float(uint16_t b) {
  uint32_t u = (uint32_t)b << 16;
  float f;
  memcpy(&f, &u, sizeof f);
  return f;
}

/* float -> bfloat16, round to nearest even (what .type_as() applies after the
 * double has been narrowed to float) */
static uint16_t float_to_bf16(float f) {
  uint32_t u;
  memcpy(&u, &f, sizeof u);
  if ((u & 0x7fffffffu) > 0x7f800000u) return 0x7fc0;
  return (uint16_t)((u + 0x7fffu + ((u >> 16) & 1u)) >> 16);
}

/*
 * x, out: [tokens, heads, 128] bf16 bit patterns (one row of the batch),
 * tokens = grid_f * grid_h * grid_w in row-major (f, h, w) order.
 * table: complex128 [freq_rows, 64] as (re, im) doubles.  Pair p of a head
 * uses table row (start_frame + f) for p < 22, row h for 22 <= p < 43, row w
 * for p >= 43, always at column p (causal_model.py:64-68, 77-78).
 * Returns 0, or -1 when a position lies outside the table.
 */
int sdv2_ref_rope(const uint16_t* x, uint16_t* out, int heads, const double* table, int freq_rows, int grid_f,
                  int grid_h, int grid_w, long start_frame) {
  const int pairs = 64, third = pairs / 3, split_t = pairs - 2 * third, split_h = split_t + third;
  if (start_frame < 0 || start_frame + grid_f > freq_rows || grid_h > freq_rows || grid_w > freq_rows) return -1;
  for (int f = 0; f < grid_f; ++f)
    for (int h = 0; h < grid_h; ++h)
      for (int w = 0; w < grid_w; ++w) {
        const long tok = ((long)f * grid_h + h) * grid_w + w;
        for (int hd = 0; hd < heads; ++hd) {
          const uint16_t* src = x + (tok * heads + hd) * 128;
          uint16_t* dst = out + (tok * heads + hd) * 128;
          for (int p = 0; p < pairs; ++p) {
            const long row = p < split_t ? start_frame + f : (p < split_h ? h : w);
            const double c = table[(row * pairs + p) * 2], s = table[(row * pairs + p) * 2 + 1];
            const double a = (double)bf16_to_float(src[2 * p]), b = (double)bf16_to_float(src[2 * p + 1]);
            const double re = a * c - b * s;
            const double im = a * s + b * c;
            dst[2 * p] = float_to_bf16((float)re);
            dst[2 * p + 1] = float_to_bf16((float)im);
          }
        }
      }
  return 0;
}

/*
 * One call of the placement logic for one cache row.
 * queue / queue_len: the row's eviction queue (slot END offsets), capacity
 * queue_cap; global_end / local_end: the row's two indices; current_step /
 * total_steps: the dict's pass counters.  Returns the first cache token the
 * chunk is written to, -1 when the cache is full and the queue is empty
 * (IndexError in the reference, :306), -2 when the queue would overflow
 * queue_cap.
 */
long sdv2_ref_ring_step(long* queue, int* queue_len, int queue_cap, long* global_end, long* local_end,
                        int* current_step, int total_steps, int cache_rows, long cap, long current_start,
                        long tokens, long frame_tokens, int sink_size) {
  const long sink_tokens = (long)sink_size * frame_tokens;
  const long c_end = current_start + tokens;
  long dst_end;
  if (c_end > cap || *local_end >= cap) {
    *global_end = current_start;
    *local_end = cap;
    if (*queue_len == 0) return -1;
    dst_end = queue[0];
    if (cache_rows == 1 && *current_step > 1) {
      *current_step -= 1;
    } else {
      const long head = queue[0];
      memmove(queue, queue + 1, (size_t)(*queue_len - 1) * sizeof(long));
      *queue_len -= 1;
      if (head > sink_tokens) queue[(*queue_len)++] = head;
      *current_step = total_steps;
    }
  } else {
    const long local_new = *local_end + c_end - *global_end;
    const long next_end = c_end + tokens;
    if (sink_tokens < next_end && next_end <= cap && (*queue_len == 0 || queue[*queue_len - 1] != next_end)) {
      if (*queue_len >= queue_cap) return -2;
      queue[(*queue_len)++] = next_end;
    }
    *local_end = local_new;
    dst_end = local_new;
  }
  *global_end = c_end;
  return dst_end - tokens;
}
