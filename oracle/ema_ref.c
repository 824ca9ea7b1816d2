/* Plain-C restatement of two reference operations, used to cross-check the
 * PyTorch restatement in ts_oracle.py bit for bit.  Test infrastructure only.
 *
 * ema_ref: benchmarks/byol/trainer.py:207-210 / benchmarks/moco-v3/main.py:
 *   138-143.  `detached * m + param_q.data * (1. - m)` is three fp32 tensor
 *   ops: t*fl32(m), s*fl32(1.-m) (the subtraction is done on Python doubles),
 *   and their sum, each rounded to fp32.  Compile with -ffp-contract=off.
 * cat_ref: torch.cat on dim 0 of contiguous pieces (tspipe/batch_ops.py:
 *   186-205) is a byte concatenation.
 */
#include <stdint.h>
#include <string.h>

void ema_ref(const float* t, const float* s, float* out, int64_t n, double m) {
  const float m32 = (float)m;
  const float c32 = (float)(1.0 - m);
  for (int64_t i = 0; i < n; ++i) {
    volatile float a = t[i] * m32;
    volatile float b = s[i] * c32;
    out[i] = a + b;
  }
}

void cat_ref(const void* const* pieces, const int64_t* bytes, int64_t n_pieces, void* out) {
  char* dst = (char*)out;
  for (int64_t i = 0; i < n_pieces; ++i) {
    memcpy(dst, pieces[i], (size_t)bytes[i]);
    dst += bytes[i];
  }
}
