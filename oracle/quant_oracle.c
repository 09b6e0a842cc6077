/*
 * TEST INFRASTRUCTURE ONLY -- CPU restatement of the reference's per-token
 * asymmetric INT8 quantizer.  Nothing in the shipped package may link, load or
 * call this file; it exists so tests and the CPU-baseline leg of the benchmark
 * have an independent answer to compare the HIP kernels with.
 *
 * Follows /root/reference/asymmetric_quant.py:66-106 step by step:
 *   :80-81   min / max of the token row (as fp32 values)
 *   :84-86   scale = (max - min) / (127 - (-128))         fp32 sub, fp32 IEEE div
 *   :87      scale == 0  ->  1.0
 *   :89      zero_point_float = -128 - min / scale        fp32 div, then fp32 sub
 *   :90-91   zero_point = clamp(roundf(.), -128, 127)     roundf: half AWAY from zero
 *   :103-104 code = clamp(roundf(x / scale + zero_point), -128, 127)
 *            (uses the unrounded fp32 scale, not the fp16 copy that is stored)
 * The additional row sum of the codes is not in the reference: it is the
 * side output the INT8 attention kernels use for the zero-point cross term.
 *
 * Build:  make -C oracle      (gcc -O2 -ffp-contract=off, no fast-math: every
 * operation below is a single correctly rounded IEEE-754 binary32 operation).
 */
#include <math.h>
#include <stdint.h>

static inline float clampf(float v, float lo, float hi) {
  /* reference: tl.maximum(q_min, tl.minimum(q_max, v)) */
  float t = v < hi ? v : hi;
  return t > lo ? t : lo;
}

void qfa_oracle_quant_rows_f32(const float *x, int64_t rows, int64_t D,
                               int8_t *codes, float *scale_out, int8_t *zp_out,
                               int32_t *rowsum_out) {
  for (int64_t r = 0; r < rows; ++r) {
    const float *row = x + r * D;
    float mn = INFINITY, mx = -INFINITY;
    for (int64_t d = 0; d < D; ++d) {
      float v = row[d];
      if (v < mn) mn = v;
      if (v > mx) mx = v;
    }
    volatile float range = mx - mn;          /* volatile: forbid re-association */
    volatile float scale = range / 255.0f;
    if (scale == 0.0f) scale = 1.0f;
    volatile float ratio = mn / scale;
    volatile float zpf = -128.0f - ratio;
    float zp = clampf(roundf(zpf), -128.0f, 127.0f);
    int32_t sum = 0;
    for (int64_t d = 0; d < D; ++d) {
      volatile float q = row[d] / scale;
      volatile float y = q + zp;
      float c = clampf(roundf(y), -128.0f, 127.0f);
      int8_t ci = (int8_t)c;
      codes[r * D + d] = ci;
      sum += ci;
    }
    scale_out[r] = scale;
    zp_out[r] = (int8_t)zp;
    if (rowsum_out) rowsum_out[r] = sum;
  }
}

/* dequantize: /root/reference/asymmetric_quant.py:160
 *   (codes.float() - zp.float()) * scale.float()                             */
void qfa_oracle_dequant_rows_f32(const int8_t *codes, const float *scale,
                                 const int8_t *zp, int64_t rows, int64_t D,
                                 float *out) {
  for (int64_t r = 0; r < rows; ++r)
    for (int64_t d = 0; d < D; ++d) {
      volatile float diff = (float)codes[r * D + d] - (float)zp[r];
      out[r * D + d] = diff * scale[r];
    }
}
