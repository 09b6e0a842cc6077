// Host-side declarations shared by the translation units of libqfa.so: the error
// channel behind qfa_last_error() and the launchers the C entry points dispatch to.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/qfa.h"

namespace qfa {

// Records a thread-local message and returns `code` (so `return set_error(...)` reads naturally).
int set_error(int code, const char *fmt, ...) __attribute__((format(printf, 2, 3)));
// hipGetLastError() after a launch; 0 or the positive hipError_t, with the message recorded.
int check_launch(const char *what);

int launch_quant(const void *x, int x_dtype, int8_t *codes, float *scale, void *scale_lp, int scale_lp_dtype,
                 int8_t *zp, int32_t *rowsum, int64_t B, int64_t H, int64_t N, int D, int64_t sxb, int64_t sxh,
                 int64_t sxn, int64_t scb, int64_t sch, int64_t scn, hipStream_t st);
// the same for two tensors of one element type and head dimension in one launch (no 16-bit scale copy)
int launch_quant_pair(const void *const x[2], int x_dtype, int8_t *const codes[2], float *const scale[2],
                      int8_t *const zp[2], int32_t *const rowsum[2], int64_t B, int64_t H, const int64_t N[2], int D,
                      const int64_t sx[2][3], const int64_t sc[2][3], hipStream_t st);
int launch_rowsum(const int8_t *codes, int32_t *rowsum, int64_t B, int64_t H, int64_t N, int D, int64_t scb,
                  int64_t sch, int64_t scn, hipStream_t st);
int launch_dequant(const int8_t *codes, const void *scale, int scale_dtype, const int8_t *zp, void *out,
                   int out_dtype, int64_t B, int64_t H, int64_t N, int D, int64_t scb, int64_t sch, int64_t scn,
                   int64_t sob, int64_t soh, int64_t son, hipStream_t st);

// Tensors of one attention call, after validation.  Strides in elements.
struct AttnArgs {
  const int8_t *qc; const float *sq; const int8_t *zq; const int32_t *rq;
  const int8_t *kc; const float *sk; const int8_t *zk; const int32_t *rk;
  const void *v; void *o; float *lse;
  const void *dout; void *workspace; void *dq; void *dk; void *dv;   // backward only
  int64_t B, H, Nq, Nk;
  int64_t sqb, sqh, sqn, skb, skh, skn, svb, svh, svn, sob, soh, son;
  int64_t sdob, sdoh, sdon, sdqb, sdqh, sdqn, sdkb, sdkh, sdkn, sdvb, sdvh, sdvn;
  float sm_scale;
  int causal;
  int D;
  int io_dtype;
};

int launch_fwd(const AttnArgs &a, hipStream_t st, bool qk_only = false);
int launch_delta(const void *o, const void *dout, float *delta, int io_dtype, int64_t B, int64_t H, int64_t N, int D,
                 int64_t sob, int64_t soh, int64_t son, int64_t sdb, int64_t sdh, int64_t sdn, hipStream_t st);
int launch_bwd(const AttnArgs &a, hipStream_t st);
int launch_sum16(const void *a, const void *b, void *out, int dtype, int64_t n, hipStream_t st);   // out = a + b, n % 8 == 0
int64_t bwd_workspace_bytes(int64_t B, int64_t H, int64_t Nq, int64_t Nk, int D);

// Shared-KV attention (K = V = one quantized tensor, Q in 16-bit float), after validation.
struct SkvAttnArgs {
  const void *q; const int8_t *codes; const void *scale; const int8_t *zp;
  void *o; float *lse;
  const void *dout; void *dq; void *dkv;   // backward only
  void *workspace;                         // forward only, nullable: partial results when the keys are split
  int64_t B, H, Nq, Nk;
  int64_t sqb, sqh, sqn, scb, sch, scn, sob, soh, son;
  int64_t sdob, sdoh, sdon, sdqb, sdqh, sdqn, sdkb, sdkh, sdkn;
  float sm_scale;
  int D, io_dtype, scale_dtype;
  int grad_dtype; const float *grad_scale;   // backward only: type of dq / dkv, optional device scalar multiplying them
};
int launch_skv_fwd(const SkvAttnArgs &a, hipStream_t st);
int64_t skv_fwd_workspace_bytes(int64_t B, int64_t H, int64_t Nq, int64_t Nk, int D);
// the same with the partial results of a split in the library's own static device array (a.workspace is ignored)
int launch_skv_fwd_static(const SkvAttnArgs &a, hipStream_t st);
int launch_skv_bwd(const SkvAttnArgs &a, hipStream_t st);        // io_dtype QFA_F16, Nq <= 32: one fused pass
// dO * 2^k as binary16 plus 2^-k for the binary16 backward kernels (k from max|dO| and the largest key scale);
// partials: dout_normalise_workspace_bytes() of scratch
int64_t dout_normalise_workspace_bytes();
int launch_dout_normalise(const void *dout, int dout_dtype, int64_t n, const void *scale, int scale_dtype, int64_t ns,
                          float *partials, void *out, float *back, hipStream_t st);
int launch_skv_bwd_long(const SkvAttnArgs &a, hipStream_t st);   // io_dtype QFA_F16, any Nq: dQ kernel + dKV kernel

}  // namespace qfa
