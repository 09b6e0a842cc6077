// C entry points of libqfa.so: argument validation, then dispatch to the kernel launchers.
// Validation touches no HIP API, so a rejected call works (and is testable) without a GPU.
#include <stdarg.h>
#include <stdio.h>
#include <string.h>

#include "qfa_host.h"

namespace qfa {

static thread_local char g_err[512] = "";

int set_error(int code, const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

int check_launch(const char *what) {
  const hipError_t e = hipGetLastError();
  if (e == hipSuccess) return 0;
  set_error((int)e, "%s: launch failed: %s", what, hipGetErrorString(e));
  return (int)e;
}

static constexpr int64_t kMaxTokens = 1LL << 28;   // longest sequence (Nq, Nk) the attention entry points take
static bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }
static bool aligned8(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 7u) == 0; }
static bool is_float_dtype(int d) { return d == QFA_F32 || d == QFA_F16 || d == QFA_BF16; }
static int elem_size(int d) { return d == QFA_F32 ? 4 : 2; }

// strides (elements) of a [B,H,N,D] tensor with element size `es`: positive, 16-byte multiples,
// and the token stride must at least span a row
static bool strides_ok(int64_t sb, int64_t sh, int64_t sn, int D, int es) {
  if (sb <= 0 || sh <= 0 || sn < D) return false;
  return (sb * es) % 16 == 0 && (sh * es) % 16 == 0 && (sn * es) % 16 == 0;
}

}  // namespace qfa

using namespace qfa;

extern "C" {

int qfa_version(void) { return QFA_VERSION; }

const char *qfa_last_error(void) { return g_err; }

int qfa_quant_per_token(const void *x, int x_dtype, int8_t *codes, float *scale_f32, void *scale_lp,
                        int scale_lp_dtype, int8_t *zp, int32_t *rowsum, int64_t B, int64_t H, int64_t N, int D,
                        int64_t sxb, int64_t sxh, int64_t sxn, int64_t scb, int64_t sch, int64_t scn, void *stream) {
  if (!x || !codes || !scale_f32 || !zp) return set_error(QFA_EINVAL, "quant: null x/codes/scale_f32/zp pointer");
  if (!is_float_dtype(x_dtype)) return set_error(QFA_EINVAL, "quant: x_dtype %d is not QFA_F32/F16/BF16", x_dtype);
  if (scale_lp && scale_lp_dtype != QFA_F16 && scale_lp_dtype != QFA_BF16)
    return set_error(QFA_EINVAL, "quant: scale_lp_dtype %d is not QFA_F16/BF16", scale_lp_dtype);
  if (B <= 0 || H <= 0 || N <= 0) return set_error(QFA_EINVAL, "quant: B, H, N must be positive");
  if (D < 8 || D > 256 || D % 8 != 0)
    return set_error(QFA_EUNSUPPORTED, "quant: head_dim %d is not a multiple of 8 between 8 and 256", D);
  if (!aligned16(x) || !aligned8(codes)) return set_error(QFA_EINVAL, "quant: x must be 16-byte, codes 8-byte aligned");
  if (!strides_ok(sxb, sxh, sxn, D, elem_size(x_dtype)))
    return set_error(QFA_EINVAL, "quant: x strides must be positive multiples of 16 bytes, token stride >= D");
  if (scb <= 0 || sch <= 0 || scn < D || scb % 8 != 0 || sch % 8 != 0 || scn % 8 != 0)
    return set_error(QFA_EINVAL, "quant: codes strides must be positive multiples of 8 bytes, token stride >= D");
  return launch_quant(x, x_dtype, codes, scale_f32, scale_lp, scale_lp_dtype, zp, rowsum, B, H, N, D, sxb, sxh, sxn,
                      scb, sch, scn, (hipStream_t)stream);
}

int qfa_quant_per_token_pair(const void *x0, const void *x1, int x_dtype, int8_t *codes0, int8_t *codes1,
                             float *scale0, float *scale1, int8_t *zp0, int8_t *zp1, int32_t *rowsum0, int32_t *rowsum1,
                             int64_t B, int64_t H, int64_t N0, int64_t N1, int D, int64_t sx0b, int64_t sx0h,
                             int64_t sx0n, int64_t sx1b, int64_t sx1h, int64_t sx1n, int64_t sc0b, int64_t sc0h,
                             int64_t sc0n, int64_t sc1b, int64_t sc1h, int64_t sc1n, void *stream) {
  const void *const x[2] = {x0, x1};
  int8_t *const codes[2] = {codes0, codes1};
  float *const scale[2] = {scale0, scale1};
  int8_t *const zp[2] = {zp0, zp1};
  int32_t *const rowsum[2] = {rowsum0, rowsum1};
  const int64_t N[2] = {N0, N1};
  const int64_t sx[2][3] = {{sx0b, sx0h, sx0n}, {sx1b, sx1h, sx1n}}, sc[2][3] = {{sc0b, sc0h, sc0n}, {sc1b, sc1h, sc1n}};
  if (!is_float_dtype(x_dtype)) return set_error(QFA_EINVAL, "quant_pair: x_dtype %d is not QFA_F32/F16/BF16", x_dtype);
  if (B <= 0 || H <= 0 || N0 <= 0 || N1 <= 0) return set_error(QFA_EINVAL, "quant_pair: B, H, N0, N1 must be positive");
  if (D < 8 || D > 256 || D % 8 != 0)
    return set_error(QFA_EUNSUPPORTED, "quant_pair: head_dim %d is not a multiple of 8 between 8 and 256", D);
  for (int i = 0; i < 2; ++i) {
    if (!x[i] || !codes[i] || !scale[i] || !zp[i]) return set_error(QFA_EINVAL, "quant_pair: null x/codes/scale/zp pointer");
    if (!aligned16(x[i]) || !aligned8(codes[i])) return set_error(QFA_EINVAL, "quant_pair: x must be 16-byte, codes 8-byte aligned");
    if (!strides_ok(sx[i][0], sx[i][1], sx[i][2], D, elem_size(x_dtype)))
      return set_error(QFA_EINVAL, "quant_pair: x strides must be positive multiples of 16 bytes, token stride >= D");
    if (sc[i][0] <= 0 || sc[i][1] <= 0 || sc[i][2] < D || sc[i][0] % 8 != 0 || sc[i][1] % 8 != 0 || sc[i][2] % 8 != 0)
      return set_error(QFA_EINVAL, "quant_pair: codes strides must be positive multiples of 8 bytes, token stride >= D");
  }
  return launch_quant_pair(x, x_dtype, codes, scale, zp, rowsum, B, H, N, D, sx, sc, (hipStream_t)stream);
}

int qfa_dequant_per_token(const int8_t *codes, const void *scale, int scale_dtype, const int8_t *zp, void *out,
                          int out_dtype, int64_t B, int64_t H, int64_t N, int D, int64_t scb, int64_t sch,
                          int64_t scn, int64_t sob, int64_t soh, int64_t son, void *stream) {
  if (!codes || !scale || !zp || !out) return set_error(QFA_EINVAL, "dequant: null pointer");
  if (!is_float_dtype(scale_dtype) || !is_float_dtype(out_dtype))
    return set_error(QFA_EINVAL, "dequant: bad scale_dtype/out_dtype");
  if (B <= 0 || H <= 0 || N <= 0) return set_error(QFA_EINVAL, "dequant: B, H, N must be positive");
  if (D < 8 || D > 256 || D % 8 != 0)
    return set_error(QFA_EUNSUPPORTED, "dequant: head_dim %d is not a multiple of 8 between 8 and 256", D);
  if (!aligned8(codes) || !aligned16(out)) return set_error(QFA_EINVAL, "dequant: codes must be 8-byte, out 16-byte aligned");
  if (scb <= 0 || sch <= 0 || scn < D || scb % 8 != 0 || sch % 8 != 0 || scn % 8 != 0 ||
      !strides_ok(sob, soh, son, D, elem_size(out_dtype)))
    return set_error(QFA_EINVAL, "dequant: strides must be positive, token stride >= D, multiples of 8 bytes (codes) and 16 bytes (out)");
  return launch_dequant(codes, scale, scale_dtype, zp, out, out_dtype, B, H, N, D, scb, sch, scn, sob, soh, son,
                        (hipStream_t)stream);
}

int qfa_code_rowsum(const int8_t *codes, int32_t *rowsum, int64_t B, int64_t H, int64_t N, int D, int64_t scb,
                    int64_t sch, int64_t scn, void *stream) {
  if (!codes || !rowsum) return set_error(QFA_EINVAL, "code_rowsum: null pointer");
  if (B <= 0 || H <= 0 || N <= 0) return set_error(QFA_EINVAL, "code_rowsum: B, H, N must be positive");
  if (D < 8 || D > 256 || D % 8 != 0)
    return set_error(QFA_EUNSUPPORTED, "code_rowsum: head_dim %d is not a multiple of 8 between 8 and 256", D);
  if (!aligned8(codes)) return set_error(QFA_EINVAL, "code_rowsum: codes must be 8-byte aligned");
  if (scb <= 0 || sch <= 0 || scn < D || scb % 8 != 0 || sch % 8 != 0 || scn % 8 != 0)
    return set_error(QFA_EINVAL, "code_rowsum: strides must be positive multiples of 8 bytes, token stride >= D");
  return launch_rowsum(codes, rowsum, B, H, N, D, scb, sch, scn, (hipStream_t)stream);
}

static int check_attn_common(const char *who, const AttnArgs &a) {
  if (!a.qc || !a.sq || !a.zq || !a.rq || !a.kc || !a.sk || !a.zk || !a.rk || !a.v || !a.o || !a.lse)
    return set_error(QFA_EINVAL, "%s: null pointer argument", who);
  if (a.io_dtype != QFA_BF16 && a.io_dtype != QFA_F16)
    return set_error(QFA_EINVAL, "%s: io_dtype must be QFA_BF16 or QFA_F16", who);
  if (a.B <= 0 || a.H <= 0 || a.Nq <= 0 || a.Nk <= 0) return set_error(QFA_EINVAL, "%s: B, H, Nq, Nk must be positive", who);
  // the kernels form byte offsets into the per-token vectors (4 bytes per token) in 31 bits
  if (a.Nq > kMaxTokens || a.Nk > kMaxTokens)
    return set_error(QFA_EUNSUPPORTED, "%s: sequences of more than 2^28 tokens are not supported", who);
  if (a.D != 64 && a.D != 128 && a.D != 256)
    return set_error(QFA_EUNSUPPORTED, "%s: head_dim %d not in {64, 128, 256}", who, a.D);
  if (!(a.sm_scale > 0.0f) || !(a.sm_scale < 3.0e38f))
    return set_error(QFA_EINVAL, "%s: sm_scale must be a positive finite number", who);
  if (a.causal && a.Nq > a.Nk)
    return set_error(QFA_EUNSUPPORTED, "%s: causal needs Nq <= Nk (the mask is aligned to the last key)", who);
  if (!aligned16(a.qc) || !aligned16(a.kc) || !aligned16(a.v) || !aligned16(a.o))
    return set_error(QFA_EINVAL, "%s: qc, kc, v, o must be 16-byte aligned", who);
  if (!strides_ok(a.sqb, a.sqh, a.sqn, a.D, 1) || !strides_ok(a.skb, a.skh, a.skn, a.D, 1) ||
      !strides_ok(a.svb, a.svh, a.svn, a.D, 2) || !strides_ok(a.sob, a.soh, a.son, a.D, 2))
    return set_error(QFA_EINVAL, "%s: strides must be positive multiples of 16 bytes, token stride >= D", who);
  // offsets inside a 64-token tile are formed in 31 bits
  if (a.skn >= (1 << 23) || a.svn >= (1 << 23) || a.sqn >= (1 << 23))
    return set_error(QFA_EUNSUPPORTED, "%s: token strides of 2^23 elements or more are not supported", who);
  return 0;
}

int qfa_attn_fwd(const int8_t *qc, const float *sq, const int8_t *zq, const int32_t *rq, const int8_t *kc,
                 const float *sk, const int8_t *zk, const int32_t *rk, const void *v, void *o, float *lse,
                 int io_dtype, int64_t B, int64_t H, int64_t Nq, int64_t Nk, int D, int64_t sqb, int64_t sqh,
                 int64_t sqn, int64_t skb, int64_t skh, int64_t skn, int64_t svb, int64_t svh, int64_t svn,
                 int64_t sob, int64_t soh, int64_t son, float sm_scale, int causal, void *stream) {
  AttnArgs a;
  memset(&a, 0, sizeof(a));
  a.qc = qc; a.sq = sq; a.zq = zq; a.rq = rq; a.kc = kc; a.sk = sk; a.zk = zk; a.rk = rk;
  a.v = v; a.o = o; a.lse = lse; a.io_dtype = io_dtype;
  a.B = B; a.H = H; a.Nq = Nq; a.Nk = Nk; a.D = D;
  a.sqb = sqb; a.sqh = sqh; a.sqn = sqn; a.skb = skb; a.skh = skh; a.skn = skn;
  a.svb = svb; a.svh = svh; a.svn = svn; a.sob = sob; a.soh = soh; a.son = son;
  a.sm_scale = sm_scale; a.causal = causal;
  if (int e = check_attn_common("attn_fwd", a)) return e;
  return launch_fwd(a, (hipStream_t)stream);
}

static int check_shared_kv(const char *who, const SkvAttnArgs &a) {
  if (!a.q || !a.codes || !a.scale || !a.zp || !a.o || !a.lse) return set_error(QFA_EINVAL, "%s: null pointer argument", who);
  if (a.io_dtype != QFA_BF16 && a.io_dtype != QFA_F16)
    return set_error(QFA_EINVAL, "%s: io_dtype must be QFA_BF16 or QFA_F16", who);
  if (a.scale_dtype != QFA_F32 && a.scale_dtype != a.io_dtype)
    return set_error(QFA_EINVAL, "%s: scale_dtype must be QFA_F32 or equal to io_dtype", who);
  if (a.B <= 0 || a.H <= 0 || a.Nq <= 0 || a.Nk <= 0) return set_error(QFA_EINVAL, "%s: B, H, Nq, Nk must be positive", who);
  // the kernels form byte offsets into the per-token vectors (4 bytes per token) in 31 bits
  if (a.Nq > kMaxTokens || a.Nk > kMaxTokens)
    return set_error(QFA_EUNSUPPORTED, "%s: sequences of more than 2^28 tokens are not supported", who);
  if (a.D != 64 && a.D != 128 && a.D != 256)
    return set_error(QFA_EUNSUPPORTED, "%s: head_dim %d not in {64, 128, 256}", who, a.D);
  if (!(a.sm_scale > 0.0f) || !(a.sm_scale < 3.0e38f))
    return set_error(QFA_EINVAL, "%s: sm_scale must be a positive finite number", who);
  if (!aligned16(a.q) || !aligned16(a.codes) || !aligned16(a.o))
    return set_error(QFA_EINVAL, "%s: q, codes, o must be 16-byte aligned", who);
  if (!strides_ok(a.sqb, a.sqh, a.sqn, a.D, 2) || !strides_ok(a.scb, a.sch, a.scn, a.D, 1) ||
      !strides_ok(a.sob, a.soh, a.son, a.D, 2))
    return set_error(QFA_EINVAL, "%s: strides must be positive multiples of 16 bytes, token stride >= D", who);
  if (a.scn >= (1 << 23)) return set_error(QFA_EUNSUPPORTED, "%s: token strides of 2^23 elements or more are not supported", who);
  return 0;
}

int64_t qfa_attn_fwd_shared_kv_workspace_bytes(int64_t B, int64_t H, int64_t Nq, int64_t Nk, int D) {
  if (B <= 0 || H <= 0 || Nq <= 0 || Nk <= 0 || (D != 64 && D != 128 && D != 256)) return 0;
  return skv_fwd_workspace_bytes(B, H, Nq, Nk, D);
}

int qfa_attn_fwd_shared_kv(const void *q, const int8_t *codes, const void *scale, int scale_dtype, const int8_t *zp,
                           void *o, float *lse, int io_dtype, int64_t B, int64_t H, int64_t Nq, int64_t Nk, int D,
                           int64_t sqb, int64_t sqh, int64_t sqn, int64_t scb, int64_t sch, int64_t scn, int64_t sob,
                           int64_t soh, int64_t son, float sm_scale, void *workspace, int64_t workspace_bytes,
                           void *stream) {
  SkvAttnArgs a;
  memset(&a, 0, sizeof(a));
  a.q = q; a.codes = codes; a.scale = scale; a.zp = zp; a.o = o; a.lse = lse;
  a.B = B; a.H = H; a.Nq = Nq; a.Nk = Nk; a.D = D; a.io_dtype = io_dtype; a.scale_dtype = scale_dtype;
  a.sqb = sqb; a.sqh = sqh; a.sqn = sqn; a.scb = scb; a.sch = sch; a.scn = scn; a.sob = sob; a.soh = soh; a.son = son;
  a.sm_scale = sm_scale;
  if (int e = check_shared_kv("attn_fwd_shared_kv", a)) return e;
  if (workspace) {
    const int64_t need = skv_fwd_workspace_bytes(B, H, Nq, Nk, D);
    if (!aligned16(workspace) || workspace_bytes < need)
      return set_error(QFA_EINVAL, "attn_fwd_shared_kv: workspace must be 16-byte aligned and hold %lld bytes "
                       "(qfa_attn_fwd_shared_kv_workspace_bytes), got %lld", (long long)need, (long long)workspace_bytes);
    a.workspace = need > 0 ? workspace : nullptr;
  }
  return launch_skv_fwd(a, (hipStream_t)stream);
}

int qfa_attn_fwd_shared_kv_static(const void *q, const int8_t *codes, const void *scale, int scale_dtype,
                                  const int8_t *zp, void *o, float *lse, int io_dtype, int64_t B, int64_t H, int64_t Nq,
                                  int64_t Nk, int D, int64_t sqb, int64_t sqh, int64_t sqn, int64_t scb, int64_t sch,
                                  int64_t scn, int64_t sob, int64_t soh, int64_t son, float sm_scale, void *stream) {
  SkvAttnArgs a;
  memset(&a, 0, sizeof(a));
  a.q = q; a.codes = codes; a.scale = scale; a.zp = zp; a.o = o; a.lse = lse;
  a.B = B; a.H = H; a.Nq = Nq; a.Nk = Nk; a.D = D; a.io_dtype = io_dtype; a.scale_dtype = scale_dtype;
  a.sqb = sqb; a.sqh = sqh; a.sqn = sqn; a.scb = scb; a.sch = sch; a.scn = scn; a.sob = sob; a.soh = soh; a.son = son;
  a.sm_scale = sm_scale;
  if (int e = check_shared_kv("attn_fwd_shared_kv_static", a)) return e;
  return launch_skv_fwd_static(a, (hipStream_t)stream);
}

int qfa_attn_bwd_shared_kv(const void *q, const int8_t *codes, const void *scale, int scale_dtype, const int8_t *zp,
                           const void *o, const void *dout, const float *lse, void *dq, void *dkv, int io_dtype,
                           int grad_dtype, const float *grad_scale,
                           int64_t B, int64_t H, int64_t Nq, int64_t Nk, int D, int64_t sqb, int64_t sqh, int64_t sqn,
                           int64_t scb, int64_t sch, int64_t scn, int64_t sob, int64_t soh, int64_t son, int64_t sdob,
                           int64_t sdoh, int64_t sdon, int64_t sdqb, int64_t sdqh, int64_t sdqn, int64_t sdkb,
                           int64_t sdkh, int64_t sdkn, float sm_scale, void *stream) {
  const char *who = "attn_bwd_shared_kv";
  SkvAttnArgs a;
  memset(&a, 0, sizeof(a));
  a.q = q; a.codes = codes; a.scale = scale; a.zp = zp; a.o = const_cast<void *>(o); a.lse = const_cast<float *>(lse);
  a.dout = dout; a.dq = dq; a.dkv = dkv; a.grad_dtype = grad_dtype; a.grad_scale = grad_scale;
  a.B = B; a.H = H; a.Nq = Nq; a.Nk = Nk; a.D = D; a.io_dtype = io_dtype; a.scale_dtype = scale_dtype;
  a.sqb = sqb; a.sqh = sqh; a.sqn = sqn; a.scb = scb; a.sch = sch; a.scn = scn; a.sob = sob; a.soh = soh; a.son = son;
  a.sdob = sdob; a.sdoh = sdoh; a.sdon = sdon; a.sdqb = sdqb; a.sdqh = sdqh; a.sdqn = sdqn;
  a.sdkb = sdkb; a.sdkh = sdkh; a.sdkn = sdkn;
  a.sm_scale = sm_scale;
  if (int e = check_shared_kv(who, a)) return e;
  if (!dout || !dq || !dkv) return set_error(QFA_EINVAL, "%s: null pointer argument", who);
  if (io_dtype != QFA_F16) return set_error(QFA_EUNSUPPORTED, "%s: io_dtype (q, o, dout) must be QFA_F16", who);
  if (grad_dtype != QFA_F16 && grad_dtype != QFA_BF16)
    return set_error(QFA_EINVAL, "%s: grad_dtype (dq, dkv) must be QFA_F16 or QFA_BF16", who);
  if (!aligned16(dout) || !aligned16(dq) || !aligned16(dkv))
    return set_error(QFA_EINVAL, "%s: dout, dq, dkv must be 16-byte aligned", who);
  if (!strides_ok(sdob, sdoh, sdon, D, 2) || !strides_ok(sdqb, sdqh, sdqn, D, 2) || !strides_ok(sdkb, sdkh, sdkn, D, 2))
    return set_error(QFA_EINVAL, "%s: strides must be positive multiples of 16 bytes, token stride >= D", who);
  // the row copies of the two-kernel path form offsets inside a 32-row block in 31 bits
  if (sqn >= (1 << 23) || son >= (1 << 23) || sdon >= (1 << 23))
    return set_error(QFA_EUNSUPPORTED, "%s: token strides of 2^23 elements or more are not supported", who);
  // one fused pass keeps a (batch, head)'s dQ in registers: at most 32 queries, head_dim up to 128
  // one fused pass while the per-wave accumulators fit: 32 queries up to head_dim 128, 16 at 256
  const bool one_pass = (Nq <= 32 && D <= 128) || (Nq <= 16 && D == 256);
  return one_pass ? launch_skv_bwd(a, (hipStream_t)stream) : launch_skv_bwd_long(a, (hipStream_t)stream);
}

int qfa_bench_qk_stage(const int8_t *qc, const float *sq, const int8_t *zq, const int32_t *rq, const int8_t *kc,
                       const float *sk, const int8_t *zk, const int32_t *rk, const void *v, void *o, float *lse,
                       int io_dtype, int64_t B, int64_t H, int64_t Nq, int64_t Nk, int D, int64_t sqb, int64_t sqh,
                       int64_t sqn, int64_t skb, int64_t skh, int64_t skn, int64_t svb, int64_t svh, int64_t svn,
                       int64_t sob, int64_t soh, int64_t son, float sm_scale, int causal, void *stream) {
  AttnArgs a;
  memset(&a, 0, sizeof(a));
  a.qc = qc; a.sq = sq; a.zq = zq; a.rq = rq; a.kc = kc; a.sk = sk; a.zk = zk; a.rk = rk;
  a.v = v; a.o = o; a.lse = lse; a.io_dtype = io_dtype;
  a.B = B; a.H = H; a.Nq = Nq; a.Nk = Nk; a.D = D;
  a.sqb = sqb; a.sqh = sqh; a.sqn = sqn; a.skb = skb; a.skh = skh; a.skn = skn;
  a.svb = svb; a.svh = svh; a.svn = svn; a.sob = sob; a.soh = soh; a.son = son;
  a.sm_scale = sm_scale; a.causal = causal;
  if (int e = check_attn_common("bench_qk_stage", a)) return e;
  return launch_fwd(a, (hipStream_t)stream, true);
}

int qfa_bwd_delta(const void *o, const void *dout, float *delta, int io_dtype, int64_t B, int64_t H, int64_t N,
                  int D, int64_t sob, int64_t soh, int64_t son, int64_t sdb, int64_t sdh, int64_t sdn,
                  void *stream) {
  if (!o || !dout || !delta) return set_error(QFA_EINVAL, "bwd_delta: null pointer argument");
  if (io_dtype != QFA_BF16 && io_dtype != QFA_F16) return set_error(QFA_EINVAL, "bwd_delta: io_dtype must be QFA_BF16 or QFA_F16");
  if (B <= 0 || H <= 0 || N <= 0) return set_error(QFA_EINVAL, "bwd_delta: B, H, N must be positive");
  if (D != 64 && D != 128 && D != 256) return set_error(QFA_EUNSUPPORTED, "bwd_delta: head_dim %d not in {64, 128, 256}", D);
  if (!aligned16(o) || !aligned16(dout)) return set_error(QFA_EINVAL, "bwd_delta: o and dout must be 16-byte aligned");
  if (!strides_ok(sob, soh, son, D, 2) || !strides_ok(sdb, sdh, sdn, D, 2))
    return set_error(QFA_EINVAL, "bwd_delta: strides must be positive multiples of 16 bytes, token stride >= D");
  return launch_delta(o, dout, delta, io_dtype, B, H, N, D, sob, soh, son, sdb, sdh, sdn, (hipStream_t)stream);
}

int qfa_sum_grads(const void *a, const void *b, void *out, int dtype, int64_t n, void *stream) {
  if (!a || !b || !out) return set_error(QFA_EINVAL, "sum_grads: null pointer argument");
  if (dtype != QFA_BF16 && dtype != QFA_F16) return set_error(QFA_EINVAL, "sum_grads: dtype must be QFA_BF16 or QFA_F16");
  if (n <= 0 || n % 8 != 0) return set_error(QFA_EINVAL, "sum_grads: the element count must be a positive multiple of 8");
  if (!aligned16(a) || !aligned16(b) || !aligned16(out)) return set_error(QFA_EINVAL, "sum_grads: pointers must be 16-byte aligned");
  return launch_sum16(a, b, out, dtype, n, (hipStream_t)stream);
}

int64_t qfa_dout_normalise_workspace_bytes(void) { return dout_normalise_workspace_bytes(); }

int qfa_dout_normalise(const void *dout, int dout_dtype, int64_t n, const void *kv_scale, int scale_dtype, int64_t n_scale,
                       void *workspace, void *out, float *back, void *stream) {
  if (!dout || !kv_scale || !workspace || !out || !back) return set_error(QFA_EINVAL, "dout_normalise: null pointer argument");
  if (dout_dtype != QFA_BF16 && dout_dtype != QFA_F16) return set_error(QFA_EINVAL, "dout_normalise: dout_dtype must be QFA_BF16 or QFA_F16");
  if (scale_dtype != QFA_F32 && scale_dtype != QFA_F16) return set_error(QFA_EINVAL, "dout_normalise: scale_dtype must be QFA_F32 or QFA_F16");
  if (n <= 0 || n % 8 != 0) return set_error(QFA_EINVAL, "dout_normalise: the element count must be a positive multiple of 8");
  if (n_scale <= 0) return set_error(QFA_EINVAL, "dout_normalise: n_scale must be positive");
  if (!aligned16(dout) || !aligned16(out) || !aligned16(kv_scale))
    return set_error(QFA_EINVAL, "dout_normalise: dout, kv_scale and out must be 16-byte aligned");
  return launch_dout_normalise(dout, dout_dtype, n, kv_scale, scale_dtype, n_scale, static_cast<float *>(workspace), out, back,
                               (hipStream_t)stream);
}

int64_t qfa_attn_bwd_workspace_bytes(int64_t B, int64_t H, int64_t Nq, int64_t Nk, int D) {
  if (B <= 0 || H <= 0 || Nq <= 0 || Nk <= 0 || (D != 64 && D != 128 && D != 256)) return 0;
  return bwd_workspace_bytes(B, H, Nq, Nk, D);
}

int qfa_attn_bwd(const int8_t *qc, const float *sq, const int8_t *zq, const int32_t *rq, const int8_t *kc,
                 const float *sk, const int8_t *zk, const int32_t *rk, const void *v, const void *o,
                 const void *dout, const float *lse, void *workspace, int64_t workspace_bytes, void *dq, void *dk,
                 void *dv, int io_dtype,
                 int64_t B, int64_t H, int64_t Nq, int64_t Nk, int D, int64_t sqb, int64_t sqh, int64_t sqn,
                 int64_t skb, int64_t skh, int64_t skn, int64_t svb, int64_t svh, int64_t svn, int64_t sob,
                 int64_t soh, int64_t son, int64_t sdob, int64_t sdoh, int64_t sdon, int64_t sdqb, int64_t sdqh,
                 int64_t sdqn, int64_t sdkb, int64_t sdkh, int64_t sdkn, int64_t sdvb, int64_t sdvh,
                 int64_t sdvn, float sm_scale, int causal, void *stream) {
  AttnArgs a;
  memset(&a, 0, sizeof(a));
  a.qc = qc; a.sq = sq; a.zq = zq; a.rq = rq; a.kc = kc; a.sk = sk; a.zk = zk; a.rk = rk;
  a.v = v; a.o = const_cast<void *>(o); a.lse = const_cast<float *>(lse); a.io_dtype = io_dtype;
  a.dout = dout; a.workspace = workspace; a.dq = dq; a.dk = dk; a.dv = dv;
  a.B = B; a.H = H; a.Nq = Nq; a.Nk = Nk; a.D = D;
  a.sqb = sqb; a.sqh = sqh; a.sqn = sqn; a.skb = skb; a.skh = skh; a.skn = skn;
  a.svb = svb; a.svh = svh; a.svn = svn; a.sob = sob; a.soh = soh; a.son = son;
  a.sdob = sdob; a.sdoh = sdoh; a.sdon = sdon; a.sdqb = sdqb; a.sdqh = sdqh; a.sdqn = sdqn;
  a.sdkb = sdkb; a.sdkh = sdkh; a.sdkn = sdkn; a.sdvb = sdvb; a.sdvh = sdvh; a.sdvn = sdvn;
  a.sm_scale = sm_scale; a.causal = causal;
  if (int e = check_attn_common("attn_bwd", a)) return e;
  if (!dout || !workspace || !dq || !dk || !dv) return set_error(QFA_EINVAL, "attn_bwd: null pointer argument");
  if (!aligned16(dout) || !aligned16(dq) || !aligned16(dk) || !aligned16(dv) || !aligned16(workspace))
    return set_error(QFA_EINVAL, "attn_bwd: dout, dq, dk, dv, workspace must be 16-byte aligned");
  const int64_t need = bwd_workspace_bytes(B, H, Nq, Nk, D);
  if (workspace_bytes < need)
    return set_error(QFA_EINVAL, "attn_bwd: workspace of %lld bytes is too small, need %lld (qfa_attn_bwd_workspace_bytes)",
                     (long long)workspace_bytes, (long long)need);
  if (!strides_ok(sdob, sdoh, sdon, D, 2) || !strides_ok(sdqb, sdqh, sdqn, D, 2) ||
      !strides_ok(sdkb, sdkh, sdkn, D, 2) || !strides_ok(sdvb, sdvh, sdvn, D, 2))
    return set_error(QFA_EINVAL, "attn_bwd: strides must be positive multiples of 16 bytes, token stride >= D");
  return launch_bwd(a, (hipStream_t)stream);
}

}  // extern "C"
