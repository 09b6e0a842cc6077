/*
 * qfa.h -- C ABI of libqfa.so: per-token asymmetric INT8 quantizer and INT8-QK^T
 * flash attention (forward + backward) for AMD MI355X (gfx950).
 *
 * Conventions shared by every entry point
 *   - Every pointer is a DEVICE pointer owned by the caller.  Nothing is allocated,
 *     freed or retained by the library.
 *   - Tensors are [B, H, N, D] (batch, heads, tokens, head_dim) with the last axis
 *     contiguous.  s?b / s?h / s?n are strides in ELEMENTS of the b, h and n axes.
 *   - Per-token vectors (scale, zero point, row sum, LSE, delta) are dense [B*H*N].
 *   - `stream` is a hipStream_t passed as void* (NULL = the default stream).  Work is
 *     enqueued asynchronously; the call returns as soon as the launches are queued.
 *   - Return value: 0 = success, < 0 = one of the QFA_E* argument errors (nothing was
 *     launched), > 0 = the hipError_t of a failed launch.  qfa_last_error() returns a
 *     thread-local, human readable description of the last failure on this thread.
 *   - The library keeps no mutable global state and calls from several host threads are safe; the one
 *     exception is qfa_attn_fwd_shared_kv_static, which owns a static device scratch array (see there).
 *
 * Reference interface each entry point replaces (paths in yisunlp/quant_flash_attn):
 * the reference has no FFI; the boundary is the Triton launch made by its Python operators.
 */
#ifndef QFA_H_
#define QFA_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define QFA_VERSION 100 /* major*10000 + minor*100 + patch */

/* element types of floating-point tensors */
#define QFA_F32 0
#define QFA_F16 1
#define QFA_BF16 2

/* argument errors */
#define QFA_EINVAL (-1)       /* null pointer, non-positive size, bad dtype code, misaligned pointer/stride */
#define QFA_EUNSUPPORTED (-2) /* well-formed but not implemented (head_dim, causal with Nq > Nk, ...) */

int qfa_version(void);
const char *qfa_last_error(void);

/*
 * Per-token asymmetric INT8 quantization over the last axis.
 * Replaces the launch of _asymmetric_quant_kernel made by asymmetric_quant_per_token
 * (asymmetric_quant.py:22-106 kernel, :109-149 wrapper).  For every token row x[0..D):
 *     scale = (max - min) / 255  (1.0 if that is 0);  zp = clamp(roundf(-128 - min/scale))
 *     code[d] = clamp(roundf(x[d]/scale + zp))         -- all IEEE binary32, roundf = ties away
 *   x         [B,H,N,D] of x_dtype (QFA_F32 / QFA_F16 / QFA_BF16), strides sxb,sxh,sxn
 *   codes     [B,H,N,D] int8, strides scb,sch,scn (the reference uses the input's strides)
 *   scale_f32 [B*H*N] float: the unrounded scale the codes were computed with
 *   scale_lp  nullable; [B*H*N] copy of the scale rounded to scale_lp_dtype (QFA_F16/QFA_BF16)
 *             -- the fp16 scale tensor the reference returns (asymmetric_quant.py:93,128)
 *   zp        [B*H*N] int8
 *   rowsum    nullable; [B*H*N] int32 sum of the token's codes (feeds the zero-point
 *             cross term of qfa_attn_fwd / qfa_attn_bwd; not produced by the reference)
 *   D any multiple of 8 up to 256 (the reference masks the tail of its power-of-two block the same way,
 *   asymmetric_quant.py:72-75,97-99).  x 16-byte aligned with strides that are multiples of 16 bytes; codes
 *   8-byte aligned with strides that are multiples of 8 bytes (the attention entry points want 16).
 * A token row that holds an infinity or a NaN gets unspecified codes (the formulas above send NaN through
 * roundf and the int8 conversion, in the reference as here); the other rows are not affected.
 */
int qfa_quant_per_token(const void *x, int x_dtype, int8_t *codes, float *scale_f32, void *scale_lp,
                        int scale_lp_dtype, int8_t *zp, int32_t *rowsum, int64_t B, int64_t H, int64_t N,
                        int D, int64_t sxb, int64_t sxh, int64_t sxn, int64_t scb, int64_t sch, int64_t scn,
                        void *stream);

/*
 * qfa_quant_per_token for TWO tensors of one element type and head dimension in one launch: the queries and the keys
 * of an attention call (tensor 0: [B,H,N0,D], tensor 1: [B,H,N1,D]).  Replaces the two launches of
 * _asymmetric_quant_kernel (asymmetric_quant.py:132-147) that quantizing q and k costs; same arithmetic, same
 * outputs per tensor (codes, fp32 scale, zero point, optional row sum; no 16-bit copy of the scale), one launch
 * ramp and one tail instead of two.  Strides in elements: x per tensor (b, h, n), codes per tensor (b, h, n).
 */
int qfa_quant_per_token_pair(const void *x0, const void *x1, int x_dtype, int8_t *codes0, int8_t *codes1,
                             float *scale0, float *scale1, int8_t *zp0, int8_t *zp1, int32_t *rowsum0, int32_t *rowsum1,
                             int64_t B, int64_t H, int64_t N0, int64_t N1, int D, int64_t sx0b, int64_t sx0h,
                             int64_t sx0n, int64_t sx1b, int64_t sx1h, int64_t sx1n, int64_t sc0b, int64_t sc0h,
                             int64_t sc0n, int64_t sc1b, int64_t sc1h, int64_t sc1n, void *stream);

/*
 * out = (codes - zp) * scale, per token (asymmetric_quant.py:158-160, and the in-kernel
 * dequantization quant_flash_attn.py:65).  scale_dtype is the element type of `scale`
 * (QFA_F32 / QFA_F16 / QFA_BF16); out has out_dtype and strides sob,soh,son.
 */
int qfa_dequant_per_token(const int8_t *codes, const void *scale, int scale_dtype, const int8_t *zp, void *out,
                          int out_dtype, int64_t B, int64_t H, int64_t N, int D, int64_t scb, int64_t sch,
                          int64_t scn, int64_t sob, int64_t soh, int64_t son, void *stream);

/*
 * rowsum[b,h,n] = sum_d codes[b,h,n,d] (int32, dense [B*H*N]): the side output of qfa_quant_per_token, for
 * codes that arrive already quantized.  qfa_attn_fwd / qfa_attn_bwd need it for the exact zero-point term of the
 * INT8 score product; the reference has no counterpart (its kernels dequantize K before the product,
 * quant_flash_attn.py:65).  D any multiple of 8 up to 256; codes 8-byte aligned, strides multiples of 8 bytes.
 */
int qfa_code_rowsum(const int8_t *codes, int32_t *rowsum, int64_t B, int64_t H, int64_t N, int D, int64_t scb,
                    int64_t sch, int64_t scn, void *stream);

/*
 * Attention forward on quantized Q and K:
 *     S = sm_scale * Q^ K^T,  Q^ = sq*(qc - zq),  K^ = sk*(kc - zk)   [causal: keep col <= row]
 *     O = softmax(S) V,   LSE = logsumexp(S) (natural log)
 * QK^T runs on INT8 MFMA with int32 accumulation; the zero points enter through the exact
 * integer cross term (uses the row sums rq, rk).  Softmax is fp32; P.V is bf16/fp16 MFMA.
 * Replaces the launch of _attn_fwd_kernel_quantized made by QuantFlashAttention.forward
 * (quant_flash_attn.py:22-83 kernel, :178-204 wrapper), generalised to a quantized Q,
 * separate K and V, a causal flag (rule of flash_attn_triton.py:50) and tiled queries.
 *   qc,kc  int8 [B,H,Nq|Nk,D];  sq,sk float, zq,zk int8, rq,rk int32: dense [B*H*Nq|Nk]
 *   v, o   [B,H,Nk|Nq,D] of io_dtype (QFA_BF16 or QFA_F16);  lse float [B*H*Nq]
 *   D in {64, 128, 256} (the widths compute_flops.py:94 sweeps; also for qfa_attn_bwd and qfa_bwd_delta).
 *   causal != 0: query i keeps the keys j <= i + (Nk - Nq), the mask aligned to the last key, which needs
 *   Nq <= Nk (with Nq == Nk the rule row >= col of flash_attn_triton.py:50; the reference has no other case:
 *   a block of queries at the end of a longer key sequence).  All tensors 16-byte aligned, strides
 *   multiples of 16 bytes, token strides below 2^23 elements, Nq and Nk at most 2^28
 *   (QFA_EUNSUPPORTED otherwise).
 */
int qfa_attn_fwd(const int8_t *qc, const float *sq, const int8_t *zq, const int32_t *rq, const int8_t *kc,
                 const float *sk, const int8_t *zk, const int32_t *rk, const void *v, void *o, float *lse,
                 int io_dtype, int64_t B, int64_t H, int64_t Nq, int64_t Nk, int D, int64_t sqb, int64_t sqh,
                 int64_t sqn, int64_t skb, int64_t skh, int64_t skn, int64_t svb, int64_t svh, int64_t svn,
                 int64_t sob, int64_t soh, int64_t son, float sm_scale, int causal, void *stream);

/*
 * Attention forward of the reference's own operator, for short query blocks:
 *     O = softmax(sm_scale * Q KV^T) KV,   KV = scale * (codes - zp) per token,   LSE = logsumexp
 * One quantized tensor serves as K and V and Q stays in 16-bit float, exactly as in
 * _attn_fwd_kernel_quantized (quant_flash_attn.py:22-83; launched from :178-204 with one program
 * per (batch, head) and the whole query block in it).  The kernel streams the INT8 codes once per
 * block of 32 queries and feeds them to the 16-bit MFMAs as exact binary16 integers, so it is bound
 * by reading the codes; it is the right entry point while Nq is small against Nk (decoding, the
 * reference's benchmark shape Nq=16, Nk=3000 of compute_flops.py:96).  For long query blocks
 * qfa_attn_fwd (quantized Q, INT8 MFMA) is the faster path.
 *   q, o   [B,H,Nq,D] of io_dtype (QFA_F16 or QFA_BF16; bf16 queries enter the products rounded
 *          to binary16), strides sq?, so?;  lse float [B*H*Nq]
 *   codes  int8 [B,H,Nk,D], strides sc?;  zp int8 [B*H*Nk]
 *   scale  [B*H*Nk] of scale_dtype: QFA_F32, or the same 16-bit type as io_dtype
 *   D in {64, 128, 256}.  q, codes, o 16-byte aligned, strides multiples of 16 bytes, scn < 2^23.
 *   The codes' binary16 offset (1152) is removed through the sum of a query's D elements: |sum| must
 *   stay below 2^21, and the scores carry an absolute error of a few fp32 ulp of 1152 * |sum| code
 *   units (nothing for |q| of order 10; about a percent of a score once every element is near 500).
 *   Binary16 ranges, not checked: the queries enter the products as binary16 (a bf16 query above 65504 in
 *   magnitude becomes an infinity and the row NaN), and the probabilities are multiplied by the key scale
 *   before they are packed to binary16 (p * scale below 65504: scales up to about 4e3).  Nq, Nk at most 2^28.
 *   workspace  nullable.  With few (batch, head) pairs one workgroup per 16 queries leaves most of the
 *              chip idle (the reference launches one program per (batch, head)); given a caller-owned
 *              scratch of qfa_attn_fwd_shared_kv_workspace_bytes(...) bytes (16-byte aligned; the
 *              function returns 0 when no split pays) the keys of a query block are split over several
 *              workgroups and a second small kernel merges their partial (O, m, l).  NULL: never split.
 */
int64_t qfa_attn_fwd_shared_kv_workspace_bytes(int64_t B, int64_t H, int64_t Nq, int64_t Nk, int D);

int qfa_attn_fwd_shared_kv(const void *q, const int8_t *codes, const void *scale, int scale_dtype, const int8_t *zp,
                           void *o, float *lse, int io_dtype, int64_t B, int64_t H, int64_t Nq, int64_t Nk, int D,
                           int64_t sqb, int64_t sqh, int64_t sqn, int64_t scb, int64_t sch, int64_t scn, int64_t sob,
                           int64_t soh, int64_t son, float sm_scale, void *workspace, int64_t workspace_bytes,
                           void *stream);

/*
 * qfa_attn_fwd_shared_kv for callers that cannot allocate device memory (code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc): no counterpart in the reference.  Same
 * computation, same kernels and bit-identical results as qfa_attn_fwd_shared_kv given a workspace, but the
 * partial results of a split over keys live in a static device array of QFA_STATIC_SCRATCH_BYTES inside the
 * library (every GPU the library runs on holds its own copy until the process ends).  The call allocates
 * and frees nothing; its first use on a device looks up that array's device address (hipGetSymbolAddress)
 * and keeps it.  A shape whose split needs more than QFA_STATIC_SCRATCH_BYTES
 * (qfa_attn_fwd_shared_kv_workspace_bytes tells) is rejected with QFA_EUNSUPPORTED before anything is
 * launched.  All calls on one GPU share the one array: calls that overlap in time on the same GPU (two
 * streams, two threads) race on it -- serialise them, or use the workspace form.  Nothing in the array has
 * to be cleared between calls (every partial result is written before it is read).
 */
#define QFA_STATIC_SCRATCH_BYTES (16 << 20)
int qfa_attn_fwd_shared_kv_static(const void *q, const int8_t *codes, const void *scale, int scale_dtype,
                                  const int8_t *zp, void *o, float *lse, int io_dtype, int64_t B, int64_t H, int64_t Nq,
                                  int64_t Nk, int D, int64_t sqb, int64_t sqh, int64_t sqn, int64_t scb, int64_t sch,
                                  int64_t scn, int64_t sob, int64_t soh, int64_t son, float sm_scale, void *stream);

/*
 * Backward of qfa_attn_fwd_shared_kv, fp16:
 *     P = exp(sm_scale Q KV^T - LSE),  dP = dO KV^T,  dS = sm_scale P o (dP - delta),  delta = rowsum(O o dO)
 *     dQ = dS KV,    dKV = P^T dO + dS^T Q
 * Replaces the launches made by QuantFlashAttention.backward (quant_flash_attn.py:207-237):
 * _bwd_preprocess_kernel (:87-101; delta is computed inside) and _attn_bwd_kernel_quantized
 * (:104-166), which also stores the single gradient dKV = dV + dK (:161).  Up to 32 queries per
 * (batch, head) run in one fused pass (one workgroup per (batch, head) streams the codes once and
 * writes each dKV row once); longer query blocks run a dQ kernel (one workgroup per 16 queries) and
 * a dKV kernel (one workgroup per 128 keys walking over the queries).
 *   q, o, dout [B,H,Nq,D] fp16 (io_dtype must be QFA_F16: the kernels compute in binary16), strides as given;
 *   dq [B,H,Nq,D], dkv [B,H,Nk,D] of grad_dtype (QFA_F16 or QFA_BF16);
 *   grad_scale  nullable DEVICE pointer to one float that multiplies dq and dkv before they are rounded.
 *               dQ and dKV are linear in dO: a caller whose dO does not fit binary16 (bf16 training) hands
 *               over dO * 2^k and *grad_scale = 2^-k without a host synchronisation;
 *   codes, scale, scale_dtype, zp, lse as in the forward.  D in {64, 128, 256} (256: one pass up to 16 queries).
 *   The sums of a query's and of a dO row's D elements must stay inside binary16 range.
 *   Range of dout: the kernels do not multiply by dO itself but by  ds = sm_scale * p * (dP - delta)  and by
 *   ds * scale_j,  both packed to binary16 (the reference rounds ds to fp16 as well, quant_flash_attn.py:159).
 *   With |dO| well below one these operands fall into binary16's subnormals and the gradients lose precision
 *   (a few percent at |dO| ~ 2^-6 for unit-variance K = V, everything at 2^-14).  dQ and dKV are linear in dO:
 *   hand over dO * 2^k with the largest |dO| * 2^k * max(scale) near 8 (and |dO| * 2^k below 2^14) and
 *   *grad_scale = 2^-k, as the Python entry point does on the device.
 */
int qfa_attn_bwd_shared_kv(const void *q, const int8_t *codes, const void *scale, int scale_dtype, const int8_t *zp,
                           const void *o, const void *dout, const float *lse, void *dq, void *dkv, int io_dtype,
                           int grad_dtype, const float *grad_scale,
                           int64_t B, int64_t H, int64_t Nq, int64_t Nk, int D, int64_t sqb, int64_t sqh, int64_t sqn,
                           int64_t scb, int64_t sch, int64_t scn, int64_t sob, int64_t soh, int64_t son, int64_t sdob,
                           int64_t sdoh, int64_t sdon, int64_t sdqb, int64_t sdqh, int64_t sdqn, int64_t sdkb,
                           int64_t sdkh, int64_t sdkn, float sm_scale, void *stream);

/*
 * Measurement hook, same arguments as qfa_attn_fwd: runs the forward kernel with the exponentials
 * and the P.V product compiled out (same K/V/Q loads, INT8 QK^T MFMAs, zero-point correction, key
 * scaling and running row maximum).  O is left untouched; lse receives the scaled row maxima.
 * Used by bench.py to time the QK^T stage alone against the INT8 MFMA peak; no counterpart in
 * the reference (its compute_flops.py:89-151 times whole kernels only).
 */
int qfa_bench_qk_stage(const int8_t *qc, const float *sq, const int8_t *zq, const int32_t *rq, const int8_t *kc,
                       const float *sk, const int8_t *zk, const int32_t *rk, const void *v, void *o, float *lse,
                       int io_dtype, int64_t B, int64_t H, int64_t Nq, int64_t Nk, int D, int64_t sqb, int64_t sqh,
                       int64_t sqn, int64_t skb, int64_t skh, int64_t skn, int64_t svb, int64_t svh, int64_t svn,
                       int64_t sob, int64_t soh, int64_t son, float sm_scale, int causal, void *stream);

/*
 * out = dout * 2^k as binary16 and back[0] = 2^-k, for a dense 16-bit dout of n elements (n a multiple of 8) and the
 * n_scale per-token scales of the shared K = V tensor (QFA_F32 or QFA_F16); dout, kv_scale and out 16-byte aligned.
 * qfa_attn_bwd_shared_kv computes in binary16 and forms sm_scale * p * (dP - delta) * scale_j as a matrix operand;
 * dQ and dKV are linear in dO, so callers hand it this scaled dO and pass `back` as grad_scale.  k is the largest
 * integer with  max|dout| * 2^k * max|scale| <= 8  and  max|dout| * 2^k <= 2^14  (within [-100, 100]), found on the
 * device: two launches, no synchronisation, no atomics.  workspace: qfa_dout_normalise_workspace_bytes() bytes of
 * device scratch (4-byte aligned), contents irrelevant before and after.  No counterpart in the reference, whose
 * Triton kernel runs the same products in fp16 on dO as it comes (quant_flash_attn.py:130-161) and loses small
 * gradients to fp16's subnormals.
 */
int64_t qfa_dout_normalise_workspace_bytes(void);
int qfa_dout_normalise(const void *dout, int dout_dtype, int64_t n, const void *kv_scale, int scale_dtype, int64_t n_scale,
                       void *workspace, void *out, float *back, void *stream);

/*
 * out[i] = a[i] + b[i] for two dense 16-bit tensors of n elements (n a multiple of 8, pointers 16-byte aligned;
 * out may be a or b), added in fp32 and rounded once.  The merged gradient dkv = dv + dk that _bwd_kernel_quantized
 * stores for its shared K = V tensor (quant_flash_attn.py:161), for callers that obtained dK and dV from
 * qfa_attn_bwd (query blocks too long for qfa_attn_bwd_shared_kv).
 */
int qfa_sum_grads(const void *a, const void *b, void *out, int dtype, int64_t n, void *stream);

/*
 * delta[b,h,n] = sum_d O[b,h,n,d] * dO[b,h,n,d], accumulated in fp32.
 * Replaces the launch of _bwd_preprocess_kernel (quant_flash_attn.py:87-101, :217-223).
 * qfa_attn_bwd computes delta inside its own staging pass; this entry point is for callers that
 * only need the preprocess step.
 */
int qfa_bwd_delta(const void *o, const void *dout, float *delta, int io_dtype, int64_t B, int64_t H, int64_t N,
                  int D, int64_t sob, int64_t soh, int64_t son, int64_t sdb, int64_t sdh, int64_t sdn,
                  void *stream);

/*
 * Attention backward.  Recomputes P = exp(S - LSE) with the same INT8 score path as the
 * forward, then   dV = P^T dO,  dP = dO V^T,  dS = P o (dP - delta),
 *                 dQ = sm_scale dS K^,  dK = sm_scale dS^T Q^      (gradients w.r.t. Q^, K^).
 * Replaces the launches made by QuantFlashAttention.backward (quant_flash_attn.py:104-166
 * kernel, :207-237 wrapper); the reference's single dKV tensor is dK + dV (:161).
 *   workspace  caller-owned scratch of at least qfa_attn_bwd_workspace_bytes(B,H,Nq,Nk,D) bytes,
 *              16-byte aligned, overwritten: two staging passes fill it with delta = rowsum(O o dO),
 *              the transposed 16-bit tiles Q^^T, K^^T (the dequantized Q and K rounded to
 *              io_dtype, the operands of the dK and dQ products) and per-token constants, once
 *              per call, so that the two MFMA kernels stream ready-made tiles.  The scores S, and
 *              with them P, come from the INT8 codes exactly as in the forward.
 *   dq [B,H,Nq,D], dk, dv [B,H,Nk,D] of io_dtype, strides as given.
 */
int64_t qfa_attn_bwd_workspace_bytes(int64_t B, int64_t H, int64_t Nq, int64_t Nk, int D);

int qfa_attn_bwd(const int8_t *qc, const float *sq, const int8_t *zq, const int32_t *rq, const int8_t *kc,
                 const float *sk, const int8_t *zk, const int32_t *rk, const void *v, const void *o,
                 const void *dout, const float *lse, void *workspace, int64_t workspace_bytes, void *dq, void *dk,
                 void *dv, int io_dtype,
                 int64_t B, int64_t H, int64_t Nq, int64_t Nk, int D, int64_t sqb, int64_t sqh, int64_t sqn,
                 int64_t skb, int64_t skh, int64_t skn, int64_t svb, int64_t svh, int64_t svn, int64_t sob,
                 int64_t soh, int64_t son, int64_t sdob, int64_t sdoh, int64_t sdon, int64_t sdqb, int64_t sdqh,
                 int64_t sdqn, int64_t sdkb, int64_t sdkh, int64_t sdkn, int64_t sdvb, int64_t sdvh,
                 int64_t sdvn, float sm_scale, int causal, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* QFA_H_ */
