// Backward kernels for gfx950: two staging passes, then two MFMA kernels that recompute
// P = exp(S - LSE) from the INT8 codes exactly as the forward does.
//
//   prep_q       per 64-query tile: delta = rowsum(O o dO) in fp32; Qz^T = ((Qc - zq) * sq)^T as a
//                16-bit tile [d][query] in the key order the MFMA layouts want; per-query constants
//   prep_k       per 64-key tile: Kz^T = ((Kc - zk) * sk)^T likewise; per-key constants
//                (both write into the caller's workspace; every tile is converted and transposed
//                once instead of once per consuming workgroup)
//   dq kernel    one workgroup = 128 queries (32 per wave), loops over 64-key tiles.
//                S^T = Kc.Qc^T (INT8 MFMA), dP^T = V.dO^T, dS^T = P^T o (dP^T - delta),
//                dQ^T += Kz^T.dS^T                with Kz = (Kc - zk) * sk, the dequantized K rounded to 16 bits
//   dkdv kernel  one workgroup = 128 keys (32 per wave), loops over 64-query tiles.
//                S = Qc.Kc^T (INT8 MFMA), dP = dO.V^T, dV^T += dO^T.P (dO^T read out of the dO tile by
//                the transposing LDS reads),
//                dK^T += Qz^T.dS                  with Qz = (Qc - zq) * sq, the dequantized Q rounded to 16 bits
// In both, the wave's own operand (queries resp. keys) stays in registers as the MFMA B operand
// for the whole loop and the streamed operand comes from LDS as the A operand.  The 32x32
// accumulator layout then leaves P / dS in registers exactly in the B-operand layout of the next
// product; the transposed LDS tiles (Kz^T, Qz^T) are written in the matching permuted order.
// dQ is produced by its own kernel instead of atomics, so results are deterministic.
// The scales of the streamed operand are folded into its transposed 16-bit tile (Kz^T, Qz^T) by the staging
// pass, so dS is used as it comes: the tiles then hold the dequantized K and Q rounded to the 16-bit type, the
// operands an unquantized backward would use.  The dK/dV kernel is bound by LDS reads (48 KB per 32x32 block
// and wave pair, 16 KB of it per-query constants), and the fold takes one constant vector out of its loop.
#include <type_traits>

#include "qfa_device.h"
#include "qfa_host.h"

namespace qfa {

// ------------------------------------------------------------------------------------------ delta
struct DeltaArgs {
  const void *o; const void *dout; float *delta;
  int64_t N, H;
  int64_t sob, soh, son, sdb, sdh, sdn;
  int chunks_per_bh;
};

template <typename T, int D> __global__ __launch_bounds__(256) void delta_kernel(DeltaArgs a) {
  constexpr int LPT = D / 8;
  constexpr int TPP = 256 / LPT;
  const int tid = threadIdx.x, sub = tid % LPT;
  const int64_t bh = blockIdx.x / a.chunks_per_bh, chunk = blockIdx.x % a.chunks_per_bh;
  const int64_t b = bh / a.H, h = bh % a.H;
  const int64_t n = chunk * (int64_t)TPP + tid / LPT;
  const int64_t nn = n < a.N ? n : a.N - 1;
  const u32x4 ow = *reinterpret_cast<const u32x4 *>(reinterpret_cast<const T *>(a.o) + b * a.sob + h * a.soh +
                                                     nn * a.son + sub * 8);
  const u32x4 gw = *reinterpret_cast<const u32x4 *>(reinterpret_cast<const T *>(a.dout) + b * a.sdb + h * a.sdh +
                                                     nn * a.sdn + sub * 8);
  float s = 0.f;
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    s = __builtin_fmaf(lo_to_f32<T>(ow[e]), lo_to_f32<T>(gw[e]), s);
    s = __builtin_fmaf(hi_to_f32<T>(ow[e]), hi_to_f32<T>(gw[e]), s);
  }
  s += dpp_f<0xB1>(s);
  s += dpp_f<0x4E>(s);
  s += dpp_f<0x141>(s);
  if (LPT >= 16) s += dpp_f<0x140>(s);
  if (LPT >= 32) s += __shfl_xor(s, 16);
  if (n < a.N && sub == 0) a.delta[bh * a.N + n] = s;
}

// out = a + b for two 16-bit tensors of the same dense shape, added in fp32 and rounded once: dKV = dK + dV of the
// shared K = V contract (quant_flash_attn.py:161) when the two gradients come from the INT8-score kernels.
template <typename T> __global__ __launch_bounds__(256) void sum16_kernel(const T *a, const T *b, T *out, int64_t n8) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= n8) return;
  const u32x4 x = reinterpret_cast<const u32x4 *>(a)[i], y = reinterpret_cast<const u32x4 *>(b)[i];
  u32x4 r;
#pragma unroll
  for (int e = 0; e < 4; ++e)
    r[e] = pack2<T>(lo_to_f32<T>(x[e]) + lo_to_f32<T>(y[e]), hi_to_f32<T>(x[e]) + hi_to_f32<T>(y[e]));
  reinterpret_cast<u32x4 *>(out)[i] = r;
}
int launch_sum16(const void *a, const void *b, void *out, int dtype, int64_t n, hipStream_t st) {
  const int64_t n8 = n / 8, blocks = (n8 + 255) / 256;
  if (blocks > 0x7fffffffLL) return set_error(QFA_EUNSUPPORTED, "sum_grads: too many elements for one launch");
  if (dtype == QFA_BF16)
    sum16_kernel<__bf16><<<dim3((unsigned)blocks), dim3(256), 0, st>>>((const __bf16 *)a, (const __bf16 *)b, (__bf16 *)out, n8);
  else
    sum16_kernel<_Float16><<<dim3((unsigned)blocks), dim3(256), 0, st>>>((const _Float16 *)a, (const _Float16 *)b, (_Float16 *)out, n8);
  return check_launch("qfa_sum_grads");
}

int launch_delta(const void *o, const void *dout, float *delta, int io_dtype, int64_t B, int64_t H, int64_t N, int D,
                 int64_t sob, int64_t soh, int64_t son, int64_t sdb, int64_t sdh, int64_t sdn, hipStream_t st) {
  DeltaArgs a;
  a.o = o; a.dout = dout; a.delta = delta; a.N = N; a.H = H;
  a.sob = sob; a.soh = soh; a.son = son; a.sdb = sdb; a.sdh = sdh; a.sdn = sdn;
  const int tpp = 256 / (D / 8);
  const int64_t chunks = (N + tpp - 1) / tpp;
  if (chunks * B * H > 0x7fffffffLL) return set_error(QFA_EUNSUPPORTED, "bwd_delta: too many tokens for one launch");
  a.chunks_per_bh = (int)chunks;
  const dim3 grid((unsigned)(chunks * B * H)), block(256);
  if (io_dtype == QFA_BF16) {
    if (D == 256) delta_kernel<__bf16, 256><<<grid, block, 0, st>>>(a);
    else if (D == 128) delta_kernel<__bf16, 128><<<grid, block, 0, st>>>(a);
    else delta_kernel<__bf16, 64><<<grid, block, 0, st>>>(a);
  } else {
    if (D == 256) delta_kernel<_Float16, 256><<<grid, block, 0, st>>>(a);
    else if (D == 128) delta_kernel<_Float16, 128><<<grid, block, 0, st>>>(a);
    else delta_kernel<_Float16, 64><<<grid, block, 0, st>>>(a);
  }
  return check_launch("qfa_bwd_delta");
}

// ------------------------------------------------------------------------------------------ shared
// Rows streamed per step: 64, or 32 at head_dim 256, where a 64-row step of codes, 16-bit rows and transposed tile
// (80 KB) could not be double-buffered in a CU's 160 KB.
// Workspace layout: per (batch*head, query tile) a Q-side blob, then per (batch*head, key tile)
// a K-side blob.  Transposed tiles are [D][TILE] 16-bit values (128- or 64-byte rows), positions permuted.
template <int D> struct BwdWs {
  static constexpr int TILE = D > 128 ? 32 : 64;
  static constexpr int CSH = D > 128 ? 8 : 7;             // bits per digit of rq - D*zq (|.| <= 65280 at head_dim 256)
  static constexpr int T_BYTES = D * TILE * 2;            // one transposed tile
  static constexpr int CQ_BYTES = 5 * TILE * 4;           // digits (2 dwords/query), a, -lse*log2e, -delta
  static constexpr int CK_BYTES = 3 * TILE * 4;           // digits (2 dwords/key), key scale
  static constexpr int Q_BLOB = T_BYTES + CQ_BYTES;           // Qz^T, constants
  static constexpr int K_BLOB = T_BYTES + CK_BYTES;           // Kz^T, constants
};

int64_t bwd_workspace_bytes(int64_t B, int64_t H, int64_t Nq, int64_t Nk, int D) {
  const int64_t tile = D == 256 ? BwdWs<256>::TILE : 64;
  const int64_t tq = (Nq + tile - 1) / tile, tk = (Nk + tile - 1) / tile;
  const int64_t qb = D == 256 ? BwdWs<256>::Q_BLOB : D == 128 ? BwdWs<128>::Q_BLOB : BwdWs<64>::Q_BLOB;
  const int64_t kb = D == 256 ? BwdWs<256>::K_BLOB : D == 128 ? BwdWs<128>::K_BLOB : BwdWs<64>::K_BLOB;
  return B * H * (tq * qb + tk * kb);
}

struct BwdArgs {
  const int8_t *qc; const float *sq; const int8_t *zq; const int32_t *rq;
  const int8_t *kc; const float *sk; const int8_t *zk; const int32_t *rk;
  const void *v; const void *o; const void *dout; const float *lse;
  unsigned char *ws_q; unsigned char *ws_k;
  void *dq; void *dk; void *dv;
  int64_t H;
  int Nq, Nk;
  int tiles_q, tiles_k;
  int64_t sqb, sqh, sqn, skb, skh, skn, svb, svh, svn, sob, soh, son;
  int64_t sdob, sdoh, sdon, sdqb, sdqh, sdqn, sdkb, sdkh, sdkn, sdvb, sdvh, sdvn;
  float sm_scale, sm_scale_log2;
  int nblocks;          // query blocks (dq) or key blocks (dkdv) per (b,h)
  int total_blocks, blocks_per_xcd;
  int group_log2;       // causal: log2 of the number of heads whose blocks are dispatched together (set per launch)
};

// position of streamed row r (0..63, or 0..31 in a 32-row tile) inside a transposed tile: the order in which the 32x32
// accumulator layout hands out rows to a lane (two runs of 4 per 16-row MFMA k-slice)
__device__ __forceinline__ int perm_pos4(int r4) {   // r4 = r / 4
  return 32 * (r4 / 8) + 16 * ((r4 / 4) % 2) + 8 * (r4 % 2) + 4 * ((r4 / 2) % 2);
}

// (code - zp) for the 8 codes in two dwords of 4 rows, as exact 16-bit floats, transposed:
// writes, for each of the 8 columns, the 4 rows as 8 bytes at dst + column * stride
template <typename T>
__device__ __forceinline__ void store_codes_transposed(const u32x2 (&c)[4], const float (&zp)[4], const float (&sc)[4],
                                                       unsigned char *dst, int stride) {
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    float f[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) f[r] = ((float)(int)(int8_t)((c[r][e / 4] >> (8 * (e % 4))) & 0xff) - zp[r]) * sc[r];
    u32x2 o;
    o[0] = pack2<T>(f[0], f[1]);
    o[1] = pack2<T>(f[2], f[3]);
    *reinterpret_cast<u32x2 *>(dst + e * stride) = o;
  }
}
// integer n -> (2^SH * floor(n / 2^SH), n mod 2^SH) resp. their negatives, as a packed pair of 16-bit floats
template <typename T, int SH = 7> __device__ __forceinline__ unsigned base128_pair(int n, float sign) {
  const int hi = n >> SH, lo = n & ((1 << SH) - 1);
  return pack2<T>(sign * (float)(hi * (1 << SH)), sign * (float)lo);
}

// ------------------------------------------------------------------------------------------ prep
// One block per (b,h, 64-query tile): delta, Qz^T and the per-query constants.
template <typename T, int D> __global__ __launch_bounds__(256) void bwd_prep_q_kernel(BwdArgs a) {
  typedef BwdWs<D> WS;
  constexpr int BWD_TILE = WS::TILE;
  static_assert((BWD_TILE / 4) * (D / 8) <= 256, "one thread per 4 rows x 8 columns");
  __shared__ float red[D / 8][BWD_TILE];
  const int tid = threadIdx.x;
  const int bh = blockIdx.x / a.tiles_q, tile = blockIdx.x % a.tiles_q;
  const int64_t b = bh / a.H, h = bh % a.H;
  const int i0 = tile * BWD_TILE;
  const int64_t tq0 = (int64_t)bh * a.Nq;
  unsigned char *blob = a.ws_q + ((int64_t)bh * a.tiles_q + tile) * WS::Q_BLOB;
  const int r4 = tid % (BWD_TILE / 4), dc = tid / (BWD_TILE / 4);
  if (dc < D / 8) {
    const int8_t *qc_bh = a.qc + b * a.sqb + h * a.sqh;
    const T *do_bh = reinterpret_cast<const T *>(a.dout) + b * a.sdob + h * a.sdoh;
    const T *o_bh = reinterpret_cast<const T *>(a.o) + b * a.sob + h * a.soh;
    u32x2 creg[4];
    u32x4 greg[4];
    float zreg[4], sreg[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int i = min(i0 + 4 * r4 + r, a.Nq - 1);
      creg[r] = *reinterpret_cast<const u32x2 *>(qc_bh + (int64_t)i * a.sqn + dc * 8);
      greg[r] = *reinterpret_cast<const u32x4 *>(do_bh + (int64_t)i * a.sdon + dc * 8);
      const u32x4 ow = *reinterpret_cast<const u32x4 *>(o_bh + (int64_t)i * a.son + dc * 8);
      zreg[r] = (float)a.zq[tq0 + i];
      sreg[r] = a.sq[tq0 + i];
      float s = 0.f;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        s = __builtin_fmaf(lo_to_f32<T>(ow[e]), lo_to_f32<T>(greg[r][e]), s);
        s = __builtin_fmaf(hi_to_f32<T>(ow[e]), hi_to_f32<T>(greg[r][e]), s);
      }
      red[dc][4 * r4 + r] = s;
    }
    const int pos = perm_pos4(r4);
    // the dequantized Q itself, rounded to the 16-bit type (what dK = sm * dS^T Q^ contracts with)
    store_codes_transposed<T>(creg, zreg, sreg, blob + (dc * 8) * (BWD_TILE * 2) + pos * 2, BWD_TILE * 2);
  }
  __syncthreads();
  if (tid < BWD_TILE) {
    const int i = min(i0 + tid, a.Nq - 1);
    float delta = 0.f;
#pragma unroll
    for (int x = 0; x < D / 8; ++x) delta += red[x][tid];
    const int zq = (int)a.zq[tq0 + i];
    const int c = a.rq[tq0 + i] - D * zq;
    unsigned *cq = reinterpret_cast<unsigned *>(blob + WS::T_BYTES);
    u32x2 dg;
    dg[0] = pack2<T>((float)(-zq), (float)(-zq));      // k-group 0: times the two digits of rk
    dg[1] = base128_pair<T, WS::CSH>(c, -1.0f);        // k-group 1: minus the digits of rq - D*zq, times zk
    reinterpret_cast<u32x2 *>(cq)[tid] = dg;
    reinterpret_cast<float *>(cq)[2 * BWD_TILE + tid] = a.sq[tq0 + i] * a.sm_scale_log2;
    reinterpret_cast<float *>(cq)[3 * BWD_TILE + tid] = -a.lse[tq0 + i] * kLog2e;
    reinterpret_cast<float *>(cq)[4 * BWD_TILE + tid] = -delta;   // the dP accumulators start from it
  }
}

// One block per (b,h, 64-key tile): Kz^T and the per-key constants.
template <typename T, int D> __global__ __launch_bounds__(256) void bwd_prep_k_kernel(BwdArgs a) {
  typedef BwdWs<D> WS;
  constexpr int BWD_TILE = WS::TILE;
  const int tid = threadIdx.x;
  const int bh = blockIdx.x / a.tiles_k, tile = blockIdx.x % a.tiles_k;
  const int64_t b = bh / a.H, h = bh % a.H;
  const int j0 = tile * BWD_TILE;
  const int64_t tk0 = (int64_t)bh * a.Nk;
  unsigned char *blob = a.ws_k + ((int64_t)bh * a.tiles_k + tile) * WS::K_BLOB;
  const int r4 = tid % (BWD_TILE / 4), dc = tid / (BWD_TILE / 4);
  if (dc < D / 8) {
    const int8_t *kc_bh = a.kc + b * a.skb + h * a.skh;
    u32x2 creg[4];
    float zreg[4], sreg[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int j = min(j0 + 4 * r4 + r, a.Nk - 1);
      creg[r] = *reinterpret_cast<const u32x2 *>(kc_bh + (int64_t)j * a.skn + dc * 8);
      zreg[r] = (float)a.zk[tk0 + j];
      sreg[r] = a.sk[tk0 + j];
    }
    // the dequantized K, rounded to the 16-bit type (what dQ = sm * dS K^ contracts with)
    store_codes_transposed<T>(creg, zreg, sreg, blob + (dc * 8) * (BWD_TILE * 2) + perm_pos4(r4) * 2, BWD_TILE * 2);
  }
  if (tid < BWD_TILE) {
    const int j = min(j0 + tid, a.Nk - 1);
    const int zk = (int)a.zk[tk0 + j];
    unsigned *ck = reinterpret_cast<unsigned *>(blob + WS::T_BYTES);
    u32x2 dg;
    dg[0] = base128_pair<T>(a.rk[tk0 + j], 1.0f);      // k-group 0: digits of rk
    dg[1] = pack2<T>((float)zk, (float)zk);            // k-group 1: zk, zk
    reinterpret_cast<u32x2 *>(ck)[tid] = dg;
    reinterpret_cast<float *>(ck)[2 * BWD_TILE + tid] = a.sk[tk0 + j];
  }
}

// ------------------------------------------------------------------------------------------ dQ
// Threads per workgroup (32 queries per wave) and waves per SIMD the registers are budgeted for.  D=128:
// 8 waves = 256 queries, one workgroup per CU (two 41 KB tile buffers).  D=64: the loop fits 170 registers
// and the buffers 42 KB, so three workgroups of 4 waves run per CU (3 waves per SIMD; backward of
// B16 H16 N2048 D64 causal 0.90 -> 0.84 ms against 8-wave workgroups, 2-wave ones are slower again).
// D=256: 4 waves, one per SIMD (128 accumulators, 96 operand registers), two 41 KB buffers of 32-key tiles.
template <int D> struct DqShape {
  static constexpr int THREADS = D == 128 ? 512 : 256;
  static constexpr int WAVES_PER_SIMD = D == 64 ? 3 : D == 128 ? 2 : 1;
  static constexpr int BLK = 32 * (THREADS / 64);
};

template <typename T, int D, bool CAUSAL>
__global__ __launch_bounds__(DqShape<D>::THREADS, DqShape<D>::WAVES_PER_SIMD) void bwd_dq_kernel(BwdArgs a) {
  constexpr int DQ_THREADS = DqShape<D>::THREADS, DQ_BLK = DqShape<D>::BLK;
  typedef BwdWs<D> WS;
  constexpr int BWD_TILE = WS::TILE, NBLK = BWD_TILE / 32;
  typedef Swz<D> SK;            // K code rows
  typedef Swz<2 * D> SV;        // V rows
  typedef Swz<BWD_TILE * 2> ST; // transposed rows
  constexpr int KS = D / 32, DB = D / 32, KD = D / 16;
  constexpr int K_BYTES = BWD_TILE * D, V_BYTES = BWD_TILE * 2 * D, T_BYTES = WS::T_BYTES;
  constexpr int OFF_V = K_BYTES, OFF_T = OFF_V + V_BYTES, OFF_C = OFF_T + T_BYTES, BUF = OFF_C + WS::CK_BYTES;
  __shared__ __attribute__((aligned(16))) unsigned char smem[2 * BUF];

  const int L = blockIdx.x;
  const int vid = (L % 8) * a.blocks_per_xcd + (L / 8);
  if (vid >= a.total_blocks) return;
  int bh = vid / a.nblocks;
  int mb = vid % a.nblocks;
  if (CAUSAL) {
    // longest rows first, 2^group_log2 heads at a time (ids cycle through the heads of a group): with one
    // head after the other the last head's long blocks start while the chip is already draining
    const int GL = a.group_log2;
    const int pb = bh >> GL << GL;
    if (pb + (1 << GL) <= a.total_blocks / a.nblocks) {
      const int idx = (bh - pb) * a.nblocks + mb;
      bh = pb + (idx & ((1 << GL) - 1));
      mb = idx >> GL;
    }
    mb = a.nblocks - 1 - mb;
  }
  const int64_t b = bh / a.H, h = bh % a.H;
  const int m0 = mb * DQ_BLK;
  const int tid = threadIdx.x, wave = tid / 64, lane = tid % 64, lr = lane % 32, g = lane / 32;

  const int8_t *qc_bh = a.qc + b * a.sqb + h * a.sqh;
  const unsigned char *kc_bh = reinterpret_cast<const unsigned char *>(a.kc + b * a.skb + h * a.skh);
  const unsigned char *v_bh = reinterpret_cast<const unsigned char *>(reinterpret_cast<const T *>(a.v) + b * a.svb + h * a.svh);
  const T *do_bh = reinterpret_cast<const T *>(a.dout) + b * a.sdob + h * a.sdoh;
  T *dq_bh = reinterpret_cast<T *>(a.dq) + b * a.sdqb + h * a.sdqh;
  const unsigned char *wsk_bh = a.ws_k + (int64_t)bh * a.tiles_k * WS::K_BLOB;
  const unsigned char *wsq_bh = a.ws_q + (int64_t)bh * a.tiles_q * WS::Q_BLOB;

  const int qi = m0 + wave * 32 + lr;
  const int qi_c = qi < a.Nq ? qi : a.Nq - 1;
  i32x4 qf[KS];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks)
    qf[ks] = *reinterpret_cast<const i32x4 *>(qc_bh + (int64_t)qi_c * a.sqn + ks * 32 + g * 16);
  u32x4 dof[KD];
#pragma unroll
  for (int kd = 0; kd < KD; ++kd)
    dof[kd] = *reinterpret_cast<const u32x4 *>(do_bh + (int64_t)qi_c * a.sdon + kd * 16 + g * 8);
  // per-query constants prepared by prep_q: correction digits, a = sq*sm*log2e, -lse*log2e, -delta
  const unsigned *cq = reinterpret_cast<const unsigned *>(wsq_bh + (int64_t)(qi_c / BWD_TILE) * WS::Q_BLOB + WS::T_BYTES);
  const int ql = qi_c % BWD_TILE;
  const u32x4 corr_q = {cq[2 * ql + g], 0u, 0u, 0u};
  const float a_i = __builtin_bit_cast(float, cq[2 * BWD_TILE + ql]);
  const float nlse2 = __builtin_bit_cast(float, cq[3 * BWD_TILE + ql]);
  const float ndelta_i = __builtin_bit_cast(float, cq[4 * BWD_TILE + ql]);   // -delta
  const int q_first = m0 + wave * 32, q_last = q_first + 31;

  int kv_end = a.Nk;
  const int coff = CAUSAL ? a.Nk - a.Nq : 0;   // causal: query i keeps keys j <= i + coff (mask aligned to the last key)
  if (CAUSAL) kv_end = min(a.Nk, m0 + DQ_BLK + coff);
  const int ntiles = (kv_end + BWD_TILE - 1) / BWD_TILE;

  // full tiles: per-thread offsets computed once, one copy instruction per chunk afterwards
  const int wave_u = __builtin_amdgcn_readfirstlane(wave);
  TileCopy<D, BWD_TILE, DQ_THREADS> cp_k;
  TileCopy<2 * D, BWD_TILE, DQ_THREADS> cp_v;
  TileCopy<BWD_TILE * 2, D, DQ_THREADS> cp_t;
  TileCopy<WS::CK_BYTES, 1, DQ_THREADS, NoSwz<WS::CK_BYTES>> cp_c;
  cp_k.init((unsigned)a.skn, tid);
  cp_v.init((unsigned)a.svn * 2u, tid);
  cp_t.init(BWD_TILE * 2, tid);
  cp_c.init(0, tid);
  // the copy of a tile goes out in two halves (one before each 32-key block of the tile in work), so
  // that the memory pipe is not handed all of it in one burst
  auto load_tile_a = [&](int t) {
    unsigned char *base = smem + (t & 1) * BUF;
    if ((t + 1) * BWD_TILE <= a.Nk) {
      cp_k.issue(kc_bh + (int64_t)t * BWD_TILE * a.skn, base, wave_u, tid);
      cp_v.issue(v_bh + (int64_t)t * BWD_TILE * a.svn * 2, base + OFF_V, wave_u, tid);
    } else {
      dma_rows<D, BWD_TILE, DQ_THREADS>(kc_bh, a.skn, t * BWD_TILE, a.Nk - 1, base, tid);
      dma_rows<2 * D, BWD_TILE, DQ_THREADS>(v_bh, a.svn * 2, t * BWD_TILE, a.Nk - 1, base + OFF_V, tid);
    }
  };
  auto load_tile_b = [&](int t) {
    unsigned char *base = smem + (t & 1) * BUF;
    const unsigned char *blob = wsk_bh + (int64_t)t * WS::K_BLOB;
    cp_t.issue(blob, base + OFF_T, wave_u, tid);
    cp_c.issue(blob + WS::T_BYTES, base + OFF_C, wave_u, tid);
  };
  auto load_tile = [&](int t) {
    load_tile_a(t);
    load_tile_b(t);
  };

  f32x16 dqacc[DB];
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int v = 0; v < 16; ++v) dqacc[db][v] = 0.f;

  // one 32-key block of tile t
  auto block = [&](int t, int nb, auto masked_tag) {
    constexpr bool MASKED = decltype(masked_tag)::value;
    const unsigned char *base = smem + (t & 1) * BUF;
    const unsigned *dgp = reinterpret_cast<const unsigned *>(base + OFF_C);
    const float *skp = reinterpret_cast<const float *>(base + OFF_C) + 2 * BWD_TILE;
    const int j0 = t * BWD_TILE;
    i32x16 acc;
    f32x16 dp;
#pragma unroll
    for (int v = 0; v < 16; ++v) { acc[v] = 0; dp[v] = ndelta_i; }   // dp = dP^T - delta straight from the MFMAs
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const i32x4 kf = *reinterpret_cast<const i32x4 *>(base + SK::off(32 * nb + lr, 2 * ks + g));
      acc = mfma_i8(kf, qf[ks], acc);
    }
#pragma unroll
    for (int kd = 0; kd < KD; ++kd) {
      const u32x4 vf = *reinterpret_cast<const u32x4 *>(base + OFF_V + SV::off(32 * nb + lr, 2 * kd + g));
      dp = mfma_16b<T>(vf, dof[kd], dp);
    }
    f32x16 f;
#pragma unroll
    for (int v = 0; v < 16; ++v) f[v] = (float)acc[v];
    const u32x4 corr_k = {dgp[2 * (32 * nb + lr) + g], 0u, 0u, 0u};
    f = mfma_16b<T>(corr_k, corr_q, f);
    float ds[16];
#pragma unroll
    for (int aa = 0; aa < 4; ++aa) {
      const int jl = 32 * nb + 8 * aa + 4 * g;
      const f32x4 sk4 = *reinterpret_cast<const f32x4 *>(skp + jl);
#pragma unroll
      for (int bb = 0; bb < 4; ++bb) {
        const int v = 4 * aa + bb;
        float p = __builtin_amdgcn_exp2f(__builtin_fmaf(a_i, f[v] * sk4[bb], nlse2));
        if (MASKED) {
          const int j = j0 + jl + bb;
          if ((CAUSAL && j > qi + coff) || j >= a.Nk) p = 0.f;
        }
        ds[v] = p * dp[v];
      }
    }
#pragma unroll
    for (int hh = 0; hh < 2; ++hh) {
      u32x4 dsf;
#pragma unroll
      for (int e = 0; e < 4; ++e) dsf[e] = pack2<T>(ds[8 * hh + 2 * e], ds[8 * hh + 2 * e + 1]);
#pragma unroll
      for (int db = 0; db < DB; ++db) {
        const u32x4 ktf = *reinterpret_cast<const u32x4 *>(base + OFF_T + ST::off(32 * db + lr, 4 * nb + 2 * hh + g));
        dqacc[db] = mfma_16b<T>(ktf, dsf, dqacc[db]);
      }
    }
  };

  load_tile(0);
  dma_wait();
  __syncthreads();
  for (int t = 0; t < ntiles; ++t) {
    const int j0 = t * BWD_TILE;
#pragma unroll
    for (int nb = 0; nb < NBLK; ++nb) {
      if (t + 1 < ntiles) {
        if (nb == 0) load_tile_a(t + 1);
        if (nb == NBLK - 1) load_tile_b(t + 1);
      }
      const int jb = j0 + 32 * nb;
      if ((jb >= a.Nk) || (CAUSAL && jb > q_last + coff)) continue;        // wave-uniform
      if ((CAUSAL && jb + 31 > q_first + coff) || (jb + 32 > a.Nk)) block(t, nb, std::true_type{});
      else block(t, nb, std::false_type{});
    }
    dma_wait();
    __syncthreads();
  }

  // dQ leaves as whole rows through LDS (the tile buffers are free after the last barrier)
  static_assert((DQ_THREADS / 64) * 32 * 2 * D <= 2 * BUF, "output staging fits the tile buffers");
  store_tile_rows<T, D>(dqacc, a.sm_scale, smem + (tid / 64) * (32 * 2 * D), dq_bh, a.sdqn, q_first, a.Nq, tid % 64);
}

// ------------------------------------------------------------------------------------------ dK, dV
// One workgroup = 4 (head_dim 128) or 6 (head_dim 64) wave pairs of 32 keys each.  The dK^T and dV^T
// accumulators of 32 keys take 128 registers at head_dim 128, too many for two waves per SIMD, so each 32-key
// slice is shared by a PAIR of waves (w and w + pairs; with 4 pairs they sit on the same SIMD):
//   P-wave  (w < pairs):  S = Qc.Kc^T (INT8 MFMA), P = exp2(.), hands P to its partner through LDS (rounded to
//                     the 16-bit type, as its own dV product uses it: half the exchange traffic of fp32),
//                     dV^T += dO^T.P
//   dS-wave (the others): dP = dO.V^T, then dS = P o (dP - delta) with the partner's P,
//                     dK^T += Qz^T.dS
// No product is computed twice, each wave keeps 64 accumulator registers, and within a SIMD one wave
// is in its VALU phase while the other feeds the matrix pipe.  One barrier per 32-query block: P goes
// to the exchange slot of the block's parity, so the slot written for block b is read before barrier
// b+1 and not written again before that barrier has passed.
// Wave pairs per workgroup (32 keys per pair) and waves per SIMD the registers are budgeted for.  One
// workgroup runs per CU (the two tile buffers and the exchange fill the LDS).  D=128: 4 pairs, 2 waves per
// SIMD (the loop takes 220 registers).  D=64: 6 pairs, 3 waves per SIMD (145 registers); backward of
// B16 H16 N2048 D64 causal 0.84 -> 0.805 ms against 4 pairs; 3 pairs with two workgroups per CU are slower
// (0.95 ms), 8 pairs need 128 registers and spill.
// D=256: 2 pairs, one wave per SIMD (128 accumulators and up to 200 operand registers), 32-query tiles.
template <int D> struct DkvShape {
  static constexpr int PAIRS = D == 64 ? 6 : D == 128 ? 4 : 2;
  static constexpr int WAVES_PER_SIMD = D == 64 ? 3 : D == 128 ? 2 : 1;
  static constexpr int THREADS = 128 * PAIRS, BLK = 32 * PAIRS;
};

// two 16-bit floats of one dword -> fp32
template <typename T> __device__ __forceinline__ float unpack_lo(unsigned w);
template <typename T> __device__ __forceinline__ float unpack_hi(unsigned w);
template <> __device__ __forceinline__ float unpack_lo<__bf16>(unsigned w) { return __builtin_bit_cast(float, w << 16); }
template <> __device__ __forceinline__ float unpack_hi<__bf16>(unsigned w) { return __builtin_bit_cast(float, w & 0xffff0000u); }
template <> __device__ __forceinline__ float unpack_lo<_Float16>(unsigned w) {
  return (float)__builtin_bit_cast(_Float16, (unsigned short)(w & 0xffffu));
}
template <> __device__ __forceinline__ float unpack_hi<_Float16>(unsigned w) {
  return (float)__builtin_bit_cast(_Float16, (unsigned short)(w >> 16));
}

template <typename T, int D, bool CAUSAL>
__global__ __launch_bounds__(DkvShape<D>::THREADS, DkvShape<D>::WAVES_PER_SIMD) void bwd_dkdv_kernel(BwdArgs a) {
  constexpr int NP = DkvShape<D>::PAIRS, DKV_THREADS = DkvShape<D>::THREADS;
  typedef BwdWs<D> WS;
  constexpr int BWD_TILE = WS::TILE, NBLK = BWD_TILE / 32;
  typedef Swz<D> SQ;            // Q code rows
  typedef SwzDual<2 * D> SG;    // dO rows: read row-wise for dP and through transposing reads for dV
  typedef Swz<BWD_TILE * 2> ST; // transposed rows
  constexpr int KS = D / 32, DB = D / 32, KD = D / 16;
  constexpr int Q_BYTES = BWD_TILE * D, G_BYTES = BWD_TILE * 2 * D, T_BYTES = WS::T_BYTES;
  constexpr int OFF_DO = Q_BYTES, OFF_QT = OFF_DO + G_BYTES, OFF_C = OFF_QT + T_BYTES,
                BUF = OFF_C + WS::CQ_BYTES;
  constexpr int OFF_X = 2 * BUF;             // P exchange: per pair 2 slots x 64 lanes x 16 packed 16-bit floats
  __shared__ __attribute__((aligned(16))) unsigned char smem[2 * BUF + NP * 4096];

  const int L = blockIdx.x;
  const int vid = (L % 8) * a.blocks_per_xcd + (L / 8);
  if (vid >= a.total_blocks) return;
  int bh = vid / a.nblocks;
  int nbk = vid % a.nblocks;   // causal: early key blocks see the most queries and come first
  if (CAUSAL && a.group_log2 > 0) {
    // key blocks of 2^group_log2 heads dispatched together, from the longest down (as in the dQ kernel);
    // the launcher allows it only while the query-side tiles of the group fit an XCD's L2
    const int GL = a.group_log2;
    const int pb = bh >> GL << GL;
    if (pb + (1 << GL) <= a.total_blocks / a.nblocks) {
      const int idx = (bh - pb) * a.nblocks + nbk;
      bh = pb + (idx & ((1 << GL) - 1));
      nbk = idx >> GL;
    }
  }
  const int64_t b = bh / a.H, h = bh % a.H;
  const int n0 = nbk * DkvShape<D>::BLK;
  const int tid = threadIdx.x, wave = tid / 64, lane = tid % 64, lr = lane % 32, g = lane / 32;
  const int pair = wave % NP;
  const bool p_role = wave < NP;     // wave-uniform

  const unsigned char *qc_bh = reinterpret_cast<const unsigned char *>(a.qc + b * a.sqb + h * a.sqh);
  const int8_t *kc_bh = a.kc + b * a.skb + h * a.skh;
  const T *v_bh = reinterpret_cast<const T *>(a.v) + b * a.svb + h * a.svh;
  const unsigned char *do_bh = reinterpret_cast<const unsigned char *>(reinterpret_cast<const T *>(a.dout) + b * a.sdob + h * a.sdoh);
  T *dk_bh = reinterpret_cast<T *>(a.dk) + b * a.sdkb + h * a.sdkh;
  T *dv_bh = reinterpret_cast<T *>(a.dv) + b * a.sdvb + h * a.sdvh;
  const unsigned char *wsk_bh = a.ws_k + (int64_t)bh * a.tiles_k * WS::K_BLOB;
  const unsigned char *wsq_bh = a.ws_q + (int64_t)bh * a.tiles_q * WS::Q_BLOB;

  // ---- this lane's key: INT8 codes + correction digits + scale for the P role, V row for the dS role
  const int kj = n0 + pair * 32 + lr;
  const int kj_c = kj < a.Nk ? kj : a.Nk - 1;
  u32x4 breg[KD];   // persistent B operand: K codes (first KS entries) or V (KD entries)
  if (p_role) {
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
      breg[ks] = *reinterpret_cast<const u32x4 *>(kc_bh + (int64_t)kj_c * a.skn + ks * 32 + g * 16);
  } else {
#pragma unroll
    for (int kd = 0; kd < KD; ++kd)
      breg[kd] = *reinterpret_cast<const u32x4 *>(v_bh + (int64_t)kj_c * a.svn + kd * 16 + g * 8);
  }
  const unsigned *ck = reinterpret_cast<const unsigned *>(wsk_bh + (int64_t)(kj_c / BWD_TILE) * WS::K_BLOB + WS::T_BYTES);
  const int kl = kj_c % BWD_TILE;
  const u32x4 corr_k = {ck[2 * kl + g], 0u, 0u, 0u};
  const float sk_j = __builtin_bit_cast(float, ck[2 * BWD_TILE + kl]);
  const int k_first = n0 + pair * 32, k_last = k_first + 31;

  const int coff = CAUSAL ? a.Nk - a.Nq : 0;   // causal: key j is seen by the queries i >= j - coff
  const int it0 = CAUSAL ? max(n0 - coff, 0) / BWD_TILE : 0;
  const int ntiles = a.tiles_q;

  // full tiles: per-thread offsets computed once, one copy instruction per chunk afterwards
  const int wave_u = __builtin_amdgcn_readfirstlane(wave);
  TileCopy<D, BWD_TILE, DKV_THREADS> cp_q;
  TileCopy<2 * D, BWD_TILE, DKV_THREADS, SG> cp_g;
  TileCopy<BWD_TILE * 2, D, DKV_THREADS> cp_t;
  TileCopy<WS::CQ_BYTES, 1, DKV_THREADS, NoSwz<WS::CQ_BYTES>> cp_c;
  cp_q.init((unsigned)a.sqn, tid);
  cp_g.init((unsigned)a.sdon * 2u, tid);
  cp_t.init(BWD_TILE * 2, tid);
  cp_c.init(0, tid);
  // the copy of a tile goes out in two halves (parts 0-1, 2), one before each 32-query block of the
  // tile in work, so that the memory pipe is not handed all of it in one burst (four quarters, one
  // per phase, measured slower)
  auto load_part = [&](int t, int part) {
    unsigned char *base = smem + (t & 1) * BUF;
    const unsigned char *blob = wsq_bh + (int64_t)t * WS::Q_BLOB;
    const bool full = (t + 1) * BWD_TILE <= a.Nq;
    if (part == 0) {
      if (full) cp_q.issue(qc_bh + (int64_t)t * BWD_TILE * a.sqn, base, wave_u, tid);
      else dma_rows<D, BWD_TILE, DKV_THREADS>(qc_bh, a.sqn, t * BWD_TILE, a.Nq - 1, base, tid);
      cp_c.issue(blob + WS::T_BYTES, base + OFF_C, wave_u, tid);
    } else if (part == 1) {
      if (full) cp_g.issue(do_bh + (int64_t)t * BWD_TILE * a.sdon * 2, base + OFF_DO, wave_u, tid);
      else dma_rows<2 * D, BWD_TILE, DKV_THREADS, SG>(do_bh, a.sdon * 2, t * BWD_TILE, a.Nq - 1, base + OFF_DO, tid);
    } else if (part == 2) {
      cp_t.issue(blob, base + OFF_QT, wave_u, tid);
    }
  };
  auto load_tile = [&](int t) {
    for (int part = 0; part < 3; ++part) load_part(t, part);
  };

  f32x16 oacc[DB];   // dV^T (P role) or dK^T (dS role) for this lane's key
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int v = 0; v < 16; ++v) oacc[db][v] = 0.f;

  // [slot][2][64 lanes] of 8 packed 16-bit floats; the slot is the block's parity, so that one barrier per block is
  // enough: P(b) is written before barrier b and read before barrier b+1, P(b+2) is written after it
  u32x4 *xch0 = reinterpret_cast<u32x4 *>(smem + OFF_X + pair * 4096);

  // LDS operands are fetched in groups well ahead of the MFMAs that consume them (a 16-byte LDS read
  // takes far longer than an MFMA issue slot, and the compiler keeps loads next to their use), the
  // groups are pinned in place with scheduling barriers.
  // ---- P role, first half of a block: S, correction, P; P goes to LDS and stays packed in pf;
  // the dO^T fragments of the second half are requested here as well
  // dO^T comes out of the dO tile through ds_read_b64_tr_b16: lane (d, k-group g) gets queries
  // 16hh + 4g + {0..3} and those + 8 of its d, the order in which pf holds P.  Offsets inside the tile:
  const int t_row = (lane % 16) / 4;
  const unsigned t_off = (unsigned)((4 * g + t_row) * (2 * D) +
                                    ((((SG::quarter(t_row)) << 2) | ((2 * ((lane / 16) % 2) + (lane % 4) / 2) ^ g)) << 4) +
                                    8 * (lane % 2));   // XOR 64*db: d block; XOR 32 with +8 rows: the second four queries
  auto p_first = [&](const unsigned char *base, int i0, int mbk, int slot, u32x4 (&pf)[2], u32x2 (&ta)[2 * DB],
                     u32x2 (&tb)[2 * DB], auto masked_tag) {
    constexpr bool MASKED = decltype(masked_tag)::value;
    const unsigned *dgp = reinterpret_cast<const unsigned *>(base + OFF_C);
    const float *cs = reinterpret_cast<const float *>(base + OFF_C);
    i32x4 qfr[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
      qfr[ks] = *reinterpret_cast<const i32x4 *>(base + SQ::off(32 * mbk + lr, 2 * ks + g));
    const u32x4 corr_q = {dgp[2 * (32 * mbk + lr) + g], 0u, 0u, 0u};
    f32x4 a4[4], nl4[4];
#pragma unroll
    for (int aa = 0; aa < 4; ++aa) {
      const int il = 32 * mbk + 8 * aa + 4 * g;
      a4[aa] = *reinterpret_cast<const f32x4 *>(cs + 2 * BWD_TILE + il);
      nl4[aa] = *reinterpret_cast<const f32x4 *>(cs + 3 * BWD_TILE + il);
    }
    __builtin_amdgcn_sched_barrier(0);
    i32x16 acc;
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[v] = 0;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) acc = mfma_i8(qfr[ks], __builtin_bit_cast(i32x4, breg[ks]), acc);
    f32x16 f;
#pragma unroll
    for (int v = 0; v < 16; ++v) f[v] = (float)acc[v];
    f = mfma_16b<T>(corr_q, corr_k, f);
    float pp[16];
#pragma unroll
    for (int aa = 0; aa < 4; ++aa) {
      const int il = 32 * mbk + 8 * aa + 4 * g;
#pragma unroll
      for (int bb = 0; bb < 4; ++bb) {
        float p = __builtin_amdgcn_exp2f(__builtin_fmaf(a4[aa][bb], f[4 * aa + bb] * sk_j, nl4[aa][bb]));
        if (MASKED) {
          const int i = i0 + il + bb;
          if ((CAUSAL && kj > i + coff) || i >= a.Nq || kj >= a.Nk) p = 0.f;
        }
        pp[4 * aa + bb] = p;
      }
    }
#pragma unroll
    for (int hh = 0; hh < 2; ++hh) {
#pragma unroll
      for (int e = 0; e < 4; ++e) pf[hh][e] = pack2<T>(pp[8 * hh + 2 * e], pp[8 * hh + 2 * e + 1]);
      xch0[slot * 128 + hh * 64 + lane] = pf[hh];
    }
    __builtin_amdgcn_sched_barrier(0);
    // requested behind the compiler's back; the barrier that follows waits for every LDS operation of the
    // wave, and lds_wait_async after it ties the registers to that wait
    const unsigned tbase = lds_addr(base + OFF_DO) + mbk * 32 * (2 * D);
#pragma unroll
    for (int db = 0; db < DB; ++db) {
      const unsigned ad = tbase + (t_off ^ (64 * db)), ad2 = tbase + (t_off ^ (64 * db) ^ 32);
      ta[2 * db] = lds_read_tr16_async<0>(ad);
      ta[2 * db + 1] = lds_read_tr16_async<8 * 2 * D>(ad2);
      tb[2 * db] = lds_read_tr16_async<16 * 2 * D>(ad);
      tb[2 * db + 1] = lds_read_tr16_async<24 * 2 * D>(ad2);
    }
  };
  // ---- dS role, first half: dP = dO.V^T; then the Qz^T fragments and constants of the second half
  auto ds_first = [&](const unsigned char *base, int mbk, f32x16 &dp, u32x4 (&tf)[2 * DB]) {
    const float *cs = reinterpret_cast<const float *>(base + OFF_C);
    u32x4 gf[KD];
    // the accumulators start from -delta of their rows, so that the MFMAs leave dP - delta
#pragma unroll
    for (int aa = 0; aa < 4; ++aa) {
      const f32x4 nd = *reinterpret_cast<const f32x4 *>(cs + 4 * BWD_TILE + 32 * mbk + 8 * aa + 4 * g);
#pragma unroll
      for (int bb = 0; bb < 4; ++bb) dp[4 * aa + bb] = nd[bb];
    }
#pragma unroll
    for (int kd = 0; kd < KD; ++kd)
      gf[kd] = *reinterpret_cast<const u32x4 *>(base + OFF_DO + SG::off(32 * mbk + lr, 2 * kd + g));
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int kd = 0; kd < KD; ++kd) dp = mfma_16b<T>(gf[kd], breg[kd], dp);
#pragma unroll
    for (int hh = 0; hh < 2; ++hh)
#pragma unroll
      for (int db = 0; db < DB; ++db)
        tf[hh * DB + db] = *reinterpret_cast<const u32x4 *>(base + OFF_QT + ST::off(32 * db + lr, 4 * mbk + 2 * hh + g));
  };
  // ---- second half: accumulate with the prefetched transposed fragments
  auto accumulate = [&](const u32x4 (&tf)[2 * DB], const u32x4 (&bf)[2]) {
#pragma unroll
    for (int hh = 0; hh < 2; ++hh)
#pragma unroll
      for (int db = 0; db < DB; ++db) oacc[db] = mfma_16b<T>(tf[hh * DB + db], bf[hh], oacc[db]);
  };
  // ---- dS role, second half prologue: dS = P (from partner) * (dP - delta), packed (dp holds dP - delta)
  auto ds_second = [&](int slot, const f32x16 &dp, u32x4 (&dsf)[2]) {
    u32x4 pw[2];
#pragma unroll
    for (int hh = 0; hh < 2; ++hh) pw[hh] = xch0[slot * 128 + hh * 64 + lane];
    float ds[16];
#pragma unroll
    for (int hh = 0; hh < 2; ++hh)
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int v = 8 * hh + 2 * e;
        ds[v] = unpack_lo<T>(pw[hh][e]) * dp[v];
        ds[v + 1] = unpack_hi<T>(pw[hh][e]) * dp[v + 1];
      }
#pragma unroll
    for (int hh = 0; hh < 2; ++hh)
#pragma unroll
      for (int e = 0; e < 4; ++e) dsf[hh][e] = pack2<T>(ds[8 * hh + 2 * e], ds[8 * hh + 2 * e + 1]);
  };

  if (it0 < ntiles) load_tile(it0);
  if (NBLK == 1 && it0 + 1 < ntiles) load_tile(it0 + 1);
  dma_wait();
  __syncthreads();
  // The two roles run separate loops with the same barrier sequence (one per 32-query block).
  auto block_flags = [&](int t, int mbk, bool &on, bool &masked) {
    const int ib = t * BWD_TILE + 32 * mbk;
    on = (ib < a.Nq) && (!CAUSAL || ib + 31 + coff >= k_first);                        // wave-uniform
    masked = (CAUSAL && ib + coff < k_last) || (ib + 32 > a.Nq) || (k_last >= a.Nk);
  };
  // Block (t, mbk): first phase | barrier | second phase; all reads of the tile buffers happen in first phases.
  // 64-query tiles (two blocks): the next tile's copy goes out in two halves around the barrier of the tile's first
  // block and must have landed before the barrier of its second block (its buffer was last read before the
  // previous tile's last barrier).  32-query tiles (one block): after the block's barrier nobody reads the tile's
  // buffer any more, so the tile after the next one is copied into it right there and must have landed before the
  // next block's barrier.
  auto before_first = [&](int t, int mbk) {
    if (NBLK == 2 && mbk == 0 && t + 1 < ntiles) {
      load_part(t + 1, 0);
      load_part(t + 1, 1);
    }
  };
  auto barrier = [&](int mbk) {
    if (mbk == NBLK - 1) dma_wait();
    lds_barrier();   // P of this block is in LDS
  };
  auto after_barrier = [&](int t, int mbk) {
    if (NBLK == 2) {
      if (mbk == 0 && t + 1 < ntiles) load_part(t + 1, 2);
    } else if (t + 2 < ntiles) {
      load_tile(t + 2);
    }
  };
  if (p_role) {
    for (int t = it0; t < ntiles; ++t) {
      const unsigned char *base = smem + (t & 1) * BUF;
#pragma unroll
      for (int mbk = 0; mbk < NBLK; ++mbk) {
        const int slot = NBLK == 2 ? mbk : (t & 1);
        before_first(t, mbk);
        bool on, masked;
        block_flags(t, mbk, on, masked);
        u32x4 pf[2];
        u32x2 ta[2 * DB], tb[2 * DB];
        if (on) {
          if (masked) p_first(base, t * BWD_TILE, mbk, slot, pf, ta, tb, std::true_type{});
          else p_first(base, t * BWD_TILE, mbk, slot, pf, ta, tb, std::false_type{});
        }
        barrier(mbk);
        after_barrier(t, mbk);
        if (on) {
          lds_wait_async<0>(ta);
          lds_wait_async<0>(tb);
#pragma unroll
          for (int db = 0; db < DB; ++db)
            oacc[db] = mfma_16b<T>(u32x4{ta[2 * db][0], ta[2 * db][1], ta[2 * db + 1][0], ta[2 * db + 1][1]}, pf[0], oacc[db]);
#pragma unroll
          for (int db = 0; db < DB; ++db)
            oacc[db] = mfma_16b<T>(u32x4{tb[2 * db][0], tb[2 * db][1], tb[2 * db + 1][0], tb[2 * db + 1][1]}, pf[1], oacc[db]);
        }
      }
    }
  } else {
    for (int t = it0; t < ntiles; ++t) {
      const unsigned char *base = smem + (t & 1) * BUF;
#pragma unroll
      for (int mbk = 0; mbk < NBLK; ++mbk) {
        const int slot = NBLK == 2 ? mbk : (t & 1);
        before_first(t, mbk);
        bool on, masked;
        block_flags(t, mbk, on, masked);
        u32x4 dsf[2], tf[2 * DB];
        f32x16 dp;
        if (on) ds_first(base, mbk, dp, tf);
        barrier(mbk);
        after_barrier(t, mbk);
        if (on) {
          ds_second(slot, dp, dsf);
          accumulate(tf, dsf);
        }
      }
    }
  }

  // dK / dV leave as whole rows through LDS: a barrier first, the last block's exchange slots and fragments may
  // still be read by the partner waves
  __syncthreads();
  static_assert((DKV_THREADS / 64) * 32 * 2 * D <= 2 * BUF + NP * 4096, "output staging fits the workgroup's LDS");
  if (p_role) store_tile_rows<T, D>(oacc, 1.0f, smem + (tid / 64) * (32 * 2 * D), dv_bh, a.sdvn, k_first, a.Nk, tid % 64);
  else store_tile_rows<T, D>(oacc, a.sm_scale, smem + (tid / 64) * (32 * 2 * D), dk_bh, a.sdkn, k_first, a.Nk, tid % 64);
}

template <typename T, int D> static int launch_bwd_td(const AttnArgs &x, hipStream_t st) {
  typedef BwdWs<D> WS;
  BwdArgs a;
  a.qc = x.qc; a.sq = x.sq; a.zq = x.zq; a.rq = x.rq; a.kc = x.kc; a.sk = x.sk; a.zk = x.zk; a.rk = x.rk;
  a.v = x.v; a.o = x.o; a.dout = x.dout; a.lse = x.lse; a.dq = x.dq; a.dk = x.dk; a.dv = x.dv;
  a.H = x.H; a.Nq = (int)x.Nq; a.Nk = (int)x.Nk;
  a.tiles_q = (int)((x.Nq + WS::TILE - 1) / WS::TILE);
  a.tiles_k = (int)((x.Nk + WS::TILE - 1) / WS::TILE);
  a.ws_q = reinterpret_cast<unsigned char *>(x.workspace);
  a.ws_k = a.ws_q + x.B * x.H * (int64_t)a.tiles_q * WS::Q_BLOB;
  a.sqb = x.sqb; a.sqh = x.sqh; a.sqn = x.sqn; a.skb = x.skb; a.skh = x.skh; a.skn = x.skn;
  a.svb = x.svb; a.svh = x.svh; a.svn = x.svn; a.sob = x.sob; a.soh = x.soh; a.son = x.son;
  a.sdob = x.sdob; a.sdoh = x.sdoh; a.sdon = x.sdon; a.sdqb = x.sdqb; a.sdqh = x.sdqh; a.sdqn = x.sdqn;
  a.sdkb = x.sdkb; a.sdkh = x.sdkh; a.sdkn = x.sdkn; a.sdvb = x.sdvb; a.sdvh = x.sdvh; a.sdvn = x.sdvn;
  a.sm_scale = x.sm_scale; a.sm_scale_log2 = x.sm_scale * kLog2e;
  a.nblocks = 0; a.total_blocks = 0; a.blocks_per_xcd = 0; a.group_log2 = 0;
  const dim3 block(256);
  const int64_t BH = x.B * x.H;
  if (BH * a.tiles_q > 0x7fffffffLL || BH * a.tiles_k > 0x7fffffffLL)
    return set_error(QFA_EUNSUPPORTED, "attn_bwd: too many tiles for one launch");
  // staging passes
  bwd_prep_q_kernel<T, D><<<dim3((unsigned)(BH * a.tiles_q)), block, 0, st>>>(a);
  if (int e = check_launch("qfa_attn_bwd (prep q)")) return e;
  bwd_prep_k_kernel<T, D><<<dim3((unsigned)(BH * a.tiles_k)), block, 0, st>>>(a);
  if (int e = check_launch("qfa_attn_bwd (prep k)")) return e;
  // dK, dV
  {
    constexpr int DKV_THREADS = DkvShape<D>::THREADS;
    a.nblocks = (int)((x.Nk + DkvShape<D>::BLK - 1) / DkvShape<D>::BLK);
    // per head the kernel streams Qc, dO and Qz^T (5 bytes per query and d): group heads while that stays
    // within about 6 MB (pairs at N=4096, D=128: 5.2 MB against the XCD's 4 MB L2, measured 1 % better than
    // single heads; four heads are not)
    const int64_t head_bytes = x.Nq * (int64_t)D * 5;
    a.group_log2 = 0;
    while (a.group_log2 < 2 && (head_bytes << (a.group_log2 + 1)) <= (6 << 20)) ++a.group_log2;
    const int64_t total = (int64_t)a.nblocks * BH;
    if (total > 0x3fffffffLL) return set_error(QFA_EUNSUPPORTED, "attn_bwd: too many key blocks for one launch");
    a.total_blocks = (int)total;
    a.blocks_per_xcd = (a.total_blocks + 7) / 8;
    const dim3 grid((unsigned)(a.blocks_per_xcd * 8));
    if (x.causal) bwd_dkdv_kernel<T, D, true><<<grid, dim3(DKV_THREADS), 0, st>>>(a);
    else bwd_dkdv_kernel<T, D, false><<<grid, dim3(DKV_THREADS), 0, st>>>(a);
    if (int e = check_launch("qfa_attn_bwd (dk, dv)")) return e;
  }
  // dQ
  {
    constexpr int DQ_THREADS = DqShape<D>::THREADS, DQ_BLK = DqShape<D>::BLK;
    a.nblocks = (int)((x.Nq + DQ_BLK - 1) / DQ_BLK);
    // per head the kernel streams Kc, V and Kz^T (5 bytes per key and d): two to eight heads together, within
    // about 6 MB (pairs at N=4096, D=128, measured)
    const int64_t head_bytes_k = x.Nk * (int64_t)D * 5;
    a.group_log2 = 1;
    while (a.group_log2 < 3 && (head_bytes_k << (a.group_log2 + 1)) <= (6 << 20)) ++a.group_log2;
    const int64_t total = (int64_t)a.nblocks * BH;
    if (total > 0x3fffffffLL) return set_error(QFA_EUNSUPPORTED, "attn_bwd: too many query blocks for one launch");
    a.total_blocks = (int)total;
    a.blocks_per_xcd = (a.total_blocks + 7) / 8;
    const dim3 grid((unsigned)(a.blocks_per_xcd * 8));
    if (x.causal) bwd_dq_kernel<T, D, true><<<grid, dim3(DQ_THREADS), 0, st>>>(a);
    else bwd_dq_kernel<T, D, false><<<grid, dim3(DQ_THREADS), 0, st>>>(a);
    if (int e = check_launch("qfa_attn_bwd (dq)")) return e;
  }
  return 0;
}

int launch_bwd(const AttnArgs &x, hipStream_t st) {
  if (x.io_dtype == QFA_BF16) {
    if (x.D == 256) return launch_bwd_td<__bf16, 256>(x, st);
    if (x.D == 128) return launch_bwd_td<__bf16, 128>(x, st);
    if (x.D == 64) return launch_bwd_td<__bf16, 64>(x, st);
  } else if (x.io_dtype == QFA_F16) {
    if (x.D == 256) return launch_bwd_td<_Float16, 256>(x, st);
    if (x.D == 128) return launch_bwd_td<_Float16, 128>(x, st);
    if (x.D == 64) return launch_bwd_td<_Float16, 64>(x, st);
  } else {
    return set_error(QFA_EINVAL, "attn_bwd: io_dtype must be QFA_BF16 or QFA_F16");
  }
  return set_error(QFA_EUNSUPPORTED, "attn_bwd: head_dim must be 64, 128 or 256");
}

}  // namespace qfa
