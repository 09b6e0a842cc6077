// Backward kernels for gfx950: delta = rowsum(O o dO), then two MFMA kernels that recompute
// P = exp(S - LSE) from the INT8 codes exactly as the forward does.
//
//   dq kernel    one workgroup = 128 queries (32 per wave), loops over 64-key tiles.
//                S^T = Kc.Qc^T (INT8 MFMA), dP^T = V.dO^T, dS^T = P^T o (dP^T - delta),
//                dQ^T += Kz^T.(dS^T * sk)         with Kz = (Kc - zk) held as exact 16-bit floats
//   dkdv kernel  one workgroup = 128 keys (32 per wave), loops over 64-query tiles.
//                S = Qc.Kc^T (INT8 MFMA), dP = dO.V^T, dV^T += dO^T.P,
//                dK^T += Qz^T.(dS * sq)           with Qz = (Qc - zq)
// In both, the wave's own operand (queries resp. keys) stays in registers as the MFMA B operand
// for the whole loop and the streamed operand comes from LDS as the A operand.  The 32x32
// accumulator layout then leaves P / dS in registers exactly in the B-operand layout of the next
// product; the transposed LDS tiles (Kz^T, dO^T, Qz^T) are written in the matching permuted order.
// dQ is produced by its own kernel instead of atomics, so results are deterministic.
// (Kc - zk) and (Qc - zq) are integers in [-255, 255]: exact in bf16 and fp16, so the scales are
// folded into dS in fp32 and dequantization adds no rounding error.
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
  if (n < a.N && sub == 0) a.delta[bh * a.N + n] = s;
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
    if (D == 128) delta_kernel<__bf16, 128><<<grid, block, 0, st>>>(a);
    else delta_kernel<__bf16, 64><<<grid, block, 0, st>>>(a);
  } else {
    if (D == 128) delta_kernel<_Float16, 128><<<grid, block, 0, st>>>(a);
    else delta_kernel<_Float16, 64><<<grid, block, 0, st>>>(a);
  }
  return check_launch("qfa_bwd_delta");
}

// ------------------------------------------------------------------------------------------ shared
struct BwdArgs {
  const int8_t *qc; const float *sq; const int8_t *zq; const int32_t *rq;
  const int8_t *kc; const float *sk; const int8_t *zk; const int32_t *rk;
  const void *v; const void *dout; const float *lse; const float *delta;
  void *dq; void *dk; void *dv;
  int64_t H;
  int Nq, Nk;
  int64_t sqb, sqh, sqn, skb, skh, skn, svb, svh, svn;
  int64_t sdob, sdoh, sdon, sdqb, sdqh, sdqn, sdkb, sdkh, sdkn, sdvb, sdvh, sdvn;
  float sm_scale, sm_scale_log2;
  int nblocks;          // query blocks (dq) or key blocks (dkdv) per (b,h)
  int total_blocks, blocks_per_xcd;
};

constexpr int BWD_BLK = 128;   // rows owned by a workgroup
constexpr int BWD_TILE = 64;   // rows streamed per step

// position of streamed row r (0..63) inside a transposed LDS tile: the order in which the 32x32
// accumulator layout hands out rows to a lane (two runs of 4 per 16-row MFMA k-slice)
__device__ __forceinline__ int perm_pos4(int r4) {   // r4 = r / 4
  return 32 * (r4 / 8) + 16 * ((r4 / 4) % 2) + 8 * (r4 % 2) + 4 * ((r4 / 2) % 2);
}

// (code - zp) for the 8 codes in two dwords of 4 rows, as exact 16-bit floats, transposed:
// writes, for each of the 8 columns, the 4 rows as 8 bytes at dst + column * stride
template <typename T>
__device__ __forceinline__ void store_codes_transposed(const u32x2 (&c)[4], const float (&zp)[4], unsigned char *dst,
                                                       int stride) {
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    float f[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) f[r] = (float)(int)(int8_t)((c[r][e / 4] >> (8 * (e % 4))) & 0xff) - zp[r];
    u32x2 o;
    o[0] = pack2<T>(f[0], f[1]);
    o[1] = pack2<T>(f[2], f[3]);
    *reinterpret_cast<u32x2 *>(dst + e * stride) = o;
  }
}
// 4 rows x 8 columns of 16-bit floats (one 16-byte register per row), transposed the same way
__device__ __forceinline__ void store_16b_transposed(const u32x4 (&w)[4], unsigned char *dst, int stride) {
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    const int x = e / 2;
    u32x2 o;
    if (e % 2 == 0) {
      o[0] = (w[0][x] & 0xffffu) | (w[1][x] << 16);
      o[1] = (w[2][x] & 0xffffu) | (w[3][x] << 16);
    } else {
      o[0] = (w[0][x] >> 16) | (w[1][x] & 0xffff0000u);
      o[1] = (w[2][x] >> 16) | (w[3][x] & 0xffff0000u);
    }
    *reinterpret_cast<u32x2 *>(dst + e * stride) = o;
  }
}

template <int D> struct BwdSmem {
  static constexpr int CSTR = D + 16;                // int8 code rows
  static constexpr int RSTR = 2 * D + 16;            // row-major 16-bit rows
  static constexpr int TSTR = (BWD_TILE + 8) * 2;    // transposed 16-bit rows
  static constexpr int C_BYTES = BWD_TILE * CSTR;
  static constexpr int R_BYTES = BWD_TILE * RSTR;
  static constexpr int T_BYTES = D * TSTR;
};

// ------------------------------------------------------------------------------------------ dQ
template <typename T, int D, bool CAUSAL>
__global__ __launch_bounds__(256, 2) void bwd_dq_kernel(BwdArgs a) {
  typedef BwdSmem<D> SM;
  constexpr int KS = D / 32, DB = D / 32, KD = D / 16;
  constexpr int KCH = (BWD_TILE * D / 16) / 256;
  constexpr int VCH = (BWD_TILE * D / 8) / 256;
  constexpr int OFF_V = SM::C_BYTES, OFF_T = OFF_V + SM::R_BYTES, OFF_C = OFF_T + SM::T_BYTES;
  __shared__ __attribute__((aligned(16))) unsigned char smem[OFF_C + 3 * BWD_TILE * 4];

  const int L = blockIdx.x;
  const int vid = (L % 8) * a.blocks_per_xcd + (L / 8);
  if (vid >= a.total_blocks) return;
  const int bh = vid / a.nblocks;
  int mb = vid % a.nblocks;
  if (CAUSAL) mb = a.nblocks - 1 - mb;
  const int64_t b = bh / a.H, h = bh % a.H;
  const int m0 = mb * BWD_BLK;
  const int tid = threadIdx.x, wave = tid / 64, lane = tid % 64, lr = lane % 32, g = lane / 32;

  const int8_t *qc_bh = a.qc + b * a.sqb + h * a.sqh;
  const int8_t *kc_bh = a.kc + b * a.skb + h * a.skh;
  const T *v_bh = reinterpret_cast<const T *>(a.v) + b * a.svb + h * a.svh;
  const T *do_bh = reinterpret_cast<const T *>(a.dout) + b * a.sdob + h * a.sdoh;
  T *dq_bh = reinterpret_cast<T *>(a.dq) + b * a.sdqb + h * a.sdqh;
  const int64_t tq0 = (int64_t)bh * a.Nq, tk0 = (int64_t)bh * a.Nk;

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
  const float zqf = (float)a.zq[tq0 + qi_c];
  const float a_i = a.sq[tq0 + qi_c] * a.sm_scale_log2;
  const float nzq = -zqf;
  const float nc = -((float)a.rq[tq0 + qi_c] - (float)D * zqf);
  const float nlse2 = -a.lse[tq0 + qi_c] * kLog2e;
  const float delta_i = a.delta[tq0 + qi_c];
  const int q_first = m0 + wave * 32, q_last = q_first + 31;

  int kv_end = a.Nk;
  if (CAUSAL) kv_end = min(a.Nk, m0 + BWD_BLK);
  const int ntiles = (kv_end + BWD_TILE - 1) / BWD_TILE;

  const int t_r4 = tid % 16, t_dc = tid / 16;
  const bool t_active = t_dc < D / 8;
  const int t_pos = perm_pos4(t_r4);

  u32x4 kreg[KCH], vreg[VCH];
  u32x2 creg[4];
  float zreg[4];
  float cst[3];

  auto load_tile = [&](int t) {
    const int j0 = t * BWD_TILE;
#pragma unroll
    for (int i = 0; i < KCH; ++i) {
      const int c = tid + 256 * i, row = c / (D / 16), col = c % (D / 16);
      const int j = min(j0 + row, a.Nk - 1);
      kreg[i] = *reinterpret_cast<const u32x4 *>(kc_bh + (int64_t)j * a.skn + col * 16);
    }
#pragma unroll
    for (int i = 0; i < VCH; ++i) {
      const int c = tid + 256 * i, row = c / (D / 8), col = c % (D / 8);
      const int j = min(j0 + row, a.Nk - 1);
      vreg[i] = *reinterpret_cast<const u32x4 *>(v_bh + (int64_t)j * a.svn + col * 8);
    }
    if (t_active) {
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int j = min(j0 + 4 * t_r4 + r, a.Nk - 1);
        creg[r] = *reinterpret_cast<const u32x2 *>(kc_bh + (int64_t)j * a.skn + t_dc * 8);
        zreg[r] = (float)a.zk[tk0 + j];
      }
    }
    if (tid < BWD_TILE) {
      const int j = min(j0 + tid, a.Nk - 1);
      cst[0] = a.sk[tk0 + j];
      cst[1] = (float)a.rk[tk0 + j];
      cst[2] = (float)a.zk[tk0 + j];
    }
  };
  auto store_tile = [&]() {
#pragma unroll
    for (int i = 0; i < KCH; ++i) {
      const int c = tid + 256 * i, row = c / (D / 16), col = c % (D / 16);
      *reinterpret_cast<u32x4 *>(smem + row * SM::CSTR + col * 16) = kreg[i];
    }
#pragma unroll
    for (int i = 0; i < VCH; ++i) {
      const int c = tid + 256 * i, row = c / (D / 8), col = c % (D / 8);
      *reinterpret_cast<u32x4 *>(smem + OFF_V + row * SM::RSTR + col * 16) = vreg[i];
    }
    if (t_active)
      store_codes_transposed<T>(creg, zreg, smem + OFF_T + (t_dc * 8) * SM::TSTR + t_pos * 2, SM::TSTR);
    if (tid < BWD_TILE) {
      float *cs = reinterpret_cast<float *>(smem + OFF_C);
      cs[tid] = cst[0];
      cs[BWD_TILE + tid] = cst[1];
      cs[2 * BWD_TILE + tid] = cst[2];
    }
  };

  f32x16 dqacc[DB];
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int v = 0; v < 16; ++v) dqacc[db][v] = 0.f;

  load_tile(0);
  for (int t = 0; t < ntiles; ++t) {
    store_tile();
    __syncthreads();
    if (t + 1 < ntiles) load_tile(t + 1);

    const float *cs = reinterpret_cast<const float *>(smem + OFF_C);
    const int j0 = t * BWD_TILE;
#pragma unroll
    for (int nb = 0; nb < 2; ++nb) {
      const int jb = j0 + 32 * nb;
      const bool on = (jb < a.Nk) && (!CAUSAL || jb <= q_last);
      if (!on) continue;
      i32x16 acc;
      f32x16 dp;
#pragma unroll
      for (int v = 0; v < 16; ++v) { acc[v] = 0; dp[v] = 0.f; }
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        const i32x4 kf = *reinterpret_cast<const i32x4 *>(smem + (32 * nb + lr) * SM::CSTR + ks * 32 + g * 16);
        acc = mfma_i8(kf, qf[ks], acc);
      }
#pragma unroll
      for (int kd = 0; kd < KD; ++kd) {
        const u32x4 vf = *reinterpret_cast<const u32x4 *>(smem + OFF_V + (32 * nb + lr) * SM::RSTR + kd * 32 + g * 16);
        dp = mfma_16b<T>(vf, dof[kd], dp);
      }
      const bool need_mask = (CAUSAL && jb + 31 > q_first) || (jb + 32 > a.Nk);
      float ds[16];
#pragma unroll
      for (int aa = 0; aa < 4; ++aa) {
        const int jl = 32 * nb + 8 * aa + 4 * g;
        const f32x4 sk4 = *reinterpret_cast<const f32x4 *>(cs + jl);
        const f32x4 rk4 = *reinterpret_cast<const f32x4 *>(cs + BWD_TILE + jl);
        const f32x4 zk4 = *reinterpret_cast<const f32x4 *>(cs + 2 * BWD_TILE + jl);
#pragma unroll
        for (int bb = 0; bb < 4; ++bb) {
          const int v = 4 * aa + bb;
          float f = (float)acc[v];
          f = __builtin_fmaf(nzq, rk4[bb], f);
          f = __builtin_fmaf(nc, zk4[bb], f);
          float p = __builtin_amdgcn_exp2f(__builtin_fmaf(a_i, f * sk4[bb], nlse2));
          if (need_mask) {
            const int j = j0 + jl + bb;
            if ((CAUSAL && j > qi) || j >= a.Nk) p = 0.f;
          }
          ds[v] = p * (dp[v] - delta_i) * sk4[bb];
        }
      }
#pragma unroll
      for (int hh = 0; hh < 2; ++hh) {
        u32x4 dsf;
#pragma unroll
        for (int e = 0; e < 4; ++e) dsf[e] = pack2<T>(ds[8 * hh + 2 * e], ds[8 * hh + 2 * e + 1]);
#pragma unroll
        for (int db = 0; db < DB; ++db) {
          const u32x4 ktf = *reinterpret_cast<const u32x4 *>(smem + OFF_T + (32 * db + lr) * SM::TSTR +
                                                             (32 * nb + 16 * hh + 8 * g) * 2);
          dqacc[db] = mfma_16b<T>(ktf, dsf, dqacc[db]);
        }
      }
    }
    __syncthreads();
  }

  if (qi < a.Nq) {
    T *row = dq_bh + (int64_t)qi * a.sdqn;
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int aa = 0; aa < 4; ++aa) {
        u32x2 w;
        w[0] = pack2<T>(dqacc[db][4 * aa + 0] * a.sm_scale, dqacc[db][4 * aa + 1] * a.sm_scale);
        w[1] = pack2<T>(dqacc[db][4 * aa + 2] * a.sm_scale, dqacc[db][4 * aa + 3] * a.sm_scale);
        *reinterpret_cast<u32x2 *>(row + 32 * db + 8 * aa + 4 * g) = w;
      }
  }
}

// ------------------------------------------------------------------------------------------ dK, dV
template <typename T, int D, bool CAUSAL>
__global__ __launch_bounds__(256, 1) void bwd_dkdv_kernel(BwdArgs a) {
  typedef BwdSmem<D> SM;
  constexpr int KS = D / 32, DB = D / 32, KD = D / 16;
  constexpr int OFF_DO = SM::C_BYTES, OFF_DOT = OFF_DO + SM::R_BYTES, OFF_QT = OFF_DOT + SM::T_BYTES,
                OFF_C = OFF_QT + SM::T_BYTES;
  __shared__ __attribute__((aligned(16))) unsigned char smem[OFF_C + 5 * BWD_TILE * 4];

  const int L = blockIdx.x;
  const int vid = (L % 8) * a.blocks_per_xcd + (L / 8);
  if (vid >= a.total_blocks) return;
  const int bh = vid / a.nblocks;
  const int nbk = vid % a.nblocks;   // causal: early key blocks see the most queries and come first
  const int64_t b = bh / a.H, h = bh % a.H;
  const int n0 = nbk * BWD_BLK;
  const int tid = threadIdx.x, wave = tid / 64, lane = tid % 64, lr = lane % 32, g = lane / 32;

  const int8_t *qc_bh = a.qc + b * a.sqb + h * a.sqh;
  const int8_t *kc_bh = a.kc + b * a.skb + h * a.skh;
  const T *v_bh = reinterpret_cast<const T *>(a.v) + b * a.svb + h * a.svh;
  const T *do_bh = reinterpret_cast<const T *>(a.dout) + b * a.sdob + h * a.sdoh;
  T *dk_bh = reinterpret_cast<T *>(a.dk) + b * a.sdkb + h * a.sdkh;
  T *dv_bh = reinterpret_cast<T *>(a.dv) + b * a.sdvb + h * a.sdvh;
  const int64_t tq0 = (int64_t)bh * a.Nq, tk0 = (int64_t)bh * a.Nk;

  // ---- this lane's key
  const int kj = n0 + wave * 32 + lr;
  const int kj_c = kj < a.Nk ? kj : a.Nk - 1;
  i32x4 kf[KS];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks)
    kf[ks] = *reinterpret_cast<const i32x4 *>(kc_bh + (int64_t)kj_c * a.skn + ks * 32 + g * 16);
  u32x4 vf[KD];
#pragma unroll
  for (int kd = 0; kd < KD; ++kd)
    vf[kd] = *reinterpret_cast<const u32x4 *>(v_bh + (int64_t)kj_c * a.svn + kd * 16 + g * 8);
  const float zkf = (float)a.zk[tk0 + kj_c];
  const float sk_j = a.sk[tk0 + kj_c];
  const float nzk = -zkf;
  const float nck = -((float)a.rk[tk0 + kj_c] - (float)D * zkf);
  const int k_first = n0 + wave * 32, k_last = k_first + 31;

  const int it0 = CAUSAL ? n0 / BWD_TILE : 0;
  const int ntiles = (a.Nq + BWD_TILE - 1) / BWD_TILE;

  const int t_r4 = tid % 16, t_dc = tid / 16;
  const bool t_active = t_dc < D / 8;
  const int t_pos = perm_pos4(t_r4);

  u32x2 creg[4];
  u32x4 greg[4];
  float zreg[4];
  float cst[5];

  auto load_tile = [&](int t) {
    const int i0 = t * BWD_TILE;
    if (t_active) {
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int i = min(i0 + 4 * t_r4 + r, a.Nq - 1);
        creg[r] = *reinterpret_cast<const u32x2 *>(qc_bh + (int64_t)i * a.sqn + t_dc * 8);
        greg[r] = *reinterpret_cast<const u32x4 *>(do_bh + (int64_t)i * a.sdon + t_dc * 8);
        zreg[r] = (float)a.zq[tq0 + i];
      }
    }
    if (tid < BWD_TILE) {
      const int i = min(i0 + tid, a.Nq - 1);
      const float zq = (float)a.zq[tq0 + i];
      cst[0] = (float)a.rq[tq0 + i];
      cst[1] = zq;
      cst[2] = a.sq[tq0 + i] * a.sm_scale_log2;
      cst[3] = -a.lse[tq0 + i] * kLog2e;
      cst[4] = a.delta[tq0 + i];
    }
  };
  auto store_tile = [&]() {
    if (t_active) {
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        *reinterpret_cast<u32x2 *>(smem + (4 * t_r4 + r) * SM::CSTR + t_dc * 8) = creg[r];
        *reinterpret_cast<u32x4 *>(smem + OFF_DO + (4 * t_r4 + r) * SM::RSTR + t_dc * 16) = greg[r];
      }
      store_16b_transposed(greg, smem + OFF_DOT + (t_dc * 8) * SM::TSTR + t_pos * 2, SM::TSTR);
      store_codes_transposed<T>(creg, zreg, smem + OFF_QT + (t_dc * 8) * SM::TSTR + t_pos * 2, SM::TSTR);
    }
    if (tid < BWD_TILE) {
      float *cs = reinterpret_cast<float *>(smem + OFF_C);
#pragma unroll
      for (int x = 0; x < 5; ++x) cs[x * BWD_TILE + tid] = cst[x];
    }
  };

  f32x16 dkacc[DB], dvacc[DB];
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int v = 0; v < 16; ++v) { dkacc[db][v] = 0.f; dvacc[db][v] = 0.f; }

  if (it0 < ntiles) load_tile(it0);
  for (int t = it0; t < ntiles; ++t) {
    store_tile();
    __syncthreads();
    if (t + 1 < ntiles) load_tile(t + 1);

    const float *cs = reinterpret_cast<const float *>(smem + OFF_C);
    const int i0 = t * BWD_TILE;
#pragma unroll
    for (int mbk = 0; mbk < 2; ++mbk) {
      const int ib = i0 + 32 * mbk;
      const bool on = (ib < a.Nq) && (!CAUSAL || ib + 31 >= k_first);
      if (!on) continue;
      i32x16 acc;
      f32x16 dp;
#pragma unroll
      for (int v = 0; v < 16; ++v) { acc[v] = 0; dp[v] = 0.f; }
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        const i32x4 qfr = *reinterpret_cast<const i32x4 *>(smem + (32 * mbk + lr) * SM::CSTR + ks * 32 + g * 16);
        acc = mfma_i8(qfr, kf[ks], acc);
      }
#pragma unroll
      for (int kd = 0; kd < KD; ++kd) {
        const u32x4 gf = *reinterpret_cast<const u32x4 *>(smem + OFF_DO + (32 * mbk + lr) * SM::RSTR + kd * 32 + g * 16);
        dp = mfma_16b<T>(gf, vf[kd], dp);
      }
      const bool need_mask = (CAUSAL && ib < k_last) || (ib + 32 > a.Nq) || (k_last >= a.Nk);
      float pp[16], ds[16];
#pragma unroll
      for (int aa = 0; aa < 4; ++aa) {
        const int il = 32 * mbk + 8 * aa + 4 * g;
        const f32x4 rq4 = *reinterpret_cast<const f32x4 *>(cs + il);
        const f32x4 zq4 = *reinterpret_cast<const f32x4 *>(cs + BWD_TILE + il);
        const f32x4 a4 = *reinterpret_cast<const f32x4 *>(cs + 2 * BWD_TILE + il);
        const f32x4 nl4 = *reinterpret_cast<const f32x4 *>(cs + 3 * BWD_TILE + il);
        const f32x4 dl4 = *reinterpret_cast<const f32x4 *>(cs + 4 * BWD_TILE + il);
#pragma unroll
        for (int bb = 0; bb < 4; ++bb) {
          const int v = 4 * aa + bb;
          float f = (float)acc[v];
          f = __builtin_fmaf(nzk, rq4[bb], f);
          f = __builtin_fmaf(nck, zq4[bb], f);
          float p = __builtin_amdgcn_exp2f(__builtin_fmaf(a4[bb], f * sk_j, nl4[bb]));
          if (need_mask) {
            const int i = i0 + il + bb;
            if ((CAUSAL && kj > i) || i >= a.Nq || kj >= a.Nk) p = 0.f;
          }
          pp[v] = p;
          ds[v] = p * (dp[v] - dl4[bb]) * a4[bb];   // dS * sq * sm_scale * log2(e)
        }
      }
#pragma unroll
      for (int hh = 0; hh < 2; ++hh) {
        u32x4 pf, dsf;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          pf[e] = pack2<T>(pp[8 * hh + 2 * e], pp[8 * hh + 2 * e + 1]);
          dsf[e] = pack2<T>(ds[8 * hh + 2 * e], ds[8 * hh + 2 * e + 1]);
        }
#pragma unroll
        for (int db = 0; db < DB; ++db) {
          const int off = (32 * db + lr) * SM::TSTR + (32 * mbk + 16 * hh + 8 * g) * 2;
          const u32x4 gtf = *reinterpret_cast<const u32x4 *>(smem + OFF_DOT + off);
          dvacc[db] = mfma_16b<T>(gtf, pf, dvacc[db]);
          const u32x4 qtf = *reinterpret_cast<const u32x4 *>(smem + OFF_QT + off);
          dkacc[db] = mfma_16b<T>(qtf, dsf, dkacc[db]);
        }
      }
    }
    __syncthreads();
  }

  if (kj < a.Nk) {
    T *krow = dk_bh + (int64_t)kj * a.sdkn;
    T *vrow = dv_bh + (int64_t)kj * a.sdvn;
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int aa = 0; aa < 4; ++aa) {
        u32x2 w;
        w[0] = pack2<T>(dkacc[db][4 * aa + 0] * kLn2, dkacc[db][4 * aa + 1] * kLn2);
        w[1] = pack2<T>(dkacc[db][4 * aa + 2] * kLn2, dkacc[db][4 * aa + 3] * kLn2);
        *reinterpret_cast<u32x2 *>(krow + 32 * db + 8 * aa + 4 * g) = w;
        w[0] = pack2<T>(dvacc[db][4 * aa + 0], dvacc[db][4 * aa + 1]);
        w[1] = pack2<T>(dvacc[db][4 * aa + 2], dvacc[db][4 * aa + 3]);
        *reinterpret_cast<u32x2 *>(vrow + 32 * db + 8 * aa + 4 * g) = w;
      }
  }
}

template <typename T, int D> static int launch_bwd_td(const AttnArgs &x, hipStream_t st) {
  BwdArgs a;
  a.qc = x.qc; a.sq = x.sq; a.zq = x.zq; a.rq = x.rq; a.kc = x.kc; a.sk = x.sk; a.zk = x.zk; a.rk = x.rk;
  a.v = x.v; a.dout = x.dout; a.lse = x.lse; a.delta = x.delta; a.dq = x.dq; a.dk = x.dk; a.dv = x.dv;
  a.H = x.H; a.Nq = (int)x.Nq; a.Nk = (int)x.Nk;
  a.sqb = x.sqb; a.sqh = x.sqh; a.sqn = x.sqn; a.skb = x.skb; a.skh = x.skh; a.skn = x.skn;
  a.svb = x.svb; a.svh = x.svh; a.svn = x.svn;
  a.sdob = x.sdob; a.sdoh = x.sdoh; a.sdon = x.sdon; a.sdqb = x.sdqb; a.sdqh = x.sdqh; a.sdqn = x.sdqn;
  a.sdkb = x.sdkb; a.sdkh = x.sdkh; a.sdkn = x.sdkn; a.sdvb = x.sdvb; a.sdvh = x.sdvh; a.sdvn = x.sdvn;
  a.sm_scale = x.sm_scale; a.sm_scale_log2 = x.sm_scale * kLog2e;
  const dim3 block(256);
  // dK, dV
  {
    a.nblocks = (int)((x.Nk + BWD_BLK - 1) / BWD_BLK);
    const int64_t total = (int64_t)a.nblocks * x.B * x.H;
    if (total > 0x3fffffffLL) return set_error(QFA_EUNSUPPORTED, "attn_bwd: too many key blocks for one launch");
    a.total_blocks = (int)total;
    a.blocks_per_xcd = (a.total_blocks + 7) / 8;
    const dim3 grid((unsigned)(a.blocks_per_xcd * 8));
    if (x.causal) bwd_dkdv_kernel<T, D, true><<<grid, block, 0, st>>>(a);
    else bwd_dkdv_kernel<T, D, false><<<grid, block, 0, st>>>(a);
    if (int e = check_launch("qfa_attn_bwd (dk, dv)")) return e;
  }
  // dQ
  {
    a.nblocks = (int)((x.Nq + BWD_BLK - 1) / BWD_BLK);
    const int64_t total = (int64_t)a.nblocks * x.B * x.H;
    if (total > 0x3fffffffLL) return set_error(QFA_EUNSUPPORTED, "attn_bwd: too many query blocks for one launch");
    a.total_blocks = (int)total;
    a.blocks_per_xcd = (a.total_blocks + 7) / 8;
    const dim3 grid((unsigned)(a.blocks_per_xcd * 8));
    if (x.causal) bwd_dq_kernel<T, D, true><<<grid, block, 0, st>>>(a);
    else bwd_dq_kernel<T, D, false><<<grid, block, 0, st>>>(a);
    if (int e = check_launch("qfa_attn_bwd (dq)")) return e;
  }
  return 0;
}

int launch_bwd(const AttnArgs &x, hipStream_t st) {
  if (x.io_dtype == QFA_BF16) {
    if (x.D == 128) return launch_bwd_td<__bf16, 128>(x, st);
    if (x.D == 64) return launch_bwd_td<__bf16, 64>(x, st);
  } else if (x.io_dtype == QFA_F16) {
    if (x.D == 128) return launch_bwd_td<_Float16, 128>(x, st);
    if (x.D == 64) return launch_bwd_td<_Float16, 64>(x, st);
  } else {
    return set_error(QFA_EINVAL, "attn_bwd: io_dtype must be QFA_BF16 or QFA_F16");
  }
  return set_error(QFA_EUNSUPPORTED, "attn_bwd: head_dim must be 64 or 128");
}

}  // namespace qfa
