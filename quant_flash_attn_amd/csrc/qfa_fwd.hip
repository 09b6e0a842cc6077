// Forward kernel: O = softmax(sm_scale * Q^ K^T) V with Q^, K^ given as per-token asymmetric
// INT8 codes (scale, zero point, row sum per token).  gfx950, wave64.
//
// Work split.  One workgroup = 4 waves = 128 query rows of one (batch, head); each wave owns
// 32 queries.  K/V stream through LDS in tiles of 64 keys, double buffered (global -> registers
// while the previous tile is being consumed, registers -> LDS afterwards, one barrier per tile).
//
// Score tile.  Each wave computes S^T = Kc . Qc^T with v_mfma_i32_32x32x32_i8: the K rows come
// from LDS (A operand), the wave's 32 queries stay in registers for the whole kernel (B operand).
// In the 32x32 accumulator layout a lane then holds 16 keys of ONE query (column l%32), so the
// per-query softmax state (running max, sum, rescale factor) is lane-local, and the exponentiated
// scores, packed to 16-bit floats, already are the B operand of the second product
// O^T = V^T . P^T (v_mfma_f32_32x32x16_bf16/f16) without leaving registers.
//
// Zero points.  With integer codes,  sum_d (qc-zq)(kc-zk) = A - zq*rk - zk*(rq - D*zq), A the int32
// MFMA result and rq, rk the code row sums.  The two corrections are applied as exact fp32 FMAs on
// the converted accumulator (every intermediate is an integer below 2^24), then one multiply by
// the key scale; the query scale, sm_scale and log2(e) are folded into the exp2 argument.
//
// V is transposed on its way into LDS (Vt[d][key]) so a lane reads its 8 keys of one d as one
// 16-byte LDS load; keys are stored in the permuted order in which the S^T accumulator layout
// hands out P, so no shuffle is needed between the two products.
#include "qfa_device.h"
#include "qfa_host.h"

namespace qfa {

struct FwdArgs {
  const int8_t *qc; const float *sq; const int8_t *zq; const int32_t *rq;
  const int8_t *kc; const float *sk; const int8_t *zk; const int32_t *rk;
  const void *v; void *o; float *lse;
  int64_t H;
  int Nq, Nk;
  int64_t sqb, sqh, sqn, skb, skh, skn, svb, svh, svn, sob, soh, son;
  float sm_scale_log2;   // sm_scale * log2(e)
  int mblocks;           // ceil(Nq / 128)
  int total_blocks;      // mblocks * B * H
  int blocks_per_xcd;    // ceil(total_blocks / 8)
};

constexpr int FWD_BM = 128;
constexpr int FWD_BN = 64;

template <int D> struct FwdSmem {
  static constexpr int KSTR = D + 16;            // bytes per K row (+16: conflict-free 16-byte reads)
  static constexpr int VSTR = (FWD_BN + 8) * 2;  // bytes per Vt row
  static constexpr int K_BYTES = FWD_BN * KSTR;
  static constexpr int V_BYTES = D * VSTR;
  static constexpr int C_BYTES = 3 * FWD_BN * 4;  // sk, float(rk), float(zk)
  static constexpr int BUF_BYTES = K_BYTES + V_BYTES + C_BYTES;
};

template <typename T, int D, bool CAUSAL>
__global__ __launch_bounds__(256, 2) void fwd_kernel(FwdArgs a) {
  typedef FwdSmem<D> SM;
  constexpr int KS = D / 32;   // int8 k-steps of 32
  constexpr int DB = D / 32;   // 32-row blocks of O^T
  constexpr int KCH = (FWD_BN * D / 16) / 256;   // 16-byte K chunks per thread (2 for D=128, 1 for D=64)
  __shared__ __attribute__((aligned(16))) unsigned char smem[2 * SM::BUF_BYTES];

  // ---- block -> (batch*head, query block); consecutive ids of one XCD share a head's K/V in its L2
  const int L = blockIdx.x;
  const int vid = (L % 8) * a.blocks_per_xcd + (L / 8);
  if (vid >= a.total_blocks) return;
  const int bh = vid / a.mblocks;
  int mb = vid % a.mblocks;
  if (CAUSAL) mb = a.mblocks - 1 - mb;   // longest rows first
  const int64_t b = bh / a.H, h = bh % a.H;
  const int m0 = mb * FWD_BM;

  const int tid = threadIdx.x;
  const int wave = tid / 64;
  const int lane = tid % 64;
  const int lr = lane % 32;   // row (A) / column (B, D) index inside a 32x32 MFMA block
  const int g = lane / 32;    // k-group

  const int8_t *qc_bh = a.qc + b * a.sqb + h * a.sqh;
  const int8_t *kc_bh = a.kc + b * a.skb + h * a.skh;
  const T *v_bh = reinterpret_cast<const T *>(a.v) + b * a.svb + h * a.svh;
  T *o_bh = reinterpret_cast<T *>(a.o) + b * a.sob + h * a.soh;
  const int64_t tq0 = (int64_t)bh * a.Nq;
  const int64_t tk0 = (int64_t)bh * a.Nk;

  // ---- this lane's query
  const int qi = m0 + wave * 32 + lr;
  const int qi_c = qi < a.Nq ? qi : a.Nq - 1;
  i32x4 qf[KS];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks)
    qf[ks] = *reinterpret_cast<const i32x4 *>(qc_bh + (int64_t)qi_c * a.sqn + ks * 32 + g * 16);
  const float zqf = (float)a.zq[tq0 + qi_c];
  const float a_i = a.sq[tq0 + qi_c] * a.sm_scale_log2;        // > 0
  const float nzq = -zqf;
  const float nc = -((float)a.rq[tq0 + qi_c] - (float)D * zqf);  // exact: |.| < 2^16
  const int q_first = m0 + wave * 32, q_last = q_first + 31;

  // ---- tile range
  int kv_end = a.Nk;
  if (CAUSAL) kv_end = min(a.Nk, m0 + FWD_BM);
  const int ntiles = (kv_end + FWD_BN - 1) / FWD_BN;

  // ---- loader roles
  const int v_kv4 = tid % 16;   // group of 4 consecutive keys
  const int v_dc = tid / 16;    // chunk of 8 consecutive d
  const bool v_active = v_dc < D / 8;
  const int v_pos = 32 * (v_kv4 / 8) + 16 * ((v_kv4 / 4) % 2) + 8 * (v_kv4 % 2) + 4 * ((v_kv4 / 2) % 2);

  u32x4 kreg[KCH];
  u32x4 vreg[4];
  float creg[3];

  auto load_tile = [&](int t) {
    const int j0 = t * FWD_BN;
#pragma unroll
    for (int i = 0; i < KCH; ++i) {
      const int c = tid + 256 * i;
      const int row = c / (D / 16), col = c % (D / 16);
      const int j = min(j0 + row, a.Nk - 1);
      kreg[i] = *reinterpret_cast<const u32x4 *>(kc_bh + (int64_t)j * a.skn + col * 16);
    }
    if (v_active) {
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int j = min(j0 + 4 * v_kv4 + r, a.Nk - 1);
        vreg[r] = *reinterpret_cast<const u32x4 *>(v_bh + (int64_t)j * a.svn + v_dc * 8);
      }
    }
    if (tid < FWD_BN) {
      const int j = min(j0 + tid, a.Nk - 1);
      creg[0] = a.sk[tk0 + j];
      creg[1] = (float)a.rk[tk0 + j];
      creg[2] = (float)a.zk[tk0 + j];
    }
  };
  auto store_tile = [&](int buf) {
    unsigned char *base = smem + buf * SM::BUF_BYTES;
#pragma unroll
    for (int i = 0; i < KCH; ++i) {
      const int c = tid + 256 * i;
      const int row = c / (D / 16), col = c % (D / 16);
      *reinterpret_cast<u32x4 *>(base + row * SM::KSTR + col * 16) = kreg[i];
    }
    if (v_active) {
      unsigned char *vt = base + SM::K_BYTES;
#pragma unroll
      for (int e = 0; e < 8; ++e) {   // d = 8*v_dc + e: gather the 4 keys of that d
        const int w = e / 2;
        u32x2 o;
        if (e % 2 == 0) {
          o[0] = (vreg[0][w] & 0xffffu) | (vreg[1][w] << 16);
          o[1] = (vreg[2][w] & 0xffffu) | (vreg[3][w] << 16);
        } else {
          o[0] = (vreg[0][w] >> 16) | (vreg[1][w] & 0xffff0000u);
          o[1] = (vreg[2][w] >> 16) | (vreg[3][w] & 0xffff0000u);
        }
        *reinterpret_cast<u32x2 *>(vt + (v_dc * 8 + e) * SM::VSTR + v_pos * 2) = o;
      }
    }
    if (tid < FWD_BN) {
      float *cs = reinterpret_cast<float *>(base + SM::K_BYTES + SM::V_BYTES);
      cs[tid] = creg[0];
      cs[FWD_BN + tid] = creg[1];
      cs[2 * FWD_BN + tid] = creg[2];
    }
  };

  f32x16 oacc[DB];
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int v = 0; v < 16; ++v) oacc[db][v] = 0.f;
  float m_run = -INFINITY;   // running max of u = score / a_i
  float l_run = 0.f;         // this lane's share of the row sum

  load_tile(0);
  store_tile(0);
  __syncthreads();

  for (int t = 0; t < ntiles; ++t) {
    const int buf = t & 1;
    if (t + 1 < ntiles) load_tile(t + 1);

    const unsigned char *base = smem + buf * SM::BUF_BYTES;
    const unsigned char *ks_ = base;
    const unsigned char *vt_ = base + SM::K_BYTES;
    const float *cs = reinterpret_cast<const float *>(base + SM::K_BYTES + SM::V_BYTES);
    const int j0 = t * FWD_BN;

    bool blk_on[2];
    float u[2][16];
    float mt = -INFINITY;
#pragma unroll
    for (int nb = 0; nb < 2; ++nb) {
      const int jb = j0 + 32 * nb;
      blk_on[nb] = (jb < a.Nk) && (!CAUSAL || jb <= q_last);   // wave-uniform
      if (!blk_on[nb]) continue;
      i32x16 acc;
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[v] = 0;
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        const i32x4 kf = *reinterpret_cast<const i32x4 *>(ks_ + (32 * nb + lr) * SM::KSTR + ks * 32 + g * 16);
        acc = mfma_i8(kf, qf[ks], acc);
      }
      const bool need_mask = (CAUSAL && jb + 31 > q_first) || (jb + 32 > a.Nk);   // wave-uniform
#pragma unroll
      for (int aa = 0; aa < 4; ++aa) {
        const int jl = 32 * nb + 8 * aa + 4 * g;
        const f32x4 sk4 = *reinterpret_cast<const f32x4 *>(cs + jl);
        const f32x4 rk4 = *reinterpret_cast<const f32x4 *>(cs + FWD_BN + jl);
        const f32x4 zk4 = *reinterpret_cast<const f32x4 *>(cs + 2 * FWD_BN + jl);
#pragma unroll
        for (int bb = 0; bb < 4; ++bb) {
          float f = (float)acc[4 * aa + bb];
          f = __builtin_fmaf(nzq, rk4[bb], f);
          f = __builtin_fmaf(nc, zk4[bb], f);
          float uu = f * sk4[bb];
          if (need_mask) {
            const int j = j0 + jl + bb;
            if ((CAUSAL && j > qi) || j >= a.Nk) uu = -INFINITY;
          }
          u[nb][4 * aa + bb] = uu;
          mt = fmaxf(mt, uu);
        }
      }
    }
    mt = fmaxf(mt, swap32_f(mt));
    const float m_new = fmaxf(m_run, mt);
    const float alpha = __builtin_amdgcn_exp2f(a_i * (m_run - m_new));
    const float nm = -a_i * m_new;
    m_run = m_new;
    l_run *= alpha;
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int v = 0; v < 16; ++v) oacc[db][v] *= alpha;

#pragma unroll
    for (int nb = 0; nb < 2; ++nb) {
      if (!blk_on[nb]) continue;
      float psum = 0.f;
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const float p = __builtin_amdgcn_exp2f(__builtin_fmaf(a_i, u[nb][v], nm));
        u[nb][v] = p;
        psum += p;
      }
      l_run += psum;
#pragma unroll
      for (int hh = 0; hh < 2; ++hh) {
        u32x4 pf;
#pragma unroll
        for (int e = 0; e < 4; ++e) pf[e] = pack2<T>(u[nb][8 * hh + 2 * e], u[nb][8 * hh + 2 * e + 1]);
#pragma unroll
        for (int db = 0; db < DB; ++db) {
          const u32x4 vf =
              *reinterpret_cast<const u32x4 *>(vt_ + (32 * db + lr) * SM::VSTR + (32 * nb + 16 * hh + 8 * g) * 2);
          oacc[db] = mfma_16b<T>(vf, pf, oacc[db]);
        }
      }
    }

    if (t + 1 < ntiles) store_tile(buf ^ 1);
    __syncthreads();
  }

  // ---- epilogue: normalise, store O (lane holds 4 consecutive d per register quad) and LSE
  const float l_tot = l_run + swap32_f(l_run);
  const float inv = 1.0f / l_tot;
  if (qi < a.Nq) {
    T *orow = o_bh + (int64_t)qi * a.son;
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int aa = 0; aa < 4; ++aa) {
        u32x2 w;
        w[0] = pack2<T>(oacc[db][4 * aa + 0] * inv, oacc[db][4 * aa + 1] * inv);
        w[1] = pack2<T>(oacc[db][4 * aa + 2] * inv, oacc[db][4 * aa + 3] * inv);
        *reinterpret_cast<u32x2 *>(orow + 32 * db + 8 * aa + 4 * g) = w;
      }
    if (g == 0) a.lse[tq0 + qi] = (a_i * m_run + __log2f(l_tot)) * kLn2;
  }
}

template <typename T, int D> static int launch_fwd_td(const AttnArgs &x, hipStream_t st) {
  FwdArgs a;
  a.qc = x.qc; a.sq = x.sq; a.zq = x.zq; a.rq = x.rq;
  a.kc = x.kc; a.sk = x.sk; a.zk = x.zk; a.rk = x.rk;
  a.v = x.v; a.o = x.o; a.lse = x.lse;
  a.H = x.H; a.Nq = (int)x.Nq; a.Nk = (int)x.Nk;
  a.sqb = x.sqb; a.sqh = x.sqh; a.sqn = x.sqn; a.skb = x.skb; a.skh = x.skh; a.skn = x.skn;
  a.svb = x.svb; a.svh = x.svh; a.svn = x.svn; a.sob = x.sob; a.soh = x.soh; a.son = x.son;
  a.sm_scale_log2 = x.sm_scale * kLog2e;
  a.mblocks = (int)((x.Nq + FWD_BM - 1) / FWD_BM);
  const int64_t total = (int64_t)a.mblocks * x.B * x.H;
  if (total > 0x3fffffffLL) return set_error(QFA_EUNSUPPORTED, "attn_fwd: too many query blocks for one launch");
  a.total_blocks = (int)total;
  a.blocks_per_xcd = (a.total_blocks + 7) / 8;
  const dim3 grid((unsigned)(a.blocks_per_xcd * 8)), block(256);
  if (x.causal) fwd_kernel<T, D, true><<<grid, block, 0, st>>>(a);
  else fwd_kernel<T, D, false><<<grid, block, 0, st>>>(a);
  return check_launch("qfa_attn_fwd");
}

int launch_fwd(const AttnArgs &x, hipStream_t st) {
  if (x.io_dtype == QFA_BF16) {
    if (x.D == 128) return launch_fwd_td<__bf16, 128>(x, st);
    if (x.D == 64) return launch_fwd_td<__bf16, 64>(x, st);
  } else if (x.io_dtype == QFA_F16) {
    if (x.D == 128) return launch_fwd_td<_Float16, 128>(x, st);
    if (x.D == 64) return launch_fwd_td<_Float16, 64>(x, st);
  } else {
    return set_error(QFA_EINVAL, "attn_fwd: io_dtype must be QFA_BF16 or QFA_F16");
  }
  return set_error(QFA_EUNSUPPORTED, "attn_fwd: head_dim must be 64 or 128");
}

}  // namespace qfa
