// Forward kernel: O = softmax(sm_scale * Q^ K^T) V with Q^, K^ given as per-token asymmetric
// INT8 codes (scale, zero point, row sum per token).  gfx950, wave64.
//
// Work split.  One workgroup = 4 waves = 128 query rows of one (batch, head); each wave owns
// 32 queries.  K (3 buffers) and V (2 buffers) stream through LDS in tiles of 64 keys: K and the
// per-key constants are resident one tile ahead of V because the score product runs ahead.
//
// Score tile.  Each wave computes S^T = Kc . Qc^T with v_mfma_i32_32x32x32_i8: the K rows come
// from LDS (A operand), the wave's 32 queries stay in registers for the whole kernel (B operand).
// In the 32x32 accumulator layout a lane then holds 16 keys of ONE query (column l%32), so the
// per-query softmax state (running max, sum, rescale factor) is lane-local, and the exponentiated
// scores, packed to 16-bit floats, already are the B operand of the second product
// O^T = V^T . P^T (v_mfma_f32_32x32x16_bf16/f16) without leaving registers.
//
// Zero points.  With integer codes,  sum_d (qc-zq)(kc-zk) = A - zq*rk - zk*(rq - D*zq), A the int32
// MFMA result and rq, rk the code row sums.  The correction is a rank-4 update with integer
// entries below 2^8 (rk and rq - D*zq split into base-128 digits), so it runs as ONE extra 16-bit
// MFMA on the converted accumulator instead of per-score VALU work; every product and partial sum
// is an integer below 2^24, hence exact in fp32.  Then one multiply by the key scale; the query
// scale, sm_scale and log2(e) are folded into the exp2 argument.
//
// The kernel is bound by softmax VALU work, not by MFMA, so the design goal is to keep the vector
// pipe busy and hide the matrix pipe under it:
//  * the running maximum is only moved (and O rescaled) when some row of the wave exceeds it by
//    more than 2^8 (any reference maximum gives the same O after the final division), so the
//    rescale is a rare branch instead of 64 multiplies per tile;
//  * row sums are taken over packed pairs with v_dot2;
//  * tiles without any masked score run a software-pipelined loop whose body is one straight
//    basic block per 32-key block: exp2/pack of block b, the P.V MFMAs of block b, the INT8 MFMAs
//    of block b+2 and the convert/correct/scale/max of block b+1 are independent of each other,
//    so MFMA and VALU instructions interleave; diagonal and ragged tiles run a simple masked loop.
//
// V is transposed on its way into LDS (Vt[d][key]) so a lane reads its 8 keys of one d as one
// 16-byte LDS load; keys are stored in the permuted order in which the S^T accumulator layout
// hands out P, so no shuffle is needed between the two products.
#include <type_traits>

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
constexpr float FWD_RESCALE_THRESHOLD = 8.0f;   // log2 units the running max may lag behind

template <int D> struct FwdSmem {
  static constexpr int KSTR = D + 16;            // bytes per K row (+16: conflict-free 16-byte reads)
  static constexpr int VSTR = (FWD_BN + 8) * 2;  // bytes per Vt row
  static constexpr int K_BYTES = FWD_BN * KSTR;
  static constexpr int V_BYTES = D * VSTR;
  static constexpr int C_BYTES = FWD_BN * 4 + FWD_BN * 8;  // key scale; correction digits (2 dwords/key)
  static constexpr int OFF_K = 0;                     // 3 buffers
  static constexpr int OFF_V = 3 * K_BYTES;           // 2 buffers
  static constexpr int OFF_C = OFF_V + 2 * V_BYTES;   // 3 buffers
  static constexpr int TOTAL = OFF_C + 3 * C_BYTES;
};

// integer n in [-32768, 32767] -> (128*floor(n/128), n mod 128) as a packed pair of 16-bit floats
template <typename T> __device__ __forceinline__ unsigned base128_pair(int n) {
  const int hi = n >> 7, lo = n & 127;
  return pack2<T>((float)(hi * 128), (float)lo);
}

// QK_ONLY is the measurement variant of the same kernel: identical loads, INT8 product, zero-point
// correction, scaling and running maximum, with the exponentials and the P.V product compiled out
// (it writes the scaled row maximum where the LSE would go and leaves O untouched).  It exists to
// time the QK^T stage by itself against the INT8 MFMA peak.
template <typename T, int D, bool CAUSAL, bool QK_ONLY = false>
__global__ __launch_bounds__(256, 2) void fwd_kernel(FwdArgs a) {
  typedef FwdSmem<D> SM;
  constexpr int KS = D / 32;   // int8 k-steps of 32
  constexpr int DB = D / 32;   // 32-row blocks of O^T
  constexpr int KCH = (FWD_BN * D / 16) / 256;   // 16-byte K chunks per thread (2 for D=128, 1 for D=64)
  __shared__ __attribute__((aligned(16))) unsigned char smem[SM::TOTAL];

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
  const int zq_i = (int)a.zq[tq0 + qi_c];
  const float a_i = a.sq[tq0 + qi_c] * a.sm_scale_log2;        // > 0
  // query side of the rank-4 correction: k-group 0 multiplies the two digits of rk by -zq,
  // k-group 1 multiplies zk (stored twice) by minus the two digits of c = rq - D*zq
  u32x4 corr_q = {0u, 0u, 0u, 0u};
  {
    const int c = a.rq[tq0 + qi_c] - D * zq_i;     // |c| <= 32640
    const int hi = c >> 7, lo = c & 127;
    corr_q[0] = g == 0 ? pack2<T>((float)(-zq_i), (float)(-zq_i)) : pack2<T>((float)(-128 * hi), (float)(-lo));
  }
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
  float c_sk;
  int c_rk, c_zk;

  auto load_k = [&](int t) {
    const int j0 = t * FWD_BN;
#pragma unroll
    for (int i = 0; i < KCH; ++i) {
      const int c = tid + 256 * i;
      const int row = c / (D / 16), col = c % (D / 16);
      const int j = min(j0 + row, a.Nk - 1);
      kreg[i] = *reinterpret_cast<const u32x4 *>(kc_bh + (int64_t)j * a.skn + col * 16);
    }
    if (tid < FWD_BN) {
      const int j = min(j0 + tid, a.Nk - 1);
      c_sk = a.sk[tk0 + j];
      c_rk = a.rk[tk0 + j];
      c_zk = (int)a.zk[tk0 + j];
    }
  };
  auto store_k = [&](int buf) {
    unsigned char *base = smem + SM::OFF_K + buf * SM::K_BYTES;
#pragma unroll
    for (int i = 0; i < KCH; ++i) {
      const int c = tid + 256 * i;
      const int row = c / (D / 16), col = c % (D / 16);
      *reinterpret_cast<u32x4 *>(base + row * SM::KSTR + col * 16) = kreg[i];
    }
    if (tid < FWD_BN) {
      unsigned char *cb = smem + SM::OFF_C + buf * SM::C_BYTES;
      reinterpret_cast<float *>(cb)[tid] = c_sk;
      u32x2 dg;
      dg[0] = base128_pair<T>(c_rk);                      // k-group 0: digits of rk
      dg[1] = pack2<T>((float)c_zk, (float)c_zk);         // k-group 1: zk, zk
      reinterpret_cast<u32x2 *>(cb + FWD_BN * 4)[tid] = dg;
    }
  };
  auto load_v = [&](int t) {
    const int j0 = t * FWD_BN;
    if (v_active) {
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int j = min(j0 + 4 * v_kv4 + r, a.Nk - 1);
        vreg[r] = *reinterpret_cast<const u32x4 *>(v_bh + (int64_t)j * a.svn + v_dc * 8);
      }
    }
  };
  auto store_v = [&](int buf) {
    if (v_active) {
      unsigned char *vt = smem + SM::OFF_V + buf * SM::V_BYTES;
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
  };
  // S^T block nb (32 keys) of the tile held in K buffer `buf`, for this wave's 32 queries
  auto qk_block = [&](int buf, int nb, i32x16 &s) {
    const unsigned char *ks_ = smem + SM::OFF_K + buf * SM::K_BYTES;
#pragma unroll
    for (int v = 0; v < 16; ++v) s[v] = 0;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const i32x4 kf = *reinterpret_cast<const i32x4 *>(ks_ + (32 * nb + lr) * SM::KSTR + ks * 32 + g * 16);
      s = mfma_i8(kf, qf[ks], s);
    }
  };

  f32x16 oacc[DB];
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int v = 0; v < 16; ++v) oacc[db][v] = 0.f;
  float m_ref = -INFINITY;   // reference maximum of u = score / a_i used in the exponent
  float nm = INFINITY;       // -a_i * m_ref
  float l_run = 0.f;         // this lane's share of the row sum

  // raw int32 block -> u = sk * (S + zero-point correction); returns the block maximum of the row
  auto prep = [&](int cbuf, int nb, const i32x16 &s, float (&u)[16], int j0, auto masked_tag) -> float {
    constexpr bool MASKED = decltype(masked_tag)::value;
    const unsigned char *cb = smem + SM::OFF_C + cbuf * SM::C_BYTES;
    const float *skp = reinterpret_cast<const float *>(cb);
    const unsigned *dgp = reinterpret_cast<const unsigned *>(cb + FWD_BN * 4);
    f32x16 f;
#pragma unroll
    for (int v = 0; v < 16; ++v) f[v] = (float)s[v];
    u32x4 corr_k = {dgp[2 * (32 * nb + lr) + g], 0u, 0u, 0u};
    f = mfma_16b<T>(corr_k, corr_q, f);
    float mt = -INFINITY;
#pragma unroll
    for (int aa = 0; aa < 4; ++aa) {
      const int jl = 32 * nb + 8 * aa + 4 * g;
      const f32x4 sk4 = *reinterpret_cast<const f32x4 *>(skp + jl);
#pragma unroll
      for (int bb = 0; bb < 4; ++bb) {
        float uu = f[4 * aa + bb] * sk4[bb];
        if (MASKED) {
          const int j = j0 + jl + bb;
          if ((CAUSAL && j > qi) || j >= a.Nk) uu = -INFINITY;
        }
        u[4 * aa + bb] = uu;
        mt = fmaxf(mt, uu);
      }
    }
    return fmaxf(mt, swap32_f(mt));
  };
  // move the reference maximum only when some row of the wave outgrew it by > 2^threshold
  auto rescale_if_needed = [&](float mt) {
    if (__builtin_amdgcn_ballot_w64(a_i * (mt - m_ref) > FWD_RESCALE_THRESHOLD) != 0) {
      const float m_new = fmaxf(m_ref, mt);
      const float alpha = __builtin_amdgcn_exp2f(a_i * (m_ref - m_new));
      m_ref = m_new;
      nm = -a_i * m_new;
      l_run *= alpha;
#pragma unroll
      for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int v = 0; v < 16; ++v) oacc[db][v] *= alpha;
    }
  };
  // p = exp2(a_i*u - a_i*m_ref), packed; row sum; O^T += V^T . P^T for the 32 keys of block nb
  auto exp_pv = [&](int vbuf, int nb, const float (&u)[16]) {
    if (QK_ONLY) {   // keep the scores alive without exponentials or MFMAs
      float s = 0.f;
#pragma unroll
      for (int v = 0; v < 16; ++v) s = fmaxf(s, u[v]);
      l_run = fmaxf(l_run, s);
      return;
    }
    const unsigned char *vt_ = smem + SM::OFF_V + vbuf * SM::V_BYTES;
#pragma unroll
    for (int hh = 0; hh < 2; ++hh) {
      u32x4 pf;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const float p0 = __builtin_amdgcn_exp2f(__builtin_fmaf(a_i, u[8 * hh + 2 * e], nm));
        const float p1 = __builtin_amdgcn_exp2f(__builtin_fmaf(a_i, u[8 * hh + 2 * e + 1], nm));
        pf[e] = pack2<T>(p0, p1);
        l_run = dot2_ones<T>(pf[e], l_run);   // sum of the rounded pair, fp32 accumulate
      }
#pragma unroll
      for (int db = 0; db < DB; ++db) {
        const u32x4 vf =
            *reinterpret_cast<const u32x4 *>(vt_ + (32 * db + lr) * SM::VSTR + (32 * nb + 16 * hh + 8 * g) * 2);
        oacc[db] = mfma_16b<T>(vf, pf, oacc[db]);
      }
    }
  };

  // ---- prologue: K(0), K(1) (with their constants) and V(0) resident
  load_k(0);
  load_v(0);
  store_k(0);
  store_v(0);
  if (ntiles > 1) {
    load_k(1);
    store_k(1);
  }
  __syncthreads();

  // tiles [0, t_hot) contain no masked score for this wave (wave-uniform)
  int t_hot = a.Nk / FWD_BN;
  if (CAUSAL) t_hot = min(t_hot, (q_first + 1) / FWD_BN);
  t_hot = min(t_hot, ntiles);

  int kb_cur = 0, kb_nxt = 1, kb_free = 2;   // K/constant buffers of tile t, t+1, and the one to refill
  int t = 0;
  {
    // ---- pipelined loop over unmasked tiles.  Entering tile t: u_a = prepared block 2t,
    // s_y = raw S of block 2t+1; the reference maximum already covers block 2t.
    float u_a[16], u_b[16];
    i32x16 s_x, s_y;
    if (t_hot > 0) {
      qk_block(0, 0, s_x);
      qk_block(0, 1, s_y);
      rescale_if_needed(prep(0, 0, s_x, u_a, 0, std::false_type{}));
    }
    for (; t < t_hot; ++t) {
      if (t + 2 < ntiles) load_k(t + 2);
      if (t + 1 < ntiles) load_v(t + 1);
      // block 2t: consume u_a; raw S(2t+2) -> s_x; prepare block 2t+1 from s_y
      qk_block(kb_nxt, 0, s_x);
      exp_pv(t & 1, 0, u_a);
      rescale_if_needed(prep(kb_cur, 1, s_y, u_b, 0, std::false_type{}));
      // block 2t+1: consume u_b; raw S(2t+3) -> s_y; prepare block 2t+2 from s_x (only a
      // candidate maximum if that block belongs to the unmasked range)
      qk_block(kb_nxt, 1, s_y);
      exp_pv(t & 1, 1, u_b);
      const float mt = prep(kb_nxt, 0, s_x, u_a, 0, std::false_type{});
      rescale_if_needed(t + 1 < t_hot ? mt : -INFINITY);

      if (t + 2 < ntiles) store_k(kb_free);
      if (t + 1 < ntiles) store_v((t + 1) & 1);
      const int tmp = kb_cur; kb_cur = kb_nxt; kb_nxt = kb_free; kb_free = tmp;
      __syncthreads();
    }
  }
  // ---- masked tiles (diagonal, ragged end): one block at a time, nothing carried between blocks
  for (; t < ntiles; ++t) {
    if (t + 2 < ntiles) load_k(t + 2);
    if (t + 1 < ntiles) load_v(t + 1);
    const int j0 = t * FWD_BN;
#pragma unroll
    for (int nb = 0; nb < 2; ++nb) {
      const int jb = j0 + 32 * nb;
      if ((CAUSAL && jb > q_last) || jb >= a.Nk) continue;   // wave-uniform: nothing to keep
      i32x16 s;
      float u[16];
      qk_block(kb_cur, nb, s);
      rescale_if_needed(prep(kb_cur, nb, s, u, j0, std::true_type{}));
      exp_pv(t & 1, nb, u);
    }
    if (t + 2 < ntiles) store_k(kb_free);
    if (t + 1 < ntiles) store_v((t + 1) & 1);
    const int tmp = kb_cur; kb_cur = kb_nxt; kb_nxt = kb_free; kb_free = tmp;
    __syncthreads();
  }

  // ---- epilogue: normalise, store O (lane holds 4 consecutive d per register quad) and LSE
  if (QK_ONLY) {
    if (qi < a.Nq && g == 0) a.lse[tq0 + qi] = a_i * fmaxf(m_ref, l_run);
    return;
  }
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
    if (g == 0) a.lse[tq0 + qi] = (a_i * m_ref + __log2f(l_tot)) * kLn2;
  }
}

template <typename T, int D> static int launch_fwd_td(const AttnArgs &x, hipStream_t st, bool qk_only) {
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
  if (qk_only) {
    if (x.causal) fwd_kernel<T, D, true, true><<<grid, block, 0, st>>>(a);
    else fwd_kernel<T, D, false, true><<<grid, block, 0, st>>>(a);
  } else {
    if (x.causal) fwd_kernel<T, D, true><<<grid, block, 0, st>>>(a);
    else fwd_kernel<T, D, false><<<grid, block, 0, st>>>(a);
  }
  return check_launch("qfa_attn_fwd");
}

int launch_fwd(const AttnArgs &x, hipStream_t st, bool qk_only) {
  if (x.io_dtype == QFA_BF16) {
    if (x.D == 128) return launch_fwd_td<__bf16, 128>(x, st, qk_only);
    if (x.D == 64) return launch_fwd_td<__bf16, 64>(x, st, qk_only);
  } else if (x.io_dtype == QFA_F16) {
    if (x.D == 128) return launch_fwd_td<_Float16, 128>(x, st, qk_only);
    if (x.D == 64) return launch_fwd_td<_Float16, 64>(x, st, qk_only);
  } else {
    return set_error(QFA_EINVAL, "attn_fwd: io_dtype must be QFA_BF16 or QFA_F16");
  }
  return set_error(QFA_EUNSUPPORTED, "attn_fwd: head_dim must be 64 or 128");
}

}  // namespace qfa
