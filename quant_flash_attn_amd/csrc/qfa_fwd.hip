// Forward kernel: O = softmax(sm_scale * Q^ K^T) V with Q^, K^ given as per-token asymmetric
// INT8 codes (scale, zero point, row sum per token).  gfx950, wave64.
//
// Work split.  One workgroup = 4 waves = 128 query rows of one (batch, head) (8 waves per workgroup
// halve the tile copies per query but measured 9 % slower: the barrier then waits for the slowest of
// 8 waves); each wave owns
// 32 queries.  K, V and the per-key constants stream through LDS in tiles of 64 keys, three buffers each
// (tile t in buffer t % 3), copied by
// direct global->LDS loads (no staging registers, no address or repacking work on the vector
// pipe); K and the per-key constants are resident one tile ahead of V because the score product
// runs ahead.
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
// entries of at most 8 significant bits (rk and rq - D*zq split into two digits), so it runs as ONE extra 16-bit
// MFMA instead of per-score VALU work; every product and partial sum
// is an integer below 2^24, hence exact in fp32.  Then one multiply by the key scale; the query
// scale, sm_scale and log2(e) are folded into the exp2 argument.
//
// With two waves per SIMD (64 O accumulators per wave leave no room for a third at head_dim 128) every vector
// instruction takes about 4.5 cycles of issue and an MFMA about twice that, whatever else overlaps, and no pipe is
// saturated (matrix 52 %, vector 53 % busy at the headline size): the time is the length of a wave's instruction
// stream plus the latency two waves cannot cover.  So the design goal is the smallest number of instructions per score:
//  * the reference maximum is only moved (and O rescaled) when it has to be (any reference gives the
//    same O after the final division): the masked loop moves it when a row exceeds it by more than
//    2^8, the pipelined loop takes no maximum at all and watches the running sum of the probabilities
//    instead (one compare per 16 keys; see check_half), so the rescale is a rare branch instead of 64 multiplies
//    and 8 maxima per block;
//  * row sums are taken over packed pairs with v_dot2;
//  * the int32 -> fp32 conversion of the scores is done by the matrix pipe (see "biased accumulators" below);
//  * the hot loop is unrolled over three tiles, so that every LDS address in it is a loop-invariant register plus
//    an immediate offset;
//  * tiles without any masked score run a software-pipelined loop whose body is one straight
//    basic block per 32-key block: exp2/pack of block b, the P.V MFMAs of block b, the INT8 MFMAs
//    of block b+2 and the correct/scale of block b+1 are independent of each other,
//    so MFMA and VALU instructions interleave; ragged tiles run a simple masked loop, and so does the
//    causal diagonal except where the pipeline already holds its scores (see the end of the pipelined part).
//
// Biased accumulators.  The correction MFMA runs FIRST, from a zero accumulator, with one more product term that
// adds c0 = 1.5 * 2^23: its fp32 result c0 + corr lies in [2^23, 2^24), where consecutive floats are consecutive
// integers and the bit pattern is 0x4B000000 + (value - 2^23).  The INT8 MFMAs then accumulate A onto that BIT
// PATTERN (integer adds), which read as a float is c0 + corr + A = c0 + S exactly, as long as it stays inside the
// binade; a third small MFMA adds -c0 and leaves the integer score S as an fp32 number.  Sixteen v_cvt_f32_i32 per
// block become one MFMA.  The two range conditions (|corr| and |S| below 2^22, intermediate sums of the first
// MFMA below 2^24 in any order) are checked per query in the prologue from quantities the wave has anyway
// (|zq|, |rq - D zq| and sum_d |qc_d - zq|, bounded against the worst key); a wave with a query that could leave
// the window -- rows pinned at one end of the code range, e.g. all-positive rows -- runs the instance of the same
// loop that converts explicitly (2 % slower).
//
// Head dimensions 64, 128 and 256 are instances of the same code: three, two and one workgroup per CU.
//
// V lies in LDS as it does in memory ([key][d] rows, 64-byte quarters XOR-swizzled against bank
// conflicts) and is transposed on the way out: ds_read_b64_tr_b16 hands lane (d, k-group) four
// consecutive keys of its d, and two such reads give exactly the 8 keys whose probabilities the
// S^T accumulator layout left in that k-group's registers, so no shuffle is needed between the two
// products.
#include <type_traits>

#include "qfa_fwd_common.h"

namespace qfa {

template <typename X> struct is_static_int : std::false_type {};
template <int V> struct is_static_int<std::integral_constant<int, V>> : std::true_type {};
template <int V> using ic = std::integral_constant<int, V>;

// QK_ONLY is the measurement variant of the same kernel: identical K and constant loads, INT8 product, zero-point
// correction, scaling and a maximum over the scores, with the V copies, the exponentials and the P.V product compiled
// out (it writes the scaled row maximum where the LSE would go and leaves O untouched).  It exists to
// time the QK^T stage by itself against the INT8 MFMA peak.
template <typename T, int D, bool CAUSAL, bool QK_ONLY = false, int NW = FWD_WAVES>
__global__ __launch_bounds__(64 * NW, FwdSmem<D>::WG_PER_CU) void fwd_kernel(FwdArgs a) {
  constexpr int NT = 64 * NW;        // threads per workgroup
  constexpr int FWD_BM = 32 * NW;    // queries per workgroup
  typedef FwdSmem<D> SM;
  constexpr int KS = D / 32;   // int8 k-steps of 32
  constexpr int DB = D / 32;   // 32-row blocks of O^T
  // Biased accumulators (see the head of the file) up to head_dim 128.  At head_dim 256 a wave is alone on its SIMD
  // and the longer dependent chain (correction -> 8 INT8 products -> unbias) is not hidden by anybody: measured 35 %
  // slower there than converting explicitly.
  constexpr bool BIAS_POSSIBLE = D <= 128;
  __shared__ __attribute__((aligned(256))) unsigned char smem[SM::TOTAL];

  // ---- block -> (batch*head, query block); consecutive ids of one XCD share a head's K/V in its L2
  const int L = blockIdx.x;
  const int vid = (L % 8) * a.blocks_per_xcd + (L / 8);
  if (vid >= a.total_blocks) return;
  int bh = vid / a.mblocks;
  int mb = vid % a.mblocks;
  if (CAUSAL) {
    // Longest rows first, and a group of heads at a time: ids run over the query blocks of 2^group_log2
    // heads, cycling through them from the longest block down.  With one head after the other the last
    // head's long blocks start when the chip is already draining (10 % longer makespan in a list-scheduling
    // model of 32 blocks per head on 64 workgroup slots per XCD; measured 5 % at D=128, 10 % at D=64); the
    // launcher sizes the group so that its K and V stay within reach of an XCD's L2.
    const int gsz = 1 << a.group_log2;
    const int pb = bh >> a.group_log2 << a.group_log2;
    if (pb + gsz <= a.total_blocks / a.mblocks) {
      const int idx = (bh - pb) * a.mblocks + mb;
      bh = pb + (idx & (gsz - 1));
      mb = idx >> a.group_log2;
    }
    mb = a.mblocks - 1 - mb;
  }
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
  // Query side (B operand) of the correction product, 4 k-slots per k-group: k-group 0 multiplies the two digits of
  // rk by -zq and the constant 2^11 by 3*2^11 (= c0, the bias of the pipelined loop); k-group 1 multiplies zk
  // (stored twice) by minus the two digits of c = rq - D*zq.
  // Two digits of 7 bits each (|c| <= 32640) up to head_dim 128, of 8 bits at head_dim 256 (|c| <= 65280): either
  // way each digit, shifted into place, has at most 8 significant bits and is exact in the 16-bit type.
  constexpr int SH = D > 128 ? 8 : 7;
  const int c_i = a.rq[tq0 + qi_c] - D * zq_i;
  u32x2 corr_q;
  {
    const int hi = c_i >> SH, lo = c_i & ((1 << SH) - 1);
    corr_q[0] = g == 0 ? pack2<T>((float)(-zq_i), (float)(-zq_i)) : pack2<T>((float)(-(hi * (1 << SH))), (float)(-lo));
    corr_q[1] = g == 0 ? pack2<T>(6144.0f, 0.0f) : 0u;
  }
  // A operand that takes the bias out again: -2^11 in the slot that meets 3*2^11
  const u32x2 unbias_a = {0u, g == 0 ? pack2<T>(-2048.0f, 0.0f) : 0u};
  const int q_first = m0 + wave * 32, q_last = q_first + 31;

  // ---- may this wave's queries use biased accumulators (see the head of the file)?  For every key:
  //   |terms of the first MFMA| <= |zq| (128 D + 127) + 128 (|c| + 2 * 2^SH) =: tq   (|rk digit sum| <= 128 D + 127, |zk| <= 128)
  //   |S| <= 255 * sum_d |qc_d - zq| =: 255 mq
  // and both must stay below 2^22.
  // (at head_dim 64 both bounds hold for every possible row: 255 * 64 * 255 and 128 * 8319 + 128 * 16576 are below 2^22)
  constexpr bool BIAS_ALWAYS = D <= 64;
  bool bias_ok = true;
  if constexpr (!BIAS_ALWAYS && BIAS_POSSIBLE) {
    const unsigned zb = ((unsigned)(zq_i + 128) & 0xffu) * 0x01010101u;
    unsigned mq = 0;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
#pragma unroll
      for (int j = 0; j < 4; ++j) mq = __builtin_amdgcn_sad_u8((unsigned)qf[ks][j] ^ 0x80808080u, zb, mq);
    mq += (unsigned)__shfl_xor((int)mq, 32, 64);
    const unsigned tq = (unsigned)abs(zq_i) * (128u * D + 127u) + 128u * ((unsigned)abs(c_i) + (2u << SH));
    const bool ok = 255u * mq < (1u << 22) && tq < (1u << 22);
    bias_ok = __builtin_amdgcn_ballot_w64(!ok) == 0;
  }

  // ---- tile range
  int kv_end = a.Nk;
  // causal: query i keeps keys j <= i + coff, the mask aligned to the last key (coff = Nk - Nq >= 0; the rule
  // row >= col when Nq == Nk)
  const int coff = CAUSAL ? a.Nk - a.Nq : 0;
  if (CAUSAL) kv_end = min(a.Nk, m0 + FWD_BM + coff);
  const int ntiles = (kv_end + FWD_BN - 1) / FWD_BN;

  // ---- tile copies: K and V by direct loads, the per-key constants through registers
  typedef Swz<D> KSW;
  typedef SwzQuad<2 * D> VSW;
  float c_sk;
  int c_rk, c_zk;

  // Full tiles: one per-thread offset for all chunks (TileCopyU); ragged tiles (rows clamped to the
  // last key) take the generic path.
  TileCopyU<D, FWD_BN, NT, KSW> cp_k;
  TileCopyU<2 * D, FWD_BN, NT, VSW> cp_v;
  cp_k.init((unsigned)a.skn, tid);
  cp_v.init((unsigned)(a.svn * sizeof(T)), tid);

  // Full tiles are copied through buffer descriptors rebased to the tile's first row (scalar
  // arithmetic), so a copy costs one instruction per 16-byte chunk and thread; the per-key constant
  // vectors are read the same way, with exact bounds (keys past the end read as zero and are masked).
  const int wave_u = __builtin_amdgcn_readfirstlane(wave);
  const rsrc_t rs_sk = make_rsrc(a.sk + tk0, (unsigned)a.Nk * 4u);
  const rsrc_t rs_rk = make_rsrc(a.rk + tk0, (unsigned)a.Nk * 4u);
  const rsrc_t rs_zk = make_rsrc(a.zk + tk0, (unsigned)a.Nk);
  auto load_kc = [&](int t) {   // per-key constants of tile t -> registers
    if (tid < FWD_BN) {
      c_sk = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rs_sk, tid * 4, t * FWD_BN * 4, 0));
      c_rk = __builtin_amdgcn_raw_buffer_load_b32(rs_rk, tid * 4, t * FWD_BN * 4, 0);
      c_zk = (int)(signed char)__builtin_amdgcn_raw_buffer_load_b8(rs_zk, tid, t * FWD_BN, 0);
    }
  };
  auto load_k = [&](int t, int buf) {
    const int j0 = t * FWD_BN;
    unsigned char *dst = smem + SM::OFF_K + buf * SM::K_BYTES;
    if (j0 + FWD_BN <= a.Nk)
      cp_k.issue(reinterpret_cast<const unsigned char *>(kc_bh) + (int64_t)j0 * a.skn, dst, wave_u);
    else
      dma_rows<D, FWD_BN, NT, KSW>(reinterpret_cast<const unsigned char *>(kc_bh), a.skn, j0, a.Nk - 1, dst, tid);
    load_kc(t);
  };
  auto store_k = [&](int buf) {
    if (tid < FWD_BN) {
      unsigned char *cb = smem + SM::OFF_C + buf * SM::C_BYTES;
      reinterpret_cast<float *>(cb)[tid] = c_sk;
      // the A operand of the correction product as it is read: per k-group two dwords
      u32x4 dg = {0u, 0u, 0u, 0u};
      dg[0] = base128_pair<T>(c_rk);                      // k-group 0: digits of rk,
      dg[1] = pack2<T>(2048.0f, 0.0f);                    //            and the constant that meets 3*2^11 (the bias c0)
      dg[2] = pack2<T>((float)c_zk, (float)c_zk);         // k-group 1: zk, zk
      reinterpret_cast<u32x4 *>(cb + FWD_BN * 4)[tid] = dg;
    }
  };
  auto load_v = [&](int t, int buf) {
    if (QK_ONLY) return;   // the QK^T-stage variant multiplies nothing by V
    const int j0 = t * FWD_BN;
    unsigned char *dst = smem + SM::OFF_V + buf * SM::V_BYTES;
    const int64_t vstride = a.svn * (int64_t)sizeof(T);
    if (j0 + FWD_BN <= a.Nk)
      cp_v.issue(reinterpret_cast<const unsigned char *>(v_bh) + (int64_t)j0 * vstride, dst, wave_u);
    else
      dma_rows<2 * D, FWD_BN, NT, VSW>(reinterpret_cast<const unsigned char *>(v_bh), vstride, j0, a.Nk - 1, dst, tid);
  };
  // this lane's read offsets inside a tile (the swizzle terms only depend on the lane)
  const int k_swz = KSW::swz(lr);                                        // rows 32*nb + lr
  int kq[KS];                                                            // K fragment ks of the lane's row
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) kq[ks] = lr * SM::KSTR + (((2 * ks + g) ^ k_swz) << 4);
  const int v_row = (lane % 16) / 4;                                     // source row of the transposing read
  const int v_off = v_row * SM::VSTR + ((VSW::swz(v_row) + 2 * ((lane / 16) % 2) + (lane % 4) / 2) << 4) +
                    8 * (lane % 2);                                      // XOR with 64*db selects the d block
  unsigned vq[DB];                                                       // LDS address of the lane's V fragment of d block db
#pragma unroll
  for (int db = 0; db < DB; ++db) vq[db] = lds_addr(smem + SM::OFF_V) + 4 * g * SM::VSTR + (v_off ^ (64 * db));
  const int c_skq = 16 * g;             // key scales of the lane's k-group inside a group of 8 keys
  const int c_crq = (2 * lr + g) * 8;   // correction operand of (key lr, k-group g)
  // the constants of block (buf, nb): key scales of keys 8aa + 4g + {0..3}, correction operand of key lr
  auto sk_of = [&](auto buf, int nb, int aa) -> f32x4 {
    return *reinterpret_cast<const f32x4 *>(smem + SM::OFF_C + (int)buf * SM::C_BYTES + (32 * nb + 8 * aa) * 4 + c_skq);
  };
  auto corr_of = [&](auto buf, int nb) -> u32x2 {
    return *reinterpret_cast<const u32x2 *>(smem + SM::OFF_C + (int)buf * SM::C_BYTES + FWD_BN * 4 + 32 * nb * 16 + c_crq);
  };
  auto kfrag_of = [&](auto buf, int nb, int ks) -> i32x4 {
    return *reinterpret_cast<const i32x4 *>(smem + SM::OFF_K + (int)buf * SM::K_BYTES + 32 * nb * SM::KSTR + kq[ks]);
  };
  // S^T block nb (32 keys) of the tile held in K buffer `buf`, for this wave's 32 queries
  auto qk_block = [&](int buf, int nb, i32x16 &s) __attribute__((always_inline)) {
#pragma unroll
    for (int v = 0; v < 16; ++v) s[v] = 0;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) s = mfma_i8(kfrag_of(buf, nb, ks), qf[ks], s);
  };

  f32x16 oacc[DB];
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int v = 0; v < 16; ++v) oacc[db][v] = 0.f;
  float m_ref = -INFINITY;   // reference maximum of u = score / a_i used in the exponent
  float m_bound = -INFINITY;                        // m_ref + threshold / a_i
  const float thr_i = FWD_RESCALE_THRESHOLD / a_i;
  float nm = INFINITY;       // -a_i * m_ref
  float l_run = 0.f;         // this lane's share of the row sum

  // raw int32 block -> u = sk * (S + zero-point correction); returns the block maximum of the row
  auto prep = [&](int cbuf, int nb, const i32x16 &s, float (&u)[16], int j0, auto masked_tag)
                  __attribute__((always_inline)) -> float {
    constexpr bool MASKED = decltype(masked_tag)::value;
    f32x16 f;
#pragma unroll
    for (int v = 0; v < 16; ++v) f[v] = (float)s[v];
    // no bias here (this path also serves the rows that may not have one): the slot that meets the constant is zero
    f = mfma_16b_k8<T>(corr_of(cbuf, nb), u32x2{corr_q[0], 0u}, f);
    float mt = -INFINITY;
#pragma unroll
    for (int aa = 0; aa < 4; ++aa) {
      const int jl = 32 * nb + 8 * aa + 4 * g;
      const f32x4 sk4 = sk_of(cbuf, nb, aa);
#pragma unroll
      for (int bb = 0; bb < 4; ++bb) {
        float uu = f[4 * aa + bb] * sk4[bb];
        if (MASKED) {
          const int j = j0 + jl + bb;
          if ((CAUSAL && j > qi + coff) || j >= a.Nk) uu = -INFINITY;
        }
        u[4 * aa + bb] = uu;
        mt = fmaxf(mt, uu);
      }
    }
    return max_across_halves(mt);
  };
  // move the reference maximum only when some row of the wave outgrew it by > 2^threshold
  // (the test is one compare against m_ref + threshold / a_i, kept in m_bound: it sits at the end
  // of a dependent chain that nothing else in the wave can overlap)
  auto move_ref = [&](float mt) __attribute__((always_inline)) {
    {
      const float m_new = fmaxf(m_ref, mt);
      const float alpha = __builtin_amdgcn_exp2f(a_i * (m_ref - m_new));
      m_ref = m_new;
      m_bound = m_new + thr_i;
      nm = -a_i * m_new;
      l_run *= alpha;
#pragma unroll
      for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int v = 0; v < 16; ++v) oacc[db][v] *= alpha;
    }
  };
  auto rescale_if_needed = [&](float mt) __attribute__((always_inline)) {
    if (__builtin_amdgcn_ballot_w64(mt > m_bound) != 0) move_ref(mt);
  };
  // p = exp2(a_i*u - a_i*m_ref), packed; row sum; O^T += V^T . P^T for the 32 keys of block nb
  auto exp_pv = [&](int vbuf, int nb, const float (&u)[16]) __attribute__((always_inline)) {
    if (QK_ONLY) {   // keep the scores alive without exponentials or MFMAs
      float s = 0.f;
#pragma unroll
      for (int v = 0; v < 16; ++v) s = fmaxf(s, u[v]);
      l_run = fmaxf(l_run, s);
      return;
    }
    // keys 32nb + 16hh + 4g + {0..3} and those + 8: the order in which pf holds the probabilities.
    // The reads are issued behind the compiler's back (see lds_read_tr16_async) and waited for below.
    const unsigned voff = vbuf * SM::V_BYTES + 32 * nb * SM::VSTR;
#pragma unroll
    for (int hh = 0; hh < 2; ++hh) {
      u32x2 vr[2 * DB];
#pragma unroll
      for (int db = 0; db < DB; ++db) {
        const unsigned ad = vq[db] + voff + hh * (16 * SM::VSTR);
        vr[2 * db] = lds_read_tr16_async<0>(ad);
        vr[2 * db + 1] = lds_read_tr16_async<8 * SM::VSTR>(ad);
      }
      u32x4 pf;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const float p0 = __builtin_amdgcn_exp2f(__builtin_fmaf(a_i, u[8 * hh + 2 * e], nm));
        const float p1 = __builtin_amdgcn_exp2f(__builtin_fmaf(a_i, u[8 * hh + 2 * e + 1], nm));
        pf[e] = pack2<T>(p0, p1);
        l_run = dot2_ones<T>(pf[e], l_run);   // sum of the rounded pair, fp32 accumulate
      }
      lds_wait_async<0>(vr);
#pragma unroll
      for (int db = 0; db < DB; ++db)
        oacc[db] = mfma_16b<T>(u32x4{vr[2 * db][0], vr[2 * db][1], vr[2 * db + 1][0], vr[2 * db + 1][1]}, pf, oacc[db]);
    }
  };

  // ---- prologue: K(0), K(1) (with their constants) and V(0) resident
  load_k(0, 0);
  load_v(0, 0);
  store_k(0);
  if (ntiles > 1) {
    load_k(1, 1);
    store_k(1);
  }
  dma_wait();
  __syncthreads();

  // tiles [0, t_hot) contain no masked score for this wave (wave-uniform)
  int t_hot = a.Nk / FWD_BN;
  if (CAUSAL) t_hot = min(t_hot, (q_first + coff + 1) / FWD_BN);
  t_hot = min(t_hot, ntiles);

  int kb_cur = 0, kb_nxt = 1, kb_free = 2;   // buffers of tile t, t+1, and the one to refill: t % 3, (t+1) % 3, (t+2) % 3
  int t = 0;
  auto pipelined = [&](auto bias_tag) __attribute__((always_inline)) {
    constexpr bool BIAS = decltype(bias_tag)::value;
    // ---- pipelined loop over unmasked tiles, one straight-line body per 32-key block b:
    //   exp2/pack and P.V of block b | correction + INT8 product of block b+1 | unbias/scale of b+1,
    // with every LDS operand requested a phase (or a body) before the MFMA that consumes it and every MFMA
    // result read a phase after the MFMA was issued.  The
    // phases are fenced so that the requests stay where they are; inside a phase MFMA and VALU
    // instructions are independent and interleave.  A wave raises its issue priority for the phases that
    // hold MFMAs and drops it for the ones that wait and request, so that of the two waves of a SIMD the
    // one that can feed the matrix pipe goes first (2 % at the non-causal sizes, nothing at the causal ones).
    // Carried between bodies: u = prepared scores of block b, kf / ck = K fragments and correction operand of block b+1.
    float u[16];
    i32x4 kf[KS];
    u32x2 ck;
    // buffer indices are either ints or integral constants (the loop unrolled over three tiles): with constants
    // every address below is a loop-invariant register plus an immediate
    auto k_frags = [&](auto buf, int nb) {
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) kf[ks] = kfrag_of(buf, nb, ks);
      ck = corr_of(buf, nb);
    };
    // V fragments of keys 32nb + 16hh + 4g + {0..3} and those + 8 (the order in which pf holds the
    // probabilities), requested without the compiler's knowledge: pair every call with lds_wait_async
    auto v_frags = [&](auto vbuf, auto nb_tag, auto hh_tag, u32x2 (&vr)[2 * DB]) {
      constexpr int ROW0 = (32 * decltype(nb_tag)::value + 16 * decltype(hh_tag)::value) * SM::VSTR;
      if constexpr (is_static_int<decltype(vbuf)>::value && 2 * SM::V_BYTES + 56 * SM::VSTR < 65536) {
        constexpr int IMM = decltype(vbuf)::value * SM::V_BYTES + ROW0;
#pragma unroll
        for (int db = 0; db < DB; ++db) {
          vr[2 * db] = lds_read_tr16_async<IMM>(vq[db]);
          vr[2 * db + 1] = lds_read_tr16_async<IMM + 8 * SM::VSTR>(vq[db]);
        }
      } else {
#pragma unroll
        for (int db = 0; db < DB; ++db) {
          const unsigned ad = vq[db] + (int)vbuf * SM::V_BYTES;
          vr[2 * db] = lds_read_tr16_async<ROW0>(ad);
          vr[2 * db + 1] = lds_read_tr16_async<ROW0 + 8 * SM::VSTR>(ad);
        }
      }
    };
    // lnew = l_run + the 8 probabilities (the running sum continues in a second register, so that l_run is still
    // there if the probabilities have to be formed again)
    auto exp_half = [&](int hh, u32x4 &pf, float &lnew) {
      float l = l_run;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const float p0 = __builtin_amdgcn_exp2f(__builtin_fmaf(a_i, u[8 * hh + 2 * e], nm));
        const float p1 = __builtin_amdgcn_exp2f(__builtin_fmaf(a_i, u[8 * hh + 2 * e + 1], nm));
        pf[e] = pack2<T>(p0, p1);
        l = e == 0 ? dot2_ones_keep<T>(pf[e], l) : dot2_ones<T>(pf[e], l);   // sum of the rounded pair, fp32 accumulate
      }
      lnew = l;
    };
    // The pipelined loop takes no running maximum.  The probabilities of 16 keys are formed against the
    // current reference and the running sum is looked at before they reach the P.V MFMAs: only if some lane's
    // sum left the range below (scores outgrew the reference by about 2^60, or overflowed) is the
    // maximum of the block taken, the reference moved (O and the row sum rescaled) and the 16
    // probabilities formed again.  Any reference gives the same O after the final division.  The reference
    // moves at least far enough to bring the sum so far back to order one (a sum that crept up to the limit
    // through many terms is not brought down by the maximum of the current block alone).
    constexpr float SUM_LIMIT = 0x1p60f;
    auto check_half = [&](int hh, u32x4 &pf, float &lnew) {
      if (__builtin_expect(__builtin_amdgcn_ballot_w64(!(lnew <= SUM_LIMIT)) != 0, 0)) {
        float mt = m_ref + __log2f(fmaxf(l_run, 1.0f)) / a_i;
#pragma unroll
        for (int v = 8 * hh; v < 16; ++v) mt = fmaxf(mt, u[v]);   // first half: the whole block
        move_ref(max_across_halves(mt));
        exp_half(hh, pf, lnew);
      }
      l_run = lnew;
    };
    // one body: P.V of V block (vbuf, NB) with the scores in u; scores of the next block from kf / ck, scaled with the
    // key scales of block (cbuf, CNB); then kf / ck are refilled from block (kbuf, KNB).
    // `copy(i)`, i = 0..2, is called between phases: the steady loop issues chunks of the next
    // tiles' copies there, so that the memory pipe sees a few requests at a time instead of a burst per tile
    auto body = [&](auto vbuf, auto nb_tag, auto cbuf, auto cnb_tag, auto kbuf, auto knb_tag, auto &&copy)
                    __attribute__((always_inline)) {
      static_assert(DB == 8 || DB == 4 || DB == 2, "fragment arrays are sized for head_dim 256, 128 or 64");
      constexpr int CNB = decltype(cnb_tag)::value, KNB = decltype(knb_tag)::value;
      u32x2 vr0[2 * DB], vr1[2 * DB];
      u32x4 pf0, pf1;
      const auto NB = nb_tag;
      // The K fragments were requested a body ago.  The compiler's counted wait for them must come HERE,
      // before the V requests it does not know of: in front of the INT8 MFMAs it would cover those too
      // (LDS returns in order) and the matrix pipe would idle for a full LDS round trip per block.
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) asm volatile("" : "+v"(kf[ks]));
      asm volatile("" : "+v"(ck));
      if (!QK_ONLY) v_frags(vbuf, NB, ic<0>{}, vr0);
      __builtin_amdgcn_sched_barrier(0);
      __builtin_amdgcn_s_setprio(1);
      // zero-point correction plus bias first (exact: an integer in [2^23, 2^24)), then the INT8 product of block b+1
      // accumulated onto its bit pattern, under the exponentials of the first 16 keys of block b
      i32x16 s;
      if constexpr (BIAS) {
        f32x16 y;
#pragma unroll
        for (int v = 0; v < 16; ++v) y[v] = 0.f;
        y = mfma_16b_k8<T>(ck, corr_q, y);
        s = __builtin_bit_cast(i32x16, y);
      } else {
#pragma unroll
        for (int v = 0; v < 16; ++v) s[v] = 0;
      }
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) s = mfma_i8(kf[ks], qf[ks], s);
      float l0, l1;
      if (!QK_ONLY) exp_half(0, pf0, l0);
      __builtin_amdgcn_sched_barrier(0);
      __builtin_amdgcn_s_setprio(0);
      copy(ic<0>{});
      if (!QK_ONLY) {
        check_half(0, pf0, l0);
        v_frags(vbuf, NB, ic<1>{}, vr1);
        lds_wait_async<(2 * DB < 15 ? 2 * DB : 15)>(vr0);   // the 2*DB requests just made may still be in flight (the counter holds 15)
      }
      f32x4 sk4[4];
#pragma unroll
      for (int aa = 0; aa < 4; ++aa) sk4[aa] = sk_of(cbuf, CNB, aa);
      __builtin_amdgcn_sched_barrier(0);
      // The MFMA that takes the bias out of the next block's scores, and P.V of the first 16 keys under the
      // exponentials of the second 16.  The unbias MFMA has no side effect, so instruction selection is free to place it
      // anywhere in the phase whatever the fence below says: it ends up behind the four P.V products, and its result is
      // still there before the next phase scales it.  Pinned to the head of the phase (an empty asm on f) the kernel
      // measured 0.6 % slower at all sizes.
      __builtin_amdgcn_s_setprio(1);
      f32x16 f;
      if constexpr (BIAS) {
        f = mfma_16b_k8<T>(unbias_a, corr_q, __builtin_bit_cast(f32x16, s));
        __builtin_amdgcn_sched_barrier(0);
      }
      if (!QK_ONLY) {
#pragma unroll
        for (int db = 0; db < DB; ++db)
          oacc[db] = mfma_16b<T>(u32x4{vr0[2 * db][0], vr0[2 * db][1], vr0[2 * db + 1][0], vr0[2 * db + 1][1]}, pf0,
                                 oacc[db]);
        exp_half(1, pf1, l1);
      } else {
        float sm = 0.f;
#pragma unroll
        for (int v = 0; v < 16; ++v) sm = fmaxf(sm, u[v]);
        l_run = fmaxf(l_run, sm);
      }
      if constexpr (!BIAS) {
        // explicit conversion, then the correction product (its query side without the bias slot)
#pragma unroll
        for (int v = 0; v < 16; ++v) f[v] = (float)s[v];
        __builtin_amdgcn_sched_barrier(0);
        f = mfma_16b_k8<T>(ck, u32x2{corr_q[0], 0u}, f);
      }
      __builtin_amdgcn_sched_barrier(0);
      __builtin_amdgcn_s_setprio(0);
      if (!QK_ONLY) {
        check_half(1, pf1, l1);
        lds_wait_async<0>(vr1);   // everything requested so far was requested a phase ago
      }
      copy(ic<1>{});
      k_frags(kbuf, KNB);
      __builtin_amdgcn_sched_barrier(0);
      // P.V of the second 16 keys under the scaling of the next block's scores
      __builtin_amdgcn_s_setprio(1);
      if (!QK_ONLY) {
#pragma unroll
        for (int db = 0; db < DB; ++db)
          oacc[db] = mfma_16b<T>(u32x4{vr1[2 * db][0], vr1[2 * db][1], vr1[2 * db + 1][0], vr1[2 * db + 1][1]}, pf1,
                                 oacc[db]);
      }
#pragma unroll
      for (int aa = 0; aa < 4; ++aa)
#pragma unroll
        for (int bb = 0; bb < 4; ++bb) u[4 * aa + bb] = f[4 * aa + bb] * sk4[aa][bb];
      __builtin_amdgcn_sched_barrier(0);
      __builtin_amdgcn_s_setprio(0);
      copy(ic<2>{});
    };

    {   // block 0 prepared, fragments of block 1 in flight
      i32x16 s0;
      qk_block(0, 0, s0);
      float u0[16];
      rescale_if_needed(prep(0, 0, s0, u0, 0, std::false_type{}));
#pragma unroll
      for (int v = 0; v < 16; ++v) u[v] = u0[v];
      k_frags(0, 1);
    }
    auto no_copy = [](auto) {};
    // steady state (tile t in buffers t % 3 = b0, b1 and b2 the next two): K(t+2) and V(t+1) are full tiles; their
    // chunks (K first, then V) go out two at a time between the phases of the tile's first body, so that the last
    // of them has the whole second body to land before the wait at the end of the tile (2 % at the causal headline
    // size against one chunk per phase over both bodies; all six at once, or three and three, are slower again)
    auto steady_tile = [&](auto b0, auto b1, auto b2, int tt) __attribute__((always_inline)) {
      load_kc(tt + 2);
      const rsrc_t rs_k =
          make_rsrc(reinterpret_cast<const unsigned char *>(kc_bh) + (int64_t)(tt + 2) * FWD_BN * a.skn, 0x7fffffffu);
      const rsrc_t rs_v = make_rsrc(
          reinterpret_cast<const unsigned char *>(v_bh) + (int64_t)(tt + 1) * FWD_BN * a.svn * (int64_t)sizeof(T), 0x7fffffffu);
      unsigned char *kd = smem + SM::OFF_K + (int)b2 * SM::K_BYTES, *vd = smem + SM::OFF_V + (int)b1 * SM::V_BYTES;
      constexpr int KCH = decltype(cp_k)::N, VCH = decltype(cp_v)::N;
      auto chunk = [&](int i) {   // i is a compile-time constant at every call site
        if (i < KCH) cp_k.issue_one(rs_k, kd, wave_u, i);
        else if (i < KCH + VCH && !QK_ONLY) cp_v.issue_one(rs_v, vd, wave_u, i - KCH);
      };
      constexpr int PER = (KCH + VCH + 2) / 3;   // chunks per slot: 2 at head_dim 128, 4 at 256
      body(b0, ic<0>{}, b0, ic<1>{}, b1, ic<0>{}, [&](auto i) {
#pragma unroll
        for (int c = 0; c < PER; ++c) chunk(PER * decltype(i)::value + c);
      });
      body(b0, ic<1>{}, b1, ic<0>{}, b1, ic<1>{}, no_copy);
      store_k((int)b2);
      dma_wait();
      __syncthreads();
    };
    {
      // tiles [0, t_steady) are unmasked for this wave, and their copies (two tiles ahead) are full tiles
      const int t_steady = min(t_hot, min(ntiles - 2, a.Nk / FWD_BN - 2));
      if constexpr (D <= 128 && !QK_ONLY) {
        // three tiles per trip with constant buffer indices
        for (; t + 3 <= t_steady; t += 3) {
          steady_tile(ic<0>{}, ic<1>{}, ic<2>{}, t);
          steady_tile(ic<1>{}, ic<2>{}, ic<0>{}, t + 1);
          steady_tile(ic<2>{}, ic<0>{}, ic<1>{}, t + 2);
        }
      } else {
        // head_dim 256: one tile per trip (the unrolled loop is three times 1 400 instructions there, and the V
        // offsets exceed the immediate field anyway)
        for (; t < t_steady; ++t) {
          steady_tile(kb_cur, kb_nxt, kb_free, t);
          const int tmp = kb_cur; kb_cur = kb_nxt; kb_nxt = kb_free; kb_free = tmp;
        }
      }
    }
    // the rest of the unmasked tiles (at most two of the steady kind, then the ones whose copies are ragged or
    // missing), with run-time buffer indices (kb_cur == t % 3 here)
    for (; t < t_hot; ++t) {
      if (t + 2 < ntiles) load_k(t + 2, kb_free);
      if (t + 1 < ntiles) load_v(t + 1, kb_nxt);
      body(kb_cur, ic<0>{}, kb_cur, ic<1>{}, kb_nxt, ic<0>{}, no_copy);
      body(kb_cur, ic<1>{}, kb_nxt, ic<0>{}, kb_nxt, ic<1>{}, no_copy);
      if (t + 2 < ntiles) store_k(kb_free);
      const int tmp = kb_cur; kb_cur = kb_nxt; kb_nxt = kb_free; kb_free = tmp;
      dma_wait();
      __syncthreads();
    }
    // ---- the wave's diagonal tile, as far as the pipeline has it already.  When the mask sits on a 32-key boundary
    // (always with Nq == Nk) the tile holds one block cut by the diagonal, before it at most one block that is fully
    // visible, behind it only invisible ones.  The scores of the tile's first block are in u, prepared by the last
    // body; a visible first block goes through one more body, which also prepares the diagonal block.  The diagonal
    // block then only needs the mask, the maximum and the P.V step: no score product is formed twice and the visible
    // block keeps the pipelined pace (the generic loop below took 2 900 cycles per block where this takes 1 600).
    if (!QK_ONLY && CAUSAL && D <= 128 && t < ntiles && coff % 32 == 0 && t == (q_first + coff + 1) / FWD_BN &&
        (t + 1) * FWD_BN <= a.Nk) {
      if (t + 2 < ntiles) load_k(t + 2, kb_free);
      if (t + 1 < ntiles) load_v(t + 1, kb_nxt);
      const int j0 = t * FWD_BN;
      const int nb_d = (q_first + coff - j0) / 32;   // 0 or 1, wave-uniform: the block that holds the diagonal
      if (nb_d == 1) body(kb_cur, ic<0>{}, kb_cur, ic<1>{}, kb_nxt, ic<0>{}, no_copy);
      float mt = -INFINITY;
#pragma unroll
      for (int aa = 0; aa < 4; ++aa)
#pragma unroll
        for (int bb = 0; bb < 4; ++bb) {
          const int j = j0 + 32 * nb_d + 8 * aa + 4 * g + bb;
          if (j > qi + coff) u[4 * aa + bb] = -INFINITY;
          mt = fmaxf(mt, u[4 * aa + bb]);
        }
      rescale_if_needed(max_across_halves(mt));
      exp_pv(kb_cur, nb_d, u);
      if (t + 2 < ntiles) store_k(kb_free);
      const int tmp = kb_cur; kb_cur = kb_nxt; kb_nxt = kb_free; kb_free = tmp;
      dma_wait();
      __syncthreads();
      ++t;
    }
  };
  // Two instances of the pipelined part: with biased accumulators for the waves whose queries allow them, with the
  // explicit conversion for the others (rows pinned at an end of the code range; all-positive rows are the common case)
  if (t_hot > 0) {
    if constexpr (BIAS_ALWAYS) {
      pipelined(std::true_type{});
    } else if constexpr (BIAS_POSSIBLE) {
      if (bias_ok) pipelined(std::true_type{});
      else pipelined(std::false_type{});
    } else {
      pipelined(std::false_type{});
    }
  }
  // ---- masked tiles (diagonal, ragged end): one block at a time, nothing carried between blocks
  for (; t < ntiles; ++t) {
    if (t + 2 < ntiles) load_k(t + 2, kb_free);
    if (t + 1 < ntiles) load_v(t + 1, kb_nxt);
    const int j0 = t * FWD_BN;
#pragma unroll
    for (int nb = 0; nb < 2; ++nb) {
      const int jb = j0 + 32 * nb;
      if ((CAUSAL && jb > q_last + coff) || jb >= a.Nk) continue;   // wave-uniform: nothing to keep
      i32x16 s;
      float u[16];
      qk_block(kb_cur, nb, s);
      rescale_if_needed(prep(kb_cur, nb, s, u, j0, std::true_type{}));
      exp_pv(kb_cur, nb, u);
    }
    if (t + 2 < ntiles) store_k(kb_free);
    const int tmp = kb_cur; kb_cur = kb_nxt; kb_nxt = kb_free; kb_free = tmp;
    dma_wait();
    __syncthreads();
  }

  // ---- epilogue: normalise, store O (as whole rows, through LDS) and LSE
  if (QK_ONLY) {
    if (qi < a.Nq && g == 0) a.lse[tq0 + qi] = a_i * fmaxf(m_ref, l_run);
    return;
  }
  const float l_tot = l_run + swap32_f(l_run);
  const float inv = 1.0f / l_tot;
  // O leaves as whole rows through LDS (all tile buffers are free after the last barrier; every wave takes 32 * 2D
  // bytes at the start of the K area)
  static_assert(SM::OFF_K + FWD_WAVES * 32 * 2 * D <= SM::TOTAL, "output staging fits the tile buffers");
  store_tile_rows<T, D>(oacc, inv, smem + SM::OFF_K + wave * (32 * 2 * D), o_bh, a.son, m0 + wave * 32, a.Nq, lane);
  if (qi < a.Nq && g == 0) a.lse[tq0 + qi] = (a_i * m_ref + __log2f(l_tot)) * kLn2;
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
  constexpr int FWD_BM = 32 * FWD_WAVES;
  a.mblocks = (int)((x.Nq + FWD_BM - 1) / FWD_BM);
  const int64_t total = (int64_t)a.mblocks * x.B * x.H;
  if (total > 0x3fffffffLL) return set_error(QFA_EUNSUPPORTED, "attn_fwd: too many query blocks for one launch");
  a.total_blocks = (int)total;
  a.blocks_per_xcd = (a.total_blocks + 7) / 8;
  // heads dispatched together (causal): as many as keep K (1 byte) and V (2 bytes) within about 6 MB --
  // one and a half times an XCD's L2, what measured best -- between 2 and 8
  const int64_t head_bytes = x.Nk * (int64_t)D * 3;
  a.group_log2 = 1;
  while (a.group_log2 < 3 && (head_bytes << (a.group_log2 + 1)) <= (6 << 20)) ++a.group_log2;
  const dim3 grid((unsigned)(a.blocks_per_xcd * 8)), block(64 * FWD_WAVES);
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
    if (x.D == 256) return launch_fwd_td<__bf16, 256>(x, st, qk_only);
    if (x.D == 128) return launch_fwd_td<__bf16, 128>(x, st, qk_only);
    if (x.D == 64) return launch_fwd_td<__bf16, 64>(x, st, qk_only);
  } else if (x.io_dtype == QFA_F16) {
    if (x.D == 256) return launch_fwd_td<_Float16, 256>(x, st, qk_only);
    if (x.D == 128) return launch_fwd_td<_Float16, 128>(x, st, qk_only);
    if (x.D == 64) return launch_fwd_td<_Float16, 64>(x, st, qk_only);
  } else {
    return set_error(QFA_EINVAL, "attn_fwd: io_dtype must be QFA_BF16 or QFA_F16");
  }
  return set_error(QFA_EUNSUPPORTED, "attn_fwd: head_dim must be 64, 128 or 256");
}

}  // namespace qfa
