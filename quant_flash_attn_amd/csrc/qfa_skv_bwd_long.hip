// Backward of the shared-KV attention for query blocks of any length, in two kernels (the fused
// one-pass kernel of qfa_skv_bwd.hip keeps a (batch, head)'s whole dQ in registers and is limited to
// 32 queries).  Same mathematics (quant_flash_attn.py:104-166):
//     P = exp(sm_scale * Q KV^T - LSE),   dP = dO KV^T,   dS = sm_scale * P o (dP - delta),
//     dQ = dS KV,   dKV = P^T dO + dS^T Q,   delta = rowsum(O o dO)
//
// skv_dq_kernel   one workgroup per block of 16 queries, built like the forward: the 32-key tiles are
//                 dealt to the four waves, streamed through private LDS rings, S^T and dP^T share the
//                 expanded code operands, dS * scale_j is the operand of dQ^T += C^T (dS*scale)^T, the
//                 four partial dQ are summed at the end.  LSE is known, so there is no running maximum.
// skv_dkv_kernel  one workgroup per 128 keys of a (batch, head): every wave owns ONE 32-key tile for the
//                 whole kernel (its code operands expanded once into registers, its dKV^T accumulators in
//                 registers) and the workgroup walks over the query blocks of 32, whose Q / dO / O rows
//                 arrive in a double-buffered LDS area by direct global->LDS loads.  Every (tile, query
//                 block) pair is visited once; each dKV row is written once, as whole 128-byte lines.
//                 At D = 256 the accumulators of a tile do not fit one wave: two waves share a tile, each
//                 keeping 128 of the 256 columns (both compute S and dP), a workgroup covers 64 keys and
//                 the row area is single-buffered.
// Both recompute delta from O and dO (no workspace), S and dP are computed in both kernels.
#include <type_traits>

#include "qfa_host.h"
#include "qfa_skv_common.h"

namespace qfa {

struct SkvBwdLongArgs {
  const _Float16 *q, *o, *dout;
  const int8_t *codes; const void *scale; const int8_t *zp;
  const float *lse;
  _Float16 *dq, *dkv;          // 16-bit outputs: binary16, or bfloat16 when grad_bf16 is set
  const float *grad_scale;     // nullable device scalar: dq and dkv are multiplied by it before rounding
  int grad_bf16;
  int64_t H;
  int Nq, Nk, BH, qblocks, kchunks, cpw;   // cpw: key chunks per workgroup of the dKV kernel
  int64_t sqb, sqh, sqn, scb, sch, scn, sob, soh, son, sdob, sdoh, sdon, sdqb, sdqh, sdqn, sdkb, sdkh, sdkn;
  float sm_scale, sm_scale_log2;
};

// ------------------------------------------------------------------------------------------ dQ

template <typename S, int D> __global__ __launch_bounds__(256, 2) void skv_dq_kernel(SkvBwdLongArgs a) {
  typedef SwzSkv<D> KSW;
  typedef TileCopy<D, SKV_TILE, 64, KSW> Copy;
  constexpr int KS = D / 32, DB = D / 16, OPS = Copy::N + 2;
  constexpr int SKVQ_NBUF = D == 256 ? 2 : 3;   // ring depth per wave (8 KB tiles at D = 256)
  constexpr int K_BYTES = SKV_TILE * D, SLOT = K_BYTES + 2 * SKV_TILE * 4, WAVE = SKVQ_NBUF * SLOT;
  constexpr int MG = 16 * D;   // floats of one partial dQ^T [D][16]
  static_assert(3 * MG * 4 <= 4 * WAVE, "the merge area overlays the rings");
  __shared__ __attribute__((aligned(16))) unsigned char smem[4 * WAVE];

  // query blocks of one (batch, head) get ids that differ by 8: same XCD, shared L2 copy of the codes
  const int bh = (int)(blockIdx.x / (8 * a.qblocks)) * 8 + (int)(blockIdx.x % 8);
  const int qb = (int)(blockIdx.x / 8) % a.qblocks;
  if (bh >= a.BH) return;
  const int64_t b = bh / a.H, h = bh % a.H;
  const int tid = threadIdx.x, lane = tid % 64, q16 = lane % 16, G = lane / 16;
  const int wave = __builtin_amdgcn_readfirstlane(tid / 64);
  const int wave_off = wave * WAVE;

  const unsigned char *codes_bh = reinterpret_cast<const unsigned char *>(a.codes + b * a.scb + h * a.sch);
  const int64_t tk0 = (int64_t)bh * a.Nk, tq0 = (int64_t)bh * a.Nq;
  const int ntiles = (a.Nk + SKV_TILE - 1) / SKV_TILE;
  const int my_tiles = ntiles > wave ? (ntiles - wave + 3) / 4 : 0;

  Copy cp;
  cp.init((unsigned)a.scn, lane);
  auto issue = [&](int i, int slot_idx) {
    skv_issue_tile<S, D>(cp, smem + wave_off + slot_idx * SLOT, codes_bh, a.scale, a.zp, tk0, wave + 4 * i, a.Nk, a.scn, lane);
  };
  auto scale_of = [](unsigned w) -> float {
    return std::is_same<S, float>::value ? __builtin_bit_cast(float, w) : lo_to_f32<_Float16>(w);
  };
  const float osc = a.grad_scale ? *a.grad_scale : 1.0f;
  auto pack_out = [&](float x, float y) -> unsigned {
    return a.grad_bf16 ? pack2<__bf16>(x * osc, y * osc) : pack2<_Float16>(x * osc, y * osc);
  };
#pragma unroll
  for (int i = 0; i < SKVQ_NBUF - 1; ++i)
    if (i < my_tiles) issue(i, i);

  // ---- this lane's query and dO row as B operands (k-step m, k-group G: d = 64(m/2) + 16G + 8(m%2) + {0..7}),
  //      their sums, delta and LSE
  const int qi = 16 * qb + q16;
  const bool q_ok = qi < a.Nq;
  const int qi_c = q_ok ? qi : a.Nq - 1;
  const _Float16 *qrow = a.q + b * a.sqb + h * a.sqh + (int64_t)qi_c * a.sqn;
  const _Float16 *orow = a.o + b * a.sob + h * a.soh + (int64_t)qi_c * a.son;
  const _Float16 *drow = a.dout + b * a.sdob + h * a.sdoh + (int64_t)qi_c * a.sdon;
  u32x4 qf[KS], dof[KS];
  float rq = 0.f, rd = 0.f, delta = 0.f;
#pragma unroll
  for (int m = 0; m < KS; ++m) {
    const int d0 = 64 * (m / 2) + 16 * G + 8 * (m % 2);
    qf[m] = *reinterpret_cast<const u32x4 *>(qrow + d0);
    dof[m] = *reinterpret_cast<const u32x4 *>(drow + d0);
    const u32x4 ov = *reinterpret_cast<const u32x4 *>(orow + d0);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const unsigned qw = qf[m][e], dw = dof[m][e], ow = ov[e];
      const float d0f = lo_to_f32<_Float16>(dw), d1f = hi_to_f32<_Float16>(dw);
      rq += lo_to_f32<_Float16>(qw) + hi_to_f32<_Float16>(qw);
      rd += d0f + d1f;
      delta += lo_to_f32<_Float16>(ow) * d0f + hi_to_f32<_Float16>(ow) * d1f;
    }
  }
#pragma unroll
  for (int m = 16; m < 64; m *= 2) {
    rq += __shfl_xor(rq, m, 64);
    rd += __shfl_xor(rd, m, 64);
    delta += __shfl_xor(delta, m, 64);
  }
  const bool big = offset_needs_x32(fmaxf(fabsf(rq), fabsf(rd)));
  u32x4 corr_q = {0u, 0u, 0u, 0u}, corr_do = {0u, 0u, 0u, 0u};
  if (G == 0) {
    const u32x2 cq2 = offset_query_operand(rq, big), cd2 = offset_query_operand(rd, big);
    corr_q[0] = cq2[0];
    corr_q[1] = cq2[1];
    corr_do[0] = cd2[0];
    corr_do[1] = cd2[1];
  }
  const float a_s = a.sm_scale_log2;
  const float nlse2 = q_ok ? -a.lse[tq0 + qi] * kLog2e : -INFINITY;   // padding rows: p = 0

  int k_off[2];
#pragma unroll
  for (int rb = 0; rb < 2; ++rb) k_off[rb] = (16 * rb + q16) * D + ((G ^ KSW::swz(16 * rb + q16)) << 4);
  int vt_off;
  {
    const int s = lane % 16, j = s / 2;
    const int key = 16 * (j / 4) + 4 * G + j % 4;
    vt_off = key * D + (KSW::swz(key) << 4) + 8 * (s % 2);
  }
  const unsigned lds0 = lds_addr(smem);

  f32x4 acc[DB];
#pragma unroll
  for (int db = 0; db < DB; ++db) acc[db] = f32x4{0.f, 0.f, 0.f, 0.f};
  float w_run = 0.f;

  auto tile = [&](int i, int slot_idx) {
    const int slot_off = wave_off + slot_idx * SLOT;
    const unsigned char *slot = smem + slot_off;
    const unsigned *skp = reinterpret_cast<const unsigned *>(slot + K_BYTES);
    const unsigned *zpp = skp + SKV_TILE;
    const int krem = a.Nk - (wave + 4 * i) * SKV_TILE;   // keys of this tile that exist (>= 32: all)
    const unsigned z_a[2] = {zpp[q16], zpp[16 + q16]};
    // (per-block read addresses are re-formed from these every tile: one XOR each instead of registers
    // held across the loop)
    int vt = vt_off, ko[2] = {k_off[0], k_off[1]};
    asm volatile("" : "+v"(vt), "+v"(ko[0]), "+v"(ko[1]));
    constexpr int VG = DB < 8 ? DB : 8;   // transposed fragments in groups of 8 blocks, the first one now
    u32x2 vr[VG];
#pragma unroll
    for (int db = 0; db < VG; ++db) vr[db] = lds_read_tr8_async(lds0 + slot_off + (vt ^ (db << 4)));
    // ---- S^T and dP^T from the same expanded code operands
    f32x4 f[2], gq[2];
#pragma unroll
    for (int rb = 0; rb < 2; ++rb) {
      f[rb] = f32x4{0.f, 0.f, 0.f, 0.f};
      gq[rb] = f32x4{0.f, 0.f, 0.f, 0.f};
      u32x4 kw[(KS + 1) / 2];
#pragma unroll
      for (int mm = 0; mm < (KS + 1) / 2; ++mm)
        kw[mm] = *reinterpret_cast<const u32x4 *>(slot + (ko[rb] ^ ((4 * mm) << 4)));
#pragma unroll
      for (int m = 0; m < KS; ++m) {
        const u32x4 ca = expand_codes(kw[m / 2][2 * (m % 2)], kw[m / 2][2 * (m % 2) + 1]);
        f[rb] = mfma_h16(ca, qf[m], f[rb]);
        gq[rb] = mfma_h16(ca, dof[m], gq[rb]);
      }
      u32x4 corr_k = {0u, 0u, 0u, 0u};
      if (G == 0) {
        const u32x2 ck2 = offset_key_operand(z_a[rb], big);
        corr_k[0] = ck2[0];
        corr_k[1] = ck2[1];
      }
      f[rb] = mfma_h16(corr_k, corr_q, f[rb]);
      gq[rb] = mfma_h16(corr_k, corr_do, gq[rb]);
    }
    // ---- p, ds, x = ds * scale_j as binary16 (keys 16rb + 4G + v), offset term
    u32x4 xf;
#pragma unroll
    for (int rb = 0; rb < 2; ++rb) {
      const u32x4 sk4 = *reinterpret_cast<const u32x4 *>(skp + 16 * rb + 4 * G);
      const u32x4 zk4 = *reinterpret_cast<const u32x4 *>(zpp + 16 * rb + 4 * G);
      float x[4];
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        const float sk = scale_of(sk4[v]);
        float p = __builtin_amdgcn_exp2f(__builtin_fmaf(a_s * sk, f[rb][v], nlse2));
        if (16 * rb + 4 * G + v >= krem) p = 0.f;
        x[v] = a.sm_scale * p * (gq[rb][v] * sk - delta) * sk;
      }
#pragma unroll
      for (int e = 0; e < 2; ++e) {
        const unsigned xx = pack_h2(x[2 * e], x[2 * e + 1]);
        xf[2 * rb + e] = xx;
        const unsigned cpair = magic_zp_pair(zk4[2 * e], zk4[2 * e + 1]);
        w_run = __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2, xx), __builtin_bit_cast(f16x2, cpair), w_run, false);
      }
    }
    // ---- dQ^T += (1152 + codes)^T . x^T
#pragma unroll
    for (int g0 = 0; g0 < DB; g0 += VG) {
      lds_wait_all();
      u32x2 now[VG];
#pragma unroll
      for (int db = 0; db < VG; ++db) now[db] = tie(vr[db]);
      if (g0 + VG < DB) {
#pragma unroll
        for (int db = 0; db < VG; ++db) vr[db] = lds_read_tr8_async(lds0 + slot_off + (vt ^ ((g0 + VG + db) << 4)));
      }
#pragma unroll
      for (int db = 0; db < VG; ++db) acc[g0 + db] = mfma_h16(expand_codes(now[db][0], now[db][1]), xf, acc[g0 + db]);
    }
  };

  int cur = 0, nxt = SKVQ_NBUF - 1;
  for (int i = 0; i < my_tiles; ++i) {
    if (i + SKVQ_NBUF - 1 < my_tiles) {
      issue(i + SKVQ_NBUF - 1, nxt);
      asm volatile("s_waitcnt vmcnt(%0)" ::"n"((SKVQ_NBUF - 1) * OPS) : "memory");
    } else {
      dma_wait();
    }
    tile(i, cur);
    cur = cur + 1 == SKVQ_NBUF ? 0 : cur + 1;
    nxt = nxt + 1 == SKVQ_NBUF ? 0 : nxt + 1;
  }

  float w_tot = w_run + __shfl_xor(w_run, 16, 64);
  w_tot += __shfl_xor(w_tot, 32, 64);
  __syncthreads();
  float *mg = reinterpret_cast<float *>(smem);
  if (wave > 0) {
    float *dst = mg + (wave - 1) * MG;
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int v = 0; v < 4; ++v) dst[(16 * db + 4 * G + v) * 16 + q16] = acc[db][v] - w_tot;
  }
  __syncthreads();
  if (wave == 0 && q_ok) {
    _Float16 *out = a.dq + b * a.sdqb + h * a.sdqh + (int64_t)qi * a.sdqn;
#pragma unroll
    for (int db = 0; db < DB; ++db) {
      float r[4];
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        const int d = 16 * db + 4 * G + v;
        r[v] = acc[db][v] - w_tot + mg[d * 16 + q16] + mg[MG + d * 16 + q16] + mg[2 * MG + d * 16 + q16];
      }
      u32x2 o2;
      o2[0] = pack_out(r[0], r[1]);
      o2[1] = pack_out(r[2], r[3]);
      *reinterpret_cast<u32x2 *>(out + 16 * db + 4 * G) = o2;
    }
  }
}

// ------------------------------------------------------------------------------------------ dKV
// Chunk swizzle of the binary16 Q / dO / O rows in LDS (see row_swizzle in qfa_skv_bwd.hip): distinct for 16
// consecutive rows at one chunk index, whole 32-byte pairs apart for 4 consecutive rows.
template <int D> struct RowSwz {
  static constexpr int CPR = D / 8;
  static __device__ __forceinline__ int swz(int i) { return (2 * (i % 4) + (i / 4) % 2 + 8 * ((i / 8) % 2)) % CPR; }
};

template <int D> struct SkvDkvSmem {
  static constexpr int DS = D == 256 ? 2 : 1;                    // waves sharing one tile (each keeps D / DS columns of dKV)
  static constexpr int NRB = D == 256 ? 1 : 2;                   // row buffers
  static constexpr bool O_IN_LDS = NRB == 2;                     // one buffer: O (needed for delta only) is read from memory
  static constexpr int SLOT = SKV_TILE * D + 2 * SKV_TILE * 4;   // one tile copy per wave, used in the prologue only
  static constexpr int ROWS = 32 * D * 2;                        // one block of 32 binary16 rows
  static constexpr int BUF = (O_IN_LDS ? 3 : 2) * ROWS;          // Q, dO (, O) of one query block
  static constexpr int OFF_SLOT = NRB * BUF;                     // tile copies behind the row buffers: both are
  static constexpr int OFF_STAT = OFF_SLOT + 4 * SLOT;           //   copied at once in the prologue
  static constexpr int STAGE = 32 * 128;                         // per wave: 64 columns of its tile's dKV rows on their way out
  // where the stages live while the rows stay resident: in the O rows (not needed after the statistics) when
  // two stages fit one block of them, else in the tile slot when a stage fits it, else in an area of their own
  static constexpr int STAGE_MODE = O_IN_LDS && 2 * STAGE <= ROWS ? 0 : (!O_IN_LDS && STAGE <= SLOT ? 2 : 1);
  static constexpr int OFF_STAGE = OFF_STAT + NRB * 4 * 32 * 4;  // per buffer: lse (log2), delta, rowsum(Q), rowsum(dO)
  static constexpr int TOTAL = OFF_STAGE + (STAGE_MODE == 1 ? 4 * STAGE : 0);
  static_assert(4 * STAGE <= NRB * BUF, "the output stage overlays the row buffers");
  static_assert(ROWS % 256 == 0, "row offsets are XOR-ed with block offsets");
  static_assert(2 * TOTAL <= 160 * 1024, "two workgroups per CU");
};

// KEEP: all query blocks fit the row buffers (Nq <= 32 * NRB).  They are copied once, their statistics are
// computed once, and the workgroup then walks over `cpw` consecutive 128-key chunks of its (batch, head)
// with no barrier at all: each wave waits for its own tile copy, expands it into registers, puts the copy
// of its next tile into the same slot, and computes.  Otherwise (longer query blocks) one workgroup per
// chunk, the row blocks cycling through the buffers with two barriers a block.
template <typename S, int D, bool KEEP> __global__ __launch_bounds__(256, 2) void skv_dkv_kernel(SkvBwdLongArgs a) {
  typedef SkvDkvSmem<D> SM;
  typedef Swz<D> KSW;
  typedef TileCopy<D, SKV_TILE, 64, KSW> Copy;
  typedef TileCopy<D * 2, 32, 256, RowSwz<D>> RowCopy;
  constexpr int DS = SM::DS, NRB = SM::NRB;
  constexpr int DB = D / 32, DBW = DB / DS, CPR = D / 8, KD = D / 16;
  __shared__ __attribute__((aligned(256))) unsigned char smem[SM::TOTAL];

  const int wgs_per_bh = (a.kchunks + a.cpw - 1) / a.cpw;
  const int bh = blockIdx.x / wgs_per_bh;
  const int c_begin = (blockIdx.x % wgs_per_bh) * a.cpw, c_end = min(a.kchunks, c_begin + a.cpw);
  const int64_t b = bh / a.H, h = bh % a.H;
  const int tid = threadIdx.x, lane = tid % 64, lr = lane % 32, g = lane / 32;
  const int wave = __builtin_amdgcn_readfirstlane(tid / 64);
  const int ntiles = (a.Nk + SKV_TILE - 1) / SKV_TILE;
  const int db0 = (wave % DS) * DBW;              // first of this wave's 32-column blocks of dKV
  unsigned char *slot = smem + SM::OFF_SLOT + wave * SM::SLOT;
  const unsigned char *codes_bh = reinterpret_cast<const unsigned char *>(a.codes + b * a.scb + h * a.sch);
  const int64_t tk0 = (int64_t)bh * a.Nk, tq0 = (int64_t)bh * a.Nq;
  const int nqb = (a.Nq + 31) / 32;
  auto tile_of = [&](int chunk) { return (4 / DS) * chunk + wave / DS; };   // this wave's tile in a chunk
  const float osc = a.grad_scale ? *a.grad_scale : 1.0f;
  auto pack_out = [&](float x, float y) -> unsigned {
    return a.grad_bf16 ? pack2<__bf16>(x * osc, y * osc) : pack2<_Float16>(x * osc, y * osc);
  };

  // ---- row copies of a query block: Q, dO (, O) -> buffer (direct loads)
  RowCopy cq, cd, co;
  cq.init((unsigned)(a.sqn * 2), tid);
  cd.init((unsigned)(a.sdon * 2), tid);
  co.init((unsigned)(a.son * 2), tid);
  const _Float16 *q_bh = a.q + b * a.sqb + h * a.sqh, *d_bh = a.dout + b * a.sdob + h * a.sdoh, *o_bh = a.o + b * a.sob + h * a.soh;
  auto issue_rows = [&](int qb) {
    unsigned char *buf = smem + (qb % NRB) * SM::BUF;
    const int rows = min(32, a.Nq - 32 * qb);
    // rows past Nq read as zeros (exact bounds)
    const rsrc_t rq = make_rsrc(q_bh + (int64_t)32 * qb * a.sqn, (unsigned)(((rows - 1) * (int)a.sqn + D) * 2));
    const rsrc_t rd = make_rsrc(d_bh + (int64_t)32 * qb * a.sdon, (unsigned)(((rows - 1) * (int)a.sdon + D) * 2));
    const rsrc_t ro = make_rsrc(o_bh + (int64_t)32 * qb * a.son, (unsigned)(((rows - 1) * (int)a.son + D) * 2));
#pragma unroll
    for (int c = 0; c < RowCopy::N; ++c) {
      cq.issue_one(rq, buf, wave, tid, c);
      cd.issue_one(rd, buf + SM::ROWS, wave, tid, c);
      if (SM::O_IN_LDS) co.issue_one(ro, buf + 2 * SM::ROWS, wave, tid, c);
    }
  };
  // delta, row sums, LSE of block qb from its buffer (thread = row tid/8, chunks tid%8 + 8k).  One buffer:
  // O does not pass through LDS, `og` holds this thread's chunks of it.
  auto block_stats = [&](int qb, const u32x4 *og) {
    const unsigned char *buf = smem + (qb % NRB) * SM::BUF;
    float *stat = reinterpret_cast<float *>(smem + SM::OFF_STAT) + (qb % NRB) * 128;
    const int pi = tid / 8, part = tid % 8;
    float dsum = 0.f, rq = 0.f, rd = 0.f;
#pragma unroll
    for (int c = part; c < CPR; c += 8) {
      const int off = pi * (D * 2) + ((c ^ RowSwz<D>::swz(pi)) << 4);
      const u32x4 qv = *reinterpret_cast<const u32x4 *>(buf + off);
      const u32x4 dv = *reinterpret_cast<const u32x4 *>(buf + SM::ROWS + off);
      const u32x4 ov = SM::O_IN_LDS ? *reinterpret_cast<const u32x4 *>(buf + 2 * SM::ROWS + off) : og[c / 8];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const unsigned qw = qv[e], dw = dv[e], ow = ov[e];
        const float d0 = lo_to_f32<_Float16>(dw), d1 = hi_to_f32<_Float16>(dw);
        rq += lo_to_f32<_Float16>(qw) + hi_to_f32<_Float16>(qw);
        rd += d0 + d1;
        dsum += lo_to_f32<_Float16>(ow) * d0 + hi_to_f32<_Float16>(ow) * d1;
      }
    }
#pragma unroll
    for (int m = 1; m < 8; m *= 2) {
      dsum += __shfl_xor(dsum, m, 64);
      rq += __shfl_xor(rq, m, 64);
      rd += __shfl_xor(rd, m, 64);
    }
    if (part == 0) {
      const int qi = 32 * qb + pi;
      stat[pi] = qi < a.Nq ? a.lse[tq0 + qi] * kLog2e : INFINITY;
      stat[32 + pi] = dsum;
      stat[64 + pi] = rq;
      stat[96 + pi] = rd;
    }
  };
  auto load_o = [&](int qb, u32x4 *og) {   // one buffer: this thread's chunks of O straight from memory
    const int pi = tid / 8, part = tid % 8;
    const bool live = 32 * qb + pi < a.Nq;
#pragma unroll
    for (int k = 0; k < (CPR + 7) / 8; ++k)
      og[k] = live ? *reinterpret_cast<const u32x4 *>(o_bh + (int64_t)(32 * qb + pi) * a.son + (part + 8 * k) * 8)
                   : u32x4{0u, 0u, 0u, 0u};
  };

  Copy cp;
  cp.init((unsigned)a.scn, lane);
  auto issue_tile = [&](int t) {
    skv_issue_tile<S, D>(cp, slot, codes_bh, a.scale, a.zp, tk0, t, a.Nk, a.scn, lane);
  };

  // ---- per-lane LDS offsets inside a row block (as in the fused kernel)
  const unsigned lds0 = lds_addr(smem);
  const int row_off = lr * (D * 2), row_swz = RowSwz<D>::swz(lr);
  const int s16 = lane % 16, G = lane / 16;
  unsigned qt_off[2][2];
#pragma unroll
  for (int hh = 0; hh < 2; ++hh)
#pragma unroll
    for (int r = 0; r < 2; ++r) {
      const int i = 16 * hh + 8 * r + 4 * g + s16 / 4;
      const int chk = 2 * (G % 2) + (s16 % 4) / 2;
      qt_off[hh][r] = i * (D * 2) + ((chk ^ RowSwz<D>::swz(i)) << 4) + 8 * (s16 % 2);
    }

  // ---- this wave's tile in registers: code operands (B operands: column = key lr), scale, offset operand
  u32x4 cb[KD];
  float sk = 0.f;
  unsigned zw = 0u;   // this lane's zero point (low byte)
  auto expand_tile = [&]() {
    const int k_swz = KSW::swz(lr);
#pragma unroll
    for (int jj = 0; jj < D / 32; ++jj) {
      const u32x4 kw = *reinterpret_cast<const u32x4 *>(slot + lr * D + (((2 * jj + g) ^ k_swz) << 4));
      cb[2 * jj] = expand_codes(kw[0], kw[1]);
      cb[2 * jj + 1] = expand_codes(kw[2], kw[3]);
    }
    const unsigned *skp = reinterpret_cast<const unsigned *>(slot + SKV_TILE * D);
    const unsigned skw = skp[lr];
    zw = skp[SKV_TILE + lr];
    sk = std::is_same<S, float>::value ? __builtin_bit_cast(float, skw) : lo_to_f32<_Float16>(skw);
  };

  f32x16 dkv[DBW];
  // dKV^T of this wave's tile += contributions of query block qb (its rows and statistics are in LDS)
  auto add_block = [&](int qb, bool key_ok) {
    const unsigned char *buf = smem + (qb % NRB) * SM::BUF;
    const float *stat = reinterpret_cast<const float *>(smem + SM::OFF_STAT) + (qb % NRB) * 128;
    const float a_sk = key_ok ? a.sm_scale_log2 * sk : 0.f;
    const float sm_k = key_ok ? a.sm_scale : 0.f;
    // operands of the rank-1 offset removal: one scaling for the whole query block
    const float rs_q = stat[64 + lr], rs_do = stat[96 + lr];
    const bool big = offset_needs_x32(fmaxf(fabsf(rs_q), fabsf(rs_do)));
    u32x4 corr_q = {0u, 0u, 0u, 0u}, corr_do = {0u, 0u, 0u, 0u}, corr_k = {0u, 0u, 0u, 0u};
    if (g == 0) {
      const u32x2 cq2 = offset_query_operand(rs_q, big), cd2 = offset_query_operand(rs_do, big);
      const u32x2 ck2 = offset_key_operand(zw, big);
      corr_q[0] = cq2[0];
      corr_q[1] = cq2[1];
      corr_do[0] = cd2[0];
      corr_do[1] = cd2[1];
      corr_k[0] = ck2[0];
      corr_k[1] = ck2[1];
    }
    // S = Q C^T, dP = dO C^T (rows = queries, columns = keys), rank-1 offset removal
    f32x16 sacc, pacc;
#pragma unroll
    for (int v = 0; v < 16; ++v) sacc[v] = 0.f, pacc[v] = 0.f;
#pragma unroll
    for (int m = 0; m < KD; ++m) {
      const int off = row_off + (((4 * (m / 2) + 2 * g + m % 2) ^ row_swz) << 4);
      const u32x4 qa = *reinterpret_cast<const u32x4 *>(buf + off);
      const u32x4 da = *reinterpret_cast<const u32x4 *>(buf + SM::ROWS + off);
      sacc = mfma_h(qa, cb[m], sacc);
      pacc = mfma_h(da, cb[m], pacc);
    }
    sacc = mfma_h(corr_q, corr_k, sacc);
    pacc = mfma_h(corr_do, corr_k, pacc);
    // p and ds for this lane's key; registers run over the queries 8aa + 4g + bb
    u32x4 pf[2], df[2];
#pragma unroll
    for (int aa = 0; aa < 4; ++aa) {
      const f32x4 l4 = *reinterpret_cast<const f32x4 *>(stat + 8 * aa + 4 * g);
      const f32x4 d4 = *reinterpret_cast<const f32x4 *>(stat + 32 + 8 * aa + 4 * g);
      float p[4], ds[4];
#pragma unroll
      for (int bb = 0; bb < 4; ++bb) {
        const int v = 4 * aa + bb;
        p[bb] = key_ok ? __builtin_amdgcn_exp2f(__builtin_fmaf(a_sk, sacc[v], -l4[bb])) : 0.f;
        ds[bb] = sm_k * p[bb] * (pacc[v] * sk - d4[bb]);
      }
#pragma unroll
      for (int e = 0; e < 2; ++e) {
        pf[aa / 2][2 * (aa % 2) + e] = pack_h2(p[2 * e], p[2 * e + 1]);
        df[aa / 2][2 * (aa % 2) + e] = pack_h2(ds[2 * e], ds[2 * e + 1]);
      }
    }
    // dKV^T += dO^T P + Q^T dS
    const unsigned bufa = lds0 + (qb % NRB) * SM::BUF;
#pragma unroll
    for (int db = 0; db < DBW; ++db) {
      u32x2 fr[2][2][2];   // [matrix: dO, Q][hh][r]
#pragma unroll
      for (int hh = 0; hh < 2; ++hh)
#pragma unroll
        for (int r = 0; r < 2; ++r) {
          const unsigned ad = bufa + (qt_off[hh][r] ^ ((4 * (db0 + db)) << 4));
          fr[0][hh][r] = lds_read_tr16_async<SM::ROWS>(ad);
          fr[1][hh][r] = lds_read_tr16_async<0>(ad);
        }
      lds_wait_all();
#pragma unroll
      for (int hh = 0; hh < 2; ++hh) {
        const u32x2 d0 = tie(fr[0][hh][0]), d1 = tie(fr[0][hh][1]), q0 = tie(fr[1][hh][0]), q1 = tie(fr[1][hh][1]);
        dkv[db] = mfma_h(u32x4{d0[0], d0[1], d1[0], d1[1]}, pf[hh], dkv[db]);
        dkv[db] = mfma_h(u32x4{q0[0], q0[1], q1[0], q1[1]}, df[hh], dkv[db]);
      }
    }
  };
  // the tile's dKV rows leave through a 4 KB LDS stage as whole 128-byte lines (two 32-column blocks a time)
  auto write_out = [&](unsigned char *stage, int j0) {
    _Float16 *dkv_bh = a.dkv + b * a.sdkb + h * a.sdkh;
    const int st_w = lr * 128 + 8 * g, st_wswz = lr % 8;
    const int st_r = (lane / 8) * 128 + (((lane % 8) ^ (lane / 8)) << 4);
#pragma unroll
    for (int db = 0; db < DBW; ++db) {
#pragma unroll
      for (int aa = 0; aa < 4; ++aa) {
        u32x2 o2;
        o2[0] = pack_out(dkv[db][4 * aa], dkv[db][4 * aa + 1]);
        o2[1] = pack_out(dkv[db][4 * aa + 2], dkv[db][4 * aa + 3]);
        *reinterpret_cast<u32x2 *>(stage + st_w + (((4 * (db % 2) + aa) ^ st_wswz) << 4)) = o2;
      }
      if (db % 2 == 1) {
#pragma unroll
        for (int it = 0; it < 4; ++it) {
          const u32x4 row16 = *reinterpret_cast<const u32x4 *>(stage + st_r + it * 1024);
          const int j = j0 + 8 * it + lane / 8;
          if (j < a.Nk) *reinterpret_cast<u32x4 *>(dkv_bh + (int64_t)j * a.sdkn + 32 * (db0 + db - 1) + 8 * (lane % 8)) = row16;
        }
      }
    }
  };
  auto clear_dkv = [&]() {
#pragma unroll
    for (int db = 0; db < DBW; ++db)
#pragma unroll
      for (int v = 0; v < 16; ++v) dkv[db][v] = 0.f;
  };

  if (KEEP) {
    // ---- rows of every query block and the first tile, copied together; statistics once
    if (tile_of(c_begin) < ntiles) issue_tile(tile_of(c_begin));
    for (int qb = 0; qb < nqb; ++qb) issue_rows(qb);
    u32x4 og[SM::O_IN_LDS ? 1 : (CPR + 7) / 8];
    if (!SM::O_IN_LDS) load_o(0, og);
    dma_wait();
    __syncthreads();
    for (int qb = 0; qb < nqb; ++qb) block_stats(qb, og);
    __syncthreads();
    // stage: in the O rows (waves 0,1 use buffer 0's, waves 2,3 buffer 1's), in an area of its own, or in the
    // wave's tile slot once its operands are in registers
    unsigned char *stage = SM::STAGE_MODE == 0 ? smem + (wave / 2) * SM::BUF + 2 * SM::ROWS + (wave % 2) * SM::STAGE
                           : SM::STAGE_MODE == 1 ? smem + SM::OFF_STAGE + wave * SM::STAGE : slot;
    // The dKV stores share the memory counter with the tile copies, so the wait for the next tile sits
    // BEFORE the stores of the current one: by then the copy, issued a whole compute phase earlier, is the
    // only thing that can still be in flight.  (Stage in the slot: the copy can only be issued after the
    // stores, and the wait at the top of the next round also covers them.)
    for (int c = c_begin; c < c_end; ++c) {
      const int t = tile_of(c);
      if (t >= ntiles) break;   // (tiles of a wave grow with c)
      if (SM::STAGE_MODE == 2) dma_wait();
      expand_tile();
      const int tn = tile_of(c + 1);
      const bool more = c + 1 < c_end && tn < ntiles;
      if (SM::STAGE_MODE != 2 && more) {   // the slot is free once its contents are in registers
        lds_wait_all();
        issue_tile(tn);
      }
      clear_dkv();
      const int j0 = t * SKV_TILE;
      for (int qb = 0; qb < nqb; ++qb) add_block(qb, j0 + lr < a.Nk);
      if (SM::STAGE_MODE != 2) dma_wait();
      write_out(stage, j0);
      if (SM::STAGE_MODE == 2 && more) {   // the stage was the slot: refill it only now
        lds_wait_all();
        issue_tile(tn);
      }
    }
    return;
  }

  // ---- one chunk per workgroup, the row blocks cycle through the buffers
  const int t = tile_of(c_begin);
  const bool t_ok = t < ntiles;                   // (a wave without a tile still takes part in copies and barriers)
  const int j0 = t * SKV_TILE;
  if (t_ok) issue_tile(t);
  issue_rows(0);   // together with the tile: one memory latency for both
  dma_wait();
  if (t_ok) expand_tile();
  clear_dkv();
  for (int qb = 0; qb < nqb; ++qb) {
    if (NRB == 1 && qb > 0) {
      __syncthreads();   // everybody is done with block qb-1
      issue_rows(qb);
    }
    u32x4 og[SM::O_IN_LDS ? 1 : (CPR + 7) / 8];
    if (!SM::O_IN_LDS) load_o(qb, og);
    dma_wait();          // this thread's share of block qb has landed ...
    __syncthreads();     // ... and everybody's; (two buffers:) everybody is also done with block qb-1
    block_stats(qb, og);
    if (NRB == 2 && qb + 1 < nqb) issue_rows(qb + 1);   // the other buffer: nobody reads it any more
    __syncthreads();
    if (t_ok) add_block(qb, j0 + lr < a.Nk);
  }
  __syncthreads();   // the row buffers are done with: the stages overlay them
  if (t_ok) write_out(smem + wave * SM::STAGE, j0);
}

template <typename S, int D> static int launch_skv_bwd_long_sd(const SkvAttnArgs &x, hipStream_t st) {
  SkvBwdLongArgs a;
  a.q = static_cast<const _Float16 *>(x.q); a.o = static_cast<const _Float16 *>(x.o);
  a.dout = static_cast<const _Float16 *>(x.dout);
  a.codes = x.codes; a.scale = x.scale; a.zp = x.zp; a.lse = x.lse;
  a.dq = static_cast<_Float16 *>(x.dq); a.dkv = static_cast<_Float16 *>(x.dkv);
  a.grad_scale = x.grad_scale; a.grad_bf16 = x.grad_dtype == QFA_BF16;
  a.H = x.H; a.Nq = (int)x.Nq; a.Nk = (int)x.Nk;
  a.sqb = x.sqb; a.sqh = x.sqh; a.sqn = x.sqn; a.scb = x.scb; a.sch = x.sch; a.scn = x.scn;
  a.sob = x.sob; a.soh = x.soh; a.son = x.son; a.sdob = x.sdob; a.sdoh = x.sdoh; a.sdon = x.sdon;
  a.sdqb = x.sdqb; a.sdqh = x.sdqh; a.sdqn = x.sdqn; a.sdkb = x.sdkb; a.sdkh = x.sdkh; a.sdkn = x.sdkn;
  a.sm_scale = x.sm_scale;
  a.sm_scale_log2 = x.sm_scale * kLog2e;
  if (x.B * x.H > 0x7fffffffLL) return set_error(QFA_EUNSUPPORTED, "attn_bwd_shared_kv: too many (batch, head) pairs");
  a.BH = (int)(x.B * x.H);
  a.qblocks = (int)((x.Nq + 15) / 16);
  const int keys_per_wg = 4 * SKV_TILE / SkvDkvSmem<D>::DS;
  a.kchunks = (int)((x.Nk + keys_per_wg - 1) / keys_per_wg);
  // query blocks that fit the row buffers stay resident and a workgroup walks over several chunks: as many
  // as leave about 2048 workgroups (four rounds of two per CU)
  const bool keep = x.Nq <= 32 * SkvDkvSmem<D>::NRB;
  a.cpw = 1;
  if (keep) {
    const int64_t want = ((int64_t)a.kchunks * a.BH + 2047) / 2048;
    a.cpw = (int)(want < 1 ? 1 : want > a.kchunks ? a.kchunks : want);
  }
  const int64_t total_q = (int64_t)a.qblocks * ((a.BH + 7) / 8) * 8;
  const int64_t total_k = (int64_t)((a.kchunks + a.cpw - 1) / a.cpw) * a.BH;
  if (total_q > 0x7fffffffLL || total_k > 0x7fffffffLL)
    return set_error(QFA_EUNSUPPORTED, "attn_bwd_shared_kv: too many blocks for one launch");
  skv_dq_kernel<S, D><<<dim3((unsigned)total_q), dim3(256), 0, st>>>(a);
  if (int e = check_launch("qfa_attn_bwd_shared_kv (dQ)")) return e;
  if (keep) skv_dkv_kernel<S, D, true><<<dim3((unsigned)total_k), dim3(256), 0, st>>>(a);
  else skv_dkv_kernel<S, D, false><<<dim3((unsigned)total_k), dim3(256), 0, st>>>(a);
  return check_launch("qfa_attn_bwd_shared_kv (dKV)");
}

int launch_skv_bwd_long(const SkvAttnArgs &x, hipStream_t st) {
  const bool s32 = x.scale_dtype == QFA_F32;
  if (x.D == 256) return s32 ? launch_skv_bwd_long_sd<float, 256>(x, st) : launch_skv_bwd_long_sd<_Float16, 256>(x, st);
  if (x.D == 128) return s32 ? launch_skv_bwd_long_sd<float, 128>(x, st) : launch_skv_bwd_long_sd<_Float16, 128>(x, st);
  if (x.D == 64) return s32 ? launch_skv_bwd_long_sd<float, 64>(x, st) : launch_skv_bwd_long_sd<_Float16, 64>(x, st);
  return set_error(QFA_EUNSUPPORTED, "attn_bwd_shared_kv: head_dim must be 64, 128 or 256");
}

}  // namespace qfa
