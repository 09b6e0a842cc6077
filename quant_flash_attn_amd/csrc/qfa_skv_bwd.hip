// Backward of the shared-KV attention for one short query block (at most 32 queries), the
// reference's _attn_bwd_kernel_quantized (quant_flash_attn.py:104-166): per (batch, head)
//     P = exp(sm_scale * Q KV^T - LSE),   dP = dO KV^T,   dS = sm_scale * P o (dP - delta),
//     dQ = dS KV,   dKV = P^T dO + dS^T Q                                      (:153-161)
// with KV = scale * (codes - zero_point) per token and delta = rowsum(O o dO) (:97-99).
// Everything is computed in binary16 products with fp32 accumulation, like the reference.
//
// One workgroup = 4 waves = one (batch, head).  The 32-key tiles are dealt round-robin to the
// waves; a wave streams its tiles through two private LDS slots (direct global->LDS loads, no
// workgroup barrier in the loop), writes the dKV rows of a tile as soon as they are complete and
// keeps a partial dQ in registers; the four partial dQ are summed at the end.  The last step of a
// tile (step 4 below) no longer reads the codes, so the copy of the tile after the next one is
// issued into the same slot just before it, and the wait for the next tile sits right behind that
// issue: the only younger vector-memory operations are then the ones just issued (the dKV stores,
// which share the counter, come after the wait).  Q and dO sit in
// LDS as binary16 rows for the whole kernel and are read as MFMA operands both ways (rows for the
// products contracted over d, transposed through ds_read_b64_tr_b16 for those contracted over
// the queries).  The codes enter the MFMAs as exact binary16 integers (qfa_skv_common.h).
//
// Per tile, with S-layout accumulators (lane = key j, registers = queries i):
//   1. S  = Q . C^T  and dP = dO . C^T       C = 1152 + codes; rank-1 MFMA removes (1152 + zp_j) * rowsum
//   2. p, ds = sm_scale * p * (dp - delta)   per-lane scale_j, zp_j;  LSE and delta per register
//      ds * scale_j goes through a small LDS buffer to become an operand contracted over keys
//   3. dQ^T += C^T . (ds * scale)^T          codes transposed by ds_read_b64_tr_b8; offset via v_dot2
//   4. dKV^T = dO^T . P + Q^T . dS           one 32-column block of d at a time, stored right away
#include <type_traits>

#include "qfa_host.h"
#include "qfa_skv_common.h"

namespace qfa {

struct SkvBwdArgs {
  const _Float16 *q, *o, *dout;
  const int8_t *codes; const void *scale; const int8_t *zp;
  const float *lse;
  _Float16 *dq, *dkv;          // 16-bit outputs: binary16, or bfloat16 when grad_bf16 is set
  const float *grad_scale;     // nullable device scalar: dq and dkv are multiplied by it before rounding
  int grad_bf16;
  int64_t H;
  int Nq, Nk;
  int64_t sqb, sqh, sqn, scb, sch, scn, sob, soh, son, sdob, sdoh, sdon, sdqb, sdqh, sdqn, sdkb, sdkh, sdkn;
  float sm_scale, sm_scale_log2;
};

constexpr int SKVB_NBUF = 2;   // LDS slots per wave: the tile in work and the next one

template <int D> struct SkvBwdSmem {
  static constexpr int K_BYTES = SKV_TILE * D;
  static constexpr int SLOT = K_BYTES + 2 * SKV_TILE * 4;   // codes, one dword per key for scale and zero point
  static constexpr int XT = 32 * 128;                       // (ds * scale) as binary16 [key][query] (first half); later
                                                            // 64 columns of the tile's dKV rows on their way out
  static constexpr int WAVE = SKVB_NBUF * SLOT + XT;
  static constexpr int ROWS = 32 * D * 2;                   // Q, then dO: binary16 [32][D], chunks swizzled
  static constexpr int OFF_Q = 4 * WAVE;
  static constexpr int OFF_DO = OFF_Q + ROWS;
  static constexpr int OFF_STAT = OFF_DO + ROWS;            // lse (log2 units), delta, rowsum(Q), rowsum(dO): 32 floats each
  static constexpr int TOTAL = OFF_STAT + 4 * 32 * 4;
  static constexpr int MG = 32 * D;                         // floats of one partial dQ^T
  static_assert(3 * MG * 4 <= OFF_STAT, "the dQ merge area overlays the slots and the Q / dO rows");
  static_assert(OFF_Q % 256 == 0, "row offsets are XOR-ed with block offsets");
};

// Chunk swizzle of the binary16 Q / dO rows (CPR 16-byte chunks each): distinct for 8 (16) consecutive
// rows read at one chunk index, and moving whole 32-byte pairs apart for 4 consecutive rows, which is
// what the transposing reads touch together.
template <int CPR> __device__ __forceinline__ int row_swizzle(int i) {
  return (2 * (i % 4) + (i / 4) % 2 + 8 * ((i / 8) % 2)) % CPR;
}

template <int OFF> __device__ __forceinline__ u32x2 lds_tr16(unsigned addr) { return lds_read_tr16_async<OFF>(addr); }

// S: element type of the scale vector (float or _Float16).  HALF: at most 16 queries -- rows 16..31 of the
// query block are padding, so their share of steps 2 and 4 is skipped (P and dS are zero there).
template <typename S, int D, bool HALF> __global__ __launch_bounds__(256, D == 256 ? 1 : 2) void skv_bwd_kernel(SkvBwdArgs a) {
  constexpr int QH = HALF ? 1 : 2;   // 16-query halves of the block that hold queries
  typedef SkvBwdSmem<D> SM;
  typedef Swz<D> KSW;
  typedef TileCopy<D, SKV_TILE, 64, KSW> Copy;
  constexpr int DB = D / 32;     // 32-row blocks of d
  constexpr int CPR = D / 8;     // 16-byte chunks in a binary16 row
  constexpr int OPS = Copy::N + 2;
  __shared__ __attribute__((aligned(256))) unsigned char smem[SM::TOTAL];

  const int bh = blockIdx.x;
  const int64_t b = bh / a.H, h = bh % a.H;
  const int tid = threadIdx.x, lane = tid % 64, lr = lane % 32, g = lane / 32;
  const int wave = __builtin_amdgcn_readfirstlane(tid / 64);
  const int wave_off = wave * SM::WAVE;
  float *stat = reinterpret_cast<float *>(smem + SM::OFF_STAT);
  const float osc = a.grad_scale ? *a.grad_scale : 1.0f;
  auto pack_out = [&](float x, float y) -> unsigned {
    return a.grad_bf16 ? pack2<__bf16>(x * osc, y * osc) : pack2<_Float16>(x * osc, y * osc);
  };

  const unsigned char *codes_bh = reinterpret_cast<const unsigned char *>(a.codes + b * a.scb + h * a.sch);
  const int64_t tk0 = (int64_t)bh * a.Nk, tq0 = (int64_t)bh * a.Nq;
  const int ntiles = (a.Nk + SKV_TILE - 1) / SKV_TILE;
  const int my_tiles = ntiles > wave ? (ntiles - wave + 3) / 4 : 0;

  // ---- tile copies (as in the forward)
  Copy cp;
  cp.init((unsigned)a.scn, lane);
  auto issue = [&](int i) {
    const int t = wave + 4 * i;
    unsigned char *slot = smem + wave_off + (i % SKVB_NBUF) * SM::SLOT;
    const int rows = min(SKV_TILE, a.Nk - t * SKV_TILE);
    const rsrc_t rs_k = make_rsrc(codes_bh + (int64_t)t * SKV_TILE * a.scn, (unsigned)((rows - 1) * (int)a.scn + D));
#pragma unroll
    for (int c = 0; c < Copy::N; ++c) cp.issue_one(rs_k, slot, 0, lane, c);
    const rsrc_t rs_s = make_rsrc(reinterpret_cast<const S *>(a.scale) + tk0 + (int64_t)t * SKV_TILE,
                                  (unsigned)rows * (unsigned)sizeof(S));
    const rsrc_t rs_z = make_rsrc(a.zp + tk0 + (int64_t)t * SKV_TILE, (unsigned)rows);
    if (lane < SKV_TILE) {
      if constexpr (sizeof(S) == 4)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_s, (lptr_t)(slot + SM::K_BYTES), 4, lane * 4, 0, 0, 0);
      else
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_s, (lptr_t)(slot + SM::K_BYTES), 2, lane * 2, 0, 0, 0);
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_z, (lptr_t)(slot + SM::K_BYTES + SKV_TILE * 4), 1, lane, 0, 0, 0);
    }
  };
  auto scale_of = [](unsigned w) -> float {
    return std::is_same<S, float>::value ? __builtin_bit_cast(float, w) : lo_to_f32<_Float16>(w);
  };
#pragma unroll
  for (int i = 0; i < SKVB_NBUF; ++i)
    if (i < my_tiles) issue(i);

  // ---- Q and dO into LDS (rows past Nq as zeros), delta, row sums, LSE in log2 units
  {
    const int pi = tid / 8, part = tid % 8;
    const bool valid = pi < a.Nq;
    const int pi_c = valid ? pi : 0;
    const _Float16 *qrow = a.q + b * a.sqb + h * a.sqh + (int64_t)pi_c * a.sqn;
    const _Float16 *orow = a.o + b * a.sob + h * a.soh + (int64_t)pi_c * a.son;
    const _Float16 *drow = a.dout + b * a.sdob + h * a.sdoh + (int64_t)pi_c * a.sdon;
    float dsum = 0.f, rq = 0.f, rd = 0.f;
#pragma unroll
    for (int c = part; c < CPR; c += 8) {
      u32x4 qv = {0u, 0u, 0u, 0u}, dv = qv, ov = qv;
      if (valid) {
        qv = *reinterpret_cast<const u32x4 *>(qrow + c * 8);
        dv = *reinterpret_cast<const u32x4 *>(drow + c * 8);
        ov = *reinterpret_cast<const u32x4 *>(orow + c * 8);
      }
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const float d0 = lo_to_f32<_Float16>(dv[e]), d1 = hi_to_f32<_Float16>(dv[e]);
        rq += lo_to_f32<_Float16>(qv[e]) + hi_to_f32<_Float16>(qv[e]);
        rd += d0 + d1;
        dsum += lo_to_f32<_Float16>(ov[e]) * d0 + hi_to_f32<_Float16>(ov[e]) * d1;
      }
      const int off = pi * (D * 2) + ((c ^ row_swizzle<CPR>(pi)) << 4);
      *reinterpret_cast<u32x4 *>(smem + SM::OFF_Q + off) = qv;
      *reinterpret_cast<u32x4 *>(smem + SM::OFF_DO + off) = dv;
    }
#pragma unroll
    for (int m = 1; m < 8; m *= 2) {
      dsum += __shfl_xor(dsum, m, 64);
      rq += __shfl_xor(rq, m, 64);
      rd += __shfl_xor(rd, m, 64);
    }
    if (part == 0) {
      stat[pi] = valid ? a.lse[tq0 + pi] * kLog2e : INFINITY;   // p = exp2(. - inf) = 0 for the padding rows
      stat[32 + pi] = dsum;
      stat[64 + pi] = rq;
      stat[96 + pi] = rd;
    }
  }
  __syncthreads();

  // query-side operands of the rank-1 updates (A operand: row = query lr), one scaling for the whole block
  const float rs_q = stat[64 + lr], rs_do = stat[96 + lr];
  const bool big = offset_needs_x32(fmaxf(fabsf(rs_q), fabsf(rs_do)));
  u32x4 corr_q = {0u, 0u, 0u, 0u}, corr_do = {0u, 0u, 0u, 0u};
  if (g == 0) {
    const u32x2 cq2 = offset_query_operand(rs_q, big), cd2 = offset_query_operand(rs_do, big);
    corr_q[0] = cq2[0];
    corr_q[1] = cq2[1];
    corr_do[0] = cd2[0];
    corr_do[1] = cd2[1];
  }
  const float a_s = a.sm_scale_log2;

  // ---- per-lane LDS offsets
  const unsigned lds0 = lds_addr(smem);
  // (a) rows of Q / dO as A operands: row lr, chunk 4jj + 2g + hf for k-step 2jj + hf
  const int row_off = lr * (D * 2), row_swz = row_swizzle<CPR>(lr);
  // (b) code rows as B operands: row lr, chunk 2jj + g (16 bytes = two k-steps)
  const int k_off = lr * D, k_swz = KSW::swz(lr);
  const int s16 = lane % 16, G = lane / 16;
  // (c) Q^T / dO^T fragments through transposing reads: lane s of a group addresses row
  //     i = 16hh + 8r + 4g + s/4 at d = 32db + 16(G%2) + 4(s%4); lane L of the group receives d = .. + L
  //     and the four rows as its elements.  Block db enters as an XOR of 4db on the chunk index.
  unsigned qt_off[2][2];
#pragma unroll
  for (int hh = 0; hh < 2; ++hh)
#pragma unroll
    for (int r = 0; r < 2; ++r) {
      const int i = 16 * hh + 8 * r + 4 * g + s16 / 4;
      const int chunk = 2 * (G % 2) + (s16 % 4) / 2;
      qt_off[hh][r] = lds0 + SM::OFF_Q + i * (D * 2) + ((chunk ^ row_swizzle<CPR>(i)) << 4) + 8 * (s16 % 2);
    }
  // (d) ds*scale: written as [key lr][query], 8-byte segment seg = 2aa + g at position seg ^ ((key/2) % 8);
  //     read back transposed: lane s addresses key 16kk + 8g + 4r + s/4, segment 4(G%2) + s%4
  const int xt_w = lr * 64, xt_wswz = (lr / 2) % 8;
  unsigned xt_r[2][2];
#pragma unroll
  for (int kk = 0; kk < 2; ++kk)
#pragma unroll
    for (int r = 0; r < 2; ++r) {
      const int j = 16 * kk + 8 * g + 4 * r + s16 / 4;
      const int seg = 4 * (G % 2) + s16 % 4;
      xt_r[kk][r] = lds0 + wave_off + SKVB_NBUF * SM::SLOT + j * 64 + ((seg ^ ((j / 2) % 8)) << 3);
    }
  // (e) codes transposed (ds_read_b64_tr_b8): lane s addresses key 16kk + 8g + s/2, 8 bytes at
  //     d = 32db + 16(G%2) + 8(s%2); block db enters as an XOR of 2db on the chunk index
  unsigned vt_off[2];
#pragma unroll
  for (int kk = 0; kk < 2; ++kk) {
    const int key = 16 * kk + 8 * g + s16 / 2;
    vt_off[kk] = key * D + (((G % 2) ^ KSW::swz(key)) << 4) + 8 * (s16 % 2);
  }

  f32x16 dq[DB];
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int v = 0; v < 16; ++v) dq[db][v] = 0.f;
  float w_run = 0.f;
  _Float16 *dkv_bh = a.dkv + b * a.sdkb + h * a.sdkh;

  u32x4 pf[2], df[2];   // P and dS of the tile in work: B operands of step 4
  auto tile_scores = [&](int i) {
    const int slot_off = wave_off + (i % SKVB_NBUF) * SM::SLOT;
    const unsigned char *slot = smem + slot_off;
    const unsigned *skp = reinterpret_cast<const unsigned *>(slot + SM::K_BYTES);
    const unsigned *zpp = skp + SKV_TILE;
    const int j0 = (wave + 4 * i) * SKV_TILE;
    const bool key_ok = j0 + lr < a.Nk;
    const float sk = scale_of(skp[lr]);
    const unsigned zmine = zpp[lr];
    // ---- 1. S = Q C^T, dP = dO C^T  (rows = queries, columns = keys)
    f32x16 sacc, pacc;
#pragma unroll
    for (int v = 0; v < 16; ++v) sacc[v] = 0.f, pacc[v] = 0.f;
#pragma unroll
    for (int jj = 0; jj < D / 32; ++jj) {
      const u32x4 kw = *reinterpret_cast<const u32x4 *>(slot + k_off + (((2 * jj + g) ^ k_swz) << 4));
#pragma unroll
      for (int hf = 0; hf < 2; ++hf) {
        const u32x4 cb = expand_codes(kw[2 * hf], kw[2 * hf + 1]);
        const int off = row_off + (((4 * jj + 2 * g + hf) ^ row_swz) << 4);
        const u32x4 qa = *reinterpret_cast<const u32x4 *>(smem + SM::OFF_Q + off);
        const u32x4 da = *reinterpret_cast<const u32x4 *>(smem + SM::OFF_DO + off);
        sacc = mfma_h(qa, cb, sacc);
        pacc = mfma_h(da, cb, pacc);
      }
    }
    {
      u32x4 corr_k = {0u, 0u, 0u, 0u};
      if (g == 0) {
        const u32x2 ck2 = offset_key_operand(zmine, big);
        corr_k[0] = ck2[0];
        corr_k[1] = ck2[1];
      }
      sacc = mfma_h(corr_q, corr_k, sacc);
      pacc = mfma_h(corr_do, corr_k, pacc);
    }
    __builtin_amdgcn_sched_barrier(0);
    // ---- 2. p and ds for this lane's key; registers run over the queries 8aa + 4g + bb
    const float a_sk = key_ok ? a_s * sk : 0.f;
    const float sm_k = key_ok ? a.sm_scale : 0.f;   // a key past the end contributes nothing
#pragma unroll
    for (int aa = 0; aa < 2 * QH; ++aa) {
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
      u32x2 x;
      x[0] = pack_h2(ds[0] * sk, ds[1] * sk);
      x[1] = pack_h2(ds[2] * sk, ds[3] * sk);
      *reinterpret_cast<u32x2 *>(smem + wave_off + SKVB_NBUF * SM::SLOT + xt_w + (((2 * aa + g) ^ xt_wswz) << 3)) = x;
    }
    __builtin_amdgcn_sched_barrier(0);
    // ---- 3. dQ^T += C^T (ds*scale)^T, contracted over the keys; the 1152 + zp offsets accumulate in w_run
#pragma unroll
    for (int kk = 0; kk < 2; ++kk) {
      u32x2 x0 = lds_tr16<0>(xt_r[kk][0]), x1 = lds_tr16<0>(xt_r[kk][1]);
      u32x2 vr[DB];
#pragma unroll
      for (int db = 0; db < DB; ++db) vr[db] = lds_read_tr8_async(lds0 + slot_off + (vt_off[kk] ^ ((2 * db) << 4)));
      const u32x4 z0 = *reinterpret_cast<const u32x4 *>(zpp + 16 * kk + 8 * g);
      const u32x4 z1 = *reinterpret_cast<const u32x4 *>(zpp + 16 * kk + 8 * g + 4);
      lds_wait_all();
      x0 = tie(x0);
      x1 = tie(x1);
      if (HALF && G % 2 == 1) x0 = x1 = u32x2{0u, 0u};   // lanes of queries 16..31: nothing was written for them
      const u32x4 xb = {x0[0], x0[1], x1[0], x1[1]};
      const unsigned zc[4] = {magic_zp_pair(z0[0], z0[1]), magic_zp_pair(z0[2], z0[3]), magic_zp_pair(z1[0], z1[1]),
                              magic_zp_pair(z1[2], z1[3])};
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const unsigned xe = xb[e], ze = zc[e];   // (bit_cast of a vector element lvalue reads element 0)
        w_run = __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2, xe), __builtin_bit_cast(f16x2, ze), w_run, false);
      }
#pragma unroll
      for (int db = 0; db < DB; ++db) {
        const u32x2 w = tie(vr[db]);
        dq[db] = mfma_h(expand_codes(w[0], w[1]), xb, dq[db]);
      }
    }
  };
  auto tile_dkv = [&](int i) {
    // ---- 4. dKV^T = dO^T P + Q^T dS for one block of 32 d at a time; column = this lane's key
    const int j0 = (wave + 4 * i) * SKV_TILE;
    unsigned char *stage = smem + wave_off + SKVB_NBUF * SM::SLOT;
    // two blocks (64 columns, 128 bytes a row) are staged in LDS and leave as whole 128-byte lines:
    // 16-byte pair p of row j sits at position p ^ (j % 8)
    const int st_w = lr * 128 + 8 * g, st_wswz = lr % 8;
    const int st_r = (lane / 8) * 128 + (((lane % 8) ^ (lane / 8)) << 4);
#pragma unroll
    for (int db = 0; db < DB; ++db) {
      u32x2 fr[2][2][2];   // [matrix: dO, Q][hh][r]
#pragma unroll
      for (int hh = 0; hh < QH; ++hh)
#pragma unroll
        for (int r = 0; r < 2; ++r) {
          const unsigned ad = qt_off[hh][r] ^ ((4 * db) << 4);
          fr[0][hh][r] = lds_tr16<SM::ROWS>(ad);
          fr[1][hh][r] = lds_tr16<0>(ad);
        }
      lds_wait_all();
      f32x16 acc;
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[v] = 0.f;
#pragma unroll
      for (int hh = 0; hh < QH; ++hh) {
        const u32x2 d0 = tie(fr[0][hh][0]), d1 = tie(fr[0][hh][1]), q0 = tie(fr[1][hh][0]), q1 = tie(fr[1][hh][1]);
        acc = mfma_h(u32x4{d0[0], d0[1], d1[0], d1[1]}, pf[hh], acc);
        acc = mfma_h(u32x4{q0[0], q0[1], q1[0], q1[1]}, df[hh], acc);
      }
#pragma unroll
      for (int aa = 0; aa < 4; ++aa) {
        u32x2 o2;
        o2[0] = pack_out(acc[4 * aa], acc[4 * aa + 1]);
        o2[1] = pack_out(acc[4 * aa + 2], acc[4 * aa + 3]);
        *reinterpret_cast<u32x2 *>(stage + st_w + (((4 * (db % 2) + aa) ^ st_wswz) << 4)) = o2;
      }
      if (db % 2 == 1) {
#pragma unroll
        for (int it = 0; it < 4; ++it) {
          const u32x4 row16 = *reinterpret_cast<const u32x4 *>(stage + st_r + it * 1024);
          const int j = j0 + 8 * it + lane / 8;
          if (j < a.Nk) *reinterpret_cast<u32x4 *>(dkv_bh + (int64_t)j * a.sdkn + 32 * (db - 1) + 8 * (lane % 8)) = row16;
        }
      }
    }
  };

  if (my_tiles > 1) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(OPS) : "memory");   // tile 0 has landed
  else dma_wait();
  for (int i = 0; i < my_tiles; ++i) {
    tile_scores(i);
    if (i + 2 < my_tiles) {
      issue(i + 2);   // into the slot of tile i, which step 4 does not read
      asm volatile("s_waitcnt vmcnt(%0)" ::"n"(OPS) : "memory");   // everything older, tile i+1 included, is there
    } else {
      dma_wait();
    }
    tile_dkv(i);
  }

  // ---- dQ = sum of the four partial results, offsets removed; wave 0 writes it
  const float w_tot = w_run + swap32_f(w_run);
  __syncthreads();   // slots and rows are done with: the merge area overlays them
  float *mg = reinterpret_cast<float *>(smem);
  constexpr int MG = SM::MG;
  if (wave > 0) {
    float *dst = mg + (wave - 1) * MG;
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int v = 0; v < 16; ++v) dst[(32 * db + 8 * (v / 4) + 4 * g + v % 4) * 32 + lr] = dq[db][v] - w_tot;
  }
  __syncthreads();
  if (wave == 0 && lr < a.Nq) {
    _Float16 *qrow = a.dq + b * a.sdqb + h * a.sdqh + (int64_t)lr * a.sdqn;
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int aa = 0; aa < 4; ++aa) {
        float r[4];
#pragma unroll
        for (int bb = 0; bb < 4; ++bb) {
          const int d = 32 * db + 8 * aa + 4 * g + bb;
          r[bb] = dq[db][4 * aa + bb] - w_tot + mg[d * 32 + lr] + mg[MG + d * 32 + lr] + mg[2 * MG + d * 32 + lr];
        }
        u32x2 o2;
        o2[0] = pack_out(r[0], r[1]);
        o2[1] = pack_out(r[2], r[3]);
        *reinterpret_cast<u32x2 *>(qrow + 32 * db + 8 * aa + 4 * g) = o2;
      }
  }
}

template <typename S, int D> static int launch_skv_bwd_sd(const SkvAttnArgs &x, hipStream_t st) {
  SkvBwdArgs a;
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
  const int64_t total = x.B * x.H;
  if (total > 0x7fffffffLL) return set_error(QFA_EUNSUPPORTED, "attn_bwd_shared_kv: too many (batch, head) pairs for one launch");
  if (x.Nq <= 16) skv_bwd_kernel<S, D, true><<<dim3((unsigned)total), dim3(256), 0, st>>>(a);
  else if constexpr (D <= 128) skv_bwd_kernel<S, D, false><<<dim3((unsigned)total), dim3(256), 0, st>>>(a);
  else return set_error(QFA_EUNSUPPORTED, "attn_bwd_shared_kv: the one-pass kernel takes at most 16 queries at head_dim 256");
  return check_launch("qfa_attn_bwd_shared_kv");
}

int launch_skv_bwd(const SkvAttnArgs &x, hipStream_t st) {
  const bool s32 = x.scale_dtype == QFA_F32;
  if (x.D == 128) return s32 ? launch_skv_bwd_sd<float, 128>(x, st) : launch_skv_bwd_sd<_Float16, 128>(x, st);
  if (x.D == 64) return s32 ? launch_skv_bwd_sd<float, 64>(x, st) : launch_skv_bwd_sd<_Float16, 64>(x, st);
  if (x.D == 256) return s32 ? launch_skv_bwd_sd<float, 256>(x, st) : launch_skv_bwd_sd<_Float16, 256>(x, st);
  return set_error(QFA_EUNSUPPORTED, "attn_bwd_shared_kv: head_dim must be 64, 128 or 256");
}

// ---- dO handed to the binary16 backward kernels: dO * 2^k as binary16, and 2^-k for the kernels to scale dQ and dKV
// back with.  dQ and dKV are linear in dO, and what the kernels feed the matrix pipe is sm_scale * p * (dP - delta)
// and that times the key's scale: k puts  max|dO| * 2^k * (largest key scale)  into (4, 8] and keeps
// max|dO| * 2^k at or below 2^14, so that neither ordinary small gradients sink into binary16's subnormals nor large
// key scales leave its range.  Two launches, no atomics: every block of the first writes its two partial maxima,
// every block of the second reduces all of them again (a few KB out of the L2) before it scales its share.
constexpr int NORM_BLOCKS = 2048;   // blocks of the first launch = pairs of floats in the partials buffer

template <typename T> __device__ __forceinline__ float max_abs8(const u32x4 w, float m) {
#pragma unroll
  for (int e = 0; e < 4; ++e) m = fmaxf(m, fmaxf(fabsf(lo_to_f32<T>(w[e])), fabsf(hi_to_f32<T>(w[e]))));
  return m;
}
// largest magnitude of the 16 bytes of scales a thread loads at a time
template <typename S> __device__ __forceinline__ float max_abs_chunk(const u32x4 w, float m) {
  if constexpr (sizeof(S) == 2) {
    return max_abs8<S>(w, m);
  } else {
#pragma unroll
    for (int e = 0; e < 4; ++e) m = fmaxf(m, fabsf(__builtin_bit_cast(float, w[e])));
    return m;
  }
}
__device__ __forceinline__ float block_max_256(float m, float *red) {
  for (int off = 32; off > 0; off >>= 1) m = fmaxf(m, __shfl_xor(m, off, 64));
  __syncthreads();
  if (threadIdx.x % 64 == 0) red[threadIdx.x / 64] = m;
  __syncthreads();
  return fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
}
// floor(log2(c / y)) for c = 2^ce and a positive normal y, exactly (no logarithm): y = m * 2^e with m in [1, 2)
__device__ __forceinline__ int floor_log2_quot(int ce, float y) {
  const unsigned b = __builtin_bit_cast(unsigned, y);
  const int e = (int)((b >> 23) & 0xff) - 127;
  return ce - e - ((b & 0x7fffffu) != 0 ? 1 : 0);
}

// 16 bytes per thread and trip for both vectors (the scales' last ns % (16 / sizeof(S)) elements one by one)
template <typename T, typename S>
__global__ __launch_bounds__(256) void dout_max_kernel(const T *dout, int64_t n8, const S *scale, int64_t ns, float *partials) {
  __shared__ float red[4];
  constexpr int EPC = 16 / sizeof(S);
  const int64_t tid = (int64_t)blockIdx.x * 256 + threadIdx.x, nth = (int64_t)NORM_BLOCKS * 256, nsc = ns / EPC;
  float m = 0.f, ms = 0.f;
  for (int64_t i = tid; i < n8; i += nth) m = max_abs8<T>(reinterpret_cast<const u32x4 *>(dout)[i], m);
  for (int64_t i = tid; i < nsc; i += nth) ms = max_abs_chunk<S>(reinterpret_cast<const u32x4 *>(scale)[i], ms);
  if (tid < ns - nsc * EPC) ms = fmaxf(ms, fabsf((float)scale[nsc * EPC + tid]));
  m = block_max_256(m, red);
  ms = block_max_256(ms, red);
  if (threadIdx.x == 0) {
    partials[2 * blockIdx.x] = m;
    partials[2 * blockIdx.x + 1] = ms;
  }
}

template <typename T>
__global__ __launch_bounds__(256) void dout_scale_kernel(const T *dout, int64_t n8, const float *partials, _Float16 *out,
                                                         float *back) {
  __shared__ float red[4];
  float m = 0.f, ms = 0.f;
  for (int i = threadIdx.x; i < NORM_BLOCKS; i += 256) {
    m = fmaxf(m, partials[2 * i]);
    ms = fmaxf(ms, partials[2 * i + 1]);
  }
  m = fmaxf(block_max_256(m, red), 1e-30f);     // inf stays inf: k = -100 below
  ms = fmaxf(block_max_256(ms, red), 1e-30f);
  int k = min(floor_log2_quot(3, m * ms), floor_log2_quot(14, m));
  k = max(-100, min(100, k));
  const float f = __builtin_ldexpf(1.0f, k);
  if (blockIdx.x == 0 && threadIdx.x == 0) back[0] = __builtin_ldexpf(1.0f, -k);
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= n8) return;
  const u32x4 w = reinterpret_cast<const u32x4 *>(dout)[i];
  u32x4 r;
#pragma unroll
  for (int e = 0; e < 4; ++e) r[e] = pack2<_Float16>(lo_to_f32<T>(w[e]) * f, hi_to_f32<T>(w[e]) * f);
  reinterpret_cast<u32x4 *>(out)[i] = r;
}

template <typename T, typename S>
static int launch_dout_normalise_ts(const void *dout, int64_t n, const void *scale, int64_t ns, float *partials,
                                    void *out, float *back, hipStream_t st) {
  const int64_t n8 = n / 8, blocks = (n8 + 255) / 256;
  if (blocks > 0x7fffffffLL) return set_error(QFA_EUNSUPPORTED, "dout_normalise: too many elements for one launch");
  dout_max_kernel<T, S><<<dim3(NORM_BLOCKS), dim3(256), 0, st>>>((const T *)dout, n8, (const S *)scale, ns, partials);
  dout_scale_kernel<T><<<dim3((unsigned)blocks), dim3(256), 0, st>>>((const T *)dout, n8, partials, (_Float16 *)out, back);
  return check_launch("qfa_dout_normalise");
}

int64_t dout_normalise_workspace_bytes() { return (int64_t)NORM_BLOCKS * 2 * sizeof(float); }

int launch_dout_normalise(const void *dout, int dout_dtype, int64_t n, const void *scale, int scale_dtype, int64_t ns,
                          float *partials, void *out, float *back, hipStream_t st) {
  const bool s32 = scale_dtype == QFA_F32;
  if (dout_dtype == QFA_BF16)
    return s32 ? launch_dout_normalise_ts<__bf16, float>(dout, n, scale, ns, partials, out, back, st)
               : launch_dout_normalise_ts<__bf16, _Float16>(dout, n, scale, ns, partials, out, back, st);
  return s32 ? launch_dout_normalise_ts<_Float16, float>(dout, n, scale, ns, partials, out, back, st)
             : launch_dout_normalise_ts<_Float16, _Float16>(dout, n, scale, ns, partials, out, back, st);
}

}  // namespace qfa
