// Shared-KV attention for short query blocks: the reference's own operator and benchmark shape
// (quant_flash_attn.py:22-83; compute_flops.py:96: Z=512, H=16, 16 queries against 3000 keys).
//     O = softmax(sm_scale * Q K^^T) K^,    K^ = V^ = scale * (codes - zero_point)  per token,
// with Q left in 16-bit floating point exactly as the reference does (:50-52).  The operator is
// bound by reading the INT8 codes once: per (batch, head) there are only a few queries, so the
// kernel streams the codes -- and nothing else -- through LDS and keeps the matrix pipe fed from them.
//
// Work split.  One workgroup = 4 waves = one block of 16 queries of one (batch, head); the 32-key
// tiles of the sequence are dealt round-robin to the waves, every wave runs its own online softmax
// over its tiles from a private ring of LDS buffers filled by direct global->LDS loads (no
// workgroup barrier in the loop), and the four partial results are merged at the end.  Longer query
// blocks are split into several workgroups that run on the same XCD and share its L2 copy of the codes.
//
// Codes as MFMA operands.  A code byte c (two's complement) with its top bit flipped is the
// unsigned byte c + 128; OR-ed under the constant 0x6400 it is the binary16 number 1152 + c
// exactly, so one XOR per dword and one byte permute per pair of elements turn codes into a
// 16-bit MFMA operand.  The offset is taken out again exactly:
//     sum_d (1152 + c_jd) q_d  - (1152 + zp_j) * sum_d q_d        = sum_d (c_jd - zp_j) q_d
//     sum_j (1152 + c_jd) p'_j - sum_j (1152 + zp_j) p'_j         = sum_j (c_jd - zp_j) p'_j
// The first subtraction is a rank-1 update done by one more MFMA (sum_d q_d split into three
// binary16 terms, products exact in fp32); the second is a per-query scalar accumulated with
// v_dot2 over the same rounded p' = p * scale_j that the MFMA consumed, so the offsets cancel
// exactly and only the usual rounding of P remains.
//
// V^T fragments come out of the row-major code tile through ds_read_b64_tr_b8: inside a group of 16
// lanes, lane i receives byte i%8 of the 8-byte rows addressed by lanes (i%16)/8 + {0,2,..,14}.
#include <mutex>
#include <type_traits>

#include "qfa_host.h"
#include "qfa_skv_common.h"

namespace qfa {

struct SkvArgs {
  const void *q; const int8_t *codes; const void *scale; const int8_t *zp;
  void *o; float *lse;
  int64_t H;
  int Nq, Nk;
  int64_t sqb, sqh, sqn, scb, sch, scn, sob, soh, son;
  float sm_scale_log2;
  int qblocks;   // query blocks per (batch, head)
  int BH;        // batch * heads
  int splits;    // workgroups sharing the keys of one query block (1: the result goes straight to o / lse)
  int tiles_per_split;
  float *partial;   // splits > 1: [BH][qblocks][splits][16*D + 32] floats (O^T unnormalised, m in log2 units, l)
};

// ring depth per wave: three tiles, two at D = 256 (8 KB tiles)
template <int D> constexpr int skv_nbuf() { return D == 256 ? 2 : 3; }

template <typename T, typename S, int D> __global__ __launch_bounds__(256, 2) void skv_fwd_kernel(SkvArgs a) {
  typedef SwzSkv<D> KSW;
  typedef TileCopy<D, SKV_TILE, 64, KSW> Copy;
  constexpr int KS = D / 32;     // 32-wide k-steps of the score product
  constexpr int DB = D / 16;     // 16-row blocks of O^T
  constexpr int OPS = Copy::N + 2, SKV_NBUF = skv_nbuf<D>();
  constexpr int K_BYTES = SKV_TILE * D, SLOT = K_BYTES + 2 * SKV_TILE * 4, WAVE = SKV_NBUF * SLOT;
  constexpr int MG = 16 * D + 32;   // floats of one partial result: O^T [D][16], m[16], l[16]
  static_assert(3 * MG * 4 <= 4 * WAVE, "the merge area overlays the rings");
  __shared__ __attribute__((aligned(16))) unsigned char smem[4 * WAVE];

  // block id -> (batch*head, query block): the query blocks of one (batch, head) get ids that differ
  // by 8, i.e. run on the same XCD close in time, and share its L2 copy of the codes
  const int per_bh = a.qblocks * a.splits;
  const int bh = (int)(blockIdx.x / (8 * per_bh)) * 8 + (int)(blockIdx.x % 8);
  const int qb = (int)(blockIdx.x / 8) % a.qblocks;
  const int split = ((int)(blockIdx.x / 8) % per_bh) / a.qblocks;
  if (bh >= a.BH) return;
  const int64_t b = bh / a.H, h = bh % a.H;
  const int tid = threadIdx.x, lane = tid % 64, q16 = lane % 16, G = lane / 16;
  const int wave = __builtin_amdgcn_readfirstlane(tid / 64);
  const int wave_off = wave * WAVE;

  const unsigned char *codes_bh = reinterpret_cast<const unsigned char *>(a.codes + b * a.scb + h * a.sch);
  const int64_t tk0 = (int64_t)bh * a.Nk, tq0 = (int64_t)bh * a.Nq;
  // this workgroup's tiles t0 .. t0 + ntiles - 1 (all of them unless the keys are split); wave w takes
  // t0 + w, t0 + w + 4, ...
  const int t0 = split * a.tiles_per_split;
  const int ntiles = min(a.tiles_per_split, (a.Nk + SKV_TILE - 1) / SKV_TILE - t0);
  const int my_tiles = ntiles > wave ? (ntiles - wave + 3) / 4 : 0;

  Copy cp;
  cp.init((unsigned)a.scn, lane);
  auto issue = [&](int i, int slot_idx) {
    const int t = t0 + wave + 4 * i;
    unsigned char *slot = smem + wave_off + slot_idx * SLOT;
    const int rows = min(SKV_TILE, a.Nk - t * SKV_TILE);
    const rsrc_t rs_k = make_rsrc(codes_bh + (int64_t)t * SKV_TILE * a.scn, (unsigned)((rows - 1) * (int)a.scn + D));
#pragma unroll
    for (int c = 0; c < Copy::N; ++c) cp.issue_one(rs_k, slot, 0, lane, c);
    const rsrc_t rs_s = make_rsrc(reinterpret_cast<const S *>(a.scale) + tk0 + (int64_t)t * SKV_TILE,
                                  (unsigned)rows * (unsigned)sizeof(S));
    const rsrc_t rs_z = make_rsrc(a.zp + tk0 + (int64_t)t * SKV_TILE, (unsigned)rows);
    if (lane < SKV_TILE) {
      if constexpr (sizeof(S) == 4)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_s, (lptr_t)(slot + K_BYTES), 4, lane * 4, 0, 0, 0);
      else
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_s, (lptr_t)(slot + K_BYTES), 2, lane * 2, 0, 0, 0);
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_z, (lptr_t)(slot + K_BYTES + SKV_TILE * 4), 1, lane, 0, 0, 0);
    }
  };
  auto scale_of = [](unsigned w) -> float {
    return std::is_same<S, float>::value ? __builtin_bit_cast(float, w) : lo_to_f32<T>(w);
  };
#pragma unroll
  for (int i = 0; i < SKV_NBUF - 1; ++i)
    if (i < my_tiles) issue(i, i);

  // ---- this lane's query as B operand: k-step m, k-group G holds d = 64(m/2) + 16G + 8(m%2) + {0..7}
  const int qi = 16 * qb + q16;
  const int qi_c = qi < a.Nq ? qi : a.Nq - 1;
  const T *qrow = reinterpret_cast<const T *>(a.q) + b * a.sqb + h * a.sqh + (int64_t)qi_c * a.sqn;
  u32x4 qf[KS];
  float rs = 0.f;
#pragma unroll
  for (int m = 0; m < KS; ++m) {
    const u32x4 raw = *reinterpret_cast<const u32x4 *>(qrow + 64 * (m / 2) + 16 * G + 8 * (m % 2));
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const unsigned w = raw[e];
      const unsigned hw = std::is_same<T, _Float16>::value ? w : pack_h2(lo_to_f32<T>(w), hi_to_f32<T>(w));
      qf[m][e] = hw;
      rs += lo_to_f32<_Float16>(hw) + hi_to_f32<_Float16>(hw);
    }
  }
  rs += __shfl_xor(rs, 16, 64);
  rs += __shfl_xor(rs, 32, 64);
  const bool big = offset_needs_x32(rs);
  u32x4 corr_q = {0u, 0u, 0u, 0u};
  if (G == 0) {
    const u32x2 cq2 = offset_query_operand(rs, big);
    corr_q[0] = cq2[0];
    corr_q[1] = cq2[1];
  }
  const float a_s = a.sm_scale_log2;

  // ---- per-lane read offsets inside a tile
  int k_off[2];   // code rows as A operands: key 16rb + lane%16, chunk 4mm + G (two k-steps per 16 bytes)
#pragma unroll
  for (int rb = 0; rb < 2; ++rb) k_off[rb] = (16 * rb + q16) * D + ((G ^ KSW::swz(16 * rb + q16)) << 4);
  // transposing reads: source lane s of group G addresses key 16((s/2)/4) + 4G + (s/2)%4 (the keys whose
  // probabilities sit in k-group G of the P operand), 8 bytes at d = 16db + 8(s%2)
  int vt_off;
  {
    const int s = lane % 16, j = s / 2;
    const int key = 16 * (j / 4) + 4 * G + j % 4;
    vt_off = key * D + (KSW::swz(key) << 4) + 8 * (s % 2);
  }
  const unsigned lds0 = lds_addr(smem);

  f32x4 oacc[DB];
#pragma unroll
  for (int db = 0; db < DB; ++db) oacc[db] = f32x4{0.f, 0.f, 0.f, 0.f};
  float m_ref = -INFINITY, m_bound = -INFINITY, nm = 0.f, l_run = 0.f, w_run = 0.f;
  const float thr = SKV_RESCALE_THRESHOLD / a_s;

  auto tile = [&](int i, int slot_idx, auto masked_tag) {
    constexpr bool MASKED = decltype(masked_tag)::value;
    const int slot_off = wave_off + slot_idx * SLOT;
    const unsigned char *slot = smem + slot_off;
    const unsigned *skp = reinterpret_cast<const unsigned *>(slot + K_BYTES);
    const unsigned *zpp = skp + SKV_TILE;
    const int j0 = (t0 + wave + 4 * i) * SKV_TILE;
    const unsigned z_a[2] = {zpp[q16], zpp[16 + q16]};
    // (the per-block read addresses are re-formed from these three every tile: one XOR each, instead of
    // two dozen registers held across the loop)
    int vt = vt_off, ko[2] = {k_off[0], k_off[1]};
    asm volatile("" : "+v"(vt), "+v"(ko[0]), "+v"(ko[1]));
    // transposed fragments for P.V in groups of 8 blocks (one group, two at D = 256), the first one now
    constexpr int VG = DB < 8 ? DB : 8;
    u32x2 vr[VG];
#pragma unroll
    for (int db = 0; db < VG; ++db) vr[db] = lds_read_tr8_async(lds0 + slot_off + (vt ^ (db << 4)));
    // ---- scores: two 16-key row blocks
    f32x4 f[2];
#pragma unroll
    for (int rb = 0; rb < 2; ++rb) {
      f[rb] = f32x4{0.f, 0.f, 0.f, 0.f};
      u32x4 kw[(KS + 1) / 2];
#pragma unroll
      for (int mm = 0; mm < (KS + 1) / 2; ++mm)
        kw[mm] = *reinterpret_cast<const u32x4 *>(slot + (ko[rb] ^ ((4 * mm) << 4)));
#pragma unroll
      for (int m = 0; m < KS; ++m)
        f[rb] = mfma_h16(expand_codes(kw[m / 2][2 * (m % 2)], kw[m / 2][2 * (m % 2) + 1]), qf[m], f[rb]);
      u32x4 corr_k = {0u, 0u, 0u, 0u};
      if (G == 0) {
        const u32x2 ck2 = offset_key_operand(z_a[rb], big);
        corr_k[0] = ck2[0];
        corr_k[1] = ck2[1];
      }
      f[rb] = mfma_h16(corr_k, corr_q, f[rb]);
    }
    // ---- scale, lane-local maximum (keys 16rb + 4G + v)
    u32x4 sk4[2], zk4[2];
    float mt = -INFINITY;
#pragma unroll
    for (int rb = 0; rb < 2; ++rb) {
      sk4[rb] = *reinterpret_cast<const u32x4 *>(skp + 16 * rb + 4 * G);
      zk4[rb] = *reinterpret_cast<const u32x4 *>(zpp + 16 * rb + 4 * G);
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        float uu = f[rb][v] * scale_of(sk4[rb][v]);
        if (MASKED && j0 + 16 * rb + 4 * G + v >= a.Nk) uu = -INFINITY;
        f[rb][v] = uu;
        mt = fmaxf(mt, uu);
      }
    }
    if (__builtin_amdgcn_ballot_w64(mt > m_bound) != 0) {
      // the reference maximum is common to the four lanes of a query
      mt = fmaxf(mt, __shfl_xor(mt, 16, 64));
      mt = fmaxf(mt, __shfl_xor(mt, 32, 64));
      const float m_new = fmaxf(m_ref, mt);
      const float alpha = m_new == m_ref ? 1.0f : __builtin_amdgcn_exp2f(a_s * (m_ref - m_new));
      m_ref = m_new;
      m_bound = m_new + thr;
      nm = -a_s * m_new;
      l_run *= alpha;
      w_run *= alpha;
#pragma unroll
      for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int v = 0; v < 4; ++v) oacc[db][v] *= alpha;
    }
    // ---- p, p' = p * scale_j as binary16, row sum, offset term
    u32x4 pf;
#pragma unroll
    for (int rb = 0; rb < 2; ++rb)
#pragma unroll
      for (int e = 0; e < 2; ++e) {
        const float p0 = __builtin_amdgcn_exp2f(__builtin_fmaf(a_s, f[rb][2 * e], nm));
        const float p1 = __builtin_amdgcn_exp2f(__builtin_fmaf(a_s, f[rb][2 * e + 1], nm));
        l_run += p0 + p1;
        const unsigned pp = pack_h2(p0 * scale_of(sk4[rb][2 * e]), p1 * scale_of(sk4[rb][2 * e + 1]));
        pf[2 * rb + e] = pp;
        const unsigned cpair = magic_zp_pair(zk4[rb][2 * e], zk4[rb][2 * e + 1]);
        w_run = __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2, pp), __builtin_bit_cast(f16x2, cpair), w_run, false);
      }
    // ---- O^T += (1152 + codes)^T . P'^T, one k-step of 32 keys
#pragma unroll
    for (int g0 = 0; g0 < DB; g0 += VG) {
      lds_wait_all();
      u32x2 cur[VG];
#pragma unroll
      for (int db = 0; db < VG; ++db) cur[db] = tie(vr[db]);
      if (g0 + VG < DB) {
#pragma unroll
        for (int db = 0; db < VG; ++db) vr[db] = lds_read_tr8_async(lds0 + slot_off + (vt ^ ((g0 + VG + db) << 4)));
      }
#pragma unroll
      for (int db = 0; db < VG; ++db) oacc[g0 + db] = mfma_h16(expand_codes(cur[db][0], cur[db][1]), pf, oacc[g0 + db]);
    }
  };

  int cur = 0, nxt = SKV_NBUF - 1;   // slot of the tile in work, slot the next copy goes to
  for (int i = 0; i < my_tiles; ++i) {
    if (i + SKV_NBUF - 1 < my_tiles) {
      issue(i + SKV_NBUF - 1, nxt);
      asm volatile("s_waitcnt vmcnt(%0)" ::"n"((SKV_NBUF - 1) * OPS) : "memory");
    } else {
      dma_wait();
    }
    if ((t0 + wave + 4 * i + 1) * SKV_TILE > a.Nk) tile(i, cur, std::true_type{});
    else tile(i, cur, std::false_type{});
    cur = cur + 1 == SKV_NBUF ? 0 : cur + 1;
    nxt = nxt + 1 == SKV_NBUF ? 0 : nxt + 1;
  }

  
  // ---- merge the four partial results
  float l_tot = l_run + __shfl_xor(l_run, 16, 64), w_tot = w_run + __shfl_xor(w_run, 16, 64);
  l_tot += __shfl_xor(l_tot, 32, 64);
  w_tot += __shfl_xor(w_tot, 32, 64);
  __syncthreads();
  float *mg = reinterpret_cast<float *>(smem);
  if (wave > 0) {
    float *dst = mg + (wave - 1) * MG;
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int v = 0; v < 4; ++v) dst[(16 * db + 4 * G + v) * 16 + q16] = oacc[db][v] - w_tot;
    if (G == 0) {
      dst[16 * D + q16] = m_ref;
      dst[16 * D + 16 + q16] = l_tot;
    }
  }
  __syncthreads();
  if (wave == 0) {
    float m_all = m_ref;   // finite: wave 0 always owns the first tile
#pragma unroll
    for (int w = 0; w < 3; ++w) m_all = fmaxf(m_all, mg[w * MG + 16 * D + q16]);
    const float s0 = __builtin_amdgcn_exp2f(a_s * (m_ref - m_all));
    float l_all = l_tot * s0;
    float sw[3];
#pragma unroll
    for (int w = 0; w < 3; ++w) {
      sw[w] = __builtin_amdgcn_exp2f(a_s * (mg[w * MG + 16 * D + q16] - m_all));   // -inf for a wave without tiles
      l_all += mg[w * MG + 16 * D + 16 + q16] * sw[w];
    }
    if (a.splits > 1) {   // hand the unnormalised block result to the merge kernel
      float *dst = a.partial + ((int64_t)(bh * a.qblocks + qb) * a.splits + split) * MG;
#pragma unroll
      for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int v = 0; v < 4; ++v) {
          const int d = 16 * db + 4 * G + v;
          float acc = (oacc[db][v] - w_tot) * s0;
#pragma unroll
          for (int w = 0; w < 3; ++w) acc += mg[w * MG + d * 16 + q16] * sw[w];
          dst[d * 16 + q16] = acc;
        }
      if (G == 0) {
        dst[16 * D + q16] = a_s * m_all;
        dst[16 * D + 16 + q16] = l_all;
      }
      return;
    }
    const float inv = 1.0f / l_all;
    if (qi < a.Nq) {
      T *orow = reinterpret_cast<T *>(a.o) + b * a.sob + h * a.soh + (int64_t)qi * a.son;
#pragma unroll
      for (int db = 0; db < DB; ++db) {
        float r[4];
#pragma unroll
        for (int v = 0; v < 4; ++v) {
          const int d = 16 * db + 4 * G + v;
          float acc = (oacc[db][v] - w_tot) * s0;
#pragma unroll
          for (int w = 0; w < 3; ++w) acc += mg[w * MG + d * 16 + q16] * sw[w];
          r[v] = acc * inv;
        }
        u32x2 o2;
        o2[0] = pack2<T>(r[0], r[1]);
        o2[1] = pack2<T>(r[2], r[3]);
        *reinterpret_cast<u32x2 *>(orow + 16 * db + 4 * G) = o2;
      }
      if (G == 0) a.lse[tq0 + qi] = (a_s * m_all + __log2f(l_all)) * kLn2;
    }
  }
}

// Sum of the `splits` partial results of every query block: O = sum_s O_s 2^(m_s - m) / sum_s l_s 2^(m_s - m).
// One workgroup per (batch*head, query block); thread = (query tid%16, columns tid/16 + 16k).
template <typename T, int D> __global__ __launch_bounds__(256) void skv_merge_kernel(SkvArgs a) {
  constexpr int MG = 16 * D + 32;
  const int bh = blockIdx.x / a.qblocks, qb = blockIdx.x % a.qblocks;
  const int64_t b = bh / a.H, h = bh % a.H;
  const int q16 = threadIdx.x % 16, dg = threadIdx.x / 16;
  const int qi = 16 * qb + q16;
  const float *src = a.partial + (int64_t)blockIdx.x * a.splits * MG;
  float m = -INFINITY;
  for (int s = 0; s < a.splits; ++s) m = fmaxf(m, src[s * MG + 16 * D + q16]);
  float l = 0.f, acc[D / 16];
#pragma unroll
  for (int k = 0; k < D / 16; ++k) acc[k] = 0.f;
  for (int s = 0; s < a.splits; ++s) {
    const float w = __builtin_amdgcn_exp2f(src[s * MG + 16 * D + q16] - m);
    l += src[s * MG + 16 * D + 16 + q16] * w;
#pragma unroll
    for (int k = 0; k < D / 16; ++k) acc[k] += src[s * MG + (dg + 16 * k) * 16 + q16] * w;
  }
  if (qi >= a.Nq) return;
  const float inv = 1.0f / l;
  T *orow = reinterpret_cast<T *>(a.o) + b * a.sob + h * a.soh + (int64_t)qi * a.son;
#pragma unroll
  for (int k = 0; k < D / 16; ++k) orow[dg + 16 * k] = (T)(acc[k] * inv);
  if (dg == 0) a.lse[(int64_t)bh * a.Nq + qi] = (m + __log2f(l)) * kLn2;
}

// How the keys of one query block are split over workgroups: enough workgroups to fill the chip
// (about four per CU), never fewer than 8 tiles per workgroup; 1 = no split.
static void skv_split_plan(int64_t BH, int64_t Nq, int64_t Nk, int *splits, int *tiles_per_split) {
  const int64_t ntiles = (Nk + SKV_TILE - 1) / SKV_TILE, wgs = BH * ((Nq + 15) / 16);
  int64_t want = wgs >= 512 ? 1 : (1024 + wgs - 1) / wgs;
  if (want > ntiles / 8) want = ntiles / 8;
  if (want < 1) want = 1;
  const int64_t tps = (ntiles + want - 1) / want;
  *tiles_per_split = (int)tps;
  *splits = (int)((ntiles + tps - 1) / tps);
}

int64_t skv_fwd_workspace_bytes(int64_t B, int64_t H, int64_t Nq, int64_t Nk, int D) {
  int splits, tps;
  skv_split_plan(B * H, Nq, Nk, &splits, &tps);
  return splits > 1 ? B * H * ((Nq + 15) / 16) * splits * (int64_t)(16 * D + 32) * 4 : 0;
}

template <typename T, typename S, int D> static int launch_skv_fwd_tsd(const SkvAttnArgs &x, hipStream_t st) {
  SkvArgs a;
  a.q = x.q; a.codes = x.codes; a.scale = x.scale; a.zp = x.zp; a.o = x.o; a.lse = x.lse;
  a.H = x.H; a.Nq = (int)x.Nq; a.Nk = (int)x.Nk;
  a.sqb = x.sqb; a.sqh = x.sqh; a.sqn = x.sqn; a.scb = x.scb; a.sch = x.sch; a.scn = x.scn;
  a.sob = x.sob; a.soh = x.soh; a.son = x.son;
  a.sm_scale_log2 = x.sm_scale * kLog2e;
  if (x.B * x.H > 0x7fffffffLL) return set_error(QFA_EUNSUPPORTED, "attn_fwd_shared_kv: too many (batch, head) pairs");
  a.BH = (int)(x.B * x.H);
  a.qblocks = (int)((x.Nq + 15) / 16);
  a.splits = 1;
  a.tiles_per_split = (int)((x.Nk + SKV_TILE - 1) / SKV_TILE);
  a.partial = nullptr;
  if (x.workspace) {   // validated: large enough for the plan below
    skv_split_plan(x.B * x.H, x.Nq, x.Nk, &a.splits, &a.tiles_per_split);
    a.partial = static_cast<float *>(x.workspace);
  }
  const int64_t total = (int64_t)a.qblocks * a.splits * ((a.BH + 7) / 8) * 8;   // ids past batch*heads exit at once
  if (total > 0x7fffffffLL) return set_error(QFA_EUNSUPPORTED, "attn_fwd_shared_kv: too many query blocks for one launch");
  skv_fwd_kernel<T, S, D><<<dim3((unsigned)total), dim3(256), 0, st>>>(a);
  if (int e = check_launch("qfa_attn_fwd_shared_kv")) return e;
  if (a.splits > 1) {
    skv_merge_kernel<T, D><<<dim3((unsigned)(a.BH * a.qblocks)), dim3(256), 0, st>>>(a);
    return check_launch("qfa_attn_fwd_shared_kv (merge)");
  }
  return 0;
}

template <typename T, int D> static int launch_skv_fwd_td(const SkvAttnArgs &x, hipStream_t st) {
  if (x.scale_dtype == QFA_F32) return launch_skv_fwd_tsd<T, float, D>(x, st);
  return launch_skv_fwd_tsd<T, T, D>(x, st);   // validated: scale_dtype == io_dtype
}

// ---- scratch for callers that cannot allocate --------------------------------------------------------
// The split over keys needs device memory beyond the inputs and outputs (the partial results).  This array
// is that memory for qfa_attn_fwd_shared_kv_static: every GPU the library runs on holds its own copy until
// the process ends.  In host code the array's NAME is only a stand-in for the symbol; the device address is
// asked for once per device (with that device current) and only that address is handed to kernels.
static __device__ __align__(256) unsigned char scratch[QFA_STATIC_SCRATCH_BYTES];

static constexpr int kMaxDevices = 64;
static std::mutex g_scratch_mutex;
static void *g_scratch_ptr[kMaxDevices];   // device address of `scratch` on device i, nullptr until asked for

// Device address of the current device's scratch array (0 and the address in *out, or an error code).
static int static_scratch(void **out) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return set_error((int)e, "attn_fwd_shared_kv_static: hipGetDevice: %s", hipGetErrorString(e));
  if (dev < 0 || dev >= kMaxDevices)
    return set_error(QFA_EUNSUPPORTED, "attn_fwd_shared_kv_static: device index %d outside [0, %d)", dev, kMaxDevices);
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_ptr[dev]) {
    void *p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !p)
      return set_error(e != hipSuccess ? (int)e : QFA_EINVAL, "attn_fwd_shared_kv_static: hipGetSymbolAddress: %s",
                       hipGetErrorString(e));
    g_scratch_ptr[dev] = p;
  }
  *out = g_scratch_ptr[dev];
  return 0;
}

int launch_skv_fwd_static(const SkvAttnArgs &x, hipStream_t st) {
  const int64_t need = skv_fwd_workspace_bytes(x.B, x.H, x.Nq, x.Nk, x.D);
  if (need > (int64_t)QFA_STATIC_SCRATCH_BYTES)
    return set_error(QFA_EUNSUPPORTED,
                     "attn_fwd_shared_kv_static: this shape splits its keys into partial results of %lld bytes, more "
                     "than the built-in scratch of %lld bytes; use qfa_attn_fwd_shared_kv with a caller workspace",
                     (long long)need, (long long)QFA_STATIC_SCRATCH_BYTES);
  SkvAttnArgs y = x;
  y.workspace = nullptr;
  if (need > 0) {   // every partial result is written by the first kernel before the merge reads it: nothing to clear
    if (int e = static_scratch(&y.workspace)) return e;
  }
  return launch_skv_fwd(y, st);
}

int launch_skv_fwd(const SkvAttnArgs &x, hipStream_t st) {
  if (x.io_dtype == QFA_F16) {
    if (x.D == 256) return launch_skv_fwd_td<_Float16, 256>(x, st);
    if (x.D == 128) return launch_skv_fwd_td<_Float16, 128>(x, st);
    if (x.D == 64) return launch_skv_fwd_td<_Float16, 64>(x, st);
  } else {
    if (x.D == 256) return launch_skv_fwd_td<__bf16, 256>(x, st);
    if (x.D == 128) return launch_skv_fwd_td<__bf16, 128>(x, st);
    if (x.D == 64) return launch_skv_fwd_td<__bf16, 64>(x, st);
  }
  return set_error(QFA_EUNSUPPORTED, "attn_fwd_shared_kv: head_dim must be 64, 128 or 256");
}

}  // namespace qfa
