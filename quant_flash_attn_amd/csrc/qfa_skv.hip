// Shared-KV attention for short query blocks: the reference's own operator and benchmark shape
// (quant_flash_attn.py:22-83; compute_flops.py:96: Z=512, H=16, 16 queries against 3000 keys).
//     O = softmax(sm_scale * Q K^^T) K^,    K^ = V^ = scale * (codes - zero_point)  per token,
// with Q left in 16-bit floating point exactly as the reference does (:50-52).  The operator is
// bound by reading the INT8 codes once: per (batch, head) there are only a few queries, so the
// kernel streams the codes -- and nothing else -- through LDS and keeps the matrix pipe fed from them.
//
// Work split.  One workgroup = 4 waves = one block of 32 queries of one (batch, head); the 32-key
// tiles of the sequence are dealt round-robin to the waves, every wave runs its own online softmax
// over its tiles from a private ring of LDS buffers filled by direct global->LDS loads (no
// workgroup barrier in the loop), and the four partial results are merged at the end.
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
  int qblocks;   // ceil(Nq / 32)
};

constexpr int SKV_NBUF = 4;      // ring depth per wave

template <int D> struct SkvSmem {
  static constexpr int K_BYTES = SKV_TILE * D;             // codes of a tile, rows dense, chunks swizzled (Swz<D>)
  static constexpr int SLOT = K_BYTES + 2 * SKV_TILE * 4;  // + one dword per key for the scale, one for the zero point
  static constexpr int WAVE = SKV_NBUF * SLOT;
  static constexpr int MG = 32 * D + 64;                   // floats of one partial result: O^T [D][32], m[32], l[32]
  static constexpr int MERGE = 3 * MG * 4;
  static constexpr int TOTAL = 4 * WAVE > MERGE ? 4 * WAVE : MERGE;
};

// T: element type of Q and O.  S: element type of the scale vector (float, or T).
template <typename T, typename S, int D> __global__ __launch_bounds__(256, 2) void skv_fwd_kernel(SkvArgs a) {
  typedef SkvSmem<D> SM;
  typedef Swz<D> KSW;
  typedef TileCopy<D, SKV_TILE, 64, KSW> Copy;
  constexpr int KD = D / 16;    // 16-wide k-steps of the score product
  constexpr int DB = D / 32;    // 32-row blocks of O^T
  constexpr int OPS = Copy::N + 2;   // vector-memory instructions per tile
  __shared__ __attribute__((aligned(16))) unsigned char smem[SM::TOTAL];

  const int bh = blockIdx.x / a.qblocks, qb = blockIdx.x % a.qblocks;
  const int64_t b = bh / a.H, h = bh % a.H;
  const int tid = threadIdx.x, lane = tid % 64, lr = lane % 32, g = lane / 32;
  const int wave = __builtin_amdgcn_readfirstlane(tid / 64);
  unsigned char *ring = smem + wave * SM::WAVE;

  const unsigned char *codes_bh = reinterpret_cast<const unsigned char *>(a.codes + b * a.scb + h * a.sch);
  const int64_t tk0 = (int64_t)bh * a.Nk, tq0 = (int64_t)bh * a.Nq;
  const int ntiles = (a.Nk + SKV_TILE - 1) / SKV_TILE;
  const int my_tiles = ntiles > wave ? (ntiles - wave + 3) / 4 : 0;    // tiles wave, wave+4, ...

  // ---- this lane's query as binary16 B operand of the score product, and sum_d q_d
  const int qi = qb * 32 + lr;
  const int qi_c = qi < a.Nq ? qi : a.Nq - 1;
  const T *qrow = reinterpret_cast<const T *>(a.q) + b * a.sqb + h * a.sqh + (int64_t)qi_c * a.sqn;
  u32x4 qf[KD];
  float rs = 0.f;
#pragma unroll
  for (int m = 0; m < KD; ++m) {
    // k-step m = 2j + hf covers d = 32j + 16g + 8hf + {0..7}: the two halves of one 16-byte code chunk
    const int d0 = 32 * (m / 2) + 16 * g + 8 * (m % 2);
    const u32x4 raw = *reinterpret_cast<const u32x4 *>(qrow + d0);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      // bf16 input enters through its binary16 rounding
      qf[m][e] = std::is_same<T, _Float16>::value ? raw[e] : pack_h2(lo_to_f32<T>(raw[e]), hi_to_f32<T>(raw[e]));
      rs += lo_to_f32<_Float16>(qf[m][e]) + hi_to_f32<_Float16>(qf[m][e]);
    }
  }
  rs += swap32_f(rs);
  // -sum_d q_d as three binary16 terms, k-group 0 of the correction MFMA's B operand
  u32x4 corr_q = {0u, 0u, 0u, 0u};
  {
    const _Float16 h0 = (_Float16)rs;
    const float r1 = rs - (float)h0;
    const _Float16 h1 = (_Float16)r1;
    const _Float16 h2 = (_Float16)(r1 - (float)h1);
    if (g == 0) {
      corr_q[0] = pack_h2(-(float)h0, -(float)h1);
      corr_q[1] = pack_h2(-(float)h2, 0.f);
    }
  }
  const float a_s = a.sm_scale_log2;

  // ---- tile copies: codes through a per-lane offset table; scale and zero point one dword per key
  // (sub-dword direct loads write lane l's zero-extended value to the dword at 4*l)
  Copy cp;
  cp.init((unsigned)a.scn, lane);
  auto issue = [&](int i) {   // own tile i -> ring slot i % NBUF
    const int t = wave + 4 * i;
    unsigned char *slot = ring + (i % SKV_NBUF) * SM::SLOT;
    const int rows = min(SKV_TILE, a.Nk - t * SKV_TILE);
    // rows past the end read as zero (exact bounds); their scores are masked
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
    return std::is_same<S, float>::value ? __builtin_bit_cast(float, w) : lo_to_f32<T>(w);
  };

  // ---- per-lane read offsets inside a tile
  const int k_off = lr * D;
  const int k_swz = KSW::swz(lr);
  // transposing reads: source lane s of a 16-lane group G addresses 8 bytes of key list[g][s/2] at
  // d = 32db + 16(G%2) + 8(s%2);  list[g] = {16hh + 4g + 0..3, 16hh + 8 + 4g + 0..3}, the keys whose
  // probabilities sit in k-group g of the P operand.
  // (block db enters as an XOR of 2db on the chunk index: smem is aligned to a whole row)
  unsigned vt_off[2];
  {
    const int s = lane % 16, G = lane / 16, j = s / 2;
#pragma unroll
    for (int hh = 0; hh < 2; ++hh) {
      const int key = 16 * hh + (j < 4 ? 4 * g + j : 8 + 4 * g + (j - 4));
      vt_off[hh] = key * D + (((G % 2) ^ KSW::swz(key)) << 4) + 8 * (s % 2);
    }
  }

  f32x16 oacc[DB];
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int v = 0; v < 16; ++v) oacc[db][v] = 0.f;
  float m_ref = -INFINITY, m_bound = -INFINITY, nm = 0.f, l_run = 0.f, w_run = 0.f;
  const float thr = SKV_RESCALE_THRESHOLD / a_s;

  auto tile = [&](int i, auto masked_tag) {
    constexpr bool MASKED = decltype(masked_tag)::value;
    const int slot_off = wave * SM::WAVE + (i % SKV_NBUF) * SM::SLOT;
    const unsigned char *slot = smem + slot_off;
    const unsigned *skp = reinterpret_cast<const unsigned *>(slot + SM::K_BYTES);
    const unsigned *zpp = skp + SKV_TILE;
    const int j0 = (wave + 4 * i) * SKV_TILE;
    // ---- code rows for the scores (plain reads), then the transposed fragments for P.V (asynchronous)
    u32x4 kw[D / 32];
#pragma unroll
    for (int j = 0; j < D / 32; ++j)
      kw[j] = *reinterpret_cast<const u32x4 *>(slot + k_off + (((2 * j + g) ^ k_swz) << 4));
    const unsigned zmine = zpp[lr];
    // ---- scores: S^T = (1152 + codes) . Q^T, offset removed by the rank-1 MFMA
    f32x16 f;
#pragma unroll
    for (int v = 0; v < 16; ++v) f[v] = 0.f;
#pragma unroll
    for (int j = 0; j < D / 32; ++j) {
      f = mfma_h(expand_codes(kw[j][0], kw[j][1]), qf[2 * j], f);
      f = mfma_h(expand_codes(kw[j][2], kw[j][3]), qf[2 * j + 1], f);
    }
    {
      const unsigned cz = magic_zp_pair(zmine, zmine);      // binary16 pair of 1152 + zp
      u32x4 corr_k = {0u, 0u, 0u, 0u};
      if (g == 0) {
        corr_k[0] = cz;
        corr_k[1] = cz & 0xffffu;
      }
      f = mfma_h(corr_k, corr_q, f);
    }
    u32x2 vr[2][DB];
#pragma unroll
    for (int hh = 0; hh < 2; ++hh)
#pragma unroll
      for (int db = 0; db < DB; ++db) vr[hh][db] = lds_read_tr8_async(lds_addr(smem) + slot_off + (vt_off[hh] ^ ((2 * db) << 4)));
    // ---- scale, running maximum
    float mt0 = -INFINITY, mt1 = -INFINITY;
#pragma unroll
    for (int aa = 0; aa < 4; ++aa) {
      const u32x4 sk4 = *reinterpret_cast<const u32x4 *>(skp + 8 * aa + 4 * g);
#pragma unroll
      for (int bb = 0; bb < 4; ++bb) {
        float uu = f[4 * aa + bb] * scale_of(sk4[bb]);
        if (MASKED && j0 + 8 * aa + 4 * g + bb >= a.Nk) uu = -INFINITY;
        f[4 * aa + bb] = uu;
        if (aa & 1) mt1 = fmaxf(mt1, uu); else mt0 = fmaxf(mt0, uu);
      }
    }
    const float mt = max_across_halves(fmaxf(mt0, mt1));
    if (__builtin_amdgcn_ballot_w64(mt > m_bound) != 0) {
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
        for (int v = 0; v < 16; ++v) oacc[db][v] *= alpha;
    }
    // ---- p = exp2(.);  p' = p * scale_j rounded to binary16;  row sum of p;  offset term of p'
    u32x4 pf[2];
#pragma unroll
    for (int aa = 0; aa < 4; ++aa) {
      const u32x4 sk4 = *reinterpret_cast<const u32x4 *>(skp + 8 * aa + 4 * g);
      const u32x4 zk4 = *reinterpret_cast<const u32x4 *>(zpp + 8 * aa + 4 * g);
#pragma unroll
      for (int e = 0; e < 2; ++e) {
        const int v0 = 4 * aa + 2 * e;
        const float p0 = __builtin_amdgcn_exp2f(__builtin_fmaf(a_s, f[v0], nm));
        const float p1 = __builtin_amdgcn_exp2f(__builtin_fmaf(a_s, f[v0 + 1], nm));
        l_run += p0 + p1;
        const unsigned pp = pack_h2(p0 * scale_of(sk4[2 * e]), p1 * scale_of(sk4[2 * e + 1]));
        pf[aa / 2][2 * (aa % 2) + e] = pp;
        const unsigned cpair = magic_zp_pair(zk4[2 * e], zk4[2 * e + 1]);
        w_run = __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2, pp), __builtin_bit_cast(f16x2, cpair), w_run, false);
      }
    }
    // ---- O^T += (1152 + codes)^T . P'^T
    lds_wait_all();
#pragma unroll
    for (int hh = 0; hh < 2; ++hh)
#pragma unroll
      for (int db = 0; db < DB; ++db) {
        const u32x2 w = tie(vr[hh][db]);
        oacc[db] = mfma_h(expand_codes(w[0], w[1]), pf[hh], oacc[db]);
      }
  };

  // ---- ring: NBUF-1 tiles in flight ahead of the one in work
#pragma unroll
  for (int i = 0; i < SKV_NBUF - 1; ++i)
    if (i < my_tiles) issue(i);
  for (int i = 0; i < my_tiles; ++i) {
    if (i + SKV_NBUF - 1 < my_tiles) {
      issue(i + SKV_NBUF - 1);
      asm volatile("s_waitcnt vmcnt(%0)" ::"n"((SKV_NBUF - 1) * OPS) : "memory");   // all but the newest NBUF-1 tiles
    } else {
      dma_wait();
    }
    if ((wave + 4 * i + 1) * SKV_TILE > a.Nk) tile(i, std::true_type{});
    else tile(i, std::false_type{});
  }

  // ---- merge the four partial results (waves 1..3 -> LDS -> wave 0)
  const float l_tot = l_run + swap32_f(l_run);
  const float w_tot = w_run + swap32_f(w_run);
  __syncthreads();   // every ring is done with: the merge area overlays them
  float *mg = reinterpret_cast<float *>(smem);
  constexpr int MG = SM::MG;
  if (wave > 0) {
    float *dst = mg + (wave - 1) * MG;
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int d = 32 * db + 8 * (v / 4) + 4 * g + v % 4;
        dst[d * 32 + lr] = oacc[db][v] - w_tot;   // offset term removed
      }
    if (g == 0) {
      dst[32 * D + lr] = m_ref;
      dst[32 * D + 32 + lr] = l_tot;
    }
  }
  __syncthreads();
  if (wave == 0) {
    float m_all = m_ref;   // finite: wave 0 always owns tile 0
#pragma unroll
    for (int w = 0; w < 3; ++w) m_all = fmaxf(m_all, mg[w * MG + 32 * D + lr]);
    const float s0 = __builtin_amdgcn_exp2f(a_s * (m_ref - m_all));
    float l_all = l_tot * s0;
    float sw[3];
#pragma unroll
    for (int w = 0; w < 3; ++w) {
      const float mw = mg[w * MG + 32 * D + lr];   // -inf for a wave without tiles: weight 0
      sw[w] = __builtin_amdgcn_exp2f(a_s * (mw - m_all));
      l_all += mg[w * MG + 32 * D + 32 + lr] * sw[w];
    }
    const float inv = 1.0f / l_all;
    if (qi < a.Nq) {
      T *orow = reinterpret_cast<T *>(a.o) + b * a.sob + h * a.soh + (int64_t)qi * a.son;
#pragma unroll
      for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int aa = 0; aa < 4; ++aa) {
          float r[4];
#pragma unroll
          for (int bb = 0; bb < 4; ++bb) {
            const int v = 4 * aa + bb, d = 32 * db + 8 * aa + 4 * g + bb;
            float acc = (oacc[db][v] - w_tot) * s0;
#pragma unroll
            for (int w = 0; w < 3; ++w) acc += mg[w * MG + d * 32 + lr] * sw[w];
            r[bb] = acc * inv;
          }
          u32x2 o2;
          o2[0] = pack2<T>(r[0], r[1]);
          o2[1] = pack2<T>(r[2], r[3]);
          *reinterpret_cast<u32x2 *>(orow + 32 * db + 8 * aa + 4 * g) = o2;
        }
      if (g == 0) a.lse[tq0 + qi] = (a_s * m_all + __log2f(l_all)) * kLn2;
    }
  }
}

// ---------------------------------------------------------------------------------------------------
// The same operator for at most 16 queries per (batch, head) -- the reference's benchmark shape --
// on the 16x16x32 MFMA: a 32-key tile is two 16-key row blocks of S^T, one k-step of O^T.  A lane
// owns query lane%16 and the keys 16rb + 4(lane/16) + {0..3} of each tile; half the registers and
// half the softmax work of the 32-query kernel, so three workgroups fit a CU.
typedef float f32x4v __attribute__((ext_vector_type(4)));
__device__ __forceinline__ f32x4 mfma_h16(u32x4 a, u32x4 b, f32x4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
}
// Chunk swizzle of a code tile for this kernel: as Swz<D>, plus a term in row/16 so that the eight keys
// one transposing read touches (4G + {0..3} and 16 + 4G + {0..3}) fall into different bank groups.
template <int D> struct SwzSkv16 {
  static constexpr int CPR = D / 16;
  static __device__ __forceinline__ int swz(int row) {
    return D == 128 ? ((row / 2) ^ ((row / 16) * 4)) % 8 : ((row / 4) ^ ((row / 16) * 2)) % 4;
  }
};
constexpr int SKV16_NBUF = 3;

template <typename T, typename S, int D> __global__ __launch_bounds__(256, 2) void skv_fwd16_kernel(SkvArgs a) {
  typedef SwzSkv16<D> KSW;
  typedef TileCopy<D, SKV_TILE, 64, KSW> Copy;
  constexpr int KS = D / 32;     // 32-wide k-steps of the score product
  constexpr int DB = D / 16;     // 16-row blocks of O^T
  constexpr int OPS = Copy::N + 2;
  constexpr int K_BYTES = SKV_TILE * D, SLOT = K_BYTES + 2 * SKV_TILE * 4, WAVE = SKV16_NBUF * SLOT;
  constexpr int MG = 16 * D + 32;   // floats of one partial result: O^T [D][16], m[16], l[16]
  static_assert(3 * MG * 4 <= 4 * WAVE, "the merge area overlays the rings");
  __shared__ __attribute__((aligned(16))) unsigned char smem[4 * WAVE];

  const int bh = blockIdx.x;
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
    const int t = wave + 4 * i;
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
  for (int i = 0; i < SKV16_NBUF - 1; ++i)
    if (i < my_tiles) issue(i, i);

  // ---- this lane's query as B operand: k-step m, k-group G holds d = 64(m/2) + 16G + 8(m%2) + {0..7}
  const int qi_c = q16 < a.Nq ? q16 : a.Nq - 1;
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
  u32x4 corr_q = {0u, 0u, 0u, 0u};
  {
    const _Float16 h0 = (_Float16)rs;
    const float r1 = rs - (float)h0;
    const _Float16 h1 = (_Float16)r1;
    const _Float16 h2 = (_Float16)(r1 - (float)h1);
    if (G == 0) {
      corr_q[0] = pack_h2(-(float)h0, -(float)h1);
      corr_q[1] = pack_h2(-(float)h2, 0.f);
    }
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
    const int j0 = (wave + 4 * i) * SKV_TILE;
    u32x4 kw[2][(KS + 1) / 2];
#pragma unroll
    for (int rb = 0; rb < 2; ++rb)
#pragma unroll
      for (int mm = 0; mm < (KS + 1) / 2; ++mm)
        kw[rb][mm] = *reinterpret_cast<const u32x4 *>(slot + (k_off[rb] ^ ((4 * mm) << 4)));
    const unsigned z_a[2] = {zpp[q16], zpp[16 + q16]};
    u32x2 vr[DB];
#pragma unroll
    for (int db = 0; db < DB; ++db) vr[db] = lds_read_tr8_async(lds0 + slot_off + (vt_off ^ (db << 4)));
    // ---- scores: two 16-key row blocks
    f32x4 f[2];
#pragma unroll
    for (int rb = 0; rb < 2; ++rb) {
      f[rb] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int m = 0; m < KS; ++m)
        f[rb] = mfma_h16(expand_codes(kw[rb][m / 2][2 * (m % 2)], kw[rb][m / 2][2 * (m % 2) + 1]), qf[m], f[rb]);
      const unsigned cz = magic_zp_pair(z_a[rb], z_a[rb]);
      u32x4 corr_k = {0u, 0u, 0u, 0u};
      if (G == 0) {
        corr_k[0] = cz;
        corr_k[1] = cz & 0xffffu;
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
    lds_wait_all();
#pragma unroll
    for (int db = 0; db < DB; ++db) {
      const u32x2 w = tie(vr[db]);
      oacc[db] = mfma_h16(expand_codes(w[0], w[1]), pf, oacc[db]);
    }
  };

  int cur = 0, nxt = SKV16_NBUF - 1;   // slot of the tile in work, slot the next copy goes to
  for (int i = 0; i < my_tiles; ++i) {
    if (i + SKV16_NBUF - 1 < my_tiles) {
      issue(i + SKV16_NBUF - 1, nxt);
      asm volatile("s_waitcnt vmcnt(%0)" ::"n"((SKV16_NBUF - 1) * OPS) : "memory");
    } else {
      dma_wait();
    }
    if ((wave + 4 * i + 1) * SKV_TILE > a.Nk) tile(i, cur, std::true_type{});
    else tile(i, cur, std::false_type{});
    cur = cur + 1 == SKV16_NBUF ? 0 : cur + 1;
    nxt = nxt + 1 == SKV16_NBUF ? 0 : nxt + 1;
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
    float m_all = m_ref;   // finite: wave 0 always owns tile 0
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
    const float inv = 1.0f / l_all;
    if (q16 < a.Nq) {
      T *orow = reinterpret_cast<T *>(a.o) + b * a.sob + h * a.soh + (int64_t)q16 * a.son;
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
      if (G == 0) a.lse[tq0 + q16] = (a_s * m_all + __log2f(l_all)) * kLn2;
    }
  }
}

template <typename T, typename S, int D> static int launch_skv_fwd_tsd(const SkvAttnArgs &x, hipStream_t st) {
  SkvArgs a;
  a.q = x.q; a.codes = x.codes; a.scale = x.scale; a.zp = x.zp; a.o = x.o; a.lse = x.lse;
  a.H = x.H; a.Nq = (int)x.Nq; a.Nk = (int)x.Nk;
  a.sqb = x.sqb; a.sqh = x.sqh; a.sqn = x.sqn; a.scb = x.scb; a.sch = x.sch; a.scn = x.scn;
  a.sob = x.sob; a.soh = x.soh; a.son = x.son;
  a.sm_scale_log2 = x.sm_scale * kLog2e;
  a.qblocks = (int)((x.Nq + 31) / 32);
  const int64_t total = (int64_t)a.qblocks * x.B * x.H;
  if (total > 0x7fffffffLL) return set_error(QFA_EUNSUPPORTED, "attn_fwd_shared_kv: too many query blocks for one launch");
  if (x.Nq <= 16) skv_fwd16_kernel<T, S, D><<<dim3((unsigned)total), dim3(256), 0, st>>>(a);
  else skv_fwd_kernel<T, S, D><<<dim3((unsigned)total), dim3(256), 0, st>>>(a);
  return check_launch("qfa_attn_fwd_shared_kv");
}

template <typename T, int D> static int launch_skv_fwd_td(const SkvAttnArgs &x, hipStream_t st) {
  if (x.scale_dtype == QFA_F32) return launch_skv_fwd_tsd<T, float, D>(x, st);
  return launch_skv_fwd_tsd<T, T, D>(x, st);   // validated: scale_dtype == io_dtype
}

int launch_skv_fwd(const SkvAttnArgs &x, hipStream_t st) {
  if (x.io_dtype == QFA_F16) {
    if (x.D == 128) return launch_skv_fwd_td<_Float16, 128>(x, st);
    if (x.D == 64) return launch_skv_fwd_td<_Float16, 64>(x, st);
  } else {
    if (x.D == 128) return launch_skv_fwd_td<__bf16, 128>(x, st);
    if (x.D == 64) return launch_skv_fwd_td<__bf16, 64>(x, st);
  }
  return set_error(QFA_EUNSUPPORTED, "attn_fwd_shared_kv: head_dim must be 64 or 128");
}

}  // namespace qfa
