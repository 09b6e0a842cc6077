// Per-token asymmetric INT8 quantizer and its inverse for gfx950.
//
// Arithmetic contract (asymmetric_quant.py:66-106 of the reference): per token row,
//   scale = (max - min) / 255 (1 if 0);  zp = clamp(roundf(-128 - min/scale));
//   code  = clamp(roundf(x/scale + zp)),  every step one IEEE binary32 operation.
// This file is compiled with -ffp-contract=off and without fast-math so that `/` is the
// correctly rounded division and nothing is fused or re-associated: codes and zero points
// are bit-identical to a CPU evaluation of the same expressions.
//
// Mapping: a token of D elements is held by D/8 adjacent lanes, rounded up to a power of two (head dimensions
// that are not one leave the group's last lanes idle: they hold a second copy of the token's first eight
// elements, which changes no minimum or maximum, and neither add to the row sum nor store -- the reference
// masks its tail lanes the same way, asymmetric_quant.py:72-75,97-99) (8 elements = one 16-byte
// load per lane for 16-bit inputs, two for fp32), so one wave64 load instruction covers
// 512/D tokens with fully coalesced 16-byte accesses.  The row is read once, kept in
// registers, reduced with DPP lane permutes inside the lane group (no LDS), and the codes
// leave as one 8-byte store per lane.  HBM-bound in principle (D*sizeof(in) + D + 9 bytes per token,
// +2 with the 16-bit scale copy); in practice the exact arithmetic makes VALU issue the limiter, so
// the per-element instruction count is kept low (see the division and packing notes below).
#include "qfa_device.h"
#include "qfa_host.h"

namespace qfa {

// One reduction step = one instruction: the lane permute is the DPP modifier of the min / max itself.
// (Written as asm: through the builtin the permuted value comes back as an integer, and the compiler
// then spends a v_mov_b32_dpp and a canonicalising v_max on every step.  The s_nop covers the two wait
// states a DPP read needs after a vector write of the same register, which the compiler does not
// insert for instructions it cannot see.)
#define QFA_DPP_STEP(OP, CTRL)                                                                           \
  asm("s_nop 1\n\t" OP " %0, %1, %1 " CTRL " row_mask:0xf bank_mask:0xf" : "=v"(r) : "v"(v))
template <int LPT> __device__ __forceinline__ float group_min(float v) {
  float r;
  QFA_DPP_STEP("v_min_f32_dpp", "quad_perm:[1,0,3,2]"); v = r;
  if (LPT >= 4) { QFA_DPP_STEP("v_min_f32_dpp", "quad_perm:[2,3,0,1]"); v = r; }
  if (LPT >= 8) { QFA_DPP_STEP("v_min_f32_dpp", "row_half_mirror"); v = r; }
  if (LPT >= 16) { QFA_DPP_STEP("v_min_f32_dpp", "row_mirror"); v = r; }
  if (LPT >= 32) v = fminf(v, __shfl_xor(v, 16, 64));
  return v;
}
template <int LPT> __device__ __forceinline__ float group_max(float v) {
  float r;
  QFA_DPP_STEP("v_max_f32_dpp", "quad_perm:[1,0,3,2]"); v = r;
  if (LPT >= 4) { QFA_DPP_STEP("v_max_f32_dpp", "quad_perm:[2,3,0,1]"); v = r; }
  if (LPT >= 8) { QFA_DPP_STEP("v_max_f32_dpp", "row_half_mirror"); v = r; }
  if (LPT >= 16) { QFA_DPP_STEP("v_max_f32_dpp", "row_mirror"); v = r; }
  if (LPT >= 32) v = fmaxf(v, __shfl_xor(v, 16, 64));
  return v;
}
#undef QFA_DPP_STEP
// integer sum: `old` = 0, the identity of the addition (never used: every lane reads a valid lane),
// lets the compiler fold the permute into v_add_u32_dpp
template <int CTRL> __device__ __forceinline__ int dpp_zero(int x) { return __builtin_amdgcn_update_dpp(0, x, CTRL, 0xf, 0xf, false); }
template <int LPT> __device__ __forceinline__ int group_sum(int v) {
  v += dpp_zero<0xB1>(v);
  if (LPT >= 4) v += dpp_zero<0x4E>(v);
  if (LPT >= 8) v += dpp_zero<0x141>(v);
  if (LPT >= 16) v += dpp_zero<0x140>(v);
  if (LPT >= 32) v += __shfl_xor(v, 16, 64);
  return v;
}

template <typename T> struct Load8;
template <> struct Load8<float> {
  static __device__ __forceinline__ void run(const void *p, float (&v)[8]) {
    const f32x4 *q = reinterpret_cast<const f32x4 *>(p);
    f32x4 a = __builtin_nontemporal_load(q), b = __builtin_nontemporal_load(q + 1);
#pragma unroll
    for (int e = 0; e < 4; ++e) { v[e] = a[e]; v[4 + e] = b[e]; }
  }
};
template <> struct Load8<__bf16> {
  static __device__ __forceinline__ void run(const void *p, float (&v)[8]) {
    u32x4 w = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(p));
#pragma unroll
    for (int e = 0; e < 4; ++e) {   // bf16 -> fp32 is a 16-bit shift
      v[2 * e] = __builtin_bit_cast(float, w[e] << 16);
      v[2 * e + 1] = __builtin_bit_cast(float, w[e] & 0xffff0000u);
    }
  }
};
template <> struct Load8<_Float16> {
  static __device__ __forceinline__ void run(const void *p, float (&v)[8]) {
    f16x8 w = __builtin_bit_cast(f16x8, __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(p)));
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] = (float)w[e];
  }
};

struct QuantArgs {
  const void *x;
  int8_t *codes;
  float *scale;
  void *scale_lp;
  int8_t *zp;
  int32_t *rowsum;
  int64_t N;
  int64_t H;
  int64_t sxb, sxh, sxn, scb, sch, scn;
  int chunks_per_bh;  // ceil(N / tokens per block)
  int scale_lp_dtype;
  int D;              // head dimension (a multiple of 8, at most the kernel's DP)
};

// One block = 256 threads = U passes over 256/(DP/8) tokens of one (b,h) slice.  DP = the head dimension
// rounded up to a power of two; PARTIAL: the head dimension is smaller than DP.
template <typename T, int DP, int U, bool PARTIAL>
__device__ __forceinline__ void quant_block(const QuantArgs &a, unsigned block) {
  constexpr int LPT = DP / 8;         // lanes per token
  constexpr int TPP = 256 / LPT;      // tokens per pass
  const int tid = threadIdx.x;
  const int sub = tid % LPT;
  const bool lane_used = !PARTIAL || sub * 8 < a.D;
  const int sub_ld = lane_used ? sub : 0;   // idle lanes duplicate the token's first eight elements
  const int64_t bh = block / a.chunks_per_bh;
  const int64_t chunk = block % a.chunks_per_bh;
  const int64_t b = bh / a.H, h = bh % a.H;
  const int64_t n0 = chunk * (int64_t)(TPP * U) + tid / LPT;
  const T *xb = reinterpret_cast<const T *>(a.x) + b * a.sxb + h * a.sxh;
  int8_t *cb = a.codes + b * a.scb + h * a.sch;

  float v[U][8];
  bool live[U];
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const int64_t n = n0 + (int64_t)u * TPP;
    live[u] = n < a.N;
    const int64_t nn = live[u] ? n : a.N - 1;   // tail lanes re-read the last token, never store
    Load8<T>::run(xb + nn * a.sxn + sub_ld * 8, v[u]);
  }
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const int64_t n = n0 + (int64_t)u * TPP;
    float mn = v[u][0], mx = v[u][0];
#pragma unroll
    for (int e = 1; e < 8; ++e) { mn = fminf(mn, v[u][e]); mx = fmaxf(mx, v[u][e]); }
    mn = group_min<LPT>(mn);
    mx = group_max<LPT>(mx);
    float scale = (mx - mn) / 255.0f;
    scale = (scale == 0.0f) ? 1.0f : scale;
    // Division by the per-token scale.  In the common exponent range the quotient is formed with the
    // same FMA refinement the hardware division sequence uses (reciprocal refined once, two residual
    // corrections of the quotient), which gives the correctly rounded x/scale without the per-element
    // operand scaling; outside that range (tiny scale, huge values, NaN) the IEEE `/` is used.
    // Quotients below 2^-30 in magnitude may differ in their last bits, which cannot matter: they
    // vanish in the addition of the zero point or round to zero.
    const bool fast = (scale >= 0x1p-60f) && (fmaxf(fabsf(mn), fabsf(mx)) <= 0x1p60f);
    float r = __builtin_amdgcn_rcpf(scale);
    r = __builtin_fmaf(__builtin_fmaf(-scale, r, 1.0f), r, r);
    auto fdiv = [&](float x) -> float {
      float q = x * r;
      q = __builtin_fmaf(__builtin_fmaf(-scale, q, x), r, q);
      q = __builtin_fmaf(__builtin_fmaf(-scale, q, x), r, q);
      return q;
    };
    // roundf (ties away from zero) in three instructions: add the largest float below one half with the
    // sign of y, truncate.  Equal to roundf for every binary32 value (checked exhaustively on the CPU; the
    // classic y + 0.5 fails at 0.49999997).
    auto round_away = [](float y) -> float {
      return __builtin_truncf(y + __builtin_copysignf(0x1.fffffep-2f, y));
    };
    float q[8], qmn;
    if (fast) {
      qmn = fdiv(mn);
#pragma unroll
      for (int e = 0; e < 8; ++e) q[e] = fdiv(v[u][e]);
    } else {
      qmn = mn / scale;
#pragma unroll
      for (int e = 0; e < 8; ++e) q[e] = v[u][e] / scale;
    }
    const float zpf = -128.0f - qmn;
    const float zp = fmaxf(-128.0f, fminf(127.0f, round_away(zpf)));
    // codes leave as biased bytes: roundf(.) + 128 converted with unsigned saturation (= the clamp to
    // [-128, 127]), flipped back to two's complement with one XOR per dword
    u32x2 w = {0u, 0u};
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float y = q[e] + zp;
      const float c = round_away(y) + 128.0f;
      w[e / 4] = __builtin_amdgcn_cvt_pk_u8_f32(c, e % 4, w[e / 4]);
    }
    int sum = (int)__builtin_amdgcn_sad_u8(w[0], 0u, 0u);
    sum = (int)__builtin_amdgcn_sad_u8(w[1], 0u, (unsigned)sum) - 8 * 128;
    if (PARTIAL && !lane_used) sum = 0;
    w[0] ^= 0x80808080u;
    w[1] ^= 0x80808080u;
    sum = group_sum<LPT>(sum);
    if (live[u] && lane_used) {
      *reinterpret_cast<u32x2 *>(cb + n * a.scn + sub * 8) = w;
      if (sub == 0) {
        const int64_t t = bh * a.N + n;
        a.scale[t] = scale;
        a.zp[t] = (int8_t)(int)zp;
        if (a.rowsum) a.rowsum[t] = sum;
        if (a.scale_lp) {
          if (a.scale_lp_dtype == QFA_F16) reinterpret_cast<_Float16 *>(a.scale_lp)[t] = (_Float16)scale;
          else reinterpret_cast<__bf16 *>(a.scale_lp)[t] = (__bf16)scale;
        }
      }
    }
  }
}

template <typename T, int DP, int U, bool PARTIAL> __global__ __launch_bounds__(256) void quant_kernel(QuantArgs a) {
  quant_block<T, DP, U, PARTIAL>(a, blockIdx.x);
}
// Two tensors of one element type and head dimension in one launch (the queries and the keys of an attention call):
// the first blocks0 workgroups take tensor 0, the others tensor 1.  One launch ramp and one tail instead of two.
struct QuantPairArgs {
  QuantArgs t[2];
  unsigned blocks0;
};
template <typename T, int DP, int U, bool PARTIAL> __global__ __launch_bounds__(256) void quant_pair_kernel(QuantPairArgs p) {
  if (blockIdx.x < p.blocks0) quant_block<T, DP, U, PARTIAL>(p.t[0], blockIdx.x);
  else quant_block<T, DP, U, PARTIAL>(p.t[1], blockIdx.x - p.blocks0);
}

template <typename T, int DP> static int launch_quant_d(const QuantArgs &a0, int64_t BH, hipStream_t st) {
  constexpr int U = 4;
  constexpr int TOK = (256 / (DP / 8)) * U;
  QuantArgs a = a0;
  const int64_t chunks = (a.N + TOK - 1) / TOK;
  if (chunks * BH > 0x7fffffffLL) return set_error(QFA_EUNSUPPORTED, "quant: too many tokens for one launch");
  a.chunks_per_bh = (int)chunks;
  const dim3 grid((unsigned)(chunks * BH)), block(256);
  if (a.D == DP) quant_kernel<T, DP, U, false><<<grid, block, 0, st>>>(a);
  else quant_kernel<T, DP, U, true><<<grid, block, 0, st>>>(a);
  return check_launch("qfa_quant_per_token");
}
// head dimension rounded up to a power of two (the lane groups the reductions run over), 32 at least
static int padded_head_dim(int D) { return D <= 32 ? 32 : D <= 64 ? 64 : D <= 128 ? 128 : 256; }
template <typename T> static int launch_quant_t(const QuantArgs &a, int64_t BH, hipStream_t st) {
  switch (padded_head_dim(a.D)) {
    case 32: return launch_quant_d<T, 32>(a, BH, st);
    case 64: return launch_quant_d<T, 64>(a, BH, st);
    case 128: return launch_quant_d<T, 128>(a, BH, st);
  }
  return launch_quant_d<T, 256>(a, BH, st);
}

int launch_quant(const void *x, int x_dtype, int8_t *codes, float *scale, void *scale_lp, int scale_lp_dtype,
                 int8_t *zp, int32_t *rowsum, int64_t B, int64_t H, int64_t N, int D, int64_t sxb, int64_t sxh,
                 int64_t sxn, int64_t scb, int64_t sch, int64_t scn, hipStream_t st) {
  QuantArgs a;
  a.x = x; a.codes = codes; a.scale = scale; a.scale_lp = scale_lp; a.zp = zp; a.rowsum = rowsum;
  a.N = N; a.H = H; a.sxb = sxb; a.sxh = sxh; a.sxn = sxn; a.scb = scb; a.sch = sch; a.scn = scn;
  a.chunks_per_bh = 0; a.scale_lp_dtype = scale_lp_dtype; a.D = D;
  if (D < 8 || D > 256 || D % 8 != 0) return set_error(QFA_EUNSUPPORTED, "quant: head_dim must be a multiple of 8, at most 256");
  switch (x_dtype) {
    case QFA_F32: return launch_quant_t<float>(a, B * H, st);
    case QFA_F16: return launch_quant_t<_Float16>(a, B * H, st);
    case QFA_BF16: return launch_quant_t<__bf16>(a, B * H, st);
  }
  return set_error(QFA_EINVAL, "quant: bad x_dtype");
}

template <typename T, int DP> static int launch_quant_pair_d(QuantPairArgs p, int64_t BH, hipStream_t st) {
  constexpr int U = 4;
  constexpr int TOK = (256 / (DP / 8)) * U;
  int64_t blocks[2];
  for (int i = 0; i < 2; ++i) {
    const int64_t chunks = (p.t[i].N + TOK - 1) / TOK;
    p.t[i].chunks_per_bh = (int)chunks;
    blocks[i] = chunks * BH;
  }
  if (blocks[0] + blocks[1] > 0x7fffffffLL) return set_error(QFA_EUNSUPPORTED, "quant_pair: too many tokens for one launch");
  p.blocks0 = (unsigned)blocks[0];
  const dim3 grid((unsigned)(blocks[0] + blocks[1])), block(256);
  if (p.t[0].D == DP) quant_pair_kernel<T, DP, U, false><<<grid, block, 0, st>>>(p);
  else quant_pair_kernel<T, DP, U, true><<<grid, block, 0, st>>>(p);
  return check_launch("qfa_quant_per_token_pair");
}
template <typename T> static int launch_quant_pair_t(const QuantPairArgs &p, int64_t BH, hipStream_t st) {
  switch (padded_head_dim(p.t[0].D)) {
    case 32: return launch_quant_pair_d<T, 32>(p, BH, st);
    case 64: return launch_quant_pair_d<T, 64>(p, BH, st);
    case 128: return launch_quant_pair_d<T, 128>(p, BH, st);
  }
  return launch_quant_pair_d<T, 256>(p, BH, st);
}

int launch_quant_pair(const void *const x[2], int x_dtype, int8_t *const codes[2], float *const scale[2],
                      int8_t *const zp[2], int32_t *const rowsum[2], int64_t B, int64_t H, const int64_t N[2], int D,
                      const int64_t sx[2][3], const int64_t sc[2][3], hipStream_t st) {
  QuantPairArgs p;
  for (int i = 0; i < 2; ++i) {
    QuantArgs &a = p.t[i];
    a.x = x[i]; a.codes = codes[i]; a.scale = scale[i]; a.scale_lp = nullptr; a.zp = zp[i]; a.rowsum = rowsum[i];
    a.N = N[i]; a.H = H; a.sxb = sx[i][0]; a.sxh = sx[i][1]; a.sxn = sx[i][2];
    a.scb = sc[i][0]; a.sch = sc[i][1]; a.scn = sc[i][2];
    a.chunks_per_bh = 0; a.scale_lp_dtype = 0; a.D = D;
  }
  p.blocks0 = 0;
  switch (x_dtype) {
    case QFA_F32: return launch_quant_pair_t<float>(p, B * H, st);
    case QFA_F16: return launch_quant_pair_t<_Float16>(p, B * H, st);
    case QFA_BF16: return launch_quant_pair_t<__bf16>(p, B * H, st);
  }
  return set_error(QFA_EINVAL, "quant_pair: bad x_dtype");
}

// ---------------------------------------------------------------------------------------------
// Dequantize: out = (code - zp) * scale  (asymmetric_quant.py:160), 8 elements per lane.
struct DequantArgs {
  const int8_t *codes;
  const void *scale;
  const int8_t *zp;
  void *out;
  int64_t N, H;
  int64_t scb, sch, scn, sob, soh, son;
  int chunks_per_bh;
  int scale_dtype;
  int D;   // head dimension (a multiple of 8, at most the kernel's DP)
};

template <typename TO, int DP> __global__ __launch_bounds__(256) void dequant_kernel(DequantArgs a) {
  constexpr int LPT = DP / 8;
  constexpr int TPP = 256 / LPT;
  const int tid = threadIdx.x;
  const int sub = tid % LPT;
  const int64_t bh = blockIdx.x / a.chunks_per_bh;
  const int64_t chunk = blockIdx.x % a.chunks_per_bh;
  const int64_t b = bh / a.H, h = bh % a.H;
  const int64_t n = chunk * (int64_t)TPP + tid / LPT;
  if (n >= a.N || sub * 8 >= a.D) return;
  const int64_t t = bh * a.N + n;
  float scale;
  if (a.scale_dtype == QFA_F32) scale = reinterpret_cast<const float *>(a.scale)[t];
  else if (a.scale_dtype == QFA_F16) scale = (float)reinterpret_cast<const _Float16 *>(a.scale)[t];
  else scale = (float)reinterpret_cast<const __bf16 *>(a.scale)[t];
  const float zp = (float)a.zp[t];
  const u32x2 w = *reinterpret_cast<const u32x2 *>(a.codes + b * a.scb + h * a.sch + n * a.scn + sub * 8);
  float f[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    const int c = (int)(int8_t)((w[e / 4] >> (8 * (e % 4))) & 0xff);
    f[e] = ((float)c - zp) * scale;
  }
  TO *o = reinterpret_cast<TO *>(a.out) + b * a.sob + h * a.soh + n * a.son + sub * 8;
  if constexpr (sizeof(TO) == 4) {
    f32x4 lo = {f[0], f[1], f[2], f[3]}, hi = {f[4], f[5], f[6], f[7]};
    reinterpret_cast<f32x4 *>(o)[0] = lo;
    reinterpret_cast<f32x4 *>(o)[1] = hi;
  } else {
    u32x4 p;
#pragma unroll
    for (int e = 0; e < 4; ++e) p[e] = pack2<TO>(f[2 * e], f[2 * e + 1]);
    *reinterpret_cast<u32x4 *>(o) = p;
  }
}

template <typename TO> static int launch_dequant_t(DequantArgs a, int D, int64_t BH, hipStream_t st) {
  if (D < 8 || D > 256 || D % 8 != 0) return set_error(QFA_EUNSUPPORTED, "dequant: head_dim must be a multiple of 8, at most 256");
  a.D = D;
  D = padded_head_dim(D);
  const int tpp = 256 / (D / 8);
  const int64_t chunks = (a.N + tpp - 1) / tpp;
  if (chunks * BH > 0x7fffffffLL) return set_error(QFA_EUNSUPPORTED, "dequant: too many tokens for one launch");
  a.chunks_per_bh = (int)chunks;
  const dim3 grid((unsigned)(chunks * BH)), block(256);
  switch (D) {
    case 32: dequant_kernel<TO, 32><<<grid, block, 0, st>>>(a); break;
    case 64: dequant_kernel<TO, 64><<<grid, block, 0, st>>>(a); break;
    case 128: dequant_kernel<TO, 128><<<grid, block, 0, st>>>(a); break;
    case 256: dequant_kernel<TO, 256><<<grid, block, 0, st>>>(a); break;
    default: return set_error(QFA_EUNSUPPORTED, "dequant: head_dim must be a multiple of 8, at most 256");
  }
  return check_launch("qfa_dequant_per_token");
}

int launch_dequant(const int8_t *codes, const void *scale, int scale_dtype, const int8_t *zp, void *out,
                   int out_dtype, int64_t B, int64_t H, int64_t N, int D, int64_t scb, int64_t sch, int64_t scn,
                   int64_t sob, int64_t soh, int64_t son, hipStream_t st) {
  DequantArgs a;
  a.codes = codes; a.scale = scale; a.zp = zp; a.out = out; a.N = N; a.H = H;
  a.scb = scb; a.sch = sch; a.scn = scn; a.sob = sob; a.soh = soh; a.son = son;
  a.chunks_per_bh = 0; a.scale_dtype = scale_dtype; a.D = D;
  switch (out_dtype) {
    case QFA_F32: return launch_dequant_t<float>(a, D, B * H, st);
    case QFA_F16: return launch_dequant_t<_Float16>(a, D, B * H, st);
    case QFA_BF16: return launch_dequant_t<__bf16>(a, D, B * H, st);
  }
  return set_error(QFA_EINVAL, "dequant: bad out_dtype");
}

// ---------------------------------------------------------------------------------------------
// Row sums of given codes: rowsum[t] = sum_d codes[t][d], the side output the quantizer emits, for codes that
// arrive already quantized (the zero-point term of the INT8 score product needs them).
struct RowsumArgs {
  const int8_t *codes;
  int32_t *rowsum;
  int64_t N, H;
  int64_t scb, sch, scn;
  int chunks_per_bh;
  int D;
};

template <int DP> __global__ __launch_bounds__(256) void rowsum_kernel(RowsumArgs a) {
  constexpr int LPT = DP / 8;
  constexpr int TPP = 256 / LPT;
  const int tid = threadIdx.x;
  const int sub = tid % LPT;
  const int64_t bh = blockIdx.x / a.chunks_per_bh;
  const int64_t chunk = blockIdx.x % a.chunks_per_bh;
  const int64_t b = bh / a.H, h = bh % a.H;
  const int64_t n = chunk * (int64_t)TPP + tid / LPT;
  const int64_t nn = n < a.N ? n : a.N - 1;          // every lane takes part in the reduction
  int sum = 0;
  if (sub * 8 < a.D) {
    u32x2 w = *reinterpret_cast<const u32x2 *>(a.codes + b * a.scb + h * a.sch + nn * a.scn + sub * 8);
    w[0] ^= 0x80808080u;                               // biased bytes: code + 128
    w[1] ^= 0x80808080u;
    sum = (int)__builtin_amdgcn_sad_u8(w[0], 0u, 0u);
    sum = (int)__builtin_amdgcn_sad_u8(w[1], 0u, (unsigned)sum) - 8 * 128;
  }
  sum = group_sum<LPT>(sum);
  if (n < a.N && sub == 0) a.rowsum[bh * a.N + n] = sum;
}

int launch_rowsum(const int8_t *codes, int32_t *rowsum, int64_t B, int64_t H, int64_t N, int D, int64_t scb,
                  int64_t sch, int64_t scn, hipStream_t st) {
  if (D < 8 || D > 256 || D % 8 != 0) return set_error(QFA_EUNSUPPORTED, "code_rowsum: head_dim must be a multiple of 8, at most 256");
  RowsumArgs a;
  a.codes = codes; a.rowsum = rowsum; a.N = N; a.H = H; a.scb = scb; a.sch = sch; a.scn = scn; a.D = D;
  const int DP = padded_head_dim(D);
  const int tpp = 256 / (DP / 8);
  const int64_t chunks = (N + tpp - 1) / tpp;
  if (chunks * B * H > 0x7fffffffLL) return set_error(QFA_EUNSUPPORTED, "code_rowsum: too many tokens for one launch");
  a.chunks_per_bh = (int)chunks;
  const dim3 grid((unsigned)(chunks * B * H)), block(256);
  switch (DP) {
    case 32: rowsum_kernel<32><<<grid, block, 0, st>>>(a); break;
    case 64: rowsum_kernel<64><<<grid, block, 0, st>>>(a); break;
    case 128: rowsum_kernel<128><<<grid, block, 0, st>>>(a); break;
    default: rowsum_kernel<256><<<grid, block, 0, st>>>(a); break;
  }
  return check_launch("qfa_code_rowsum");
}

}  // namespace qfa
