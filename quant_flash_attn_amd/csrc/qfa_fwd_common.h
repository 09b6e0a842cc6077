// Argument block, tile constants and LDS layout of the forward kernel (qfa_fwd.hip).
#pragma once
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
  int mblocks;           // query blocks of one workgroup each per (batch, head)
  int total_blocks;      // mblocks * B * H
  int blocks_per_xcd;    // ceil(total_blocks / 8)
  int group_log2;        // causal: log2 of the number of heads whose query blocks are dispatched together
};

#ifndef QFA_FWD_WAVES
#define QFA_FWD_WAVES 4
#endif
constexpr int FWD_WAVES = QFA_FWD_WAVES;   // waves (32 queries each) per workgroup
constexpr int FWD_BN = 64;
constexpr float FWD_RESCALE_THRESHOLD = 8.0f;   // log2 units the running max may lag behind

template <int D> struct FwdSmem {
  static constexpr int KSTR = D;                 // bytes per K row (dense, chunks swizzled: Swz<D>)
  static constexpr int VSTR = 2 * D;             // bytes per V row (dense, quarters swizzled: SwzQuad<2D>)
  static constexpr int K_BYTES = FWD_BN * KSTR;
  static constexpr int V_BYTES = FWD_BN * VSTR;
  static constexpr int C_BYTES = FWD_BN * 4 + FWD_BN * 16;  // key scale; correction operands (per key and k-group two dwords)
  // Tile t lives in buffer t % 3 of each of the three rings, so that a loop unrolled over three tiles addresses
  // all of them with immediate offsets
  static constexpr int NBUF = 3;
  static constexpr int OFF_C = 0;                     // the small ring first: its reads keep 16-bit immediate offsets
  static constexpr int OFF_K = OFF_C + NBUF * C_BYTES;
  static constexpr int OFF_V = OFF_K + NBUF * K_BYTES;
  static constexpr int TOTAL = OFF_V + NBUF * V_BYTES;
  static_assert(OFF_K % 256 == 0 && OFF_V % 256 == 0, "tile buffers start on a bank line");
  // head_dim 128: two workgroups per CU (2 waves per SIMD of up to 256 registers; 76 KB of LDS each); head_dim 64:
  // three (the loop fits the 168 registers of three waves per SIMD: 10 % faster than two); head_dim 256: 148 KB,
  // one workgroup, each wave has the SIMD's whole register file (the 128 O accumulators live in AccVGPRs)
  static constexpr int WG_PER_CU = D <= 64 ? 3 : D <= 128 ? 2 : 1;
  static_assert(WG_PER_CU * TOTAL <= 160 * 1024, "the workgroups of a CU share 160 KB of LDS");
};

// integer n in [-32768, 32767] -> (128*floor(n/128), n mod 128) as a packed pair of 16-bit floats
template <typename T> __device__ __forceinline__ unsigned base128_pair(int n) {
  const int hi = n >> 7, lo = n & 127;
  return pack2<T>((float)(hi * 128), (float)lo);
}


}  // namespace qfa
