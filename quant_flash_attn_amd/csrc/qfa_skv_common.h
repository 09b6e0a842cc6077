// Shared pieces of the shared-KV kernels (forward and backward): tile geometry and the helpers that
// turn INT8 codes into exact binary16 MFMA operands.
//
// A code byte c (two's complement) with its top bit flipped is the unsigned byte c + 128; placed
// under the constant high byte 0x64 it is the binary16 number 1152 + c exactly.  One XOR per dword
// and one byte permute per pair of elements therefore make a 16-bit MFMA operand out of codes, and
// the offset 1152 + zero_point is taken out again exactly by the kernels (a rank-1 MFMA update where
// the codes are contracted over d, a v_dot2 accumulation where they are contracted over tokens).
#pragma once
#include "qfa_device.h"

namespace qfa {

constexpr int SKV_TILE = 32;     // keys per tile
constexpr float SKV_RESCALE_THRESHOLD = 4.0f;   // p <= 2^4: p * scale stays inside binary16 for any fp16 K

__device__ __forceinline__ f32x16 mfma_h(u32x4 a, u32x4 b, f32x16 c) { return mfma_16b<_Float16>(a, b, c); }
// two unsigned bytes (positions A and A+1 of w) -> packed binary16 pair (1024 + byte)
template <int A> __device__ __forceinline__ unsigned magic_pair(unsigned w) {
  constexpr unsigned sel = 0x04000400u | (unsigned)A | ((unsigned)(A + 1) << 16);
  return __builtin_amdgcn_perm(0x64646464u, w, sel);
}
// 8 code bytes (two dwords) -> 8 binary16 values 1152 + code
__device__ __forceinline__ u32x4 expand_codes(unsigned w0, unsigned w1) {
  w0 ^= 0x80808080u;
  w1 ^= 0x80808080u;
  return u32x4{magic_pair<0>(w0), magic_pair<2>(w0), magic_pair<0>(w1), magic_pair<2>(w1)};
}
__device__ __forceinline__ unsigned pack_h2(float a, float b) { return pack2<_Float16>(a, b); }
// binary16 pair (1152 + za, 1152 + zb) from two zero points held in the low bytes of za and zb
__device__ __forceinline__ unsigned magic_zp_pair(unsigned za, unsigned zb) {
  return __builtin_amdgcn_perm(za, zb, 0x0c000c04u) ^ 0x64806480u;
}
// Operands of the rank-1 MFMA that removes the offset where codes are contracted over d:
//     sum_d (1152 + c_jd) x_d  -  (1152 + zp_j) * rs,      rs = sum_d x_d.
// The key side carries 1152 + zp_j in three k-slots, the query side -rs as three binary16 terms (33
// significant bits, every product exact in fp32).  When some |rs| of the block reaches 2^15 (`big`, decided
// for all queries of the MFMA together) the key side carries 32 * (1152 + zp_j) instead -- bits
// 0x7800 | (zp_j + 128), still exact -- and the query side -rs / 32, which extends the range to 2^21.
__device__ __forceinline__ bool offset_needs_x32(float rs) {
  return __builtin_amdgcn_ballot_w64(!(fabsf(rs) < 32768.0f)) != 0;
}
// dwords 0 and 1 of the key-side operand (the caller zeroes them outside k-group 0; dwords 2, 3 are zero)
__device__ __forceinline__ u32x2 offset_key_operand(unsigned z, bool big) {
  const unsigned cz = __builtin_amdgcn_perm(z, z, 0x0c000c04u) ^ (big ? 0x78807880u : 0x64806480u);
  return u32x2{cz, cz & 0xffffu};
}
// dwords 0 and 1 of the query-side operand
__device__ __forceinline__ u32x2 offset_query_operand(float rs, bool big) {
  const float x = big ? rs * 0.03125f : rs;
  const _Float16 h0 = (_Float16)x;
  const float r1 = x - (float)h0;
  const _Float16 h1 = (_Float16)r1;
  const _Float16 h2 = (_Float16)(r1 - (float)h1);
  return u32x2{pack_h2(-(float)h0, -(float)h1), pack_h2(-(float)h2, 0.f)};
}

// ds_read_b64_tr_b8, issued like lds_read_tr16_async: invisible to the compiler's wait bookkeeping
// (which would make it wait for every direct-to-LDS load in flight); use the result only after
// lds_wait_all() and through tie().
__device__ __forceinline__ u32x2 lds_read_tr8_async(unsigned addr) {
  u32x2 r;
  asm volatile("ds_read_b64_tr_b8 %0, %1" : "=v"(r) : "v"(addr) : "memory");
  return r;
}

// 16x16x32 MFMA, used on blocks of 16 queries: a 32-key tile is two 16-key row blocks of S^T and one
// k-step of the products contracted over keys.  A lane owns query lane%16 and the keys
// 16rb + 4(lane/16) + {0..3} of each tile.
__device__ __forceinline__ f32x4 mfma_h16(u32x4 a, u32x4 b, f32x4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
}
// Chunk swizzle of a code tile for the 16-query kernels: as Swz<D>, plus a term in row/16 so that the eight
// keys one transposing read touches (4G + {0..3} and 16 + 4G + {0..3}) fall into different bank groups.
template <int D> struct SwzSkv {
  static constexpr int CPR = D / 16;
  static __device__ __forceinline__ int swz(int row) {
    return D == 256 ? (row ^ ((row / 16) * 4)) % 16
           : D == 128 ? ((row / 2) ^ ((row / 16) * 4)) % 8 : ((row / 4) ^ ((row / 16) * 2)) % 4;
  }
};

// Copy of 32-key tile t of one (batch, head) into an LDS slot by direct global->LDS loads: the codes
// through `cp` (rows dense, chunks swizzled), then one dword per key for the scale and one for the zero
// point (sub-dword direct loads write lane l's zero-extended value to the dword at 4*l).  Rows past the
// end of the sequence read as zeros.  Copy::N + 2 vector-memory instructions per wave.
template <typename S, int D, typename Copy>
__device__ __forceinline__ void skv_issue_tile(const Copy &cp, unsigned char *slot, const unsigned char *codes_bh,
                                               const void *scale, const int8_t *zp, int64_t tk0, int t, int Nk,
                                               int64_t scn, int lane) {
  const int rows = min(SKV_TILE, Nk - t * SKV_TILE);
  const rsrc_t rs_k = make_rsrc(codes_bh + (int64_t)t * SKV_TILE * scn, (unsigned)((rows - 1) * (int)scn + D));
#pragma unroll
  for (int c = 0; c < Copy::N; ++c) cp.issue_one(rs_k, slot, 0, lane, c);
  const rsrc_t rs_s = make_rsrc(reinterpret_cast<const S *>(scale) + tk0 + (int64_t)t * SKV_TILE,
                                (unsigned)rows * (unsigned)sizeof(S));
  const rsrc_t rs_z = make_rsrc(zp + tk0 + (int64_t)t * SKV_TILE, (unsigned)rows);
  if (lane < SKV_TILE) {
    if constexpr (sizeof(S) == 4)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_s, (lptr_t)(slot + SKV_TILE * D), 4, lane * 4, 0, 0, 0);
    else
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_s, (lptr_t)(slot + SKV_TILE * D), 2, lane * 2, 0, 0, 0);
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_z, (lptr_t)(slot + SKV_TILE * D + SKV_TILE * 4), 1, lane, 0, 0, 0);
  }
}

// wait for every LDS operation of this wave; `tie` keeps the users of an asynchronously loaded
// register pair behind the wait that precedes it in program order
__device__ __forceinline__ void lds_wait_all() { asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); }
__device__ __forceinline__ u32x2 tie(u32x2 w) {
  asm volatile("" : "+v"(w));
  return w;
}

}  // namespace qfa
