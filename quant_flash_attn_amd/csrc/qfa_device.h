// Device-side helpers shared by the gfx950 kernels: vector types, MFMA wrappers,
// DPP lane exchanges, 16-bit float conversions.  gfx950 (CDNA4) only, wave64.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace qfa {

typedef int i32x2 __attribute__((ext_vector_type(2)));
typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef int i32x16 __attribute__((ext_vector_type(16)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef unsigned u32x2 __attribute__((ext_vector_type(2)));
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));

constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;

// ---- 16-bit float element traits ------------------------------------------------------------
template <typename T> struct Elem;
template <> struct Elem<__bf16> {
  typedef bf16x2 x2;
  typedef bf16x4 x4;
  typedef bf16x8 x8;
};
template <> struct Elem<_Float16> {
  typedef f16x2 x2;
  typedef f16x4 x4;
  typedef f16x8 x8;
};

// two fp32 -> packed pair of 16-bit floats (round to nearest even), as one dword
template <typename T> __device__ __forceinline__ unsigned pack2(float a, float b) {
  f32x2 p = {a, b};
  typename Elem<T>::x2 q = __builtin_convertvector(p, typename Elem<T>::x2);
  return __builtin_bit_cast(unsigned, q);
}
template <typename T> __device__ __forceinline__ float lo_to_f32(unsigned w) {
  typename Elem<T>::x2 q = __builtin_bit_cast(typename Elem<T>::x2, w);
  return (float)q[0];
}
template <typename T> __device__ __forceinline__ float hi_to_f32(unsigned w) {
  typename Elem<T>::x2 q = __builtin_bit_cast(typename Elem<T>::x2, w);
  return (float)q[1];
}

// c + lo(w) + hi(w) for a packed pair of 16-bit floats (v_dot2 with a pair of ones), fp32 accumulate
template <typename T> __device__ __forceinline__ float dot2_ones(unsigned w, float c);
template <> __device__ __forceinline__ float dot2_ones<__bf16>(unsigned w, float c) {
  const bf16x2 ones = {(__bf16)1.0f, (__bf16)1.0f};
  return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, w), ones, c, false);
}
template <> __device__ __forceinline__ float dot2_ones<_Float16>(unsigned w, float c) {
  const f16x2 ones = {(_Float16)1.0f, (_Float16)1.0f};
  return __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2, w), ones, c, false);
}

// The same sum written to a NEW register (the three-operand encoding; the compiler only forms the accumulate-in-place
// one and would copy c first): for a chain that starts from a value which must survive
template <typename T> __device__ __forceinline__ float dot2_ones_keep(unsigned w, float c);
template <> __device__ __forceinline__ float dot2_ones_keep<__bf16>(unsigned w, float c) {
  float r;
  asm("v_dot2_f32_bf16 %0, %1, %2, %3" : "=v"(r) : "v"(w), "s"(0x3f803f80u), "v"(c));
  return r;
}
template <> __device__ __forceinline__ float dot2_ones_keep<_Float16>(unsigned w, float c) {
  float r;
  asm("v_dot2_f32_f16 %0, %1, %2, %3" : "=v"(r) : "v"(w), "s"(0x3c003c00u), "v"(c));
  return r;
}

// ---- MFMA wrappers (A and B: 16 bytes per lane; C/D: 16 dwords per lane) ------------------------
// 32x32x32 int8:  A lane l = row l%32, 16 consecutive k at k-group l/32;  B lane l = column l%32,
// same k slots;  D lane l = column l%32, register v = row 8*(v/4) + 4*(l/32) + v%4.
__device__ __forceinline__ i32x16 mfma_i8(i32x4 a, i32x4 b, i32x16 c) {
  return __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, c, 0, 0, 0);
}
// 32x32x16 bf16/f16: A lane l = row l%32, 8 consecutive k at k-group l/32; B likewise; D as above.
template <typename T> __device__ __forceinline__ f32x16 mfma_16b(u32x4 a, u32x4 b, f32x16 c);
template <> __device__ __forceinline__ f32x16 mfma_16b<__bf16>(u32x4 a, u32x4 b, f32x16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0,
                                                 0, 0);
}
template <> __device__ __forceinline__ f32x16 mfma_16b<_Float16>(u32x4 a, u32x4 b, f32x16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0,
                                                0);
}

// 32x32x8, the older 16-bit shape (A and B: 4 elements = 8 bytes per lane, k-group l/32 holds k = 4g..4g+3): the same
// 32 cycles on the matrix pipe as the x16 shape, half the operand registers -- for products of rank <= 8
typedef short s16x4 __attribute__((ext_vector_type(4)));
template <typename T> __device__ __forceinline__ f32x16 mfma_16b_k8(u32x2 a, u32x2 b, f32x16 c);
template <> __device__ __forceinline__ f32x16 mfma_16b_k8<__bf16>(u32x2 a, u32x2 b, f32x16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x8bf16_1k(__builtin_bit_cast(s16x4, a), __builtin_bit_cast(s16x4, b), c, 0, 0, 0);
}
template <> __device__ __forceinline__ f32x16 mfma_16b_k8<_Float16>(u32x2 a, u32x2 b, f32x16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x8f16(__builtin_bit_cast(f16x4, a), __builtin_bit_cast(f16x4, b), c, 0, 0, 0);
}

// ---- lane exchanges ---------------------------------------------------------------------------
// DPP controls: quad_perm [1,0,3,2] = 0xB1, [2,3,0,1] = 0x4E, row_half_mirror = 0x141, row_mirror = 0x140
template <int CTRL> __device__ __forceinline__ float dpp_f(float x) {
  int xi = __builtin_bit_cast(int, x);
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(xi, xi, CTRL, 0xf, 0xf, false));
}
template <int CTRL> __device__ __forceinline__ int dpp_i(int x) {
  return __builtin_amdgcn_update_dpp(x, x, CTRL, 0xf, 0xf, false);
}
// value held by lane (l ^ 32)
__device__ __forceinline__ float swap32_f(float x) { return __shfl_xor(x, 32, 64); }

// max of x over the lane pair (l, l ^ 32).  v_permlane32_swap exchanges the upper half of its first
// register with the lower half of its second; fed two copies of x it leaves {lo,lo} and {hi,hi}.
// (Inline asm: the builtin's second result is not usable with this compiler; the instruction needs
// two wait states after a vector write of its operands.)
__device__ __forceinline__ float max_across_halves(float x) {
  float lo = x, hi = x;
  asm("s_nop 1\n\tv_permlane32_swap_b32 %0, %1" : "+v"(lo), "+v"(hi));
  return fmaxf(lo, hi);
}

// ---- direct global -> LDS tile copies -------------------------------------------------------------
// global_load_lds_dwordx4 writes lane l's 16 bytes to LDS[wave-uniform base + 16*l], so a tile lands
// in LDS as dense rows without padding.  Bank conflicts are avoided by an XOR swizzle applied on the
// global side: the 16-byte slot (row r, position q) holds the row's chunk q ^ swz(r), with swz
// chosen so that 16 consecutive rows read at the same logical chunk hit 16 different 16-byte slots
// of the 256-byte bank line.
template <int ROW_BYTES> struct Swz {
  static constexpr int CPR = ROW_BYTES / 16;                 // chunks per row (4, 8, 16 or 32)
  static constexpr int RP = CPR >= 16 ? 1 : 16 / CPR;        // rows per 256 bytes (1 for rows of one or more lines)
  static constexpr int MOD = CPR >= 16 ? 16 : CPR;           // only the slot inside the 256-byte line matters
  static constexpr int PERIOD = RP * MOD;                    // swz(row + PERIOD) == swz(row)
  static __device__ __forceinline__ int swz(int row) { return (row / RP) % MOD; }
  // byte offset of logical chunk c of row r inside the tile
  static __device__ __forceinline__ int off(int r, int c) { return r * ROW_BYTES + ((c ^ swz(r)) << 4); }
};

// Raw buffer descriptor over [p, p + bytes): loads through it take a per-lane 32-bit offset plus a
// scalar offset (no 64-bit address arithmetic on the vector pipe) and return zero out of range.
typedef __amdgpu_buffer_rsrc_t rsrc_t;
__device__ __forceinline__ rsrc_t make_rsrc(const void *p, unsigned bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(p), 0, (int)bytes, 0x00020000);
}

typedef const __attribute__((address_space(1))) void *gptr_t;
typedef __attribute__((address_space(3))) void *lptr_t;

// Swizzle for tiles of 16-bit elements that are read back with ds_read_b64_tr_b16: there the 32 lanes
// of one k-group read 64 contiguous bytes from each of 4 consecutive rows, so the XOR moves whole
// 64-byte quarters of the 256-byte bank line: position q of row r holds chunk q ^ swz(r).
template <int ROW_BYTES> struct SwzQuad {
  static constexpr int CPR = ROW_BYTES / 16;
  static constexpr int RPL = ROW_BYTES >= 256 ? 1 : 256 / ROW_BYTES;   // rows per 256-byte line
  static constexpr int QPR = ROW_BYTES >= 256 ? 4 : ROW_BYTES / 64;      // quarters the XOR moves over (one line at most)
  static constexpr int PERIOD = RPL * QPR;                               // swz(row + PERIOD) == swz(row)
  static __device__ __forceinline__ int swz(int row) { return 4 * ((row / RPL) % QPR); }
};

// Layout for a [row][d] tile of 16-bit floats that is read BOTH ways: row-wise (16 lanes = 16 consecutive
// rows at one logical chunk) and through the transposing reads (32 lanes = 4 consecutive rows x 64
// contiguous bytes).  The row's low bits move the 64-byte quarter, bits 2-3 the chunk inside the quarter, so
// either pattern lands on 16 different 16-byte slots of the 256-byte bank line.
template <int ROW_BYTES> struct SwzDual {
  static_assert(ROW_BYTES == 512 || ROW_BYTES == 256 || ROW_BYTES == 128, "rows of 256, 128 or 64 16-bit floats");
  static constexpr int CPR = ROW_BYTES / 16;
  // the part of the XOR that moves quarters (a function of the row's low bits only)
  static __device__ __forceinline__ int quarter(int row) { return ROW_BYTES >= 256 ? (row & 3) : ((row >> 1) & 1); }
  static __device__ __forceinline__ int swz(int row) { return (quarter(row) << 2) | ((row >> 2) & 3); }
  static __device__ __forceinline__ int off(int r, int c) { return r * ROW_BYTES + ((c ^ swz(r)) << 4); }
};

// rows [row0, row0+ROWS) (clamped to row_max) of a row-major global array -> swizzled LDS tile; NT threads
template <int ROW_BYTES, int ROWS, int NT, typename S = Swz<ROW_BYTES>>
__device__ __forceinline__ void dma_rows(const unsigned char *g, int64_t gstride, int row0, int row_max,
                                         unsigned char *lds, int tid) {
  constexpr int TOTAL = ROWS * S::CPR;
#pragma unroll
  for (int i = 0; i < (TOTAL + NT - 1) / NT; ++i) {
    const int p = tid + NT * i;
    if (TOTAL % NT == 0 || p < TOTAL) {
      const int row = p / S::CPR, pos = p % S::CPR;
      const int c = pos ^ S::swz(row);
      const int rr = min(row0 + row, row_max);
      __builtin_amdgcn_global_load_lds((gptr_t)(g + (int64_t)rr * gstride + c * 16),
                                       (lptr_t)(lds + ((tid & ~63) + NT * i) * 16), 16, 0, 0);
    }
  }
}
// The same copy for FULL tiles (no row clamping), with everything per-thread computed once: off[]
// holds the thread's byte offsets from the tile's first row, and each copy rebases a buffer
// descriptor to that row with scalar arithmetic, so a tile costs one instruction per chunk and thread.
template <int ROW_BYTES, int ROWS, int NT, typename S = Swz<ROW_BYTES>> struct TileCopy {
  static constexpr int TOTAL = ROWS * S::CPR;
  static constexpr int N = (TOTAL + NT - 1) / NT;
  unsigned off[N];
  __device__ __forceinline__ void init(unsigned gstride, int tid) {
#pragma unroll
    for (int i = 0; i < N; ++i) {
      const int p = tid + NT * i, row = p / S::CPR, pos = p % S::CPR;
      off[i] = (unsigned)row * gstride + (unsigned)((pos ^ S::swz(row)) << 4);
    }
  }
  // one chunk (index i < N) of a copy whose descriptor the caller made with make_rsrc(tile_base, ...)
  __device__ __forceinline__ void issue_one(rsrc_t rs, unsigned char *lds, int wave_u, int tid, int i) const {
    if (TOTAL % NT == 0 || tid + NT * i < TOTAL)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, (lptr_t)(lds + (wave_u * 64 + NT * i) * 16), 16, (int)off[i], 0, 0, 0);
  }
  // tile_base and lds must be wave-uniform; wave_u = wave index held in a scalar register
  __device__ __forceinline__ void issue(const void *tile_base, unsigned char *lds, int wave_u, int tid) const {
    const rsrc_t rs = make_rsrc(tile_base, 0x7fffffffu);
#pragma unroll
    for (int i = 0; i < N; ++i)
      if (TOTAL % NT == 0 || tid + NT * i < TOTAL)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, (lptr_t)(lds + (wave_u * 64 + NT * i) * 16), 16, (int)off[i], 0, 0, 0);
  }
};
// TileCopy for tiles whose chunks all look alike from a thread's point of view: chunk i of a thread lies
// i * (NT / CPR) rows below its chunk 0 at the same swizzled position (the rows per chunk are a multiple of the
// swizzle's period), so ONE per-thread offset serves every chunk and the step goes into the scalar offset of the load.
template <int ROW_BYTES, int ROWS, int NT, typename S = Swz<ROW_BYTES>> struct TileCopyU {
  static constexpr int TOTAL = ROWS * S::CPR;
  static constexpr int N = TOTAL / NT;
  static constexpr int RPC = NT / S::CPR;   // rows per chunk
  static_assert(TOTAL % NT == 0 && NT % S::CPR == 0 && RPC % S::PERIOD == 0, "chunks must repeat the swizzle");
  unsigned off0;    // per thread
  unsigned step;    // uniform: bytes between a thread's consecutive chunks
  __device__ __forceinline__ void init(unsigned gstride, int tid) {
    const int row = tid / S::CPR, pos = tid % S::CPR;
    off0 = (unsigned)row * gstride + (unsigned)((pos ^ S::swz(row)) << 4);
    step = (unsigned)RPC * gstride;
  }
  // chunk i (a compile-time constant at the call site) of a copy through the descriptor of the tile's first row
  __device__ __forceinline__ void issue_one(rsrc_t rs, unsigned char *lds, int wave_u, int i) const {
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, (lptr_t)(lds + (wave_u * 64 + NT * i) * 16), 16, (int)off0,
                                             (int)(step * (unsigned)i), 0, 0);
  }
  __device__ __forceinline__ void issue(const void *tile_base, unsigned char *lds, int wave_u) const {
    const rsrc_t rs = make_rsrc(tile_base, 0x7fffffffu);
#pragma unroll
    for (int i = 0; i < N; ++i) issue_one(rs, lds, wave_u, i);
  }
};
// dense swizzle-free layout for TileCopy (contiguous bytes)
template <int ROW_BYTES> struct NoSwz {
  static constexpr int CPR = ROW_BYTES / 16;
  static __device__ __forceinline__ int swz(int) { return 0; }
};

// BYTES contiguous bytes, copied as they are
template <int BYTES, int NT>
__device__ __forceinline__ void dma_flat(const unsigned char *g, unsigned char *lds, int tid) {
  constexpr int TOTAL = BYTES / 16;
#pragma unroll
  for (int i = 0; i < (TOTAL + NT - 1) / NT; ++i) {
    const int p = tid + NT * i;
    if (TOTAL % NT == 0 || p < TOTAL)
      __builtin_amdgcn_global_load_lds((gptr_t)(g + p * 16), (lptr_t)(lds + ((tid & ~63) + NT * i) * 16), 16, 0, 0);
  }
}
// all direct loads of this wave have landed (vmcnt(0)); follow with a barrier before other waves read
__device__ __forceinline__ void dma_wait() { __builtin_amdgcn_s_waitcnt(0x0f70); }
// ds_read_b64_tr_b16: inside each group of 16 lanes, lane i receives element i%4 of the four 8-byte
// rows addressed by lanes (i%16)/4, +4, +8, +12 of its group -- a 16-bit transpose on the way out of LDS.
// It is issued behind the compiler's back, with an explicit wait: the compiler makes every such read
// it knows of (__builtin_amdgcn_ds_read_tr16_b64) wait for ALL outstanding direct-to-LDS loads (it
// cannot tell which buffer they fill), which would expose the latency of the next tile's copy once
// per tile.  The asm form is invisible to that bookkeeping, so the result must not be used before
// one of the waits below, which take the loaded registers as operands to keep their consumers
// behind them.
// LDS operations return in order: lgkmcnt(N) guarantees everything but the last N issued is there.
__device__ __forceinline__ unsigned lds_addr(const void *p) { return (unsigned)(size_t)(lptr_t)p; }
template <int OFF> __device__ __forceinline__ u32x2 lds_read_tr16_async(unsigned addr) {
  u32x2 r;
  asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(r) : "v"(addr), "n"(OFF));
  return r;
}
// The same for plain 16-byte and 8-byte reads (a loop that times every LDS request itself issues all of them this way)
template <int OFF> __device__ __forceinline__ u32x4 lds_read_b128_async(unsigned addr) {
  u32x4 r;
  asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(r) : "v"(addr), "n"(OFF));
  return r;
}
template <int OFF> __device__ __forceinline__ u32x2 lds_read_b64_async(unsigned addr) {
  u32x2 r;
  asm volatile("ds_read_b64 %0, %1 offset:%2" : "=v"(r) : "v"(addr), "n"(OFF));
  return r;
}
// wait until at most N LDS operations of this wave are outstanding; the values named are tied behind the wait
template <typename A> __device__ __forceinline__ void lds_tie(A &a) { asm volatile("" : "+v"(a)); }
template <typename A, int K> __device__ __forceinline__ void lds_tie(A (&a)[K]) {
#pragma unroll
  for (int i = 0; i < K; ++i) asm volatile("" : "+v"(a[i]));
}
template <int N, typename... A> __device__ __forceinline__ void lds_wait_for(A &...a) {
  asm volatile("s_waitcnt lgkmcnt(%0)" : : "n"(N) : "memory");
  (lds_tie(a), ...);
}
template <int N> __device__ __forceinline__ void lds_wait_async(u32x2 (&r)[8]) {
  asm volatile("s_waitcnt lgkmcnt(%8)"
               : "+v"(r[0]), "+v"(r[1]), "+v"(r[2]), "+v"(r[3]), "+v"(r[4]), "+v"(r[5]), "+v"(r[6]), "+v"(r[7])
               : "n"(N)
               : "memory");
}
template <int N> __device__ __forceinline__ void lds_wait_async(u32x2 (&r)[16]) {
  asm volatile("s_waitcnt lgkmcnt(%16)"
               : "+v"(r[0]), "+v"(r[1]), "+v"(r[2]), "+v"(r[3]), "+v"(r[4]), "+v"(r[5]), "+v"(r[6]), "+v"(r[7]),
                 "+v"(r[8]), "+v"(r[9]), "+v"(r[10]), "+v"(r[11]), "+v"(r[12]), "+v"(r[13]), "+v"(r[14]), "+v"(r[15])
               : "n"(N)
               : "memory");
}
template <int N> __device__ __forceinline__ void lds_wait_async(u32x2 (&r)[4]) {
  asm volatile("s_waitcnt lgkmcnt(%4)" : "+v"(r[0]), "+v"(r[1]), "+v"(r[2]), "+v"(r[3]) : "n"(N) : "memory");
}
// A wave's 32 x D result tile, held as the transposed accumulators of the 32x32 MFMAs (lane l: row l%32, register
// quad aa of block db: columns 32db + 8aa + 4(l/32) + {0..3}), scaled, rounded to T and written to rows
// row0 .. row0+31 (those below nrows) of a row-major tensor.  Stored directly, one instruction would write 16 bytes
// to each of 32 rows; the tile goes through `stage` (32 * 2D bytes of LDS owned by this wave, not in use by anybody
// else) and leaves as whole rows, 16 bytes per lane.  Chunks are XORed with the row so that the 32 rows of one LDS
// write spread over the banks.
template <typename T, int D>
__device__ __forceinline__ void store_tile_rows(const f32x16 (&acc)[D / 32], float scale, unsigned char *stage,
                                                T *base, int64_t row_stride, int row0, int nrows, int lane) {
  constexpr int ROWB = 2 * D, CPR = ROWB / 16;
  asm volatile("" : "+v"(lane));   // addresses are formed here, not hoisted above the caller's main loop
  const int lr = lane % 32, g = lane / 32;
#pragma unroll
  for (int db = 0; db < D / 32; ++db)
#pragma unroll
    for (int aa = 0; aa < 4; ++aa) {
      u32x2 w;
      w[0] = pack2<T>(acc[db][4 * aa + 0] * scale, acc[db][4 * aa + 1] * scale);
      w[1] = pack2<T>(acc[db][4 * aa + 2] * scale, acc[db][4 * aa + 3] * scale);
      *reinterpret_cast<u32x2 *>(stage + lr * ROWB + (((4 * db + aa) ^ (lr % CPR)) * 16) + 8 * g) = w;
    }
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // the wave reads back only what it wrote itself
#pragma unroll
  for (int i = 0; i < 32 * CPR / 64; ++i) {
    const int p = lane + 64 * i, row = p / CPR, c = p % CPR;
    const u32x4 w = *reinterpret_cast<const u32x4 *>(stage + row * ROWB + ((c ^ (row % CPR)) * 16));
    if (row0 + row < nrows) *reinterpret_cast<u32x4 *>(base + (int64_t)(row0 + row) * row_stride + c * 8) = w;
  }
}

// Workgroup barrier that orders LDS traffic only.  __syncthreads() also waits for every outstanding
// global access, including direct-to-LDS loads issued for a LATER tile, which would serialise the
// prefetch; this one leaves them in flight (pair it with dma_wait() where a tile must have landed).
__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

}  // namespace qfa
