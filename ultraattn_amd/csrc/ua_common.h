// Shared device/host helpers for the gfx950 attention kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include "../../include/ultraattn.h"

namespace ua {

typedef __bf16 bf16;
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(8))) float f32x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;

constexpr int kTile = UA_TILE;          // 128 x 128 kernel tile
constexpr int kHeadDim = UA_HEAD_DIM;   // 128
constexpr int kRowBytes = kHeadDim * 2; // one K/V/Q row of bf16 in LDS
constexpr int kTileBytes = kTile * kRowBytes;  // 32 KiB
constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;

struct Strides3 { int64_t b, s, h; };   // element strides of (batch, token, head)

// LDS address (bytes) of 16-byte chunk `c` (0..15) of row `r` in a [128][128] bf16 tile.
// K-type layout: chunk index XOR (row mod 16): 16 consecutive rows at one logical column
// land in 16 different 16-byte slots, so 128-bit row-fragment reads are conflict free.
__device__ __forceinline__ int lds_off_k(int r, int c) { return r * kRowBytes + ((c ^ (r & 15)) << 4); }
// V-type layout: 64-byte group index XOR (row mod 4): the 4 consecutive rows that one
// transposing 64-bit read gathers land in 4 different bank groups.
__device__ __forceinline__ int lds_off_v(int r, int c) { return r * kRowBytes + ((c ^ ((r & 3) << 2)) << 4); }

// Universal layout: chunk index XOR (row mod 16 with its two 2-bit fields swapped).  Serves
// both access patterns on one tile: 16 consecutive rows still hit 16 different slots, and 4
// consecutive rows still hit 4 different 64-byte groups.
__device__ __forceinline__ int lds_off_u(int r, int c) {
  return r * kRowBytes + ((c ^ (((r & 3) << 2) | ((r >> 2) & 3))) << 4);
}

__device__ __forceinline__ bf16x8 lds_read_b128(const unsigned char* smem, int off) {
  return *reinterpret_cast<const bf16x8*>(smem + off);
}
// Transposing LDS read: across each group of 16 lanes, lane i receives element (i) of the
// 16-element row that lanes 4j..4j+3 point at, for j = 0..3 (4 rows x 16 columns -> column i).
__device__ __forceinline__ bf16x4 lds_read_tr16_b64(const unsigned char* smem, int off) {
  typedef __attribute__((address_space(3))) bf16x4 lds_bf16x4;
  return __builtin_amdgcn_ds_read_tr16_b64_v4bf16((lds_bf16x4*)(smem + off));
}

__device__ __forceinline__ float xhalf_max(float x) {   // max over lane l and lane l^32
  auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float xhalf_sum(float x) {   // sum over lane l and lane l^32
  auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

__device__ __forceinline__ f32x16 mfma32(bf16x8 a, bf16x8 b, f32x16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
}

// Copy one [128][128] bf16 tile from global memory into LDS with the layout `OFF`
// (256 threads, 16 bytes per thread per pass, each pass covers 16 full rows).
template <int (*OFF)(int, int)>
__device__ __forceinline__ void stage_tile(unsigned char* smem, const bf16* g, int64_t row_stride, int tid) {
  const int c = tid & 15, r0 = tid >> 4;
  u32x4 val[8];
#pragma unroll
  for (int p = 0; p < 8; ++p)
    val[p] = *reinterpret_cast<const u32x4*>(g + (int64_t)(p * 16 + r0) * row_stride + c * 8);
#pragma unroll
  for (int p = 0; p < 8; ++p)
    *reinterpret_cast<u32x4*>(smem + OFF(p * 16 + r0, c)) = val[p];
}

// Per-lane constants of the transposing reads that build an A operand of X^T from a
// row-major tile X[row][col] in LDS: the MFMA row index is the tile column
// (32*mb + lane%32), the contraction index runs over tile rows.  For a 16-row step starting
// at row0, lane half hi = lane/32 supplies contraction slots j = 0..7 = tile rows
// row0 + 8*(j/4) + 4*hi + j%4, the same slots that a 32x32 accumulator block hands to the
// next product when it is reused as the B operand.
struct TrLane {
  int row_in, chunk_in, sub;
  __device__ __forceinline__ explicit TrLane(int lane) {
    const int i16 = lane & 15, grp = (lane >> 4) & 1, hi = lane >> 5;
    row_in = (i16 >> 2) + 4 * hi;
    chunk_in = 2 * grp + ((i16 & 3) >> 1);
    sub = (i16 & 1) * 8;
  }
};
template <int (*OFF)(int, int)>
__device__ __forceinline__ bf16x8 lds_read_tr_frag(const unsigned char* smem, const TrLane& t, int row0, int mb) {
  const bf16x4 lo = lds_read_tr16_b64(smem, OFF(row0 + t.row_in, 4 * mb + t.chunk_in) + t.sub);
  const bf16x4 hi = lds_read_tr16_b64(smem, OFF(row0 + 8 + t.row_in, 4 * mb + t.chunk_in) + t.sub);
  return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
}

// blockIdx -> (position in the launch order, batch*head).  Consecutive workgroups go to
// consecutive XCDs; each XCD gets its own heads so that tiles which share operands meet in
// one L2.  heads_per_xcd = batch*n_heads/8 when divisible, else 0 (plain mapping).
__device__ __forceinline__ void map_block(int bid, int nbh, int heads_per_xcd, int& pos, int& bh) {
  if (heads_per_xcd > 0) {
    const int xcd = bid & 7, idx = bid >> 3;
    pos = idx / heads_per_xcd;
    bh = xcd * heads_per_xcd + idx % heads_per_xcd;
  } else {
    pos = bid / nbh;
    bh = bid % nbh;
  }
}

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }
inline bool strides_ok(const int64_t* s) { return s && s[0] % 8 == 0 && s[1] % 8 == 0 && s[2] % 8 == 0 && s[1] > 0; }

int check_device();   // UA_OK when the current device is gfx950

}  // namespace ua
