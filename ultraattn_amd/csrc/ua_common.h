// Shared device/host helpers for the gfx950 attention kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include "../../include/ultraattn.h"

namespace ua {

typedef __bf16 bf16;
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(16))) float f32x16;
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

__device__ __forceinline__ void wait_vmem_all() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }
// Keeps a wave-uniform branch a branch (the optimiser may not turn its body into selects).
__device__ __forceinline__ void keep_branch() { asm volatile("" ::: "memory"); }

// Wave-uniform reads of the (read-only) tile-list arrays through the scalar cache.
__device__ __forceinline__ int32_t sload(const int32_t* p, int i) {
  return ((const __attribute__((address_space(4))) int32_t*)p)[i];
}
__device__ __forceinline__ int sload(const uint8_t* p, int i) {
  // the scalar unit loads dwords: fetch the aligned word that holds byte i (the entry points
  // require p on a 4-byte boundary and the array padded to a multiple of 4 bytes)
  const uintptr_t a = reinterpret_cast<uintptr_t>(p) + (uintptr_t)i;
  const uint32_t w = *reinterpret_cast<const __attribute__((address_space(4))) uint32_t*>(a & ~(uintptr_t)3);
  return (w >> (8 * (a & 3))) & 0xff;
}

// Asynchronous global -> LDS copy (buffer_load_dwordx4 ... lds), 16 bytes per lane: the wave's
// 64 lanes fill 1 KiB starting at the wave-uniform LDS address `lds_dst`, lane l at +16*l.  The
// source address is descriptor base + per-lane byte offset `voff` + wave-uniform byte offset
// `soff`, so a tile's address arithmetic stays on the scalar unit; reads beyond the descriptor's
// extent return 0.  Completion is tracked by vmcnt.
__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* base, uint32_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, bytes, 0x00020000);
}
__device__ __forceinline__ void dma16_buf(__amdgpu_buffer_rsrc_t r, unsigned char* lds_dst, int voff, int soff) {
  __builtin_amdgcn_raw_ptr_buffer_load_lds(r, (__attribute__((address_space(3))) void*)lds_dst, 16, voff, soff, 0, 0);
}
// Per-thread byte offsets for staging a [64][128] bf16 half tile (16 KiB) with NW waves: each
// thread issues 16/NW copies; copy i of wave w fills LDS rows 4*(NW*i + w) .. +3; lane l lands in
// that group's row l/16, physical 16-byte slot l%16, so it must fetch the logical chunk that the
// XOR layout `OFF` maps to that slot.
template <int (*OFF)(int, int), int NW>
__device__ __forceinline__ void dma_voffsets(int (&off)[16 / NW], int row_stride, int wave, int lane) {
#pragma unroll
  for (int i = 0; i < 16 / NW; ++i) {
    const int r = 4 * (NW * i + wave) + (lane >> 4);
    const int c = ((OFF(r, 0) - r * kRowBytes) >> 4) ^ (lane & 15);
    off[i] = (r * row_stride + c * 8) * 2;
  }
}
template <int NW>
__device__ __forceinline__ void dma_half_tile_buf(unsigned char* lds, __amdgpu_buffer_rsrc_t r, const int (&voff)[16 / NW],
                                                  int soff, int wave) {
#pragma unroll
  for (int i = 0; i < 16 / NW; ++i) dma16_buf(r, lds + (NW * i + wave) * 1024, voff[i], soff);
}

// blockIdx -> (position in the launch order, batch*head).  Consecutive workgroups go to
// consecutive XCDs.  Each XCD gets its own heads (heads_per_xcd = batch*n_heads/8 when
// divisible, else 0 = plain mapping) and works on them kHeadGroup at a time, so that the
// workgroups resident on an XCD belong to few heads and share K/V (or Q/dO) tiles in its L2.
// Within a head group the dispatch order goes team by team: a team is kTeam consecutive
// positions of the launch order (rows with the same or nearly the same tile lists); its
// members are dispatched back to back, start together and walk their lists in step.
constexpr int kHeadGroup = 2;
constexpr int kTeam = 4;
__device__ __forceinline__ void map_block(int bid, int nbh, int heads_per_xcd, int n_pos, int& pos, int& bh) {
  if (heads_per_xcd > 0) {
    const int xcd = bid & 7, idx = bid >> 3;
    const int g = (heads_per_xcd % kHeadGroup == 0) ? kHeadGroup : 1;
    const int per_group = n_pos * g;
    const int hg = idx / per_group, r = idx % per_group;
    const int full = (n_pos / kTeam) * kTeam;        // positions in complete teams
    int hs;
    if (r < full * g) {
      const int team = r / (kTeam * g), rr = r % (kTeam * g);
      hs = rr / kTeam;
      pos = team * kTeam + rr % kTeam;
    } else {                                         // the last, shorter team
      const int t = n_pos - full, rr = r - full * g;
      hs = rr / t;
      pos = full + rr % t;
    }
    bh = xcd * heads_per_xcd + hg * g + hs;
  } else {
    pos = bid / nbh;
    bh = bid % nbh;
  }
}

inline bool aligned4(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 3) == 0; }
inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }
inline bool strides_ok(const int64_t* s) { return s && s[0] % 8 == 0 && s[1] % 8 == 0 && s[2] % 8 == 0 && s[1] > 0; }

int check_device();   // UA_OK when the current device is gfx950

// ---- dense rectangles: how many parts a walk is cut into -------------------------------------
// A dense rectangle launches one workgroup per (tile line, head); with few lines and heads the
// device (256 CUs, two resident workgroups each for the row walks) stays empty while every
// workgroup walks a long list.  The walk is then cut into parts that run as workgroups of their
// own and leave partial results, combined by a second, HBM-bound kernel.  No split when the launch
// fills the device anyway or the list is short; else enough parts for ~2 workgroups per CU, at
// least two tiles each, at most UA_MAX_PARTS.
constexpr int kDenseFullLaunch = 384, kDenseTargetGroups = 512;
inline int dense_parts(int64_t n_workgroups, int list_len) {
  if (n_workgroups >= kDenseFullLaunch || list_len < 4) return 1;
  int64_t want = (kDenseTargetGroups + n_workgroups - 1) / n_workgroups;
  if (want > UA_MAX_PARTS) want = UA_MAX_PARTS;
  if (want > list_len / 2) want = list_len / 2;
  return want >= 2 ? (int)want : 1;
}
inline int64_t align256(int64_t x) { return (x + 255) / 256 * 256; }
struct DenseSplit {     // parts and workspace layout of one dense call (bytes, 256-byte aligned blocks)
  int fwd_parts, dq_parts, dkdv_parts;
  int64_t fwd_o_bytes, fwd_lse_bytes;          // per part
  int64_t dq_bytes, dkdv_bytes;                // per part (dkdv: dK then dV)
  int64_t fwd_total, bwd_total;
};
inline DenseSplit dense_split(int batch, int n_heads, int n_qtiles, int n_ktiles) {
  DenseSplit d;
  const int64_t nbh = (int64_t)batch * n_heads;
  d.fwd_parts = d.dq_parts = dense_parts(nbh * n_qtiles, n_ktiles);
  d.dkdv_parts = dense_parts(nbh * n_ktiles * 2, n_qtiles);      // one dK/dV workgroup fills a CU
  const int64_t q_elems = nbh * n_qtiles * kTile * kHeadDim, k_elems = nbh * n_ktiles * kTile * kHeadDim;
  d.fwd_o_bytes = align256(q_elems * 2);
  d.fwd_lse_bytes = align256(nbh * n_qtiles * kTile * 4);
  d.dq_bytes = align256(q_elems * 4);
  d.dkdv_bytes = 2 * align256(k_elems * 4);
  d.fwd_total = d.fwd_parts > 1 ? d.fwd_parts * (d.fwd_o_bytes + d.fwd_lse_bytes) : 0;
  d.bwd_total = (d.dq_parts > 1 ? d.dq_parts * d.dq_bytes : 0) + (d.dkdv_parts > 1 ? d.dkdv_parts * d.dkdv_bytes : 0);
  return d;
}
int launch_grad_sum(const void* const* parts, int n_parts, bool parts_fp32, void* out, const int64_t* out_strides,
                    int batch, int seqlen, int n_heads, float scale, hipStream_t st);

}  // namespace ua
