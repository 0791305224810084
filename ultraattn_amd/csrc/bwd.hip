// Block-sparse flash-attention backward for gfx950 (MI355X): two deterministic kernels that
// recompute P from the rows' LSE, no atomics.
//
//  dkdv_kernel : one workgroup per (key tile, head) walks the CSC column of query tiles.
//                A wavefront owns 32 key rows; K and V fragments stay in registers, the Q and
//                dO tiles stream through LDS.  Products (all 32x32x16 bf16 MFMA):
//                  S [q,key]  = Q K^T          dP[q,key]  = dO V^T
//                  dV^T[d,key] += dO^T P       dK^T[d,key] += Q^T dS
//                In the accumulator layout a lane holds one key column, so S / dP blocks
//                become, after the pointwise step, the B operands of the last two products.
//  dq_kernel   : one workgroup per (query tile, head) walks the CSR row of key tiles.
//                A wavefront owns 32 query rows; Q and dO fragments stay in registers, the K
//                and V tiles stream through LDS:
//                  S^T[key,q] = K Q^T          dP^T[key,q] = V dO^T
//                  dQ^T[d,q] += K^T dS^T
//                Here a lane holds one query column, so lse and delta are per-lane scalars.
//  P = exp2(scale*log2e*S - lse*log2e);  dS = P * (dP - delta);  dQ, dK are scaled by
//  softmax_scale on output.
#include <type_traits>
#include "ua_common.h"

namespace ua {

struct BwdParams {
  const bf16* q; const bf16* k; const bf16* v; const bf16* dout;
  const float* lse; const float* delta;
  bf16* out0; bf16* out1;                  // dkdv: dk, dv; dq: dq, unused
  const int32_t* ptr; const int32_t* idx; const uint8_t* flag; const int32_t* order;
  int batch, n_heads, n_qtiles, n_ktiles, nnz;
  Strides3 qs, ks, vs, ds, o0s, o1s;
  float scale_log2, scale;
  int heads_per_xcd;
  // Dense rectangle (no list arrays).  dq walks key tiles [0, n_ktiles) of a query tile, with
  // dense_causal [0, qt + diag_off], the last one causal; dkdv walks query tiles [0, n_qtiles) of a
  // key tile, with dense_causal [kt - diag_off, n_qtiles), the first one causal.  The walk is cut
  // into n_parts parts of part_len tiles; with out_f32 part i leaves an fp32 partial result at
  // out + i * o*_part (fp32 elements, contiguous [batch, tokens, heads, 128]) for a later sum.
  int dense, dense_causal, diag_off, n_parts, part_len, out_f32;
  int64_t o0_part, o1_part;
};

__device__ __forceinline__ void store_acc_t(bf16* row_ptr, const f32x16 (&acc)[4], float mul, int hi) {
  // acc[mb][4g+j] holds column (32*mb + 8*g + 4*hi + j) of this lane's output row
#pragma unroll
  for (int mb = 0; mb < 4; ++mb)
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      bf16x4 w;
#pragma unroll
      for (int j = 0; j < 4; ++j) w[j] = (bf16)(acc[mb][4 * g + j] * mul);
      *reinterpret_cast<bf16x4*>(row_ptr + 32 * mb + 8 * g + 4 * hi) = w;
    }
}

__device__ __forceinline__ void store_acc_f32(float* row_ptr, const f32x16 (&acc)[4], float mul, int hi) {
#pragma unroll
  for (int mb = 0; mb < 4; ++mb)
#pragma unroll
    for (int g = 0; g < 4; ++g)
      *reinterpret_cast<f32x4*>(row_ptr + 32 * mb + 8 * g + 4 * hi) =
          f32x4{acc[mb][4 * g] * mul, acc[mb][4 * g + 1] * mul, acc[mb][4 * g + 2] * mul, acc[mb][4 * g + 3] * mul};
}
// Output row of a result tensor: the caller's strided bf16 tensor, or part `part` of the fp32 partials.
__device__ __forceinline__ void store_result(const BwdParams& p, bf16* out, const Strides3& os, int64_t part_stride, int part,
                                             int b, int64_t row, int h, int64_t seq, const f32x16 (&acc)[4], float mul, int hi) {
  if (p.out_f32) {
    float* base = reinterpret_cast<float*>(out) + part * part_stride;
    store_acc_f32(base + (((int64_t)b * seq + row) * p.n_heads + h) * kHeadDim, acc, mul, hi);
  } else {
    store_acc_t(out + b * os.b + row * os.s + h * os.h, acc, mul, hi);
  }
}

constexpr int kHalf = 64;
constexpr int kHalfBytes = kHalf * kRowBytes;      // 16 KiB

// Per-lane LDS byte offsets into a tile held in the universal layout, for the first 32-row
// block; later blocks add 32*kRowBytes per block (the XOR term repeats every 16 rows).
struct LaneOffsU {
  int nat[8];      // 128-bit row-fragment reads: row lane%32, chunk 2*ks + lane/32
  int tr[4][2];    // transposing reads for d-block mbd: rows row_in (+8)
  __device__ __forceinline__ LaneOffsU(int l32, int hi, const TrLane& t) {
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) nat[ks] = lds_off_u(l32, 2 * ks + hi);
#pragma unroll
    for (int mbd = 0; mbd < 4; ++mbd) {
      tr[mbd][0] = lds_off_u(t.row_in, 4 * mbd + t.chunk_in) + t.sub;
      tr[mbd][1] = lds_off_u(t.row_in + 8, 4 * mbd + t.chunk_in) + t.sub;
    }
  }
};
// ---- dK/dV ------------------------------------------------------------------------------------
// The workgroup has 8 wavefronts in two groups of 4; wave w of either group owns key rows
// 32w..32w+31 of the key tile, and each SIMD hosts one wave of each group.  Work is handed out
// in half tiles of 64 query rows (two blocks of 32):
//   group A, half tile i  :  S = Q K^T -> P = exp2(..), left in LDS for its partner;  dV^T += dO^T P
//   group B, half tile i-1:  dS = P * dP' (dP' = dO V^T - delta, kept from the step before);
//                            dK^T += Q^T dS;   then dP' of half tile i for the next step
// Group B thus runs one half tile behind group A, nothing inside a step depends on the other
// group, and one workgroup barrier per half tile is the only synchronisation.  Both groups issue
// 32 MFMAs per step; A's order is MFMA, vector, MFMA and B's is vector, MFMA, MFMA, so one
// group's MFMAs cover the other's exp2 / pointwise work.
//
// Q / dO half tiles, P and the rows' statistics live in rings of three stages inside one LDS
// array: copies into stage i+1 are in flight while A reads stage i and B reads stage i-1.  All
// LDS accesses use absolute addresses = one per-lane register + a compile-time constant that
// names ring and stage (it fits the instructions' 16-bit offset field), so the three stages cost
// no extra address registers.  The asynchronous copies are issued from inline assembly: the
// compiler then does not order the LDS reads of other stages behind them; completion is awaited
// explicitly (s_waitcnt vmcnt(0)) before the barrier that ends the step.
#define UA_LDS __attribute__((address_space(3)))
constexpr int kPBlockBytes = 4 * 2048;      // P of one 32-row block: 4 waves x (64 lanes x 32 B)
constexpr int kPHalfBytes = 2 * kPBlockBytes;
constexpr int kStatBytes = 2 * kHalf * 4;   // -lse/scale and -delta of one half tile
constexpr int kRingQ = 0, kRingDO = 3 * kHalfBytes, kRingP = 6 * kHalfBytes, kRingStat = kRingP + 3 * kPHalfBytes;
constexpr int kDkdvLdsBytes = kRingStat + 3 * kStatBytes;
static_assert(2 * kHalfBytes + kHalfBytes / 2 + 16 * kRowBytes + 8 * kRowBytes + 256 < 65536, "stage constants fit the offset field");

__device__ __forceinline__ void keep_in_register(uint32_t& x) { asm volatile("" : "+v"(x)); }
__device__ __forceinline__ bf16x8 lds_abs_b128(uint32_t a) { return *reinterpret_cast<const UA_LDS bf16x8*>(a); }
__device__ __forceinline__ bf16x8 lds_abs_tr_pair(uint32_t a_lo, uint32_t a_hi) {
  const bf16x4 x = __builtin_amdgcn_ds_read_tr16_b64_v4bf16(reinterpret_cast<UA_LDS bf16x4*>(a_lo));
  const bf16x4 y = __builtin_amdgcn_ds_read_tr16_b64_v4bf16(reinterpret_cast<UA_LDS bf16x4*>(a_hi));
  return __builtin_shufflevector(x, y, 0, 1, 2, 3, 4, 5, 6, 7);
}
// buffer_load_dwordx4 ... lds with the LDS destination (wave-uniform) in M0; see dma16_buf.
// M0 is declared clobbered; "memory" is left out on purpose so that LDS reads of the other
// stages may be scheduled across the copy (completion is awaited explicitly at the step's end).
__device__ __forceinline__ void dma16_abs(u32x4 rsrc, uint32_t lds_addr, int voff, int soff) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
               :: "s"(lds_addr), "v"(voff), "s"(rsrc), "s"(soff) : "m0");
}
__device__ __forceinline__ u32x4 make_rsrc_words(const void* base, uint32_t bytes) {
  const uint64_t a = reinterpret_cast<uint64_t>(base);
  u32x4 r;
  r[0] = __builtin_amdgcn_readfirstlane((uint32_t)a);
  r[1] = __builtin_amdgcn_readfirstlane((uint32_t)(a >> 32) & 0xffffu);
  r[2] = __builtin_amdgcn_readfirstlane(bytes);
  r[3] = 0x00020000u;
  return r;
}

// Per-lane absolute LDS addresses (stage 0, first 32-row block) of one wave group.
struct DkdvAddr {
  uint32_t nat[8];      // 128-bit row fragments of the operand that is read row-wise
  uint32_t tr[4][2];    // transposing reads of the other operand
  uint32_t p;           // this lane's 32 bytes of P per block
  uint32_t stat;        // this lane half's 4 consecutive row statistics
};

// A block of 8 MFMAs reads 8 operand fragments from LDS.  Every block is split in two calls: the
// first issues the reads of its first fragments (and, for a row-wise block, the 4 reads that
// start the accumulator from the rows' statistic), the second runs the MFMAs, each preceded by
// the read of the fragment kAhead positions later.  The first call of block n+1 is placed ahead
// of the second call of block n, so a block never starts by waiting for LDS.
constexpr int kTrAhead = 3, kNatAhead = 4;

// Transposed operand: acc[mbd] += X^T * bfrag[t], 2 steps of 16 rows x 4 d-blocks.
template <int kImm>
__device__ __forceinline__ bf16x8 dkdv_tr_frag(const DkdvAddr& ad, int i) {
  return lds_abs_tr_pair(ad.tr[i & 3][0] + (kImm + 16 * (i >> 2) * kRowBytes), ad.tr[i & 3][1] + (kImm + 16 * (i >> 2) * kRowBytes));
}
template <int kImm>
__device__ __forceinline__ void dkdv_tr_first(const DkdvAddr& ad, bf16x8 (&fr)[8]) {
#pragma unroll
  for (int i = 0; i < kTrAhead; ++i) fr[i] = dkdv_tr_frag<kImm>(ad, i);
  __builtin_amdgcn_sched_group_barrier(0x100, 2 * kTrAhead, 0);
}
template <int kImm>
__device__ __forceinline__ void dkdv_tr_run(const DkdvAddr& ad, bf16x8 (&fr)[8], const bf16x8 (&bfrag)[2], f32x16 (&acc)[4]) {
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    if (i + kTrAhead < 8) fr[i + kTrAhead] = dkdv_tr_frag<kImm>(ad, i + kTrAhead);
    acc[i & 3] = mfma32(fr[i], bfrag[i >> 2], acc[i & 3]);
    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
    if (i + kTrAhead < 8) __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
  }
}

// Row-wise operand: one 32x32 block = stat + X[32 rows, :] * frag^T over head_dim.  The
// accumulator starts from the rows' statistic instead of zero, which folds the "- lse" /
// "- delta" of the pointwise step into the product.
template <int kImm, int kStatImm>
__device__ __forceinline__ void dkdv_nat_first(const DkdvAddr& ad, bf16x8 (&fr)[8], f32x16& acc) {
#pragma unroll
  for (int ks = 0; ks < kNatAhead; ++ks) fr[ks] = lds_abs_b128(ad.nat[ks] + kImm);
  // element i: row 8*(i/4) + 4*hi + i%4 of the block
#pragma unroll
  for (int g = 0; g < 4; ++g) {
    const f32x4 v = *reinterpret_cast<const UA_LDS f32x4*>(ad.stat + (kStatImm + 32 * g));
    acc[4 * g] = v[0]; acc[4 * g + 1] = v[1]; acc[4 * g + 2] = v[2]; acc[4 * g + 3] = v[3];
  }
  __builtin_amdgcn_sched_group_barrier(0x100, kNatAhead + 4, 0);
}
template <int kImm>
__device__ __forceinline__ void dkdv_nat_run(const DkdvAddr& ad, bf16x8 (&fr)[8], const bf16x8 (&frag)[8], f32x16& acc) {
#pragma unroll
  for (int ks = 0; ks < 8; ++ks) {
    if (ks + kNatAhead < 8) fr[ks + kNatAhead] = lds_abs_b128(ad.nat[ks + kNatAhead] + kImm);
    acc = mfma32(fr[ks], frag[ks], acc);
    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
    if (ks + kNatAhead < 8) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
  }
}

// P = exp2(scale_log2 * S') with S' = Q K^T - lse/scale (bf16, accumulator layout), written to
// the partner's slot.  nb = block of the query tile (0..3).
template <int kPImm>
__device__ __forceinline__ void dkdv_p_from_s(f32x16 s, const DkdvAddr& ad, float scale_log2,
                                              int nb, int hi, int key_l, bool causal, bf16x8 (&pb)[2]) {
  // element i: query row 32*nb + 8*(i/4) + 4*hi + i%4, key column key_l
  if (causal) {
    keep_branch();
#pragma unroll
    for (int i = 0; i < 16; ++i)
      if (key_l > 32 * nb + 8 * (i >> 2) + 4 * hi + (i & 3)) s[i] = -INFINITY;
  }
#pragma unroll
  for (int i = 0; i < 16; ++i) pb[i >> 3][i & 7] = (bf16)fast_exp2(s[i] * scale_log2);
  *reinterpret_cast<UA_LDS bf16x8*>(ad.p + kPImm) = pb[0];
  *reinterpret_cast<UA_LDS bf16x8*>(ad.p + (kPImm + 1024)) = pb[1];
}

// dS = P * dP' for one block, P (two 128-bit words per lane) read from the partner's slot.
template <int kPImm>
__device__ __forceinline__ void dkdv_p_read(const DkdvAddr& ad, u32x4 (&praw)[2]) {
  praw[0] = *reinterpret_cast<const UA_LDS u32x4*>(ad.p + kPImm);
  praw[1] = *reinterpret_cast<const UA_LDS u32x4*>(ad.p + (kPImm + 1024));
}
__device__ __forceinline__ void dkdv_ds_from_p(const u32x4 (&praw)[2], const f32x16& dp, bf16x8 (&dsb)[2]) {
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const uint32_t w = praw[i >> 3][(i & 7) >> 1];
    const float pv = __uint_as_float((i & 1) ? (w & 0xffff0000u) : (w << 16));
    dsb[i >> 3][i & 7] = (bf16)(pv * dp[i]);
  }
}

// The whole key-tile column for one wave group (kGroupB: dK, else dV).  Both groups execute the
// same sequence of barriers.
template <bool kGroupB>
__device__ __forceinline__ void dkdv_run(const BwdParams& p, uint32_t lds_base, int kt, int b,
                                         int h, int tid, int lane, int wave8, int e0, int e1, int diag, int part) {
  const int wave = wave8 & 3, l32 = lane & 31, hi = lane >> 5;
  const int64_t seq_q = (int64_t)p.n_qtiles * kTile;
  // group A keeps the K fragments, group B the V fragments (B operands): lane holds key row
  // 32*wave + lane%32, d = 16*ks + 8*hi .. +7
  const int krow = kt * kTile + wave * 32 + l32;
  const bf16* fp = kGroupB ? p.v + b * p.vs.b + (int64_t)krow * p.vs.s + h * p.vs.h + hi * 8
                           : p.k + b * p.ks.b + (int64_t)krow * p.ks.s + h * p.ks.h + hi * 8;
  bf16x8 frag[8];
#pragma unroll
  for (int ks = 0; ks < 8; ++ks) frag[ks] = *reinterpret_cast<const bf16x8*>(fp + ks * 16);
  f32x16 acc[4];       // group A: dV^T, group B: dK^T
#pragma unroll
  for (int i = 0; i < 4; ++i) acc[i] = f32x16{0};
  f32x16 dp[2];        // group B: dP' of the half tile it finishes in the next step
  dp[0] = f32x16{0};
  dp[1] = f32x16{0};

  const bf16* qbase = p.q + b * p.qs.b + h * p.qs.h;
  const bf16* dobase = p.dout + b * p.ds.b + h * p.ds.h;
  const float* lse_row = p.lse + ((int64_t)b * p.n_heads + h) * seq_q;
  const float* delta_row = p.delta + ((int64_t)b * p.n_heads + h) * seq_q;
  const int key_l = wave * 32 + l32;

  // group A reads Q row-wise (S) and dO transposed (dV); group B reads dO row-wise (dP) and Q
  // transposed (dK)
  DkdvAddr ad;
  {
    const TrLane tr(lane);
    const LaneOffsU lo(l32, hi, tr);
    const uint32_t nat_ring = lds_base + (kGroupB ? kRingDO : kRingQ), tr_ring = lds_base + (kGroupB ? kRingQ : kRingDO);
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) { ad.nat[ks] = nat_ring + lo.nat[ks]; keep_in_register(ad.nat[ks]); }
#pragma unroll
    for (int m = 0; m < 4; ++m)
#pragma unroll
      for (int t = 0; t < 2; ++t) { ad.tr[m][t] = tr_ring + lo.tr[m][t]; keep_in_register(ad.tr[m][t]); }
    ad.p = lds_base + kRingP + wave * 2048 + lane * 16;
    keep_in_register(ad.p);
    ad.stat = lds_base + kRingStat + (kGroupB ? kHalf * 4 : 0) + 16 * hi;
    keep_in_register(ad.stat);
  }

  const int q_stride = (int)p.qs.s, do_stride = (int)p.ds.s;
  int qoff[2], dooff[2];
  dma_voffsets<lds_off_u, 8>(qoff, q_stride, wave8, lane);
  dma_voffsets<lds_off_u, 8>(dooff, do_stride, wave8, lane);
  const int q_half = kHalf * q_stride * 2, do_half = kHalf * do_stride * 2;
  const uint32_t q_extent = (uint32_t)((kTile - 1) * q_stride + kHeadDim) * 2;
  const uint32_t do_extent = (uint32_t)((kTile - 1) * do_stride + kHeadDim) * 2;
  const int n_half = 2 * (e1 - e0);
  // half tile i = half (i & 1) of list entry e0 + i / 2.  The list entry (query tile, causal
  // flag) of half tile i+1 is fetched one step before it is needed, so that no step starts by
  // waiting for a scalar load.
  auto entry = [&](int i) {           // query tile | causal flag << 30
    if (n_half == 0) return 0;        // an empty column owns no list entry (the arrays may be NULL)
    const int e = min(e0 + (i >> 1), e1 - 1);
    if (p.dense) return e | ((int)(e == diag) << 30);      // the entry is the query tile itself
    return min(max(sload(p.idx, e), 0), p.n_qtiles - 1) | (sload(p.flag, e) << 30);
  };
  // rows' statistics, staged in the form the accumulators start from: threads 0..63 carry
  // -lse/softmax_scale (lse = -inf, a row without keys, stays -inf so that P = 0), threads
  // 64..127 carry -delta
  // (the raw value is only touched when it is stored to LDS at the end of a step: no wait for
  // the global load may land between the copies' issue and the step's work)
  const float neg_inv_scale = -1.f / p.scale;
  const float* stat_src = (tid < kHalf ? lse_row : delta_row) + (tid & (kHalf - 1));
  auto load_stat = [&](int i, int qt) {
    float x = 0.f;
    if (tid < 2 * kHalf) x = stat_src[qt * kTile + (i & 1) * kHalf];
    return x;
  };
  const uint32_t dma_lds = __builtin_amdgcn_readfirstlane(lds_base + wave8 * 1024);
  auto copy_in = [&](int i, int qt, int stage) {       // 8 waves x 2 copies x 1 KiB per operand
    const u32x4 rq = make_rsrc_words(qbase + (int64_t)qt * kTile * q_stride, q_extent);
    const u32x4 rd = make_rsrc_words(dobase + (int64_t)qt * kTile * do_stride, do_extent);
    const int sq = __builtin_amdgcn_readfirstlane((i & 1) * q_half), sd = __builtin_amdgcn_readfirstlane((i & 1) * do_half);
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      dma16_abs(rq, dma_lds + kRingQ + stage * kHalfBytes + j * 8192, qoff[j], sq);
      dma16_abs(rd, dma_lds + kRingDO + stage * kHalfBytes + j * 8192, dooff[j], sd);
    }
  };
  auto put_stat = [&](int stage, float x) {
    if (tid < 2 * kHalf) {
      x = tid < kHalf ? ((x == -INFINITY) ? -INFINITY : x * neg_inv_scale) : -x;
      *reinterpret_cast<UA_LDS float*>(lds_base + kRingStat + stage * kStatBytes + tid * 4) = x;
    }
  };
  int ent[2] = {0, 0};
  // One step on stage kCur = i mod 3: copies for half tile i+1 go in flight into the next stage;
  // group A works on half tile i; group B finishes half tile i-1 (previous stage) and computes dP'
  // of half tile i.
  auto step = [&](int i, auto cur_tag) {
    constexpr int kCur = decltype(cur_tag)::value, kPrev = (kCur + 2) % 3, kNext = (kCur + 1) % 3;
    if (i > n_half) return;            // workgroup-uniform: the column is done
    const bool more = i + 1 < n_half;
    const int ent_cur = ent[0], ent_next = ent[1];     // entries of half tiles i and i+1
    ent[0] = ent_next;
    ent[1] = entry(i + 2);
    float stat = 0.f;
    if (more) {
      stat = load_stat(i + 1, ent_next & 0x3fffffff);
      copy_in(i + 1, ent_next & 0x3fffffff, kNext);
    }
    constexpr int kQ0 = kCur * kHalfBytes, kQ1 = kQ0 + 32 * kRowBytes;          // blocks of this half tile
    constexpr int kPrev0 = kPrev * kHalfBytes, kPrev1 = kPrev0 + 32 * kRowBytes;  // blocks of the previous one
    bf16x8 f0[8], f1[8];       // operand fragments of the block being run / the block after it
    if (kGroupB) {
      // unconditional: in step 0 P and dP' are zero (dK += 0), in the last step the new dP' is
      // computed from stale rows and never used
      u32x4 p0[2], p1[2];
      bf16x8 ds0[2], ds1[2];
      dkdv_p_read<kPrev * kPHalfBytes>(ad, p0);
      dkdv_p_read<kPrev * kPHalfBytes + kPBlockBytes>(ad, p1);
      __builtin_amdgcn_sched_group_barrier(0x100, 4, 0);
      dkdv_tr_first<kPrev0>(ad, f0);
      dkdv_ds_from_p(p0, dp[0], ds0);
      dkdv_ds_from_p(p1, dp[1], ds1);
      dkdv_tr_first<kPrev1>(ad, f1);
      dkdv_tr_run<kPrev0>(ad, f0, ds0, acc);
      dkdv_nat_first<kQ0, kCur * kStatBytes>(ad, f0, dp[0]);
      dkdv_tr_run<kPrev1>(ad, f1, ds1, acc);
      dkdv_nat_first<kQ1, kCur * kStatBytes + 128>(ad, f1, dp[1]);
      dkdv_nat_run<kQ0>(ad, f0, frag, dp[0]);
      dkdv_nat_run<kQ1>(ad, f1, frag, dp[1]);
    } else if (i < n_half) {
      const bool causal = (ent_cur >> 30) != 0;
      bf16x8 pb0[2], pb1[2];
      f32x16 s0, s1;
      dkdv_nat_first<kQ0, kCur * kStatBytes>(ad, f0, s0);
      dkdv_nat_first<kQ1, kCur * kStatBytes + 128>(ad, f1, s1);
      dkdv_nat_run<kQ0>(ad, f0, frag, s0);
      dkdv_tr_first<kQ0>(ad, f0);
      dkdv_nat_run<kQ1>(ad, f1, frag, s1);
      dkdv_tr_first<kQ1>(ad, f1);
      dkdv_p_from_s<kCur * kPHalfBytes>(s0, ad, p.scale_log2, 2 * (i & 1), hi, key_l, causal, pb0);
      dkdv_p_from_s<kCur * kPHalfBytes + kPBlockBytes>(s1, ad, p.scale_log2, 2 * (i & 1) + 1, hi, key_l, causal, pb1);
      dkdv_tr_run<kQ0>(ad, f0, pb0, acc);
      dkdv_tr_run<kQ1>(ad, f1, pb1, acc);
    }
    if (more) put_stat(kNext, stat);
    wait_vmem_all();
    __syncthreads();     // next stage has landed, P of half tile i is visible, everyone is done with the previous stage
  };

  if (n_half > 0) {
    ent[0] = entry(0);
    ent[1] = entry(1);
    const float st0 = load_stat(0, ent[0] & 0x3fffffff);
    copy_in(0, ent[0] & 0x3fffffff, 0);
    put_stat(0, st0);
  }
  // step 0 lets group B "finish" a half tile that does not exist: its P and its Q rows (stage 2)
  // must be zero, not whatever the LDS held (0 x NaN would reach dK)
  for (int o = tid * 16; o < kPHalfBytes; o += 512 * 16)
    *reinterpret_cast<UA_LDS u32x4*>(lds_base + kRingP + 2 * kPHalfBytes + o) = u32x4{0, 0, 0, 0};
  for (int o = tid * 16; o < kHalfBytes; o += 512 * 16)
    *reinterpret_cast<UA_LDS u32x4*>(lds_base + kRingQ + 2 * kHalfBytes + o) = u32x4{0, 0, 0, 0};
  wait_vmem_all();
  __syncthreads();
  // steps 0 .. n_half (the last one only lets group B finish), three at a time so that the
  // stage is a compile-time constant
  for (int i = 0; i <= n_half; i += 3) {
    step(i, std::integral_constant<int, 0>{});
    step(i + 1, std::integral_constant<int, 1>{});
    step(i + 2, std::integral_constant<int, 2>{});
  }
  const int64_t seq_k = (int64_t)p.n_ktiles * kTile;
  if (kGroupB) store_result(p, p.out0, p.o0s, p.o0_part, part, b, krow, h, seq_k, acc, p.scale, hi);
  else         store_result(p, p.out1, p.o1s, p.o1_part, part, b, krow, h, seq_k, acc, 1.f, hi);
}

__global__ __launch_bounds__(512) void dkdv_kernel(const BwdParams p) {
  __shared__ __attribute__((aligned(1024))) unsigned char smem[kDkdvLdsBytes];
  const uint32_t lds_base = (uint32_t)(uintptr_t)(UA_LDS unsigned char*)smem;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave8 = __builtin_amdgcn_readfirstlane(tid >> 6);      // 0..7
  int pos, bh;
  map_block(blockIdx.x, p.batch * p.n_heads, p.heads_per_xcd, p.n_ktiles * p.n_parts, pos, bh);
  const int b = bh / p.n_heads, h = bh % p.n_heads;
  int kt, e0, e1, diag = -1, part = 0;
  if (p.dense) {
    part = pos / p.n_ktiles;
    kt = pos - part * p.n_ktiles;                          // column 0 is the longest of a causal rectangle
    if (p.dense_causal) diag = kt - p.diag_off;            // query tile on the diagonal (may lie outside)
    const int qbeg = p.dense_causal ? min(max(diag, 0), p.n_qtiles) : 0;
    e0 = min(max(part * p.part_len, qbeg), p.n_qtiles);
    e1 = max(min((part + 1) * p.part_len, p.n_qtiles), e0);
  } else {
    kt = min(max(sload(p.order, pos), 0), p.n_ktiles - 1);
    e0 = min(max(sload(p.ptr, kt), 0), p.nnz);
    e1 = min(max(sload(p.ptr, kt + 1), e0), p.nnz);
  }
  if (wave8 >= 4) dkdv_run<true>(p, lds_base, kt, b, h, tid, lane, wave8, e0, e1, diag, part);
  else            dkdv_run<false>(p, lds_base, kt, b, h, tid, lane, wave8, e0, e1, diag, part);
}

// dQ: one 64-key half tile for this wave's 32 query rows.
__device__ __forceinline__ void dq_half_tile(const unsigned char* sK, const unsigned char* sV, const bf16x8 (&qf)[8],
                                             const bf16x8 (&dof)[8], f32x16 (&dq)[4], const TrLane& tr,
                                             float scale_log2, float lse2, float neg_delta, int l32, int hi, int q_l,
                                             int key0, bool mask) {
#pragma unroll
  for (int mb = 0; mb < 2; ++mb) {     // 32 keys at a time
    // S^T and dP^T blocks: 16 row fragments (K and V alternating), fetched kAhead reads ahead
    // dP' = V dO^T - delta: the accumulator starts from -delta (a per-lane scalar here)
    f32x16 s = f32x16{0}, dp;
#pragma unroll
    for (int i = 0; i < 16; ++i) dp[i] = neg_delta;
    {
      constexpr int kAhead = 4;
      bf16x8 fr[16];
      auto rd = [&](int i) {
        return (i & 1) ? lds_read_b128(sV, lds_off_k(32 * mb + l32, 2 * (i >> 1) + hi))
                       : lds_read_b128(sK, lds_off_u(32 * mb + l32, 2 * (i >> 1) + hi));
      };
#pragma unroll
      for (int i = 0; i < kAhead; ++i) fr[i] = rd(i);
      __builtin_amdgcn_sched_group_barrier(0x100, kAhead, 0);
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        if (i + kAhead < 16) fr[i + kAhead] = rd(i + kAhead);
        if (i & 1) dp = mfma32(fr[i], dof[i >> 1], dp);
        else       s = mfma32(fr[i], qf[i >> 1], s);
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      }
    }
    // the first K^T fragments of the dQ product are fetched now, behind the pointwise work
    constexpr int kTAhead = 3;
    bf16x8 tfr[8];
#pragma unroll
    for (int i = 0; i < kTAhead; ++i) tfr[i] = lds_read_tr_frag<lds_off_u>(sK, tr, 32 * mb + 16 * (i >> 2), i & 3);
    // element i: key key0 + 32*mb + 8*(i/4) + 4*hi + i%4, query column q_l
    if (mask) {
      keep_branch();
#pragma unroll
      for (int i = 0; i < 16; ++i)
        if (key0 + 32 * mb + 8 * (i >> 2) + 4 * hi + (i & 3) > q_l) s[i] = -INFINITY;
    }
    bf16x8 dsb[2];
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const float pv = fast_exp2(fmaf(s[i], scale_log2, -lse2));
      dsb[i >> 3][i & 7] = (bf16)(pv * dp[i]);
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      if (i + kTAhead < 8) tfr[i + kTAhead] = lds_read_tr_frag<lds_off_u>(sK, tr, 32 * mb + 16 * ((i + kTAhead) >> 2), (i + kTAhead) & 3);
      dq[i & 3] = mfma32(tfr[i], dsb[i >> 2], dq[i & 3]);
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
    }
  }
}

__global__ __launch_bounds__(256, 2) void dq_kernel(const BwdParams p) {
  __shared__ __attribute__((aligned(1024))) unsigned char sKA[kHalfBytes];
  __shared__ __attribute__((aligned(1024))) unsigned char sVA[kHalfBytes];
  __shared__ __attribute__((aligned(1024))) unsigned char sKB[kHalfBytes];
  __shared__ __attribute__((aligned(1024))) unsigned char sVB[kHalfBytes];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l32 = lane & 31, hi = lane >> 5;
  int pos, bh;
  map_block(blockIdx.x, p.batch * p.n_heads, p.heads_per_xcd, p.n_qtiles * p.n_parts, pos, bh);
  const int b = bh / p.n_heads, h = bh % p.n_heads;
  const int64_t seq_q = (int64_t)p.n_qtiles * kTile;
  int qt, e0, e1, diag = -1, part = 0;
  if (p.dense) {
    part = pos / p.n_qtiles;
    const int line = pos - part * p.n_qtiles;
    qt = p.dense_causal ? p.n_qtiles - 1 - line : line;    // longest rows first
    if (p.dense_causal) diag = qt + p.diag_off;
    const int kend = p.dense_causal ? min(max(diag + 1, 0), p.n_ktiles) : p.n_ktiles;
    e0 = min(part * p.part_len, kend);
    e1 = min(e0 + p.part_len, kend);
  } else {
    qt = min(max(sload(p.order, pos), 0), p.n_qtiles - 1);
    e0 = min(max(sload(p.ptr, qt), 0), p.nnz);
    e1 = min(max(sload(p.ptr, qt + 1), e0), p.nnz);
  }

  const bf16* kbase = p.k + b * p.ks.b + h * p.ks.h;
  const bf16* vbase = p.v + b * p.vs.b + h * p.vs.h;
  const int k_stride = (int)p.ks.s, v_stride = (int)p.vs.s;
  int koff[4], voff[4];
  dma_voffsets<lds_off_u, 4>(koff, k_stride, wave, lane);
  dma_voffsets<lds_off_k, 4>(voff, v_stride, wave, lane);
  const int k_half = kHalf * k_stride * 2, v_half = kHalf * v_stride * 2;
  const uint32_t k_extent = (uint32_t)((kTile - 1) * k_stride + kHeadDim) * 2;
  const uint32_t v_extent = (uint32_t)((kTile - 1) * v_stride + kHeadDim) * 2;
  auto k_rsrc = [&](int kt) { return make_rsrc(kbase + (int64_t)kt * kTile * k_stride, k_extent); };
  auto v_rsrc = [&](int kt) { return make_rsrc(vbase + (int64_t)kt * kTile * v_stride, v_extent); };
  auto ktile = [&](int e) { return p.dense ? e : min(max(sload(p.idx, e), 0), p.n_ktiles - 1); };
  auto is_causal = [&](int e) { return p.dense ? (int)(e == diag) : sload(p.flag, e); };

  int kt = e0 < e1 ? ktile(e0) : 0;
  if (e0 < e1) {
    dma_half_tile_buf<4>(sKA, k_rsrc(kt), koff, 0, wave);
    dma_half_tile_buf<4>(sVA, v_rsrc(kt), voff, 0, wave);
  }

  const int q_l = wave * 32 + l32;
  const int qrow = qt * kTile + q_l;
  const bf16* qp = p.q + b * p.qs.b + (int64_t)qrow * p.qs.s + h * p.qs.h + hi * 8;
  const bf16* dop = p.dout + b * p.ds.b + (int64_t)qrow * p.ds.s + h * p.ds.h + hi * 8;
  bf16x8 qf[8], dof[8];
#pragma unroll
  for (int ks = 0; ks < 8; ++ks) {
    qf[ks] = *reinterpret_cast<const bf16x8*>(qp + ks * 16);
    dof[ks] = *reinterpret_cast<const bf16x8*>(dop + ks * 16);
  }
  const float lse_raw = p.lse[((int64_t)b * p.n_heads + h) * seq_q + qrow];
  const float lse2 = (lse_raw == -INFINITY) ? INFINITY : lse_raw * kLog2e;
  const float neg_delta = -p.delta[((int64_t)b * p.n_heads + h) * seq_q + qrow];

  f32x16 dq[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) dq[i] = f32x16{0};
  const TrLane tr(lane);

  for (int e = e0; e < e1; ++e) {
    const int causal = is_causal(e);
    const int kt_next = e + 1 < e1 ? ktile(e + 1) : kt;
    wait_vmem_all();
    __syncthreads();            // stage A (keys 0..63) landed; everyone is done with stage B
    dma_half_tile_buf<4>(sKB, k_rsrc(kt), koff, k_half, wave);
    dma_half_tile_buf<4>(sVB, v_rsrc(kt), voff, v_half, wave);
    // causal tile: queries 64..127 (waves 2, 3) see all of keys 0..63
    dq_half_tile(sKA, sVA, qf, dof, dq, tr, p.scale_log2, lse2, neg_delta, l32, hi, q_l, 0, causal && wave < 2);
    wait_vmem_all();
    __syncthreads();            // stage B landed; everyone is done with stage A
    if (e + 1 < e1) {
      dma_half_tile_buf<4>(sKA, k_rsrc(kt_next), koff, 0, wave);
      dma_half_tile_buf<4>(sVA, v_rsrc(kt_next), voff, 0, wave);
    }
    // causal tile: queries 0..63 (waves 0, 1) see none of keys 64..127
    if (!causal || wave >= 2)
      dq_half_tile(sKB, sVB, qf, dof, dq, tr, p.scale_log2, lse2, neg_delta, l32, hi, q_l, kHalf, causal);
    kt = kt_next;
  }
  store_result(p, p.out0, p.o0s, p.o0_part, part, b, qrow, h, seq_q, dq, p.scale, hi);
}

static int fill_common(BwdParams& p, const void* q, const void* k, const void* v, const void* dout,
                       const float* lse, const float* delta, const int32_t* idx, const uint8_t* flag,
                       int batch, int n_heads, int n_qtiles,
                       int n_ktiles, int nnz, int head_dim, const int64_t* qs, const int64_t* ks,
                       const int64_t* vs, const int64_t* ds, float softmax_scale) {
  if (!q || !k || !v || !dout || !lse || !delta || !qs || !ks || !vs || !ds) return UA_ERR_NULL;
  if (batch <= 0 || n_heads <= 0 || n_qtiles <= 0 || n_ktiles <= 0 || nnz < 0) return UA_ERR_SHAPE;
  if (nnz > 0 && (!idx || !flag)) return UA_ERR_NULL;          // only an empty list may leave them out
  if (flag && !aligned4(flag)) return UA_ERR_ALIGN;            // read one aligned 32-bit word at a time
  if ((int64_t)batch * n_heads * n_qtiles * UA_MAX_PARTS > INT32_MAX ||
      (int64_t)batch * n_heads * n_ktiles * UA_MAX_PARTS > INT32_MAX) return UA_ERR_SHAPE;
  if (head_dim != kHeadDim || !(softmax_scale > 0.f)) return UA_ERR_UNSUPPORTED;
  if (!aligned16(q) || !aligned16(k) || !aligned16(v) || !aligned16(dout)) return UA_ERR_ALIGN;
  if (!strides_ok(qs) || !strides_ok(ks) || !strides_ok(vs) || !strides_ok(ds)) return UA_ERR_ALIGN;
  for (const int64_t* st : {qs, ks, vs, ds})
    if (st[1] > (INT32_MAX >> 9)) return UA_ERR_SHAPE;
  p.q = (const bf16*)q; p.k = (const bf16*)k; p.v = (const bf16*)v; p.dout = (const bf16*)dout;
  p.lse = lse; p.delta = delta;
  p.batch = batch; p.n_heads = n_heads; p.n_qtiles = n_qtiles; p.n_ktiles = n_ktiles; p.nnz = nnz;
  p.qs = {qs[0], qs[1], qs[2]}; p.ks = {ks[0], ks[1], ks[2]};
  p.vs = {vs[0], vs[1], vs[2]}; p.ds = {ds[0], ds[1], ds[2]};
  p.scale = softmax_scale; p.scale_log2 = softmax_scale * kLog2e;
  const int nbh = batch * n_heads;
  p.heads_per_xcd = (nbh % 8 == 0) ? nbh / 8 : 0;
  p.ptr = nullptr; p.idx = idx; p.flag = flag; p.order = nullptr;
  p.dense = 0; p.dense_causal = 0; p.diag_off = 0; p.n_parts = 1; p.part_len = 0; p.out_f32 = 0; p.o0_part = 0; p.o1_part = 0;
  return check_device();
}

static int launch_dkdv(const BwdParams& p, hipStream_t st) {
  hipLaunchKernelGGL(dkdv_kernel, dim3((unsigned)(p.batch * p.n_heads * p.n_ktiles * p.n_parts)), dim3(512), 0, st, p);
  return hipGetLastError() == hipSuccess ? UA_OK : UA_ERR_LAUNCH;
}
static int launch_dq(const BwdParams& p, hipStream_t st) {
  hipLaunchKernelGGL(dq_kernel, dim3((unsigned)(p.batch * p.n_heads * p.n_qtiles * p.n_parts)), dim3(256), 0, st, p);
  return hipGetLastError() == hipSuccess ? UA_OK : UA_ERR_LAUNCH;
}

}  // namespace ua

extern "C" int ua_bsa_bwd_dkdv(const void* q, const void* k, const void* v, const void* dout,
                               const float* lse, const float* delta, void* dk, void* dv,
                               const int32_t* col_ptr, const int32_t* row_idx, const uint8_t* cflag,
                               const int32_t* k_order,
                               int batch, int n_heads, int n_qtiles, int n_ktiles, int nnz, int head_dim,
                               const int64_t* q_strides, const int64_t* k_strides, const int64_t* v_strides,
                               const int64_t* do_strides, const int64_t* dk_strides, const int64_t* dv_strides,
                               float softmax_scale, void* stream) {
  using namespace ua;
  BwdParams p;
  if (int rc = fill_common(p, q, k, v, dout, lse, delta, row_idx, cflag, batch, n_heads, n_qtiles, n_ktiles, nnz,
                           head_dim, q_strides, k_strides, v_strides, do_strides, softmax_scale)) return rc;
  if (!dk || !dv || !col_ptr || !k_order || !dk_strides || !dv_strides) return UA_ERR_NULL;
  if (!aligned16(dk) || !aligned16(dv) || !strides_ok(dk_strides) || !strides_ok(dv_strides)) return UA_ERR_ALIGN;
  p.out0 = (bf16*)dk; p.out1 = (bf16*)dv;
  p.o0s = {dk_strides[0], dk_strides[1], dk_strides[2]};
  p.o1s = {dv_strides[0], dv_strides[1], dv_strides[2]};
  p.ptr = col_ptr; p.idx = row_idx; p.flag = cflag; p.order = k_order;
  return launch_dkdv(p, (hipStream_t)stream);
}

extern "C" int ua_bsa_bwd_dq(const void* q, const void* k, const void* v, const void* dout,
                             const float* lse, const float* delta, void* dq,
                             const int32_t* row_ptr, const int32_t* col_idx, const uint8_t* flag,
                             const int32_t* q_order,
                             int batch, int n_heads, int n_qtiles, int n_ktiles, int nnz, int head_dim,
                             const int64_t* q_strides, const int64_t* k_strides, const int64_t* v_strides,
                             const int64_t* do_strides, const int64_t* dq_strides,
                             float softmax_scale, void* stream) {
  using namespace ua;
  BwdParams p;
  if (int rc = fill_common(p, q, k, v, dout, lse, delta, col_idx, flag, batch, n_heads, n_qtiles, n_ktiles, nnz,
                           head_dim, q_strides, k_strides, v_strides, do_strides, softmax_scale)) return rc;
  if (!dq || !row_ptr || !q_order || !dq_strides) return UA_ERR_NULL;
  if (!aligned16(dq) || !strides_ok(dq_strides)) return UA_ERR_ALIGN;
  p.out0 = (bf16*)dq; p.out1 = nullptr;
  p.o0s = {dq_strides[0], dq_strides[1], dq_strides[2]};
  p.o1s = p.o0s;
  p.ptr = row_ptr; p.idx = col_idx; p.flag = flag; p.order = q_order;
  return launch_dq(p, (hipStream_t)stream);
}

extern "C" int ua_dense_bwd(const void* dout, const void* q, const void* k, const void* v,
                            const float* lse, const float* delta, void* dq, void* dk, void* dv,
                            int batch, int n_heads, int seqlen_q, int seqlen_k, int head_dim,
                            const int64_t* q_strides, const int64_t* k_strides, const int64_t* v_strides,
                            const int64_t* do_strides, const int64_t* dq_strides, const int64_t* dk_strides,
                            const int64_t* dv_strides, float softmax_scale, int causal,
                            void* workspace, int64_t workspace_bytes, void* stream) {
  using namespace ua;
  if (seqlen_q <= 0 || seqlen_k <= 0 || seqlen_q % kTile || seqlen_k % kTile) return UA_ERR_SHAPE;
  const int n_qtiles = seqlen_q / kTile, n_ktiles = seqlen_k / kTile;
  if (!dq || !dk || !dv || !dq_strides || !dk_strides || !dv_strides) return UA_ERR_NULL;
  if (!aligned16(dq) || !aligned16(dk) || !aligned16(dv) || !strides_ok(dq_strides) || !strides_ok(dk_strides) ||
      !strides_ok(dv_strides)) return UA_ERR_ALIGN;
  BwdParams p;
  if (int rc = fill_common(p, q, k, v, dout, lse, delta, nullptr, nullptr, batch, n_heads, n_qtiles, n_ktiles, 0,
                           head_dim, q_strides, k_strides, v_strides, do_strides, softmax_scale)) return rc;
  hipStream_t st = (hipStream_t)stream;
  p.dense = 1; p.dense_causal = causal != 0; p.diag_off = n_ktiles - n_qtiles;
  const DenseSplit d = dense_split(batch, n_heads, n_qtiles, n_ktiles);
  unsigned char* ws = static_cast<unsigned char*>(workspace);
  const bool ws_ok = workspace && aligned16(workspace) && workspace_bytes >= d.bwd_total;
  const void* parts[UA_MAX_PARTS];

  // dK, dV: one workgroup per (key tile, head) walks the query tiles; few key tiles -> parts of the query range
  {
    BwdParams c = p;
    c.out0 = (bf16*)dk; c.out1 = (bf16*)dv;
    c.o0s = {dk_strides[0], dk_strides[1], dk_strides[2]};
    c.o1s = {dv_strides[0], dv_strides[1], dv_strides[2]};
    c.part_len = n_qtiles;
    if (d.dkdv_parts > 1 && ws_ok) {
      const int len = (n_qtiles + d.dkdv_parts - 1) / d.dkdv_parts;
      const int n = (n_qtiles + len - 1) / len;
      float* base = reinterpret_cast<float*>(ws);
      ws += (int64_t)d.dkdv_parts * d.dkdv_bytes;
      c.n_parts = n; c.part_len = len; c.out_f32 = 1;
      c.o0_part = c.o1_part = d.dkdv_bytes / 4;
      c.out0 = reinterpret_cast<bf16*>(base);
      c.out1 = reinterpret_cast<bf16*>(base + d.dkdv_bytes / 8);
      if (int rc = launch_dkdv(c, st)) return rc;
      for (int i = 0; i < n; ++i) parts[i] = base + i * c.o0_part;
      if (int rc = launch_grad_sum(parts, n, true, dk, dk_strides, batch, seqlen_k, n_heads, 1.f, st)) return rc;
      for (int i = 0; i < n; ++i) parts[i] = base + d.dkdv_bytes / 8 + i * c.o1_part;
      if (int rc = launch_grad_sum(parts, n, true, dv, dv_strides, batch, seqlen_k, n_heads, 1.f, st)) return rc;
    } else if (int rc = launch_dkdv(c, st)) {
      return rc;
    }
  }
  // dQ: one workgroup per (query tile, head) walks the key tiles; few query tiles -> parts of the key range
  {
    BwdParams c = p;
    c.out0 = (bf16*)dq; c.out1 = nullptr;
    c.o0s = {dq_strides[0], dq_strides[1], dq_strides[2]};
    c.o1s = c.o0s;
    c.part_len = n_ktiles;
    if (d.dq_parts > 1 && ws_ok) {
      const int len = (n_ktiles + d.dq_parts - 1) / d.dq_parts;
      const int n = (n_ktiles + len - 1) / len;
      float* base = reinterpret_cast<float*>(ws);
      c.n_parts = n; c.part_len = len; c.out_f32 = 1;
      c.o0_part = d.dq_bytes / 4;
      c.out0 = reinterpret_cast<bf16*>(base);
      if (int rc = launch_dq(c, st)) return rc;
      for (int i = 0; i < n; ++i) parts[i] = base + i * c.o0_part;
      return launch_grad_sum(parts, n, true, dq, dq_strides, batch, seqlen_q, n_heads, 1.f, st);
    }
    return launch_dq(c, st);
  }
}
