// Block mask -> compacted active-tile list (CSR over query tiles, CSC over key tiles).
//
// Refinement rule (one block -> rate x rate tiles): EMPTY stays empty, FULL becomes all full,
// CAUSAL becomes causal on the sub-diagonal, full below it and empty above it.  Tiles are
// emitted row-major (query tile outer, key tile inner).
#include <algorithm>
#include <atomic>
#include <numeric>
#include <vector>
#include "ua_common.h"

// Scratch of the entry point that allocates nothing (ua_tilelist_build_device_noalloc): the
// per-row and per-column tile counts that the device builder otherwise keeps in the caller's
// `work` argument.  Every GPU the library runs on holds its own copy (256 KiB) until the process
// ends; calls on one GPU share it, so two such calls must not overlap.
static __device__ __align__(256) int32_t scratch[UA_NOALLOC_MAX_LINES + 8];

namespace ua {

// type of tile (qt, kt): 0 empty, 1 full, 2 causal
__host__ __device__ __forceinline__ int tile_type(const uint8_t* mask, int nkb, int rate, int qt, int kt) {
  const int t = mask[(int64_t)(qt / rate) * nkb + kt / rate];
  if (t != 2) return t == 1 ? 1 : 0;
  const int a = qt % rate, b = kt % rate;
  return a == b ? 2 : (a > b ? 1 : 0);
}

// Launch order: does line a (a row of the CSR, or a column of the CSC) come before line b?
//  1. Lines much longer than average (len * n > 2 * nnz) first, so that they cannot end up as
//     the tail of the launch; among them the longer block lines first (see 3), then as in 4.
//  2. The rest by their anchor index, ascending.  The anchor is the first index of the list, or
//     the last one when `from_end`: lines that share it walk common tiles (the rows of a causal
//     mask share their oldest keys, its columns their latest queries).
//  3. Among those, the lines of longer block lines first (the length of a tile's block line =
//     the list length of that block's longest tile: sub-tile rate-1 of a row block, sub-tile 0 of
//     a column block): the short lists end the group, and a list that leaves the common part
//     early does not run ahead of the lists that still walk it.
//  4. Then lexicographic order of the index lists read from the anchor, a list that is a prefix
//     (from_end: a suffix) of another sorting after it; ties by line number.  Lines that walk the
//     same K/V (or Q/dO) tiles thus sit next to each other in the launch and share them in L2.
__host__ __device__ __forceinline__ bool very_long(const int32_t* ptr, int n, int a) {
  return (int64_t)(ptr[a + 1] - ptr[a]) * n > 2 * (int64_t)ptr[n];
}
__host__ __device__ __forceinline__ bool row_precedes(const int32_t* ptr, const int32_t* idx, int n, int rate, int longest_sub,
                                                      bool from_end, int a, int b) {
  const int pa = ptr[a], pb = ptr[b];
  const int la = ptr[a + 1] - pa, lb = ptr[b + 1] - pb;
  const bool va = very_long(ptr, n, a), vb = very_long(ptr, n, b);
  if (va != vb) return va;
  if (la > 0 && lb > 0) {
    // element t of a list, counted from its anchor
    const int sa = from_end ? pa + la - 1 : pa, sb = from_end ? pb + lb - 1 : pb, step = from_end ? -1 : 1;
    const int fa = idx[sa], fb = idx[sb];
    const int ra = a / rate * rate + longest_sub, rb = b / rate * rate + longest_sub;
    const int ba = ptr[ra + 1] - ptr[ra], bb = ptr[rb + 1] - ptr[rb];
    if (va) {                       // rule 1: block-line length decides before the anchor
      if (ba != bb) return ba > bb;
      if (fa != fb) return fa < fb;
    } else {
      if (fa != fb) return fa < fb;
      if (ba != bb) return ba > bb;
    }
    const int m = la < lb ? la : lb;
    for (int t = 1; t < m; ++t) {
      const int ca = idx[sa + t * step], cb = idx[sb + t * step];
      if (ca != cb) return ca < cb;
    }
  }
  if (la != lb) return la > lb;
  return a < b;
}
// Which end anchors the order of one side: the one with FEWER distinct values over the lines that
// rule 2 applies to (more lines share it); the start on a tie.
inline bool anchor_from_end(const int32_t* ptr, const int32_t* idx, int n) {
  std::vector<int32_t> first, last;
  for (int i = 0; i < n; ++i)
    if (ptr[i + 1] > ptr[i] && !very_long(ptr, n, i)) { first.push_back(idx[ptr[i]]); last.push_back(idx[ptr[i + 1] - 1]); }
  auto distinct = [](std::vector<int32_t>& v) { std::sort(v.begin(), v.end()); return std::unique(v.begin(), v.end()) - v.begin(); };
  return distinct(last) < distinct(first);
}

static int check_mask(const uint8_t* mask, int nqb, int nkb, int rate) {
  if (!mask) return UA_ERR_NULL;
  if (nqb <= 0 || nkb <= 0 || rate <= 0) return UA_ERR_SHAPE;
  if ((int64_t)nqb * rate > (1 << 24) || (int64_t)nkb * rate > (1 << 24)) return UA_ERR_SHAPE;
  for (int64_t i = 0; i < (int64_t)nqb * nkb; ++i)
    if (mask[i] > 2) return UA_ERR_MASK;
  return UA_OK;
}

// ---- device variant -----------------------------------------------------------------------
// One wavefront per query tile (a "row" of the list) and per key tile (a "column"); lanes
// stride over the blocks of that row or column of the block mask.  Number of active tiles
// that block (qb, kb) gives to query tile qt = qb*rate + a: FULL rate, CAUSAL a + 1 (key
// sub-tiles 0..a); to key tile kt = kb*rate + b: FULL rate, CAUSAL rate - b (query sub-tiles
// b..rate-1).
constexpr int kWavesPerGroup = 4;

struct Line {          // one row or one column of the tile grid, as seen by its wavefront
  bool is_row;
  int id;              // tile index of the row or column
  int n_blocks;        // blocks along it
  int sub;             // id % rate
  int64_t base, step;  // block (i) of the line sits at mask[base + i*step]
};
__device__ __forceinline__ bool line_of_wave(int nqb, int nkb, int rate, Line& ln) {
  const int w = blockIdx.x * kWavesPerGroup + (threadIdx.x >> 6);
  const int nqt = nqb * rate, nkt = nkb * rate;
  if (w >= nqt + nkt) return false;
  ln.is_row = w < nqt;
  ln.id = ln.is_row ? w : w - nqt;
  ln.n_blocks = ln.is_row ? nkb : nqb;
  ln.sub = ln.id % rate;
  ln.base = ln.is_row ? (int64_t)(ln.id / rate) * nkb : ln.id / rate;
  ln.step = ln.is_row ? 1 : nkb;
  return true;
}
__device__ __forceinline__ int tiles_of_block(const Line& ln, int type, int rate) {
  return type == 1 ? rate : (type == 2 ? (ln.is_row ? ln.sub + 1 : rate - ln.sub) : 0);
}
__device__ __forceinline__ int wave_sum(int v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off);
  return v;
}

__global__ __launch_bounds__(64 * kWavesPerGroup) void tl_count_kernel(const uint8_t* mask, int nqb, int nkb, int rate,
                                                                        int32_t* qcnt, int32_t* kcnt) {
  Line ln;
  if (!line_of_wave(nqb, nkb, rate, ln)) return;
  const int lane = threadIdx.x & 63;
  int n = 0;
  for (int i = lane; i < ln.n_blocks; i += 64) n += tiles_of_block(ln, mask[ln.base + i * ln.step], rate);
  n = wave_sum(n);
  if (lane == 0) (ln.is_row ? qcnt : kcnt)[ln.id] = n;
}

// init: zeroes the counters that the later kernels of the stream accumulate into.
__global__ void tl_init_kernel(int32_t* n_invalid, int32_t* anchor_cnt) {
  if (threadIdx.x == 0) *n_invalid = 0;
  if (threadIdx.x < 4) anchor_cnt[threadIdx.x] = 0;
}

// check: counts the mask entries that are not a Block_Type (> 2); the builder treats them as
// EMPTY, and the count lets the caller detect them after the stream has been synchronised (the
// host builder returns UA_ERR_MASK for the same input).  Grid-stride over the mask, one atomic per
// workgroup.
__global__ __launch_bounds__(1024) void tl_check_kernel(const uint8_t* mask, int64_t n, int32_t* n_invalid) {
  __shared__ int32_t part[16];
  int bad = 0;
  for (int64_t i = (int64_t)blockIdx.x * 1024 + threadIdx.x; i < n; i += (int64_t)gridDim.x * 1024) bad += mask[i] > 2;
  bad = wave_sum(bad);
  if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = bad;
  __syncthreads();
  if (threadIdx.x == 0) {
    int s = 0;
    for (int i = 0; i < 16; ++i) s += part[i];
    if (s) atomicAdd(n_invalid, s);
  }
}

// scan: a single workgroup turns counts into exclusive prefix sums.
__global__ __launch_bounds__(1024) void tl_scan_kernel(const int32_t* cnt, int n, int32_t* ptr) {
  __shared__ int32_t part[1024];
  const int tid = threadIdx.x;
  const int per = (n + 1023) / 1024;
  const int lo = min(n, tid * per), hi = min(n, lo + per);
  int s = 0;
  for (int i = lo; i < hi; ++i) s += cnt[i];
  part[tid] = s;
  __syncthreads();
  for (int off = 1; off < 1024; off <<= 1) {
    const int v = tid >= off ? part[tid - off] : 0;
    __syncthreads();
    part[tid] += v;
    __syncthreads();
  }
  int run = tid ? part[tid - 1] : 0;
  for (int i = lo; i < hi; ++i) { ptr[i] = run; run += cnt[i]; }
  if (tid == 1023) ptr[n] = part[1023];
}

// fill: the wavefront walks its line 64 blocks at a time; an exclusive scan of the per-block
// tile counts gives every lane the slot where its block's tiles go, in ascending tile order.
__global__ __launch_bounds__(64 * kWavesPerGroup) void tl_fill_kernel(const uint8_t* mask, int nqb, int nkb, int rate,
                                                                       const int32_t* row_ptr, int32_t* col_idx, uint8_t* flag,
                                                                       const int32_t* col_ptr, int32_t* row_idx, uint8_t* cflag) {
  Line ln;
  if (!line_of_wave(nqb, nkb, rate, ln)) return;
  const int lane = threadIdx.x & 63;
  int32_t* idx = ln.is_row ? col_idx : row_idx;
  uint8_t* flg = ln.is_row ? flag : cflag;
  int e = (ln.is_row ? row_ptr : col_ptr)[ln.id];
  for (int i0 = 0; i0 < ln.n_blocks; i0 += 64) {
    const int i = i0 + lane;
    const int type = i < ln.n_blocks ? mask[ln.base + i * ln.step] : 0;
    const int c = tiles_of_block(ln, type, rate);
    int incl = c;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
      const int v = __shfl_up(incl, off);
      if (lane >= off) incl += v;
    }
    int at = e + incl - c;
    // sub-tiles along the line: a row takes key sub-tiles 0..sub of a causal block (the last one
    // causal), a column takes query sub-tiles sub..rate-1 (the first one causal)
    const int first = (type == 2 && !ln.is_row) ? ln.sub : 0;
    for (int t = 0; t < c; ++t) {
      const int s = first + t;
      idx[at] = i * rate + s;
      flg[at] = type == 2 && s == ln.sub;
      ++at;
    }
    e += __shfl(incl, 63);
  }
}

// anchor: number of distinct first and of distinct last indices over the lines of each side that are
// neither empty nor very long -> anchor_cnt[0..1] for the rows, [2..3] for the columns.  Linear in
// the number of lines: every line marks its two anchor values in a flag array indexed by tile id
// (bit 0 = seen as a first index, bit 1 = as a last index), then the set bits are counted.  The flag
// arrays are the launch-order outputs themselves, which are only written afterwards: a row's anchors
// are key tiles (flags in k_order, n_ktiles entries), a column's are query tiles (flags in q_order).
__global__ __launch_bounds__(256) void tl_anchor_clear_kernel(int32_t* q_order, int nq, int32_t* k_order, int nk) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i < nq) q_order[i] = 0;
  else if (i < nq + nk) k_order[i - nq] = 0;
}
__global__ __launch_bounds__(256) void tl_anchor_mark_kernel(const int32_t* qptr, const int32_t* qidx, int nq,
                                                             const int32_t* kptr, const int32_t* kidx, int nk,
                                                             int32_t* q_order, int32_t* k_order) {
  const int t = blockIdx.x * 256 + threadIdx.x;
  if (t >= nq + nk) return;
  const bool is_row = t < nq;
  const int32_t* ptr = is_row ? qptr : kptr;
  const int32_t* idx = is_row ? qidx : kidx;
  const int n = is_row ? nq : nk, i = is_row ? t : t - nq;
  if (ptr[i + 1] == ptr[i] || very_long(ptr, n, i)) return;
  int32_t* flags = is_row ? k_order : q_order;
  const int limit = is_row ? nk : nq;
  const int first = idx[ptr[i]], last = idx[ptr[i + 1] - 1];
  if (first >= 0 && first < limit) atomicOr(&flags[first], 1);
  if (last >= 0 && last < limit) atomicOr(&flags[last], 2);
}
__global__ __launch_bounds__(256) void tl_anchor_count_kernel(const int32_t* q_order, int nq, const int32_t* k_order, int nk,
                                                              int32_t* anchor_cnt) {
  const int t = blockIdx.x * 256 + threadIdx.x;
  // flags in k_order belong to the rows (anchor_cnt[0..1]), flags in q_order to the columns ([2..3])
  const int f = t < nq ? q_order[t] : (t < nq + nk ? k_order[t - nq] : 0);
  const bool rows_side = t >= nq;
  // a wavefront may straddle the boundary between the two arrays: its two sides are summed separately
  const int r0 = wave_sum(rows_side ? (f & 1) : 0), r1 = wave_sum(rows_side ? ((f >> 1) & 1) : 0);
  const int c0 = wave_sum(rows_side ? 0 : (f & 1)), c1 = wave_sum(rows_side ? 0 : ((f >> 1) & 1));
  if ((threadIdx.x & 63) == 0) {
    if (r0) atomicAdd(&anchor_cnt[0], r0);
    if (r1) atomicAdd(&anchor_cnt[1], r1);
    if (c0) atomicAdd(&anchor_cnt[2], c0);
    if (c1) atomicAdd(&anchor_cnt[3], c1);
  }
}

// order: rank of a line = number of lines that precede it; one workgroup per line, its threads
// share the comparisons.
__global__ __launch_bounds__(256) void tl_order_kernel(const int32_t* qptr, const int32_t* qidx, int nq, int32_t* q_order,
                                                       const int32_t* kptr, const int32_t* kidx, int nk, int32_t* k_order, int rate,
                                                       const int32_t* anchor_cnt) {
  __shared__ int rank_s;
  const int t = blockIdx.x;
  const int32_t* ptr = t < nq ? qptr : kptr;
  const int32_t* idx = t < nq ? qidx : kidx;
  const int n = t < nq ? nq : nk;
  int32_t* order = t < nq ? q_order : k_order;
  const int i = t < nq ? t : t - nq;
  const int longest_sub = t < nq ? rate - 1 : 0;
  const int32_t* cnt = anchor_cnt + (t < nq ? 0 : 2);
  const bool from_end = cnt[1] < cnt[0];
  if (threadIdx.x == 0) rank_s = 0;
  __syncthreads();
  int rank = 0;
  for (int j = threadIdx.x; j < n; j += 256) rank += (j != i) && row_precedes(ptr, idx, n, rate, longest_sub, from_end, j, i);
  rank = wave_sum(rank);
  if ((threadIdx.x & 63) == 0) atomicAdd(&rank_s, rank);
  __syncthreads();
  if (threadIdx.x == 0) order[rank_s] = i;
}

}  // namespace ua

extern "C" int ua_tilelist_size(const uint8_t* block_mask, int n_qblocks, int n_kblocks, int rate,
                                int64_t* n_qtiles, int64_t* n_ktiles, int64_t* nnz) {
  using namespace ua;
  if (!n_qtiles || !n_ktiles || !nnz) return UA_ERR_NULL;
  if (int rc = check_mask(block_mask, n_qblocks, n_kblocks, rate)) return rc;
  int64_t n = 0;
  for (int64_t i = 0; i < (int64_t)n_qblocks * n_kblocks; ++i) {
    const int t = block_mask[i];
    n += t == 1 ? (int64_t)rate * rate : (t == 2 ? (int64_t)rate * (rate + 1) / 2 : 0);
  }
  if (n > INT32_MAX) return UA_ERR_SHAPE;
  *n_qtiles = (int64_t)n_qblocks * rate;
  *n_ktiles = (int64_t)n_kblocks * rate;
  *nnz = n;
  return UA_OK;
}

extern "C" int ua_tilelist_build(const uint8_t* block_mask, int n_qblocks, int n_kblocks, int rate,
                                 int32_t* row_ptr, int32_t* col_idx, uint8_t* flag,
                                 int32_t* col_ptr, int32_t* row_idx, uint8_t* cflag,
                                 int32_t* q_order, int32_t* k_order) {
  using namespace ua;
  if (int rc = check_mask(block_mask, n_qblocks, n_kblocks, rate)) return rc;
  if (!row_ptr || !col_ptr || !q_order || !k_order) return UA_ERR_NULL;
  const int nqt = n_qblocks * rate, nkt = n_kblocks * rate;
  std::vector<int32_t> kcnt(nkt, 0);
  int64_t e = 0;
  for (int qt = 0; qt < nqt; ++qt) {
    row_ptr[qt] = (int32_t)e;
    for (int kb = 0; kb < n_kblocks; ++kb) {
      if (!block_mask[(int64_t)(qt / rate) * n_kblocks + kb]) continue;
      for (int kt = kb * rate; kt < (kb + 1) * rate; ++kt) {
        const int ty = tile_type(block_mask, n_kblocks, rate, qt, kt);
        if (!ty) continue;
        if (!col_idx || !flag) return UA_ERR_NULL;
        col_idx[e] = kt; flag[e] = ty == 2; ++e; ++kcnt[kt];
      }
    }
  }
  row_ptr[nqt] = (int32_t)e;
  col_ptr[0] = 0;
  for (int kt = 0; kt < nkt; ++kt) col_ptr[kt + 1] = col_ptr[kt] + kcnt[kt];
  if (e > 0 && (!row_idx || !cflag)) return UA_ERR_NULL;
  std::vector<int32_t> cur(col_ptr, col_ptr + nkt);
  for (int qt = 0; qt < nqt; ++qt)
    for (int32_t i = row_ptr[qt]; i < row_ptr[qt + 1]; ++i) {
      const int32_t pos = cur[col_idx[i]]++;
      row_idx[pos] = qt; cflag[pos] = flag[i];
    }
  std::iota(q_order, q_order + nqt, 0);
  const bool q_end = anchor_from_end(row_ptr, col_idx, nqt), k_end = anchor_from_end(col_ptr, row_idx, nkt);
  std::sort(q_order, q_order + nqt, [&](int32_t a, int32_t b) { return row_precedes(row_ptr, col_idx, nqt, rate, rate - 1, q_end, a, b); });
  std::iota(k_order, k_order + nkt, 0);
  std::sort(k_order, k_order + nkt, [&](int32_t a, int32_t b) { return row_precedes(col_ptr, row_idx, nkt, rate, 0, k_end, a, b); });
  return UA_OK;
}

namespace ua {

static int build_device_impl(const uint8_t* block_mask, int n_qblocks, int n_kblocks, int rate,
                             int32_t* row_ptr, int32_t* col_idx, uint8_t* flag,
                             int32_t* col_ptr, int32_t* row_idx, uint8_t* cflag,
                             int32_t* q_order, int32_t* k_order, int32_t* work, int32_t* n_invalid, hipStream_t st) {
  const int nqt = n_qblocks * rate, nkt = n_kblocks * rate;
  int32_t* qcnt = work;
  int32_t* kcnt = work + nqt + 1;
  int32_t* anchor_cnt = work + nqt + nkt + 3;
  hipLaunchKernelGGL(tl_init_kernel, dim3(1), dim3(64), 0, st, n_invalid, anchor_cnt);
  const int64_t n_mask = (int64_t)n_qblocks * n_kblocks;
  hipLaunchKernelGGL(tl_check_kernel, dim3((unsigned)std::min<int64_t>((n_mask + 1023) / 1024, 2048)), dim3(1024), 0, st,
                     block_mask, n_mask, n_invalid);
  const int blocks = (nqt + nkt + kWavesPerGroup - 1) / kWavesPerGroup;
  hipLaunchKernelGGL(tl_count_kernel, dim3(blocks), dim3(64 * kWavesPerGroup), 0, st, block_mask, n_qblocks, n_kblocks, rate, qcnt, kcnt);
  hipLaunchKernelGGL(tl_scan_kernel, dim3(1), dim3(1024), 0, st, (const int32_t*)qcnt, nqt, row_ptr);
  hipLaunchKernelGGL(tl_scan_kernel, dim3(1), dim3(1024), 0, st, (const int32_t*)kcnt, nkt, col_ptr);
  hipLaunchKernelGGL(tl_fill_kernel, dim3(blocks), dim3(64 * kWavesPerGroup), 0, st, block_mask, n_qblocks, n_kblocks, rate,
                     (const int32_t*)row_ptr, col_idx, flag, (const int32_t*)col_ptr, row_idx, cflag);
  const int line_blocks = (nqt + nkt + 255) / 256;
  hipLaunchKernelGGL(tl_anchor_clear_kernel, dim3(line_blocks), dim3(256), 0, st, q_order, nqt, k_order, nkt);
  hipLaunchKernelGGL(tl_anchor_mark_kernel, dim3(line_blocks), dim3(256), 0, st,
                     (const int32_t*)row_ptr, (const int32_t*)col_idx, nqt,
                     (const int32_t*)col_ptr, (const int32_t*)row_idx, nkt, q_order, k_order);
  hipLaunchKernelGGL(tl_anchor_count_kernel, dim3(line_blocks), dim3(256), 0, st,
                     (const int32_t*)q_order, nqt, (const int32_t*)k_order, nkt, anchor_cnt);
  hipLaunchKernelGGL(tl_order_kernel, dim3(nqt + nkt), dim3(256), 0, st,
                     (const int32_t*)row_ptr, (const int32_t*)col_idx, nqt, q_order,
                     (const int32_t*)col_ptr, (const int32_t*)row_idx, nkt, k_order, rate, (const int32_t*)anchor_cnt);
  return hipGetLastError() == hipSuccess ? UA_OK : UA_ERR_LAUNCH;
}

static int check_device_builder_args(const uint8_t* block_mask, int n_qblocks, int n_kblocks, int rate,
                                     const void* row_ptr, const void* col_idx, const void* flag, const void* col_ptr,
                                     const void* row_idx, const void* cflag, const void* q_order, const void* k_order) {
  if (!block_mask || !row_ptr || !col_idx || !flag || !col_ptr || !row_idx || !cflag || !q_order || !k_order)
    return UA_ERR_NULL;
  if (n_qblocks <= 0 || n_kblocks <= 0 || rate <= 0) return UA_ERR_SHAPE;
  if ((int64_t)n_qblocks * rate > (1 << 24) || (int64_t)n_kblocks * rate > (1 << 24)) return UA_ERR_SHAPE;
  return UA_OK;
}

}  // namespace ua

extern "C" int ua_tilelist_build_device(const uint8_t* block_mask, int n_qblocks, int n_kblocks, int rate,
                                        int32_t* row_ptr, int32_t* col_idx, uint8_t* flag,
                                        int32_t* col_ptr, int32_t* row_idx, uint8_t* cflag,
                                        int32_t* q_order, int32_t* k_order, int32_t* work, void* stream) {
  using namespace ua;
  if (!work) return UA_ERR_NULL;
  if (int rc = check_device_builder_args(block_mask, n_qblocks, n_kblocks, rate, row_ptr, col_idx, flag, col_ptr,
                                         row_idx, cflag, q_order, k_order)) return rc;
  if (int rc = check_device()) return rc;
  const int nqt = n_qblocks * rate, nkt = n_kblocks * rate;
  return build_device_impl(block_mask, n_qblocks, n_kblocks, rate, row_ptr, col_idx, flag, col_ptr, row_idx, cflag,
                           q_order, k_order, work, work + nqt + nkt + 2, (hipStream_t)stream);
}

// The device address of `scratch`, looked up once per device with that device current.  In host
// code the array's name is only a handle for this lookup, never an address to pass on.
static int scratch_of_current_device(int32_t** out) {
  static std::atomic<int32_t*> ptrs[64];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return UA_ERR_DEVICE;
  int32_t* p = ptrs[dev].load(std::memory_order_acquire);
  if (!p) {
    void* sym = nullptr;
    if (hipGetSymbolAddress(&sym, HIP_SYMBOL(scratch)) != hipSuccess || !sym) return UA_ERR_DEVICE;
    p = static_cast<int32_t*>(sym);
    ptrs[dev].store(p, std::memory_order_release);
  }
  *out = p;
  return UA_OK;
}

// Everything the entry points resolve lazily per device, resolved now (outside any graph capture).
extern "C" int ua_init(void) {
  if (int rc = ua::check_device()) return rc;
  int32_t* p = nullptr;
  return scratch_of_current_device(&p);
}

extern "C" int ua_tilelist_build_device_noalloc(const uint8_t* block_mask, int n_qblocks, int n_kblocks, int rate,
                                                int32_t* row_ptr, int32_t* col_idx, uint8_t* flag,
                                                int32_t* col_ptr, int32_t* row_idx, uint8_t* cflag,
                                                int32_t* q_order, int32_t* k_order, int32_t* n_invalid, void* stream) {
  using namespace ua;
  if (int rc = check_device_builder_args(block_mask, n_qblocks, n_kblocks, rate, row_ptr, col_idx, flag, col_ptr,
                                         row_idx, cflag, q_order, k_order)) return rc;
  const int64_t lines = (int64_t)n_qblocks * rate + (int64_t)n_kblocks * rate;
  if (lines > UA_NOALLOC_MAX_LINES) return UA_ERR_TOO_LARGE;
  if (int rc = check_device()) return rc;
  int32_t* work = nullptr;
  if (int rc = scratch_of_current_device(&work)) return rc;
  // the counts are written before they are read and the invalid-entry count is stored, not
  // accumulated: nothing in the scratch has to start at zero
  return build_device_impl(block_mask, n_qblocks, n_kblocks, rate, row_ptr, col_idx, flag, col_ptr, row_idx, cflag,
                           q_order, k_order, work, n_invalid ? n_invalid : work + lines + 2, (hipStream_t)stream);
}
