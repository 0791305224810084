// LSE-weighted merge of partial attention outputs, and the backward's row statistic
// delta = rowsum(dO * O).  Both are HBM-bandwidth bound streaming kernels.
//
// A workgroup owns a few consecutive tokens (kTok, kMergeTok) of all heads.  The per-row statistics are laid out
// [batch, head, token] while the rows themselves are [batch, token, head, 128]; the workgroup
// first handles the statistics with token-contiguous (coalesced) accesses and parks the row
// weights in LDS, then streams the rows as 16-byte vectors (16 lanes per 256-byte row).
#include "ua_common.h"

namespace ua {

constexpr int kTok = 16;          // tokens per workgroup (delta, single update)
// The merge runs best with many small workgroups: with 2 tokens x 32 heads a workgroup issues
// all of its row loads in one step (4 x 16 bytes per thread and partial) and retires; the
// device then streams 4 reads : 1 write at the rate a bare copy kernel of the same shape reaches.
constexpr int kMergeTok = 2;
constexpr int kMaxHeadsLds = 256; // rows per workgroup = kTok * n_heads <= 4096

struct MergeParams {
  const bf16* o_parts[UA_MAX_PARTS];
  const float* lse_parts[UA_MAX_PARTS];
  bf16* o; float* lse;
  int n_parts, seqlen, n_heads;
};

template <int P>
__global__ __launch_bounds__(256) void merge_kernel(const MergeParams p) {
  extern __shared__ float w_lds[];              // [P][rows], rows = kMergeTok * n_heads
  const int tid = threadIdx.x;
  const int tiles_per_batch = (p.seqlen + kMergeTok - 1) / kMergeTok;
  const int b = blockIdx.x / tiles_per_batch;
  const int s0 = (blockIdx.x % tiles_per_batch) * kMergeTok;
  const int ntok = min(kMergeTok, p.seqlen - s0);       // the last workgroup of a batch may be ragged
  const int rows = ntok * p.n_heads;

  // The rows are streamed as 16-byte chunks (chunk c = 8 bf16 of row c/16), kUnroll chunks per
  // thread per step, and the loads of step n+1 are issued before step n is combined, so that
  // P * kUnroll (..2x) 16-byte loads per thread are always in flight.
  const int64_t base = ((int64_t)b * p.seqlen + s0) * p.n_heads * kHeadDim;
  const int n_chunks = rows * 16;
  constexpr int kUnroll = P <= 4 ? 4 : (P <= 8 ? 2 : 1);
  constexpr int kStep = 256 * kUnroll;
  u32x4 raw[kUnroll][P];
  auto load = [&](int c0) {
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
      const int c = c0 + u * 256;
      if (c < n_chunks) {
#pragma unroll
        for (int i = 0; i < P; ++i)
          raw[u][i] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p.o_parts[i] + base) + c);
      }
    }
  };
  load(tid);        // first step's rows are in flight while the statistics are handled

  // phase 1: one thread per (head, token): statistics, coalesced along the token axis
  for (int t = tid; t < kMergeTok * p.n_heads; t += 256) {
    const int h = t / kMergeTok, sl = t % kMergeTok;
    if (sl >= ntok) continue;
    const int64_t li = ((int64_t)b * p.n_heads + h) * p.seqlen + s0 + sl;
    float l[P];
    float m = -INFINITY;
#pragma unroll
    for (int i = 0; i < P; ++i) { l[i] = p.lse_parts[i][li]; m = fmaxf(m, l[i]); }
    const float ms = (m == -INFINITY) ? 0.f : m;
    float den = 0.f;
#pragma unroll
    for (int i = 0; i < P; ++i) { l[i] = fast_exp2((l[i] - ms) * kLog2e); den += l[i]; }
    const float inv = den > 0.f ? 1.f / den : 0.f;
    const int row = sl * p.n_heads + h;
#pragma unroll
    for (int i = 0; i < P; ++i) w_lds[i * rows + row] = l[i] * inv;
    p.lse[li] = den > 0.f ? ms + __builtin_amdgcn_logf(den) * kLn2 : -INFINITY;
  }
  __syncthreads();

  // phase 2: combine
  for (int c0 = tid; c0 < n_chunks; c0 += kStep) {
    u32x4 cur[kUnroll][P];
#pragma unroll
    for (int u = 0; u < kUnroll; ++u)
#pragma unroll
      for (int i = 0; i < P; ++i) cur[u][i] = raw[u][i];
    load(c0 + kStep);
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
      const int c = c0 + u * 256;
      if (c >= n_chunks) break;
      const int row = c >> 4;
      float acc[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) acc[j] = 0.f;
#pragma unroll
      for (int i = 0; i < P; ++i) {
        const float w = w_lds[i * rows + row];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          acc[2 * j] = fmaf(w, __uint_as_float(cur[u][i][j] << 16), acc[2 * j]);
          acc[2 * j + 1] = fmaf(w, __uint_as_float(cur[u][i][j] & 0xffff0000u), acc[2 * j + 1]);
        }
      }
      bf16x8 out;
#pragma unroll
      for (int j = 0; j < 8; ++j) out[j] = (bf16)acc[j];
      __builtin_nontemporal_store(out, reinterpret_cast<bf16x8*>(p.o + base) + c);
    }
  }
}

struct DeltaParams {
  const bf16* o; const bf16* dout; float* delta;
  int seqlen, n_heads;
  Strides3 os, ds;
};

__global__ __launch_bounds__(256) void delta_kernel(const DeltaParams p) {
  extern __shared__ float d_lds[];               // [n_heads][kTok]
  const int tid = threadIdx.x;
  const int tiles_per_batch = (p.seqlen + kTok - 1) / kTok;
  const int b = blockIdx.x / tiles_per_batch;
  const int s0 = (blockIdx.x % tiles_per_batch) * kTok;
  const int ntok = min(kTok, p.seqlen - s0);
  const int rows = ntok * p.n_heads;
  const int sub = tid & 15;
  // 16 lanes per row; kRows rows per thread and step so that 2 * kRows 16-byte loads are in flight
  constexpr int kRows = 4;
  for (int row0 = tid >> 4; row0 < rows; row0 += 16 * kRows) {
    u32x4 a[kRows], g[kRows];
#pragma unroll
    for (int u = 0; u < kRows; ++u) {
      const int row = row0 + 16 * u;
      if (row < rows) {
        const int sl = row / p.n_heads, h = row % p.n_heads;
        const int64_t s = s0 + sl;
        a[u] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p.o + b * p.os.b + s * p.os.s + h * p.os.h + sub * 8));
        g[u] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p.dout + b * p.ds.b + s * p.ds.s + h * p.ds.h + sub * 8));
      }
    }
#pragma unroll
    for (int u = 0; u < kRows; ++u) {
      const int row = row0 + 16 * u;
      if (row >= rows) break;
      const int sl = row / p.n_heads, h = row % p.n_heads;
      float acc = 0.f;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        acc = fmaf(__uint_as_float(a[u][j] << 16), __uint_as_float(g[u][j] << 16), acc);
        acc = fmaf(__uint_as_float(a[u][j] & 0xffff0000u), __uint_as_float(g[u][j] & 0xffff0000u), acc);
      }
      acc += __shfl_xor(acc, 1); acc += __shfl_xor(acc, 2); acc += __shfl_xor(acc, 4); acc += __shfl_xor(acc, 8);
      if (sub == 0) d_lds[h * kTok + sl] = acc;
    }
  }
  __syncthreads();
  for (int t = tid; t < kTok * p.n_heads; t += 256) {
    const int h = t / kTok, sl = t % kTok;
    if (sl >= ntok) continue;
    p.delta[((int64_t)b * p.n_heads + h) * p.seqlen + s0 + sl] = d_lds[t];
  }
}

// ---- in-place update of a running (out, lse) by one more partial -------------------------------
// new_lse = logaddexp(lse, block_lse);  new_out = exp(lse - new_lse) out + exp(block_lse - new_lse) block_out
// in the max-stabilised form (a partial with lse = -inf contributes nothing, two of them give
// out = 0, lse = -inf).  All six tensors are addressed through (batch, token, head) element
// strides, so a row range of a larger tensor, the [B, S, Nh, 1] statistics of the hierarchy
// executor and the kernel's own [B, Nh, S] layout are all the same call.  Rows may be bf16 or
// fp32 (the reference's running output becomes fp32 after its first update).
struct UpdateParams {
  const void* out; const float* lse; const void* blk; const float* blk_lse;
  void* new_out; float* new_lse;
  int n_rows, n_heads;
  Strides3 os, ls, bs, bls, ns, nls;
  int token_major;          // 1: lse's head axis is the contiguous one, 0: its token axis
};

template <bool kF32>
__device__ __forceinline__ void load8(const void* base, int64_t elem_off, float (&x)[8]) {
  if (kF32) {
    const f32x4* p = reinterpret_cast<const f32x4*>(static_cast<const float*>(base) + elem_off);
    const f32x4 a = p[0], b = p[1];
#pragma unroll
    for (int j = 0; j < 4; ++j) { x[j] = a[j]; x[4 + j] = b[j]; }
  } else {
    const u32x4 r = *reinterpret_cast<const u32x4*>(static_cast<const bf16*>(base) + elem_off);
#pragma unroll
    for (int j = 0; j < 4; ++j) { x[2 * j] = __uint_as_float(r[j] << 16); x[2 * j + 1] = __uint_as_float(r[j] & 0xffff0000u); }
  }
}
template <bool kF32>
__device__ __forceinline__ void store8(void* base, int64_t elem_off, const float (&x)[8]) {
  if (kF32) {
    f32x4* p = reinterpret_cast<f32x4*>(static_cast<float*>(base) + elem_off);
    p[0] = f32x4{x[0], x[1], x[2], x[3]};
    p[1] = f32x4{x[4], x[5], x[6], x[7]};
  } else {
    bf16x8 w;
#pragma unroll
    for (int j = 0; j < 8; ++j) w[j] = (bf16)x[j];
    *reinterpret_cast<bf16x8*>(static_cast<bf16*>(base) + elem_off) = w;
  }
}

template <bool kOutF32, bool kBlkF32, bool kNewF32>
__global__ __launch_bounds__(256) void merge_update_kernel(const UpdateParams p) {
  extern __shared__ float w_lds[];              // [2][rows]: weight of the running output, of the block
  const int tid = threadIdx.x;
  const int tiles_per_batch = (p.n_rows + kTok - 1) / kTok;
  const int b = blockIdx.x / tiles_per_batch;
  const int s0 = (blockIdx.x % tiles_per_batch) * kTok;
  const int ntok = min(kTok, p.n_rows - s0);
  const int rows = ntok * p.n_heads;
  // statistics: one thread per (token, head), walking the running lse along its contiguous axis
  for (int t = tid; t < kTok * p.n_heads; t += 256) {
    const int sl = p.token_major ? t / p.n_heads : t % kTok;
    const int h = p.token_major ? t % p.n_heads : t / kTok;
    if (sl >= ntok) continue;
    const int64_t s = s0 + sl;
    const float a = p.lse[b * p.ls.b + s * p.ls.s + h * p.ls.h];
    const float c = p.blk_lse[b * p.bls.b + s * p.bls.s + h * p.bls.h];
    const float m = fmaxf(a, c);
    const float ms = (m == -INFINITY) ? 0.f : m;
    const float ea = fast_exp2((a - ms) * kLog2e), ec = fast_exp2((c - ms) * kLog2e);
    const float den = ea + ec;
    const float inv = den > 0.f ? 1.f / den : 0.f;
    const int row = sl * p.n_heads + h;
    w_lds[row] = ea * inv;
    w_lds[rows + row] = ec * inv;
    p.new_lse[b * p.nls.b + s * p.nls.s + h * p.nls.h] = den > 0.f ? ms + __builtin_amdgcn_logf(den) * kLn2 : -INFINITY;
  }
  __syncthreads();
  // rows: 16 chunks of 8 elements each
  for (int c = tid; c < rows * 16; c += 256) {
    const int row = c >> 4, part = (c & 15) * 8;
    const int sl = row / p.n_heads, h = row % p.n_heads;
    const int64_t s = s0 + sl;
    float x[8], y[8];
    load8<kOutF32>(p.out, b * p.os.b + s * p.os.s + h * p.os.h + part, x);
    load8<kBlkF32>(p.blk, b * p.bs.b + s * p.bs.s + h * p.bs.h + part, y);
    const float wa = w_lds[row], wc = w_lds[rows + row];
    // a weight of exactly 0 drops its operand (a partial without keys may hold anything)
#pragma unroll
    for (int j = 0; j < 8; ++j) x[j] = (wa != 0.f ? wa * x[j] : 0.f) + (wc != 0.f ? wc * y[j] : 0.f);
    store8<kNewF32>(p.new_out, b * p.ns.b + s * p.ns.s + h * p.ns.h + part, x);
  }
}

template <int P>
static int launch_merge(const MergeParams& p, int blocks, size_t lds, hipStream_t st) {
  hipLaunchKernelGGL(merge_kernel<P>, dim3(blocks), dim3(256), lds, st, p);
  return hipGetLastError() == hipSuccess ? UA_OK : UA_ERR_LAUNCH;
}

}  // namespace ua

extern "C" int ua_merge(const void* const* o_parts, const float* const* lse_parts, int n_parts,
                        void* o, float* lse, int batch, int seqlen, int n_heads, int head_dim, void* stream) {
  using namespace ua;
  if (!o_parts || !lse_parts || !o || !lse) return UA_ERR_NULL;
  if (n_parts < 1 || n_parts > UA_MAX_PARTS) return UA_ERR_UNSUPPORTED;
  if (head_dim != kHeadDim) return UA_ERR_UNSUPPORTED;
  if (batch <= 0 || seqlen <= 0 || n_heads <= 0 || n_heads > kMaxHeadsLds) return UA_ERR_SHAPE;
  if ((int64_t)batch * ((seqlen + kMergeTok - 1) / kMergeTok) > INT32_MAX) return UA_ERR_SHAPE;
  if (!aligned16(o)) return UA_ERR_ALIGN;
  MergeParams p;
  for (int i = 0; i < n_parts; ++i) {
    if (!o_parts[i] || !lse_parts[i]) return UA_ERR_NULL;
    if (!aligned16(o_parts[i])) return UA_ERR_ALIGN;
    p.o_parts[i] = (const bf16*)o_parts[i];
    p.lse_parts[i] = lse_parts[i];
  }
  for (int i = n_parts; i < UA_MAX_PARTS; ++i) { p.o_parts[i] = nullptr; p.lse_parts[i] = nullptr; }
  p.o = (bf16*)o; p.lse = lse; p.n_parts = n_parts; p.seqlen = seqlen; p.n_heads = n_heads;
  if (int rc = check_device()) return rc;
  const int blocks = batch * ((seqlen + kMergeTok - 1) / kMergeTok);
  const size_t lds = (size_t)n_parts * kMergeTok * n_heads * sizeof(float);
  if (lds > 65536) return UA_ERR_SHAPE;   // n_parts * n_heads <= 1024
  hipStream_t st = (hipStream_t)stream;
  switch (n_parts) {
#define UA_CASE(N) case N: return launch_merge<N>(p, blocks, lds, st);
    UA_CASE(1) UA_CASE(2) UA_CASE(3) UA_CASE(4) UA_CASE(5) UA_CASE(6) UA_CASE(7) UA_CASE(8)
    UA_CASE(9) UA_CASE(10) UA_CASE(11) UA_CASE(12) UA_CASE(13) UA_CASE(14) UA_CASE(15) UA_CASE(16)
#undef UA_CASE
  }
  return UA_ERR_UNSUPPORTED;
}

extern "C" int ua_bsa_bwd_delta(const void* o, const void* dout, float* delta,
                                int batch, int seqlen_q, int n_heads, int head_dim,
                                const int64_t* o_strides, const int64_t* do_strides, void* stream) {
  using namespace ua;
  if (!o || !dout || !delta || !o_strides || !do_strides) return UA_ERR_NULL;
  if (head_dim != kHeadDim) return UA_ERR_UNSUPPORTED;
  if (batch <= 0 || seqlen_q <= 0 || n_heads <= 0 || n_heads > kMaxHeadsLds) return UA_ERR_SHAPE;
  if ((int64_t)batch * ((seqlen_q + kTok - 1) / kTok) > INT32_MAX) return UA_ERR_SHAPE;
  if (!aligned16(o) || !aligned16(dout) || !strides_ok(o_strides) || !strides_ok(do_strides)) return UA_ERR_ALIGN;
  if (int rc = check_device()) return rc;
  DeltaParams p;
  p.o = (const bf16*)o; p.dout = (const bf16*)dout; p.delta = delta; p.seqlen = seqlen_q; p.n_heads = n_heads;
  p.os = {o_strides[0], o_strides[1], o_strides[2]};
  p.ds = {do_strides[0], do_strides[1], do_strides[2]};
  hipLaunchKernelGGL(delta_kernel, dim3(batch * ((seqlen_q + kTok - 1) / kTok)), dim3(256),
                     (size_t)kTok * n_heads * sizeof(float), (hipStream_t)stream, p);
  return hipGetLastError() == hipSuccess ? UA_OK : UA_ERR_LAUNCH;
}

extern "C" int ua_merge_update(const void* out, const float* lse, const void* block_out, const float* block_lse,
                               void* new_out, float* new_lse, int batch, int n_rows, int n_heads, int head_dim,
                               int out_is_fp32, int block_is_fp32, int new_is_fp32,
                               const int64_t* out_strides, const int64_t* lse_strides,
                               const int64_t* block_out_strides, const int64_t* block_lse_strides,
                               const int64_t* new_out_strides, const int64_t* new_lse_strides, void* stream) {
  using namespace ua;
  if (!out || !lse || !block_out || !block_lse || !new_out || !new_lse || !out_strides || !lse_strides ||
      !block_out_strides || !block_lse_strides || !new_out_strides || !new_lse_strides) return UA_ERR_NULL;
  if (head_dim != kHeadDim) return UA_ERR_UNSUPPORTED;
  if (batch <= 0 || n_rows <= 0 || n_heads <= 0 || n_heads > kMaxHeadsLds) return UA_ERR_SHAPE;
  if ((int64_t)batch * ((n_rows + kTok - 1) / kTok) > INT32_MAX) return UA_ERR_SHAPE;
  // every row must start on a 16-byte boundary: strides in multiples of 8 (bf16) or 4 (fp32) elements
  auto rows_ok = [](const void* ptr, const int64_t* st, int is_fp32) {
    const int64_t q = is_fp32 ? 4 : 8;
    return aligned16(ptr) && st[0] % q == 0 && st[1] % q == 0 && st[2] % q == 0;
  };
  if (!rows_ok(out, out_strides, out_is_fp32) || !rows_ok(block_out, block_out_strides, block_is_fp32) ||
      !rows_ok(new_out, new_out_strides, new_is_fp32)) return UA_ERR_ALIGN;
  // in place (the slice_ path): same pointer means same element type and the same strides, else
  // one thread's store would land on rows that other threads have not read yet
  auto same3 = [](const int64_t* a, const int64_t* b) { return a[0] == b[0] && a[1] == b[1] && a[2] == b[2]; };
  if (new_out == out && (out_is_fp32 != new_is_fp32 || !same3(out_strides, new_out_strides))) return UA_ERR_SHAPE;
  if (new_lse == lse && !same3(lse_strides, new_lse_strides)) return UA_ERR_SHAPE;
  if (int rc = check_device()) return rc;
  UpdateParams p;
  p.out = out; p.lse = lse; p.blk = block_out; p.blk_lse = block_lse; p.new_out = new_out; p.new_lse = new_lse;
  p.n_rows = n_rows; p.n_heads = n_heads;
  auto s3 = [](const int64_t* st) { return Strides3{st[0], st[1], st[2]}; };
  p.os = s3(out_strides); p.ls = s3(lse_strides); p.bs = s3(block_out_strides); p.bls = s3(block_lse_strides);
  p.ns = s3(new_out_strides); p.nls = s3(new_lse_strides);
  p.token_major = lse_strides[2] == 1 && lse_strides[1] != 1;
  const int blocks = batch * ((n_rows + kTok - 1) / kTok);
  const size_t lds = (size_t)2 * kTok * n_heads * sizeof(float);
  hipStream_t st = (hipStream_t)stream;
  const int sel = (out_is_fp32 ? 4 : 0) | (block_is_fp32 ? 2 : 0) | (new_is_fp32 ? 1 : 0);
  switch (sel) {
#define UA_CASE(N, A, B, C) case N: hipLaunchKernelGGL((merge_update_kernel<A, B, C>), dim3(blocks), dim3(256), lds, st, p); break;
    UA_CASE(0, false, false, false) UA_CASE(1, false, false, true) UA_CASE(2, false, true, false) UA_CASE(3, false, true, true)
    UA_CASE(4, true, false, false) UA_CASE(5, true, false, true) UA_CASE(6, true, true, false) UA_CASE(7, true, true, true)
#undef UA_CASE
  }
  return hipGetLastError() == hipSuccess ? UA_OK : UA_ERR_LAUNCH;
}
