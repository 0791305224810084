// Block-sparse flash-attention forward for gfx950 (MI355X).
//
// One workgroup (4 wavefronts) per (query tile of 128 rows, head).  It walks the query tile's
// CSR entries; each 128x128 K/V tile is streamed as two 64-key half tiles through two LDS
// stages (A, B) that are filled by asynchronous global->LDS copies while the other stage is
// being consumed.  Each wavefront owns 32 query rows and computes the TRANSPOSED products
//     S^T[key, q] = K Q^T      (A = K fragment from LDS, B = Q fragment held in registers)
//     O^T[d,  q] += V^T P^T    (A = V^T fragment via transposing LDS reads, B = P^T)
// with v_mfma_f32_32x32x16_bf16.  In the 32x32 accumulator layout a lane holds ONE query
// column (lane % 32) and 16 rows, so the online-softmax statistics of a query row live in one
// lane (mirrored in lane ^ 32): the row max needs a single cross-half exchange, the rescale of
// O^T is lane local, and S^T's accumulator registers are, after exp2 and bf16 packing, exactly
// the B operand of the second product.
#include "ua_common.h"

namespace ua {

struct FwdParams {
  const bf16* q; const bf16* k; const bf16* v; bf16* o; float* lse;
  const int32_t* row_ptr; const int32_t* col_idx; const uint8_t* flag; const int32_t* q_order;
  int batch, n_heads, n_qtiles, n_ktiles, nnz;
  Strides3 qs, ks, vs, os;
  float scale_log2;      // softmax_scale * log2(e)
  int heads_per_xcd;     // batch*n_heads / 8 when divisible, else 0
  // Dense rectangle (no list arrays): query tile qt walks key tiles [0, n_ktiles), or with
  // dense_causal [0, qt + diag_off] with the last one causal.  The key range is cut into n_parts
  // parts of part_len tiles; part i writes its partial (O, LSE) at o + i * o_part, lse + i * lse_part
  // (elements).  Longest rows are launched first.
  int dense, dense_causal, diag_off, n_parts, part_len;
  int64_t o_part, lse_part;
};

constexpr int kHalf = 64;                          // keys per pipeline stage
constexpr int kHalfBytes = kHalf * kRowBytes;      // 16 KiB
// P is computed against the row's current reference max without looking at the new scores'
// max; only when a block's row sum shows that some score exceeded the reference by more than
// ~2^kRaiseLog2 is the reference raised (and O, l rescaled, P recomputed).  O/l stay exact
// because numerator and denominator always share the reference.
constexpr float kRaiseSum = 16777216.f;     // 2^24

struct SoftmaxState {
  float m_run = -INFINITY;   // reference max of the row (log2 domain, scaled)
  float m_use = 0.f;         // m_run, or 0 while the row has not seen a visible key
  float l_run = 0.f;         // this half-wave's partial row sum
};

// One 64-key half tile for this wave's 32 query rows.  With `mask` (wave-uniform) keys beyond
// the query's own tile-local index are hidden; `key0` = tile-local index of the half's first key.
__device__ __forceinline__ void half_tile(const unsigned char* sK, const unsigned char* sV, const bf16x8 (&qf)[8],
                                          f32x16 (&oacc)[4], SoftmaxState& st, const TrLane& tr, float scale_log2,
                                          int l32, int hi, int q_local, int key0, bool mask, bool first) {
  // ---- S^T = K Q^T : 2 blocks of 32 keys x 32 queries ------------------------------------
  // The 16 K fragments are fetched kAhead reads ahead of the MFMA that consumes them, so the
  // LDS latency is covered by the preceding MFMAs instead of being paid before each one.
  f32x16 s[2];
  s[0] = f32x16{0};
  s[1] = f32x16{0};
  {
    constexpr int kAhead = 4;
    bf16x8 kfr[16];
#pragma unroll
    for (int i = 0; i < kAhead; ++i) kfr[i] = lds_read_b128(sK, lds_off_k(32 * (i & 1) + l32, 2 * (i >> 1) + hi));
    __builtin_amdgcn_sched_group_barrier(0x100, kAhead, 0);   // kAhead LDS reads up front
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      if (i + kAhead < 16) {
        const int j = i + kAhead;
        kfr[j] = lds_read_b128(sK, lds_off_k(32 * (j & 1) + l32, 2 * (j >> 1) + hi));
      }
      s[i & 1] = mfma32(kfr[i], qf[i >> 1], s[i & 1]);
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);   // then 1 MFMA, 1 LDS read, ...
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
    }
  }
  // element (mb, i) of this lane: key key0 + 32*mb + 8*(i/4) + 4*hi + i%4, query q_local
  if (mask) {
#pragma unroll
    for (int mb = 0; mb < 2; ++mb)
#pragma unroll
      for (int i = 0; i < 16; ++i)
        if (key0 + 32 * mb + 8 * (i >> 2) + 4 * hi + (i & 3) > q_local) s[mb][i] = -INFINITY;
  }
  // the first V^T fragments are fetched now: their latency hides behind the softmax
  constexpr int kVAhead = 3;
  bf16x8 vfr[4];
#pragma unroll
  for (int i = 0; i < kVAhead; ++i) vfr[i] = lds_read_tr_frag<lds_off_v>(sV, tr, 16 * (i >> 2), i & 3);
  // ---- online softmax (fp32, log2 domain) ---------------------------------------------------
  float rs = 0.f;
  bf16x8 pf[4];
  bool raise = first;
  if (!first) {
#pragma unroll
    for (int mb = 0; mb < 2; ++mb)
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const float pv = fast_exp2(fmaf(s[mb][i], scale_log2, -st.m_use));
        rs += pv;
        pf[mb * 2 + (i >> 3)][i & 7] = (bf16)pv;
      }
    raise = __builtin_amdgcn_ballot_w64(!(rs < kRaiseSum)) != 0;       // wave-uniform, rare
  }
  if (raise) {
    float mx = fmaxf(s[0][0], s[1][0]);
#pragma unroll
    for (int i = 1; i < 16; ++i) mx = fmaxf(mx, fmaxf(s[0][i], s[1][i]));
    mx = xhalf_max(mx) * scale_log2;
    const float m_new = fmaxf(st.m_run, mx);
    const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
    const float alpha = (m_new == st.m_run) ? 1.f : fast_exp2(st.m_run - m_use);      // m_run = -inf -> 0
    st.m_run = m_new;
    st.m_use = m_use;
    st.l_run *= alpha;
#pragma unroll
    for (int mbd = 0; mbd < 4; ++mbd)
#pragma unroll
      for (int i = 0; i < 16; ++i) oacc[mbd][i] *= alpha;
    rs = 0.f;
#pragma unroll
    for (int mb = 0; mb < 2; ++mb)
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const float pv = fast_exp2(fmaf(s[mb][i], scale_log2, -m_use));
        rs += pv;
        pf[mb * 2 + (i >> 3)][i & 7] = (bf16)pv;
      }
  }
  st.l_run += rs;
  // ---- O^T += V^T P^T : 4 blocks of 32 d x 32 queries, 4 steps of 16 keys -------------------
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    if (i + kVAhead < 16) vfr[(i + kVAhead) & 3] = lds_read_tr_frag<lds_off_v>(sV, tr, 16 * ((i + kVAhead) >> 2), (i + kVAhead) & 3);
    oacc[i & 3] = mfma32(vfr[i & 3], pf[i >> 2], oacc[i & 3]);
    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);   // 1 MFMA
    __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);   // 2 LDS reads (one fragment)
  }
}

__global__ __launch_bounds__(256, 2) void fwd_kernel(const FwdParams p) {
  // two pipeline stages, distinct arrays so that reads of one stage need not wait for the
  // copies in flight into the other
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
  int qt, e0, e1, diag = -1, part = 0;
  if (p.dense) {
    part = pos / p.n_qtiles;
    const int line = pos - part * p.n_qtiles;
    qt = p.dense_causal ? p.n_qtiles - 1 - line : line;
    if (p.dense_causal) diag = qt + p.diag_off;          // key tile on the diagonal (may lie outside the rectangle)
    const int kend = p.dense_causal ? min(max(diag + 1, 0), p.n_ktiles) : p.n_ktiles;
    e0 = min(part * p.part_len, kend);
    e1 = min(e0 + p.part_len, kend);
  } else {
    qt = min(max(sload(p.q_order, pos), 0), p.n_qtiles - 1);
    // list bounds are clamped to the arrays' extent: an inconsistent row_ptr cannot read beyond them
    e0 = min(max(sload(p.row_ptr, qt), 0), p.nnz);
    e1 = min(max(sload(p.row_ptr, qt + 1), e0), p.nnz);
  }
  // entry e of the walk: its key tile, and whether it is a causal tile
  auto ktile = [&](int e) { return p.dense ? e : min(max(sload(p.col_idx, e), 0), p.n_ktiles - 1); };
  auto is_causal = [&](int e) { return p.dense ? (int)(e == diag) : sload(p.flag, e); };

  const bf16* kbase = p.k + b * p.ks.b + h * p.ks.h;
  const bf16* vbase = p.v + b * p.vs.b + h * p.vs.h;
  const int k_stride = (int)p.ks.s, v_stride = (int)p.vs.s;
  int koff[4], voff[4];
  dma_voffsets<lds_off_k, 4>(koff, k_stride, wave, lane);
  dma_voffsets<lds_off_v, 4>(voff, v_stride, wave, lane);
  const int k_half = kHalf * k_stride * 2, v_half = kHalf * v_stride * 2;                 // bytes
  const uint32_t k_extent = (uint32_t)((kTile - 1) * k_stride + kHeadDim) * 2;            // bytes of one tile
  const uint32_t v_extent = (uint32_t)((kTile - 1) * v_stride + kHeadDim) * 2;
  auto k_rsrc = [&](int kt) { return make_rsrc(kbase + (int64_t)kt * kTile * k_stride, k_extent); };
  auto v_rsrc = [&](int kt) { return make_rsrc(vbase + (int64_t)kt * kTile * v_stride, v_extent); };

  // first half tile of the first entry goes in flight before anything else
  int kt = e0 < e1 ? ktile(e0) : 0;
  if (e0 < e1) {
    dma_half_tile_buf<4>(sKA, k_rsrc(kt), koff, 0, wave);
    dma_half_tile_buf<4>(sVA, v_rsrc(kt), voff, 0, wave);
  }

  // Q fragment (B operand of S^T): lane holds query row 32*wave + lane%32,
  // d = 16*ks + 8*(lane/32) .. +7 for ks = 0..7.
  const int q_local = wave * 32 + l32;
  const int qrow = qt * kTile + q_local;
  const bf16* qp = p.q + b * p.qs.b + (int64_t)qrow * p.qs.s + h * p.qs.h + hi * 8;
  bf16x8 qf[8];
#pragma unroll
  for (int ks = 0; ks < 8; ++ks) qf[ks] = *reinterpret_cast<const bf16x8*>(qp + ks * 16);

  f32x16 oacc[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) oacc[i] = f32x16{0};
  SoftmaxState st;
  const TrLane tr(lane);

  for (int e = e0; e < e1; ++e) {
    const int causal = is_causal(e);
    const int kt_next = e + 1 < e1 ? ktile(e + 1) : kt;
    // stage A (keys 0..63 of this tile) has landed; everyone is done with stage B
    wait_vmem_all();
    __syncthreads();
    dma_half_tile_buf<4>(sKB, k_rsrc(kt), koff, k_half, wave);
    dma_half_tile_buf<4>(sVB, v_rsrc(kt), voff, v_half, wave);
    // causal tile: queries 64..127 (waves 2, 3) see all of keys 0..63
    half_tile(sKA, sVA, qf, oacc, st, tr, p.scale_log2, l32, hi, q_local, 0, causal && wave < 2, e == e0);
    // stage B has landed; everyone is done with stage A
    wait_vmem_all();
    __syncthreads();
    if (e + 1 < e1) {
      dma_half_tile_buf<4>(sKA, k_rsrc(kt_next), koff, 0, wave);
      dma_half_tile_buf<4>(sVA, v_rsrc(kt_next), voff, 0, wave);
    }
    // causal tile: queries 0..63 (waves 0, 1) see none of keys 64..127
    if (!causal || wave >= 2)
      half_tile(sKB, sVB, qf, oacc, st, tr, p.scale_log2, l32, hi, q_local, kHalf, causal, false);
    kt = kt_next;
  }

  // ---- epilogue: normalise, write O (bf16) and LSE (natural log) -------------------------
  const float l_tot = xhalf_sum(st.l_run);
  const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
  bf16* op = p.o + part * p.o_part + b * p.os.b + (int64_t)qrow * p.os.s + h * p.os.h;
#pragma unroll
  for (int mbd = 0; mbd < 4; ++mbd)
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      bf16x4 w;
#pragma unroll
      for (int j = 0; j < 4; ++j) w[j] = (bf16)(oacc[mbd][4 * g + j] * inv);
      *reinterpret_cast<bf16x4*>(op + 32 * mbd + 8 * g + 4 * hi) = w;
    }
  if (hi == 0) {
    const float lse = l_tot > 0.f ? (st.m_run + __builtin_amdgcn_logf(l_tot)) * kLn2 : -INFINITY;
    p.lse[part * p.lse_part + ((int64_t)b * p.n_heads + h) * ((int64_t)p.n_qtiles * kTile) + qrow] = lse;
  }
}

}  // namespace ua

namespace ua {

static int fwd_common(FwdParams& p, const void* q, const void* k, const void* v, void* o, float* lse,
                      int batch, int n_heads, int n_qtiles, int n_ktiles, int head_dim,
                      const int64_t* q_strides, const int64_t* k_strides, const int64_t* v_strides,
                      const int64_t* o_strides, float softmax_scale) {
  if (!q || !k || !v || !o || !lse || !q_strides || !k_strides || !v_strides || !o_strides) return UA_ERR_NULL;
  if (batch <= 0 || n_heads <= 0 || n_qtiles <= 0 || n_ktiles <= 0) return UA_ERR_SHAPE;
  if ((int64_t)batch * n_heads * n_qtiles * UA_MAX_PARTS > INT32_MAX) return UA_ERR_SHAPE;
  if (head_dim != kHeadDim || !(softmax_scale > 0.f)) return UA_ERR_UNSUPPORTED;
  if (!aligned16(q) || !aligned16(k) || !aligned16(v) || !aligned16(o)) return UA_ERR_ALIGN;
  if (!strides_ok(q_strides) || !strides_ok(k_strides) || !strides_ok(v_strides) || !strides_ok(o_strides))
    return UA_ERR_ALIGN;
  if (k_strides[1] > (INT32_MAX >> 9) || v_strides[1] > (INT32_MAX >> 9)) return UA_ERR_SHAPE;
  p.q = (const bf16*)q; p.k = (const bf16*)k; p.v = (const bf16*)v; p.o = (bf16*)o; p.lse = lse;
  p.row_ptr = nullptr; p.col_idx = nullptr; p.flag = nullptr; p.q_order = nullptr;
  p.batch = batch; p.n_heads = n_heads; p.n_qtiles = n_qtiles; p.n_ktiles = n_ktiles; p.nnz = 0;
  p.qs = {q_strides[0], q_strides[1], q_strides[2]};
  p.ks = {k_strides[0], k_strides[1], k_strides[2]};
  p.vs = {v_strides[0], v_strides[1], v_strides[2]};
  p.os = {o_strides[0], o_strides[1], o_strides[2]};
  p.scale_log2 = softmax_scale * kLog2e;
  const int nbh = batch * n_heads;
  p.heads_per_xcd = (nbh % 8 == 0) ? nbh / 8 : 0;
  p.dense = 0; p.dense_causal = 0; p.diag_off = 0; p.n_parts = 1; p.part_len = n_ktiles; p.o_part = 0; p.lse_part = 0;
  return check_device();
}

static int fwd_launch(const FwdParams& p, hipStream_t st) {
  hipLaunchKernelGGL(fwd_kernel, dim3((unsigned)(p.batch * p.n_heads * p.n_qtiles * p.n_parts)), dim3(256), 0, st, p);
  return hipGetLastError() == hipSuccess ? UA_OK : UA_ERR_LAUNCH;
}

static bool contiguous_bshd(const int64_t* st, int seqlen, int n_heads) {
  return st[2] == kHeadDim && st[1] == (int64_t)n_heads * kHeadDim && st[0] == (int64_t)seqlen * n_heads * kHeadDim;
}

}  // namespace ua

extern "C" int ua_bsa_fwd(const void* q, const void* k, const void* v, void* o, float* lse,
                          const int32_t* row_ptr, const int32_t* col_idx, const uint8_t* flag,
                          const int32_t* q_order,
                          int batch, int n_heads, int n_qtiles, int n_ktiles, int nnz, int head_dim,
                          const int64_t* q_strides, const int64_t* k_strides, const int64_t* v_strides,
                          const int64_t* o_strides, float softmax_scale, void* stream) {
  using namespace ua;
  if (!row_ptr || !q_order) return UA_ERR_NULL;
  if (nnz < 0) return UA_ERR_SHAPE;
  if (nnz > 0 && (!col_idx || !flag)) return UA_ERR_NULL;      // only an empty list may leave them out
  if (flag && !aligned4(flag)) return UA_ERR_ALIGN;            // read one aligned 32-bit word at a time
  FwdParams p;
  if (int rc = fwd_common(p, q, k, v, o, lse, batch, n_heads, n_qtiles, n_ktiles, head_dim, q_strides, k_strides,
                          v_strides, o_strides, softmax_scale)) return rc;
  p.row_ptr = row_ptr; p.col_idx = col_idx; p.flag = flag; p.q_order = q_order; p.nnz = nnz;
  return fwd_launch(p, (hipStream_t)stream);
}

extern "C" int64_t ua_dense_workspace_bytes(int batch, int n_heads, int seqlen_q, int seqlen_k, int backward) {
  using namespace ua;
  if (batch <= 0 || n_heads <= 0 || seqlen_q <= 0 || seqlen_k <= 0 || seqlen_q % kTile || seqlen_k % kTile) return 0;
  const DenseSplit d = dense_split(batch, n_heads, seqlen_q / kTile, seqlen_k / kTile);
  return backward ? d.bwd_total : d.fwd_total;
}

extern "C" int ua_dense_fwd(const void* q, const void* k, const void* v, void* o, float* lse,
                            int batch, int n_heads, int seqlen_q, int seqlen_k, int head_dim,
                            const int64_t* q_strides, const int64_t* k_strides, const int64_t* v_strides,
                            const int64_t* o_strides, float softmax_scale, int causal,
                            void* workspace, int64_t workspace_bytes, void* stream) {
  using namespace ua;
  if (seqlen_q <= 0 || seqlen_k <= 0 || seqlen_q % kTile || seqlen_k % kTile) return UA_ERR_SHAPE;
  const int n_qtiles = seqlen_q / kTile, n_ktiles = seqlen_k / kTile;
  FwdParams p;
  if (int rc = fwd_common(p, q, k, v, o, lse, batch, n_heads, n_qtiles, n_ktiles, head_dim, q_strides, k_strides,
                          v_strides, o_strides, softmax_scale)) return rc;
  p.dense = 1; p.dense_causal = causal != 0; p.diag_off = n_ktiles - n_qtiles;
  hipStream_t st = (hipStream_t)stream;
  const DenseSplit d = dense_split(batch, n_heads, n_qtiles, n_ktiles);
  // the split path needs the caller's workspace and a contiguous output for the merge
  const bool split = d.fwd_parts > 1 && workspace && aligned16(workspace) && workspace_bytes >= d.fwd_total &&
                     contiguous_bshd(o_strides, seqlen_q, n_heads);
  if (!split) return fwd_launch(p, st);
  const int len = (n_ktiles + d.fwd_parts - 1) / d.fwd_parts;
  const int parts = (n_ktiles + len - 1) / len;
  unsigned char* ws = static_cast<unsigned char*>(workspace);
  p.o = reinterpret_cast<bf16*>(ws);
  p.lse = reinterpret_cast<float*>(ws + (int64_t)parts * d.fwd_o_bytes);
  p.o_part = d.fwd_o_bytes / 2; p.lse_part = d.fwd_lse_bytes / 4;
  p.os = {(int64_t)seqlen_q * n_heads * kHeadDim, (int64_t)n_heads * kHeadDim, kHeadDim};
  p.n_parts = parts; p.part_len = len;
  if (int rc = fwd_launch(p, st)) return rc;
  const void* op[UA_MAX_PARTS];
  const float* lp[UA_MAX_PARTS];
  for (int i = 0; i < parts; ++i) { op[i] = p.o + i * p.o_part; lp[i] = p.lse + i * p.lse_part; }
  return ua_merge(op, lp, parts, o, lse, batch, seqlen_q, n_heads, head_dim, stream);
}
