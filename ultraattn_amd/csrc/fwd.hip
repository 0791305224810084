// Block-sparse flash-attention forward for gfx950 (MI355X).
//
// One workgroup (4 wavefronts) per (query tile of 128 rows, head).  It walks the query tile's
// CSR entries; per entry the 128x128 K and V tiles are staged in LDS.  Each wavefront owns 32
// query rows and computes the TRANSPOSED products
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
  int batch, n_heads, n_qtiles, n_ktiles;
  Strides3 qs, ks, vs, os;
  float scale_log2;      // softmax_scale * log2(e)
  int heads_per_xcd;     // batch*n_heads / 8 when divisible, else 0
};

__global__ __launch_bounds__(256, 2) void fwd_kernel(const FwdParams p) {
  __shared__ __attribute__((aligned(16))) unsigned char smem[2 * kTileBytes];
  unsigned char* sK = smem;
  unsigned char* sV = smem + kTileBytes;

  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int l32 = lane & 31, hi = lane >> 5;

  int pos, bh;
  map_block(blockIdx.x, p.batch * p.n_heads, p.heads_per_xcd, pos, bh);
  const int qt = p.q_order[pos];
  const int b = bh / p.n_heads, h = bh % p.n_heads;

  // Q fragment (B operand of S^T): lane holds query row 32*wave + lane%32,
  // d = 16*ks + 8*(lane/32) .. +7 for ks = 0..7.
  const int qrow = qt * kTile + wave * 32 + l32;
  const bf16* qp = p.q + b * p.qs.b + (int64_t)qrow * p.qs.s + h * p.qs.h + hi * 8;
  bf16x8 qf[8];
#pragma unroll
  for (int ks = 0; ks < 8; ++ks) qf[ks] = *reinterpret_cast<const bf16x8*>(qp + ks * 16);

  f32x16 oacc[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) oacc[i] = f32x16{0};
  float m_run = -INFINITY;   // running row max, log2 domain (already scaled)
  float l_run = 0.f;         // this half-wave's partial row sum

  const bf16* kbase = p.k + b * p.ks.b + h * p.ks.h;
  const bf16* vbase = p.v + b * p.vs.b + h * p.vs.h;
  const int e0 = p.row_ptr[qt], e1 = p.row_ptr[qt + 1];

  const TrLane tr(lane);

  for (int e = e0; e < e1; ++e) {
    const int kt = p.col_idx[e];
    const int causal = p.flag[e];
    if ((unsigned)kt >= (unsigned)p.n_ktiles) continue;   // uniform: never index outside K/V
    __syncthreads();
    stage_tile<lds_off_k>(sK, kbase + (int64_t)kt * kTile * p.ks.s, p.ks.s, tid);
    stage_tile<lds_off_v>(sV, vbase + (int64_t)kt * kTile * p.vs.s, p.vs.s, tid);
    __syncthreads();

    // ---- S^T = K Q^T : 4 blocks of 32 keys x 32 queries --------------------------------
    f32x16 s[4];
#pragma unroll
    for (int mb = 0; mb < 4; ++mb) {
      s[mb] = f32x16{0};
#pragma unroll
      for (int ks = 0; ks < 8; ++ks) {
        bf16x8 a = lds_read_b128(sK, lds_off_k(32 * mb + l32, 2 * ks + hi));
        s[mb] = mfma32(a, qf[ks], s[mb]);
      }
    }
    // element (mb, i) of this lane: key 32*mb + 8*(i/4) + 4*hi + i%4, query 32*wave + l32
    if (causal) {
      const int ql = wave * 32 + l32;
#pragma unroll
      for (int mb = 0; mb < 4; ++mb)
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          const int key = 32 * mb + 8 * (i >> 2) + 4 * hi + (i & 3);
          if (key > ql) s[mb][i] = -INFINITY;
        }
    }
    // ---- online softmax (fp32, log2 domain) ---------------------------------------------
    float mx = -INFINITY;
#pragma unroll
    for (int mb = 0; mb < 4; ++mb)
#pragma unroll
      for (int i = 0; i < 16; ++i) mx = fmaxf(mx, s[mb][i]);
    mx = xhalf_max(mx) * p.scale_log2;
    const float m_new = fmaxf(m_run, mx);
    const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
    const float alpha = fast_exp2(m_run - m_use);
    m_run = m_new;
    float rs = 0.f;
    bf16x8 pf[8];
#pragma unroll
    for (int mb = 0; mb < 4; ++mb) {
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const float pv = fast_exp2(fmaf(s[mb][i], p.scale_log2, -m_use));
        rs += pv;
        pf[mb * 2 + (i >> 3)][i & 7] = (bf16)pv;
      }
    }
    l_run = l_run * alpha + rs;
#pragma unroll
    for (int mbd = 0; mbd < 4; ++mbd)
#pragma unroll
      for (int i = 0; i < 16; ++i) oacc[mbd][i] *= alpha;

    // ---- O^T += V^T P^T : 4 blocks of 32 d x 32 queries, 8 steps of 16 keys ----------------
#pragma unroll
    for (int kk = 0; kk < 8; ++kk) {
#pragma unroll
      for (int mbd = 0; mbd < 4; ++mbd) {
        const bf16x8 a = lds_read_tr_frag<lds_off_v>(sV, tr, 16 * kk, mbd);
        oacc[mbd] = mfma32(a, pf[kk], oacc[mbd]);
      }
    }
  }

  // ---- epilogue: normalise, write O (bf16) and LSE (natural log) -------------------------
  const float l_tot = xhalf_sum(l_run);
  const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
  bf16* op = p.o + b * p.os.b + (int64_t)qrow * p.os.s + h * p.os.h;
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
    const float lse = l_tot > 0.f ? (m_run + __builtin_amdgcn_logf(l_tot)) * kLn2 : -INFINITY;
    p.lse[((int64_t)b * p.n_heads + h) * ((int64_t)p.n_qtiles * kTile) + qrow] = lse;
  }
}

}  // namespace ua

extern "C" int ua_bsa_fwd(const void* q, const void* k, const void* v, void* o, float* lse,
                          const int32_t* row_ptr, const int32_t* col_idx, const uint8_t* flag,
                          const int32_t* q_order,
                          int batch, int n_heads, int n_qtiles, int n_ktiles, int head_dim,
                          const int64_t* q_strides, const int64_t* k_strides, const int64_t* v_strides,
                          const int64_t* o_strides, float softmax_scale, void* stream) {
  using namespace ua;
  if (!q || !k || !v || !o || !lse || !row_ptr || !q_order || !q_strides || !k_strides || !v_strides || !o_strides)
    return UA_ERR_NULL;
  if (batch <= 0 || n_heads <= 0 || n_qtiles <= 0 || n_ktiles <= 0) return UA_ERR_SHAPE;
  if ((int64_t)batch * n_heads * n_qtiles > INT32_MAX) return UA_ERR_SHAPE;
  if (head_dim != kHeadDim || !(softmax_scale > 0.f)) return UA_ERR_UNSUPPORTED;
  if (!aligned16(q) || !aligned16(k) || !aligned16(v) || !aligned16(o)) return UA_ERR_ALIGN;
  if (!strides_ok(q_strides) || !strides_ok(k_strides) || !strides_ok(v_strides) || !strides_ok(o_strides))
    return UA_ERR_ALIGN;
  if (int rc = check_device()) return rc;
  FwdParams p;
  p.q = (const bf16*)q; p.k = (const bf16*)k; p.v = (const bf16*)v; p.o = (bf16*)o; p.lse = lse;
  p.row_ptr = row_ptr; p.col_idx = col_idx; p.flag = flag; p.q_order = q_order;
  p.batch = batch; p.n_heads = n_heads; p.n_qtiles = n_qtiles; p.n_ktiles = n_ktiles;
  p.qs = {q_strides[0], q_strides[1], q_strides[2]};
  p.ks = {k_strides[0], k_strides[1], k_strides[2]};
  p.vs = {v_strides[0], v_strides[1], v_strides[2]};
  p.os = {o_strides[0], o_strides[1], o_strides[2]};
  p.scale_log2 = softmax_scale * kLog2e;
  const int nbh = batch * n_heads;
  p.heads_per_xcd = (nbh % 8 == 0) ? nbh / 8 : 0;
  hipLaunchKernelGGL(fwd_kernel, dim3((unsigned)(nbh * n_qtiles)), dim3(256), 0, (hipStream_t)stream, p);
  return hipGetLastError() == hipSuccess ? UA_OK : UA_ERR_LAUNCH;
}
