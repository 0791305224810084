/*
 * ultraattn.h — C ABI of the MI355X (gfx950) block-sparse attention tile library.
 *
 * The reference (oliverYoung2001/UltraAttn) has no FFI of its own for this path: its executors
 * call the Python functions `_flash_attn_forward` / `_flash_attn_backward` of an un-vendored
 * flash-attention fork and a pure-torch merge.  Each entry point below names the reference
 * interface it replaces (paths relative to the reference's root).
 *
 * Conventions
 *  - All tensor arguments are DEVICE pointers owned by the caller; the library never allocates,
 *    frees or synchronises.  Work is enqueued on `stream` (a hipStream_t, NULL = default stream).
 *  - q, o, dout, dq : [batch, n_qtiles*128, n_heads, 128] bf16, k, v, dk, dv :
 *    [batch, n_ktiles*128, n_heads, 128] bf16; the innermost (head_dim) axis is contiguous and
 *    `*_strides` give the element strides of (batch, token, head), each a multiple of 8.
 *  - lse, delta : [batch, n_heads, n_qtiles*128] fp32, contiguous (the fork's softmax_lse layout,
 *    orchestrated_attn/orchestrated_attn_impl.py:326 "lse: [mbs, Nh, S]").  Natural log.
 *  - A tile list is the compacted form of a block mask at 128x128 granularity: CSR over query
 *    tiles (row_ptr/col_idx/flag, row-major order = search_algo/dependent_graph.py:235-240) and
 *    the transposed CSC over key tiles.  flag 0 = full tile, 1 = causal tile (key j visible to
 *    query i iff j <= i on tile-local indices; such tiles sit on the mask's diagonal,
 *    orchestrated_attn/orchestrated_attn_impl.py:91).  `*_order` is a permutation of the tile
 *    rows (columns) giving the launch order, a performance hint that does not change results:
 *    rows much longer than average first, the rest grouped by their first (or, where that is
 *    shared by more rows, last) index, longer block rows first, then lexicographically, so that
 *    rows sharing K/V tiles run together.
 *    `nnz` is the number of entries of col_idx/flag (row_idx/cflag): the kernels clamp every
 *    list bound to it, and only an empty list (nnz = 0) may pass NULL for those arrays.
 *    flag / cflag are read one aligned 32-bit word at a time: they must start on a 4-byte boundary
 *    (else UA_ERR_ALIGN) and be readable up to the next multiple of 4 bytes after entry nnz-1, i.e.
 *    allocate (nnz + 3) / 4 * 4 bytes; the padding bytes are never interpreted.
 *  - Every function returns 0 (UA_OK) or a negative UA_ERR_* code; ua_strerror() names it.
 *    No exceptions cross this boundary and nothing aborts.
 *  - Functions may be called from several host threads on different streams.  The only state
 *    the library keeps is per-device and write-once (the device check's result and the address of
 *    the fixed scratch), set by ua_init() or by the first call on a device; the one exception is the
 *    CONTENT of that scratch, which ua_tilelist_build_device_noalloc calls on one GPU share (see
 *    there).
 */
#ifndef ULTRAATTN_H
#define ULTRAATTN_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define UA_OK 0
#define UA_ERR_NULL (-1)        /* a required pointer is NULL */
#define UA_ERR_SHAPE (-2)       /* non-positive or inconsistent sizes */
#define UA_ERR_UNSUPPORTED (-3) /* head_dim != 128, softmax_scale <= 0, too many partials */
#define UA_ERR_ALIGN (-4)       /* pointer not 16-byte aligned or stride not a multiple of 8 */
#define UA_ERR_MASK (-5)        /* block mask holds a value other than 0, 1, 2 */
#define UA_ERR_LAUNCH (-6)      /* the HIP runtime rejected the launch */
#define UA_ERR_DEVICE (-7)      /* current device is not a gfx950 GPU */
#define UA_ERR_TOO_LARGE (-8)   /* input exceeds the fixed scratch of a no-allocation entry point */

#define UA_TILE 128        /* rows and columns of one kernel tile */
#define UA_HEAD_DIM 128    /* the only supported head dimension */
#define UA_MAX_PARTS 16    /* most partial outputs one ua_merge call combines */
#define UA_NOALLOC_MAX_LINES 65532   /* most query tiles + key tiles of ua_tilelist_build_device_noalloc */

/* 100 * major + minor.  102: `nnz` argument of the attention entry points, ua_merge_update, the
 * no-allocation builder, `work` of ua_tilelist_build_device grown to n_qtiles + n_ktiles + 7.  */
#define UA_VERSION 103
int ua_version(void);
const char *ua_strerror(int rc);

/* No counterpart in the reference.  Resolves, for the CURRENT device, everything the entry points
 * otherwise look up on their first call there: the device's architecture (hipGetDeviceProperties)
 * and the address of the library's fixed scratch (hipGetSymbolAddress, which also loads the code
 * object).  Those lookups are not legal while a stream is being captured into a HIP graph, so a
 * caller that captures a FIRST call of any entry point calls ua_init() once per device
 * beforehand, outside capture.  Allocates nothing; idempotent; UA_ERR_DEVICE if the device is not
 * gfx950.                                                                                      */
int ua_init(void);

/* ---- block mask -> active-tile list (host) ------------------------------------------------
 * Replaces the reference's Python enumeration of Comp_Kernels from a block table:
 * search_algo/dependent_graph.py:235-263 (row-major order over schedule_table >= 0) with the
 * refinement rule of search_algo/bsa_config.py:177-213 (complicate_block / complicate).
 * `block_mask` is a HOST array [n_qblocks, n_kblocks] of Block_Type values
 * (search_algo/utils.py:140-143: 0 EMPTY, 1 FULL, 2 CAUSAL); every block is refined into
 * rate x rate tiles (rate = block tokens / 128).  ua_tilelist_size reports the array sizes,
 * ua_tilelist_build fills caller-allocated HOST arrays:
 *   row_ptr[n_qtiles+1], col_idx[nnz], flag[nnz]      CSR over query tiles
 *   col_ptr[n_ktiles+1], row_idx[nnz], cflag[nnz]     CSC over key tiles
 *   q_order[n_qtiles], k_order[n_ktiles]              launch orders                         */
int ua_tilelist_size(const uint8_t *block_mask, int n_qblocks, int n_kblocks, int rate,
                     int64_t *n_qtiles, int64_t *n_ktiles, int64_t *nnz);
int ua_tilelist_build(const uint8_t *block_mask, int n_qblocks, int n_kblocks, int rate,
                      int32_t *row_ptr, int32_t *col_idx, uint8_t *flag,
                      int32_t *col_ptr, int32_t *row_idx, uint8_t *cflag,
                      int32_t *q_order, int32_t *k_order);

/* Device-side variant: `block_mask` and all outputs are DEVICE arrays (sizes as above, from
 * ua_tilelist_size on a host copy or an upper bound nnz <= n_qtiles*n_ktiles); `work` is a
 * device scratch of (n_qtiles + n_ktiles + 7) int32.  Produces the same arrays bit for bit.
 * The mask cannot be validated without a synchronisation: an entry that is not 0, 1 or 2 is
 * treated as EMPTY, and work[n_qtiles + n_ktiles + 2] receives the number of such entries (0 for
 * a valid mask; the host builder returns UA_ERR_MASK instead) for the caller to read later.
 * Cost: counting, filling and the anchor statistics are linear in the mask; the launch order ranks
 * every line against every other line of its side (comparisons stop at the first differing
 * index), i.e. it grows with the square of the number of lines.  Measured on MI355X, n_qtiles +
 * n_ktiles lines: 2 048 lines 0.1-0.3 ms, 8 192 lines 0.4-1.0 ms (dense causal: 0.4 ms),
 * 16 384 lines 1.1-2.7 ms, 32 768 lines 5-10 ms, 65 532 lines 34-45 ms (band and causal-band masks);
 * the benchmark masks have 2 048 to 4 608 lines (0.07-0.1 ms).                                */
int ua_tilelist_build_device(const uint8_t *block_mask, int n_qblocks, int n_kblocks, int rate,
                             int32_t *row_ptr, int32_t *col_idx, uint8_t *flag,
                             int32_t *col_ptr, int32_t *row_idx, uint8_t *cflag,
                             int32_t *q_order, int32_t *k_order, int32_t *work, void *stream);

/* No counterpart in the reference.  For callers that cannot allocate device memory (code under
 * HIP graph capture, tight serving loops, harnesses that forbid it): the same builder as
 * ua_tilelist_build_device with the `work` scratch taken from a fixed array inside the library
 * (256 KiB + 16 B per GPU, held until the process ends) instead of from the caller.  Limit:
 * n_qtiles + n_ktiles <= UA_NOALLOC_MAX_LINES, else UA_ERR_TOO_LARGE.  `n_invalid` (device,
 * may be NULL) receives the number of mask entries that are not 0, 1 or 2.  It calls no
 * hipMalloc/hipFree.  All calls on one GPU share the array: calls that overlap in time on the
 * same GPU (different streams or threads) race; serialise them.  The first call on a device looks
 * up the scratch address (see ua_init): under graph capture call ua_init() first.              */
int ua_tilelist_build_device_noalloc(const uint8_t *block_mask, int n_qblocks, int n_kblocks, int rate,
                                     int32_t *row_ptr, int32_t *col_idx, uint8_t *flag,
                                     int32_t *col_ptr, int32_t *row_idx, uint8_t *cflag,
                                     int32_t *q_order, int32_t *k_order, int32_t *n_invalid, void *stream);

/* ---- forward ------------------------------------------------------------------------------
 * Replaces the N dense `_flash_attn_forward(q, k, v, dropout_p, softmax_scale, causal=, ...,
 * out=)` launches of fwd_comp_func (orchestrated_attn/orchestrated_attn_impl.py:320-338; same
 * call hierarchy_attn/hierarchy_attn_impl.py:40-53) by one launch over the tile list.
 * Writes o (bf16) and lse (fp32) for every query row; rows without an active tile get o = 0,
 * lse = -inf.                                                                               */
int ua_bsa_fwd(const void *q, const void *k, const void *v, void *o, float *lse,
               const int32_t *row_ptr, const int32_t *col_idx, const uint8_t *flag,
               const int32_t *q_order,
               int batch, int n_heads, int n_qtiles, int n_ktiles, int nnz, int head_dim,
               const int64_t *q_strides, const int64_t *k_strides, const int64_t *v_strides,
               const int64_t *o_strides, float softmax_scale, void *stream);

/* ---- backward -----------------------------------------------------------------------------
 * Replace `_flash_attn_backward(dout, q, k, v, out, softmax_lse, dq, dk, dv, ..., softmax_d=)`
 * of bwd_comp_func (orchestrated_attn/orchestrated_attn_impl.py:574-597).
 * ua_bsa_bwd_delta : delta = rowsum(dout * o), the `softmax_d` the reference precomputes.
 * ua_bsa_bwd_dkdv  : dk, dv for every key row (walks the CSC, no atomics); key rows without an
 *                    active tile get 0.
 * ua_bsa_bwd_dq    : dq for every query row (walks the CSR).
 * lse and delta are the rows' global statistics, the same for every tile of a row
 * (ring_flash_attn/ring_flash_attn.py:91-108).  Outputs are overwritten, not accumulated. */
int ua_bsa_bwd_delta(const void *o, const void *dout, float *delta,
                     int batch, int seqlen_q, int n_heads, int head_dim,
                     const int64_t *o_strides, const int64_t *do_strides, void *stream);
int ua_bsa_bwd_dkdv(const void *q, const void *k, const void *v, const void *dout,
                    const float *lse, const float *delta, void *dk, void *dv,
                    const int32_t *col_ptr, const int32_t *row_idx, const uint8_t *cflag,
                    const int32_t *k_order,
                    int batch, int n_heads, int n_qtiles, int n_ktiles, int nnz, int head_dim,
                    const int64_t *q_strides, const int64_t *k_strides, const int64_t *v_strides,
                    const int64_t *do_strides, const int64_t *dk_strides, const int64_t *dv_strides,
                    float softmax_scale, void *stream);
int ua_bsa_bwd_dq(const void *q, const void *k, const void *v, const void *dout,
                  const float *lse, const float *delta, void *dq,
                  const int32_t *row_ptr, const int32_t *col_idx, const uint8_t *flag,
                  const int32_t *q_order,
                  int batch, int n_heads, int n_qtiles, int n_ktiles, int nnz, int head_dim,
                  const int64_t *q_strides, const int64_t *k_strides, const int64_t *v_strides,
                  const int64_t *do_strides, const int64_t *dq_strides,
                  float softmax_scale, void *stream);

/* ---- dense rectangles: the reference's tile kernel itself ------------------------------------
 * One call = one `_flash_attn_forward(q, k, v, dropout_p=0, softmax_scale, causal, ..., out=)`
 * (orchestrated_attn/orchestrated_attn_impl.py:326-337, hierarchy_attn/hierarchy_attn_impl.py:41-51)
 * or one `_flash_attn_backward(dout, q, k, v, out, softmax_lse, dq, dk, dv, ..., softmax_d=)`
 * (orchestrated_attn_impl.py:578-596) over a dense seqlen_q x seqlen_k rectangle (multiples of 128),
 * with no tile list: the kernels enumerate the tiles themselves.  causal != 0 aligns the diagonal
 * to the bottom-right corner as flash-attn >= 2.1 does (query i sees key j iff
 * j <= i + seqlen_k - seqlen_q; rows that see no key get o = 0, lse = -inf, zero gradients).
 * Rectangles with few tile lines (B * Nh * seqlen / 128 well below two workgroups per CU) and long
 * walks are cut into up to UA_MAX_PARTS parts that run as workgroups of their own: the forward
 * leaves partial (O, LSE) and finishes with ua_merge's kernel, the backward leaves fp32 partial
 * dQ (parts of the key range) and dK, dV (parts of the query range) and sums them in one pass.
 * The partials live in `workspace` (device memory, 16-byte aligned, caller-owned, overwritten by
 * every call: calls that share it must not overlap); ua_dense_workspace_bytes() gives the size
 * that lets a shape split (0 = it never splits).  With workspace == NULL or too small, or a
 * forward output that is not contiguous, the call runs unsplit: same results, one workgroup per
 * line.                                                                                       */
int64_t ua_dense_workspace_bytes(int batch, int n_heads, int seqlen_q, int seqlen_k, int backward);
int ua_dense_fwd(const void *q, const void *k, const void *v, void *o, float *lse,
                 int batch, int n_heads, int seqlen_q, int seqlen_k, int head_dim,
                 const int64_t *q_strides, const int64_t *k_strides, const int64_t *v_strides,
                 const int64_t *o_strides, float softmax_scale, int causal,
                 void *workspace, int64_t workspace_bytes, void *stream);
int ua_dense_bwd(const void *dout, const void *q, const void *k, const void *v,
                 const float *lse, const float *delta, void *dq, void *dk, void *dv,
                 int batch, int n_heads, int seqlen_q, int seqlen_k, int head_dim,
                 const int64_t *q_strides, const int64_t *k_strides, const int64_t *v_strides,
                 const int64_t *do_strides, const int64_t *dq_strides, const int64_t *dk_strides,
                 const int64_t *dv_strides, float softmax_scale, int causal,
                 void *workspace, int64_t workspace_bytes, void *stream);

/* ---- merge of partial outputs ---------------------------------------------------------------
 * Replaces the chain of `update_out_and_lse` calls (ring_flash_attn/utils.py:38-52, 78-99;
 * hierarchy_attn/utils.py:16-56; the commented formula at orchestrated_attn/utils.py:120-133)
 * by one pass over n_parts partials:  LSE = log sum_p exp(lse_p),  O = sum_p exp(lse_p - LSE) O_p
 * (max-stabilised; a partial with lse = -inf contributes nothing).
 * o_parts / lse_parts are HOST arrays of n_parts DEVICE pointers: o_parts[p] is a contiguous
 * [batch, seqlen, n_heads, 128] bf16 tensor, lse_parts[p] a contiguous [batch, n_heads, seqlen]
 * fp32 tensor; o and lse have the same layouts.  o / lse may alias partial 0.               */
int ua_merge(const void *const *o_parts, const float *const *lse_parts, int n_parts,
             void *o, float *lse, int batch, int seqlen, int n_heads, int head_dim, void *stream);

/* In-place form of one `update_out_and_lse(out, lse, block_out, block_lse, slice_=None)` step
 * (ring_flash_attn/utils.py:78-99, called with a row slice at
 * hierarchy_attn/hierarchy_attn_impl.py:75-81): new_lse = logaddexp(lse, block_lse),
 * new_out = exp(lse - new_lse) out + exp(block_lse - new_lse) block_out, max-stabilised.
 * Every tensor is addressed through (batch, token, head) ELEMENT strides: rows
 * [batch, n_rows, n_heads, 128] with head_dim contiguous (a row range of a larger tensor is a
 * pointer offset), statistics fp32 in either the reference's running layout [B, S, Nh, 1]
 * (strides S*Nh, Nh, 1) or the kernels' [B, Nh, S] (strides Nh*S, 1, S).  `*_is_fp32` select
 * fp32 or bf16 rows (the reference's running `out` turns fp32 after its first update).
 * new_out / new_lse may be exactly out / lse (the slice_ path: same pointer, then the same element
 * type and strides are required, else UA_ERR_SHAPE) or buffers that do not overlap them; partial
 * overlap is undefined.  Row strides must keep rows
 * 16-byte aligned (multiples of 8 bf16 / 4 fp32 elements).                                   */
int ua_merge_update(const void *out, const float *lse, const void *block_out, const float *block_lse,
                    void *new_out, float *new_lse, int batch, int n_rows, int n_heads, int head_dim,
                    int out_is_fp32, int block_is_fp32, int new_is_fp32,
                    const int64_t *out_strides, const int64_t *lse_strides,
                    const int64_t *block_out_strides, const int64_t *block_lse_strides,
                    const int64_t *new_out_strides, const int64_t *new_lse_strides, void *stream);

/* ---- accumulation of partial gradients -------------------------------------------------------
 * The reduce() of the gradient packs that the reference leaves as stubs
 * (orchestrated_attn/utils.py:260-262, 296-298: `self.data.add_(other.data)` commented out), with
 * the accumulation its ring executor specifies (ring_flash_attn/ring_flash_attn.py:110-118:
 * partial dq/dk/dv are added into fp32 buffers and cast to bf16 once).
 * ua_grad_accumulate: one step of a running sum over `n` contiguous elements (n a multiple of 8),
 *   acc != NULL, init_from_out == 0 :  acc += partial;  out = bf16(acc) when out != NULL
 *   acc != NULL, init_from_out != 0 :  acc  = float(out) + partial;  out = bf16(acc)   (first step)
 *   acc == NULL                     :  out  = bf16(float(out) + partial)
 *   acc fp32, partial and out bf16; one pass (read acc + partial, write acc + out).
 * ua_grad_sum: out = bf16(scale * sum_p parts[p]) over n_parts (1..UA_MAX_PARTS) partial gradients
 *   in one pass.  `parts` is a HOST array of DEVICE pointers to contiguous
 *   [batch, seqlen, n_heads, 128] arrays, fp32 when parts_fp32 != 0, else bf16; `out` is bf16 and
 *   takes (batch, token, head) element strides (multiples of 8).                                */
int ua_grad_accumulate(float *acc, const void *partial, void *out, int64_t n, int init_from_out, void *stream);
int ua_grad_sum(const void *const *parts, int n_parts, int parts_fp32, void *out,
                int batch, int seqlen, int n_heads, int head_dim, const int64_t *out_strides,
                float scale, void *stream);

/* ---- column-buffer layout changes around a fused rectangle -----------------------------------
 * Replace the two torch transpose+contiguous copies of the X x Y path:
 *   ua_cols_gather : buf.view(Y,2,B,Skv,Nh,D).transpose(0,1).transpose(1,2).flatten(2,3).contiguous()
 *                    (orchestrated_attn/orchestrated_attn_impl.py:269 forward, :512 backward):
 *                    src [n_chunks, 2, batch, inner] -> dst [2, batch, n_chunks, inner], so that
 *                    dst is one K and one V of n_chunks*Skv keys each;
 *   ua_cols_scatter: oc.view(2, Y, K_nelem).transpose(0,1).contiguous()
 *                    (orchestrated_attn_impl.py:548): src [2, batch, n_chunks, inner] ->
 *                    dst [n_chunks, 2, batch, inner], [dK | dV] of the rectangle back to per-chunk
 *                    [dK | dV] (the reference has batch = 1 there).
 * inner_elems = Skv*Nh*D bf16 elements, a multiple of 8; src and dst are device pointers, 16-byte
 * aligned, and must not overlap; 2*n_chunks*batch <= 65535.                                      */
int ua_cols_gather(const void *src, void *dst, int n_chunks, int batch, int64_t inner_elems, void *stream);
int ua_cols_scatter(const void *src, void *dst, int n_chunks, int batch, int64_t inner_elems, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* ULTRAATTN_H */
