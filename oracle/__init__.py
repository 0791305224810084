"""CPU oracle for the block-sparse attention hot path.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package (``ultraattn_amd``) may import,
call or fall back to anything in this directory.  Only ``tests/``, the smoke check in
``__graft_entry__.py`` and the ``cpu_baseline`` leg of ``bench.py`` use it, and only as the
checker or as the timed CPU baseline, never as the product path.

It restates, in plain fp32/fp64 torch-on-CPU and numpy, the algorithm that the reference's
per-device attention path runs (reference = oliverYoung2001/UltraAttn, paths below relative to
its root):

* the attention tile itself is a call into the un-vendored ``flash_attn`` fork
  (``v2.5.7_burst``, ``.gitmodules:11-14``; call sites
  ``orchestrated_attn/orchestrated_attn_impl.py:326-337, 578-596``).  That package is absent,
  so the tile is restated from its published definition, the textbook softmax attention that
  the reference itself uses as its check (``easy_context/dist_flash_attn/lightseq_async_attn.py:482-488``);
* the merge follows ``ring_flash_attn/utils.py:38-52, 78-99`` line by line;
* the block-mask algebra follows ``search_algo/bsa_config.py:177-213`` and the tile
  enumeration order follows ``search_algo/dependent_graph.py:235-240``;
* the column-buffer gather / scatter around a fused rectangle follows
  ``orchestrated_attn/orchestrated_attn_impl.py:269, 512, 548``.

Pinning status (what each function is checked against, see tests/test_oracle_*.py):

* ``tile_fwd``        : torch SDPA / logsumexp, closed forms (Q=0, constant V, single key,
                        causal row 0), fp64 brute force with Python loops.            PINNED
* ``tile_bwd``        : torch.autograd on the dense formula in fp64, gradcheck,
                        finite differences, row-sum identities.                       PINNED
* ``update_out_and_lse`` / ``merge_partials`` : torch.logaddexp, single-pass result over the
                        union of key sets, equal-LSE average, -inf identity.          PINNED
* ``accumulate_gradients`` : left-to-right fp32 sum equals the fp64 sum rounded to fp32 on
                        exactly representable inputs; differs from a bf16 running sum.    PINNED
* ``tilelist``        : brute-force element mask, counts derived independently,
                        reference-held mask strings and allocation logs.              PINNED
* ``layout_oracle``   : explicit index loops, the reference's torch view/transpose chain,
                        round trip.                                                   PINNED
* flash_attn fork's own numerics (rounding order inside its CUDA kernel): no reference
  test or fixture pins a number at that boundary                                      PARITY UNPINNED
"""
