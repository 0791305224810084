"""MI355X-native block-sparse attention tiles (forward, backward, LSE merge, tile-list builder)."""
from .masks import (CAUSAL, EMPTY, FULL, calc_flops, canonical_block_table, config_causal, config_global_local,
                    config_streaming_shard, config_strided, total_sparsity)
from .tilelist import TILE, TileList, build_tile_list, build_tile_list_device


def __getattr__(name):
    # torch-dependent operators are imported on first use so that mask / tile-list host logic
    # works without initialising torch.
    if name in ("bsa_fwd", "bsa_bwd", "merge_partials", "softmax_delta", "update_out_and_lse", "grad_accumulate", "grad_sum"):
        from . import ops
        return getattr(ops, name)
    if name in ("BlockSparseExecutor", "mask_from_comp_kernels", "comp_kernels_from_schedule"):
        from . import executor
        return getattr(executor, name)
    if name == "create_buf_dict":
        from . import packed
        return packed.create_buf_dict
    raise AttributeError(name)
