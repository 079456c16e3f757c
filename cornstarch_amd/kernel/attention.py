"""Tile constants of the materialized-mask sibling kernel.

The reference's context-parallel split code imports ``BLOCK_M`` / ``BLOCK_N`` from
``cornstarch.kernel.attention`` (cornstarch/kernel/attention.py:51-52,
cornstarch/shardformer/layers/utils.py:11); they are the granularity of the tile flags.
The materialized-mask kernel itself (``flash_attn_func``, attention.py:1126) is not part of
this build.
"""

BLOCK_M = 128
BLOCK_N = 32


def flash_attn_func(*args, **kwargs):
    raise NotImplementedError(
        "the materialized-mask attention kernel is not part of this build; "
        "use cornstarch_amd.kernel.bitfield_attention.bitfield_attn_func"
    )
