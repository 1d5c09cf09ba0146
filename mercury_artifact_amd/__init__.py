"""MI355X (gfx950) implementation of the per-rank compute step of Mercury's ring attention.

Importing the package registers the two block operators and exposes, under the names Mercury's
generated code resolves in its ``exec`` namespace, everything that code calls:
``_flash_attn_forward``, ``_flash_attn_backward``, ``get_default_args``, ``update_out_and_lse``,
``flash_reduce`` and the rank/mesh index helpers.  ``namespace()`` returns them as a dict.
"""
from __future__ import annotations

from . import _native
from .flash_attn_interface import (_flash_attn_backward, _flash_attn_forward, attn_bwd_block,
                                   attn_fwd_block)
from .graph import GraphedStep
from .lazy import LazyLse, LazyOut, update_out_and_lse_lazy
from .merge import (LocalGroup, _update_out_and_lse, add_collective, flash_reduce, get_default_args,
                    grad_accumulate, merge_into, merge_many, pack_block, unpack_into, update_out_and_lse,
                    update_out_and_lse_collective)
from .ring import (flash_attn_backward, flash_attn_expose_reduce, flash_attn_expose_reduce_q_ring,
                   flash_attn_pack_kv,
                   flash_attn_pack_split_kv, fp8_pack_split_kv, gqa_pack_kv, quantize_e4m3,
                   zigzag_causal_pack_kv)
from .schedule import (LocalMesh, LocalRing, debug_print, double_ring_order, get_device_group, get_src_dst_ranks, local_peers,
                       n_dim_to_one_dim, one_dim_to_n_dim, reduce_buffer_route, ring_divide_order, shift_tuple_element, single_ring_order,
                       zigzag_blocks, zigzag_step)

__version__ = "0.1.0"


def namespace(lazy_merge: bool = True) -> dict:
    """Names to place in the dict generated ring code is ``exec``-ed in (the reference fills it with
    ``from utils.flash_attn_dsl import *`` and ``from mercury.backend import *``).

    By default ``update_out_and_lse`` is the recording variant of ``mercury_artifact_amd.lazy``: unchanged
    generated code then folds all block results of a step in one pass when its epilogue runs, instead of
    moving the fp32 accumulator once per chunk (same results to fp32 rounding; anything the lazy handles are
    not asked by the generated epilogue falls back to the literal chain).  ``lazy_merge=False`` binds the
    literal merge of utils/flash_attn_dsl.py:51-71, one kernel per call."""
    return {
        "_flash_attn_forward": _flash_attn_forward,
        "_flash_attn_backward": _flash_attn_backward,
        "get_default_args": get_default_args,
        "update_out_and_lse": update_out_and_lse_lazy if lazy_merge else update_out_and_lse,
        "_update_out_and_lse": _update_out_and_lse,
        "flash_reduce": flash_reduce,
        "merge_many": merge_many,
        "update_out_and_lse_collective": update_out_and_lse_collective,
        "add_collective": add_collective,
        "one_dim_to_n_dim": one_dim_to_n_dim,
        "n_dim_to_one_dim": n_dim_to_one_dim,
        "shift_tuple_element": shift_tuple_element,
        "get_src_dst_ranks": get_src_dst_ranks,
        "get_device_group": get_device_group,
        "debug_print": debug_print,
    }
