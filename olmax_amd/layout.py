"""The flat parameter layout of libolmax_hip, by leaf name: how the reference's Equinox pytree
maps onto the buffers the whole-model entry points take.

``olmax_model_layout`` (a host-only query of the library) lists every parameter leaf with its
element offset in the flat fp32 master / bf16 working / bf16 gradient buffers.  The leaves
carry the reference's pytree paths (``layers.{l}.attention.q_proj.weight`` ..., reference
src/olmax/nn/transformer/layer.py:21-24,120-121; src/olmax/nn/attention.py:113-120;
src/olmax/nn/mlp.py:14-16; ``embedding.weight``, ``norm.weight``, ``lm_head.proj.weight``,
src/olmax/nn/transformer/model.py:24-29), so a host packs its pytree ONCE into the flat buffers
and from then on hands the library four pointers.  Inside a layer q|k|v and gate|up are adjacent,
which is what lets each pair be one GEMM.

Works on any array type with ``reshape`` / ``__setitem__`` (numpy on the host, jax via
``flat.at[a:b].set``-style callers use ``leaf_table`` directly); needs no GPU.
"""
from __future__ import annotations

import ctypes
from typing import Dict, List, NamedTuple, Tuple

from . import _lib


class Leaf(NamedTuple):
    name: str       # the reference's dotted pytree path
    offset: int     # element offset in the flat parameter-layout buffers
    shape: Tuple[int, ...]
    grad_f32: bool  # gradient accumulated in fp32 (embedding, norm weights) at grad_f32_offset
    grad_f32_offset: int


def leaf_table(config, batch_size: int = 1, sequence_length: int = 1) -> List[Leaf]:
    """Leaves of ``config`` (a TransformerConfig) in layout order."""
    from .transformer import _LEAF_NAMES, CLeaf

    L = _lib.load()
    c = config.c_config(batch_size, sequence_length)
    n = L.olmax_model_layout(ctypes.byref(c), None, 0)
    if n < 0:
        raise _lib.OlmaxHipError(L.olmax_last_error_string().decode())
    arr = (CLeaf * n)()
    L.olmax_model_layout(ctypes.byref(c), arr, n)
    return [Leaf(_LEAF_NAMES[l.kind].format(l=l.layer), l.offset, (l.rows, l.cols) if l.rows > 1 else (l.cols,),
                 bool(l.grad_f32), l.grad_f32_offset) for l in arr]


def num_params(config) -> int:
    L = _lib.load()
    L.olmax_model_num_params.restype = ctypes.c_int64
    c = config.c_config(1, 1)
    return int(L.olmax_model_num_params(ctypes.byref(c)))


def pack(config, named: Dict[str, "object"], flat) -> None:
    """Copy every named leaf into its slice of ``flat`` (a 1-D array of num_params elements)."""
    table = leaf_table(config)
    missing = [l.name for l in table if l.name not in named]
    extra = sorted(set(named) - {l.name for l in table})
    if missing or extra:
        raise KeyError(f"pack: missing leaves {missing[:4]}, unknown leaves {extra[:4]}")
    for l in table:
        a = named[l.name]
        if tuple(a.shape) != l.shape:
            raise ValueError(f"{l.name}: expected shape {l.shape}, got {tuple(a.shape)}")
        n = 1
        for s in l.shape:
            n *= s
        flat[l.offset: l.offset + n] = a.reshape(-1)


def unpack(config, flat) -> Dict[str, "object"]:
    """Views (for numpy / torch) of every leaf of ``flat`` under the reference's names."""
    out = {}
    for l in leaf_table(config):
        n = 1
        for s in l.shape:
            n *= s
        out[l.name] = flat[l.offset: l.offset + n].reshape(l.shape)
    return out
