"""Minimal nested-structure helpers (dict / list / tuple of tensors).

The reference walks nested MoE inputs with dm-tree
(fmoe/layers.py:59,77,212-219); these two functions cover the calls it makes.
"""
from __future__ import annotations


def map_structure(fn, *structs):
    s = structs[0]
    if isinstance(s, dict):
        return type(s)((k, map_structure(fn, *[x[k] for x in structs])) for k in s)
    if isinstance(s, (list, tuple)):
        items = [map_structure(fn, *xs) for xs in zip(*structs)]
        if isinstance(s, tuple) and hasattr(s, "_fields"):  # namedtuple
            return type(s)(*items)
        return type(s)(items)
    return fn(*structs)


def flatten(struct):
    if isinstance(struct, dict):
        out = []
        for k in sorted(struct):
            out.extend(flatten(struct[k]))
        return out
    if isinstance(struct, (list, tuple)):
        out = []
        for x in struct:
            out.extend(flatten(x))
        return out
    return [struct]
