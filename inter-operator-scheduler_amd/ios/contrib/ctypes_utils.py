"""Marshalling helpers between Python objects and the C ABI of the runtime library."""
import ctypes
from typing import Iterable, List, Optional

import numpy as np

from ios.ir import Node, Sequential


def c_int(i: int):
    return ctypes.c_int(int(i))


def c_string(s: str):
    """NUL-terminated UTF-8 copy of ``s`` as ``char *`` (the buffer lives as long as the return value)."""
    return ctypes.c_char_p(s.encode())


def c_string_list(strings: List[str]):
    """``char **`` over copies of ``strings``; keep the returned object alive during the call."""
    array = (ctypes.c_char_p * len(strings))(*[s.encode() for s in strings])
    return array


def c_float_array(n: int):
    return (ctypes.c_float * int(n))()


def c_ndarray(a: np.ndarray):
    return a.ctypes.data_as(ctypes.c_void_p)


def c_ndarray_list(arrays: List[Optional[np.ndarray]]):
    """``float **``: element i points at arrays[i] (or is NULL when arrays[i] is not an ndarray)."""
    pointers = [a.ctypes.data_as(ctypes.c_void_p) if isinstance(a, np.ndarray) else ctypes.c_void_p(None)
                for a in arrays]
    return (ctypes.c_void_p * len(arrays))(*pointers)


def as_f32(a) -> np.ndarray:
    """C-contiguous float32 view or copy of ``a``."""
    return np.ascontiguousarray(a, dtype=np.float32)


def get_nodes_by_type(nodes: Iterable[Node], node_type):
    """Operators of ``node_type`` in order, descending into Sequential operators."""
    for node in nodes:
        if isinstance(node, node_type):
            yield node
        elif isinstance(node, Sequential):
            yield from get_nodes_by_type(node.nodes, node_type)
