"""ctypes loader of oracle/libmoe_oracle.so (TEST INFRASTRUCTURE ONLY)."""
import ctypes
import os
import subprocess

import numpy as np

_DIR = os.path.dirname(os.path.abspath(__file__))
_PATH = os.path.join(_DIR, "libmoe_oracle.so")
_lib = None


def build() -> str:
    subprocess.run(["make", "-C", _DIR, "-B", "libmoe_oracle.so"], check=True, stdout=subprocess.DEVNULL)
    return _PATH


def load():
    global _lib
    if _lib is None:
        if not os.path.exists(_PATH):
            build()
        lib = ctypes.CDLL(_PATH)
        vp, i32, i64 = ctypes.c_void_p, ctypes.c_int, ctypes.c_int64
        lib.oracle_topk_softmax.restype = i32
        lib.oracle_topk_softmax.argtypes = [vp, i64, i32, i32, i32, vp, vp]
        lib.oracle_moe_align_block_size.restype = i32
        lib.oracle_moe_align_block_size.argtypes = [vp, i64, i32, i32, vp, i64, vp, i64, vp]
        _lib = lib
    return _lib


def topk_softmax(logits: np.ndarray, topk: int, renormalize: bool):
    x = np.ascontiguousarray(logits, dtype=np.float32)
    T, E = x.shape
    w = np.empty((T, topk), dtype=np.float32)
    ids = np.empty((T, topk), dtype=np.int32)
    rc = load().oracle_topk_softmax(x.ctypes.data, T, E, topk, int(renormalize), w.ctypes.data, ids.ctypes.data)
    assert rc == 0, rc
    return w, ids


def moe_align_block_size(topk_ids: np.ndarray, num_experts: int, block_size: int):
    flat = np.ascontiguousarray(np.asarray(topk_ids).reshape(-1), dtype=np.int32)
    max_padded = flat.size + num_experts * (block_size - 1)
    sorted_ids = np.empty(max_padded, dtype=np.int32)
    expert_ids = np.empty(-(-max_padded // block_size), dtype=np.int32)
    post = np.empty(1, dtype=np.int32)
    rc = load().oracle_moe_align_block_size(flat.ctypes.data, flat.size, num_experts, block_size,
                                            sorted_ids.ctypes.data, sorted_ids.size,
                                            expert_ids.ctypes.data, expert_ids.size, post.ctypes.data)
    assert rc == 0, rc
    return sorted_ids, expert_ids, post
