"""ctypes front end of oracle/libbrute.so (test infrastructure only)."""
import ctypes
import os

import numpy as np
import torch

from . import build as _build

_lib = None


def lib():
    global _lib
    if _lib is None:
        path = _build.OUT
        if not os.path.exists(path):
            path = _build.build()
        _lib = ctypes.CDLL(path)
        _lib.brute_f16_to_f32.restype = ctypes.c_float
        _lib.brute_f16_to_f32.argtypes = [ctypes.c_uint16]
        _lib.brute_f32_to_f16.restype = ctypes.c_uint16
        _lib.brute_f32_to_f16.argtypes = [ctypes.c_float]
        _lib.brute_f32_to_bf16.restype = ctypes.c_uint16
        _lib.brute_f32_to_bf16.argtypes = [ctypes.c_float]
    return _lib


def _bits(t: torch.Tensor) -> np.ndarray:
    return t.contiguous().view(torch.int16).numpy().view(np.uint16).copy()


def _p(a: np.ndarray):
    return a.ctypes.data_as(ctypes.c_void_p)


def _i32(x) -> np.ndarray:
    return np.ascontiguousarray(np.asarray(x, dtype=np.int32))


def attention(qkv, k_cache, v_cache, qsl, lens, clens, tables, nH, nKV, d, bs, batch, maxblk):
    T = qkv.shape[0]
    out = np.zeros((T, nH * d), dtype=np.float64)
    a, b, c = _bits(qkv), _bits(k_cache), _bits(v_cache)
    q, l, cl, tb = _i32(qsl), _i32(lens), _i32(clens), _i32(tables)
    lib().brute_attention(_p(a), _p(b), _p(c), _p(out), _p(q), _p(l), _p(cl), _p(tb),
                          int(nH), int(nKV), int(d), int(bs), int(batch), int(maxblk),
                          int(qkv.dtype == torch.bfloat16))
    return torch.from_numpy(out)


def mla(qa, qr, kc, pc, qsl, lens, clens, tables, nH, R, C, bs, batch, maxblk, scale,
        topk=None, top_k=0):
    T = qa.shape[0]
    out = np.zeros((T, nH, C), dtype=np.float64)
    a, b, c, d = _bits(qa), _bits(qr), _bits(kc), _bits(pc)
    q, l, cl, tb = _i32(qsl), _i32(lens), _i32(clens), _i32(tables)
    tk = _i32(topk) if top_k else None
    f = lib().brute_mla
    f.argtypes = [ctypes.c_void_p] * 9 + [ctypes.c_int] * 6 + [ctypes.c_double, ctypes.c_void_p, ctypes.c_int]
    f(_p(a), _p(b), _p(c), _p(d), _p(out), _p(q), _p(l), _p(cl), _p(tb), int(nH), int(R), int(C),
      int(bs), int(batch), int(maxblk), float(scale), _p(tk) if top_k else None, int(top_k))
    return torch.from_numpy(out)


def rope_and_cache(inout, k_cache, v_cache, position, cosin, slots, nH, nKV, d, rot, bs):
    """Returns (inout, k_cache, v_cache) after the update, as tensors of the input dtype."""
    dt = inout.dtype
    a, b, c, cs = _bits(inout), _bits(k_cache), _bits(v_cache), _bits(cosin)
    pos = np.ascontiguousarray(position.numpy().astype(np.int64))
    sl = _i32(slots)
    lib().brute_rope_and_cache(_p(a), _p(b), _p(c), _p(pos), _p(cs), _p(sl), int(inout.shape[0]),
                               int(nH), int(nKV), int(d), int(rot), int(bs),
                               int(dt == torch.bfloat16))

    def back(x, like):
        return torch.from_numpy(x.view(np.int16)).view(dt).view(like.shape)

    return back(a, inout), back(b, k_cache), back(c, v_cache)


def rope_complex(inp, freqs_f32, position, H, step, rope):
    dt = inp.dtype
    T = inp.shape[0]
    a = _bits(inp)
    f = np.ascontiguousarray(freqs_f32.numpy().astype(np.float32))
    pos = np.ascontiguousarray(position.numpy().astype(np.int64))
    out = np.zeros((T, H, rope), dtype=np.uint16)
    lib().brute_rope_complex(_p(a), _p(f), _p(pos), _p(out), int(T), int(H), int(step), int(rope),
                             int(dt == torch.bfloat16))
    return torch.from_numpy(out.view(np.int16)).view(dt)
