"""CPU-side checks of the C-ABI library: it loads, exports every declared symbol, and its
host-only entry points agree with the oracle. No GPU compute here."""
import ctypes
import os
import random
import re

import numpy as np
import pytest
import torch

from gvirt_amd import _lib
from gvirt_amd import _C
from oracle import xlite_oracle as O

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    text = open(os.path.join(ROOT, "include", "xlite_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(xlite_hip_\w+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = _lib.load()
    names = _declared()
    assert len(names) >= 15
    for n in names:
        assert hasattr(lib, n), n
        assert n in _lib.SIGNATURES, "no ctypes signature for " + n
    assert sorted(_lib.SIGNATURES) == names
    assert lib.xlite_hip_version() == 1


def test_tile_tuner_matches_oracle_on_random_workloads():
    rnd = random.Random(7)
    for case in range(200):
        batch = rnd.choice([1, 1, 2, 3, 8, 17])
        decode = rnd.random() < 0.8
        clens = [rnd.randint(0, 140000) for _ in range(batch)]
        qlens = [1] * batch if decode else [rnd.randint(1, 3000) for _ in range(batch)]
        if decode and rnd.random() < 0.2:
            clens[0] = 0  # a padding sequence (kv length 1) is ignored by the scores
        g = rnd.choice([1, 4, 5, 7, 8, 16, 128])
        nkv = rnd.choice([1, 2, 4, 8])
        bs = rnd.choice([64, 128])
        cores = rnd.choice([20, 24, 256])
        want = O.get_tile_size_of_cached_kv_ref(clens, qlens, g, nkv, bs, cores)
        got = _C.get_tile_size_of_cached_kv(clens, qlens, g, nkv, bs, cores)
        assert got == want, (case, clens, qlens, g, nkv, bs, cores)


def test_prepare_attn_matches_oracle_and_rejects_short_tables():
    lib = _lib.load()
    rnd = random.Random(3)
    for _ in range(20):
        batch = rnd.randint(1, 6)
        bs = rnd.choice([4, 16, 128])
        lens = [rnd.randint(1, 40) for _ in range(batch)]
        clens = [rnd.randint(0, 300) for _ in range(batch)]
        rows = [[rnd.randint(0, 999) for _ in range((l + c + bs - 1) // bs + rnd.randint(0, 2))]
                for l, c in zip(lens, clens)]
        want = O.prepare_attn_ref(lens, clens, rows, bs)
        u32 = ctypes.c_uint32 * batch
        row_arrays = [(ctypes.c_int32 * len(r))(*r) for r in rows]
        ptrs = (ctypes.c_void_p * batch)(*[ctypes.addressof(a) for a in row_arrays])
        T = sum(lens)
        qsl = (ctypes.c_int32 * batch)()
        pos = (ctypes.c_int64 * T)()
        slots = (ctypes.c_int32 * T)()
        cap = batch * want["max_num_blocks"]
        dense = (ctypes.c_int32 * cap)()
        mnb, bt, dec = ctypes.c_uint32(), ctypes.c_uint32(), ctypes.c_int()
        rc = lib.xlite_hip_prepare_attn(u32(*lens), u32(*clens), batch, ptrs, u32(*[len(r) for r in rows]), bs,
                                        qsl, pos, slots, dense, cap, ctypes.byref(mnb), ctypes.byref(bt),
                                        ctypes.byref(dec))
        assert rc == 0, lib.xlite_hip_last_error()
        assert list(qsl) == want["query_start_loc"]
        assert list(pos) == want["position"]
        assert list(slots) == want["slot_mapping"]
        assert mnb.value == want["max_num_blocks"] and bt.value == want["batched_tokens"]
        assert bool(dec.value) == want["is_decode"]
        assert np.array(dense).reshape(batch, -1).tolist() == want["block_tables"].tolist()
    # a block table shorter than the sequence needs is an error, as in the reference
    u1 = ctypes.c_uint32 * 1
    short = (ctypes.c_int32 * 1)(5)
    ptrs = (ctypes.c_void_p * 1)(ctypes.addressof(short))
    buf = (ctypes.c_int32 * 64)()
    p64 = (ctypes.c_int64 * 64)()
    rc = lib.xlite_hip_prepare_attn(u1(9), u1(0), 1, ptrs, u1(1), 4, buf, p64, buf, buf, 64, None, None, None)
    assert rc < 0 and b"block table too small" in lib.xlite_hip_last_error()
    with pytest.raises(RuntimeError):
        _lib.check(rc)


def test_operators_refuse_cpu_tensors_and_bad_arguments():
    class FakeRt:
        pass
    x = torch.zeros(2, 4 * 64, dtype=torch.bfloat16)
    i32 = torch.zeros(2, dtype=torch.int32)
    with pytest.raises(RuntimeError, match="GPU tensor"):
        _C.attention(FakeRt(), x, x, x, x, i32, i32, i32, i32, 2, 1, 64, 128, 2, 1)
    with pytest.raises(RuntimeError, match="gptj"):
        _C.rope_and_cache(FakeRt(), x, x, x, i32.long(), x, i32, 2, 1, 64, 64, 128, False)
    with pytest.raises(RuntimeError, match="kvHeads"):
        _C.gather_sparse_kv_cache(FakeRt(), x, x, i32, i32, i32, i32, x, x, 1, 2, 128, 1, 512, 64, 2)
    with pytest.raises(RuntimeError, match="NZ"):
        _C.einsum_mht_htd_mhd(FakeRt(), x, x, x, 1, 1, 16, 32, True)
    with pytest.raises(RuntimeError, match="single GPU"):
        _C.Runtime(0, 0, tp_size=2)


def test_prepare_attn_accepts_the_reference_metadata_objects():
    """`ModelAttnMeta` (positions derived) and the vLLM form `AttnMeta` (host block tables, caller's positions:
    xlite/csrc/_C.cpp:666-677, xlite/csrc/runtime.cpp:535-548) through the host-side builder, on CPU tensors."""
    import torch
    from gvirt_amd import _C
    from gvirt_amd.mha import prepare_attn_meta
    lens, clens, rows, bs = [3, 1, 5], [5, 9, 0], [[7, 2], [4, 9, 1], [3, 8]], 4
    want = O.prepare_attn_ref(lens, clens, rows, bs)
    m0 = _C.ModelAttnMeta()
    m0.lens, m0.cached_lens, m0.block_tables = lens, clens, rows
    a = prepare_attn_meta(m0, bs, "cpu")
    assert a.batch == 3 and a.batched_tokens == 9 and not a.is_decode and a.max_num_blocks == want["max_num_blocks"]
    assert a.position.tolist() == list(want["position"]) and a.slot_mapping.tolist() == list(want["slot_mapping"])
    assert a.query_start_loc.tolist() == list(want["query_start_loc"])
    assert a.block_tables.tolist() == want["block_tables"].flatten().tolist()
    m1 = _C.AttnMeta()
    m1.lens, m1.cached_lens, m1.block_tables_cpu = lens, clens, rows
    m1.positions = torch.arange(100, 109, dtype=torch.int64)
    b = prepare_attn_meta(m1, bs, "cpu")
    assert b.position.tolist() == list(range(100, 109)) and b.slot_mapping.tolist() == a.slot_mapping.tolist()
    m1.positions = None
    with pytest.raises(RuntimeError):
        prepare_attn_meta(m1, bs, "cpu")
    with pytest.raises(RuntimeError):
        prepare_attn_meta(object(), bs, "cpu")
