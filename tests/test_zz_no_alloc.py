"""The allocation-free attention entry point against the entry point with a caller-provided workspace,
both through the C ABI: same bits, on two calls in a row of which the second is smaller (the built-in
buffer still holds the first call's partial results)."""
import ctypes

import pytest
import torch

from gvirt_amd import _lib
from test_gpu_attention import generic_case

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _p(t):
    return None if t is None else ctypes.c_void_p(t.data_ptr())


_set_up = [False]


def _call_both(lib, w, check=True):
    if not _set_up[0]:
        # the entry point's first call on a device is its set-up (it takes the address of the library's buffer, and
        # the runtime then maps the buffer): the driver-level check below is for the calls after it
        _set_up[0] = True
        _call_both(lib, generic_case(40, [1] * 8, [700 + 11 * i for i in range(8)], 32, 8, 128, 128, torch.bfloat16, rms=True), check=False)
    s = w["shape"]
    d = {k: (v.to(DEV) if isinstance(v, torch.Tensor) else v) for k, v in w.items()}
    T = d["qkv"].shape[0]
    dt = 1 if d["qkv"].dtype == torch.bfloat16 else 0
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    common = [_p(d["qkv"]), _p(d["k_cache"]), _p(d["v_cache"])]
    meta = [_p(d["query_start_loc"]), _p(d["lens"]), _p(d["cached_lens"]), _p(d["block_tables"]), T, s.n_heads,
            s.n_kv_heads, s.head_dim, s.block_size, w["batch"], w["max_num_block"], dt, 0, None, None]
    need = lib.xlite_hip_attention_workspace_bytes(T, s.n_heads, s.n_kv_heads, s.head_dim, s.block_size, w["batch"],
                                                   w["max_num_block"])
    ws = torch.empty(max(need, 256), dtype=torch.uint8, device=DEV)
    out_ws = torch.full_like(d["output"], 7.0)
    out_na = torch.full_like(d["output"], -7.0)
    _lib.check(lib.xlite_hip_attention(stream, *common, _p(out_ws), *meta, _p(ws), ws.numel()))
    torch.cuda.synchronize()
    before = (torch.cuda.memory_allocated(), torch.cuda.mem_get_info()[0])   # torch's allocator, and the driver's free bytes
    rc = lib.xlite_hip_attention_noalloc(stream, *common, _p(out_na), *meta)
    torch.cuda.synchronize()
    if check:
        assert (torch.cuda.memory_allocated(), torch.cuda.mem_get_info()[0]) == before
    return rc, need, out_ws, out_na


def test_noalloc_matches_workspace_entry_on_two_calls_in_a_row():
    lib = _lib.load()
    assert lib.xlite_hip_attention_noalloc_scratch_bytes() == 32 << 20
    # a decode batch whose rows are split across workgroups, then a smaller one, then a split prefill, then a
    # smaller decode batch again
    cases = [generic_case(41, [1] * 24, [3000 + 37 * i for i in range(24)], 32, 8, 128, 128, torch.bfloat16, rms=True),
             generic_case(42, [1] * 3, [900, 70, 411], 32, 8, 128, 128, torch.bfloat16, rms=True),
             generic_case(43, [100, 1], [6000, 2000], 28, 4, 128, 128, torch.bfloat16, rms=True),
             generic_case(44, [1] * 2, [129, 16], 14, 2, 64, 128, torch.float16, rms=True)]
    for w in cases:
        rc, need, out_ws, out_na = _call_both(lib, w)
        assert rc == 0, lib.xlite_hip_last_error()
        assert need > 0
        assert torch.equal(out_ws.view(torch.int16), out_na.view(torch.int16))
        assert bool(torch.isfinite(out_na.float()).all())


def test_noalloc_refuses_shapes_beyond_its_buffer():
    lib = _lib.load()
    w = generic_case(45, [1] * 2, [300, 40], 128, 8, 128, 128, torch.bfloat16, rms=True)
    rc, need, _, out_na = _call_both(lib, w)
    assert need > 32 << 20
    assert rc == -3
    assert b"built-in buffer" in lib.xlite_hip_last_error()
    assert bool((out_na == -7.0).all())   # nothing ran


def test_noalloc_captured_into_a_graph_replays_the_workspace_entry_bits():
    """The entry point is meant for code under graph capture: after one eager call on the device (which takes the
    buffer's address), a captured call replays on changed inputs with the bits of the workspace entry point."""
    lib = _lib.load()
    w = generic_case(46, [1] * 16, [2500 + 91 * i for i in range(16)], 32, 8, 128, 128, torch.bfloat16, rms=True)
    s = w["shape"]
    d = {k: (v.to(DEV) if isinstance(v, torch.Tensor) else v) for k, v in w.items()}
    T = d["qkv"].shape[0]
    common = [_p(d["qkv"]), _p(d["k_cache"]), _p(d["v_cache"])]
    meta = [_p(d["query_start_loc"]), _p(d["lens"]), _p(d["cached_lens"]), _p(d["block_tables"]), T, s.n_heads,
            s.n_kv_heads, s.head_dim, s.block_size, w["batch"], w["max_num_block"], 1, 0, None, None]
    need = lib.xlite_hip_attention_workspace_bytes(T, s.n_heads, s.n_kv_heads, s.head_dim, s.block_size, w["batch"],
                                                   w["max_num_block"])
    ws = torch.empty(max(need, 256), dtype=torch.uint8, device=DEV)
    out_ws, out_na = torch.zeros_like(d["output"]), torch.zeros_like(d["output"])
    cur = lambda: ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    assert lib.xlite_hip_attention_noalloc(cur(), *common, _p(out_na), *meta) == 0   # warm-up, eager
    torch.cuda.synchronize()
    graph, side = torch.cuda.CUDAGraph(), torch.cuda.Stream()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            assert lib.xlite_hip_attention_noalloc(cur(), *common, _p(out_na), *meta) == 0
    torch.cuda.synchronize()
    g = torch.Generator(device=DEV).manual_seed(5)
    for _ in range(3):
        d["qkv"].copy_(torch.randn(d["qkv"].shape, generator=g, device=DEV).to(d["qkv"].dtype) * 0.3)
        out_na.fill_(3.0)
        torch.cuda.synchronize()
        graph.replay()
        _lib.check(lib.xlite_hip_attention(cur(), *common, _p(out_ws), *meta, _p(ws), ws.numel()))
        torch.cuda.synchronize()
        assert torch.equal(out_ws.view(torch.int16), out_na.view(torch.int16))
