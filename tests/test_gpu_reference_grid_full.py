"""The entries of the reference's workload grids that the CPU oracle cannot take whole, at their full size
(xlite/tests/kernels/attention.py:46-48, xlite/tests/kernels/mla.py:66-69): the operator runs the whole batch,
the oracle takes sampled rows, each as the decode step it is equivalent to (row r of a sequence with c cached
positions sees the c + r positions before it and its own), and every row is checked through the convexity
property (each output column lies between the column-wise extremes of the value rows the row can see).
Tolerances: max abs <= 2e-2 and mean abs <= 2e-3."""
import numpy as np
import pytest
import torch

from oracle import xlite_oracle as O
from test_gpu_attention import check, generic_case, run_attention
from test_gpu_mla import mla_case, run_mla

pytestmark = pytest.mark.gpu
SLACK = 1e-2   # 16-bit rounding of the output


def _sample_rows(lens, per_seq, seed):
    """(sequence, row) pairs: first and last row of every sequence, rows at block ends, random ones."""
    rng = np.random.default_rng(seed)
    picks = []
    for i, n in enumerate(lens):
        if n == 0:
            continue
        rows = {0, n - 1, min(n - 1, 127), min(n - 1, 128)} | {int(x) for x in rng.integers(0, n, size=per_seq)}
        picks += [(i, r) for r in sorted(rows)]
    return picks


def _gqa_rows_as_decode_steps(w, got, picks):
    """The sampled rows of a prefill batch as one decode batch over the same cache (the prefill wrote nothing: the
    operator reads keys from the cache only, which holds every position already)."""
    s = w["shape"]
    mb = w["max_num_block"]
    qsl, clens = w["query_start_loc"].tolist(), w["cached_lens"].tolist()
    tables = w["block_tables"].view(w["batch"], mb)
    n = len(picks)
    one = dict(w)
    one["qkv"] = torch.stack([w["qkv"][qsl[i] + r] for i, r in picks]).contiguous()
    one["batch"] = n
    one["lens"] = torch.ones(n, dtype=torch.int32)
    one["cached_lens"] = torch.tensor([clens[i] + r for i, r in picks], dtype=torch.int32)
    one["query_start_loc"] = torch.arange(n, dtype=torch.int32)
    one["block_tables"] = torch.stack([tables[i] for i, _ in picks]).flatten().contiguous()
    one["output"] = torch.zeros(n, s.n_heads * s.head_dim, dtype=w["qkv"].dtype)
    ref = O.attention_ref(one["qkv"], w["k_cache"], w["v_cache"], one["query_start_loc"], one["lens"], one["cached_lens"],
                          one["block_tables"], s.n_heads, s.n_kv_heads, s.head_dim, s.block_size, n, mb)
    check(torch.stack([got[qsl[i] + r] for i, r in picks]), ref)


def _gqa_convexity(w, got):
    s = w["shape"]
    g = s.n_heads // s.n_kv_heads
    mb = w["max_num_block"]
    qsl, lens, clens = w["query_start_loc"].tolist(), w["lens"].tolist(), w["cached_lens"].tolist()
    tables = w["block_tables"].view(w["batch"], mb)
    for j in range(w["batch"]):
        if lens[j] == 0:
            continue
        v = w["v_cache"][tables[j].long()].reshape(-1, s.n_kv_heads, s.head_dim)[: clens[j] + lens[j]].float()
        hi = v.cummax(0).values[clens[j]:].unsqueeze(2)
        lo = v.cummin(0).values[clens[j]:].unsqueeze(2)
        o = got[qsl[j]: qsl[j] + lens[j]].view(lens[j], s.n_kv_heads, g, s.head_dim)
        assert bool((o <= hi + SLACK).all()) and bool((o >= lo - SLACK).all()), j


@pytest.mark.parametrize("model", [(14, 2, 64, torch.bfloat16), (32, 8, 128, torch.bfloat16), (8, 1, 128, torch.bfloat16),
                                   (20, 20, 128, torch.float16)])
@pytest.mark.parametrize("work", [([0], [24322]), ([0] * 8, [789, 65, 13, 6545, 24, 190, 2432, 124]), ([128], [1800])])
def test_attention_reference_grid_large_prefills(rt, model, work):
    nH, nKV, d, dtype = model
    clens, lens = work
    w = generic_case(71, lens, clens, nH, nKV, d, 128, dtype, rms=True)
    got = run_attention(rt, w)
    _gqa_convexity(w, got)
    _gqa_rows_as_decode_steps(w, got, _sample_rows(lens, 2, 72))


def _mla_rows_as_decode_steps(c, got, picks, scale):
    qsl, clens = c["qsl"].tolist(), c["clens"].tolist()
    tables = c["tables"].view(c["batch"], c["maxblk"])
    n = len(picks)
    qa = torch.stack([c["qa"][qsl[i] + r] for i, r in picks])
    qr = torch.stack([c["qr"][qsl[i] + r] for i, r in picks])
    tb = torch.stack([tables[i] for i, _ in picks]).flatten().contiguous()
    ref = O.mla_attention_ref(qa, qr, c["kc"], c["pc"], torch.arange(n, dtype=torch.int32), torch.ones(n, dtype=torch.int32),
                              torch.tensor([clens[i] + r for i, r in picks], dtype=torch.int32), tb, c["nH"], c["R"], c["C"],
                              c["bs"], n, c["maxblk"], scale)
    g = torch.stack([got[qsl[i] + r] for i, r in picks])
    err = (g.reshape(ref.shape) - ref).abs()
    assert float(err.max()) <= 2e-2 and float(err.mean()) <= 2e-3, (float(err.max()), float(err.mean()))


def _mla_convexity(c, got):
    qsl, lens, clens = c["qsl"].tolist(), c["lens"].tolist(), c["clens"].tolist()
    tables = c["tables"].view(c["batch"], c["maxblk"])
    for j in range(c["batch"]):
        if lens[j] == 0:
            continue
        lat = c["kc"][tables[j].long()].reshape(-1, c["C"])[: clens[j] + lens[j]].float()
        hi = lat.cummax(0).values[clens[j]:].unsqueeze(1)
        lo = lat.cummin(0).values[clens[j]:].unsqueeze(1)
        o = got[qsl[j]: qsl[j] + lens[j]]
        assert bool((o <= hi + SLACK).all()) and bool((o >= lo - SLACK).all()), j


@pytest.mark.parametrize("nH", [16, 128])
@pytest.mark.parametrize("work", [([0], [1600]), ([0], [2528]), ([0] * 8, [789, 65, 13, 6545, 24, 190, 2432, 124]),
                                  ([0] * 4, [189, 65, 13, 545]), ([128], [128]), ([0], [256])])
def test_mla_reference_grid_large_prefills(rt, nH, work):
    """Also the 128-head cases of the bounded grid that the whole-batch oracle would spend minutes on."""
    clens, lens = work
    c = mla_case(73, lens, clens, nH)
    scale = 192 ** -0.5
    got = run_mla(rt, c, scale)
    _mla_convexity(c, got)
    _mla_rows_as_decode_steps(c, got, _sample_rows(lens, 1 if nH == 128 else 2, 74), scale)


def test_mla_topk_mask_128_heads_at_2048_entries(rt):
    """The top-k mask at the full head count and list length (bounded to 16 heads in the grid test): the oracle takes
    the listed rows themselves, which are decode rows already."""
    from gvirt_amd._C import mla_attention
    from test_gpu_mla import _topk_indices, DEV
    c = mla_case(75, [1, 1, 1], [2500, 2047, 2048], 128, bs=64)
    scale = 192 ** -0.5
    topk = _topk_indices(c, 2048, 76)
    out = torch.zeros(c["T"], c["nH"], c["C"], dtype=torch.bfloat16, device=DEV)
    mla_attention(rt, c["qa"].to(DEV), c["qr"].to(DEV), c["kc"].to(DEV), c["pc"].to(DEV), out, c["qsl"].to(DEV),
                  c["lens"].to(DEV), c["clens"].to(DEV), c["tables"].to(DEV), c["nH"], c["R"], c["C"], c["bs"], c["batch"],
                  c["maxblk"], scale, topk.to(DEV), 2048)
    rt.synchronize()
    ref = O.mla_attention_ref(c["qa"], c["qr"], c["kc"], c["pc"], c["qsl"], c["lens"], c["clens"], c["tables"], c["nH"],
                              c["R"], c["C"], c["bs"], c["batch"], c["maxblk"], scale, topk, 2048)
    err = (out.float().cpu() - ref).abs()
    assert float(err.max()) <= 2e-2 and float(err.mean()) <= 2e-3
