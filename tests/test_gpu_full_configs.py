"""The benchmark configurations 3, 4 and 5 at their full sizes on the GPU, through the operator API. The CPU
oracle checks a sample (sequences re-packed into a compact cache with their own block tables; prefill rows
each as the decode step they are equivalent to); every output row is checked through a size-independent
property: it is a convex combination of the value rows it can see, so each of its columns lies between the
column-wise extremes of those rows.
Tolerances: max abs <= 2e-2 and mean abs <= 2e-3 (int8 KV: 5e-2 max)."""
import numpy as np
import pytest
import torch

from gvirt_amd import workloads as W
from oracle import xlite_oracle as O

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
SLACK = 1e-2   # 16-bit rounding of the output


def check(got, ref, max_abs=2e-2, mean_abs=2e-3):
    err = (got - ref).abs()
    assert float(err.max()) <= max_abs, "max abs err %g" % float(err.max())
    assert float(err.mean()) <= mean_abs, "mean abs err %g" % float(err.mean())


def compact(tables, max_num_block, seqs, *caches):
    """The blocks of the sequences `seqs` gathered into small CPU caches, with the block table that addresses
    them: what the oracle needs of a cache that is too large to copy whole."""
    rows = tables.view(-1, max_num_block)[seqs].long()                 # [n, MB] physical blocks
    flat = rows.flatten()
    small = [None if c is None else c[flat].cpu() for c in caches]
    new_tables = torch.arange(flat.numel(), dtype=torch.int32)
    return new_tables, small


def test_config3_qwen25_7b_chunked_prefill_full(rt):
    """All 8 seeded sequences (1024..8192 tokens), every 2048-token chunk call, as bench.py issues them."""
    from gvirt_amd._C import attention
    s = W.QWEN25_7B
    lens = W.c3_total_lengths()
    g = s.n_heads // s.n_kv_heads
    caches, ci, calls = None, 0, 0
    rng = np.random.default_rng(3)
    while True:
        w = W.gqa_prefill_chunk(s, lens, ci, 2048, W.SEED_BASE + 3, device=DEV, caches=caches)
        if w is None:
            break
        caches = w["caches"]
        attention(rt, w["qkv"], w["k_cache"], w["v_cache"], w["output"], w["query_start_loc"], w["lens"], w["cached_lens"],
                  w["block_tables"], s.n_heads, s.n_kv_heads, s.head_dim, s.block_size, w["batch"], w["max_num_block"])
        rt.synchronize()
        mb = w["max_num_block"]
        qsl, ql = w["query_start_loc"].tolist(), w["lens"].tolist()
        cached = 2048 * ci
        out = w["output"].float()
        tables = w["block_tables"].view(w["batch"], mb)
        for j in range(w["batch"]):
            # property on every row of the sequence
            v = w["v_cache"][tables[j].long()].reshape(-1, s.n_kv_heads, s.head_dim)[: cached + ql[j]].float()
            hi = v.cummax(0).values[cached:].unsqueeze(2)
            lo = v.cummin(0).values[cached:].unsqueeze(2)
            o = out[qsl[j]: qsl[j] + ql[j]].view(ql[j], s.n_kv_heads, g, s.head_dim)
            assert bool((o <= hi + SLACK).all()) and bool((o >= lo - SLACK).all()), (ci, j)
            # the oracle on sampled rows, each as its equivalent decode step over the sequence's own blocks
            t1, (kc, vc) = compact(w["block_tables"], mb, [j], w["k_cache"], w["v_cache"])
            for r in sorted({0, ql[j] - 1, int(rng.integers(0, ql[j]))}):
                row = w["qkv"][qsl[j] + r: qsl[j] + r + 1].cpu()
                ref = O.attention_ref(row, kc, vc, torch.tensor([0]), torch.tensor([1]), torch.tensor([cached + r]), t1,
                                      s.n_heads, s.n_kv_heads, s.head_dim, s.block_size, 1, mb)
                check(out[qsl[j] + r: qsl[j] + r + 1].cpu(), ref)
        calls += 1
        ci += 1
    assert calls == 4 and max(lens) > 6144


def test_config4_deepseek_r1_decode_full_batch(rt):
    """The batch of 32 sequences the benchmark times (contexts 4096..8192, 128 heads, block size 64)."""
    from gvirt_amd._C import mla_attention
    s = W.MlaShape()
    ctx = W.c4_context_lengths()
    w = W.mla_decode(s, ctx, W.SEED_BASE + 4, device=DEV)
    mla_attention(rt, w["q_absorb"], w["qr"], w["k_cache"], w["pe_cache"], w["o_absorb"], w["query_start_loc"], w["lens"],
                  w["cached_lens"], w["block_tables"], s.n_heads, s.rope_head_dim, s.kv_lora_rank, s.block_size, w["batch"],
                  w["max_num_blocks"], s.scale)
    rt.synchronize()
    mb = w["max_num_blocks"]
    out = w["o_absorb"].float()
    tables = w["block_tables"].view(32, mb)
    for i in range(32):
        lat = w["k_cache"][tables[i].long()].reshape(-1, s.kv_lora_rank)[: ctx[i]].float()
        assert bool((out[i] <= lat.max(0).values + SLACK).all()) and bool((out[i] >= lat.min(0).values - SLACK).all()), i
    sample = sorted({0, 13, 31, int(np.argmax(ctx)), int(np.argmin(ctx))})
    t1, (kc, pc) = compact(w["block_tables"], mb, sample, w["k_cache"], w["pe_cache"])
    n = len(sample)
    ref = O.mla_attention_ref(w["q_absorb"][sample].cpu(), w["qr"][sample].cpu(), kc, pc, torch.arange(n, dtype=torch.int32),
                              torch.ones(n, dtype=torch.int32), w["cached_lens"][sample].cpu(), t1, s.n_heads,
                              s.rope_head_dim, s.kv_lora_rank, s.block_size, n, mb, s.scale)
    check(out[sample].cpu().reshape(ref.shape), ref)


def test_config5_int8_kv_decode_full_batch(rt):
    """The 128 sequences of configuration 5 (contexts log-uniform in 128..32768) over the int8 cache."""
    from gvirt_amd._C import attention
    s = W.LLAMA3_8B
    ctx = W.c5_context_lengths()
    assert len(ctx) == 128
    w = W.gqa_decode(s, ctx, W.SEED_BASE + 5, device=DEV, int8_kv=True)
    attention(rt, w["qkv"], w["k_cache"], w["v_cache"], w["output"], w["query_start_loc"], w["lens"], w["cached_lens"],
              w["block_tables"], s.n_heads, s.n_kv_heads, s.head_dim, s.block_size, w["batch"], w["max_num_block"],
              k_scale=w["k_scale"], v_scale=w["v_scale"])
    rt.synchronize()
    mb = w["max_num_block"]
    g = s.n_heads // s.n_kv_heads
    out = w["output"].float().view(128, s.n_kv_heads, g, s.head_dim)
    tables = w["block_tables"].view(128, mb)
    for i in range(128):
        blocks = tables[i, : (ctx[i] + s.block_size - 1) // s.block_size].long()
        v = w["v_cache"][blocks].reshape(-1, s.n_kv_heads, s.head_dim)[: ctx[i]].float()
        v = v * w["v_scale"][blocks].reshape(-1, s.n_kv_heads)[: ctx[i]].unsqueeze(-1)
        hi, lo = v.max(0).values.unsqueeze(1), v.min(0).values.unsqueeze(1)
        assert bool((out[i] <= hi + SLACK).all()) and bool((out[i] >= lo - SLACK).all()), i
    order = np.argsort(ctx)
    sample = sorted({int(order[-1]), int(order[0]), int(order[64]), int(order[100]), 5, 40, 77, 120})
    t1, (kc, vc, ks, vs) = compact(w["block_tables"], mb, sample, w["k_cache"], w["v_cache"], w["k_scale"], w["v_scale"])
    n = len(sample)
    ref = O.attention_ref(w["qkv"][sample].cpu(), kc, vc, torch.arange(n, dtype=torch.int32), torch.ones(n, dtype=torch.int32),
                          w["cached_lens"][sample].cpu(), t1, s.n_heads, s.n_kv_heads, s.head_dim, s.block_size, n, mb, ks, vs)
    check(w["output"].float()[sample].cpu(), ref, max_abs=5e-2)
