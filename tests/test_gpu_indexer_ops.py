"""GPU parity of the operators around the DSA indexer (layernorm, muls, the general rope_complex_and_cache)
and of the MLA layer with its indexer branch, against the oracle."""
import pytest
import torch

from oracle import xlite_oracle as O

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _freqs(rope, max_pos):
    ang = torch.outer(torch.arange(max_pos).float(), 1.0 / (10000.0 ** (torch.arange(0, rope, 2).float() / rope)))
    return torch.polar(torch.ones_like(ang), ang)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_layernorm_and_muls(rt, dtype):
    from gvirt_amd._C import layernorm, muls
    g = torch.Generator().manual_seed(5)
    x = torch.randn(70, 192, generator=g).to(dtype)
    w, b = torch.randn(128, generator=g).to(dtype), torch.randn(128, generator=g).to(dtype)
    # the reference's test shape (xlite/tests/kernels/layernorm.py:25-46: 64 x 128, whole rows) and a row longer
    # than the normalised width, in place
    for rows, cols, dim in ((64, 128, 128), (70, 192, 128), (3, 40, 24)):
        xin = x[:rows, :cols].contiguous()
        out = xin.clone().to(DEV)
        layernorm(rt, out, w.to(DEV), b.to(DEV), out, 1e-6, dim)
        rt.synchronize()
        want = O.layernorm_ref(xin, w, b, 1e-6, dim)
        # two fp32 reductions in another order: at most one unit of the 16-bit result
        torch.testing.assert_close(out[:, :dim].float().cpu(), want.float(), rtol=2 ** -7 if dtype == torch.bfloat16 else 2 ** -10, atol=1e-3)
        assert torch.equal(out[:, dim:].cpu(), xin[:, dim:])
    # muls: the reference's test (xlite/tests/kernels/muls.py:19-23) and the column-range form, exact
    xm = torch.randn(8, 2048, generator=g).to(dtype)
    y = torch.zeros_like(xm).to(DEV)
    muls(rt, xm.to(DEV), 2.5, y)
    rt.synchronize()
    assert torch.equal(y.cpu(), O.muls_ref(xm, 2.5))
    z = xm.clone().to(DEV)
    muls(rt, z, 0.0883883, z, 128, 64)
    rt.synchronize()
    assert torch.equal(z.cpu(), O.muls_ref(xm, 0.0883883, 128, 64))
    with pytest.raises(RuntimeError):
        muls(rt, z, 2.0, z, 2048, 4)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_rope_complex_and_cache_general_forms(rt, dtype):
    from gvirt_amd._C import rope_complex_and_cache
    g = torch.Generator().manual_seed(6)
    T, H, step, rope = 37, 5, 128, 64
    freqs = _freqs(rope, 300)
    pos = torch.randint(0, 300, (T,), generator=g)
    inp = torch.randn(T, H * step, generator=g).to(dtype)
    # to another tensor at column offsets, bit-exact
    out = torch.full((T, H * 80), 7.0, dtype=dtype, device=DEV)
    rope_complex_and_cache(rt, H, step, rope, 32, 0, inp.to(DEV), freqs.to(DEV), pos.to(DEV), output=out, out_step_dim=80, out_offset=16)
    rt.synchronize()
    want = O.rope_complex_and_cache_ref(H, step, rope, 32, 0, inp, freqs, pos)
    got = out.cpu().view(T, H, 80)
    assert torch.equal(got[..., 16:16 + rope], want) and bool((got[..., :16] == 7.0).all()) and bool((got[..., 16 + rope:] == 7.0).all())
    # in place on the first columns of every head (the indexer's query, xlite/csrc/model.cpp:311-313)
    q = inp.clone().to(DEV)
    rope_complex_and_cache(rt, H, step, rope, 0, 0, q, freqs.to(DEV), pos.to(DEV), output=q, out_step_dim=step, out_offset=0)
    rt.synchronize()
    qc = q.cpu().view(T, H, step)
    assert torch.equal(qc[..., :rope], O.rope_complex_and_cache_ref(H, step, rope, 0, 0, inp, freqs, pos))
    assert torch.equal(qc[..., rope:], inp.view(T, H, step)[..., rope:])
    # into a paged cache: one head, vdim columns (rotated, then unchanged), nothing else written
    bs, vdim, row = 16, 128, 128 + 16
    one = torch.randn(T, row, generator=g).to(dtype)
    slots = torch.randperm(4 * bs, generator=g)[:T].int()
    cache = torch.full((4, bs, vdim), 3.0, dtype=dtype)
    cache_gpu = cache.clone().to(DEV)
    src = one.clone().to(DEV)
    rope_complex_and_cache(rt, 1, row, rope, 0, vdim, src, freqs.to(DEV), pos.to(DEV), block_size=bs, cache=cache_gpu,
                           slot_mapping=slots.to(DEV))
    rt.synchronize()
    O.rope_complex_and_cache_ref(1, row, rope, 0, vdim, one, freqs, pos, bs, cache, slots)
    assert torch.equal(cache_gpu.cpu(), cache) and torch.equal(src.cpu(), one)


@pytest.mark.parametrize("index_n_heads,topk", [(16, 64), (64, 128)])
def test_mla_layer_with_indexer_branch(rt, index_n_heads, topk):
    """Prefill, then decode steps; the contexts pass index_topk, so the later steps attend to the indexer's
    position lists only. The lists are compared with the oracle's up to the few positions whose 16-bit scores
    tie or round across the selection threshold, the layer output with the oracle's layer on the same lists."""
    from gvirt_amd.mha import prepare_attn
    from gvirt_amd.mla import IndexerWeights, MlaConfig, MlaLayer
    g = torch.Generator().manual_seed(93)
    dt = torch.bfloat16
    n_heads, block_size, D = 16, 64, 128
    cfg = MlaConfig(hidden=256, n_heads=n_heads, q_lora_rank=192, kv_lora_rank=512, nope_head_dim=128, rope_head_dim=64,
                    v_head_dim=128, block_size=block_size, softmax_scale=192 ** -0.5)
    r = lambda *s: torch.randn(*s, generator=g)
    wa = (r(cfg.hidden, cfg.q_lora_rank + cfg.kv_lora_rank + cfg.rope_head_dim) * cfg.hidden ** -0.5).to(dt)
    wqb = (r(cfg.q_lora_rank, n_heads * (cfg.nope_head_dim + cfg.rope_head_dim)) * cfg.q_lora_rank ** -0.5).to(dt)
    wuk_t = (r(n_heads, cfg.nope_head_dim, cfg.kv_lora_rank) * cfg.nope_head_dim ** -0.5).to(dt)
    wuv = (r(n_heads, cfg.kv_lora_rank, cfg.v_head_dim) * cfg.kv_lora_rank ** -0.5).to(dt)
    wo = (r(n_heads * cfg.v_head_dim, cfg.hidden) * (n_heads * cfg.v_head_dim) ** -0.5).to(dt)
    qn, kn = (1 + 0.1 * r(cfg.q_lora_rank)).to(dt), (1 + 0.1 * r(cfg.kv_lora_rank)).to(dt)
    ix = dict(wk_weights_proj=(r(cfg.hidden, D + index_n_heads) * cfg.hidden ** -0.5).to(dt), k_norm=(1 + 0.1 * r(D)).to(dt),
              k_norm_bias=(0.1 * r(D)).to(dt), wq_b=(r(cfg.q_lora_rank, index_n_heads * D) * cfg.q_lora_rank ** -0.5).to(dt),
              index_n_heads=index_n_heads, index_head_dim=D, index_topk=topk)
    freqs = _freqs(cfg.rope_head_dim, 1024)
    prompts, steps = [300, 40, 170], 2
    blocks_per_seq = (max(prompts) + steps + block_size - 1) // block_size
    NB = len(prompts) * blocks_per_seq + 2
    perm = torch.randperm(NB, generator=g).tolist()
    tables = [perm[i * blocks_per_seq:(i + 1) * blocks_per_seq] for i in range(len(prompts))]
    kc_ref, pc_ref, ic_ref = (torch.zeros(NB, block_size, n).to(dt) for n in (cfg.kv_lora_rank, cfg.rope_head_dim, D))
    kc, pc, ic = kc_ref.to(DEV), pc_ref.to(DEV), ic_ref.to(DEV)
    mv = lambda t: t.to(DEV)
    weights = IndexerWeights(mv(ix["wk_weights_proj"]), mv(ix["k_norm"]), mv(ix["k_norm_bias"]), mv(ix["wq_b"]), index_n_heads, D, topk)
    layer = MlaLayer(cfg, mv(wa), mv(qn), mv(kn), mv(wqb), mv(wuk_t), mv(wuv), mv(wo), indexer=weights)
    with pytest.raises(RuntimeError):
        layer.forward(rt, torch.zeros(1, cfg.hidden, dtype=dt, device=DEV), kc, pc, prepare_attn([1], [0], [tables[0]], block_size, DEV), mv(freqs))
    cached = [0] * len(prompts)
    for step in range(steps + 1):
        lens = prompts if step == 0 else [1] * len(prompts)
        hidden = r(sum(lens), cfg.hidden).to(dt)
        meta = prepare_attn(lens, cached, tables, block_size, DEV)
        got = layer.forward(rt, mv(hidden), kc, pc, meta, mv(freqs), index_k_cache=ic)
        rt.synchronize()
        lists = layer.last_topk_indices
        ref, own = O.mla_forward_ref(hidden, wa, qn, kn, wqb, wuk_t, wuv, wo, kc_ref, pc_ref, lens, cached, tables, freqs, n_heads,
                                     cfg.q_lora_rank, cfg.kv_lora_rank, cfg.nope_head_dim, cfg.rope_head_dim, cfg.v_head_dim,
                                     block_size, cfg.softmax_scale, cfg.norm_eps, indexer=ix, index_k_cache=ic_ref,
                                     topk_override=None if lists is None else lists.cpu())
        torch.testing.assert_close(ic.float().cpu(), ic_ref.float(), rtol=2 ** -6, atol=3e-2)
        assert (lists is None) == (own is None)
        if lists is not None:
            # the lists: at most 3 % of a row's set (plus one position, for the short lists of this test) may
            # differ from the oracle's (16-bit scores that tie or round across the threshold; the measure of
            # xlite/tests/kernels/indexer_topk.py:52-56), ascending, in range
            off = 0
            for i, n in enumerate(lens):
                for rr in range(n):
                    k = min(topk, cached[i] + n)
                    mine, theirs = lists[off + rr, :k].tolist(), own[off + rr, :k].tolist()
                    assert mine == sorted(set(mine)) and 0 <= mine[0] and mine[-1] < cached[i] + n
                    assert len(set(theirs) - set(mine)) * 100.0 <= 3.0 * k + 100.0
                off += n
        # the layer output, on the lists the GPU selected
        err = (got.float().cpu() - ref.float()).abs()
        assert float(err.max()) <= 3e-2 and float(err.mean()) <= 3e-3, "step %d: max %g mean %g" % (step, float(err.max()), float(err.mean()))
        cached = [c + l for c, l in zip(cached, lens)]
