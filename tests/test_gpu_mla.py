"""GPU parity of the MLA operators (absorbed attention, mla_v2, mla_v3, einsum) against the oracle."""
import numpy as np
import pytest
import torch

from gvirt_amd import workloads as W
from oracle import xlite_oracle as O

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def check(got, ref, max_abs=2e-2, mean_abs=2e-3):
    err = (got - ref).abs()
    assert float(err.max()) <= max_abs, "max abs err %g" % float(err.max())
    assert float(err.mean()) <= mean_abs, "mean abs err %g" % float(err.mean())


def mla_case(seed, lens, clens, nH, bs=128, C=512, R=64):
    g = torch.Generator().manual_seed(seed)
    batch, T = len(lens), sum(lens)
    maxblk = max((l + c + bs - 1) // bs for l, c in zip(lens, clens))
    NB = batch * maxblk + 1
    rms = lambda x: x / x.pow(2).mean(-1, keepdim=True).add(1e-6).sqrt()
    return dict(batch=batch, T=T, nH=nH, bs=bs, C=C, R=R, maxblk=maxblk,
                qa=(rms(torch.randn(T, nH, C, generator=g)) * 4).bfloat16(), qr=rms(torch.randn(T, nH, R, generator=g)).bfloat16(),
                kc=rms(torch.randn(NB, bs, C, generator=g).clamp(0.2, 1)).bfloat16(), pc=rms(torch.randn(NB, bs, R, generator=g)).bfloat16(),
                qsl=torch.tensor(np.cumsum([0] + lens[:-1]), dtype=torch.int32), lens=torch.tensor(lens, dtype=torch.int32),
                clens=torch.tensor(clens, dtype=torch.int32), tables=torch.randperm(NB, generator=g)[: batch * maxblk].int())


def run_mla(rt, c, scale):
    from gvirt_amd._C import mla_attention
    out = torch.zeros(c["T"], c["nH"], c["C"], dtype=torch.bfloat16, device=DEV)
    mla_attention(rt, c["qa"].to(DEV), c["qr"].to(DEV), c["kc"].to(DEV), c["pc"].to(DEV), out, c["qsl"].to(DEV),
                  c["lens"].to(DEV), c["clens"].to(DEV), c["tables"].to(DEV), c["nH"], c["R"], c["C"], c["bs"], c["batch"],
                  c["maxblk"], scale)
    rt.synchronize()
    return out.float().cpu()


def oracle_mla(c, scale):
    return O.mla_attention_ref(c["qa"], c["qr"], c["kc"], c["pc"], c["qsl"], c["lens"], c["clens"], c["tables"], c["nH"],
                               c["R"], c["C"], c["bs"], c["batch"], c["maxblk"], scale)


# workloads of xlite/tests/kernels/mla.py:61-76 (bounded) on its deepseek_v3 (16 heads) and glm5 (8 heads) shapes
MLA_WORK = [([0], [1]), ([0], [30]), ([0], [77]), ([0], [128]), ([0], [256]), ([100], [30]), ([128], [128]),
            ([0] * 4, [189, 65, 13, 545]), ([4000] * 2, [1] * 2), ([8, 13, 65, 11, 5], [1] * 5)]


@pytest.mark.parametrize("nH", [16, 8, 128])
@pytest.mark.parametrize("work", MLA_WORK)
def test_mla_attention_grid(rt, nH, work):
    clens, lens = work
    c = mla_case(31, lens, clens, nH)
    scale = 192 ** -0.5
    if nH == 128 and sum(lens) > 200:
        # the whole-batch oracle would take minutes at 128 heads: sampled rows, each as its equivalent decode step, and
        # the convexity property on every row
        from test_gpu_reference_grid_full import _mla_convexity, _mla_rows_as_decode_steps, _sample_rows
        got = run_mla(rt, c, scale)
        _mla_convexity(c, got)
        _mla_rows_as_decode_steps(c, got, _sample_rows(lens, 1, 32), scale)
        return
    check(run_mla(rt, c, scale), oracle_mla(c, scale))


@pytest.mark.parametrize("nH,C,R", [(1, 16, 64), (3, 96, 32), (2, 40, 8)])
@pytest.mark.parametrize("work", MLA_WORK)
def test_mla_attention_other_latent_sizes(rt, nH, C, R, work):
    """The reference's smallest test model (1 head, kv_lora_rank 16: xlite/tests/kernels/mla.py:54) and other
    sizes the matrix-core kernels are not built for, through the plain vector kernel; with position lists too."""
    clens, lens = work
    c = mla_case(35, lens, clens, nH, bs=16, C=C, R=R)
    scale = (C // 4 + R) ** -0.5
    check(run_mla(rt, c, scale), oracle_mla(c, scale))
    if max(cl + l for cl, l in zip(clens, lens)) > 64:
        from gvirt_amd._C import mla_attention
        topk = _topk_indices(c, 48, 7)
        out = torch.zeros(c["T"], nH, C, dtype=torch.bfloat16, device=DEV)
        mla_attention(rt, c["qa"].to(DEV), c["qr"].to(DEV), c["kc"].to(DEV), c["pc"].to(DEV), out, c["qsl"].to(DEV),
                      c["lens"].to(DEV), c["clens"].to(DEV), c["tables"].to(DEV), nH, R, C, c["bs"], c["batch"], c["maxblk"],
                      scale, topk.to(DEV), 48)
        rt.synchronize()
        check(out.float().cpu(), O.mla_attention_ref(c["qa"], c["qr"], c["kc"], c["pc"], c["qsl"], c["lens"], c["clens"],
                                                     c["tables"], nH, R, C, c["bs"], c["batch"], c["maxblk"], scale, topk, 48))


def test_config4_deepseek_r1_decode_sampled(rt):
    """Configuration 4 shape (128 heads, block 64) with 4 of the 32 sequences at full context."""
    ctx = W.c4_context_lengths()[:4]
    w = W.mla_decode(W.MlaShape(), ctx, W.SEED_BASE + 4)
    s = w["shape"]
    from gvirt_amd._C import mla_attention
    d = W.to_device(w, DEV)
    mla_attention(rt, d["q_absorb"], d["qr"], d["k_cache"], d["pe_cache"], d["o_absorb"], d["query_start_loc"], d["lens"],
                  d["cached_lens"], d["block_tables"], s.n_heads, s.rope_head_dim, s.kv_lora_rank, s.block_size, 4,
                  w["max_num_blocks"], s.scale)
    rt.synchronize()
    ref = O.mla_attention_ref(w["q_absorb"], w["qr"], w["k_cache"], w["pe_cache"], w["query_start_loc"], w["lens"],
                              w["cached_lens"], w["block_tables"], s.n_heads, s.rope_head_dim, s.kv_lora_rank, s.block_size,
                              4, w["max_num_blocks"], s.scale)
    check(d["o_absorb"].float().cpu(), ref)


@pytest.mark.parametrize("m,h,t,d", [(3, 4, 192, 512), (3, 4, 512, 192), (3, 4, 128, 512), (3, 4, 512, 128), (530, 4, 256, 512),
                                     (963, 8, 512, 128), (32, 128, 128, 512)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_einsum(rt, m, h, t, d, dtype):
    """Cases of xlite/tests/kernels/einsum_mht_mhd.py:19-33 (bounded), both weight layouts."""
    from gvirt_amd._C import einsum_mht_htd_mhd, einsum_mht_hdt_mhd
    g = torch.Generator().manual_seed(m + t)
    a = torch.randn(m, h, t, generator=g).to(dtype)
    w = (torch.randn(h, t, d, generator=g) / t ** 0.5).to(dtype)
    ref = O.einsum_ref(a, w)
    out = torch.zeros(m, h, d, dtype=dtype, device=DEV)
    einsum_mht_htd_mhd(rt, a.to(DEV), w.to(DEV), out, m, h, t, d)
    torch.testing.assert_close(out.float().cpu(), ref, atol=2e-2, rtol=1e-2)
    out2 = torch.zeros(m, h, d, dtype=dtype, device=DEV)
    einsum_mht_hdt_mhd(rt, a.to(DEV), w.transpose(1, 2).contiguous().to(DEV), out2, m, h, t, d)
    torch.testing.assert_close(out2.float().cpu(), ref, atol=2e-2, rtol=1e-2)
    # the two layouts sum the products in different orders: equal up to a rounding step of the 16-bit result
    torch.testing.assert_close(out.float().cpu(), out2.float().cpu(), atol=2e-3, rtol=2 ** -6)


@pytest.mark.parametrize("nH,nope,vd", [(16, 128, 128), (8, 192, 256)])
def test_mla_v2_three_stage(rt, nH, nope, vd):
    """deepseek_v3 / glm5 shapes of xlite/tests/kernels/mla.py:54-58, rtol 5e-2 as there (:255)."""
    from gvirt_amd._C import mla_v2
    c = mla_case(41, [1, 40], [300, 17], nH)
    g = torch.Generator().manual_seed(42)
    rms = lambda x: x / x.pow(2).mean(-1, keepdim=True).add(1e-6).sqrt()
    qwq = rms(torch.randn(c["T"], nH, nope + 64, generator=g)).bfloat16()
    wkvb = torch.randn(nH, nope + vd, 512, generator=g).clamp(0.2, 1)
    wuk_t = wkvb[:, :nope].contiguous().bfloat16()
    wuv = wkvb[:, -vd:].transpose(1, 2).contiguous().bfloat16()
    scale = (nope + 64) ** -0.5
    out = torch.zeros(c["T"], nH, vd, dtype=torch.bfloat16, device=DEV)
    empty = torch.zeros(0, dtype=torch.int32, device=DEV)
    mla_v2(rt, qwq.to(DEV), c["qr"].to(DEV), c["kc"].to(DEV), c["pc"].to(DEV), wuk_t.to(DEV), wuv.to(DEV), out, c["qsl"].to(DEV),
           c["lens"].to(DEV), c["clens"].to(DEV), c["tables"].to(DEV), nH, 64, nope, vd, 512, c["bs"], c["batch"], c["maxblk"],
           scale, empty, 0, False, True, 8192)
    ref = O.mla_v2_ref(qwq, c["qr"], c["kc"], c["pc"], wuk_t, wuv, c["qsl"], c["lens"], c["clens"], c["tables"], nH, 64, nope, vd,
                       512, c["bs"], c["batch"], c["maxblk"], scale)
    torch.testing.assert_close(out.float().cpu(), ref, atol=3e-2, rtol=5e-2)
    with pytest.raises(RuntimeError, match="NZ"):
        mla_v2(rt, qwq.to(DEV), c["qr"].to(DEV), c["kc"].to(DEV), c["pc"].to(DEV), wuk_t.to(DEV), wuv.to(DEV), out,
               c["qsl"].to(DEV), c["lens"].to(DEV), c["clens"].to(DEV), c["tables"].to(DEV), nH, 64, nope, vd, 512, c["bs"],
               c["batch"], c["maxblk"], scale, empty, 0, True)


@pytest.mark.parametrize("cached,topk", [([127], 512), ([2047, 8191, 5841], 2048), ([4096], 512), ([131071], 2048), ([32751] * 3, 512)])
def test_gather_then_mla_v3(rt, cached, topk):
    """Decode + sparse path of xlite/tests/kernels/mla_v3.py (bounded): gather, then dense attention."""
    from gvirt_amd._C import gather_sparse_kv_cache, mla_v3
    batch = len(cached)
    c = mla_case(51, [1] * batch, cached, 16)
    g = torch.Generator().manual_seed(52)
    idx = []
    for cl in cached:
        n = cl + 1
        p = torch.randperm(n, generator=g)[:topk]
        if n < topk:
            p = torch.cat([p, p[-1:].expand(topk - n)])
        idx.append(torch.sort(p).values)
    idx = torch.stack(idx).int()
    kd = torch.zeros(batch, topk, 1, 512, dtype=torch.bfloat16, device=DEV); pd = torch.zeros(batch, topk, 1, 64, dtype=torch.bfloat16, device=DEV)
    gather_sparse_kv_cache(rt, c["kc"].to(DEV), c["pc"].to(DEV), c["tables"].to(DEV), idx.to(DEV), c["lens"].to(DEV),
                           c["clens"].to(DEV), kd, pd, batch, topk, c["bs"], c["maxblk"], 512, 64, 1)
    out = torch.zeros(batch, 16, 512, dtype=torch.bfloat16, device=DEV)
    mla_v3(rt, c["qa"].to(DEV), c["qr"].to(DEV), kd, pd, out, c["qsl"].to(DEV), c["lens"].to(DEV), c["clens"].to(DEV), 16, 64,
           512, batch, topk, 192 ** -0.5)
    ref = O.mla_v3_ref(c["qa"], c["qr"], kd.cpu(), pd.cpu(), c["qsl"], c["lens"], c["clens"], 16, 64, 512, batch, topk, 192 ** -0.5)
    check(out.float().cpu(), ref)


def _topk_indices(c, top_k, seed):
    """Index lists as the reference test draws them (xlite/tests/kernels/mla.py:280-303): a random subset of the
    causal range per query row, padded with its last element when the range is shorter than top_k, ascending."""
    g = torch.Generator().manual_seed(seed)
    rows = []
    for l, cl in zip(c["lens"].tolist(), c["clens"].tolist()):
        for r in range(l):
            valid = cl + r + 1
            perm = torch.randperm(valid, generator=g)
            perm = torch.cat([perm, perm[-1:].expand(top_k - valid)]) if valid < top_k else perm[:top_k]
            rows.append(torch.sort(perm).values)
    return torch.stack(rows).int()


@pytest.mark.parametrize("nH", [16, 128])
@pytest.mark.parametrize("work,top_k", [(([300, 40, 2100], [1, 1, 1]), 64), (([100], [30]), 32), (([0, 500], [70, 3]), 128),
                                        (([2500, 2047, 2048], [1, 1, 1]), 2048)])
def test_mla_topk_index_mask(rt, nH, work, top_k):
    """Rows longer than top_k attend to their listed positions only, shorter rows to their whole range."""
    from gvirt_amd._C import mla_attention
    clens, lens = work
    if nH == 128 and top_k == 2048:
        return   # this size at 128 heads: test_mla_topk_mask_128_heads_at_2048_entries
    c = mla_case(41, lens, clens, nH, bs=64)
    scale = 192 ** -0.5
    topk = _topk_indices(c, top_k, 42)
    out = torch.zeros(c["T"], c["nH"], c["C"], dtype=torch.bfloat16, device=DEV)
    mla_attention(rt, c["qa"].to(DEV), c["qr"].to(DEV), c["kc"].to(DEV), c["pc"].to(DEV), out, c["qsl"].to(DEV),
                  c["lens"].to(DEV), c["clens"].to(DEV), c["tables"].to(DEV), c["nH"], c["R"], c["C"], c["bs"], c["batch"],
                  c["maxblk"], scale, topk.to(DEV), top_k)
    rt.synchronize()
    ref = O.mla_attention_ref(c["qa"], c["qr"], c["kc"], c["pc"], c["qsl"], c["lens"], c["clens"], c["tables"], c["nH"],
                              c["R"], c["C"], c["bs"], c["batch"], c["maxblk"], scale, topk, top_k)
    check(out.float().cpu(), ref)


@pytest.mark.parametrize("top_k", [96, 512])
def test_mla_topk_lists_with_entries_to_ignore(rt, top_k):
    """Lists as an indexer that ranks the whole sequence leaves them for prefill rows: ascending, with positions
    beyond the row's causal range; plus repeats and negative entries. Only the usable entries count, once each
    (xlite/csrc/kernels/mla_v2.h:697-699; the mask of xlite/tests/kernels/mla.py:293-333 is a set)."""
    from gvirt_amd._C import mla_attention
    lens, clens = [7, 1, 3], [700, 1500, 64]
    c = mla_case(43, lens, clens, 16, bs=64)
    g = torch.Generator().manual_seed(44)
    rows = []
    for l, cl in zip(lens, clens):
        for r in range(l):
            total = cl + l                                   # the indexer sees the whole sequence
            pick = torch.randperm(total, generator=g)[:top_k] if total >= top_k else torch.arange(total)
            pick = torch.sort(pick).values
            if pick.numel() < top_k:
                pick = torch.cat([pick, pick[-1:].expand(top_k - pick.numel())])
            pick = pick.clone()
            pick[5] = pick[4]                                # a repeat
            pick[0] = -1                                     # an unset entry
            rows.append(pick)
    topk = torch.stack(rows).int()
    scale = 192 ** -0.5
    out = torch.zeros(c["T"], c["nH"], c["C"], dtype=torch.bfloat16, device=DEV)
    mla_attention(rt, c["qa"].to(DEV), c["qr"].to(DEV), c["kc"].to(DEV), c["pc"].to(DEV), out, c["qsl"].to(DEV),
                  c["lens"].to(DEV), c["clens"].to(DEV), c["tables"].to(DEV), c["nH"], c["R"], c["C"], c["bs"], c["batch"],
                  c["maxblk"], scale, topk.to(DEV), top_k)
    rt.synchronize()
    ref = O.mla_attention_ref(c["qa"], c["qr"], c["kc"], c["pc"], c["qsl"], c["lens"], c["clens"], c["tables"], c["nH"],
                              c["R"], c["C"], c["bs"], c["batch"], c["maxblk"], scale, topk, top_k)
    check(out.float().cpu(), ref)


def test_mla_decode_large_batch_of_short_sequences(rt):
    """More rows than threads in the work-splitting scan (two rows per thread), chunks that span many rows,
    and rows far shorter than a step."""
    g = np.random.default_rng(5)
    B = 700
    clens = [int(x) for x in g.integers(0, 90, size=B)]
    clens[3] = 0
    c = mla_case(33, [1] * B, clens, 16, bs=32)
    scale = 192 ** -0.5
    check(run_mla(rt, c, scale), oracle_mla(c, scale))


def test_mla_decode_one_long_row_among_short_ones(rt):
    """A chunk boundary inside a long row and many short rows inside one chunk."""
    clens = [5, 9000, 17, 300, 2, 64, 1000]
    c = mla_case(34, [1] * len(clens), clens, 16, bs=64)
    scale = 192 ** -0.5
    check(run_mla(rt, c, scale), oracle_mla(c, scale))


@pytest.mark.parametrize("nH,clens", [(128, [20000]), (16, [50000, 77, 9000]), (128, [3000] * 4), (8, [2500] * 40)])
def test_mla_decode_few_rows_many_partials(rt, nH, clens):
    """Few (row, head)s cut into a chunk per compute unit: four waves of the merge share a (row, head); the
    last case is just above that path's limit."""
    c = mla_case(35, [1] * len(clens), clens, nH)
    scale = 192 ** -0.5
    check(run_mla(rt, c, scale), oracle_mla(c, scale))


def test_dsa_decode_pipeline_indexer_to_masked_mla(rt):
    """DeepSeek sparse attention, decode step: indexer_topk picks the positions, mla_attention attends to
    them (xlite/csrc/model.cpp:384-427). The lists go from one operator to the other untouched; the result is
    checked against the oracle attention on the same lists, and the lists against the oracle's own."""
    from gvirt_amd._C import indexer_topk, mla_attention
    clens, lens, top_k, bs = [3000, 2100, 500, 1023], [1, 1, 1, 1], 1024, 64
    c = mla_case(51, lens, clens, 16, bs=bs)
    g = torch.Generator().manual_seed(52)
    NB = c["kc"].shape[0]
    iq = torch.randn(c["T"], 64, 128, generator=g).bfloat16()
    iw = torch.randn(c["T"], 128 + 64, generator=g).bfloat16()
    ik = torch.randn(NB, bs, 128, generator=g).bfloat16()
    ld = c["maxblk"] * bs
    lists = torch.full((c["T"], top_k), -1, dtype=torch.int32, device=DEV)
    dev = lambda t: t.to(DEV)
    meta = (dev(c["qsl"]), dev(c["lens"]), dev(c["clens"]), dev(c["tables"]))
    indexer_topk(rt, dev(iq), dev(ik), dev(iw), torch.arange(ld, dtype=torch.int32, device=DEV), lists, *meta, 64, 128, bs,
                 c["batch"], c["maxblk"], top_k)
    scale = 192 ** -0.5
    out = torch.zeros(c["T"], c["nH"], c["C"], dtype=torch.bfloat16, device=DEV)
    mla_attention(rt, dev(c["qa"]), dev(c["qr"]), dev(c["kc"]), dev(c["pc"]), out, *meta, c["nH"], c["R"], c["C"], bs,
                  c["batch"], c["maxblk"], scale, lists, top_k)
    rt.synchronize()
    got_lists = lists.cpu()
    ref = O.mla_attention_ref(c["qa"], c["qr"], c["kc"], c["pc"], c["qsl"], c["lens"], c["clens"], c["tables"], c["nH"],
                              c["R"], c["C"], bs, c["batch"], c["maxblk"], scale, got_lists.clamp(min=0), top_k)
    check(out.float().cpu(), ref)
    want = O.indexer_topk_ref(O.indexer_scores_ref(iq, ik, iw, c["qsl"], c["lens"], c["clens"], c["tables"], 64, 128, bs,
                                                   c["batch"], c["maxblk"]), top_k)
    for i in range(c["batch"]):
        n = clens[i] + 1
        row = got_lists[i, :min(top_k, n)].tolist()
        assert len(set(want[i][0]) - set(row)) * 100.0 <= 3.0 * len(row)


def test_mla_prefill_128_heads_rows_of_several_sequences(rt):
    """Chunked prefill at the full head count: hundreds of query rows, each with its own causal limit, cut
    into chunks that cross row and sequence boundaries; a sequence without query rows in between."""
    c = mla_case(61, [300, 0, 77, 1], [700, 50, 0, 2000], 128, bs=64)
    scale = 192 ** -0.5
    check(run_mla(rt, c, scale), oracle_mla(c, scale))


def test_mla_decode_at_the_longest_reference_context(rt):
    """xlite/tests/kernels/mla.py:72: two sequences of 131071 cached positions, one new token each."""
    c = mla_case(36, [1, 1], [131071, 131071], 16)
    scale = 192 ** -0.5
    check(run_mla(rt, c, scale), oracle_mla(c, scale))


def test_clock_probe_reports_a_plausible_shader_clock_and_switches_off(rt):
    """xlite_hip_set_clock_probe: while a buffer is set, workgroup 0 of the streaming MLA kernel leaves shader-clock
    and 100 MHz wall-clock stamps; their ratio is a clock between 0.3 and 3 GHz; with the probe off nothing is written."""
    import ctypes
    c = mla_case(71, [1] * 4, [3000, 2000, 4000, 1000], 128)
    buf = torch.zeros(4, dtype=torch.int64, device=DEV)
    rt._lib.xlite_hip_set_clock_probe(ctypes.c_void_p(buf.data_ptr()))
    try:
        want = run_mla(rt, c, 192 ** -0.5)
    finally:
        rt._lib.xlite_hip_set_clock_probe(None)
    c0, w0, c1, w1 = [int(x) for x in buf.tolist()]
    assert w1 > w0 and c1 > c0
    ghz = (c1 - c0) / ((w1 - w0) * 10.0)
    assert 0.3 < ghz < 3.0, ghz
    buf.zero_()
    got = run_mla(rt, c, 192 ** -0.5)
    assert torch.equal(got, want)
    assert int(buf.abs().sum()) == 0


@pytest.mark.parametrize("bs", [16, 48, 8, 1])
@pytest.mark.parametrize("nH", [16, 128])
def test_mla_block_sizes_that_are_not_a_multiple_of_32(rt, bs, nH):
    """The streaming kernel walks such caches position by position (a step's 32 positions do not share a block):
    decode rows, prefill rows and a chunked prefill, against the oracle."""
    if bs == 1:
        lens, clens = [1, 5, 1], [300, 40, 77]
    else:
        lens, clens = [1, 1, 40, 1, 9], [1500, 31, 200, 4099 if nH == 16 else 1100, 0]
    c = mla_case(91, lens, clens, nH, bs=bs)
    scale = 192 ** -0.5
    check(run_mla(rt, c, scale), oracle_mla(c, scale))


@pytest.mark.parametrize("bs", [16, 48])
def test_mla_topk_lists_over_block_sizes_that_are_not_a_multiple_of_32(rt, bs):
    """Position lists over such caches: rows longer than top_k walk their lists, shorter rows their own positions."""
    from gvirt_amd._C import mla_attention
    lens, clens, top_k = [1, 1, 6, 1], [900, 100, 700, 3000], 256
    c = mla_case(92, lens, clens, 16, bs=bs)
    scale = 192 ** -0.5
    topk = _topk_indices(c, top_k, 93)
    out = torch.zeros(c["T"], c["nH"], c["C"], dtype=torch.bfloat16, device=DEV)
    mla_attention(rt, c["qa"].to(DEV), c["qr"].to(DEV), c["kc"].to(DEV), c["pc"].to(DEV), out, c["qsl"].to(DEV),
                  c["lens"].to(DEV), c["clens"].to(DEV), c["tables"].to(DEV), c["nH"], c["R"], c["C"], c["bs"], c["batch"],
                  c["maxblk"], scale, topk.to(DEV), top_k)
    rt.synchronize()
    ref = O.mla_attention_ref(c["qa"], c["qr"], c["kc"], c["pc"], c["qsl"], c["lens"], c["clens"], c["tables"], c["nH"],
                              c["R"], c["C"], c["bs"], c["batch"], c["maxblk"], scale, topk, top_k)
    check(out.float().cpu(), ref)
