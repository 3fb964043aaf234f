"""GPU parity of the cache writers / gathers against the CPU oracle: bit-exact."""
import numpy as np
import pytest
import torch

from oracle import xlite_oracle as O

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _bits(t):
    return t.detach().cpu().contiguous().view(torch.int16)


def _cosin(rot, max_pos, dtype):
    fr = torch.outer(torch.arange(max_pos).float(), 1.0 / (10000.0 ** (torch.arange(0, rot, 2).float() / rot)))
    return torch.cat([fr.cos(), fr.sin()], -1).to(dtype)


# the reference's own grid (xlite/tests/kernels/rope_and_cache.py:60-61) plus GQA shapes
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("nH,nKV,d,rot", [(32, 32, 64, 64), (32, 32, 128, 128), (32, 32, 128, 64),
                                          (14, 2, 64, 64), (32, 8, 128, 128), (28, 4, 128, 128), (5, 1, 128, 32)])
def test_rope_and_cache_bit_exact(rt, dtype, nH, nKV, d, rot):
    from gvirt_amd._C import rope_and_cache
    g = torch.Generator().manual_seed(100 + nH + d + rot)
    T, bs, NB = 80, 128, 3
    inout = torch.randn(T, (nH + 2 * nKV) * d, generator=g).to(dtype)
    kc = torch.full((NB, bs, nKV, d), 3.0).to(dtype)
    vc = torch.full((NB, bs, nKV, d), -3.0).to(dtype)
    cosin = _cosin(rot, 1024, dtype)
    pos = torch.randint(0, 1024, (T,), generator=g)
    slots = torch.randperm(NB * bs, generator=g)[:T].int()
    dev = [x.to(DEV) for x in (inout, kc, vc, pos, cosin, slots)]
    rope_and_cache(rt, *dev, nH, nKV, d, rot, bs, True)
    O.rope_and_cache_ref(inout, kc, vc, pos, cosin, slots, nH, nKV, d, rot, bs)
    assert torch.equal(_bits(dev[0]), _bits(inout))
    assert torch.equal(_bits(dev[1]), _bits(kc))
    assert torch.equal(_bits(dev[2]), _bits(vc))


def test_rope_and_cache_mrope_and_empty(rt):
    from gvirt_amd._C import rope_and_cache
    g = torch.Generator().manual_seed(5)
    T, nH, nKV, d, bs = 33, 4, 2, 128, 16
    inout = torch.randn(T, (nH + 2 * nKV) * d, generator=g).bfloat16()
    kc = torch.zeros(4, bs, nKV, d).bfloat16(); vc = torch.zeros(4, bs, nKV, d).bfloat16()
    cosin = _cosin(d, 256, torch.bfloat16)
    pos = torch.randint(0, 256, (3, T), generator=g)
    slots = torch.randperm(4 * bs, generator=g)[:T].int()
    mh, mw = 0x0000_00FF_FF00_0000, 0x0000_FF00_00FF_0000  # disjoint lane sets below 64
    dev = [x.to(DEV) for x in (inout, kc, vc, pos, cosin, slots)]
    rope_and_cache(rt, *dev, nH, nKV, d, d, bs, True, mh, mw)
    O.rope_and_cache_ref(inout, kc, vc, pos, cosin, slots, nH, nKV, d, d, bs, mh, mw)
    assert torch.equal(_bits(dev[0]), _bits(inout)) and torch.equal(_bits(dev[1]), _bits(kc))
    # zero tokens: nothing happens, nothing is touched
    empty = torch.zeros(0, (nH + 2 * nKV) * d, dtype=torch.bfloat16, device=DEV)
    rope_and_cache(rt, empty, dev[1], dev[2], torch.zeros(0, dtype=torch.int64, device=DEV), dev[4],
                   torch.zeros(0, dtype=torch.int32, device=DEV), nH, nKV, d, d, bs, True)
    assert torch.equal(_bits(dev[1]), _bits(kc))


@pytest.mark.parametrize("cached,topk", [([127], 512), ([2047, 8191, 45841], 2048), ([2047] * 4, 512), ([16384], 2048),
                                         ([131071], 2048), ([32751] * 3, 512), ([4096], 512)])
def test_gather_sparse_kv_cache_exact(rt, cached, topk):
    """Workloads of xlite/tests/kernels/gather_sparse_kv_cache.py:37-49, exact equality."""
    from gvirt_amd._C import gather_sparse_kv_cache
    g = torch.Generator().manual_seed(len(cached) * 31 + topk)
    bs, C, R = 128, 512, 64
    batch = len(cached)
    maxblk = (max(cached) + 1 + bs - 1) // bs
    NB = batch * maxblk
    kc = torch.randn(NB, bs, 1, C, generator=g).bfloat16()
    pc = torch.randn(NB, bs, 1, R, generator=g).bfloat16()
    tables = torch.randperm(NB, generator=g).int()
    idx = []
    for c in cached:
        n = c + 1
        p = torch.randperm(n, generator=g)[:topk]
        if n < topk:
            p = torch.cat([p, p[-1:].expand(topk - n)])
        idx.append(torch.sort(p).values)
    idx = torch.stack(idx).int()
    ql = torch.ones(batch, dtype=torch.int32); cl = torch.tensor(cached, dtype=torch.int32)
    kd = torch.full((batch, topk, 1, C), 9.0).bfloat16(); pd = torch.full((batch, topk, 1, R), 9.0).bfloat16()
    dkd, dpd = kd.to(DEV), pd.to(DEV)
    gather_sparse_kv_cache(rt, kc.to(DEV), pc.to(DEV), tables.to(DEV), idx.to(DEV), ql.to(DEV), cl.to(DEV), dkd, dpd,
                           batch, topk, bs, maxblk, C, R)
    O.gather_sparse_kv_cache_ref(kc, pc, tables, idx, ql, cl, kd, pd, batch, topk, bs, maxblk, C, R)
    assert torch.equal(_bits(dkd), _bits(kd)) and torch.equal(_bits(dpd), _bits(pd))  # incl. untouched tail


@pytest.mark.parametrize("dtype,rope,step", [(torch.float16, 64, 64), (torch.float16, 64, 192), (torch.bfloat16, 64, 128),
                                             (torch.bfloat16, 64, 576)])
def test_rope_complex_bit_exact(rt, dtype, rope, step):
    from gvirt_amd._C import rope_complex
    g = torch.Generator().manual_seed(rope + step)
    T, H = 80, 64
    x = torch.randn(T, H, step, generator=g).to(dtype)
    ang = torch.outer(torch.arange(1024).float(), 1.0 / (10000.0 ** (torch.arange(0, rope, 2).float() / rope)))
    freqs = torch.polar(torch.ones_like(ang), ang)
    pos = torch.randint(0, 1024, (T,), generator=g)
    out = torch.zeros(T, H, rope, dtype=dtype, device=DEV)
    rope_complex(rt, H, step, rope, x.to(DEV), freqs.to(DEV), pos.to(DEV), out)
    assert torch.equal(_bits(out), _bits(O.rope_complex_ref(H, step, rope, x, freqs, pos)))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_mla_prepare(rt, dtype):
    """Shapes of xlite/tests/kernels/mla_prepare.py:61-64; rope slice and caches exact, RMSNorm outputs
    within the reference's own tolerance (the fp32 sum of squares is reduced in a different order)."""
    from gvirt_amd._C import mla_prepare
    g = torch.Generator().manual_seed(77)
    T, ql, kl, rp, bs = 80, 2048, 512, 64, 128
    row = (torch.randn(T, ql + kl + rp, generator=g) / 10).to(dtype)
    w1, b1, w2, b2 = [(torch.randn(n, generator=g) / 10).to(dtype) for n in (ql, ql, kl, kl)]
    ang = torch.outer(torch.arange(1024).float(), 1.0 / (10000.0 ** (torch.arange(0, rp, 2).float() / rp)))
    freqs = torch.polar(torch.ones_like(ang), ang)
    pos = torch.randint(0, 1024, (T,), generator=g)
    slots = torch.randperm(bs, generator=g)[:T].int()
    qc = torch.zeros(T, ql).to(dtype); kvc = torch.zeros(T, kl).to(dtype)
    kcache = torch.zeros(1, bs, kl).to(dtype); pcache = torch.zeros(1, bs, rp).to(dtype)
    d = [x.to(DEV) for x in (row, w1, b1, qc, w2, b2, kvc, freqs, pos)]
    dk, dp, ds = kcache.to(DEV), pcache.to(DEV), slots.to(DEV)
    mla_prepare(rt, *d, ql, kl, rp, bs, dk, dp, ds, 1e-6)
    O.mla_prepare_ref(row, w1, b1, qc, w2, b2, kvc, freqs, pos, ql, kl, rp, bs, kcache, pcache, slots, 1e-6)
    torch.testing.assert_close(d[3].cpu(), qc, atol=2e-5, rtol=1e-3 if dtype == torch.float16 else 8e-3)
    torch.testing.assert_close(d[6].cpu(), kvc, atol=2e-5, rtol=1e-3 if dtype == torch.float16 else 8e-3)
    assert torch.equal(_bits(d[0][:, ql + kl:]), _bits(row[:, ql + kl:]))       # rotated slice, in place
    assert torch.equal(_bits(d[0][:, :ql + kl]), _bits(row[:, :ql + kl]))       # the rest untouched
    assert torch.equal(_bits(dp), _bits(pcache))
    assert torch.equal(_bits(dk.view(bs, kl)[ds.long()]), _bits(d[6]))          # cache row == returned row
    # block_size 0 disables the cache writes
    dk2 = torch.zeros_like(dk)
    mla_prepare(rt, *[x.to(DEV) for x in (row, w1, b1, qc, w2, b2, kvc, freqs, pos)], ql, kl, rp, 0, dk2, dp, ds, 1e-6)
    assert int(dk2.abs().sum()) == 0


QUANT = {torch.int8: O.quantize_kv_int8, torch.float8_e4m3fn: O.quantize_kv_fp8}


def _same(a, b):
    return torch.equal(a.view(torch.uint8), b.view(torch.uint8))


@pytest.mark.parametrize("kv_dtype", [torch.int8, torch.float8_e4m3fn])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_quantize_kv_matches_definition(rt, kv_dtype, dtype):
    from gvirt_amd._C import quantize_kv, quantize_kv_int8
    g = torch.Generator().manual_seed(9)
    x = (torch.randn(3, 128, 8, 128, generator=g) * torch.rand(3, 128, 8, 1, generator=g) * 4).to(dtype)
    x[0, 0, 0] = 0
    x[1, 5, 2] *= 1e-4      # a tiny row: its quotients still span the format's whole range
    q, s = quantize_kv(rt, x.to(DEV), kv_dtype)
    qr, sr = QUANT[kv_dtype](x)
    assert q.dtype == kv_dtype and _same(q.cpu(), qr) and torch.equal(s.cpu(), sr)
    if kv_dtype == torch.int8:
        q2, s2 = quantize_kv_int8(rt, x.to(DEV))
        assert torch.equal(q2, q) and torch.equal(s2, s)


@pytest.mark.parametrize("kv_dtype", [torch.int8, torch.float8_e4m3fn])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("nH,nKV,d,rot", [(32, 8, 128, 128), (14, 2, 64, 64), (8, 4, 128, 64), (4, 2, 256, 256), (4, 1, 256, 64)])
def test_rope_and_cache_quantise_on_write(rt, kv_dtype, dtype, nH, nKV, d, rot):
    """The rows land in the quantised cache as the oracle's quantisation of the oracle's rotated rows: bit-exact
    (values and scales); slots of other tokens keep their contents. One launch for heads of at most 16 items
    (all but the last shape), two for wider ones."""
    from gvirt_amd._C import rope_and_cache
    g = torch.Generator().manual_seed(300 + nH + d + rot)
    T, bs, NB = 37, 16, 5
    inout = torch.randn(T, (nH + 2 * nKV) * d, generator=g).to(dtype)
    inout[3, nH * d:(nH + 1) * d] = 0          # an all-zero K row: scale 0, values 0
    cosin = _cosin(rot, 512, dtype)
    pos = torch.randint(0, 512, (T,), generator=g)
    slots = torch.randperm(NB * bs, generator=g)[:T].int()
    fill = lambda v: torch.full((NB, bs, nKV, d), v, dtype=torch.int8).view(kv_dtype).to(DEV)
    kq, vq = fill(9), fill(-9)
    ks = torch.full((NB, bs, nKV), 5.0, device=DEV)
    vs = torch.full((NB, bs, nKV), -5.0, device=DEV)
    dev_inout = inout.to(DEV)
    rope_and_cache(rt, dev_inout, kq, vq, pos.to(DEV), cosin.to(DEV), slots.to(DEV), nH, nKV, d, rot, bs, True,
                   k_scale=ks, v_scale=vs)
    # oracle: 16-bit rope and cache write, then the quantiser on the written rows
    kc = torch.zeros(NB, bs, nKV, d).to(dtype)
    vc = torch.zeros(NB, bs, nKV, d).to(dtype)
    O.rope_and_cache_ref(inout, kc, vc, pos, cosin, slots, nH, nKV, d, rot, bs)
    assert torch.equal(_bits(dev_inout), _bits(inout))
    kq_ref, ks_ref = QUANT[kv_dtype](kc)
    vq_ref, vs_ref = QUANT[kv_dtype](vc)
    written = torch.zeros(NB * bs, dtype=torch.bool)
    written[slots.long()] = True
    w = written.view(NB, bs)
    b = lambda t: t.cpu().view(torch.int8)
    assert torch.equal(b(kq)[w], b(kq_ref)[w]) and torch.equal(b(vq)[w], b(vq_ref)[w])
    assert torch.equal(ks.cpu()[w], ks_ref[w]) and torch.equal(vs.cpu()[w], vs_ref[w])
    assert bool((b(kq)[~w] == 9).all()) and bool((b(vq)[~w] == -9).all())
    assert bool((ks.cpu()[~w] == 5.0).all()) and bool((vs.cpu()[~w] == -5.0).all())


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("nH,nKV,d,bias,full", [(32, 8, 128, True, False), (14, 2, 64, False, False), (16, 4, 128, False, True)])
def test_qk_rms_norm(rt, dtype, nH, nKV, d, bias, full):
    """Per-head (xlite/csrc/model.cpp:516-519) and whole-segment granularity; V columns bit-identical; the
    normalised values within one 16-bit unit of the oracle (the fp32 sum of squares is reduced in another
    order), as for mla_prepare."""
    from gvirt_amd._C import qk_rms_norm
    g = torch.Generator().manual_seed(400 + nH + d)
    T = 41
    x = torch.randn(T, (nH + 2 * nKV) * d, generator=g).to(dtype)
    qd, qc, kd, kc_ = (nH * d, 1, nKV * d, 1) if full else (d, nH, d, nKV)
    wq, wk = torch.randn(qd, generator=g).to(dtype), torch.randn(kd, generator=g).to(dtype)
    bq = torch.randn(qd, generator=g).to(dtype) if bias else None
    bk = torch.randn(kd, generator=g).to(dtype) if bias else None
    ref = O.qk_rms_norm_ref(x, wq, bq, wk, bk, 1e-6, qd, qc, kd, kc_, nH * d)
    dev = x.to(DEV)
    mv = lambda t: None if t is None else t.to(DEV)
    qk_rms_norm(rt, dev, mv(wq), mv(bq), mv(wk), mv(bk), dev, 1e-6, qd, qc, kd, kc_, nH * d)   # in place
    got = dev.cpu()
    assert torch.equal(_bits(got[:, (nH + nKV) * d:]), _bits(x[:, (nH + nKV) * d:]))
    torch.testing.assert_close(got[:, :(nH + nKV) * d].float(), ref[:, :(nH + nKV) * d].float(), atol=2e-5,
                               rtol=1e-3 if dtype == torch.float16 else 8e-3)
    # into a separate output: only the two segments are written
    out = torch.full_like(dev, 7.0)
    qk_rms_norm(rt, x.to(DEV), mv(wq), mv(bq), mv(wk), mv(bk), out, 1e-6, qd, qc, kd, kc_, nH * d)
    assert torch.equal(_bits(out.cpu()[:, :(nH + nKV) * d]), _bits(got[:, :(nH + nKV) * d]))
    assert bool((out.cpu()[:, (nH + nKV) * d:] == 7.0).all())
