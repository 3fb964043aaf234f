"""Pins for the CPU oracle: every check here is independent of the oracle's own formula
(brute-force fp64 C loops, closed forms, library routines, invariances)."""
import math

import numpy as np
import pytest
import torch

from oracle import brute
from oracle import xlite_oracle as O


def _paged_case(seed, batch, lens, clens, nH, nKV, d, bs, dtype, permute=True):
    g = torch.Generator().manual_seed(seed)
    T = sum(lens)
    maxblk = max((l + c + bs - 1) // bs for l, c in zip(lens, clens))
    NB = batch * maxblk + 3
    qkv = (torch.randn(T, (nH + 2 * nKV) * d, generator=g) * 0.5).to(dtype)
    kc = torch.randn(NB, bs, nKV, d, generator=g).to(dtype)
    vc = torch.randn(NB, bs, nKV, d, generator=g).to(dtype)
    perm = torch.randperm(NB, generator=g) if permute else torch.arange(NB)
    tables = perm[: batch * maxblk].to(torch.int32).view(batch, maxblk)
    qsl = np.cumsum([0] + lens[:-1]).tolist()
    return qkv, kc, vc, qsl, tables, maxblk, T


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("nH,nKV,d", [(4, 2, 64), (5, 1, 128), (2, 2, 32)])
def test_attention_vs_fp64_bruteforce(dtype, nH, nKV, d):
    bs = 16
    lens, clens = [1, 7, 3], [37, 0, 20]
    qkv, kc, vc, qsl, tables, maxblk, T = _paged_case(1, 3, lens, clens, nH, nKV, d, bs, dtype)
    ref = brute.attention(qkv, kc, vc, qsl, lens, clens, tables.flatten(), nH, nKV, d, bs, 3, maxblk)
    got = O.attention_ref(qkv, kc, vc, qsl, lens, clens, tables.flatten(), nH, nKV, d, bs, 3, maxblk)
    assert torch.allclose(got.double(), ref, atol=2e-5, rtol=1e-4)


def test_attention_vs_torch_sdpa():
    """Library cross-check: dense K/V gathered by hand, torch's own fused attention."""
    nH, nKV, d, bs = 6, 2, 64, 8
    lens, clens = [5], [11]
    qkv, kc, vc, qsl, tables, maxblk, T = _paged_case(2, 1, lens, clens, nH, nKV, d, bs, torch.bfloat16)
    n = 16
    keys = torch.stack([kc[tables[0, p // bs], p % bs] for p in range(n)]).float()
    vals = torch.stack([vc[tables[0, p // bs], p % bs] for p in range(n)]).float()
    q = qkv.view(T, nH + 2 * nKV, d)[:, :nH].float().transpose(0, 1).unsqueeze(0)  # [1,nH,q,d]
    k = keys.repeat_interleave(nH // nKV, 1).transpose(0, 1).unsqueeze(0)
    v = vals.repeat_interleave(nH // nKV, 1).transpose(0, 1).unsqueeze(0)
    allowed = torch.arange(n).unsqueeze(0) <= (11 + torch.arange(5)).unsqueeze(1)
    ref = torch.nn.functional.scaled_dot_product_attention(q, k, v, attn_mask=allowed, scale=1.0)
    ref = ref[0].transpose(0, 1).reshape(T, nH * d)
    got = O.attention_ref(qkv, kc, vc, qsl, lens, clens, tables.flatten(), nH, nKV, d, bs, 1, maxblk)
    assert torch.allclose(got, ref, atol=2e-5, rtol=1e-4)


def test_attention_closed_forms():
    nH, nKV, d, bs = 4, 2, 32, 4
    # a single visible key: the output is exactly v0 of the matching kv head
    qkv, kc, vc, qsl, tables, maxblk, T = _paged_case(3, 1, [1], [0], nH, nKV, d, bs, torch.bfloat16)
    got = O.attention_ref(qkv, kc, vc, qsl, [1], [0], tables.flatten(), nH, nKV, d, bs, 1, maxblk)
    v0 = vc[tables[0, 0], 0].float().repeat_interleave(nH // nKV, 0).reshape(1, nH * d)
    assert torch.equal(got, v0)
    # all keys equal: uniform probabilities, output = mean of V
    qkv, kc, vc, qsl, tables, maxblk, T = _paged_case(4, 1, [1], [9], nH, nKV, d, bs, torch.bfloat16)
    kc[:] = kc[0, 0]
    got = O.attention_ref(qkv, kc, vc, qsl, [1], [9], tables.flatten(), nH, nKV, d, bs, 1, maxblk)
    vals = torch.stack([vc[tables[0, p // bs], p % bs] for p in range(10)]).float().mean(0)
    assert torch.allclose(got, vals.repeat_interleave(nH // nKV, 0).reshape(1, -1), atol=1e-6)


def test_attention_block_permutation_invariance_and_decode_equivalence():
    nH, nKV, d, bs = 4, 1, 64, 8
    lens, clens = [6], [13]
    qkv, kc, vc, qsl, tables, maxblk, T = _paged_case(5, 1, lens, clens, nH, nKV, d, bs, torch.bfloat16)
    a = O.attention_ref(qkv, kc, vc, qsl, lens, clens, tables.flatten(), nH, nKV, d, bs, 1, maxblk)
    # identity table over a re-packed cache gives bit-identical results
    ident = torch.arange(maxblk, dtype=torch.int32)
    kc2, vc2 = kc[tables[0].long()].clone(), vc[tables[0].long()].clone()
    b = O.attention_ref(qkv, kc2, vc2, qsl, lens, clens, ident, nH, nKV, d, bs, 1, maxblk)
    assert torch.equal(a, b)
    # each prefill row equals the same row issued alone as a decode step
    for r in range(6):
        one = O.attention_ref(qkv[r:r + 1], kc, vc, [0], [1], [13 + r], tables.flatten(), nH, nKV,
                              d, bs, 1, maxblk)
        assert torch.allclose(one[0], a[r], atol=1e-6)


def _mla_case(seed, lens, clens, nH, R, C, bs):
    g = torch.Generator().manual_seed(seed)
    batch, T = len(lens), sum(lens)
    maxblk = max((l + c + bs - 1) // bs for l, c in zip(lens, clens))
    NB = batch * maxblk + 2
    qa = (torch.randn(T, nH, C, generator=g) * 0.3).bfloat16()
    qr = (torch.randn(T, nH, R, generator=g) * 0.3).bfloat16()
    kc = torch.randn(NB, bs, C, generator=g).bfloat16()
    pc = torch.randn(NB, bs, R, generator=g).bfloat16()
    tables = torch.randperm(NB, generator=g)[: batch * maxblk].to(torch.int32)
    qsl = np.cumsum([0] + lens[:-1]).tolist()
    return qa, qr, kc, pc, qsl, tables, maxblk, T


def test_mla_vs_fp64_bruteforce_dense_and_topk():
    nH, R, C, bs = 3, 8, 32, 8
    lens, clens = [1, 5], [20, 3]
    qa, qr, kc, pc, qsl, tables, maxblk, T = _mla_case(6, lens, clens, nH, R, C, bs)
    scale = 0.17
    ref = brute.mla(qa, qr, kc, pc, qsl, lens, clens, tables, nH, R, C, bs, 2, maxblk, scale)
    got = O.mla_attention_ref(qa, qr, kc, pc, qsl, lens, clens, tables, nH, R, C, bs, 2, maxblk, scale)
    assert torch.allclose(got.double(), ref, atol=2e-5, rtol=1e-4)
    g = torch.Generator().manual_seed(7)
    top_k = 4
    topk = torch.stack([torch.sort(torch.randperm(8, generator=g)[:top_k]).values for _ in range(T)]).int()
    ref = brute.mla(qa, qr, kc, pc, qsl, lens, clens, tables, nH, R, C, bs, 2, maxblk, scale, topk, top_k)
    got = O.mla_attention_ref(qa, qr, kc, pc, qsl, lens, clens, tables, nH, R, C, bs, 2, maxblk,
                              scale, topk, top_k)
    assert torch.allclose(got.double(), ref, atol=2e-5, rtol=1e-4)


def test_mla_absorbed_equals_naive_per_head_fp64():
    """The absorbed form must equal the textbook per-head MLA (k = W_UK latent, v = W_UV^T latent)."""
    g = torch.Generator().manual_seed(8)
    nH, nope, rope, vdim, C, n = 2, 6, 4, 5, 8, 9
    q_nope = torch.randn(1, nH, nope, generator=g, dtype=torch.float64)
    q_rope = torch.randn(1, nH, rope, generator=g, dtype=torch.float64)
    lat = torch.randn(n, C, generator=g, dtype=torch.float64)
    pe = torch.randn(n, rope, generator=g, dtype=torch.float64)
    wuk_t = torch.randn(nH, nope, C, generator=g, dtype=torch.float64)   # [h, nope, C]
    wuv = torch.randn(nH, C, vdim, generator=g, dtype=torch.float64)     # [h, C, v]
    scale = (nope + rope) ** -0.5
    k_nope = torch.einsum("nc,hdc->nhd", lat, wuk_t)
    v = torch.einsum("nc,hcv->nhv", lat, wuv)
    s = (torch.einsum("qhd,nhd->hqn", q_nope, k_nope) + torch.einsum("qhr,nr->hqn", q_rope, pe)) * scale
    naive = torch.einsum("hqn,nhv->qhv", torch.softmax(s, -1), v)
    # run the oracle on values that are exact in bf16 so no rounding enters
    def exact(x):
        return (x * 4).round().div(4).clamp(-3, 3)
    q_nope, q_rope, lat, pe, wuk_t, wuv = map(exact, (q_nope, q_rope, lat, pe, wuk_t, wuv))
    k_nope = torch.einsum("nc,hdc->nhd", lat, wuk_t)
    v = torch.einsum("nc,hcv->nhv", lat, wuv)
    s = (torch.einsum("qhd,nhd->hqn", q_nope, k_nope) + torch.einsum("qhr,nr->hqn", q_rope, pe)) * scale
    naive = torch.einsum("hqn,nhv->qhv", torch.softmax(s, -1), v)
    qwq = torch.cat([q_nope, q_rope], -1).bfloat16()
    kc = torch.zeros(2, 8, C).bfloat16(); pc = torch.zeros(2, 8, rope).bfloat16()
    kc.view(16, C)[:n] = lat.bfloat16(); pc.view(16, rope)[:n] = pe.bfloat16()
    out = O.mla_v2_ref(qwq, q_rope.bfloat16(), kc, pc, wuk_t.bfloat16(), wuv.bfloat16(), [0], [1],
                       [n - 1], torch.tensor([0, 1], dtype=torch.int32), nH, rope, nope, vdim, C, 8,
                       1, 2, scale, round_intermediates=False)
    assert torch.allclose(out.double(), naive, atol=1e-5, rtol=1e-5)


def test_mla_v3_matches_dense_prefix_of_paged():
    nH, R, C, bs = 2, 8, 16, 4
    qa, qr, kc, pc, qsl, tables, maxblk, T = _mla_case(9, [1], [10], nH, R, C, bs)
    topk = 16
    kd = torch.zeros(1, topk, C).bfloat16(); pd = torch.zeros(1, topk, R).bfloat16()
    idx = torch.arange(topk, dtype=torch.int32).clamp(max=10).view(1, topk)
    O.gather_sparse_kv_cache_ref(kc, pc, tables, idx, [1], [10], kd, pd, 1, topk, bs, maxblk, C, R)
    assert torch.equal(kd[0, 11:], torch.zeros(5, C).bfloat16())       # padding tail untouched
    a = O.mla_v3_ref(qa, qr, kd, pd, [0], [1], [10], nH, R, C, 1, topk, 0.3)
    b = O.mla_attention_ref(qa, qr, kc, pc, [0], [1], [10], tables, nH, R, C, bs, 1, maxblk, 0.3)
    assert torch.allclose(a, b, atol=1e-6)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("d,rot", [(64, 64), (128, 128), (128, 64)])
def test_rope_and_cache_bit_exact_vs_c(dtype, d, rot):
    g = torch.Generator().manual_seed(10)
    T, nH, nKV, bs, NB = 9, 3, 2, 4, 5
    inout = torch.randn(T, (nH + 2 * nKV) * d, generator=g).to(dtype)
    kc = torch.full((NB, bs, nKV, d), 7.0).to(dtype); vc = torch.full((NB, bs, nKV, d), -7.0).to(dtype)
    fr = torch.outer(torch.arange(32).float(), 1.0 / (10000.0 ** (torch.arange(0, rot, 2).float() / rot)))
    cosin = torch.cat([fr.cos(), fr.sin()], -1).to(dtype)
    pos = torch.randint(0, 32, (T,), generator=g)
    slots = torch.randperm(NB * bs, generator=g)[:T].int()
    a, b, c = brute.rope_and_cache(inout, kc, vc, pos, cosin, slots, nH, nKV, d, rot, bs)
    O.rope_and_cache_ref(inout, kc, vc, pos, cosin, slots, nH, nKV, d, rot, bs)
    for x, y in ((a, inout), (b, kc), (c, vc)):
        assert torch.equal(x.view(torch.int16), y.view(torch.int16))
    # untouched slots keep their sentinel, touched ones hold the updated k / the raw v
    touched = torch.zeros(NB * bs, dtype=torch.bool); touched[slots.long()] = True
    assert torch.equal(kc.view(NB * bs, -1)[~touched], torch.full((NB * bs - T, nKV * d), 7.0).to(dtype))
    row = inout.view(T, nH + 2 * nKV, d)
    assert torch.equal(kc.view(NB * bs, nKV, d)[slots.long()], row[:, nH:nH + nKV])
    assert torch.equal(vc.view(NB * bs, nKV, d)[slots.long()], row[:, nH + nKV:])


def test_rope_matches_reference_golden_formula_and_identities():
    """Same shape as the reference's own golden (rotate_half form, dtype arithmetic)."""
    g = torch.Generator().manual_seed(11)
    T, nH, nKV, d, bs = 4, 2, 2, 64, 8
    x = torch.randn(T, (nH + 2 * nKV) * d, generator=g).bfloat16()
    fr = torch.outer(torch.arange(16).float(), 1.0 / (10000.0 ** (torch.arange(0, d, 2).float() / d)))
    cosin = torch.cat([fr.cos(), fr.sin()], -1).bfloat16()
    pos = torch.tensor([0, 3, 7, 15])
    y = x.clone()
    kc = torch.zeros(1, bs, nKV, d).bfloat16(); vc = torch.zeros(1, bs, nKV, d).bfloat16()
    O.rope_and_cache_ref(y, kc, vc, pos, cosin, torch.arange(T).int(), nH, nKV, d, d, bs)
    xr = x.view(T, nH + 2 * nKV, d); yr = y.view(T, nH + 2 * nKV, d)
    cos = cosin[pos][:, None, : d // 2].repeat(1, 1, 2); sin = cosin[pos][:, None, d // 2:].repeat(1, 1, 2)
    k = xr[:, nH:nH + nKV]
    half = torch.cat([-k[..., d // 2:], k[..., : d // 2]], -1)
    golden_k = k * cos + half * sin                     # bf16 tensor arithmetic, as in the golden
    assert torch.equal(yr[:, nH:nH + nKV], golden_k)
    q = xr[:, :nH]
    halfq = torch.cat([-q[..., d // 2:], q[..., : d // 2]], -1)
    golden_q = (q * cos + halfq * sin) * d ** -0.5
    assert torch.equal(yr[:, :nH], golden_q)
    assert torch.equal(yr[0, nH:nH + nKV], xr[0, nH:nH + nKV])     # position 0 = identity
    assert torch.equal(yr[:, nH + nKV:], xr[:, nH + nKV:])         # v is never modified


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_rope_complex_vs_c_and_complex_product(dtype):
    g = torch.Generator().manual_seed(12)
    T, H, step, rope = 6, 3, 48, 16
    x = torch.randn(T, H, step, generator=g).to(dtype)
    ang = torch.outer(torch.arange(20).float(), 1.0 / (10000.0 ** (torch.arange(0, rope, 2).float() / rope)))
    freqs = torch.polar(torch.ones_like(ang), ang)
    pos = torch.randint(0, 20, (T,), generator=g)
    got = O.rope_complex_ref(H, step, rope, x, freqs, pos)
    ref = brute.rope_complex(x, torch.view_as_real(freqs).reshape(20, rope), pos, H, step, rope)
    assert torch.equal(got.view(torch.int16), ref.view(torch.int16))
    xc = torch.view_as_complex(x[..., step - rope:].double().reshape(T, H, rope // 2, 2))
    yc = xc * freqs[pos].to(torch.complex128).unsqueeze(1)
    exact = torch.cat([yc.real, yc.imag], -1)
    assert torch.allclose(got.double(), exact, atol=0.02, rtol=1e-2)
    assert torch.allclose(got.double().pow(2).sum(-1), x[..., step - rope:].double().pow(2).sum(-1), rtol=2e-2)


def test_rmsnorm_closed_forms_and_mla_prepare_composition():
    x = torch.full((2, 8), 3.0).bfloat16()
    out = O.rmsnorm_ref(x, torch.full((8,), 2.0).bfloat16(), torch.full((8,), 0.5).bfloat16(), 0.0)
    assert torch.equal(out, torch.full((2, 8), 2.5).bfloat16())          # x/rms = 1
    g = torch.Generator().manual_seed(13)
    T, ql, kl, rp, bs = 5, 16, 8, 4, 4
    row = (torch.randn(T, ql + kl + rp, generator=g) / 10).bfloat16()
    w1, b1 = torch.randn(ql, generator=g).bfloat16(), torch.randn(ql, generator=g).bfloat16()
    w2, b2 = torch.randn(kl, generator=g).bfloat16(), torch.randn(kl, generator=g).bfloat16()
    ang = torch.outer(torch.arange(8).float(), 1.0 / (10000.0 ** (torch.arange(0, rp, 2).float() / rp)))
    freqs = torch.polar(torch.ones_like(ang), ang)
    pos = torch.tensor([0, 1, 2, 3, 4]); slots = torch.tensor([3, 0, 5, 6, 1]).int()
    qc = torch.zeros(T, ql).bfloat16(); kvc = torch.zeros(T, kl).bfloat16()
    kcache = torch.zeros(2, bs, kl).bfloat16(); pcache = torch.zeros(2, bs, rp).bfloat16()
    before = row.clone()
    O.mla_prepare_ref(row, w1, b1, qc, w2, b2, kvc, freqs, pos, ql, kl, rp, bs, kcache, pcache, slots, 1e-6)
    xf = before[:, :ql].double()
    manual = (xf / (xf.pow(2).mean(-1, keepdim=True) + 1e-6).sqrt()) * w1.double() + b1.double()
    assert torch.allclose(qc.double(), manual, atol=0.02, rtol=1e-2)
    assert torch.equal(row[:, :ql + kl], before[:, :ql + kl])
    assert torch.equal(kcache.view(8, kl)[slots.long()], kvc)
    assert torch.equal(pcache.view(8, rp)[slots.long()], row[:, ql + kl:])
    assert torch.equal(row[:, ql + kl:], O.rope_complex_ref(1, rp, rp, before[:, ql + kl:].contiguous(), freqs, pos).view(T, rp))


def test_prepare_attn_hand_case():
    m = O.prepare_attn_ref([3, 1], [5, 9], [[7, 2], [4, 9, 1]], 4)
    assert m["query_start_loc"] == [0, 3]
    assert m["position"] == [5, 6, 7, 9]
    assert m["slot_mapping"] == [2 * 4 + 1, 2 * 4 + 2, 2 * 4 + 3, 1 * 4 + 1]
    assert m["max_num_blocks"] == 3 and m["batched_tokens"] == 4 and not m["is_decode"]
    assert m["block_tables"].tolist() == [[7, 2, 0], [4, 9, 1]]


def test_tile_size_hand_cases():
    # prefill -> fixed values by core count (auto_tuner.cpp:177-184)
    assert O.get_tile_size_of_cached_kv_ref([0], [100], 4, 8, 128, 24) == 6016
    assert O.get_tile_size_of_cached_kv_ref([0], [100], 4, 8, 128, 20) == 8192
    # batch 1 decode, cached 65536: tasks = round(1.5*8+3) = 15 -> ceil(65536/15)=4370 -> 4480
    assert O.get_tile_size_of_cached_kv_ref([65536], [1], 4, 8, 128, 24) == 4480
    # short context clamps to the 1024 floor
    assert O.get_tile_size_of_cached_kv_ref([2000], [1], 4, 8, 128, 24) == 1024
    # batch 2 decode with kv length 8192 each: tile 8192 scores 0.7*1 + 0.2*(16 % 24)/24 + 0.1
    # and no smaller tile reaches a kv remainder score of 1, so 8192 wins
    assert O.get_tile_size_of_cached_kv_ref([8191, 8191], [1, 1], 4, 8, 128, 24) == 8192


def test_int8_roundtrip_bound():
    g = torch.Generator().manual_seed(14)
    x = torch.randn(7, 3, 128, generator=g).bfloat16()
    q, s = O.quantize_kv_int8(x)
    assert q.dtype == torch.int8 and int(q.abs().max()) == 127
    err = (O.dequantize_kv_int8(q, s) - x.float()).abs()
    assert bool((err <= s.unsqueeze(-1) * 0.5 + 1e-7).all())
    z, sz = O.quantize_kv_int8(torch.zeros(2, 8))
    assert int(z.abs().max()) == 0 and float(sz.max()) == 0.0


def _e4m3_value(byte: int) -> float:
    """A byte of the OCP e4m3 format by its definition: sign, 4 exponent bits (bias 7), 3 mantissa bits; exponent
    0 is subnormal (no implicit one, 2^-6); 0x7f / 0xff are NaN and there are no infinities."""
    s, e, m = byte >> 7, (byte >> 3) & 15, byte & 7
    if e == 15 and m == 7:
        return float("nan")
    mag = (m / 8.0) * 2.0 ** -6 if e == 0 else (1.0 + m / 8.0) * 2.0 ** (e - 7)
    return -mag if s else mag


def test_fp8_quantiser_against_the_format_definition():
    """The fp8 cache format is pinned by brute force over the format's 256 bytes: torch decodes every byte to the
    value the definition gives, and the quantiser picks, for every element, the representable value nearest to
    x / scale (ties to the even mantissa), with scale = absmax / 448; the round trip error is at most half a step
    of the format at that magnitude."""
    table = torch.tensor([_e4m3_value(b) for b in range(256)], dtype=torch.float64)
    dec = torch.arange(256, dtype=torch.uint8).view(torch.float8_e4m3fn).double()
    finite = ~torch.isnan(table)
    assert torch.equal(dec[finite], table[finite]) and bool(torch.isnan(dec[~finite]).all())
    assert float(table[finite].max()) == 448.0
    g = torch.Generator().manual_seed(16)
    x = (torch.randn(5, 4, 64, generator=g) * torch.tensor([1e-3, 1.0, 37.0, 1e3]).view(1, 4, 1)).bfloat16()
    q, s = O.quantize_kv_fp8(x)
    assert q.dtype == torch.float8_e4m3fn and s.dtype == torch.float32
    assert torch.equal(s, x.float().abs().amax(-1) / 448.0)
    y = (x.float() / s.unsqueeze(-1)).double()                      # the quotients, exactly representable in fp64
    pos = table[:127]                                                # non-negative finite values, ascending
    codes = q.view(torch.uint8).long()
    for yy, cc in zip(y.flatten().tolist(), codes.flatten().tolist()):
        d = (pos - abs(yy)).abs()
        best = float(d.min())
        cands = [i for i in range(127) if float(d[i]) == best]
        want = cands[0] if len(cands) == 1 else [i for i in cands if i % 2 == 0][0]   # tie: even mantissa
        assert (cc & 127) == want and ((cc >> 7) == (1 if yy < 0 else 0) or want == 0), (yy, cc, want)
    assert int((codes & 127).max()) == 126                           # every row reaches the format's maximum, 448
    back = O.dequantize_kv_fp8(q, s)
    step = torch.where(y.abs() >= 2.0 ** -6, 2.0 ** (torch.floor(torch.log2(y.abs().clamp_min(2.0 ** -6))) - 3), torch.tensor(2.0 ** -9, dtype=torch.float64))
    # (the quotient and the product back are fp32 operations: a few 2^-24 of |x| on top of the format's half step)
    assert bool(((back.double() - x.double()).abs() <= 0.5 * step * s.unsqueeze(-1).double() + 4e-7 * x.double().abs() + 1e-30).all())
    z, sz = O.quantize_kv_fp8(torch.zeros(2, 8))
    assert int(z.view(torch.uint8).max()) == 0 and float(sz.max()) == 0.0


def test_fp16_conversions_in_c_match_torch():
    g = torch.Generator().manual_seed(15)
    vals = torch.cat([torch.randn(2000, generator=g) * 10 ** torch.randint(-9, 6, (2000,), generator=g).float(),
                      torch.tensor([0.0, -0.0, 65504.0, 65519.9, 65520.0, 1e-8, 6e-8, 6.1e-5, float("inf")])])
    L = brute.lib()
    for v in vals.tolist():
        want = torch.tensor(v, dtype=torch.float32).half().view(torch.int16).item() & 0xFFFF
        assert L.brute_f32_to_f16(v) == want, v
        wantb = torch.tensor(v, dtype=torch.float32).bfloat16().view(torch.int16).item() & 0xFFFF
        assert L.brute_f32_to_bf16(v) == wantb, v
    for h in range(0, 65536, 7):
        f = L.brute_f16_to_f32(h)
        t = torch.tensor(h if h < 32768 else h - 65536, dtype=torch.int16).view(torch.float16).float().item()
        assert (math.isnan(f) and math.isnan(t)) or f == t


def test_indexer_scores_pins():
    """Triple loop on a tiny case; one head of weight 1 is q . k; without the intermediate rounding the
    weighted sum is linear in q."""
    torch.manual_seed(5)
    H, D, bs = 16, 128, 16
    lens, clens = [3, 1], [5, 20]
    batch = 2
    MB = max((l + c + bs - 1) // bs for l, c in zip(lens, clens))
    T = sum(lens)
    q = torch.randn(T, H, D).bfloat16()
    w = torch.randn(T, D + H).bfloat16()
    kc = torch.randn(batch * MB + 1, bs, D).bfloat16()
    perm = torch.randperm(batch * MB + 1)[:batch * MB].to(torch.int32)
    qsl = torch.tensor([0, 3], dtype=torch.int32)
    args = (qsl, torch.tensor(lens, dtype=torch.int32), torch.tensor(clens, dtype=torch.int32), perm, H, D, bs, batch, MB)
    got = O.indexer_scores_ref(q, kc, w, *args, round_heads=False)
    # brute force
    for i in range(batch):
        for r in range(lens[i]):
            t = int(qsl[i]) + r
            for j in range(clens[i] + lens[i]):
                row = kc[int(perm[i * MB + j // bs]), j % bs].float()
                acc = 0.0
                for h in range(H):
                    acc += float(w[t, D + h]) * float((q[t, h].float() * row).sum())
                assert abs(acc - float(got[i][r, j])) <= 1e-3 * max(1.0, abs(acc))
    # linearity: (sum_h w_h q_h) . k
    for i in range(batch):
        s = int(qsl[i])
        qw = torch.einsum("shd,sh->sd", q[s:s + lens[i]].double(), w[s:s + lens[i], D:].double())
        k = O.gather_paged(kc, perm.view(batch, MB)[i].tolist(), clens[i] + lens[i]).double()
        torch.testing.assert_close(got[i].double(), qw @ k.T, rtol=1e-4, atol=1e-3)
    # one head with weight 1, the others 0: the rounded product itself
    w1 = torch.zeros_like(w)
    w1[:, D + 3] = 1.0
    one = O.indexer_scores_ref(q, kc, w1, *args)
    k0 = O.gather_paged(kc, perm.view(batch, MB)[0].tolist(), clens[0] + lens[0]).float()
    torch.testing.assert_close(one[0], (q[:3, 3].float() @ k0.T).bfloat16().float(), rtol=0, atol=0)
    # the rounding of the per-head products moves the result by no more than a 16-bit rounding of each term
    rounded = O.indexer_scores_ref(q, kc, w, *args)
    for i in range(batch):
        bound = (w[int(qsl[i]):int(qsl[i]) + lens[i], D:].float().abs().sum(-1, keepdim=True)) * 2.0 ** -8 * 40
        assert ((rounded[i] - got[i]).abs() <= bound).all()


def test_indexer_topk_pins():
    torch.manual_seed(6)
    sc = [torch.randn(4, 50).bfloat16().float(), torch.randn(2, 7)]
    res = O.indexer_topk_ref(sc, 10)
    for s, rows in zip(sc, res):
        for r, sel in enumerate(rows):
            n = s.shape[1]
            assert sel == sorted(set(sel)) and len(sel) == min(10, n)
            if n > 10:
                rest = [j for j in range(n) if j not in sel]
                assert min(float(s[r, j]) for j in sel) >= max(float(s[r, j]) for j in rest)
                # ties at the threshold go to the lower positions
                thr = min(float(s[r, j]) for j in sel)
                ties_in = [j for j in sel if float(s[r, j]) == thr]
                ties_out = [j for j in rest if float(s[r, j]) == thr]
                assert not ties_out or max(ties_in) < min(ties_out)
                top = torch.topk(s[r], 10).values
                assert sorted(float(s[r, j]) for j in sel) == sorted(top.tolist())


def test_qk_rms_norm_pins():
    torch.manual_seed(8)
    nH, nKV, d = 3, 2, 16
    x = torch.randn(5, (nH + 2 * nKV) * d).bfloat16()
    wq, wk = torch.randn(d).bfloat16(), torch.randn(d).bfloat16()
    bq = torch.randn(d).bfloat16()
    got = O.qk_rms_norm_ref(x, wq, bq, wk, None, 1e-6, d, nH, d, nKV, nH * d)
    # V columns untouched; every Q / K vector by a plain Python loop in double precision
    assert torch.equal(got[:, (nH + nKV) * d:], x[:, (nH + nKV) * d:])
    for t in range(5):
        for h in range(nH + nKV):
            v = x[t, h * d:(h + 1) * d].double()
            w = (wq if h < nH else wk).double()
            b = bq.double() if h < nH else torch.zeros(d, dtype=torch.double)
            ref = v / math.sqrt(float((v * v).sum()) / d + 1e-6) * w + b
            torch.testing.assert_close(got[t, h * d:(h + 1) * d].double(), ref, rtol=2 ** -7, atol=1e-6)
    # closed form: equal entries c -> sign(c) * w + b (eps negligible)
    c = torch.full((1, (nH + 2 * nKV) * d), -3.0).bfloat16()
    one = O.qk_rms_norm_ref(c, wq, bq, wk, None, 1e-12, d, nH, d, nKV, nH * d)
    torch.testing.assert_close(one[0, :d].float(), (-wq.float() + bq.float()).bfloat16().float(), rtol=2 ** -7, atol=1e-6)
    # the whole-segment form (one vector per segment) differs from the per-head form
    full = O.qk_rms_norm_ref(x, torch.ones(nH * d).bfloat16(), None, torch.ones(nKV * d).bfloat16(), None, 1e-6,
                             nH * d, 1, nKV * d, 1, nH * d)
    torch.testing.assert_close(full[:, :nH * d].float().pow(2).mean(-1), torch.ones(5), rtol=2e-2, atol=0)


def test_mla_forward_equals_the_naive_model_form():
    """The layer composition (projection, norms, rope, absorbed attention over the paged cache, output
    projection) must equal the textbook model form of xlite/tests/models/deepseek_v3.py:656-674: per-head keys
    k = [W_UK kv | k_pe], values v = W_UV^T kv, rope as a complex product, recomputed here from the whole
    token history in float32 with no paging, no absorption and no cache."""
    g = torch.Generator().manual_seed(31)
    H, ql, kvl, nope, rope, vd, hid, bs = 3, 12, 8, 6, 4, 5, 10, 4
    scale = (nope + rope) ** -0.5
    r = lambda *s: torch.randn(*s, generator=g)
    wa, wqb, wuk_t, wuv, wo = r(hid, ql + kvl + rope) * 0.3, r(ql, H * (nope + rope)) * 0.3, r(H, nope, kvl), r(H, kvl, vd), r(H * vd, hid)
    qn, kn = 1 + 0.1 * r(ql), 1 + 0.1 * r(kvl)
    ang = torch.outer(torch.arange(64).float(), 1.0 / (100.0 ** (torch.arange(0, rope, 2).float() / rope)))
    freqs = torch.polar(torch.ones_like(ang), ang)                     # complex64 [max_pos, rope / 2]
    prompts = [7, 2, 9]
    tables = [[5, 1, 9], [0, 7, 3], [2, 8, 4]]
    kc, pc = torch.zeros(10, bs, kvl), torch.zeros(10, bs, rope)
    history = [torch.zeros(0, hid) for _ in prompts]
    cached = [0] * len(prompts)

    def rms(x, w):
        return x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + 1e-6) * w

    def crope(x, pos):                                                  # interleaved pairs -> complex product
        xc = torch.view_as_complex(x.reshape(*x.shape[:-1], -1, 2).contiguous()) * freqs[pos].reshape(len(pos), *([1] * (x.dim() - 2)), -1)
        return torch.view_as_real(xc).flatten(-2)

    for step in range(3):
        lens = prompts if step == 0 else [1] * len(prompts)
        hidden = r(sum(lens), hid)
        got = O.mla_forward_ref(hidden, wa, qn, kn, wqb, wuk_t, wuv, wo, kc, pc, lens, cached, tables, freqs, H, ql, kvl,
                                nope, rope, vd, bs, scale)
        off = 0
        for i, n in enumerate(lens):
            history[i] = torch.cat([history[i], hidden[off:off + n]])
            x = history[i]
            L = x.shape[0]
            pos = torch.arange(L)
            a = x @ wa
            q = (rms(a[:, :ql], qn) @ wqb).view(L, H, nope + rope)
            q_pe = crope(q[..., nope:], pos)
            kv = rms(a[:, ql:ql + kvl], kn)
            k_pe = crope(a[:, ql + kvl:], pos)
            k_nope = torch.einsum("tc,hdc->thd", kv, wuk_t)
            v = torch.einsum("tc,hcv->thv", kv, wuv)
            s = (torch.einsum("shd,thd->hst", q[..., :nope], k_nope) + torch.einsum("shr,tr->hst", q_pe, k_pe)) * scale
            s = s + torch.full((L, L), float("-inf")).triu(1)
            o = torch.einsum("hst,thv->shv", torch.softmax(s, -1), v).reshape(L, -1) @ wo
            assert torch.allclose(got[off:off + n], o[L - n:], atol=2e-4, rtol=2e-4), "step %d sequence %d" % (step, i)
            off += n
        cached = [c + l for c, l in zip(cached, lens)]


def test_layernorm_muls_and_general_rope_pins():
    g = torch.Generator().manual_seed(41)
    x = torch.randn(5, 40, generator=g)
    w, b = torch.randn(24, generator=g), torch.randn(24, generator=g)
    # library routine on the normalised columns; a constant row normalises to the bias
    want = torch.nn.functional.layer_norm(x[:, :24], (24,), w, b, 1e-6)
    assert torch.allclose(O.layernorm_ref(x, w, b, 1e-6, 24), want, atol=1e-6, rtol=1e-5)
    assert torch.allclose(O.layernorm_ref(torch.full((2, 30), 3.25), w, b, 1e-6, 24), b.expand(2, 24), atol=1e-5)
    # muls: exact for a power of two, other columns untouched
    xb = torch.randn(4, 16, generator=g).bfloat16()
    y = O.muls_ref(xb, 0.5, 4, 8)
    assert torch.equal(y[:, 4:12].float(), xb[:, 4:12].float() * 0.5) and torch.equal(y[:, :4], xb[:, :4]) and torch.equal(y[:, 12:], xb[:, 12:])
    # the general rope: on the last columns it is rope_complex_ref; at offset 0 it is the complex product
    T, H, step, rope = 6, 3, 20, 8
    inp = torch.randn(T, H * step, generator=g).bfloat16()
    ang = torch.randn(32, rope // 2, generator=g)
    freqs = torch.polar(torch.ones_like(ang), ang)
    pos = torch.randint(0, 32, (T,), generator=g)
    a = O.rope_complex_and_cache_ref(H, step, rope, step - rope, 0, inp, freqs, pos)
    assert torch.equal(a, O.rope_complex_ref(H, step, rope, inp, freqs, pos))
    z = torch.view_as_complex(inp.view(T, H, step)[..., :rope].double().reshape(T, H, rope // 2, 2)) * freqs[pos].to(torch.complex128).unsqueeze(1)
    got = O.rope_complex_and_cache_ref(H, step, rope, 0, 0, inp, freqs, pos).double()
    assert torch.allclose(got[..., :rope // 2], z.real, atol=2e-2, rtol=1e-2) and torch.allclose(got[..., rope // 2:], z.imag, atol=2e-2, rtol=1e-2)
    # the cache form: rotated columns, then the rest of the vdim columns unchanged, at the slot; nothing else
    bs, vdim = 4, 12
    one = torch.randn(T, step, generator=g).bfloat16()
    cache = torch.full((3, bs, vdim), 9.0).bfloat16()
    slots = torch.tensor([5, 0, 11, 7, 2, 9], dtype=torch.int32)
    O.rope_complex_and_cache_ref(1, step, rope, 2, vdim, one, freqs, pos, bs, cache, slots)
    rot = O.rope_complex_and_cache_ref(1, step, rope, 2, 0, one, freqs, pos)
    flat = cache.view(-1, vdim)
    for t in range(T):
        assert torch.equal(flat[slots[t], :rope], rot[t, 0]) and torch.equal(flat[slots[t], rope:], one[t, 2 + rope:2 + vdim])
    untouched = [i for i in range(3 * bs) if i not in slots.tolist()]
    assert bool((flat[untouched] == 9.0).all())


def test_indexer_forward_selects_the_textbook_sets():
    """The indexer composition (projection, LayerNorm, rope into the paged index cache, query projection, rope,
    scaled head weights, scores, top-k) against the textbook form of xlite/tests/models/deepseek_v3.py:543-568
    recomputed from the whole token history in float32 without cache or paging (its rotate_activation is an
    orthogonal map applied to q and k alike and cancels in q . k; the kernel path ranks every position of the
    sequence for every row, so the comparison runs on decode rows, where the golden has no mask either)."""
    g = torch.Generator().manual_seed(43)
    hid, ql, nH, D, rope, bs, topk = 12, 10, 4, 16, 8, 4, 6
    r = lambda *s: torch.randn(*s, generator=g)
    wkw, kn, kb, wqb = r(hid, D + nH) * 0.4, 1 + 0.1 * r(D), 0.1 * r(D), r(ql, nH * D) * 0.4
    ang = torch.outer(torch.arange(64).float(), 1.0 / (50.0 ** (torch.arange(0, rope, 2).float() / rope)))
    freqs = torch.polar(torch.ones_like(ang), ang)
    tables = [[4, 1, 7, 2], [0, 6, 3, 5]]
    cache = torch.zeros(8, bs, D)
    prompts = [9, 13]
    hist_x = [torch.zeros(0, hid), torch.zeros(0, hid)]
    cached = [0, 0]

    def crope(x, pos):
        xc = torch.view_as_complex(x.reshape(*x.shape[:-1], -1, 2).contiguous()) * freqs[pos].reshape(len(pos), *([1] * (x.dim() - 2)), -1)
        return torch.view_as_real(xc).flatten(-2)

    for step in range(3):
        lens = prompts if step == 0 else [1, 1]
        hidden, qc = r(sum(lens), hid), r(sum(lens), ql)
        meta = O.prepare_attn_ref(lens, cached, tables, bs)
        res = O.indexer_forward_ref(hidden, qc, wkw, kn, kb, wqb, cache, freqs, torch.tensor(meta["position"]),
                                    torch.tensor(meta["slot_mapping"], dtype=torch.int32),
                                    torch.tensor(meta["query_start_loc"], dtype=torch.int32), torch.tensor(lens, dtype=torch.int32),
                                    torch.tensor(cached, dtype=torch.int32), torch.from_numpy(meta["block_tables"]).flatten(), nH, D,
                                    rope, topk, bs, 2, meta["max_num_blocks"], 1e-6)
        off = 0
        for i, n in enumerate(lens):
            hist_x[i] = torch.cat([hist_x[i], hidden[off:off + n]])
            if step > 0:
                L = hist_x[i].shape[0]
                kwf = hist_x[i] @ wkw
                k = torch.nn.functional.layer_norm(kwf[:, :D], (D,), kn, kb, 1e-6)
                k = torch.cat([crope(k[:, :rope], torch.arange(L)), k[:, rope:]], -1)
                q = (qc[off:off + 1] @ wqb).view(1, nH, D)
                q = torch.cat([crope(q[..., :rope], torch.tensor([L - 1])), q[..., rope:]], -1)
                weights = kwf[L - 1:, D:] * nH ** -0.5
                index_score = torch.einsum("sht,sh->st", torch.einsum("shd,td->sht", q, k) * D ** -0.5, weights)
                want = sorted(index_score[0].topk(min(topk, L))[1].tolist())
                assert res[1][i][0] == want, "step %d sequence %d" % (step, i)
                assert torch.allclose(res[0][i][0], index_score[0], atol=1e-4, rtol=1e-4)
            off += n
        cached = [c + l for c, l in zip(cached, lens)]
