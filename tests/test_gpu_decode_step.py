"""`decode_step` (one call into the library: rope_and_cache, then attention) against the two separate calls on the
same inputs: the rotated rows, both caches and the output must agree bit for bit, for decode batches of several
shapes and for a chunked prefill batch; its argument checks run on the first call of a combination and refuse
what the separate calls refuse."""
import pytest
import torch

from gvirt_amd import workloads as W

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _both(rt, s, w, r):
    from gvirt_amd._C import attention, decode_step, rope_and_cache
    k0, v0, q0 = w["k_cache"].clone(), w["v_cache"].clone(), r["inout"].clone()
    rope_and_cache(rt, r["inout"], w["k_cache"], w["v_cache"], r["position"], r["cosin"], r["slot_mapping"], s.n_heads,
                   s.n_kv_heads, s.head_dim, s.head_dim, s.block_size, True)
    attention(rt, r["inout"], w["k_cache"], w["v_cache"], w["output"], w["query_start_loc"], w["lens"],
              w["cached_lens"], w["block_tables"], s.n_heads, s.n_kv_heads, s.head_dim, s.block_size, w["batch"],
              w["max_num_block"])
    rt.synchronize()
    want = [t.clone() for t in (r["inout"], w["k_cache"], w["v_cache"], w["output"])]
    w["k_cache"].copy_(k0); w["v_cache"].copy_(v0); r["inout"].copy_(q0); w["output"].fill_(5.0)
    for _ in range(2):   # the second call takes the cached plan
        w["k_cache"].copy_(k0); w["v_cache"].copy_(v0); r["inout"].copy_(q0); w["output"].fill_(5.0)
        decode_step(rt, r["inout"], w["k_cache"], w["v_cache"], w["output"], r["position"], r["cosin"],
                    r["slot_mapping"], w["query_start_loc"], w["lens"], w["cached_lens"], w["block_tables"], s.n_heads,
                    s.n_kv_heads, s.head_dim, s.head_dim, s.block_size, w["batch"], w["max_num_block"])
        rt.synchronize()
        for name, a, b in zip(("rows", "k_cache", "v_cache", "output"), want,
                              (r["inout"], w["k_cache"], w["v_cache"], w["output"])):
            assert torch.equal(a.view(torch.int16), b.view(torch.int16)), name


@pytest.mark.parametrize("shape,ctx", [(W.QWEN2_05B, [485, 17, 300, 731]), (W.LLAMA3_8B, [700, 3000, 129, 2048, 64, 1500, 4096, 33]),
                                       (W.LLAMA3_8B, [1])])
def test_decode_step_is_the_two_calls_bit_for_bit(rt, shape, ctx):
    w = W.gqa_decode(shape, ctx, 61, device=DEV)
    _both(rt, shape, w, W.rope_inputs(shape, w, 62))


def test_decode_step_on_a_prefill_chunk(rt):
    s = W.LLAMA3_8B
    w = W.gqa_prefill_chunk(s, [700, 300], 0, 2048, 63, device=DEV)
    T = w["qkv"].shape[0]
    g = torch.Generator(device=DEV).manual_seed(64)
    D, bs = s.head_dim, s.block_size
    inv = 1.0 / (10000.0 ** (torch.arange(0, D, 2, dtype=torch.float32, device=DEV) / D))
    ang = torch.outer(torch.arange(4096, dtype=torch.float32, device=DEV), inv)
    lens = w["lens"].tolist()
    pos = torch.cat([torch.arange(n, device=DEV) for n in lens]).to(torch.int64)
    tables = w["block_tables"].view(w["batch"], w["max_num_block"]).long()
    seq = torch.cat([torch.full((n,), i, device=DEV, dtype=torch.int64) for i, n in enumerate(lens)])
    r = dict(inout=(torch.randn(w["qkv"].shape, generator=g, device=DEV) * 0.5).to(s.dtype), position=pos,
             cosin=torch.cat([ang.cos(), ang.sin()], dim=-1).to(s.dtype),
             slot_mapping=(tables[seq, pos // bs] * bs + pos % bs).to(torch.int32))
    assert r["inout"].shape[0] == T
    _both(rt, s, w, r)


def test_decode_step_refuses_what_the_two_calls_refuse(rt):
    from gvirt_amd._C import decode_step
    s = W.QWEN2_05B
    w = W.gqa_decode(s, [100, 200], 65, device=DEV)
    r = W.rope_inputs(s, w, 66)
    args = lambda **kw: [kw.get("qkv", r["inout"]), w["k_cache"], w["v_cache"], kw.get("output", w["output"]),
                         kw.get("position", r["position"]), r["cosin"], r["slot_mapping"], w["query_start_loc"], w["lens"],
                         w["cached_lens"], w["block_tables"], s.n_heads, s.n_kv_heads, s.head_dim, s.head_dim,
                         s.block_size, w["batch"], w["max_num_block"]]
    decode_step(rt, *args())   # the combination is now known; the ones below are others
    with pytest.raises(RuntimeError, match="output shape mismatch"):
        decode_step(rt, *args(output=w["output"][:1]))
    with pytest.raises(RuntimeError, match="position"):
        decode_step(rt, *args(position=r["position"].to(torch.int32)))
    with pytest.raises(RuntimeError):
        decode_step(rt, *args(qkv=r["inout"].cpu()))
    with pytest.raises(RuntimeError, match="gptj"):
        decode_step(rt, *args(), is_neox=False)
