"""`decode_step` (one call into the library: rope_and_cache, then attention) against the two separate calls on the
same inputs: the rotated rows, both caches and the output must agree bit for bit, for decode batches of several
shapes and for a chunked prefill batch; its argument checks run on the first call of a combination and refuse
what the separate calls refuse."""
import pytest
import torch

from gvirt_amd import workloads as W

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _both(rt, s, w, r, rot_dim=None, **rope_kw):
    from gvirt_amd._C import attention, decode_step, rope_and_cache
    rot_dim = rot_dim or s.head_dim
    k0, v0, q0 = w["k_cache"].clone(), w["v_cache"].clone(), r["inout"].clone()
    rope_and_cache(rt, r["inout"], w["k_cache"], w["v_cache"], r["position"], r["cosin"], r["slot_mapping"], s.n_heads,
                   s.n_kv_heads, s.head_dim, rot_dim, s.block_size, True, **rope_kw)
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
                    s.n_kv_heads, s.head_dim, rot_dim, s.block_size, w["batch"], w["max_num_block"], **rope_kw)
        rt.synchronize()
        for name, a, b in zip(("rows", "k_cache", "v_cache", "output"), want,
                              (r["inout"], w["k_cache"], w["v_cache"], w["output"])):
            assert torch.equal(a.view(torch.int16), b.view(torch.int16)), name


@pytest.mark.parametrize("shape,ctx", [(W.QWEN2_05B, [485, 17, 300, 731]), (W.LLAMA3_8B, [700, 3000, 129, 2048, 64, 1500, 4096, 33]),
                                       (W.LLAMA3_8B, [1])])
def test_decode_step_is_the_two_calls_bit_for_bit(rt, shape, ctx):
    w = W.gqa_decode(shape, ctx, 61, device=DEV)
    _both(rt, shape, w, W.rope_inputs(shape, w, 62))


@pytest.mark.parametrize("shape,ctx", [
    (W.LLAMA3_8B, [100, 33, 256, 1]),                                            # head_dim 128, a workgroup per (row, kv head)
    (W.LLAMA3_8B, [(37 * i) % 255 + 1 for i in range(40)]),                      # ... a workgroup per row, all 8 kv heads
    (W.QWEN2_05B, [(53 * i) % 511 + 1 for i in range(150)]),                     # head_dim 64, more rows than compute units / kv heads
    (W.QWEN2_05B, [(29 * i) % 300 + 1 for i in range(700)]),                     # more sequences than workgroups: several per workgroup
    (W.GqaShape("g3", 12, 3, 64, 16, torch.float16), [1, 16, 17, 200, 5]),       # 3 kv heads, fp16, block size 16
    (W.GqaShape("g12", 24, 12, 128, 32, torch.bfloat16), [9, 130, 64]),          # two passes of kv heads
])
def test_one_launch_steps_of_short_contexts(rt, shape, ctx):
    """Decode batches whose rows the attention kernel takes whole are one launch: the kernel rotates and stores a
    sequence's row before it walks it. Bit for bit the two calls."""
    w = W.gqa_decode(shape, ctx, 71, device=DEV)
    _both(rt, shape, w, W.rope_inputs(shape, w, 72))


def test_one_launch_step_with_partial_rotary_span_and_mrope(rt):
    s = W.GqaShape("p", 16, 4, 128, 64, torch.bfloat16)
    w = W.gqa_decode(s, [77, 300, 12], 73, device=DEV)
    r = W.rope_inputs(s, w, 74)
    r["cosin"] = torch.cat([r["cosin"][:, :32], r["cosin"][:, 64:96]], dim=1).contiguous()   # rot_dim 64: 32 cos | 32 sin
    _both(rt, s, w, r, rot_dim=64)
    r = W.rope_inputs(s, w, 75)
    g = torch.Generator(device=DEV).manual_seed(76)
    pos3 = torch.stack([r["position"], torch.randint(0, 500, (3,), generator=g, device=DEV),
                        torch.randint(0, 500, (3,), generator=g, device=DEV)]).contiguous()
    r["position"] = pos3
    _both(rt, s, w, r, mrope_mask_h=0x00000000FFFF0000, mrope_mask_w=0x0000FFFF00000000)


def test_one_launch_step_with_several_rows_in_a_sequence(rt):
    """A batch with as many rows as sequences need not be one row each: a sequence with three rows (a short
    speculative run) next to sequences with none. A sequence's later rows read the cache rows of its earlier ones."""
    s = W.QWEN2_05B
    lens, cached = [3, 0, 1, 0, 1], [40, 7, 299, 0, 0]
    w = W.gqa_decode(s, [c + max(l, 1) for l, c in zip(lens, cached)], 77, device=DEV)
    T = sum(lens)
    assert T == w["batch"]
    w["lens"] = torch.tensor(lens, dtype=torch.int32, device=DEV)
    w["cached_lens"] = torch.tensor(cached, dtype=torch.int32, device=DEV)
    starts = [sum(lens[:i]) for i in range(len(lens))]
    w["query_start_loc"] = torch.tensor(starts, dtype=torch.int32, device=DEV)
    r = W.rope_inputs(s, w, 78)
    seq = [i for i, n in enumerate(lens) for _ in range(n)]
    pos = [cached[i] + j for i, n in enumerate(lens) for j in range(n)]
    tables = w["block_tables"].view(w["batch"], w["max_num_block"]).long()
    r["position"] = torch.tensor(pos, dtype=torch.int64, device=DEV)
    r["slot_mapping"] = torch.tensor([int(tables[i, p // s.block_size]) * s.block_size + p % s.block_size
                                      for i, p in zip(seq, pos)], dtype=torch.int32, device=DEV)
    _both(rt, s, w, r)


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
