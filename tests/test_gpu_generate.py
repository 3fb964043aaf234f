"""Generation through the operator module under its reference name: `gvirt_amd.install_as_xlite()`, then
`from xlite._C import ...` as the reference's scripts do (xlite/tests/kernels/attention.py:17, :222-225), a small
multi-layer decoder stack (gvirt_amd/generate.py) doing a ragged prefill and greedy decode steps with the step
metadata advancing through `prepare_attn`, checked token by token against the oracle's composition of the same
layers (teacher-forced with the tokens the GPU chose: at every step the chosen token's oracle logit must be the
oracle's maximum up to the 16-bit noise of the stack, and nearly all choices must be the oracle's own)."""
import pytest
import torch

from oracle import xlite_oracle as O

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
LOGIT_SLACK = 0.06   # logits are O(1); the GPU and CPU stacks differ by 16-bit roundings of every stage


def _norm(x, w, eps=1e-6):
    xf = x.float()
    return (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps) * w.float()).to(x.dtype)


def _mha_weights(g, n_layers, hidden, n_heads, n_kv, d, vocab, dt):
    r = lambda *s: torch.randn(*s, generator=g)
    cols = (n_heads + 2 * n_kv) * d
    return dict(wqkv=[(r(hidden, cols) * hidden ** -0.5).to(dt) for _ in range(n_layers)],
                wo=[(r(n_heads * d, hidden) * (n_heads * d) ** -0.5).to(dt) for _ in range(n_layers)],
                norms=[(1 + 0.1 * r(hidden)).to(dt) for _ in range(n_layers + 1)],
                embed=r(vocab, hidden).to(dt), lm_head=(r(hidden, vocab) * hidden ** -0.5).to(dt))


def _cosin(rot, max_pos, dtype):
    fr = torch.outer(torch.arange(max_pos).float(), 1.0 / (10000.0 ** (torch.arange(0, rot, 2).float() / rot)))
    return torch.cat([fr.cos(), fr.sin()], -1).to(dtype)


class OracleMhaStack:
    """The same stack on the CPU from the oracle's layer composition, with its own caches."""

    def __init__(self, w, n_heads, n_kv, d, bs, blocks_per_seq, max_batch, cosin):
        self.w, self.n_heads, self.n_kv, self.d, self.bs, self.bps, self.cosin = w, n_heads, n_kv, d, bs, blocks_per_seq, cosin
        nb = max_batch * blocks_per_seq
        dt = w["embed"].dtype
        self.caches = [(torch.zeros(nb, bs, n_kv, d, dtype=dt), torch.zeros(nb, bs, n_kv, d, dtype=dt)) for _ in w["wqkv"]]

    def step(self, flat_tokens, lens, cached, live):
        tables = [[i * self.bps + b for b in range(self.bps)] for i in live]
        x = self.w["embed"][torch.tensor(flat_tokens).long()]
        for li, (kc, vc) in enumerate(self.caches):
            h = _norm(x, self.w["norms"][li])
            x = x + O.mha_forward_ref(h, self.w["wqkv"][li], self.w["wo"][li], kc, vc, lens, cached, tables, self.cosin,
                                      self.n_heads, self.n_kv, self.d, self.d, self.bs)
        x = _norm(x, self.w["norms"][-1])
        ends = [sum(lens[: i + 1]) - 1 for i in range(len(lens))]
        return (x[torch.tensor(ends)].float() @ self.w["lm_head"].float())


def _check_replay(oracle_step, prompts, completions, eos, max_new=None, min_checked=16):
    """Feed the oracle the tokens the GPU run consumed and compare the choices step by step."""
    n = len(prompts)
    cached = [0] * n
    pending = [list(p) for p in prompts]
    produced = [0] * n
    agree = total = 0
    while sum(len(p) for p in pending):
        lens = [len(p) for p in pending]
        live = [i for i in range(n) if lens[i]]
        logits = oracle_step([t for p in pending for t in p], [lens[i] for i in live], [cached[i] for i in live], live)
        for row, i in enumerate(live):
            cached[i] += lens[i]
            pending[i] = []
            if produced[i] < len(completions[i]):
                tok = completions[i][produced[i]]
                top = float(logits[row].max())
                assert float(logits[row, tok]) >= top - LOGIT_SLACK, "sequence %d token %d: logit %g, best %g" % (
                    i, produced[i], float(logits[row, tok]), top)
                agree += int(int(logits[row].argmax()) == tok)
                total += 1
                produced[i] += 1
                pending[i] = [tok]
            elif max_new is not None and len(completions[i]) < max_new:
                # the run stopped this sequence here: the end token must have been (within the noise) the best one
                assert float(logits[row, eos]) >= float(logits[row].max()) - LOGIT_SLACK, "sequence %d did not end" % i
    assert total >= min_checked and agree >= 0.9 * total, (agree, total)


def test_operators_under_the_reference_module_name(rt):
    """`from xlite._C import ...` with the reference test's positional call shapes
    (xlite/tests/kernels/attention.py:222-225, rope_and_cache.py:105-108)."""
    import gvirt_amd
    gvirt_amd.install_as_xlite()
    from xlite._C import Runtime, attention, rope_and_cache, ModelAttnMeta, get_tile_size_of_cached_kv  # noqa: F401
    import xlite._C as xc
    from gvirt_amd import _C
    assert xc is _C and Runtime is _C.Runtime
    from test_gpu_attention import generic_case, oracle_attention, check
    w = generic_case(51, [1, 1, 1], [300, 17, 129], 8, 2, 128, 128, torch.bfloat16, rms=True)
    xrt = Runtime(0, 64)
    d = {k: (v.to(DEV) if isinstance(v, torch.Tensor) else v) for k, v in w.items()}
    attention(xrt, d["qkv"], d["k_cache"], d["v_cache"], d["output"], d["query_start_loc"], d["lens"], d["cached_lens"],
              d["block_tables"], 8, 2, 128, 128, 3, w["max_num_block"])
    check(d["output"].float().cpu(), oracle_attention(w))
    # the flash variant's two extra positional arguments are accepted (hints here)
    d["output"].zero_()
    attention(xrt, d["qkv"], d["k_cache"], d["v_cache"], d["output"], d["query_start_loc"], d["lens"], d["cached_lens"],
              d["block_tables"], 8, 2, 128, 128, 3, w["max_num_block"], True, 1024)
    check(d["output"].float().cpu(), oracle_attention(w))


@pytest.mark.parametrize("n_layers", [2, 4])
def test_generation_mha_stack_ragged_prefill_then_decode(n_layers):
    import gvirt_amd
    gvirt_amd.install_as_xlite()
    from xlite._C import Runtime
    from gvirt_amd.generate import DecoderModel, generate_ragged
    from gvirt_amd.mha import MhaConfig, MhaLayer
    g = torch.Generator().manual_seed(5 + n_layers)
    dt = torch.bfloat16
    hidden, n_heads, n_kv, d, bs, vocab, max_seq = 256, 8, 2, 128, 16, 384, 96
    w = _mha_weights(g, n_layers, hidden, n_heads, n_kv, d, vocab, dt)
    cosin = _cosin(d, 128, dt)
    cfg = MhaConfig(hidden=hidden, n_heads=n_heads, n_kv_heads=n_kv, head_dim=d, rot_dim=d, block_size=bs)
    rt = Runtime(0, 64)
    layers = [MhaLayer(cfg, w["wqkv"][i].to(DEV), w["wo"][i].to(DEV)) for i in range(n_layers)]
    prompts = [[int(x) for x in torch.randint(0, vocab, (n,), generator=g)] for n in (37, 5, 64, 12)]
    model = DecoderModel(rt, layers, [x.to(DEV) for x in w["norms"]], w["embed"].to(DEV), w["lm_head"].to(DEV), cosin.to(DEV),
                         max_batch=len(prompts), max_seq_len=max_seq)
    eos = vocab   # never produced: every sequence runs its full length
    completions, steps = generate_ragged(model, prompts, 18, eos)
    assert steps == 18 and all(len(c) == 18 for c in completions)
    oracle = OracleMhaStack(w, n_heads, n_kv, d, bs, model.blocks_per_seq, len(prompts), cosin)
    _check_replay(oracle.step, prompts, completions, eos)
    # a sequence that produces the end token takes no further part: its length is 0 in the later steps (fewer
    # query rows than sequences), and the others continue as before
    eos = completions[1][3]
    model2 = DecoderModel(rt, layers, [x.to(DEV) for x in w["norms"]], w["embed"].to(DEV), w["lm_head"].to(DEV), cosin.to(DEV),
                          max_batch=len(prompts), max_seq_len=max_seq)
    again, _ = generate_ragged(model2, prompts, 18, eos)
    assert len(again[1]) <= 3 and all(eos not in a for a in again)
    oracle2 = OracleMhaStack(w, n_heads, n_kv, d, bs, model.blocks_per_seq, len(prompts), cosin)
    _check_replay(oracle2.step, prompts, again, eos, max_new=18)


def test_generation_reference_loop_rectangular_prompts():
    """`generate` of xlite/tests/generate.py:52-103: prefill of the shortest prompt's length, then one position per
    step with the longer prompts' tokens forced; against the ragged run of the same model (same caches, same
    arithmetic per row, so the continuations agree wherever both are unforced)."""
    import gvirt_amd
    gvirt_amd.install_as_xlite()
    from xlite._C import Runtime
    from gvirt_amd.generate import DecoderModel, generate, generate_ragged
    from gvirt_amd.mha import MhaConfig, MhaLayer
    g = torch.Generator().manual_seed(17)
    dt = torch.bfloat16
    hidden, n_heads, n_kv, d, bs, vocab, max_seq = 256, 14, 2, 64, 16, 300, 64
    w = _mha_weights(g, 2, hidden, n_heads, n_kv, d, vocab, dt)
    cfg = MhaConfig(hidden=hidden, n_heads=n_heads, n_kv_heads=n_kv, head_dim=d, rot_dim=d, block_size=bs)
    rt = Runtime(0, 64)
    prompts = [[int(x) for x in torch.randint(0, vocab, (n,), generator=g)] for n in (9, 5, 7)]

    def build():
        layers = [MhaLayer(cfg, w["wqkv"][i].to(DEV), w["wo"][i].to(DEV)) for i in range(2)]
        return DecoderModel(rt, layers, [x.to(DEV) for x in w["norms"]], w["embed"].to(DEV), w["lm_head"].to(DEV),
                            _cosin(d, 128, dt).to(DEV), max_batch=3, max_seq_len=max_seq)
    rect, steps = generate(build(), prompts, 16, vocab, 0.0)
    assert steps == 9 + 16 - 5 and all(len(c) == 16 for c in rect)
    ragged, _ = generate_ragged(build(), prompts, 16, vocab)
    same = sum(int(a == b) for ra, rb in zip(rect, ragged) for a, b in zip(ra, rb))
    assert same >= 0.9 * 48, same
    with pytest.raises(RuntimeError):
        generate(build(), prompts, 4, vocab, 0.7)


def test_generation_mla_stack_ragged_prefill_then_decode():
    import gvirt_amd
    gvirt_amd.install_as_xlite()
    from xlite._C import Runtime
    from gvirt_amd.generate import DecoderModel, generate_ragged
    from gvirt_amd.mla import MlaConfig, MlaLayer
    g = torch.Generator().manual_seed(23)
    dt = torch.bfloat16
    n_layers, hidden, n_heads, vocab, bs, max_seq = 2, 256, 16, 320, 32, 128
    cfg = MlaConfig(hidden=hidden, n_heads=n_heads, q_lora_rank=192, kv_lora_rank=512, nope_head_dim=128, rope_head_dim=64,
                    v_head_dim=128, block_size=bs, softmax_scale=192 ** -0.5)
    r = lambda *s: torch.randn(*s, generator=g)
    L = []
    for _ in range(n_layers):
        L.append(dict(wa=(r(hidden, cfg.q_lora_rank + cfg.kv_lora_rank + cfg.rope_head_dim) * hidden ** -0.5).to(dt),
                      wqb=(r(cfg.q_lora_rank, n_heads * (cfg.nope_head_dim + cfg.rope_head_dim)) * cfg.q_lora_rank ** -0.5).to(dt),
                      wuk_t=(r(n_heads, cfg.nope_head_dim, cfg.kv_lora_rank) * cfg.nope_head_dim ** -0.5).to(dt),
                      wuv=(r(n_heads, cfg.kv_lora_rank, cfg.v_head_dim) * cfg.kv_lora_rank ** -0.5).to(dt),
                      wo=(r(n_heads * cfg.v_head_dim, hidden) * (n_heads * cfg.v_head_dim) ** -0.5).to(dt),
                      qn=(1 + 0.1 * r(cfg.q_lora_rank)).to(dt), kn=(1 + 0.1 * r(cfg.kv_lora_rank)).to(dt)))
    norms = [(1 + 0.1 * r(hidden)).to(dt) for _ in range(n_layers + 1)]
    embed, lm_head = r(vocab, hidden).to(dt), (r(hidden, vocab) * hidden ** -0.5).to(dt)
    ang = torch.outer(torch.arange(256).float(), 1.0 / (10000.0 ** (torch.arange(0, 64, 2).float() / 64)))
    freqs = torch.polar(torch.ones_like(ang), ang)
    rt = Runtime(0, 64)
    layers = [MlaLayer(cfg, x["wa"].to(DEV), x["qn"].to(DEV), x["kn"].to(DEV), x["wqb"].to(DEV), x["wuk_t"].to(DEV),
                       x["wuv"].to(DEV), x["wo"].to(DEV)) for x in L]
    prompts = [[int(x) for x in torch.randint(0, vocab, (n,), generator=g)] for n in (70, 3, 33)]
    model = DecoderModel(rt, layers, [x.to(DEV) for x in norms], embed.to(DEV), lm_head.to(DEV), freqs.to(DEV),
                         max_batch=3, max_seq_len=max_seq)
    completions, steps = generate_ragged(model, prompts, 17, vocab)
    assert steps == 17
    bps = model.blocks_per_seq
    caches = [(torch.zeros(3 * bps, bs, 512, dtype=dt), torch.zeros(3 * bps, bs, 64, dtype=dt)) for _ in L]

    def oracle_step(toks, lens, cached, live):
        tables = [[i * bps + b for b in range(bps)] for i in live]
        x = embed[torch.tensor(toks).long()]
        for li, (kc, pc) in enumerate(caches):
            h = _norm(x, norms[li])
            w = L[li]
            x = x + O.mla_forward_ref(h, w["wa"], w["qn"], w["kn"], w["wqb"], w["wuk_t"], w["wuv"], w["wo"], kc, pc, lens, cached,
                                      tables, freqs, n_heads, cfg.q_lora_rank, cfg.kv_lora_rank, cfg.nope_head_dim,
                                      cfg.rope_head_dim, cfg.v_head_dim, bs, cfg.softmax_scale, cfg.norm_eps)
        x = _norm(x, norms[-1])
        ends = [sum(lens[: i + 1]) - 1 for i in range(len(lens))]
        return x[torch.tensor(ends)].float() @ lm_head.float()
    _check_replay(oracle_step, prompts, completions, vocab)
