"""The model-level caller (gvirt_amd/mha.py: prepare_attn + MhaLayer) over several steps of a small batch:
one ragged prefill, then decode steps on growing caches, against the oracle's composition of the same pieces."""
import pytest
import torch

from oracle import xlite_oracle as O

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _cosin(rot, max_pos, dtype):
    fr = torch.outer(torch.arange(max_pos).float(), 1.0 / (10000.0 ** (torch.arange(0, rot, 2).float() / rot)))
    return torch.cat([fr.cos(), fr.sin()], -1).to(dtype)


@pytest.mark.parametrize("qk_norm,head_dim,rot_dim", [(False, 128, 128), (True, 128, 128), (True, 256, 64)])
def test_mha_layer_prefill_then_decode_steps(rt, qk_norm, head_dim, rot_dim):
    """The last case is the Qwen3.5 attention shape (xlite/tests/models/qwen3_5.py:67-71: 8 / 2 heads of 256 with
    qk-norm, a rotary span of a quarter of the head)."""
    from gvirt_amd.mha import MhaConfig, MhaLayer, prepare_attn
    g = torch.Generator().manual_seed(77)
    dt = torch.bfloat16
    cfg = MhaConfig(hidden=256, n_heads=8, n_kv_heads=2, head_dim=head_dim, rot_dim=rot_dim, block_size=16, qk_norm=qk_norm)
    cols = (cfg.n_heads + 2 * cfg.n_kv_heads) * cfg.head_dim
    wqkv = (torch.randn(cfg.hidden, cols, generator=g) * cfg.hidden ** -0.5).to(dt)
    wo = (torch.randn(cfg.n_heads * cfg.head_dim, cfg.hidden, generator=g) * (cfg.n_heads * cfg.head_dim) ** -0.5).to(dt)
    qn = (1 + 0.1 * torch.randn(cfg.head_dim, generator=g)).to(dt) if qk_norm else None
    kn = (1 + 0.1 * torch.randn(cfg.head_dim, generator=g)).to(dt) if qk_norm else None
    prompts, steps = [37, 5, 64], 3
    max_len = max(prompts) + steps
    blocks_per_seq = (max_len + cfg.block_size - 1) // cfg.block_size
    NB = len(prompts) * blocks_per_seq + 3
    perm = torch.randperm(NB, generator=g).tolist()
    tables = [perm[i * blocks_per_seq:(i + 1) * blocks_per_seq] for i in range(len(prompts))]
    cosin = _cosin(cfg.rot_dim, 256, dt)
    kc_ref = torch.zeros(NB, cfg.block_size, cfg.n_kv_heads, cfg.head_dim).to(dt)
    vc_ref = torch.zeros_like(kc_ref)
    kc, vc = kc_ref.to(DEV), vc_ref.to(DEV)
    mv = lambda t: None if t is None else t.to(DEV)
    layer = MhaLayer(cfg, wqkv.to(DEV), wo.to(DEV), q_norm=mv(qn), k_norm=mv(kn))
    cached = [0] * len(prompts)
    for step in range(steps + 1):
        lens = prompts if step == 0 else [1] * len(prompts)
        hidden = torch.randn(sum(lens), cfg.hidden, generator=g).to(dt)
        meta = prepare_attn(lens, cached, tables, cfg.block_size, DEV)
        assert meta.is_decode == (step > 0) and meta.batched_tokens == sum(lens)
        got = layer.forward(rt, hidden.to(DEV), kc, vc, meta, cosin.to(DEV))
        rt.synchronize()
        ref = O.mha_forward_ref(hidden, wqkv, wo, kc_ref, vc_ref, lens, cached, tables, cosin, cfg.n_heads, cfg.n_kv_heads,
                                cfg.head_dim, cfg.rot_dim, cfg.block_size, qn, kn, cfg.norm_eps)
        err = (got.float().cpu() - ref.float()).abs()
        assert float(err.max()) <= 3e-2 and float(err.mean()) <= 3e-3, "step %d: max %g mean %g" % (step, float(err.max()), float(err.mean()))
        # the caches agree up to a 16-bit unit of the projected rows (the two GEMMs sum in different orders)
        torch.testing.assert_close(kc.float().cpu(), kc_ref.float(), rtol=2 ** -7, atol=2e-2)
        torch.testing.assert_close(vc.float().cpu(), vc_ref.float(), rtol=2 ** -7, atol=2e-2)
        cached = [c + l for c, l in zip(cached, lens)]
