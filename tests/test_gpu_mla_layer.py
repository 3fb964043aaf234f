"""The model-level MLA caller (gvirt_amd/mla.py: MlaLayer over prepare_attn) across several steps of a small
batch: one ragged prefill, then decode steps on growing latent caches, against the oracle's composition of the
same pieces (itself pinned against the textbook per-head model form in tests/test_oracle_pins.py)."""
import pytest
import torch

from oracle import xlite_oracle as O

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.mark.parametrize("n_heads,block_size", [(16, 64), (128, 32)])
def test_mla_layer_prefill_then_decode_steps(rt, n_heads, block_size):
    from gvirt_amd.mha import prepare_attn
    from gvirt_amd.mla import MlaConfig, MlaLayer
    g = torch.Generator().manual_seed(91)
    dt = torch.bfloat16
    cfg = MlaConfig(hidden=256, n_heads=n_heads, q_lora_rank=192, kv_lora_rank=512, nope_head_dim=128, rope_head_dim=64,
                    v_head_dim=128, block_size=block_size, softmax_scale=192 ** -0.5)
    r = lambda *s: torch.randn(*s, generator=g)
    wa = (r(cfg.hidden, cfg.q_lora_rank + cfg.kv_lora_rank + cfg.rope_head_dim) * cfg.hidden ** -0.5).to(dt)
    wqb = (r(cfg.q_lora_rank, n_heads * (cfg.nope_head_dim + cfg.rope_head_dim)) * cfg.q_lora_rank ** -0.5).to(dt)
    wuk_t = (r(n_heads, cfg.nope_head_dim, cfg.kv_lora_rank) * cfg.nope_head_dim ** -0.5).to(dt)
    wuv = (r(n_heads, cfg.kv_lora_rank, cfg.v_head_dim) * cfg.kv_lora_rank ** -0.5).to(dt)
    wo = (r(n_heads * cfg.v_head_dim, cfg.hidden) * (n_heads * cfg.v_head_dim) ** -0.5).to(dt)
    qn, kn = (1 + 0.1 * r(cfg.q_lora_rank)).to(dt), (1 + 0.1 * r(cfg.kv_lora_rank)).to(dt)
    ang = torch.outer(torch.arange(512).float(), 1.0 / (10000.0 ** (torch.arange(0, cfg.rope_head_dim, 2).float() / cfg.rope_head_dim)))
    freqs = torch.polar(torch.ones_like(ang), ang)
    prompts, steps = [150, 3, 77], 3
    blocks_per_seq = (max(prompts) + steps + block_size - 1) // block_size
    NB = len(prompts) * blocks_per_seq + 3
    perm = torch.randperm(NB, generator=g).tolist()
    tables = [perm[i * blocks_per_seq:(i + 1) * blocks_per_seq] for i in range(len(prompts))]
    kc_ref = torch.zeros(NB, block_size, cfg.kv_lora_rank).to(dt)
    pc_ref = torch.zeros(NB, block_size, cfg.rope_head_dim).to(dt)
    kc, pc = kc_ref.to(DEV), pc_ref.to(DEV)
    layer = MlaLayer(cfg, wa.to(DEV), qn.to(DEV), kn.to(DEV), wqb.to(DEV), wuk_t.to(DEV), wuv.to(DEV), wo.to(DEV))
    cached = [0] * len(prompts)
    for step in range(steps + 1):
        lens = prompts if step == 0 else [1] * len(prompts)
        hidden = r(sum(lens), cfg.hidden).to(dt)
        meta = prepare_attn(lens, cached, tables, block_size, DEV)
        got = layer.forward(rt, hidden.to(DEV), kc, pc, meta, freqs.to(DEV))
        rt.synchronize()
        ref = O.mla_forward_ref(hidden, wa, qn, kn, wqb, wuk_t, wuv, wo, kc_ref, pc_ref, lens, cached, tables, freqs, n_heads,
                                cfg.q_lora_rank, cfg.kv_lora_rank, cfg.nope_head_dim, cfg.rope_head_dim, cfg.v_head_dim,
                                block_size, cfg.softmax_scale, cfg.norm_eps)
        err = (got.float().cpu() - ref.float()).abs()
        assert float(err.max()) <= 3e-2 and float(err.mean()) <= 3e-3, "step %d: max %g mean %g" % (step, float(err.max()), float(err.mean()))
        # the caches agree up to a 16-bit unit of the projected rows (the two GEMMs sum in different orders)
        torch.testing.assert_close(kc.float().cpu(), kc_ref.float(), rtol=2 ** -6, atol=3e-2)
        torch.testing.assert_close(pc.float().cpu(), pc_ref.float(), rtol=2 ** -6, atol=3e-2)
        cached = [c + l for c, l in zip(cached, lens)]
