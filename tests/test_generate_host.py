"""Host-side checks of the generation stack: the paged caches' bounds are enforced before anything is launched."""
import types

import pytest
import torch

from gvirt_amd.generate import DecoderModel


def _model(max_batch=2, max_seq_len=40, block_size=16):
    cfg = types.SimpleNamespace(block_size=block_size, n_kv_heads=1, head_dim=8)
    layer = types.SimpleNamespace(cfg=cfg)
    embed = torch.zeros(4, 8, dtype=torch.bfloat16)
    return DecoderModel(None, [layer], [torch.ones(8), torch.ones(8)], embed, torch.zeros(8, 4, dtype=torch.bfloat16),
                        torch.zeros(1), max_batch, max_seq_len)


def test_attn_meta_lays_out_consecutive_blocks_per_sequence():
    m = _model()
    meta = m.attn_meta([3, 1], [0, 32])
    assert meta.block_tables == [[0], [3, 4, 5]]


def test_attn_meta_refuses_batches_and_lengths_beyond_the_caches():
    m = _model()
    with pytest.raises(RuntimeError, match="max_batch"):
        m.attn_meta([1, 1, 1], [0, 0, 0])
    with pytest.raises(RuntimeError, match="max_seq_len"):
        m.attn_meta([1, 2], [0, 39])
    m.attn_meta([1, 1], [0, 39])   # exactly full is fine
