"""Model-level caller of the MLA path: one multi-head latent attention layer over the operators.

Mirrors `XModel::ForwardAttnMLACommonV2` and `XModel::ForwardAttnMLAV2` of the reference
(xlite/csrc/model.cpp:333-482): QKV_A projection -> mla_prepare (two RMSNorms, rope of the shared rotary
slice, latent / rotary cache write) -> Q_B projection -> rope_complex (per-head rotary slice of q) ->
W_UK absorb einsum -> absorbed attention over the paged latent cache -> W_UV einsum -> output projection.
With indexer weights the DSA branch `XModel::ForwardAttnIndexer` (xlite/csrc/model.cpp:285-330) runs between
mla_prepare and the attention: index key projection -> LayerNorm -> rope into the index key cache -> index
query projection -> rope -> head-weight scaling -> indexer_topk, whose position lists mask the attention.
The projections are plain GEMMs and go through torch.matmul; everything between them is this package's
operators. The step's metadata comes from `gvirt_amd.mha.prepare_attn`.
"""
from dataclasses import dataclass
from typing import Optional

import torch

from . import _C
from .mha import StepMeta


@dataclass
class MlaConfig:
    hidden: int
    n_heads: int
    q_lora_rank: int
    kv_lora_rank: int
    nope_head_dim: int
    rope_head_dim: int
    v_head_dim: int
    block_size: int
    softmax_scale: float
    norm_eps: float = 1e-6


@dataclass
class IndexerWeights:
    """The DSA indexer of a layer: `wk_weights_proj` [hidden, index_head_dim + index_n_heads] (index key, then one
    weight per index head), `k_norm`, `k_norm_bias` [index_head_dim] (LayerNorm), `wq_b` [q_lora, index_n_heads *
    index_head_dim]."""
    wk_weights_proj: torch.Tensor
    k_norm: torch.Tensor
    k_norm_bias: torch.Tensor
    wq_b: torch.Tensor
    index_n_heads: int
    index_head_dim: int
    index_topk: int


class MlaLayer:
    """Weights: `wqkv_a` [hidden, q_lora + kv_lora + rope], `q_norm` [q_lora], `kv_norm` [kv_lora] (optional
    biases of the same shapes), `wq_b` [q_lora, n_heads (nope + rope)], `wuk_t` [n_heads, nope, kv_lora],
    `wuv` [n_heads, kv_lora, v_head], `wo` [n_heads v_head, hidden]."""

    def __init__(self, cfg: MlaConfig, wqkv_a: torch.Tensor, q_norm: torch.Tensor, kv_norm: torch.Tensor,
                 wq_b: torch.Tensor, wuk_t: torch.Tensor, wuv: torch.Tensor, wo: torch.Tensor,
                 q_norm_bias: Optional[torch.Tensor] = None, kv_norm_bias: Optional[torch.Tensor] = None,
                 indexer: Optional[IndexerWeights] = None):
        self.cfg = cfg
        self.indexer = indexer
        self.last_topk_indices = None
        self.wqkv_a, self.q_norm, self.kv_norm, self.wq_b, self.wuk_t, self.wuv, self.wo = \
            wqkv_a, q_norm, kv_norm, wq_b, wuk_t, wuv, wo
        self.q_norm_bias = torch.zeros_like(q_norm) if q_norm_bias is None else q_norm_bias
        self.kv_norm_bias = torch.zeros_like(kv_norm) if kv_norm_bias is None else kv_norm_bias
        if wuk_t.numel() != cfg.n_heads * cfg.nope_head_dim * cfg.kv_lora_rank:
            raise RuntimeError("MlaLayer: wuk_t must be [n_heads, nope_head_dim, kv_lora_rank]")
        if wuv.numel() != cfg.n_heads * cfg.kv_lora_rank * cfg.v_head_dim:
            raise RuntimeError("MlaLayer: wuv must be [n_heads, kv_lora_rank, v_head_dim]")

    def index_topk(self, rt: _C.Runtime, hidden: torch.Tensor, norm_qc: torch.Tensor, index_k_cache: torch.Tensor,
                   meta: StepMeta, freqs: torch.Tensor) -> Optional[torch.Tensor]:
        """`ForwardAttnIndexer` (xlite/csrc/model.cpp:285-330): writes the step's index keys into `index_k_cache`
        [num_blocks, block_size, index_head_dim] and returns the position lists [tokens, index_topk], or None
        when no sequence can be longer than index_topk."""
        c, ix = self.cfg, self.indexer
        T = hidden.shape[0]
        kw = torch.matmul(hidden, ix.wk_weights_proj).contiguous()          # [T, index_head_dim + index_n_heads]
        _C.layernorm(rt, kw, ix.k_norm, ix.k_norm_bias, kw, c.norm_eps, ix.index_head_dim)
        _C.rope_complex_and_cache(rt, 1, ix.index_head_dim + ix.index_n_heads, c.rope_head_dim, 0, ix.index_head_dim, kw,
                                  freqs, meta.position, block_size=c.block_size, cache=index_k_cache,
                                  slot_mapping=meta.slot_mapping)
        if meta.max_num_blocks * c.block_size <= ix.index_topk:
            return None
        q = torch.matmul(norm_qc, ix.wq_b).contiguous()                      # [T, index_n_heads * index_head_dim]
        _C.rope_complex_and_cache(rt, ix.index_n_heads, ix.index_head_dim, c.rope_head_dim, 0, 0, q, freqs, meta.position,
                                  output=q, out_step_dim=ix.index_head_dim, out_offset=0)
        _C.muls(rt, kw, (ix.index_n_heads * ix.index_head_dim) ** -0.5, kw, ix.index_head_dim, ix.index_n_heads)
        topk = torch.empty(T, ix.index_topk, dtype=torch.int32, device=hidden.device)
        arange = torch.arange(meta.max_num_blocks * c.block_size, dtype=torch.int32, device=hidden.device)
        _C.indexer_topk(rt, q, index_k_cache, kw, arange, topk, meta.query_start_loc, meta.lens, meta.cached_lens,
                        meta.block_tables, ix.index_n_heads, ix.index_head_dim, c.block_size, meta.batch, meta.max_num_blocks,
                        ix.index_topk)
        return topk

    def forward(self, rt: _C.Runtime, hidden: torch.Tensor, k_cache: torch.Tensor, pe_cache: torch.Tensor,
                meta: StepMeta, freqs: torch.Tensor, topk_indices: Optional[torch.Tensor] = None,
                top_k: int = 0, index_k_cache: Optional[torch.Tensor] = None) -> torch.Tensor:
        c = self.cfg
        T = hidden.shape[0]
        new = lambda cols: torch.empty(T, cols, dtype=hidden.dtype, device=hidden.device)
        qkvc = torch.matmul(hidden, self.wqkv_a).contiguous()
        norm_qc, norm_kvc = new(c.q_lora_rank), new(c.kv_lora_rank)
        _C.mla_prepare(rt, qkvc, self.q_norm, self.q_norm_bias, norm_qc, self.kv_norm, self.kv_norm_bias, norm_kvc,
                       freqs, meta.position, c.q_lora_rank, c.kv_lora_rank, c.rope_head_dim, c.block_size, k_cache,
                       pe_cache, meta.slot_mapping, c.norm_eps)
        if self.indexer is not None:
            if index_k_cache is None:
                raise RuntimeError("MlaLayer: a layer with an indexer needs its index key cache")
            topk_indices = self.index_topk(rt, hidden, norm_qc, index_k_cache, meta, freqs)
            top_k = self.indexer.index_topk if topk_indices is not None else 0
            self.last_topk_indices = topk_indices   # what the step attended to (None: every position)
        q_with_qr = torch.matmul(norm_qc, self.wq_b).contiguous()
        q_pe = new(c.n_heads * c.rope_head_dim)
        _C.rope_complex(rt, c.n_heads, c.nope_head_dim + c.rope_head_dim, c.rope_head_dim, q_with_qr, freqs,
                        meta.position, q_pe)
        attn = new(c.n_heads * c.v_head_dim)
        _C.mla_v2(rt, q_with_qr, q_pe, k_cache, pe_cache, self.wuk_t, self.wuv, attn, meta.query_start_loc, meta.lens,
                  meta.cached_lens, meta.block_tables, c.n_heads, c.rope_head_dim, c.nope_head_dim, c.v_head_dim,
                  c.kv_lora_rank, c.block_size, meta.batch, meta.max_num_blocks, c.softmax_scale, topk_indices, top_k)
        return torch.matmul(attn, self.wo)
