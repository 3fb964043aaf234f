"""Model-level caller of the attention path: the per-step metadata and one multi-head attention layer.

Mirrors the attention part of the reference's model runner: `XRuntime::PrepareAttn`
(xlite/csrc/runtime.cpp:404-550) builds the step's metadata on the host and uploads it, and
`XModel::ForwardAttnMHA` (xlite/csrc/model.cpp:480-600) runs QKV projection -> (qk_rms_norm) ->
rope_and_cache -> attention -> output projection. The two projections are plain GEMMs and go through
torch.matmul (hipBLASLt); everything between them is this package's operators.
"""
import ctypes
from dataclasses import dataclass
from typing import List, Optional, Sequence

import torch

from . import _C, _lib


@dataclass
class StepMeta:
    """What `PrepareAttn` leaves on the device for one step (xlite/csrc/runtime.h:37-51)."""
    batch: int
    batched_tokens: int
    max_num_blocks: int
    is_decode: bool
    query_start_loc: torch.Tensor   # [batch] int32
    lens: torch.Tensor              # [batch] int32
    cached_lens: torch.Tensor       # [batch] int32
    block_tables: torch.Tensor      # [batch * max_num_blocks] int32
    position: torch.Tensor          # [batched_tokens] int64
    slot_mapping: torch.Tensor      # [batched_tokens] int32


def prepare_attn(lens: Sequence[int], cached_lens: Sequence[int], block_tables: Sequence[Sequence[int]],
                 block_size: int, device, positions: Optional[torch.Tensor] = None) -> StepMeta:
    """Host metadata of one step through the library's `xlite_hip_prepare_attn`, then one upload per array.
    `block_tables[i]` lists the physical blocks of sequence i (at least ceil((len + cached) / block_size)).
    `positions` (int64, one per token) replaces the derived positions, as the reference's version-1 metadata
    does (xlite/csrc/runtime.cpp:535-548)."""
    lib = _lib.load()
    batch = len(lens)
    if batch == 0:
        raise RuntimeError("invalid batchSize: 0")
    u32 = ctypes.c_uint32 * batch
    rows = [(ctypes.c_int32 * max(1, len(r)))(*r) for r in block_tables]
    ptrs = (ctypes.c_void_p * batch)(*[ctypes.addressof(a) for a in rows])
    T = int(sum(lens))
    cap = batch * max((int(l) + int(c) + block_size - 1) // block_size for l, c in zip(lens, cached_lens))
    qsl = torch.empty(batch, dtype=torch.int32)
    pos = torch.empty(T, dtype=torch.int64)
    slots = torch.empty(T, dtype=torch.int32)
    dense = torch.empty(max(cap, 1), dtype=torch.int32)
    mnb, bt, dec = ctypes.c_uint32(), ctypes.c_uint32(), ctypes.c_int()
    _lib.check(lib.xlite_hip_prepare_attn(
        u32(*[int(x) for x in lens]), u32(*[int(x) for x in cached_lens]), batch, ptrs, u32(*[len(r) for r in block_tables]),
        block_size, ctypes.c_void_p(qsl.data_ptr()), ctypes.c_void_p(pos.data_ptr()), ctypes.c_void_p(slots.data_ptr()),
        ctypes.c_void_p(dense.data_ptr()), cap, ctypes.byref(mnb), ctypes.byref(bt), ctypes.byref(dec)))
    up = lambda t: t.to(device, non_blocking=False)
    if positions is not None:
        if positions.dtype != torch.int64 or positions.numel() < T:
            raise RuntimeError("prepare_attn: positions must hold one int64 per token")
        pos = positions.reshape(-1)[:T]
    return StepMeta(batch=batch, batched_tokens=int(bt.value), max_num_blocks=int(mnb.value), is_decode=bool(dec.value),
                    query_start_loc=up(qsl), lens=up(torch.tensor([int(x) for x in lens], dtype=torch.int32)),
                    cached_lens=up(torch.tensor([int(x) for x in cached_lens], dtype=torch.int32)),
                    block_tables=up(dense[: batch * int(mnb.value)].contiguous()), position=up(pos), slot_mapping=up(slots))


def prepare_attn_meta(meta, block_size: int, device) -> StepMeta:
    """`prepare_attn` from one of the reference's metadata objects: `_C.ModelAttnMeta` (positions derived) or
    `_C.AttnMeta` (vLLM form: `block_tables_cpu` and the caller's `positions` tensor)."""
    if isinstance(meta, _C.ModelAttnMeta):
        return prepare_attn(meta.lens, meta.cached_lens, meta.block_tables, block_size, device)
    if isinstance(meta, _C.AttnMeta):
        if meta.positions is None:
            raise RuntimeError("prepare_attn: AttnMeta.positions is not set")
        return prepare_attn(meta.lens, meta.cached_lens, meta.block_tables_cpu, block_size, device, positions=meta.positions)
    raise RuntimeError("prepare_attn: invalid attnMeta version: " + type(meta).__name__)


@dataclass
class MhaConfig:
    hidden: int
    n_heads: int
    n_kv_heads: int
    head_dim: int
    rot_dim: int
    block_size: int
    norm_eps: float = 1e-6
    qk_norm: bool = False


class MhaLayer:
    """One attention layer: weights `wqkv` [hidden, (n_heads + 2 n_kv_heads) head_dim] (+ optional bias), `wo`
    [n_heads head_dim, hidden], optional per-head RMSNorm weights `q_norm`, `k_norm` [head_dim]."""

    def __init__(self, cfg: MhaConfig, wqkv: torch.Tensor, wo: torch.Tensor, bqkv: Optional[torch.Tensor] = None,
                 q_norm: Optional[torch.Tensor] = None, k_norm: Optional[torch.Tensor] = None):
        self.cfg, self.wqkv, self.wo, self.bqkv, self.q_norm, self.k_norm = cfg, wqkv, wo, bqkv, q_norm, k_norm
        if cfg.qk_norm and (q_norm is None or k_norm is None):
            raise RuntimeError("MhaLayer: qk_norm needs q_norm and k_norm")

    def forward(self, rt: _C.Runtime, hidden: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, meta: StepMeta,
                cosin: torch.Tensor) -> torch.Tensor:
        c = self.cfg
        qkv = torch.matmul(hidden, self.wqkv)
        if self.bqkv is not None:
            qkv = qkv + self.bqkv
        qkv = qkv.contiguous()
        if c.qk_norm:
            _C.qk_rms_norm(rt, qkv, self.q_norm, None, self.k_norm, None, qkv, c.norm_eps, c.head_dim, c.n_heads,
                           c.head_dim, c.n_kv_heads, c.n_heads * c.head_dim)
        attn = torch.empty(hidden.shape[0], c.n_heads * c.head_dim, dtype=hidden.dtype, device=hidden.device)
        # rope_and_cache, then attention (xlite/csrc/model.cpp:544-571), from one call into the library: a single
        # kernel launch for decode steps over short contexts, the two launches otherwise, the same bits either way
        _C.decode_step(rt, qkv, k_cache, v_cache, attn, meta.position, cosin, meta.slot_mapping, meta.query_start_loc,
                       meta.lens, meta.cached_lens, meta.block_tables, c.n_heads, c.n_kv_heads, c.head_dim, c.rot_dim,
                       c.block_size, meta.batch, meta.max_num_blocks)
        return torch.matmul(attn, self.wo)
