"""Seeded synthetic inputs for the five benchmark configurations of the attention path.

Everything is random-initialised (there are no datasets or checkpoints on the box): q/k/v ~ N(0,1)
in bf16, q pre-multiplied by 1/sqrt(head_dim) (the convention of `rope_and_cache`, which hands
`attention` an already scaled query), block tables a random permutation of physical blocks.
Tensors are created on `device`; a CPU copy of the same seed is bit-identical only when the
generator device is also the CPU, so parity tests build on the CPU and move the tensors over.
"""
from __future__ import annotations

import math
from dataclasses import dataclass, field
from typing import Dict, List, Optional

import numpy as np
import torch

SEED_BASE = 20260000


@dataclass
class GqaShape:
    name: str
    n_heads: int
    n_kv_heads: int
    head_dim: int
    block_size: int = 128
    dtype: torch.dtype = torch.bfloat16


QWEN2_05B = GqaShape("qwen2-0.5b", 14, 2, 64)
LLAMA3_8B = GqaShape("llama-3-8b", 32, 8, 128)
QWEN25_7B = GqaShape("qwen2.5-7b", 28, 4, 128)


def c1_context_lengths(seed: int = SEED_BASE + 1) -> List[int]:
    rng = np.random.default_rng(seed)
    return [int(x) for x in rng.integers(256, 513, size=4)]


def c3_total_lengths(seed: int = SEED_BASE + 3) -> List[int]:
    rng = np.random.default_rng(seed)
    return [int(x) for x in rng.integers(1024, 8193, size=8)]


def c4_context_lengths(seed: int = SEED_BASE + 4) -> List[int]:
    rng = np.random.default_rng(seed)
    return [int(x) for x in rng.integers(4096, 8193, size=32)]


def c5_context_lengths(seed: int = SEED_BASE + 5, batch: int = 128) -> List[int]:
    rng = np.random.default_rng(seed)
    u = rng.uniform(math.log(128.0), math.log(32768.0), size=batch)
    return [int(round(math.exp(x))) for x in u]


def _tables(ctx: List[int], block_size: int, spare: int, gen: torch.Generator, device) -> Dict:
    nblk = [(c + block_size - 1) // block_size for c in ctx]
    max_nb = max(nblk)
    total = sum(nblk) + spare
    perm = torch.randperm(total, generator=gen, device=device).to(torch.int32)
    tables = torch.zeros(len(ctx), max_nb, dtype=torch.int32, device=device)
    off = 0
    for i, n in enumerate(nblk):
        tables[i, :n] = perm[off:off + n]
        off += n
    return dict(tables=tables, max_num_block=max_nb, num_blocks=total)


def _randn(shape, gen, device, dtype, scale: float = 1.0, chunk: int = 1 << 26) -> torch.Tensor:
    """N(0,1) * scale in `dtype`, generated in fp32 pieces to bound the temporary."""
    out = torch.empty(shape, dtype=dtype, device=device)
    flat = out.view(-1)
    for s in range(0, flat.numel(), chunk):
        e = min(flat.numel(), s + chunk)
        piece = torch.randn(e - s, generator=gen, device=device, dtype=torch.float32)
        flat[s:e] = (piece * scale).to(dtype) if scale != 1.0 else piece.to(dtype)
    return out


def quantize_cache(x: torch.Tensor, kv_dtype: torch.dtype):
    """Per (position, kv head) symmetric quantisation of a cache tensor [..., head_dim] to int8 (scale =
    absmax / 127) or float8_e4m3fn (scale = absmax / 448); returns the bytes and the fp32 scales."""
    xf = x.float()
    scale = xf.abs().amax(dim=-1) / (127.0 if kv_dtype == torch.int8 else 448.0)
    safe = torch.where(scale > 0, scale, torch.ones_like(scale))
    y = xf / safe.unsqueeze(-1)
    q = torch.clamp(torch.round(y), -127, 127).to(torch.int8) if kv_dtype == torch.int8 else y.to(kv_dtype)
    return q, scale.contiguous()


def gqa_decode(shape: GqaShape, ctx: List[int], seed: int, device="cpu", int8_kv: bool = False,
               spare_blocks: int = 2, kv_dtype: Optional[torch.dtype] = None) -> Dict:
    """One decode step: every sequence has ctx[i] - 1 cached tokens and one new token whose K/V is
    already in the cache (the operator reads only the caches)."""
    gen = torch.Generator(device=device).manual_seed(seed)
    B = len(ctx)
    H, KV, D, bs = shape.n_heads, shape.n_kv_heads, shape.head_dim, shape.block_size
    t = _tables(ctx, bs, spare_blocks, gen, device)
    NB = t["num_blocks"]
    qkv = _randn((B, (H + 2 * KV) * D), gen, device, shape.dtype)
    qkv.view(B, H + 2 * KV, D)[:, :H] = (qkv.view(B, H + 2 * KV, D)[:, :H].float() * D ** -0.5).to(shape.dtype)
    k_cache = _randn((NB, bs, KV, D), gen, device, shape.dtype)
    v_cache = _randn((NB, bs, KV, D), gen, device, shape.dtype)
    w = dict(shape=shape, batch=B, ctx=ctx, qkv=qkv, k_cache=k_cache, v_cache=v_cache,
             output=torch.zeros(B, H * D, dtype=shape.dtype, device=device),
             query_start_loc=torch.arange(B, dtype=torch.int32, device=device),
             lens=torch.ones(B, dtype=torch.int32, device=device),
             cached_lens=torch.tensor([c - 1 for c in ctx], dtype=torch.int32, device=device),
             block_tables=t["tables"].flatten().contiguous(), max_num_block=t["max_num_block"],
             k_scale=None, v_scale=None)
    if int8_kv and kv_dtype is None:
        kv_dtype = torch.int8
    int8_kv = kv_dtype is not None
    if int8_kv:
        for name in ("k", "v"):
            w[name + "_cache"], w[name + "_scale"] = quantize_cache(w[name + "_cache"], kv_dtype)
    kv_elt = 1 if int8_kv else 2
    total_ctx = sum(ctx)
    w["kv_bytes"] = total_ctx * KV * D * 2 * kv_elt + (total_ctx * KV * 2 * 4 if int8_kv else 0)
    w["flops"] = 4 * H * D * total_ctx
    return w


def rope_inputs(shape: GqaShape, w: Dict, seed: int, max_pos: int = 40960) -> Dict:
    """Inputs of the reshape-and-cache step that precedes a decode step: the 64 (batch) new tokens
    are written into the slots that their block tables assign to position ctx - 1."""
    device = w["qkv"].device
    gen = torch.Generator(device=device).manual_seed(seed)
    B, D, bs = w["batch"], shape.head_dim, shape.block_size
    inv = 1.0 / (10000.0 ** (torch.arange(0, D, 2, dtype=torch.float32, device=device) / D))
    ang = torch.outer(torch.arange(max_pos, dtype=torch.float32, device=device), inv)
    cosin = torch.cat([ang.cos(), ang.sin()], dim=-1).to(shape.dtype)
    pos = torch.tensor([c - 1 for c in w["ctx"]], dtype=torch.int64, device=device)
    tables = w["block_tables"].view(B, w["max_num_block"]).long()
    slots = (tables[torch.arange(B, device=device), pos // bs] * bs + pos % bs).to(torch.int32)
    inout = _randn(tuple(w["qkv"].shape), gen, device, shape.dtype)
    return dict(inout=inout, position=pos, cosin=cosin, slot_mapping=slots)


def gqa_prefill_chunk(shape: GqaShape, total_lens: List[int], chunk_index: int, chunk: int, seed: int,
                      device="cpu", caches: Optional[Dict] = None) -> Optional[Dict]:
    """The chunk_index-th 2048-token chunk of every sequence that still has tokens left, batched in
    one call: cached_lens = chunk * chunk_index, lens = min(chunk, L - cached). `caches` (from a
    previous call) carries the paged K/V and block tables, which already hold all L tokens."""
    H, KV, D, bs = shape.n_heads, shape.n_kv_heads, shape.head_dim, shape.block_size
    gen = torch.Generator(device=device).manual_seed(seed + 97 * chunk_index)
    if caches is None:
        g0 = torch.Generator(device=device).manual_seed(seed)
        t = _tables(total_lens, bs, 2, g0, device)
        caches = dict(k_cache=_randn((t["num_blocks"], bs, KV, D), g0, device, shape.dtype),
                      v_cache=_randn((t["num_blocks"], bs, KV, D), g0, device, shape.dtype),
                      tables=t["tables"], max_num_block=t["max_num_block"])
    seqs = [i for i, L in enumerate(total_lens) if L > chunk * chunk_index]
    if not seqs:
        return None
    lens = [min(chunk, total_lens[i] - chunk * chunk_index) for i in seqs]
    T = sum(lens)
    qkv = _randn((T, (H + 2 * KV) * D), gen, device, shape.dtype)
    qkv.view(T, H + 2 * KV, D)[:, :H] = (qkv.view(T, H + 2 * KV, D)[:, :H].float() * D ** -0.5).to(shape.dtype)
    qsl = np.cumsum([0] + lens[:-1]).tolist()
    pairs = sum(l * (chunk * chunk_index) + l * (l + 1) // 2 for l in lens)
    return dict(shape=shape, batch=len(seqs), seqs=seqs, qkv=qkv, k_cache=caches["k_cache"],
                v_cache=caches["v_cache"], output=torch.zeros(T, H * D, dtype=shape.dtype, device=device),
                query_start_loc=torch.tensor(qsl, dtype=torch.int32, device=device),
                lens=torch.tensor(lens, dtype=torch.int32, device=device),
                cached_lens=torch.full((len(seqs),), chunk * chunk_index, dtype=torch.int32, device=device),
                block_tables=caches["tables"][seqs].flatten().contiguous(),
                max_num_block=caches["max_num_block"], caches=caches, flops=4 * H * D * pairs, tokens=T)


@dataclass
class MlaShape:
    name: str = "deepseek-r1"
    n_heads: int = 128
    kv_lora_rank: int = 512
    rope_head_dim: int = 64
    nope_head_dim: int = 128
    v_head_dim: int = 128
    block_size: int = 64
    scale: float = field(default=192 ** -0.5)


def mla_decode(shape: MlaShape, ctx: List[int], seed: int, device="cpu") -> Dict:
    gen = torch.Generator(device=device).manual_seed(seed)
    B, H, C, R, bs = len(ctx), shape.n_heads, shape.kv_lora_rank, shape.rope_head_dim, shape.block_size
    t = _tables(ctx, bs, 2, gen, device)
    NB = t["num_blocks"]
    dt = torch.bfloat16
    total_ctx = sum(ctx)
    return dict(shape=shape, batch=B, ctx=ctx,
                q_absorb=_randn((B, H, C), gen, device, dt), qr=_randn((B, H, R), gen, device, dt),
                k_cache=_randn((NB, bs, C), gen, device, dt), pe_cache=_randn((NB, bs, R), gen, device, dt),
                o_absorb=torch.zeros(B, H, C, dtype=dt, device=device),
                query_start_loc=torch.arange(B, dtype=torch.int32, device=device),
                lens=torch.ones(B, dtype=torch.int32, device=device),
                cached_lens=torch.tensor([c - 1 for c in ctx], dtype=torch.int32, device=device),
                block_tables=t["tables"].flatten().contiguous(), max_num_blocks=t["max_num_block"],
                kv_bytes=total_ctx * (C + R) * 2, flops=total_ctx * H * (2 * (C + R) + 2 * C))


def to_device(w: Dict, device) -> Dict:
    out = {}
    for k, v in w.items():
        if isinstance(v, torch.Tensor):
            out[k] = v.to(device)
        elif isinstance(v, dict):
            out[k] = to_device(v, device)
        else:
            out[k] = v
    return out
