"""A small decoder stack over the attention layers, and the greedy generation loop of the reference's harness.

Mirrors the attention side of `xlite/tests/generate.py:52-103` (`generate`: a rectangular token matrix, one
prefill of the shortest prompt's length, then one position per step, prompts longer than that forced) and of
`xlite/tests/models/llama.py:640-651`, `:419-427` (`prepare_xlite_attnmeta` + `forward_xlite`: the step's
`ModelAttnMeta`, every layer over the paged caches, logits of each sequence's last token). `generate_ragged`
is the serving-shaped variant: one ragged prefill of every whole prompt, then decode steps.

The stack is attention only: x += Attention(RMSNorm(x)) per layer, a final RMSNorm and the vocabulary
projection; the reference's feed-forward blocks, sampling and weight loading are outside this package's
path. Norms, embedding and projections are torch operations; the attention layers run this package's operators
(`MhaLayer` or `MlaLayer`), and the metadata goes through `prepare_attn_meta` exactly as `XRuntime::PrepareAttn`
(xlite/csrc/runtime.cpp:404-550) derives it from the lists.
"""
from typing import List, Sequence, Tuple

import torch

from . import _C
from .mha import MhaLayer, prepare_attn_meta
from .mla import MlaLayer


def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    xf = x.float()
    return (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps) * weight.float()).to(x.dtype)


class DecoderModel:
    """`layers`: MhaLayer or MlaLayer objects (all of one kind); `norms`: one RMSNorm weight [hidden] per layer and
    a final one; `embed` [vocab, hidden]; `lm_head` [hidden, vocab]; `rope`: the cos|sin table of `rope_and_cache`
    (MHA) or the complex `freqs` of `mla_prepare` (MLA). Every sequence of a batch owns `ceil(max_seq_len /
    block_size)` consecutive physical blocks, as the reference's harness lays them out."""

    def __init__(self, rt: _C.Runtime, layers: Sequence, norms: Sequence[torch.Tensor], embed: torch.Tensor,
                 lm_head: torch.Tensor, rope: torch.Tensor, max_batch: int, max_seq_len: int, norm_eps: float = 1e-6):
        if len(norms) != len(layers) + 1:
            raise RuntimeError("DecoderModel: one norm per layer and a final one")
        self.rt, self.layers, self.norms, self.embed, self.lm_head, self.rope = rt, list(layers), list(norms), embed, lm_head, rope
        self.max_seq_len, self.norm_eps = max_seq_len, norm_eps
        cfg = layers[0].cfg
        self.block_size = cfg.block_size
        self.blocks_per_seq = (max_seq_len + cfg.block_size - 1) // cfg.block_size
        nb = max_batch * self.blocks_per_seq
        dev, dt = embed.device, embed.dtype
        self.is_mla = isinstance(layers[0], MlaLayer)
        if self.is_mla:
            self.caches = [(torch.zeros(nb, cfg.block_size, cfg.kv_lora_rank, dtype=dt, device=dev),
                            torch.zeros(nb, cfg.block_size, cfg.rope_head_dim, dtype=dt, device=dev)) for _ in layers]
        else:
            self.caches = [(torch.zeros(nb, cfg.block_size, cfg.n_kv_heads, cfg.head_dim, dtype=dt, device=dev),
                            torch.zeros(nb, cfg.block_size, cfg.n_kv_heads, cfg.head_dim, dtype=dt, device=dev)) for _ in layers]

    def attn_meta(self, lens: Sequence[int], cached_lens: Sequence[int]) -> _C.ModelAttnMeta:
        """The step's host lists (xlite/tests/models/llama.py:640-651): sequence i uses blocks i * blocks_per_seq ..."""
        meta = _C.ModelAttnMeta()
        meta.lens = [int(x) for x in lens]
        meta.cached_lens = [int(x) for x in cached_lens]
        meta.block_tables = [[i * self.blocks_per_seq + b for b in range((l + c + self.block_size - 1) // self.block_size)]
                             for i, (l, c) in enumerate(zip(meta.lens, meta.cached_lens))]
        return meta

    def forward_tokens(self, tokens: torch.Tensor, lens: Sequence[int], cached_lens: Sequence[int]) -> torch.Tensor:
        """`tokens`: the step's token ids, sequence after sequence (sum(lens) of them). Returns the logits of every
        sequence's last token, [batch, vocab] in fp32. Sequences without tokens this step get a row of zeros."""
        meta = prepare_attn_meta(self.attn_meta(lens, cached_lens), self.block_size, self.embed.device)
        x = self.embed[tokens.long()]
        for layer, norm, (c0, c1) in zip(self.layers, self.norms, self.caches):
            h = rms_norm(x, norm, self.norm_eps)
            x = x + layer.forward(self.rt, h, c0, c1, meta, self.rope)
        x = rms_norm(x, self.norms[-1], self.norm_eps)
        ends, rows = [], []
        off = 0
        for i, l in enumerate(lens):
            off += int(l)
            if l > 0:
                ends.append(off - 1)
                rows.append(i)
        logits = torch.zeros(len(lens), self.lm_head.shape[1], dtype=torch.float32, device=x.device)
        if rows:
            last = x[torch.tensor(ends, device=x.device)]
            logits[torch.tensor(rows, device=x.device)] = torch.matmul(last, self.lm_head).float()
        return logits

    def forward(self, tokens: torch.Tensor, start_pos: int = 0) -> torch.Tensor:
        """The reference model's call shape (xlite/tests/models/llama.py:419-427): `tokens` [batch, seqlen], every
        sequence with `start_pos` cached tokens."""
        batch, seqlen = tokens.shape
        return self.forward_tokens(tokens.reshape(-1), [seqlen] * batch, [start_pos] * batch)


def generate(model: DecoderModel, prompt_tokens: List[List[int]], max_new_tokens: int, eos_id: int,
             temperature: float = 0.0) -> Tuple[List[List[int]], int]:
    """xlite/tests/generate.py:52-103 with greedy selection (temperature 0; sampling is outside this path)."""
    if temperature > 0:
        raise RuntimeError("generate: only greedy selection (temperature 0) is built")
    prompt_lens = [len(t) for t in prompt_tokens]
    if max(prompt_lens) > model.max_seq_len:
        raise RuntimeError("Prompt length exceeds model maximum sequence length (max_seq_len=%d)" % model.max_seq_len)
    dev = model.embed.device
    total_len = min(model.max_seq_len, max_new_tokens + max(prompt_lens))
    tokens_cpu = torch.full((len(prompt_tokens), total_len), -1, dtype=torch.int32)
    for i, t in enumerate(prompt_tokens):
        tokens_cpu[i, : len(t)] = torch.tensor(t, dtype=torch.int32)
    prompt_mask = (tokens_cpu != -1).to(dev)
    tokens = tokens_cpu.to(dev)
    finished = torch.zeros(len(prompt_tokens), dtype=torch.bool, device=dev)
    prev_pos, step = 0, 0
    for cur_pos in range(min(prompt_lens), total_len):
        logits = model.forward(tokens[:, prev_pos:cur_pos], prev_pos)
        next_token = logits.argmax(dim=-1).to(torch.int32)
        next_token = torch.where(prompt_mask[:, cur_pos], tokens[:, cur_pos], next_token)
        tokens[:, cur_pos] = next_token
        finished |= torch.logical_and(~prompt_mask[:, cur_pos], next_token == eos_id)
        prev_pos = cur_pos
        step += 1
        if bool(finished.all()):
            break
    out = []
    for i, toks in enumerate(tokens.tolist()):
        toks = toks[prompt_lens[i]: prompt_lens[i] + max_new_tokens]
        if eos_id in toks:
            toks = toks[: toks.index(eos_id)]
        out.append(toks)
    return out, step


def generate_ragged(model: DecoderModel, prompt_tokens: List[List[int]], max_new_tokens: int, eos_id: int) -> Tuple[List[List[int]], int]:
    """One ragged prefill of every whole prompt, then one decode step per new token (a sequence that has produced
    `eos_id` takes no further part: its length for the step is 0). Greedy."""
    dev = model.embed.device
    n = len(prompt_tokens)
    cached = [0] * n
    pending = [list(t) for t in prompt_tokens]     # tokens to feed next, per sequence
    out: List[List[int]] = [[] for _ in range(n)]
    done = [False] * n
    step = 0
    for _ in range(max_new_tokens):
        lens = [len(p) for p in pending]
        if sum(lens) == 0:
            break
        flat = torch.tensor([t for p in pending for t in p], dtype=torch.int32, device=dev)
        logits = model.forward_tokens(flat, lens, cached)
        nxt = logits.argmax(dim=-1).tolist()
        step += 1
        for i in range(n):
            cached[i] += lens[i]
            pending[i] = []
            if lens[i] == 0 or done[i]:
                continue
            if nxt[i] == eos_id or cached[i] + 1 > model.max_seq_len:
                done[i] = True
                continue
            out[i].append(int(nxt[i]))
            pending[i] = [int(nxt[i])]
    return out, step
