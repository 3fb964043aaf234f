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
        self.max_batch, self.max_seq_len, self.norm_eps = max_batch, max_seq_len, norm_eps
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

    def check_batch(self, batch: int, longest: int) -> None:
        """The caches hold `max_batch` sequences of `max_seq_len` positions: anything beyond would be written and
        read outside them."""
        if batch > self.max_batch:
            raise RuntimeError("DecoderModel: batch of %d sequences exceeds max_batch=%d" % (batch, self.max_batch))
        if longest > self.max_seq_len:
            raise RuntimeError("DecoderModel: a sequence of %d positions exceeds max_seq_len=%d" % (longest, self.max_seq_len))

    def attn_meta(self, lens: Sequence[int], cached_lens: Sequence[int]) -> _C.ModelAttnMeta:
        """The step's host lists (xlite/tests/models/llama.py:640-651): sequence i uses blocks i * blocks_per_seq ..."""
        meta = _C.ModelAttnMeta()
        meta.lens = [int(x) for x in lens]
        meta.cached_lens = [int(x) for x in cached_lens]
        self.check_batch(len(meta.lens), max((l + c for l, c in zip(meta.lens, meta.cached_lens)), default=0))
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
    """The rectangular loop of the reference's harness (xlite/tests/generate.py:52-103), greedy: the first call
    feeds every sequence the shortest prompt's length, every later call one position of every sequence; where a
    prompt still has a token for the position, that token stands and the model's choice is dropped. Sequences
    keep stepping after their end token so that the batch stays rectangular; the answer of each is cut at its
    first end token. Returns the new tokens per sequence and the number of model calls."""
    if temperature > 0:
        raise RuntimeError("generate: only greedy selection (temperature 0) is built")
    n = len(prompt_tokens)
    longest = max(len(t) for t in prompt_tokens)
    if longest > model.max_seq_len:
        raise RuntimeError("Prompt length exceeds model maximum sequence length (max_seq_len=%d)" % model.max_seq_len)
    model.check_batch(n, longest)
    horizon = min(model.max_seq_len, longest + max_new_tokens)
    known = [[int(x) for x in t] for t in prompt_tokens]     # per sequence: the prompt, then what was chosen
    ended = [False] * n
    fed, calls = 0, 0
    dev = model.embed.device
    for pos in range(min(len(t) for t in known), horizon):
        # every sequence holds at least `pos` tokens here: the columns fed .. pos - 1 of the token matrix
        window = torch.tensor([k[fed:pos] for k in known], dtype=torch.int32, device=dev)
        choice = model.forward(window, fed).argmax(dim=-1).tolist()
        calls += 1
        for i, k in enumerate(known):
            if len(k) == pos:          # the prompt is used up: the model's token is the sequence's next one
                k.append(int(choice[i]))
                ended[i] = ended[i] or k[-1] == eos_id
        fed = pos
        if all(ended):
            break
    answers = []
    for k, t in zip(known, prompt_tokens):
        new = k[len(t): len(t) + max_new_tokens]
        answers.append(new[: new.index(eos_id)] if eos_id in new else new)
    return answers, calls


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
