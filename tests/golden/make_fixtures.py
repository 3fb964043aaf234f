#!/usr/bin/env python3
"""Writes the golden fixtures of this directory: small seeded inputs and the outputs of the fp64
triple-loop C restatement (oracle/brute.c) on them (numpy float64 loops for the indexer), as .npz files of
plain arrays.

The reference's own tests hold no stored vectors (they draw unseeded random tensors), so these are
the vectors the HIP kernels and the PyTorch oracle are both held to. 16-bit tensors are stored as
their bit patterns (uint16). Run from the repository root:  python tests/golden/make_fixtures.py
"""
import os
import sys

import numpy as np
import torch

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__)))))
from oracle import brute  # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))


def bits(t):
    return t.contiguous().view(torch.int16).numpy().view(np.uint16).copy()


def gqa(name, seed, lens, clens, nH, nKV, d, bs, dtype):
    g = torch.Generator().manual_seed(seed)
    batch, T = len(lens), sum(lens)
    maxblk = max((l + c + bs - 1) // bs for l, c in zip(lens, clens))
    NB = batch * maxblk + 2
    qkv = (torch.randn(T, (nH + 2 * nKV) * d, generator=g) * 0.5).to(dtype)
    kc = torch.randn(NB, bs, nKV, d, generator=g).to(dtype)
    vc = torch.randn(NB, bs, nKV, d, generator=g).to(dtype)
    tables = torch.randperm(NB, generator=g)[: batch * maxblk].to(torch.int32)
    qsl = np.cumsum([0] + lens[:-1]).astype(np.int32)
    out = brute.attention(qkv, kc, vc, qsl, lens, clens, tables, nH, nKV, d, bs, batch, maxblk)
    np.savez_compressed(os.path.join(HERE, name), qkv=bits(qkv), k_cache=bits(kc), v_cache=bits(vc), block_tables=tables.numpy(),
                        query_start_loc=qsl, lens=np.int32(lens), cached_lens=np.int32(clens),
                        dims=np.int32([nH, nKV, d, bs, batch, maxblk, int(dtype == torch.bfloat16)]),
                        expected=out.numpy().astype(np.float32))


def mla(name, seed, lens, clens, nH, bs, top_k=0):
    R, C = 64, 512
    g = torch.Generator().manual_seed(seed)
    batch, T = len(lens), sum(lens)
    maxblk = max((l + c + bs - 1) // bs for l, c in zip(lens, clens))
    NB = batch * maxblk + 1
    qa = (torch.randn(T, nH, C, generator=g) * 0.3).bfloat16()
    qr = (torch.randn(T, nH, R, generator=g) * 0.3).bfloat16()
    kc = torch.randn(NB, bs, C, generator=g).bfloat16()
    pc = torch.randn(NB, bs, R, generator=g).bfloat16()
    tables = torch.randperm(NB, generator=g)[: batch * maxblk].to(torch.int32)
    qsl = np.cumsum([0] + lens[:-1]).astype(np.int32)
    scale = 192 ** -0.5
    topk = None
    if top_k:
        rows = []
        for i, (l, c) in enumerate(zip(lens, clens)):
            for r in range(l):
                rows.append(torch.sort(torch.randperm(c + r + 1, generator=g)[:top_k]).values)
        topk = torch.stack(rows).int()
    out = brute.mla(qa, qr, kc, pc, qsl, lens, clens, tables, nH, R, C, bs, batch, maxblk, scale, topk, top_k)
    np.savez_compressed(os.path.join(HERE, name), q_absorb=bits(qa), qr=bits(qr), k_cache=bits(kc), pe_cache=bits(pc),
                        block_tables=tables.numpy(), query_start_loc=qsl, lens=np.int32(lens), cached_lens=np.int32(clens),
                        dims=np.int32([nH, R, C, bs, batch, maxblk, top_k]), scale=np.float64(scale),
                        topk=(topk.numpy() if top_k else np.zeros((0, 0), np.int32)),
                        expected=out.numpy().astype(np.float32))


def rope(name, seed, T, nH, nKV, d, rot, bs, NB, dtype):
    g = torch.Generator().manual_seed(seed)
    inout = torch.randn(T, (nH + 2 * nKV) * d, generator=g).to(dtype)
    kc = torch.full((NB, bs, nKV, d), 7.0).to(dtype)
    vc = torch.full((NB, bs, nKV, d), -7.0).to(dtype)
    fr = torch.outer(torch.arange(64).float(), 1.0 / (10000.0 ** (torch.arange(0, rot, 2).float() / rot)))
    cosin = torch.cat([fr.cos(), fr.sin()], -1).to(dtype)
    pos = torch.randint(0, 64, (T,), generator=g)
    slots = torch.randperm(NB * bs, generator=g)[:T].int()
    a, b, c = brute.rope_and_cache(inout, kc, vc, pos, cosin, slots, nH, nKV, d, rot, bs)
    np.savez_compressed(os.path.join(HERE, name), inout=bits(inout), cosin=bits(cosin), position=pos.numpy().astype(np.int64),
                        slot_mapping=slots.numpy(), dims=np.int32([T, nH, nKV, d, rot, bs, NB, int(dtype == torch.bfloat16)]),
                        inout_after=bits(a), k_cache_after=bits(b), v_cache_after=bits(c))


def _round_bf16(x):
    """float64 array -> nearest bfloat16 (ties to even), as float64."""
    u = np.asarray(x, np.float32).view(np.uint32).astype(np.uint64)
    u = (u + 0x7fff + ((u >> 16) & 1)) & 0xffff0000
    return u.astype(np.uint32).view(np.float32).astype(np.float64)


def indexer(name, seed, lens, clens, nH, bs, top_k):
    """DSA indexer: numpy float64 loops (no shared code with the oracle). scores[t][j] =
    sum_h w[t][h] * bf16(q[t][h] . k[j]); the top-k positions are taken on the scores rounded to bf16, ties to
    the lower position, listed ascending."""
    D = 128
    g = torch.Generator().manual_seed(seed)
    batch, T = len(lens), sum(lens)
    maxblk = max((l + c + bs - 1) // bs for l, c in zip(lens, clens))
    NB = batch * maxblk + 1
    q = torch.randn(T, nH, D, generator=g).bfloat16()
    w = torch.randn(T, D + nH, generator=g).bfloat16()
    kc = torch.randn(NB, bs, D, generator=g).bfloat16()
    tables = torch.randperm(NB, generator=g)[: batch * maxblk].to(torch.int32)
    qsl = np.cumsum([0] + lens[:-1]).astype(np.int32)
    qn, wn, kn = q.double().numpy(), w.double().numpy(), kc.double().numpy()
    ld = maxblk * bs
    scores = np.full((T, ld), np.nan, np.float64)
    topk = np.full((T, top_k), -1, np.int32)
    for i in range(batch):
        n = lens[i] + clens[i]
        for r in range(lens[i]):
            t = int(qsl[i]) + r
            for j in range(n):
                krow = kn[int(tables[i * maxblk + j // bs]), j % bs]
                acc = 0.0
                for h in range(nH):
                    acc += wn[t, D + h] * _round_bf16(np.dot(qn[t, h], krow))
                scores[t, j] = acc
            key = _round_bf16(scores[t, :n])
            order = sorted(range(n), key=lambda j: (-key[j], j))[:top_k]
            sel = sorted(order)
            topk[t, :len(sel)] = sel
    np.savez_compressed(os.path.join(HERE, name), q=bits(q), weight=bits(w), k_cache=bits(kc), block_tables=tables.numpy(),
                        query_start_loc=qsl, lens=np.int32(lens), cached_lens=np.int32(clens),
                        dims=np.int32([nH, D, bs, batch, maxblk, top_k]), expected_scores=scores.astype(np.float32),
                        expected_topk=topk)


if __name__ == "__main__":
    gqa("gqa_decode_bf16.npz", 101, [1, 1, 1, 1], [150, 0, 31, 32], 8, 2, 128, 16, torch.bfloat16)
    gqa("gqa_decode_fp16_d64.npz", 102, [1, 1, 1], [63, 140, 17], 14, 2, 64, 16, torch.float16)
    gqa("gqa_prefill_bf16.npz", 103, [70, 9, 33], [0, 100, 64], 8, 1, 128, 16, torch.bfloat16)
    mla("mla_decode.npz", 104, [1, 1, 1], [130, 0, 65], 16, 32)
    mla("mla_prefill_topk.npz", 105, [3, 2], [40, 70], 8, 32, top_k=16)
    rope("rope_and_cache_bf16.npz", 106, 11, 8, 2, 128, 128, 16, 4, torch.bfloat16)
    rope("rope_and_cache_fp16_partial.npz", 107, 7, 4, 4, 128, 64, 16, 2, torch.float16)
    indexer("indexer_bf16.npz", 108, [2, 1, 3], [21, 40, 0], 16, 16, 8)
    print("written to", HERE)
