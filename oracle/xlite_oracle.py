"""CPU oracle for the Xlite attention hot path.

TEST INFRASTRUCTURE ONLY. Nothing in the shipped package may import this
module; it is the checker for the HIP kernels (tests, the smoke check and the
CPU-baseline leg of the benchmark), never the thing measured or shipped.

Every function restates, in plain PyTorch on CPU tensors, the arithmetic of one
piece of the reference (paths under /root/reference/):

  rope_and_cache_ref   xlite/tests/kernels/rope_and_cache.py:27-41,84-103 (golden) with the
                       rounding order and cache write of
                       xlite/csrc/kernels/rope_and_cache.h:93-129,486-501,563-600
  gather_paged         xlite/tests/kernels/attention.py:186-220 (paged layout),
                       xlite/csrc/kernels/attention.h:147,156
  attention_ref        xlite/tests/kernels/attention.py:109-117,139-184;
                       xlite/tests/models/llama.py:207-259
  mla_attention_ref    xlite/tests/kernels/mla.py:163-202, top-k mask :293-333;
                       xlite/tests/models/deepseek_v3.py:675-690
  mla_v2_ref           xlite/csrc/_C.cpp:1234-1301 (einsum + attention + einsum)
  mla_v3_ref           xlite/tests/kernels/mla_v3.py:163-192; xlite/csrc/kernels/mla_v3.h:534-536
  gather_sparse_kv_cache_ref  xlite/tests/kernels/gather_sparse_kv_cache.py:102-116
  mha_forward_ref      xlite/csrc/model.cpp:480-600 (composition of the pieces; the projections are fp32
                       matrix products rounded once)
  mla_forward_ref      xlite/csrc/model.cpp:333-482 (composition of the MLA pieces; golden of the whole layer:
                       xlite/tests/models/deepseek_v3.py:629-692)
  indexer_scores_ref   xlite/tests/kernels/indexer_scores.py:96-118 (golden) with the 16-bit rounding of
                       the per-head products of xlite/csrc/kernels/indexer_scores.h:214-217
  indexer_topk_ref     xlite/tests/kernels/indexer_topk.py:139-152
  rope_complex_ref     xlite/tests/kernels/rope_complex.py:31-41 with the fp32 operation order of
                       xlite/csrc/kernels/rope_complex_and_cache.h:165-205
  mla_prepare_ref      xlite/tests/kernels/mla_prepare.py:27-45,90-109
  layernorm_ref        xlite/tests/kernels/layernorm.py:22-23; muls_ref xlite/tests/kernels/muls.py:23
  rope_complex_and_cache_ref  xlite/csrc/kernels/rope_complex_and_cache.h:12-241 (any column offset; cache form)
  indexer_forward_ref  xlite/csrc/model.cpp:285-330 (composition; golden of the whole indexer:
                       xlite/tests/models/deepseek_v3.py:543-568)
  qk_rms_norm_ref      xlite/csrc/kernels/qk_rms_norm.h:32-54 over rmsnorm_ref
                       (xlite/tests/kernels/rmsnorm.py:24-30)
  einsum_ref           xlite/tests/kernels/einsum_mht_mhd.py:44
  prepare_attn_ref     xlite/csrc/runtime.cpp:438-534
  get_tile_size_of_cached_kv_ref  xlite/csrc/auto_tuner.cpp:10-210
  quantize_kv_int8 / dequantize_kv_int8   not in the reference (its caches are never
                       quantised); definition from the benchmark contract:
                       scale = absmax/127 per (token, kv head), symmetric.
  quantize_kv_fp8 / dequantize_kv_fp8     not in the reference either; the same layout with OCP e4m3 bytes,
                       scale = absmax/448 (the format's largest value), round to nearest even.

Pinning status (what independent evidence each function is checked against in
tests/test_oracle_pins.py):
  attention_ref, mla_attention_ref, mla_v3_ref: fp64 triple-loop C restatement
      (oracle/brute.c), torch scaled_dot_product_attention on gathered dense K/V,
      closed forms (single key -> v0; equal keys -> mean of V), block-permutation
      invariance, prefill rows == the same rows issued as decode steps, absorbed
      MLA == naive per-head MLA in fp64.
  rope_and_cache_ref, rope_complex_ref: C restatement with explicit bf16/fp16
      rounding (oracle/brute.c), rotation by position 0 is the identity, norm
      preservation, complex-multiply identity in fp64.
  mla_prepare_ref, qk_rms_norm_ref: composition of pinned pieces + RMSNorm closed forms (a vector of
      equal entries c normalises to sign(c) * w + b; scale invariance; per-vector Python loop).
  mha_forward_ref, mla_forward_ref: compositions of pinned pieces; mla_forward_ref additionally against the
      textbook model form (per-head keys and values from the whole token history, rope as a complex product,
      no paging, no absorption) over a prefill and two decode steps.
  layernorm_ref: torch.nn.functional.layer_norm; a constant row normalises to the bias. muls_ref: exact
      for power-of-two scales. rope_complex_and_cache_ref: equals rope_complex_ref on the last columns; complex
      product in fp64; the cache form against a Python loop. indexer_forward_ref: the textbook indexer (fp32,
      no cache, no paging; the golden's orthogonal rotate_activation cancels in q . k) selects the same sets.
  gather_*: brute-force Python loops.
  indexer_scores_ref: pure-Python triple loop in float (tiny case); one head with weight 1 reduces to
      q . k; with no intermediate rounding the weighted sum equals (sum_h w_h q_h) . k (linearity).
  indexer_topk_ref: numpy argsort on the same scores; every selected score >= every unselected one.
  get_tile_size_of_cached_kv_ref, prepare_attn_ref: hand-computed cases.
  int8 / fp8 KV: parity unpinned by the reference (feature absent there). int8 is pinned by the round-trip bound
      |x - dequant(quant(x))| <= scale/2; fp8 by brute force over all 256 codes of OCP e4m3 (decoded values from
      the format's definition, quantisation = nearest code, ties to even, against a search over the code table).
"""
from __future__ import annotations

import math
from typing import List, Optional, Sequence, Tuple

import numpy as np
import torch

MAX_KV_TILE_SIZE = 8192          # xlite/csrc/auto_tuner.h:13
MIN_KV_TILE_SIZE = 4096          # xlite/csrc/auto_tuner.h:12
SINGLE_BATCH_MIN_KV_TILE_SIZE = 1024  # xlite/csrc/auto_tuner.h:11
XLITE_MAX_M0 = 128               # xlite/csrc/kernels/kernel_param.h:33


# --------------------------------------------------------------------------
# paged layout
# --------------------------------------------------------------------------
def gather_paged(cache: torch.Tensor, table_row: Sequence[int], n_tokens: int) -> torch.Tensor:
    """Tokens 0..n_tokens-1 of one sequence: token p lives at cache[table[p // bs], p % bs]."""
    bs = cache.shape[1]
    nblk = (n_tokens + bs - 1) // bs
    idx = torch.as_tensor(list(table_row[:nblk]), dtype=torch.long)
    flat = cache[idx].reshape(nblk * bs, *cache.shape[2:])
    return flat[:n_tokens]


# --------------------------------------------------------------------------
# rope_and_cache
# --------------------------------------------------------------------------
def _neox_rotate(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor, rot_dim: int) -> torch.Tensor:
    """x [T, H, D] in fp16/bf16; cos/sin [T, rot_dim/2] same dtype. Each product is rounded to
    the storage dtype before the add/sub, then the sum is rounded again."""
    dt = x.dtype
    half = rot_dim // 2
    x1 = x[..., :half].float()
    x2 = x[..., half:rot_dim].float()
    c = cos.float().unsqueeze(1)
    s = sin.float().unsqueeze(1)
    a = (x1 * c).to(dt).float()
    b = (x2 * s).to(dt).float()
    e = (x2 * c).to(dt).float()
    f = (x1 * s).to(dt).float()
    out = x.clone()
    out[..., :half] = (a - b).to(dt)
    out[..., half:rot_dim] = (e + f).to(dt)
    return out


def rope_and_cache_ref(inout, k_cache, v_cache, position, cosin, slot_mapping, n_heads, n_kv_heads,
                       head_dim, rot_dim, block_size, mrope_mask_h: int = 0, mrope_mask_w: int = 0):
    """In place on CPU tensors, same contract as the operator."""
    T = inout.shape[0]
    dt = inout.dtype
    half = rot_dim // 2
    row = inout.view(T, n_heads + 2 * n_kv_heads, head_dim)
    q = row[:, :n_heads]
    k = row[:, n_heads:n_heads + n_kv_heads]
    v = row[:, n_heads + n_kv_heads:]
    if mrope_mask_h or mrope_mask_w:
        pos = position.view(3, T).long()
        cs_t, cs_h, cs_w = cosin[pos[0]], cosin[pos[1]], cosin[pos[2]]
        lane = torch.arange(half)
        in_h = torch.tensor([(mrope_mask_h >> int(j)) & 1 for j in lane], dtype=torch.bool)
        in_w = torch.tensor([(mrope_mask_w >> int(j)) & 1 for j in lane], dtype=torch.bool)
        cos = torch.where(in_h, cs_h[:, :half], torch.where(in_w, cs_w[:, :half], cs_t[:, :half]))
        sin = torch.where(in_h, cs_h[:, half:], torch.where(in_w, cs_w[:, half:], cs_t[:, half:]))
    else:
        cs = cosin[position.view(-1).long()]
        cos, sin = cs[:, :half], cs[:, half:]
    k_new = _neox_rotate(k, cos, sin, rot_dim)
    q_new = _neox_rotate(q, cos, sin, rot_dim)
    scale = 1.0 / math.sqrt(float(head_dim))
    if dt == torch.float16:
        # the fp16 kernel multiplies by the scale rounded to fp16 (rope_and_cache.h:219,595)
        scale_t = torch.tensor(scale, dtype=torch.float32).to(torch.float16).float()
    else:
        scale_t = torch.tensor(scale, dtype=torch.float32)
    q_new = (q_new.float() * scale_t).to(dt)
    slots = slot_mapping.view(-1).long() & 0xFFFFFFFF
    blk = slots // block_size
    off = slots % block_size
    for t in range(T):  # sequential: a later token wins on duplicate slots
        k_cache[blk[t], off[t]] = k_new[t]
        v_cache[blk[t], off[t]] = v[t]
    k.copy_(k_new)
    q.copy_(q_new)


# --------------------------------------------------------------------------
# attention
# --------------------------------------------------------------------------
def causal_mask(qlen: int, clen: int) -> torch.Tensor:
    """[qlen, clen + qlen] additive mask: column j is visible to row r iff j <= clen + r."""
    cols = torch.arange(clen + qlen).unsqueeze(0)
    rows = torch.arange(qlen).unsqueeze(1)
    m = torch.zeros(qlen, clen + qlen, dtype=torch.float32)
    m[cols > clen + rows] = float("-inf")
    return m


def attention_ref(qkv, k_cache, v_cache, query_start_loc, lens, cached_lens, block_tables, n_heads,
                  n_kv_heads, head_dim, block_size, batch, max_num_block,
                  k_scale: Optional[torch.Tensor] = None, v_scale: Optional[torch.Tensor] = None,
                  seqs: Optional[Sequence[int]] = None) -> torch.Tensor:
    """Returns fp32 [T, n_heads*head_dim] (rows of sequences not in `seqs` stay zero).

    fp32 accumulation from the 16-bit inputs; no softmax scale (q is pre-scaled). With
    k_scale/v_scale the caches are int8 and are dequantised first.
    """
    T = qkv.shape[0]
    g = n_heads // n_kv_heads
    out = torch.zeros(T, n_heads * head_dim, dtype=torch.float32)
    qsl = [int(x) for x in query_start_loc]
    ql = [int(x) for x in lens]
    cl = [int(x) for x in cached_lens]
    tables = block_tables.view(batch, max_num_block)
    q_all = qkv.view(T, n_heads + 2 * n_kv_heads, head_dim)[:, :n_heads]
    for i in (range(batch) if seqs is None else seqs):
        qlen, clen, st = ql[i], cl[i], qsl[i]
        if qlen == 0:
            continue
        n = clen + qlen
        row = tables[i].tolist()
        keys = gather_paged(k_cache, row, n).float()
        vals = gather_paged(v_cache, row, n).float()
        if k_scale is not None:
            keys = keys * gather_paged(k_scale, row, n).float().unsqueeze(-1)
            vals = vals * gather_paged(v_scale, row, n).float().unsqueeze(-1)
        q = q_all[st:st + qlen].float()                       # [qlen, nH, d]
        keys = keys.repeat_interleave(g, dim=1)                # [n, nH, d]
        vals = vals.repeat_interleave(g, dim=1)
        scores = torch.einsum("qhd,nhd->hqn", q, keys) + causal_mask(qlen, clen).unsqueeze(0)
        probs = torch.softmax(scores, dim=-1)
        o = torch.einsum("hqn,nhd->qhd", probs, vals)
        out[st:st + qlen] = o.reshape(qlen, n_heads * head_dim)
    return out


# --------------------------------------------------------------------------
# MLA
# --------------------------------------------------------------------------
def mla_attention_ref(q_absorb, qr, k_cache, pe_cache, query_start_loc, lens, cached_lens,
                      block_tables, n_heads, rope_head_dim, kv_lora_rank, block_size, batch,
                      max_num_blocks, scale, topk_indices: Optional[torch.Tensor] = None,
                      top_k: int = 0, seqs: Optional[Sequence[int]] = None) -> torch.Tensor:
    """Absorbed MLA attention, fp32 [T, n_heads, kv_lora_rank]."""
    T = q_absorb.shape[0]
    out = torch.zeros(T, n_heads, kv_lora_rank, dtype=torch.float32)
    qa = q_absorb.view(T, n_heads, kv_lora_rank)
    qrr = qr.view(T, n_heads, rope_head_dim)
    kc = k_cache.view(k_cache.shape[0], block_size, kv_lora_rank)
    pc = pe_cache.view(pe_cache.shape[0], block_size, rope_head_dim)
    tables = block_tables.view(batch, max_num_blocks)
    for i in (range(batch) if seqs is None else seqs):
        qlen, clen, st = int(lens[i]), int(cached_lens[i]), int(query_start_loc[i])
        if qlen == 0:
            continue
        n = clen + qlen
        row = tables[i].tolist()
        lat = gather_paged(kc, row, n).float()
        pe = gather_paged(pc, row, n).float()
        s = torch.einsum("qhc,nc->qhn", qa[st:st + qlen].float(), lat)
        s = s + torch.einsum("qhr,nr->qhn", qrr[st:st + qlen].float(), pe)
        s = s * scale + causal_mask(qlen, clen).unsqueeze(1)
        if top_k > 0:
            # the index list of a row applies only when its causal range is longer than top_k
            # (xlite/csrc/kernels/mla_v2.h:697-699); indices outside the range are ignored
            idx = topk_indices.view(T, top_k)[st:st + qlen].long()
            keep = torch.zeros(qlen, n)
            for r in range(qlen):
                limit = clen + r + 1
                if limit > top_k:
                    keep[r] = float("-inf")
                    good = idx[r][(idx[r] >= 0) & (idx[r] < limit)]
                    keep[r, good] = 0.0
            s = s + keep.unsqueeze(1)
        p = torch.softmax(s, dim=-1)
        p = torch.nan_to_num(p, nan=0.0)  # a row with no visible key yields zeros
        out[st:st + qlen] = torch.einsum("qhn,nc->qhc", p, lat)
    return out


def einsum_ref(mht: torch.Tensor, w: torch.Tensor, w_is_hdt: bool = False) -> torch.Tensor:
    """fp32 result of einsum('mht,htd->mhd') (or 'mht,hdt->mhd')."""
    if w_is_hdt:
        return torch.einsum("mht,hdt->mhd", mht.float(), w.float())
    return torch.einsum("mht,htd->mhd", mht.float(), w.float())


def mla_v2_ref(q_with_qr, qr, k_cache, pe_cache, wuk_t, wuv, query_start_loc, lens, cached_lens,
               block_tables, n_heads, rope_head_dim, nope_head_dim, v_head_dim, kv_lora_rank,
               block_size, batch, max_num_blocks, scale, topk_indices=None, top_k=0,
               round_intermediates: bool = True) -> torch.Tensor:
    """The three-stage operator. The reference stores q_absorb and o_absorb in the activation
    dtype between stages (xlite/csrc/_C.cpp:1257-1262), which `round_intermediates` reproduces."""
    T = q_with_qr.shape[0]
    dt = q_with_qr.dtype
    q_nope = q_with_qr.view(T, n_heads, nope_head_dim + rope_head_dim)[..., :nope_head_dim]
    q_abs = einsum_ref(q_nope, wuk_t.view(n_heads, nope_head_dim, kv_lora_rank))
    if round_intermediates:
        q_abs = q_abs.to(dt)
    o_abs = mla_attention_ref(q_abs, qr, k_cache, pe_cache, query_start_loc, lens, cached_lens,
                              block_tables, n_heads, rope_head_dim, kv_lora_rank, block_size, batch,
                              max_num_blocks, scale, topk_indices, top_k)
    if round_intermediates:
        o_abs = o_abs.to(dt)
    return einsum_ref(o_abs, wuv.view(n_heads, kv_lora_rank, v_head_dim))


def mla_v3_ref(q_absorb, qr, k_dense, pe_dense, query_start_loc, lens, cached_lens, n_heads,
               rope_head_dim, kv_lora_rank, batch, index_topk, scale) -> torch.Tensor:
    T = q_absorb.shape[0]
    out = torch.zeros(T, n_heads, kv_lora_rank, dtype=torch.float32)
    qa = q_absorb.view(T, n_heads, kv_lora_rank)
    qrr = qr.view(T, n_heads, rope_head_dim)
    kd = k_dense.view(batch, index_topk, kv_lora_rank)
    pd = pe_dense.view(batch, index_topk, rope_head_dim)
    for i in range(batch):
        qlen, clen, st = int(lens[i]), int(cached_lens[i]), int(query_start_loc[i])
        n = min(clen + qlen, index_topk)
        if qlen == 0 or n <= 0:
            continue
        lat = kd[i, :n].float()
        pe = pd[i, :n].float()
        s = torch.einsum("qhc,nc->qhn", qa[st:st + qlen].float(), lat)
        s = (s + torch.einsum("qhr,nr->qhn", qrr[st:st + qlen].float(), pe)) * scale
        p = torch.softmax(s, dim=-1)
        out[st:st + qlen] = torch.einsum("qhn,nc->qhc", p, lat)
    return out


def gather_sparse_kv_cache_ref(k_cache, pe_cache, block_tables, topk_indices, query_lens,
                               cached_lens, k_dense, pe_dense, batch, index_topk, block_size,
                               max_num_blocks, kv_lora_rank, rope_head_dim):
    """In place; slots beyond min(qlen + clen, index_topk) are not touched."""
    kc = k_cache.view(-1, block_size, kv_lora_rank)
    pc = pe_cache.view(-1, block_size, rope_head_dim)
    kd = k_dense.view(batch, index_topk, kv_lora_rank)
    pd = pe_dense.view(batch, index_topk, rope_head_dim)
    tables = block_tables.view(batch, max_num_blocks)
    idx = topk_indices.view(batch, index_topk)
    for b in range(batch):
        valid = min(int(query_lens[b]) + int(cached_lens[b]), index_topk)
        for i in range(valid):
            tok = int(idx[b, i])
            phys = int(tables[b, tok // block_size])
            kd[b, i] = kc[phys, tok % block_size]
            pd[b, i] = pc[phys, tok % block_size]


# --------------------------------------------------------------------------
# model-level caller
# --------------------------------------------------------------------------
def mha_forward_ref(hidden, wqkv, wo, k_cache, v_cache, lens, cached_lens, block_tables, cosin, n_heads, n_kv_heads,
                    head_dim, rot_dim, block_size, q_norm=None, k_norm=None, norm_eps=1e-6):
    """xlite/csrc/model.cpp:480-600 as a composition of the pieces above: metadata (prepare_attn_ref), QKV
    projection (fp32 accumulate, one rounding), optional per-head qk RMSNorm, rope_and_cache (in place on the
    caches), attention, output projection. `block_tables[i]` lists the blocks of sequence i."""
    dt = hidden.dtype
    meta = prepare_attn_ref(lens, cached_lens, block_tables, block_size)
    qkv = (hidden.float() @ wqkv.float()).to(dt)
    if q_norm is not None:
        qkv = qk_rms_norm_ref(qkv, q_norm, None, k_norm, None, norm_eps, head_dim, n_heads, head_dim, n_kv_heads,
                              n_heads * head_dim)
    pos = torch.tensor(meta["position"], dtype=torch.int64)
    slots = torch.tensor(meta["slot_mapping"], dtype=torch.int32)
    rope_and_cache_ref(qkv, k_cache, v_cache, pos, cosin, slots, n_heads, n_kv_heads, head_dim, rot_dim, block_size)
    batch = len(lens)
    attn = attention_ref(qkv, k_cache, v_cache, torch.tensor(meta["query_start_loc"], dtype=torch.int32),
                         torch.tensor(list(lens), dtype=torch.int32), torch.tensor(list(cached_lens), dtype=torch.int32),
                         torch.from_numpy(meta["block_tables"]).flatten(), n_heads, n_kv_heads, head_dim, block_size, batch,
                         meta["max_num_blocks"])
    return (attn.to(dt).float().reshape(hidden.shape[0], -1) @ wo.float()).to(dt)


def mla_forward_ref(hidden, wqkv_a, q_norm, kv_norm, wq_b, wuk_t, wuv, wo, k_cache, pe_cache, lens, cached_lens,
                    block_tables, freqs, n_heads, q_lora_rank, kv_lora_rank, nope_head_dim, rope_head_dim, v_head_dim,
                    block_size, scale, norm_eps=1e-6, indexer=None, index_k_cache=None, topk_override=None):
    """xlite/csrc/model.cpp:333-482 as a composition of the pieces above: metadata (prepare_attn_ref), QKV_A
    projection, mla_prepare (in place on the caches), Q_B projection, rope_complex, mla_v2 (absorb einsum,
    absorbed attention, W_UV einsum), output projection; every stage leaves its result in the activation
    dtype, as the reference's tensors between operators do. `block_tables[i]` lists the blocks of sequence i.
    `indexer`: dict with wk_weights_proj, k_norm, k_norm_bias, wq_b, index_n_heads, index_head_dim, index_topk -
    the DSA branch (indexer_forward_ref) then masks the attention with its position lists; `index_k_cache` is
    written in place. `topk_override` [T, index_topk] replaces the lists the branch selected (to check the
    attention on lists chosen elsewhere). Returns the output, and with an indexer (output, lists or None)."""
    dt = hidden.dtype
    T = hidden.shape[0]
    meta = prepare_attn_ref(lens, cached_lens, block_tables, block_size)
    pos = torch.tensor(meta["position"], dtype=torch.int64)
    slots = torch.tensor(meta["slot_mapping"], dtype=torch.int32)
    qkvc = (hidden.float() @ wqkv_a.float()).to(dt)
    norm_qc = torch.empty(T, q_lora_rank, dtype=dt)
    norm_kvc = torch.empty(T, kv_lora_rank, dtype=dt)
    mla_prepare_ref(qkvc, q_norm, torch.zeros_like(q_norm), norm_qc, kv_norm, torch.zeros_like(kv_norm), norm_kvc, freqs,
                    pos, q_lora_rank, kv_lora_rank, rope_head_dim, block_size, k_cache, pe_cache, slots, norm_eps)
    batch = len(lens)
    qsl = torch.tensor(meta["query_start_loc"], dtype=torch.int32)
    lens_t, clens_t = torch.tensor(list(lens), dtype=torch.int32), torch.tensor(list(cached_lens), dtype=torch.int32)
    tables = torch.from_numpy(meta["block_tables"]).flatten()
    topk_indices, top_k = None, 0
    if indexer is not None:
        res = indexer_forward_ref(hidden, norm_qc, indexer["wk_weights_proj"], indexer["k_norm"], indexer["k_norm_bias"],
                                  indexer["wq_b"], index_k_cache, freqs, pos, slots, qsl, lens_t, clens_t, tables,
                                  indexer["index_n_heads"], indexer["index_head_dim"], rope_head_dim, indexer["index_topk"],
                                  block_size, batch, meta["max_num_blocks"], norm_eps)
        if res is not None:
            top_k = indexer["index_topk"]
            topk_indices = torch.full((T, top_k), -1, dtype=torch.int32)
            for i in range(batch):
                for r, row in enumerate(res[1][i]):
                    topk_indices[int(qsl[i]) + r, :len(row)] = torch.tensor(row, dtype=torch.int32)
    own_lists = topk_indices
    if topk_indices is not None and topk_override is not None:
        topk_indices = topk_override
    q_with_qr = (norm_qc.float() @ wq_b.float()).to(dt)
    q_pe = rope_complex_ref(n_heads, nope_head_dim + rope_head_dim, rope_head_dim, q_with_qr, freqs, pos)
    attn = mla_v2_ref(q_with_qr, q_pe.reshape(T, -1), k_cache, pe_cache, wuk_t, wuv, qsl, lens_t, clens_t, tables,
                      n_heads, rope_head_dim, nope_head_dim, v_head_dim, kv_lora_rank, block_size, batch,
                      meta["max_num_blocks"], scale, topk_indices, top_k)
    out = (attn.to(dt).float().reshape(T, -1) @ wo.float()).to(dt)
    return out if indexer is None else (out, own_lists)


# --------------------------------------------------------------------------
# DSA indexer
# --------------------------------------------------------------------------
def indexer_scores_ref(q, k_cache, weight, query_start_loc, lens, cached_lens, block_tables, n_heads, head_dim,
                       block_size, batch, max_num_block, round_heads: bool = True) -> List[torch.Tensor]:
    """Per sequence i: fp32 tensor [lens[i], cached_lens[i] + lens[i]] of
    sum_h weight[t, head_dim + h] * (q[t, h] . k[j]); every query row sees every position of its sequence.
    `round_heads` rounds the per-head products to the activation dtype first, as the reference kernel does
    when it parks them in L1 (the golden, computed in the activation dtype, rounds there too)."""
    kc = k_cache.view(-1, block_size, head_dim)
    tables = block_tables.view(batch, max_num_block)
    out = []
    for i in range(batch):
        s, ql, cl = int(query_start_loc[i]), int(lens[i]), int(cached_lens[i])
        total = cl + ql
        k = gather_paged(kc, tables[i].tolist(), total).float()                      # [total, d]
        qi = q[s:s + ql].reshape(ql, n_heads, head_dim).float()
        w = weight[s:s + ql].reshape(ql, head_dim + n_heads)[:, head_dim:].float()    # [ql, H]
        res = torch.empty(ql, total)
        for r0 in range(0, ql, 64):      # row chunks bound the [rows, heads, positions] intermediate
            dots = torch.einsum("shd,td->sht", qi[r0:r0 + 64], k)
            if round_heads:
                dots = dots.to(q.dtype).float()
            res[r0:r0 + 64] = torch.einsum("sht,sh->st", dots, w[r0:r0 + 64])
        out.append(res)
    return out


def indexer_topk_ref(scores: Sequence[torch.Tensor], top_k: int) -> List[List[List[int]]]:
    """Per sequence, per query row: the positions of the min(top_k, n) largest scores, ascending; ties at
    the k-th score go to the lower positions."""
    res = []
    for sc in scores:
        rows = []
        n = sc.shape[1]
        for r in range(sc.shape[0]):
            if n <= top_k:
                rows.append(list(range(n)))
                continue
            v = sc[r].double().numpy()
            order = np.lexsort((np.arange(n), -v))      # by score descending, then position ascending
            rows.append(sorted(int(x) for x in order[:top_k]))
        res.append(rows)
    return res


# --------------------------------------------------------------------------
# rope_complex / mla_prepare
# --------------------------------------------------------------------------
def _freqs_as_cos_sin(freqs: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    f = torch.view_as_real(freqs) if freqs.is_complex() else freqs.view(freqs.shape[0], -1, 2)
    return f[..., 0].float(), f[..., 1].float()


def _rope_interleaved(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    """x [..., rope_dim] interleaved (re, im) pairs in fp32; cos/sin broadcastable [..., rope_dim/2].
    Four fp32 products, one fp32 add/sub each, output [re... | im...] (still fp32)."""
    xe = x[..., 0::2]
    xo = x[..., 1::2]
    re = xe * cos - xo * sin     # torch evaluates the two products separately, then subtracts
    im = xe * sin + xo * cos
    return torch.cat([re, im], dim=-1)


def rope_complex_ref(n_local_heads, step_dim, rope_dim, input_with_r, freqs, position):
    """Returns [T, n_local_heads, rope_dim] in the input dtype."""
    T = input_with_r.shape[0]
    dt = input_with_r.dtype
    x = input_with_r.view(T, n_local_heads, step_dim)[..., step_dim - rope_dim:].float()
    cos, sin = _freqs_as_cos_sin(freqs)
    pos = position.view(-1).long()
    y = _rope_interleaved(x, cos[pos].unsqueeze(1), sin[pos].unsqueeze(1))
    return y.to(dt)


def rmsnorm_ref(x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor, eps: float) -> torch.Tensor:
    xf = x.float()
    var = xf.pow(2).mean(-1, keepdim=True)
    y = xf * torch.rsqrt(var + eps)
    return (weight.float() * y + bias.float()).to(x.dtype)


def qk_rms_norm_ref(qkv, q_norm, q_norm_bias, k_norm, k_norm_bias, norm_eps, q_norm_dim, q_cnt_per_token,
                    k_norm_dim, k_cnt_per_token, k_start_offset) -> torch.Tensor:
    """xlite/csrc/kernels/qk_rms_norm.h:32-54 (two independent RMSNorm passes over disjoint column ranges of
    the same rows), each pass the golden of xlite/tests/kernels/rmsnorm.py:24-30,49-51. Returns the new rows."""
    out = qkv.clone()
    T = qkv.shape[0]
    zq = torch.zeros(q_norm_dim, dtype=qkv.dtype) if q_norm_bias is None else q_norm_bias
    zk = torch.zeros(k_norm_dim, dtype=qkv.dtype) if k_norm_bias is None else k_norm_bias
    qs = qkv[:, :q_norm_dim * q_cnt_per_token].reshape(T, q_cnt_per_token, q_norm_dim)
    out[:, :q_norm_dim * q_cnt_per_token] = rmsnorm_ref(qs, q_norm, zq, norm_eps).reshape(T, -1)
    k_end = k_start_offset + k_norm_dim * k_cnt_per_token
    ks = qkv[:, k_start_offset:k_end].reshape(T, k_cnt_per_token, k_norm_dim)
    out[:, k_start_offset:k_end] = rmsnorm_ref(ks, k_norm, zk, norm_eps).reshape(T, -1)
    return out


def layernorm_ref(x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor, eps: float, norm_dim: int) -> torch.Tensor:
    """xlite/tests/kernels/layernorm.py:22-23 over the first norm_dim columns of every row (the launcher's
    defaults, xlite/csrc/op.cpp:607-628): fp32, biased variance, one rounding. Returns those columns."""
    xf = x[:, :norm_dim].float()
    mean = xf.mean(-1, keepdim=True)
    var = (xf - mean).pow(2).mean(-1, keepdim=True)
    y = (xf - mean) * torch.rsqrt(var + eps) * weight[:norm_dim].float() + bias[:norm_dim].float()
    return y.to(x.dtype)


def muls_ref(x: torch.Tensor, scale: float, calc_offset: int = 0, calc_num: Optional[int] = None) -> torch.Tensor:
    """xlite/tests/kernels/muls.py:23 restricted to a column range (xlite/csrc/op.cpp:1644-1680): a new tensor."""
    out = x.clone()
    end = x.shape[1] if calc_num is None else min(x.shape[1], calc_offset + calc_num)
    out[:, calc_offset:end] = (x[:, calc_offset:end].float() * scale).to(x.dtype)
    return out


def rope_complex_and_cache_ref(n_local_heads, step_dim, rope_dim, offset, vdim, input_with_r, freqs, position,
                               block_size=0, cache=None, slot_mapping=None):
    """xlite/csrc/kernels/rope_complex_and_cache.h:12-241: the rope_dim columns from `offset` of every head,
    rotated and de-interleaved. Without a cache: returns them [T, heads, rope_dim]. With a cache (one head):
    writes the vdim columns from `offset` (rotated part, then the rest unchanged) to cache[slot], in place."""
    T = input_with_r.shape[0]
    dt = input_with_r.dtype
    rows = input_with_r.view(T, n_local_heads, step_dim)
    cos, sin = _freqs_as_cos_sin(freqs)
    pos = position.view(-1).long()
    y = _rope_interleaved(rows[..., offset:offset + rope_dim].float(), cos[pos].unsqueeze(1), sin[pos].unsqueeze(1)).to(dt)
    if cache is None:
        return y
    assert n_local_heads == 1
    cv = cache.view(-1, block_size, vdim)
    slots = slot_mapping.view(-1).long() & 0xFFFFFFFF
    for t in range(T):
        cv[slots[t] // block_size, slots[t] % block_size, :rope_dim] = y[t, 0]
        cv[slots[t] // block_size, slots[t] % block_size, rope_dim:] = rows[t, 0, offset + rope_dim:offset + vdim]
    return None


def indexer_forward_ref(hidden, norm_qc, wk_weights_proj, k_norm, k_norm_bias, wq_b, index_k_cache, freqs, position,
                        slot_mapping, query_start_loc, lens, cached_lens, block_tables, index_n_heads, index_head_dim,
                        rope_head_dim, index_topk, block_size, batch, max_num_blocks, norm_eps):
    """xlite/csrc/model.cpp:285-330 as a composition: index key projection, LayerNorm, rope into the index key
    cache (in place), index query projection, rope, head weights times (heads * head_dim)^-0.5, scores, top-k.
    Returns (score rows per sequence, position lists per sequence), or None when no sequence can exceed
    index_topk."""
    dt = hidden.dtype
    T = hidden.shape[0]
    kw = (hidden.float() @ wk_weights_proj.float()).to(dt)
    kw[:, :index_head_dim] = layernorm_ref(kw, k_norm, k_norm_bias, norm_eps, index_head_dim)
    rope_complex_and_cache_ref(1, index_head_dim + index_n_heads, rope_head_dim, 0, index_head_dim, kw, freqs, position,
                               block_size, index_k_cache, slot_mapping)
    if max_num_blocks * block_size <= index_topk:
        return None
    q = (norm_qc.float() @ wq_b.float()).to(dt).view(T, index_n_heads, index_head_dim).clone()
    q[..., :rope_head_dim] = rope_complex_and_cache_ref(index_n_heads, index_head_dim, rope_head_dim, 0, 0,
                                                         q.reshape(T, -1), freqs, position)
    kw = muls_ref(kw, (index_n_heads * index_head_dim) ** -0.5, index_head_dim, index_n_heads)
    scores = indexer_scores_ref(q.reshape(T, -1), index_k_cache, kw, query_start_loc, lens, cached_lens, block_tables,
                                index_n_heads, index_head_dim, block_size, batch, max_num_blocks)
    return scores, indexer_topk_ref(scores, index_topk)


def mla_prepare_ref(attn_qkvc, q_norm, q_norm_bias, attn_norm_qc, kv_norm, kv_norm_bias,
                    attn_norm_kvc, freqs, position, q_lora_rank, kv_lora_rank, rope_head_dim,
                    block_size, k_cache, pe_cache, slot_mapping, norm_eps):
    """In place on CPU tensors."""
    T = attn_qkvc.shape[0]
    dt = attn_qkvc.dtype
    rows = attn_qkvc.view(T, q_lora_rank + kv_lora_rank + rope_head_dim)
    attn_norm_qc.view(T, q_lora_rank).copy_(rmsnorm_ref(rows[:, :q_lora_rank], q_norm, q_norm_bias, norm_eps))
    kvc = rmsnorm_ref(rows[:, q_lora_rank:q_lora_rank + kv_lora_rank], kv_norm, kv_norm_bias, norm_eps)
    attn_norm_kvc.view(T, kv_lora_rank).copy_(kvc)
    cos, sin = _freqs_as_cos_sin(freqs)
    pos = position.view(-1).long()
    pe = _rope_interleaved(rows[:, q_lora_rank + kv_lora_rank:].float(), cos[pos], sin[pos]).to(dt)
    rows[:, q_lora_rank + kv_lora_rank:] = pe
    if block_size:
        kc = k_cache.view(-1, block_size, kv_lora_rank)
        pc = pe_cache.view(-1, block_size, rope_head_dim)
        slots = slot_mapping.view(-1).long() & 0xFFFFFFFF
        for t in range(T):
            kc[slots[t] // block_size, slots[t] % block_size] = kvc[t]
            pc[slots[t] // block_size, slots[t] % block_size] = pe[t]


# --------------------------------------------------------------------------
# host metadata
# --------------------------------------------------------------------------
def prepare_attn_ref(lens: Sequence[int], cached_lens: Sequence[int],
                     block_tables: Sequence[Sequence[int]], block_size: int):
    batch = len(lens)
    if batch == 0:
        raise RuntimeError("invalid batchSize: 0")
    qsl, pos, slots, nblk = [], [], [], []
    start = 0
    for i in range(batch):
        qsl.append(start)
        start += lens[i]
        nblk.append((lens[i] + cached_lens[i] + block_size - 1) // block_size)
    max_nb = max(nblk)
    for i in range(batch):
        if len(block_tables[i]) < nblk[i]:
            raise RuntimeError("block table too small")
        for j in range(lens[i]):
            p = cached_lens[i] + j
            pos.append(p)
            slots.append(block_tables[i][p // block_size] * block_size + p % block_size)
    dense = np.zeros((batch, max_nb), dtype=np.int32)
    for i in range(batch):
        dense[i, :nblk[i]] = block_tables[i][:nblk[i]]
    return dict(query_start_loc=qsl, position=pos, slot_mapping=slots, block_tables=dense,
                max_num_blocks=max_nb, batched_tokens=start,
                is_decode=all(l == 1 for l in lens))


def _calc_task_num(clen, qlen, g, n_kv, tile):
    qtile = XLITE_MAX_M0 // g
    if qtile == 0:
        qtile = XLITE_MAX_M0
    qnum = (qlen + qtile - 1) // qtile
    kvnum = (clen + qlen + tile - 1) // tile
    valid = 0
    for idx in range(qnum * n_kv * kvnum):
        kvidx = idx % kvnum
        qidx = idx // (kvnum * n_kv)
        qstart = qidx * qtile
        qtl = min(qtile, qlen - qstart)
        if clen + qstart + qtl > kvidx * tile:
            valid += 1
    return valid


def get_tile_size_of_cached_kv_ref(cached_lens: List[int], query_lens: List[int],
                                   head_num_in_group: int, n_kv_heads: int, block_size: int,
                                   aic_num: int) -> int:
    f32 = np.float32
    if any(q != 1 for q in query_lens):
        return 6016 if aic_num == 24 else 8192
    batch = len(query_lens)
    if batch == 1:
        clen = float(cached_lens[0])
        tasks = int(round(1.5 * math.sqrt(clen / 1024.0) + 3))
        tasks = max(1, min(tasks, aic_num))
        tile = (int(math.ceil(clen)) + tasks - 1) // tasks
        tile = (tile + block_size - 1) // block_size * block_size
        return max(SINGLE_BATCH_MIN_KV_TILE_SIZE, min(tile, MAX_KV_TILE_SIZE))
    best, best_score = MAX_KV_TILE_SIZE, f32(-1.0)
    tile = MAX_KV_TILE_SIZE
    while tile >= MIN_KV_TILE_SIZE:
        tot, cnt, total_tasks = f32(0.0), 0, 0
        for c, q in zip(cached_lens, query_lens):
            kv = c + q
            if kv == 1:
                continue
            rem = kv % tile
            tot = f32(tot + (f32(1.0) if rem == 0 else f32(rem) / f32(tile)))
            cnt += 1
            total_tasks += _calc_task_num(c, q, head_num_in_group, n_kv_heads, tile)
        kv_score = f32(0.0) if cnt == 0 else f32(tot / f32(cnt))
        rem = total_tasks % aic_num
        task_score = f32(1.0) if rem == 0 else f32(rem) / f32(aic_num)
        size_score = f32(tile) / f32(MAX_KV_TILE_SIZE)
        score = f32(f32(f32(kv_score * f32(0.7)) + f32(task_score * f32(0.2))) + f32(size_score * f32(0.1)))
        if score > best_score:
            best_score, best = score, tile
        tile -= block_size
    return best


# --------------------------------------------------------------------------
# int8 KV cache
# --------------------------------------------------------------------------
def quantize_kv_int8(x: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """x [..., head_dim] -> (int8 same shape, fp32 scale [...]); scale = absmax/127."""
    xf = x.float()
    amax = xf.abs().amax(dim=-1)
    scale = amax / 127.0
    safe = torch.where(scale > 0, scale, torch.ones_like(scale))
    q = torch.clamp(torch.round(xf / safe.unsqueeze(-1)), -127, 127).to(torch.int8)
    return q, scale


def dequantize_kv_int8(q: torch.Tensor, scale: torch.Tensor) -> torch.Tensor:
    return q.float() * scale.unsqueeze(-1)


def quantize_kv_fp8(x: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """x [..., head_dim] -> (float8_e4m3fn same shape, fp32 scale [...]); scale = absmax/448 (the largest e4m3
    value), the quotient rounded to nearest even by torch's conversion (the OCP e4m3 format, no infinities)."""
    xf = x.float()
    amax = xf.abs().amax(dim=-1)
    scale = amax / 448.0
    safe = torch.where(scale > 0, scale, torch.ones_like(scale))
    q = (xf / safe.unsqueeze(-1)).to(torch.float8_e4m3fn)
    return q, scale


def dequantize_kv_fp8(q: torch.Tensor, scale: torch.Tensor) -> torch.Tensor:
    return q.float() * scale.unsqueeze(-1)
