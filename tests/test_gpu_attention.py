"""GPU parity of the GQA attention operator (decode, prefill, int8 KV) against the CPU oracle.
Tolerance for bf16/fp16 outputs: max abs <= 2e-2 and mean abs <= 2e-3 (5e-2 max for int8 KV)."""
import numpy as np
import pytest
import torch

from gvirt_amd import workloads as W
from oracle import xlite_oracle as O

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
MAX_ABS, MEAN_ABS, MAX_ABS_INT8 = 2e-2, 2e-3, 5e-2


def run_attention(rt, w, **kw):
    from gvirt_amd._C import attention
    s = w["shape"]
    d = W.to_device(w, DEV)
    d["output"].zero_()
    attention(rt, d["qkv"], d["k_cache"], d["v_cache"], d["output"], d["query_start_loc"], d["lens"],
              d["cached_lens"], d["block_tables"], s.n_heads, s.n_kv_heads, s.head_dim, s.block_size, w["batch"],
              w["max_num_block"], k_scale=d.get("k_scale"), v_scale=d.get("v_scale"), **kw)
    return d["output"].float().cpu()


def oracle_attention(w, seqs=None):
    s = w["shape"]
    return O.attention_ref(w["qkv"], w["k_cache"], w["v_cache"], w["query_start_loc"], w["lens"], w["cached_lens"],
                           w["block_tables"], s.n_heads, s.n_kv_heads, s.head_dim, s.block_size, w["batch"],
                           w["max_num_block"], w.get("k_scale"), w.get("v_scale"), seqs=seqs)


def check(got, ref, max_abs=MAX_ABS, mean_abs=MEAN_ABS, rows=None):
    if rows is not None:
        got, ref = got[rows], ref[rows]
    err = (got - ref).abs()
    assert float(err.max()) <= max_abs, "max abs err %g" % float(err.max())
    assert float(err.mean()) <= mean_abs, "mean abs err %g" % float(err.mean())


def generic_case(seed, lens, clens, nH, nKV, d, bs, dtype, rms=False):
    g = torch.Generator().manual_seed(seed)
    batch, T = len(lens), sum(lens)
    maxblk = max((l + c + bs - 1) // bs for l, c in zip(lens, clens))
    NB = batch * maxblk + 1
    qkv = torch.randn(T, nH + 2 * nKV, d, generator=g)
    kc = torch.randn(NB, bs, nKV, d, generator=g)
    vc = torch.randn(NB, bs, nKV, d, generator=g)
    if rms:  # the reference test normalises q, k, v rows (xlite/tests/kernels/attention.py:72-75)
        qkv, kc, vc = [x / x.pow(2).mean(-1, keepdim=True).add(1e-6).sqrt() for x in (qkv, kc, vc)]
    else:
        qkv[:, :nH] *= d ** -0.5
    tables = torch.randperm(NB, generator=g)[: batch * maxblk].int()
    shape = W.GqaShape("t", nH, nKV, d, bs, dtype)
    return dict(shape=shape, batch=batch, qkv=qkv.reshape(T, -1).to(dtype), k_cache=kc.to(dtype), v_cache=vc.to(dtype),
                output=torch.zeros(T, nH * d, dtype=dtype), query_start_loc=torch.tensor(np.cumsum([0] + lens[:-1]), dtype=torch.int32),
                lens=torch.tensor(lens, dtype=torch.int32), cached_lens=torch.tensor(clens, dtype=torch.int32),
                block_tables=tables, max_num_block=maxblk)


def test_config1_qwen2_05b_decode(rt):
    """Benchmark configuration 1 in full: also the one the CPU golden path runs completely."""
    w = W.gqa_decode(W.QWEN2_05B, W.c1_context_lengths(), W.SEED_BASE + 1)
    check(run_attention(rt, w), oracle_attention(w))


# model shapes of xlite/tests/kernels/attention.py:28-39
MODELS = [(1, 1, 64, torch.float16), (1, 1, 64, torch.bfloat16), (1, 1, 128, torch.bfloat16), (14, 2, 64, torch.bfloat16),
          (5, 1, 128, torch.bfloat16), (8, 1, 128, torch.bfloat16), (4, 1, 128, torch.bfloat16), (32, 32, 128, torch.float16),
          (20, 20, 128, torch.float16), (32, 8, 128, torch.bfloat16),
          # head_dim 256: the Qwen3.5 shape of xlite/tests/models/qwen3_5.py:67-71 (8 / 2 heads), and a 16-bit float one
          (8, 2, 256, torch.bfloat16), (4, 4, 256, torch.float16)]
# decode workloads of the same file (:50-59), contexts bounded to what the CPU oracle does in seconds
DECODE_WORK = [([0], [1]), ([1800], [1]), ([8, 13, 65, 11, 5], [1] * 5), ([4000] * 2, [1] * 2), ([16000, 127], [1] * 2),
               ([127, 128, 129, 255, 256, 257], [1] * 6)]


@pytest.mark.parametrize("model", MODELS)
@pytest.mark.parametrize("work", DECODE_WORK)
def test_decode_model_grid(rt, model, work):
    nH, nKV, d, dtype = model
    clens, lens = work
    w = generic_case(11, lens, clens, nH, nKV, d, 128, dtype, rms=True)
    check(run_attention(rt, w), oracle_attention(w))


def test_decode_special_cases(rt):
    # single visible key: the output is v0 exactly (softmax of one element is 1.0)
    w = generic_case(12, [1, 1], [0, 0], 8, 2, 128, 128, torch.bfloat16)
    got = run_attention(rt, w)
    v0 = torch.stack([w["v_cache"][w["block_tables"][i].long(), 0] for i in range(2)]).float()
    assert torch.equal(got, v0.repeat_interleave(4, 1).reshape(2, -1))
    # block permutation invariance: identity table over a re-packed cache gives identical bits
    w = generic_case(13, [1] * 3, [700, 300, 511], 14, 2, 64, 128, torch.bfloat16)
    a = run_attention(rt, w)
    t = w["block_tables"].long()
    w2 = dict(w); w2["k_cache"] = w["k_cache"][t].contiguous(); w2["v_cache"] = w["v_cache"][t].contiguous()
    w2["block_tables"] = torch.arange(t.numel(), dtype=torch.int32)
    assert torch.equal(a, run_attention(rt, w2))
    # idempotence: the ticket counters are left at zero, a second call gives the same bits
    assert torch.equal(a, run_attention(rt, w))
    # non power-of-two block size and a block size smaller than the split granularity
    for bs in (48, 16):
        w = generic_case(14, [1] * 2, [1000, 37], 8, 2, 128, bs, torch.bfloat16)
        check(run_attention(rt, w), oracle_attention(w))


@pytest.mark.parametrize("model", [(64, 2, 128, 128, torch.bfloat16), (64, 1, 128, 64, torch.float16), (40, 2, 128, 16, torch.bfloat16),
                                   (32, 8, 128, 8, torch.bfloat16), (8, 2, 128, 4, torch.bfloat16),
                                   (48, 2, 128, 48, torch.bfloat16), (8, 2, 128, 20, torch.bfloat16),
                                   (40, 2, 64, 128, torch.bfloat16), (6, 2, 64, 8, torch.float16)])
@pytest.mark.parametrize("work", DECODE_WORK)
def test_decode_wide_groups_and_small_blocks(rt, model, work):
    """More than 16 query heads per kv head, and block sizes that are not a multiple of 16: decode batches the
    streaming prefill kernel serves (a sequence's rows are one ragged M tile, the KV range is split)."""
    nH, nKV, d, bs, dtype = model
    clens, lens = work
    w = generic_case(15, lens, clens, nH, nKV, d, bs, dtype, rms=True)
    check(run_attention(rt, w), oracle_attention(w))


@pytest.mark.parametrize("model", [(28, 4, 128, torch.bfloat16), (16, 4, 16, torch.float16), (64, 4, 48, torch.bfloat16),
                                   (14, 2, 128, torch.bfloat16), (32, 2, 16, torch.float16), (6, 2, 32, torch.bfloat16),
                                   (16, 1, 128, torch.bfloat16), (7, 1, 16, torch.float16), (1, 1, 48, torch.bfloat16)])
def test_decode_few_kv_heads_position_groups_share_a_workgroup(rt, model):
    """Decode batches with 4, 2 or 1 kv heads of 128 elements (a model's share under tensor parallelism): 2, 4 or 8
    waves share a kv head, each with its own 16 positions of a step of 32, 64 or 128, and their results meet inside
    the workgroup. Visible ranges around every multiple of 16 up to two steps and around block ends (whole groups
    beyond the end re-read the last valid group), blocks of 16, 32, 48 and 128 positions, groups of 1 to 16 heads."""
    nH, nKV, bs, dtype = model
    ctx = [1, 2, 15, 16, 17, 31, 32, 33, 47, 48, 49, 63, 64, 65, 79, 80, 81, 96, 97, 111, 112, 113, 127, 128, 129, 143, 144, 145,
           160, 191, 192, 193, 255, 256, 257, 1000, 4097, 9000]
    w = generic_case(63, [1] * len(ctx), [c - 1 for c in ctx], nH, nKV, 128, bs, dtype)
    check(run_attention(rt, w), oracle_attention(w))
    # a handful of long sequences: every workgroup gets a slice of one, partials merged by the second kernel
    w = generic_case(64, [1] * 3, [20000, 7001, 12345], nH, nKV, 128, bs, dtype)
    check(run_attention(rt, w), oracle_attention(w))


@pytest.mark.parametrize("model", [(32, 8, 128, torch.bfloat16), (28, 4, 128, torch.bfloat16), (6, 3, 128, torch.float16),
                                   (14, 2, 64, torch.bfloat16)])
@pytest.mark.parametrize("kv_dtype", [None, torch.int8])
def test_decode_block_tables_beyond_the_multiply_high_lookup(rt, model, kv_dtype):
    """Positions become (block, offset) by a multiply-high with floor(2^32 / block_size) + 1, which is exact below
    2^32 / block_size positions; a block table that reaches further (here 4096 blocks of 1024 positions) makes the
    kernels divide instead. The same batch with the table cut to what the contexts need takes the multiply-high path
    and must give the same bits."""
    nH, nKV, d, dtype = model
    w = generic_case(67, [1] * 3, [2999, 1024, 17], nH, nKV, d, 1024, dtype)
    if kv_dtype is not None:
        w = quantised(w, kv_dtype)
    ref = oracle_attention(w)
    narrow = run_attention(rt, w)
    check(narrow, ref, max_abs=MAX_ABS if kv_dtype is None else MAX_ABS_INT8)
    wide = dict(w)
    rows = w["block_tables"].reshape(w["batch"], w["max_num_block"])
    wide["block_tables"] = torch.cat([rows, torch.zeros(w["batch"], 4096 - w["max_num_block"], dtype=torch.int32)], 1).reshape(-1)
    wide["max_num_block"] = 4096
    assert torch.equal(run_attention(rt, wide), narrow)


@pytest.mark.parametrize("model,batch,lo,hi,long_ones", [((32, 8, 128, 128, torch.bfloat16), 100, 1, 3000, [9000, 5000]),
                                                        ((32, 8, 128, 128, torch.bfloat16), 700, 1, 200, [2500]),
                                                        ((16, 8, 128, 16, torch.float16), 70, 1, 900, []),
                                                        ((64, 16, 128, 64, torch.bfloat16), 40, 100, 2000, []),
                                                        ((14, 2, 64, 128, torch.bfloat16), 100, 1, 1500, [7000]),
                                                        ((28, 4, 128, 128, torch.float16), 70, 1, 2000, [6000, 33]),
                                                        ((4, 1, 128, 16, torch.bfloat16), 30, 1, 700, [])])
def test_decode_ragged_batches_balanced_split(rt, model, batch, lo, hi, long_ones):
    """Ragged decode batches on the shapes of the streaming decode kernel: the sequences' steps are cut into
    equal chunks across workgroups, so chunks hold whole short sequences, tails and heads of long ones; more
    than 64 sequences take the prefix sums through LDS, more than 512 several sequences per thread. With fewer
    than 8 kv heads the waves of a kv head share a segment and combine their parts inside the workgroup."""
    nH, nKV, d, bs, dtype = model
    rng = np.random.default_rng(batch)
    clens = [int(x) for x in rng.integers(lo, hi, size=batch)]
    for i, v in enumerate(long_ones):
        clens[(7 * i + 3) % batch] = v
    w = generic_case(16, [1] * batch, clens, nH, nKV, d, bs, dtype, rms=True)
    check(run_attention(rt, w), oracle_attention(w))


@pytest.mark.parametrize("model", [(32, 8, 128, 128, torch.bfloat16), (14, 2, 64, 128, torch.bfloat16),
                                   (28, 4, 128, 16, torch.float16), (16, 1, 64, 64, torch.float16)])
@pytest.mark.parametrize("clens", [[40000], [33000, 150, 12000], [6000] * 5])
def test_decode_few_sequences_many_partials(rt, model, clens):
    """Few (row, head)s whose rows are cut into up to a chunk per compute unit: the merge sums the partial
    slots in parallel streams (side by side in a wave's lanes and in the four waves of a workgroup)."""
    nH, nKV, d, bs, dtype = model
    w = generic_case(23, [1] * len(clens), clens, nH, nKV, d, bs, dtype, rms=True)
    check(run_attention(rt, w), oracle_attention(w))


# sequences without rows and sequences with several, with as many rows as sequences (the batch shape the
# decode kernels are chosen by) and otherwise
ZERO_LEN_WORK = [([100, 50], [2, 0]), ([10, 700, 33], [0, 3, 0]), ([5, 9, 300], [1, 0, 1]), ([100, 50], [1, 0]),
                 ([0, 0, 0], [0, 3, 0]), ([40, 2000, 7, 129], [0, 0, 4, 0]), ([300, 20], [0, 1])]


@pytest.mark.parametrize("model", [(32, 8, 128, 128, torch.bfloat16), (14, 2, 64, 128, torch.bfloat16),
                                   (8, 1, 128, 16, torch.float16), (64, 2, 128, 128, torch.bfloat16),
                                   (8, 2, 128, 20, torch.bfloat16)])
@pytest.mark.parametrize("work", ZERO_LEN_WORK)
def test_zero_length_sequences(rt, model, work):
    """Decode iff every length is 1 (xlite/csrc/runtime.cpp:466-470); a batch with as many rows as sequences
    need not be one. Rows of absent sequences do not exist; row r of a sequence sees cached + r + 1 keys."""
    nH, nKV, d, bs, dtype = model
    clens, lens = work
    w = generic_case(31, lens, clens, nH, nKV, d, bs, dtype, rms=True)
    check(run_attention(rt, w), oracle_attention(w))


@pytest.mark.parametrize("batch", [100, 700])
def test_zero_length_sequences_many_rows(rt, batch):
    """The same with more rows than a wave has lanes (prefix sums of the split through LDS): lengths of 0, 1 and
    2 that add up to the number of sequences."""
    rng = np.random.default_rng(batch)
    lens = [1] * batch
    for i in rng.choice(batch // 2, size=batch // 5, replace=False):
        lens[2 * i], lens[2 * i + 1] = 2, 0
    clens = [int(x) for x in rng.integers(1, 900, size=batch)]
    w = generic_case(32, lens, clens, 32, 8, 128, 128, torch.bfloat16, rms=True)
    assert sum(lens) == batch
    check(run_attention(rt, w), oracle_attention(w))


KV_DTYPES = [torch.int8, torch.float8_e4m3fn]


def quantised(w, kv_dtype):
    """The same workload over a quantised cache (bytes + one fp32 scale per position and kv head)."""
    q = dict(w)
    q["k_cache"], q["k_scale"] = W.quantize_cache(w["k_cache"], kv_dtype)
    q["v_cache"], q["v_scale"] = W.quantize_cache(w["v_cache"], kv_dtype)
    return q


@pytest.mark.parametrize("kv_dtype", KV_DTYPES)
def test_decode_quantised_kv(rt, kv_dtype):
    ctx = [129, 4100, 640, 17, 2048, 9000]
    w = W.gqa_decode(W.LLAMA3_8B, ctx, 77, kv_dtype=kv_dtype)
    got = run_attention(rt, w)
    check(got, oracle_attention(w), max_abs=MAX_ABS_INT8)
    # and against the unquantised cache the error stays within the budget as well (fp8 keeps 3 mantissa bits)
    w16 = W.gqa_decode(W.LLAMA3_8B, ctx, 77)
    check(got, oracle_attention(w16), max_abs=MAX_ABS_INT8 if kv_dtype == torch.int8 else 0.15,
          mean_abs=1e-2 if kv_dtype == torch.int8 else 3e-2)


@pytest.mark.parametrize("kv_dtype", KV_DTYPES)
def test_decode_quantised_kv_ragged_batch(rt, kv_dtype):
    rng = np.random.default_rng(3)
    ctx = [int(x) for x in np.exp(rng.uniform(np.log(16), np.log(6000), 90))]
    w = W.gqa_decode(W.LLAMA3_8B, ctx, 78, kv_dtype=kv_dtype)
    check(run_attention(rt, w), oracle_attention(w), max_abs=MAX_ABS_INT8)


@pytest.mark.parametrize("kv_dtype", KV_DTYPES)
@pytest.mark.parametrize("model", [(32, 8, 16, torch.float16), (16, 16, 32, torch.bfloat16), (128, 8, 128, torch.bfloat16),
                                   (8, 8, 48, torch.float16), (24, 8, 16, torch.bfloat16)])
def test_decode_quantised_kv_byte_streaming_kernel_shapes(rt, kv_dtype, model):
    """Decode batches on the kernel that copies the cache bytes straight into LDS (head_dim 128, kv heads a multiple
    of 8): both activation types, one and two passes over the kv heads, groups of 1, 3, 4 and 16 query heads, blocks
    of 16, 32 and 48 positions (a step of 32 positions then spans two blocks), and visible ranges around every
    multiple of 16 and 32 (the padding rows of the last step re-read the last position)."""
    nH, nKV, bs, dtype = model
    ctx = [1, 2, 15, 16, 17, 31, 32, 33, 47, 48, 49, 63, 64, 65, 96, 97, 1000, 4097]
    w = quantised(generic_case(62, [1] * len(ctx), [c - 1 for c in ctx], nH, nKV, 128, bs, dtype), kv_dtype)
    check(run_attention(rt, w), oracle_attention(w), max_abs=MAX_ABS_INT8)


@pytest.mark.parametrize("kv_dtype", KV_DTYPES)
@pytest.mark.parametrize("model", [(28, 4, 128, torch.bfloat16), (16, 4, 16, torch.float16), (64, 4, 48, torch.bfloat16),
                                   (14, 2, 128, torch.float16), (32, 2, 16, torch.bfloat16), (2, 2, 32, torch.bfloat16)])
def test_decode_quantised_kv_few_kv_heads_position_groups_share_a_workgroup(rt, kv_dtype, model):
    """8-bit caches with 4 or 2 kv heads of 128 elements on the kernel that copies the cache bytes straight into LDS:
    2 or 4 waves share a kv head, each with its own 32 positions of a step of 64 or 128 (a copy instruction is then 2
    or 4 positions, the scales of a wave's group travel with it), and their results meet inside the workgroup. Visible
    ranges around every multiple of 16 up to two steps, block sizes of 16, 32, 48 and 128, groups of 1 to 16 heads."""
    nH, nKV, bs, dtype = model
    ctx = [1, 2, 15, 16, 17, 31, 32, 33, 47, 48, 49, 63, 64, 65, 79, 80, 81, 96, 97, 111, 112, 113, 127, 128, 129, 143, 144, 145,
           160, 191, 192, 193, 255, 256, 257, 1000, 4097, 9000]
    w = quantised(generic_case(65, [1] * len(ctx), [c - 1 for c in ctx], nH, nKV, 128, bs, dtype), kv_dtype)
    check(run_attention(rt, w), oracle_attention(w), max_abs=MAX_ABS_INT8)
    w = quantised(generic_case(66, [1] * 3, [20000, 7001, 12345], nH, nKV, 128, bs, dtype), kv_dtype)
    check(run_attention(rt, w), oracle_attention(w), max_abs=MAX_ABS_INT8)


@pytest.mark.parametrize("kv_dtype", KV_DTYPES)
@pytest.mark.parametrize("model", [(32, 8, 128, 128, torch.bfloat16), (14, 2, 64, 128, torch.float16), (28, 4, 128, 16, torch.bfloat16),
                                   (64, 2, 128, 128, torch.bfloat16), (8, 2, 128, 20, torch.float16)])
@pytest.mark.parametrize("work", [([0], [77]), ([128], [300]), ([0] * 4, [189, 65, 13, 545]), ([2047, 1500, 0, 900], [1, 1, 300, 1]),
                                  ([3000], [100]), ([700, 45, 4000], [1, 1, 1]), ([300, 0, 40], [5, 0, 2])])
def test_quantised_kv_prefill_mixed_and_other_decode_shapes(rt, kv_dtype, model, work):
    """Prefill, chunked prefill, decode rows mixed with a prefill, and decode shapes outside the streaming kernel
    (wide groups, odd block sizes) over int8 and fp8 caches: one `attention` call serves both phases, as the
    reference's model runner issues it (xlite/csrc/model.cpp:544-569). Inputs as the reference's test draws them
    (RMS-normalised rows, unscaled queries: xlite/tests/kernels/attention.py:72-75), and as the benchmark contract
    does (N(0,1), q scaled by 1/sqrt(head_dim) as rope_and_cache leaves it)."""
    nH, nKV, d, bs, dtype = model
    clens, lens = work
    for rms in (True, False):
        w = quantised(generic_case(61, lens, clens, nH, nKV, d, bs, dtype, rms=rms), kv_dtype)
        check(run_attention(rt, w), oracle_attention(w), max_abs=MAX_ABS_INT8)


@pytest.mark.parametrize("kv_dtype", KV_DTYPES)
@pytest.mark.parametrize("model", [(32, 8, 128, 128, torch.bfloat16), (32, 8, 128, 16, torch.float16), (28, 4, 128, 16, torch.float16),
                                   (64, 16, 128, 8, torch.bfloat16)])
@pytest.mark.parametrize("work", [([500, 0, 3000], [700, 1300, 600]), ([9000], [1500]), ([0, 6, 2047, 64], [2000, 1100, 1, 900])])
def test_quantised_prefill_read_on_the_fly_against_the_copy_path(rt, kv_dtype, model, work):
    """Long chunks over a quantised cache go through an fp16 copy of the visible blocks; with too little scratch for
    the copy (and, whatever the scratch, for short chunks) the prefill kernel reads the bytes and scales itself, with
    the copy's arithmetic. Without scratch there is no KV split either, so the two agree bit for bit where the copy
    path does not split (kv heads a multiple of 8 here) and to the last places where it does; both within the budget
    of the oracle."""
    nH, nKV, d, bs, dtype = model
    clens, lens = work
    assert sum(lens) * (nH // nKV) > 2048 * len(lens)          # by default: the copy
    w = quantised(generic_case(63, lens, clens, nH, nKV, d, bs, dtype, rms=True), kv_dtype)
    by_copy = run_attention(rt, w)
    on_the_fly = run_attention(rt, w, workspace_limit=0)
    if nKV % 8 == 0:
        assert torch.equal(by_copy, on_the_fly)
    assert float((by_copy - on_the_fly).abs().max()) <= 4e-3
    check(on_the_fly, oracle_attention(w), max_abs=MAX_ABS_INT8)


def test_quantised_prefill_without_any_scratch(rt):
    """No scratch at all: no copy, no KV split, one kernel; head_dim 64 has no such path and says what it needs."""
    w = quantised(generic_case(64, [300, 40], [700, 0], 32, 8, 128, 32, torch.bfloat16, rms=True), torch.int8)
    check(run_attention(rt, w, workspace_limit=0), oracle_attention(w), max_abs=MAX_ABS_INT8)
    w = quantised(generic_case(65, [300, 40], [700, 0], 14, 2, 64, 32, torch.bfloat16, rms=True), torch.int8)
    with pytest.raises(RuntimeError, match="workspace too small"):
        run_attention(rt, w, workspace_limit=0)


@pytest.mark.parametrize("kv_dtype", KV_DTYPES)
def test_quantised_kv_prefill_then_decode_through_quantise_on_write(rt, kv_dtype):
    """A prompt written into a quantised cache by rope_and_cache (quantise-on-write), attended to as a prefill, then
    decode steps that append to the same cache - against the oracle over a 16-bit cache quantised after every write."""
    from gvirt_amd._C import rope_and_cache, attention
    from oracle import xlite_oracle as O
    nH, nKV, d, bs = 16, 4, 128, 16
    dt = torch.bfloat16
    g = torch.Generator().manual_seed(71)
    prompts, steps = [45, 130, 7], 4
    mb = (max(prompts) + steps + bs - 1) // bs
    NB = len(prompts) * mb
    tables = torch.randperm(NB, generator=g).int().view(len(prompts), mb)
    fr = torch.outer(torch.arange(256).float(), 1.0 / (10000.0 ** (torch.arange(0, d, 2).float() / d)))
    cosin = torch.cat([fr.cos(), fr.sin()], -1).to(dt)
    kq = torch.zeros(NB, bs, nKV, d, dtype=torch.int8).view(kv_dtype).to(DEV)
    vq = torch.zeros_like(kq)
    ks, vs = torch.zeros(NB, bs, nKV, device=DEV), torch.zeros(NB, bs, nKV, device=DEV)
    kc_ref, vc_ref = torch.zeros(NB, bs, nKV, d).to(dt), torch.zeros(NB, bs, nKV, d).to(dt)
    quant = O.quantize_kv_int8 if kv_dtype == torch.int8 else O.quantize_kv_fp8
    cached = [0] * len(prompts)
    for step in range(steps + 1):
        lens = prompts if step == 0 else [1] * len(prompts)
        T = sum(lens)
        qkv = torch.randn(T, (nH + 2 * nKV) * d, generator=g).to(dt)
        pos = torch.tensor([c + j for c, l in zip(cached, lens) for j in range(l)], dtype=torch.int64)
        slots = torch.tensor([int(tables[i, (c + j) // bs]) * bs + (c + j) % bs for i, (c, l) in enumerate(zip(cached, lens))
                              for j in range(l)], dtype=torch.int32)
        qsl = torch.tensor(np.cumsum([0] + lens[:-1]), dtype=torch.int32)
        dq = qkv.to(DEV)
        rope_and_cache(rt, dq, kq, vq, pos.to(DEV), cosin.to(DEV), slots.to(DEV), nH, nKV, d, d, bs, True, k_scale=ks, v_scale=vs)
        out = torch.zeros(T, nH * d, dtype=dt, device=DEV)
        attention(rt, dq, kq, vq, out, qsl.to(DEV), torch.tensor(lens, dtype=torch.int32, device=DEV),
                  torch.tensor(cached, dtype=torch.int32, device=DEV), tables.flatten().to(DEV), nH, nKV, d, bs, len(prompts), mb,
                  k_scale=ks, v_scale=vs)
        O.rope_and_cache_ref(qkv, kc_ref, vc_ref, pos, cosin, slots, nH, nKV, d, d, bs)
        kq_ref, ks_ref = quant(kc_ref)
        vq_ref, vs_ref = quant(vc_ref)
        assert torch.equal(kq.cpu().view(torch.int8), kq_ref.view(torch.int8)) and torch.equal(ks.cpu(), ks_ref)
        assert torch.equal(vq.cpu().view(torch.int8), vq_ref.view(torch.int8)) and torch.equal(vs.cpu(), vs_ref)
        ref = O.attention_ref(qkv, kq_ref, vq_ref, qsl, torch.tensor(lens), torch.tensor(cached), tables.flatten(), nH, nKV, d, bs,
                              len(prompts), mb, ks_ref, vs_ref)
        check(out.float().cpu(), ref, max_abs=MAX_ABS_INT8)
        cached = [c + l for c, l in zip(cached, lens)]


def test_config2_llama3_8b_decode_sampled(rt):
    """Configuration 2 at full size on the GPU; the oracle checks a sample of sequences, and the
    reshape-and-cache step of the 64 new tokens is checked bit-exactly first."""
    from gvirt_amd._C import rope_and_cache
    w = W.gqa_decode(W.LLAMA3_8B, [4096] * 64, W.SEED_BASE + 2, device=DEV)
    s = w["shape"]
    r = W.rope_inputs(s, w, W.SEED_BASE + 2)
    sample = [0, 17, 63]
    tables = w["block_tables"].view(64, -1)
    before = {i: (w["k_cache"][tables[i].long()].cpu(), w["v_cache"][tables[i].long()].cpu()) for i in sample}
    inout_cpu = r["inout"].cpu()
    rope_and_cache(rt, r["inout"], w["k_cache"], w["v_cache"], r["position"], r["cosin"], r["slot_mapping"],
                   s.n_heads, s.n_kv_heads, s.head_dim, s.head_dim, s.block_size, True)
    # oracle on a compact copy: the sampled sequences' blocks re-packed with an identity table
    for i in sample:
        kc, vc = before[i]
        pos = r["position"][i:i + 1].cpu()
        slot = torch.tensor([int(pos) // 128 * 128 + int(pos) % 128], dtype=torch.int32)
        row = inout_cpu[i:i + 1].clone()
        O.rope_and_cache_ref(row, kc, vc, pos, r["cosin"].cpu(), slot, s.n_heads, s.n_kv_heads, s.head_dim, s.head_dim, 128)
        assert torch.equal(w["k_cache"][tables[i].long()].cpu().view(torch.int16), kc.view(torch.int16))
        assert torch.equal(w["v_cache"][tables[i].long()].cpu().view(torch.int16), vc.view(torch.int16))
        assert torch.equal(r["inout"][i:i + 1].cpu().view(torch.int16), row.view(torch.int16))
    w["qkv"] = r["inout"]
    got = run_attention(rt, w)
    wc = W.to_device({k: v for k, v in w.items() if k != "shape"}, "cpu"); wc["shape"] = s
    ref = oracle_attention(wc, seqs=sample)
    check(got, ref, rows=sample)
    # size-independent property on all 64 sequences: each output row is a convex combination of V
    # rows, so it is bounded by the column-wise extremes of the V rows the sequence can see
    out = got.view(64, s.n_kv_heads, 4, s.head_dim)
    for i in range(0, 64, 7):
        v = w["v_cache"][tables[i].long()].reshape(-1, s.n_kv_heads, s.head_dim)[:4096].float().cpu()
        assert bool((out[i] <= v.max(0).values.unsqueeze(1) + 1e-2).all())
        assert bool((out[i] >= v.min(0).values.unsqueeze(1) - 1e-2).all())


PREFILL_WORK = [([0], [30]), ([0], [77]), ([0], [1800]), ([128], [1800]), ([0] * 8, [789, 65, 13, 2545, 24, 190, 1432, 124]),
                ([300, 0, 4000], [5, 130, 1])]


@pytest.mark.parametrize("model", [(1, 1, 64, torch.float16), (1, 1, 128, torch.bfloat16), (14, 2, 64, torch.bfloat16),
                                   (5, 1, 128, torch.bfloat16), (8, 1, 128, torch.bfloat16), (28, 4, 128, torch.bfloat16),
                                   (8, 2, 256, torch.bfloat16), (4, 4, 256, torch.float16)])
@pytest.mark.parametrize("work", PREFILL_WORK)
def test_prefill_model_grid(rt, model, work):
    """Prefill / chunked-prefill workloads of xlite/tests/kernels/attention.py:42-60 (bounded)."""
    nH, nKV, d, dtype = model
    clens, lens = work
    w = generic_case(21, lens, clens, nH, nKV, d, 128, dtype, rms=True)
    check(run_attention(rt, w), oracle_attention(w))


SPLIT_WORK = [([3000], [100]), ([16384], [128]), ([2047, 1500, 0, 4000], [1, 1, 300, 1]), ([8191] * 4 + [0], [1] * 4 + [256]),
              ([5000, 900], [257, 2])]


@pytest.mark.parametrize("model", [(8, 2, 128, 128, torch.bfloat16), (32, 8, 128, 128, torch.bfloat16),
                                   (16, 4, 128, 16, torch.float16), (28, 4, 128, 64, torch.bfloat16),
                                   (8, 2, 128, 48, torch.bfloat16), (6, 2, 128, 12, torch.float16),
                                   (14, 2, 64, 128, torch.bfloat16), (8, 8, 64, 8, torch.float16), (12, 4, 64, 24, torch.bfloat16)])
@pytest.mark.parametrize("work", SPLIT_WORK)
def test_prefill_few_tiles_over_long_context(rt, model, work):
    """Short chunks after a long cached context and decode rows mixed with a prefill: fewer M tiles than
    compute units, so each tile's KV range is split over several workgroups and merged."""
    nH, nKV, d, bs, dtype = model
    clens, lens = work
    w = generic_case(23, lens, clens, nH, nKV, d, bs, dtype, rms=True)
    check(run_attention(rt, w), oracle_attention(w))


def test_prefill_rows_equal_decode_steps(rt):
    """Row r of a prefill chunk must match the same row issued alone as a decode step."""
    w = generic_case(22, [40], [200], 8, 2, 128, 128, torch.bfloat16)
    full = run_attention(rt, w)
    for r in (0, 17, 39):
        one = dict(w); one["qkv"] = w["qkv"][r:r + 1].contiguous(); one["batch"] = 1
        one["lens"] = torch.tensor([1], dtype=torch.int32); one["cached_lens"] = torch.tensor([200 + r], dtype=torch.int32)
        one["query_start_loc"] = torch.tensor([0], dtype=torch.int32); one["output"] = torch.zeros(1, 8 * 128, dtype=torch.bfloat16)
        assert float((run_attention(rt, one)[0] - full[r]).abs().max()) <= 1e-2


def test_config3_qwen25_7b_chunked_prefill_sampled(rt):
    """Configuration 3 shape with two of the eight sequences (full-length ones are left to the
    benchmark): every 2048-token chunk attends to the prior paged KV."""
    lens = [2500, 1024]
    caches = None
    for ci in range(2):
        w = W.gqa_prefill_chunk(W.QWEN25_7B, lens, ci, 2048, W.SEED_BASE + 3, caches=caches)
        if w is None:
            break
        caches = w["caches"]
        got = run_attention(rt, w)
        ref = oracle_attention(w)
        check(got, ref)


@pytest.mark.parametrize("model", [(8, 1, 128, torch.bfloat16), (14, 2, 64, torch.bfloat16), (4, 1, 128, torch.float16)])
def test_decode_at_the_longest_reference_contexts(rt, model):
    """The two-sequence decode workloads of xlite/tests/kernels/attention.py:50-57 at their full lengths
    (60000 and 131071 cached positions), against the oracle."""
    nH, nKV, d, dtype = model
    w = generic_case(17, [1, 1], [131071, 60000], nH, nKV, d, 128, dtype, rms=True)
    check(run_attention(rt, w), oracle_attention(w))


@pytest.mark.parametrize("model", [(8, 1, 128, torch.bfloat16), (14, 2, 64, torch.bfloat16)])
def test_prefill_at_the_longest_reference_length_sampled_rows(rt, model):
    """The 32769-token prefill of xlite/tests/kernels/attention.py:46 at full length. The oracle takes sampled
    rows, each as the decode step it is equivalent to (row r of a prefill from an empty cache sees the r keys
    before it and its own)."""
    nH, nKV, d, dtype = model
    n = 32769
    w = generic_case(18, [n], [0], nH, nKV, d, 128, dtype, rms=True)
    got = run_attention(rt, w)
    # the prefill wrote nothing into the cache, which already holds the chunk's keys at positions 0 .. n-1 (the
    # operator reads keys from the cache only): a decode workload over the same cache sees what row r saw
    for r in (0, 1, 127, 128, 4099, 20000, n - 1):
        one = dict(w)
        one["qkv"] = w["qkv"][r:r + 1].contiguous()
        one["batch"] = 1
        one["lens"] = torch.tensor([1], dtype=torch.int32)
        one["cached_lens"] = torch.tensor([r], dtype=torch.int32)
        one["query_start_loc"] = torch.tensor([0], dtype=torch.int32)
        one["output"] = torch.zeros(1, nH * d, dtype=dtype)
        check(got[r:r + 1], oracle_attention(one))


@pytest.mark.parametrize("model,lens", [((8, 1, 128, 16, torch.bfloat16), [3]), ((64, 2, 128, 16, torch.bfloat16), [1]),
                                        ((14, 2, 64, 8, torch.float16), [2])])
def test_block_tables_too_long_for_the_streaming_prefill_kernel(rt, model, lens):
    """More block-table entries per sequence than the streaming prefill kernel can stage next to its KV stages
    (a 131k-token context at block size 16): the call is served by the kernels without that bound."""
    nH, nKV, d, bs, dtype = model
    w = generic_case(19, lens, [131100], nH, nKV, d, bs, dtype, rms=True)
    assert w["max_num_block"] > 8191
    check(run_attention(rt, w), oracle_attention(w))


def _mixed_lens(batch, prefills, seed):
    """`batch` sequences, one query row each except the (index, rows) pairs of `prefills`; contexts 1..3000
    (1..400 for the largest batches, which the CPU oracle would otherwise spend minutes on)."""
    rng = np.random.default_rng(seed)
    lens = [1] * batch
    clens = [int(x) for x in rng.integers(1, 3000 if batch <= 130 else 400, size=batch)]
    for i, n in prefills:
        lens[i] = n
        clens[i] = int(rng.integers(0, 2) * rng.integers(1, 700))
    return clens, lens


@pytest.mark.parametrize("kv_dtype", [None, torch.int8, torch.float8_e4m3fn])
@pytest.mark.parametrize("model", [(32, 8, 128, 128, torch.bfloat16), (14, 2, 64, 16, torch.float16), (28, 4, 128, 64, torch.bfloat16)])
@pytest.mark.parametrize("batch,prefills", [(21, [(0, 30)]), (40, [(39, 77), (5, 2)]), (130, [(64, 200), (3, 0), (129, 9)]),
                                            (700, [(0, 300), (350, 0), (699, 130)])])
def test_mixed_batch_split_between_decode_and_prefill_kernels(rt, kv_dtype, model, batch, prefills):
    """Mostly decode rows with a few prefills (and sequences without rows) among them: the sequences with one
    row go to the streaming decode kernel, the others to the prefill kernel, in one `attention` call; more than
    64 sequences take the split's prefix sums through LDS."""
    nH, nKV, d, bs, dtype = model
    clens, lens = _mixed_lens(batch, prefills, batch)
    assert batch < sum(lens) < 4 * batch
    w = generic_case(81, lens, clens, nH, nKV, d, bs, dtype, rms=True)
    if kv_dtype is not None:
        w = quantised(w, kv_dtype)
    check(run_attention(rt, w), oracle_attention(w), max_abs=MAX_ABS if kv_dtype is None else MAX_ABS_INT8)


def compact_case(seed, lens, clens, nH, nKV, d, bs, dtype):
    """generic_case with only the blocks the sequences need (a batch of thousands of short sequences and a few long
    ones would otherwise reserve the longest sequence's block count for every one); table rows are padded with 0."""
    g = torch.Generator().manual_seed(seed)
    batch, T = len(lens), sum(lens)
    need = [(l + c + bs - 1) // bs for l, c in zip(lens, clens)]
    maxblk, NB = max(need), sum(need) + 1
    rms = lambda x: x / x.pow(2).mean(-1, keepdim=True).add(1e-6).sqrt()
    qkv = rms(torch.randn(T, nH + 2 * nKV, d, generator=g))
    kc = rms(torch.randn(NB, bs, nKV, d, generator=g)).to(dtype)
    vc = rms(torch.randn(NB, bs, nKV, d, generator=g)).to(dtype)
    perm = torch.randperm(NB, generator=g).int()
    tables = torch.zeros(batch, maxblk, dtype=torch.int32)
    off = 0
    for i, n in enumerate(need):
        tables[i, :n] = perm[off:off + n]
        off += n
    shape = W.GqaShape("t", nH, nKV, d, bs, dtype)
    return dict(shape=shape, batch=batch, qkv=qkv.reshape(T, -1).to(dtype), k_cache=kc, v_cache=vc,
                output=torch.zeros(T, nH * d, dtype=dtype), query_start_loc=torch.tensor(np.cumsum([0] + lens[:-1]), dtype=torch.int32),
                lens=torch.tensor(lens, dtype=torch.int32), cached_lens=torch.tensor(clens, dtype=torch.int32),
                block_tables=tables.flatten(), max_num_block=maxblk)


@pytest.mark.parametrize("model,batch", [((32, 8, 128, 128, torch.bfloat16), 4100), ((8, 2, 64, 16, torch.float16), 9000)])
def test_decode_batches_beyond_one_launch_of_the_split(rt, model, batch):
    """More rows than one launch of the decode kernel splits (4096): the batch runs as several launches over
    slices of its rows, each followed by its merge. Short contexts, and a few long ones cut across workgroups."""
    nH, nKV, d, bs, dtype = model
    rng = np.random.default_rng(batch)
    clens = [int(x) for x in rng.integers(1, 60, size=batch)]
    for i in (7, 4095, 4096, batch - 1):
        clens[i] = int(rng.integers(3000, 9000))
    lens = [1] * batch
    lens[4097], lens[4098] = 2, 0          # and the row / sequence numbering parts ways inside the second slice
    w = compact_case(91, lens, clens, nH, nKV, d, bs, dtype)
    assert w["k_cache"].numel() * 2 < 2 << 30
    check(run_attention(rt, w), oracle_attention(w))


@pytest.mark.parametrize("bs", [16, 128, 48])
def test_head_dim_256_split_decode_and_chunked_prefill(rt, bs):
    """head_dim 256 (xlite/tests/models/qwen3_5.py:67, served by the reference's generic kernel,
    xlite/csrc/kernels/attention.h:39-74): long decode contexts whose KV range is split across workgroups, a chunked
    prefill behind a long cached context, sequences without rows, other block sizes."""
    w = generic_case(81, [1] * 5, [9000, 0, 255, 256, 4097], 8, 2, 256, bs, torch.bfloat16, rms=True)
    check(run_attention(rt, w), oracle_attention(w))
    w = generic_case(82, [200, 0, 1, 33], [5000, 10, 700, 0], 8, 2, 256, bs, torch.bfloat16, rms=True)
    check(run_attention(rt, w), oracle_attention(w))


@pytest.mark.parametrize("heads", [(4, 1), (16, 1), (6, 2), (16, 4), (32, 8), (36, 12), (5, 5)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_head_dim_256_decode_batches_of_every_kv_head_count(rt, heads, dtype):
    """head_dim-256 decode batches stream the cache with a head as two 256-byte units: one, two, four kv heads per
    pass, several passes (8 and 12 kv heads), groups that fill and do not fill the 16 columns; 5 kv heads is a count
    the streaming kernel does not take and runs through the generic one. Contexts from one position to several
    chunks, with and without a remainder of a step; narrow block tables (no split) and wide ones."""
    nH, nKV = heads
    ctx = [1, 15, 16, 17, 31, 33, 64, 100, 127, 128, 129, 255, 300]
    w = generic_case(84, [1] * len(ctx), [c - 1 for c in ctx], nH, nKV, 256, 16, dtype, rms=True)
    check(run_attention(rt, w), oracle_attention(w))
    ctx = [6000, 1, 2049, 700, 0, 4096]
    w = generic_case(85, [1 if c else 0 for c in ctx], [max(c - 1, 0) for c in ctx], nH, nKV, 256, 64, dtype, rms=True)
    check(run_attention(rt, w), oracle_attention(w))


def test_head_dim_256_quantised_cache_is_refused(rt):
    w = generic_case(83, [1], [100], 8, 2, 256, 128, torch.bfloat16)
    kq, ks = O.quantize_kv_int8(w["k_cache"].float())
    vq, vs = O.quantize_kv_int8(w["v_cache"].float())
    w.update(k_cache=kq, v_cache=vq, k_scale=ks, v_scale=vs)
    with pytest.raises(RuntimeError, match="head_dim must be 64 or 128"):
        run_attention(rt, w)


@pytest.mark.parametrize("model", [(14, 2, 64, torch.bfloat16), (32, 8, 128, torch.bfloat16), (28, 4, 128, torch.float16),
                                   (32, 8, 128, "int8")])
def test_short_block_tables_run_whole_rows_and_agree_with_the_split_path(rt, model):
    """A decode batch whose block tables are narrow (at most 16 steps per wave) is served without a split and without
    a merge launch; the same batch behind wider tables (same blocks, padding columns) takes the split path. Both
    against the oracle, and against each other."""
    nH, nKV, d, dtype = model
    int8 = dtype == "int8"
    ctx = [1, 15, 16, 17, 100, 128, 129, 200, 255, 256]
    if nKV < 8:
        ctx += [300, 511, 512]
    w = generic_case(81, [1] * len(ctx), [c - 1 for c in ctx], nH, nKV, d, 16, torch.bfloat16 if int8 else dtype, rms=int8)
    if int8:
        w = quantised(w, torch.int8)
    ref = oracle_attention(w)
    narrow = run_attention(rt, w)
    check(narrow, ref, 5e-2 if int8 else MAX_ABS, 5e-3 if int8 else MEAN_ABS)
    wide = dict(w)
    mb, pad = w["max_num_block"], 300   # 300 more columns: far beyond the whole-row bound
    t = w["block_tables"].view(w["batch"], mb)
    wide["block_tables"] = torch.cat([t, torch.zeros(w["batch"], pad, dtype=torch.int32)], dim=1).flatten().contiguous()
    wide["max_num_block"] = mb + pad
    split = run_attention(rt, wide)
    check(split, ref, 5e-2 if int8 else MAX_ABS, 5e-3 if int8 else MEAN_ABS)
    assert float((split - narrow).abs().max()) <= 1e-2


def test_whole_row_mode_with_more_rows_than_workgroups(rt):
    """600 decode rows behind narrow block tables: the whole-row kernel's workgroups take several rows each."""
    rng = np.random.default_rng(11)
    ctx = [int(x) for x in rng.integers(1, 257, size=600)]
    w = generic_case(82, [1] * len(ctx), [c - 1 for c in ctx], 32, 8, 128, 16, torch.bfloat16)
    assert w["max_num_block"] * 16 <= 256
    got = run_attention(rt, w)
    rows = list(range(0, 600, 7)) + [599]
    check(got, oracle_attention(w, seqs=rows), rows=rows)
    assert bool(torch.isfinite(got).all())
