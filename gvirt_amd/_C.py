"""Python operator API of the MI355X attention path, with the names, argument order, defaults and
error behaviour of the reference's `xlite._C` extension (xlite/xlite/_C.pyi) for the attention
operators: Runtime, rope_and_cache, attention, mla_v2, mla_v3, gather_sparse_kv_cache,
mla_prepare, rope_complex, einsum_mht_htd_mhd, einsum_mht_hdt_mhd, get_tile_size_of_cached_kv.

Tensors are borrowed for the call and results are written in place, as in the reference
(xlite/csrc/_C.cpp:174-194). Differences, all deliberate:
  * contiguity, device and dtype are checked and raise RuntimeError (the reference assumes them);
  * kernels run on torch's current HIP stream; the call blocks until they finish unless
    `Runtime.blocking` is set to False (the reference always synchronises, _C.cpp:1182);
  * `attention` and `rope_and_cache` accept keyword-only `k_scale` / `v_scale` for a quantised KV cache
    (int8 or float8_e4m3fn, one fp32 scale per token and kv head).
PyTorch is used only to own device memory and streams.
"""
from __future__ import annotations

import ctypes
from typing import List, Optional, Sequence

import torch

from . import _lib

_DT = {torch.float16: 0, torch.bfloat16: 1}
# element types of a quantised KV cache (one byte per element, fp32 scale per token and kv head)
_KV_DT = {torch.int8: 1, torch.float8_e4m3fn: 2}


def _ptr(t: Optional[torch.Tensor]):
    return None if t is None else ctypes.c_void_p(t.data_ptr())


def _req(cond: bool, msg: str) -> None:
    if not cond:
        raise RuntimeError(msg)


def _dev(name: str, t: torch.Tensor, dtype=None) -> None:
    # the checks first, the messages only when one fails: formatting a device or dtype costs more than the checks
    if isinstance(t, torch.Tensor) and t.is_cuda and t.is_contiguous() and (dtype is None or t.dtype == dtype):
        return
    _req(isinstance(t, torch.Tensor), "%s: expected a tensor" % name)
    _req(t.is_cuda, "%s: expected a GPU tensor, got %s" % (name, t.device))
    _req(t.is_contiguous(), "%s: tensor must be contiguous" % name)
    raise RuntimeError("%s: dtype %s unsupported! (expected %s)" % (name, t.dtype, dtype))


def _act_dtype(name: str, *tensors: torch.Tensor) -> int:
    dt = tensors[0].dtype
    code = _DT.get(dt)
    if code is None:
        raise RuntimeError("%s: dtype %s unsupported!" % (name, dt))
    for t in tensors:
        if t.dtype != dt:
            raise RuntimeError("%s: mixed dtypes %s / %s unsupported!" % (name, dt, t.dtype))
    return code


# torch's current stream of a device as a raw handle, without building a Stream object
_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


class Runtime:
    """Device + scratch handle passed as first argument of every operator
    (reference: XRuntime, xlite/csrc/runtime.h:60-229; Python stub _C.pyi:14-94).

    `size` is the initial scratch pool in MB (the reference's tensor pool); the pool holds the
    split-KV partial results and grows on demand. The parallel-group arguments are accepted for
    signature compatibility; this build runs on one GPU, so any size other than 1 is refused.
    """

    def __init__(self, devid: int, size: int = 0, rank: int = 0, tp_size: int = 1, dp_size: int = 1,
                 moe_tp_size: int = 1, moe_ep_size: int = 1) -> None:
        if tp_size != 1 or dp_size != 1 or moe_tp_size != 1 or moe_ep_size != 1:
            raise RuntimeError("Runtime: this build runs on a single GPU (all group sizes must be 1)")
        self._lib = _lib.load()
        if not torch.cuda.is_available():
            raise RuntimeError("Runtime: no HIP device available")
        self.devid = int(devid)
        self.device = torch.device("cuda", self.devid)
        self.rank = rank
        self.task_id = 0
        self.notify = None
        self.peer_notify = None
        self.multi_task_parallel = False
        self.blocking = True
        ncu = ctypes.c_int(0)
        lds = ctypes.c_int(0)
        arch = ctypes.create_string_buffer(64)
        _lib.check(self._lib.xlite_hip_device_info(self.devid, ctypes.byref(ncu), ctypes.byref(lds), arch, 64))
        self.num_cu = ncu.value
        self.arch = arch.value.decode()
        # names of the reference's core counts, for callers that read them
        self.aic_num = self.num_cu
        self.aiv_num = self.num_cu
        self._pool: Optional[torch.Tensor] = None
        self._retired: List[torch.Tensor] = []
        self._step_plans: dict = {}   # decode_step: argument combinations already checked
        self.init_tensor_pool(size)

    # -- reference API ---------------------------------------------------------------------
    def update_core_num(self, util: float) -> None:
        self.aic_num = max(1, int(round(self.num_cu * util)))
        self.aiv_num = self.aic_num

    def init_tensor_pool(self, size: int) -> int:
        if size:
            self._grow(int(size) << 20)
        return 0

    def set_current_context(self) -> None:
        torch.cuda.set_device(self.devid)

    def configure_swizzle(self, swizzle: int, use_swizzle_table: bool) -> None:
        return None  # matmul tiling knob of the reference; nothing on this path uses it

    # -- scratch -------------------------------------------------------------------------------
    def _grow(self, nbytes: int) -> None:
        """One scratch pool per Runtime, shared by every call on it: calls that use one Runtime from two
        streams at once race on it (the reference's Runtime is not re-entrant either,
        xlite/csrc/runtime.cpp:42). A pool that was handed out is never freed while the Runtime lives:
        kernels still queued and captured graphs keep its address. A pool that has to grow at least doubles, so
        the retired pools together stay smaller than the live one."""
        nbytes = max(nbytes, 1 << 20)
        if self._pool is None or self._pool.numel() < nbytes:
            if self._pool is not None:
                nbytes = max(nbytes, 2 * self._pool.numel())
                if torch.cuda.is_current_stream_capturing():
                    raise RuntimeError("Runtime: the scratch pool must grow to %d bytes, which cannot happen while a "
                                       "graph is being captured; run the shape once before the capture or give "
                                       "Runtime a larger size" % nbytes)
                self._retired.append(self._pool)
            self._pool = torch.empty(nbytes, dtype=torch.uint8, device=self.device)

    def workspace(self, nbytes: int) -> torch.Tensor:
        self._grow(nbytes)
        return self._pool

    def stream(self) -> ctypes.c_void_p:
        if _raw_stream is not None:
            return ctypes.c_void_p(_raw_stream(self.devid))
        return ctypes.c_void_p(torch.cuda.current_stream(self.device).cuda_stream)

    def finish(self) -> None:
        if self.blocking:
            torch.cuda.current_stream(self.device).synchronize()

    def synchronize(self) -> None:
        torch.cuda.current_stream(self.device).synchronize()


class ModelAttnMeta:
    """Host lists describing one step, as in xlite._C.ModelAttnMeta (xlite/csrc/_C.cpp:1988-1993): the metadata
    builder derives positions, slots and the dense block table from them."""

    def __init__(self):
        self.lens: List[int] = []
        self.cached_lens: List[int] = []
        self.is_prefills: List[bool] = []          # deprecated in the reference; ignored
        self.block_tables: List[List[int]] = []


class AttnMeta:
    """The vLLM-compatible form, as in xlite._C.AttnMeta (xlite/csrc/_C.cpp:1995-2001): host block tables, and
    the positions taken from the caller's tensor instead of being derived (xlite/csrc/_C.cpp:666-677)."""

    def __init__(self):
        self.lens: List[int] = []
        self.cached_lens: List[int] = []
        self.is_prefills: List[bool] = []
        self.block_tables_cpu: List[List[int]] = []
        self.positions: Optional[torch.Tensor] = None


def rope_and_cache(rt: Runtime, inout: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                   position: torch.Tensor, cosin: torch.Tensor, slot_mapping: torch.Tensor, n_heads: int,
                   n_kv_heads: int, head_dim: int, rot_dim: int, block_size: int, is_neox: bool,
                   mrope_mask_h: int = 0, mrope_mask_w: int = 0, *, k_scale: Optional[torch.Tensor] = None,
                   v_scale: Optional[torch.Tensor] = None) -> None:
    """RoPE in place on the fused q|k|v rows and the write of K and V into the paged caches
    (xlite/_C.pyi:1251-1290). Extension (keyword-only): with `k_scale` and `v_scale`
    [num_blocks, block_size, n_kv_heads] fp32 the caches are int8 or float8_e4m3fn and the rows are quantised as
    they are written (scale = absmax / 127, or absmax / 448, per token and kv head)."""
    if not is_neox:
        raise RuntimeError("rope_and_cache: unsupported rope type gptj")
    int8 = k_scale is not None or v_scale is not None
    for n, t in (("inout", inout), ("cosin", cosin)):
        _dev(n, t)
    for n, t in (("k_cache", k_cache), ("v_cache", v_cache)):
        _dev(n, t)
    if int8:
        _req(k_cache.dtype in _KV_DT and v_cache.dtype == k_cache.dtype,
             "rope_and_cache: scales given but the caches are neither int8 nor float8_e4m3fn")
    _dev("position", position, torch.int64)
    _dev("slot_mapping", slot_mapping, torch.int32)
    dt = _act_dtype("rope_and_cache", inout, cosin) if int8 else _act_dtype("rope_and_cache", inout, k_cache, v_cache, cosin)
    T = inout.shape[0]
    _req(inout.numel() == T * (n_heads + 2 * n_kv_heads) * head_dim, "rope_and_cache: inout shape mismatch")
    _req(k_cache.shape == v_cache.shape, "rope_and_cache: cache shapes differ")
    _req(k_cache.numel() % (block_size * n_kv_heads * head_dim) == 0, "rope_and_cache: cache shape mismatch")
    mrope = bool(mrope_mask_h or mrope_mask_w)
    _req(position.numel() == (3 * T if mrope else T), "rope_and_cache: position shape mismatch")
    _req(slot_mapping.numel() >= T, "rope_and_cache: slot_mapping too short")
    _req(cosin.shape[-1] == rot_dim, "rope_and_cache: cosin row must hold rot_dim values")
    if int8:
        _req(k_scale is not None and v_scale is not None, "rope_and_cache: int8 caches need k_scale and v_scale")
        for n, t in (("k_scale", k_scale), ("v_scale", v_scale)):
            _dev(n, t, torch.float32)
            _req(t.numel() * head_dim == k_cache.numel(), "rope_and_cache: %s shape mismatch" % n)
        _lib.check(rt._lib.xlite_hip_rope_and_cache_quant(
            rt.stream(), _ptr(inout), _ptr(k_cache), _ptr(v_cache), _ptr(k_scale), _ptr(v_scale), _ptr(position),
            _ptr(cosin), _ptr(slot_mapping), T, n_heads, n_kv_heads, head_dim, rot_dim, block_size, 1, mrope_mask_h,
            mrope_mask_w, dt, _KV_DT[k_cache.dtype]))
    else:
        _lib.check(rt._lib.xlite_hip_rope_and_cache(
            rt.stream(), _ptr(inout), _ptr(k_cache), _ptr(v_cache), _ptr(position), _ptr(cosin), _ptr(slot_mapping),
            T, n_heads, n_kv_heads, head_dim, rot_dim, block_size, 1, mrope_mask_h, mrope_mask_w, dt))
    rt.finish()


def attention(rt: Runtime, qkv: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
              output: torch.Tensor, query_start_loc: torch.Tensor, lens: torch.Tensor,
              cached_lens: torch.Tensor, block_tables: torch.Tensor, n_heads: int, n_kv_heads: int,
              head_dim: int, block_size: int, batch: int, max_num_block: int,
              enable_flash_attention: bool = False, tile_size_of_cached_kv: int = 8192, *,
              k_scale: Optional[torch.Tensor] = None, v_scale: Optional[torch.Tensor] = None,
              workspace_limit: Optional[int] = None) -> None:
    """Paged GQA attention, decode and causal (chunked) prefill. `enable_flash_attention` and
    `tile_size_of_cached_kv` select between two kernels in the reference; here they are hints
    only (the KV split is chosen from the batch shape). `workspace_limit` (keyword-only, bytes): hand the
    library at most that much scratch, as a caller with little memory would; paths that need more are not
    taken (a multi-row batch over a quantised cache is then read by the prefill kernel itself instead of
    through a 16-bit copy of its blocks) or fail with the library's error."""
    for n, t in (("qkv", qkv), ("k_cache", k_cache), ("v_cache", v_cache), ("output", output)):
        _dev(n, t)
    for n, t in (("query_start_loc", query_start_loc), ("lens", lens), ("cached_lens", cached_lens),
                 ("block_tables", block_tables)):
        _dev(n, t, torch.int32)
    dt = _act_dtype("attention", qkv, output)
    int8 = k_scale is not None or v_scale is not None
    if int8:
        _req(k_scale is not None and v_scale is not None, "attention: k_scale and v_scale go together")
        _dev("k_scale", k_scale, torch.float32)
        _dev("v_scale", v_scale, torch.float32)
        _req(k_cache.dtype in _KV_DT and v_cache.dtype == k_cache.dtype,
             "attention: scales given but the caches are neither int8 nor float8_e4m3fn")
        _req(k_scale.numel() * head_dim == k_cache.numel() and v_scale.numel() * head_dim == v_cache.numel(),
             "attention: one scale per (block, slot, kv head) expected")
    else:
        if k_cache.dtype != qkv.dtype or v_cache.dtype != qkv.dtype:
            raise RuntimeError("attention: qkv %s kCache %s vCache %s unsupported!" % (qkv.dtype, k_cache.dtype, v_cache.dtype))
    T = qkv.shape[0]
    _req(n_kv_heads > 0 and n_heads % n_kv_heads == 0, "attention: n_heads must be a multiple of n_kv_heads")
    _req(qkv.numel() == T * (n_heads + 2 * n_kv_heads) * head_dim, "attention: qkv shape mismatch")
    _req(output.numel() == T * n_heads * head_dim, "attention: output shape mismatch")
    _req(min(query_start_loc.numel(), lens.numel(), cached_lens.numel()) >= batch, "attention: metadata shorter than batch")
    _req(block_tables.numel() >= batch * max_num_block, "attention: block_tables shorter than batch * max_num_block")
    kv = _KV_DT[k_cache.dtype] if int8 else 0
    need = rt._lib.xlite_hip_attention_workspace_bytes_kv(T, n_heads, n_kv_heads, head_dim, block_size, batch,
                                                          max_num_block, kv)
    ws = rt.workspace(need)
    ws_bytes = ws.numel() if workspace_limit is None else min(ws.numel(), int(workspace_limit))
    _lib.check(rt._lib.xlite_hip_attention(
        rt.stream(), _ptr(qkv), _ptr(k_cache), _ptr(v_cache), _ptr(output), _ptr(query_start_loc), _ptr(lens),
        _ptr(cached_lens), _ptr(block_tables), T, n_heads, n_kv_heads, head_dim, block_size, batch, max_num_block,
        dt, kv, _ptr(k_scale), _ptr(v_scale), _ptr(ws), ws_bytes))
    rt.finish()


def decode_step(rt: Runtime, qkv: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, output: torch.Tensor,
                position: torch.Tensor, cosin: torch.Tensor, slot_mapping: torch.Tensor,
                query_start_loc: torch.Tensor, lens: torch.Tensor, cached_lens: torch.Tensor,
                block_tables: torch.Tensor, n_heads: int, n_kv_heads: int, head_dim: int, rot_dim: int,
                block_size: int, batch: int, max_num_block: int, is_neox: bool = True, mrope_mask_h: int = 0,
                mrope_mask_w: int = 0) -> None:
    """`rope_and_cache` followed by `attention` over the same rows and caches, as a layer of the reference's model
    loop runs them (xlite/csrc/model.cpp:544-571), through one call into the library. The argument checks of the
    two run once per combination of shapes, dtypes and devices: a serving loop repeats the same combination step
    after step, and for a small batch the checks cost more than the kernels. 16-bit caches."""
    tensors = (qkv, k_cache, v_cache, output, position, cosin, slot_mapping, query_start_loc, lens, cached_lens,
               block_tables)
    key = (tuple((t.shape, t.dtype, t.device, t.is_contiguous()) for t in tensors), n_heads, n_kv_heads, head_dim,
           rot_dim, block_size, batch, max_num_block, is_neox, mrope_mask_h, mrope_mask_w)
    plan = rt._step_plans.get(key)
    if plan is None:
        if not is_neox:
            raise RuntimeError("rope_and_cache: unsupported rope type gptj")
        for n, t in (("qkv", qkv), ("k_cache", k_cache), ("v_cache", v_cache), ("output", output), ("cosin", cosin)):
            _dev(n, t)
        _dev("position", position, torch.int64)
        for n, t in (("slot_mapping", slot_mapping), ("query_start_loc", query_start_loc), ("lens", lens),
                     ("cached_lens", cached_lens), ("block_tables", block_tables)):
            _dev(n, t, torch.int32)
        dt = _act_dtype("decode_step", qkv, k_cache, v_cache, cosin, output)
        T = qkv.shape[0]
        _req(n_kv_heads > 0 and n_heads % n_kv_heads == 0, "decode_step: n_heads must be a multiple of n_kv_heads")
        _req(qkv.numel() == T * (n_heads + 2 * n_kv_heads) * head_dim, "decode_step: qkv shape mismatch")
        _req(output.numel() == T * n_heads * head_dim, "decode_step: output shape mismatch")
        _req(k_cache.shape == v_cache.shape, "decode_step: cache shapes differ")
        _req(k_cache.numel() % (block_size * n_kv_heads * head_dim) == 0, "decode_step: cache shape mismatch")
        mrope = bool(mrope_mask_h or mrope_mask_w)
        _req(position.numel() == (3 * T if mrope else T), "decode_step: position shape mismatch")
        _req(slot_mapping.numel() >= T, "decode_step: slot_mapping too short")
        _req(cosin.shape[-1] == rot_dim, "decode_step: cosin row must hold rot_dim values")
        _req(min(query_start_loc.numel(), lens.numel(), cached_lens.numel()) >= batch,
             "decode_step: metadata shorter than batch")
        _req(block_tables.numel() >= batch * max_num_block, "decode_step: block_tables shorter than batch * max_num_block")
        need = rt._lib.xlite_hip_attention_workspace_bytes(T, n_heads, n_kv_heads, head_dim, block_size, batch,
                                                           max_num_block)
        plan = rt._step_plans[key] = (T, dt, need)
    T, dt, need = plan
    ws = rt.workspace(need)
    _lib.check(rt._lib.xlite_hip_decode_step(
        rt.stream(), qkv.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), output.data_ptr(), position.data_ptr(),
        cosin.data_ptr(), slot_mapping.data_ptr(), query_start_loc.data_ptr(), lens.data_ptr(), cached_lens.data_ptr(),
        block_tables.data_ptr(), T, n_heads, n_kv_heads, head_dim, rot_dim, block_size, batch, max_num_block, 1,
        mrope_mask_h, mrope_mask_w, dt, ws.data_ptr(), ws.numel()))
    rt.finish()


def _einsum(rt: Runtime, name: str, mht, w, mhd, m, h, t, d, weight_nz, hdt: bool, t_stride: Optional[int] = None):
    if weight_nz:
        raise RuntimeError(name + ": the NZ (Ascend fractal) weight layout has no meaning on this device")
    for n, x in (("mht", mht), ("w", w), ("mhd", mhd)):
        _dev(n, x)
    dt = _act_dtype(name, mht, w, mhd)
    ts = t if t_stride is None else t_stride
    _req(mht.numel() >= m * h * ts, name + ": mht too small")
    _req(w.numel() == h * t * d, name + ": weight shape mismatch")
    _req(mhd.numel() == m * h * d, name + ": mhd shape mismatch")
    _lib.check(rt._lib.xlite_hip_einsum_mht_mhd(rt.stream(), _ptr(mht), _ptr(w), _ptr(mhd), m, h, t, d, ts,
                                                1 if hdt else 0, dt))


def einsum_mht_htd_mhd(rt: Runtime, mht: torch.Tensor, htd: torch.Tensor, mhd: torch.Tensor, m: int, h: int,
                       t: int, d: int, weight_nz: bool = False) -> None:
    _einsum(rt, "einsum_mht_htd_mhd", mht, htd, mhd, m, h, t, d, weight_nz, False)
    rt.finish()


def einsum_mht_hdt_mhd(rt: Runtime, mht: torch.Tensor, hdt: torch.Tensor, mhd: torch.Tensor, m: int, h: int,
                       t: int, d: int, weight_nz: bool = False) -> None:
    _einsum(rt, "einsum_mht_hdt_mhd", mht, hdt, mhd, m, h, t, d, weight_nz, True)
    rt.finish()


def mla_attention(rt: Runtime, q_absorb: torch.Tensor, qr: torch.Tensor, k_cache: torch.Tensor,
                  pe_cache: torch.Tensor, o_absorb: torch.Tensor, query_start_loc: torch.Tensor,
                  lens: torch.Tensor, cached_lens: torch.Tensor, block_tables: torch.Tensor, n_heads: int,
                  rope_head_dim: int, kv_lora_rank: int, block_size: int, batch: int, max_num_blocks: int,
                  scale: float, topk_indices: Optional[torch.Tensor] = None, top_k: int = 0) -> None:
    """The attention stage of mla_v2 alone (q_absorb, qr -> o_absorb); the reference runs it as
    XliteOpMLAV2 / XliteOpFlashMLAV2 inside the mla_v2 binding (xlite/csrc/_C.cpp:1264-1294)."""
    for n, t in (("q_absorb", q_absorb), ("qr", qr), ("k_cache", k_cache), ("pe_cache", pe_cache),
                 ("o_absorb", o_absorb)):
        _dev(n, t)
    for n, t in (("query_start_loc", query_start_loc), ("lens", lens), ("cached_lens", cached_lens),
                 ("block_tables", block_tables)):
        _dev(n, t, torch.int32)
    if q_absorb.dtype != torch.bfloat16:
        raise RuntimeError("mla: qAbsorb dtype %s unsupported!" % q_absorb.dtype)
    dt = _act_dtype("mla", q_absorb, qr, k_cache, pe_cache, o_absorb)
    if top_k > 2048:
        raise RuntimeError("mla: topK should be less than or equal to 2048")
    T = q_absorb.shape[0]
    _req(q_absorb.numel() == T * n_heads * kv_lora_rank and o_absorb.numel() == q_absorb.numel(),
         "mla: q_absorb / o_absorb shape mismatch")
    _req(qr.numel() == T * n_heads * rope_head_dim, "mla: qr shape mismatch")
    _req(block_tables.numel() >= batch * max_num_blocks, "mla: block_tables too short")
    if top_k:
        _dev("topk_indices", topk_indices, torch.int32)
        _req(topk_indices.numel() >= T * top_k, "mla: topk_indices too short")
    need = rt._lib.xlite_hip_mla_workspace_bytes(T, n_heads, kv_lora_rank, rope_head_dim, block_size, batch, max_num_blocks, top_k)
    ws = rt.workspace(need)
    _lib.check(rt._lib.xlite_hip_mla_attention(
        rt.stream(), _ptr(q_absorb), _ptr(qr), _ptr(k_cache), _ptr(pe_cache), _ptr(o_absorb),
        _ptr(query_start_loc), _ptr(lens), _ptr(cached_lens), _ptr(block_tables), T, n_heads, rope_head_dim,
        kv_lora_rank, block_size, batch, max_num_blocks, float(scale), _ptr(topk_indices) if top_k else None,
        top_k, dt, _ptr(ws), ws.numel()))


def mla_v2(rt: Runtime, q_with_qr: torch.Tensor, qr: torch.Tensor, k_cache: torch.Tensor,
           pe_cache: torch.Tensor, wuk_t: torch.Tensor, wuv: torch.Tensor, output: torch.Tensor,
           query_start_loc: torch.Tensor, lens: torch.Tensor, cached_lens: torch.Tensor,
           block_tables: torch.Tensor, n_heads: int, rope_head_dim: int, nope_head_dim: int, v_head_dim: int,
           kv_lora_rank: int, block_size: int, batch: int, max_num_blocks: int, scale: float,
           topk_indices: torch.Tensor, top_k: int = 0, nz: bool = False, enable_flash_attention: bool = False,
           tile_size_of_cached_kv: int = 8192) -> None:
    """W_UK absorb einsum + absorbed MLA attention + W_UV einsum (xlite/csrc/_C.cpp:1234-1301)."""
    if nz:
        raise RuntimeError("mla_v2: the NZ (Ascend fractal) weight layout has no meaning on this device")
    T = q_with_qr.shape[0]
    _dev("q_with_qr", q_with_qr)
    q_absorb = torch.empty(T, n_heads * kv_lora_rank, dtype=q_with_qr.dtype, device=q_with_qr.device)
    o_absorb = torch.empty_like(q_absorb)
    _einsum(rt, "mla_v2", q_with_qr, wuk_t, q_absorb, T, n_heads, nope_head_dim, kv_lora_rank, False, False,
            t_stride=nope_head_dim + rope_head_dim)
    mla_attention(rt, q_absorb, qr, k_cache, pe_cache, o_absorb, query_start_loc, lens, cached_lens, block_tables,
                  n_heads, rope_head_dim, kv_lora_rank, block_size, batch, max_num_blocks, scale, topk_indices,
                  top_k)
    _einsum(rt, "mla_v2", o_absorb, wuv, output, T, n_heads, kv_lora_rank, v_head_dim, False, False)
    rt.finish()


def gather_sparse_kv_cache(rt: Runtime, k_cache: torch.Tensor, pe_cache: torch.Tensor, block_tables: torch.Tensor,
                           topk_indices: torch.Tensor, query_lens: torch.Tensor, cached_lens: torch.Tensor,
                           k_dense_cache: torch.Tensor, pe_dense_cache: torch.Tensor, batch: int, index_topk: int,
                           block_size: int, max_num_blocks: int, kv_lora_rank: int, rope_head_dim: int,
                           kv_heads: int = 1) -> None:
    if kv_heads != 1:
        raise RuntimeError("gather_sparse_kv_cache: kvHeads should be less than or equal to 1")
    for n, t in (("k_cache", k_cache), ("pe_cache", pe_cache), ("k_dense_cache", k_dense_cache),
                 ("pe_dense_cache", pe_dense_cache)):
        _dev(n, t)
    for n, t in (("block_tables", block_tables), ("topk_indices", topk_indices), ("query_lens", query_lens),
                 ("cached_lens", cached_lens)):
        _dev(n, t, torch.int32)
    dt = _act_dtype("gather_sparse_kv_cache", k_cache, pe_cache, k_dense_cache, pe_dense_cache)
    _req(k_dense_cache.numel() == batch * index_topk * kv_lora_rank, "gather_sparse_kv_cache: k_dense shape mismatch")
    _req(pe_dense_cache.numel() == batch * index_topk * rope_head_dim, "gather_sparse_kv_cache: pe_dense shape mismatch")
    _req(topk_indices.numel() >= batch * index_topk, "gather_sparse_kv_cache: topk_indices too short")
    _req(block_tables.numel() >= batch * max_num_blocks, "gather_sparse_kv_cache: block_tables too short")
    _lib.check(rt._lib.xlite_hip_gather_sparse_kv_cache(
        rt.stream(), _ptr(k_cache), _ptr(pe_cache), _ptr(block_tables), _ptr(topk_indices), _ptr(query_lens),
        _ptr(cached_lens), _ptr(k_dense_cache), _ptr(pe_dense_cache), batch, index_topk, block_size,
        max_num_blocks, kv_lora_rank, rope_head_dim, kv_heads, dt))
    rt.finish()


def mla_v3(rt: Runtime, q_absorb: torch.Tensor, qr: torch.Tensor, k_dense_cache: torch.Tensor,
           pe_dense_cache: torch.Tensor, o_absorb: torch.Tensor, query_start_loc: torch.Tensor, lens: torch.Tensor,
           cached_lens: torch.Tensor, n_heads: int, rope_head_dim: int, kv_lora_rank: int, batch: int,
           index_topk: int, scale: float) -> None:
    for n, t in (("q_absorb", q_absorb), ("qr", qr), ("k_dense_cache", k_dense_cache),
                 ("pe_dense_cache", pe_dense_cache), ("o_absorb", o_absorb)):
        _dev(n, t)
    for n, t in (("query_start_loc", query_start_loc), ("lens", lens), ("cached_lens", cached_lens)):
        _dev(n, t, torch.int32)
    if q_absorb.dtype != torch.bfloat16:
        raise RuntimeError("mla_v3: qAbsorb dtype %s unsupported!" % q_absorb.dtype)
    dt = _act_dtype("mla_v3", q_absorb, qr, k_dense_cache, pe_dense_cache, o_absorb)
    T = q_absorb.shape[0]
    _req(k_dense_cache.numel() == batch * index_topk * kv_lora_rank, "mla_v3: k_dense shape mismatch")
    _req(pe_dense_cache.numel() == batch * index_topk * rope_head_dim, "mla_v3: pe_dense shape mismatch")
    need = rt._lib.xlite_hip_mla_workspace_bytes(T, n_heads, kv_lora_rank, rope_head_dim, 1, batch, index_topk, 0)
    ws = rt.workspace(need)
    _lib.check(rt._lib.xlite_hip_mla_v3(
        rt.stream(), _ptr(q_absorb), _ptr(qr), _ptr(k_dense_cache), _ptr(pe_dense_cache), _ptr(o_absorb),
        _ptr(query_start_loc), _ptr(lens), _ptr(cached_lens), T, n_heads, rope_head_dim, kv_lora_rank, batch,
        index_topk, float(scale), dt, _ptr(ws), ws.numel()))
    rt.finish()


def qk_rms_norm(rt: Runtime, qkv: torch.Tensor, q_norm: torch.Tensor, q_norm_bias: Optional[torch.Tensor],
                k_norm: torch.Tensor, k_norm_bias: Optional[torch.Tensor], out: torch.Tensor, norm_eps: float,
                q_norm_dim: int, q_cnt_per_token: int, k_norm_dim: int, k_cnt_per_token: int,
                k_start_offset: int) -> None:
    """RMSNorm of the Q and K segments of the fused qkv rows, argument order of the reference's C++ operator
    (xlite/csrc/op.cpp:1177-1182; it has no Python binding there). `out` may be `qkv`."""
    for n, t in (("qkv", qkv), ("q_norm", q_norm), ("k_norm", k_norm), ("out", out)):
        _dev(n, t)
    tensors = [qkv, q_norm, k_norm, out]
    for n, t in (("q_norm_bias", q_norm_bias), ("k_norm_bias", k_norm_bias)):
        if t is not None:
            _dev(n, t)
            tensors.append(t)
    dt = _act_dtype("qk_rms_norm", *tensors)
    _req(qkv.dim() == 2 and out.shape == qkv.shape, "qk_rms_norm: qkv and out must be [tokens, row] of one shape")
    _req(q_norm.numel() == q_norm_dim and k_norm.numel() == k_norm_dim, "qk_rms_norm: weight shape mismatch")
    _req(q_norm_bias is None or q_norm_bias.numel() == q_norm_dim, "qk_rms_norm: q bias shape mismatch")
    _req(k_norm_bias is None or k_norm_bias.numel() == k_norm_dim, "qk_rms_norm: k bias shape mismatch")
    _lib.check(rt._lib.xlite_hip_qk_rms_norm(
        rt.stream(), _ptr(qkv), _ptr(out), _ptr(q_norm), _ptr(q_norm_bias), _ptr(k_norm), _ptr(k_norm_bias),
        qkv.shape[0], qkv.shape[1], q_norm_dim, q_cnt_per_token, k_norm_dim, k_cnt_per_token, k_start_offset,
        float(norm_eps), dt))
    rt.finish()


def _indexer_check(name: str, q, k_cache, weight, query_start_loc, lens, cached_lens, block_tables, n_heads: int,
                   head_dim: int, batch: int, max_num_block: int) -> int:
    for n, t in (("q", q), ("k_cache", k_cache), ("weight", weight)):
        _dev(n, t)
    for n, t in (("query_start_loc", query_start_loc), ("lens", lens), ("cached_lens", cached_lens),
                 ("block_tables", block_tables)):
        _dev(n, t, torch.int32)
    dt = _act_dtype(name, q, k_cache, weight)
    T = q.shape[0]
    _req(q.numel() == T * n_heads * head_dim, "%s: q shape mismatch" % name)
    _req(weight.numel() == T * (head_dim + n_heads), "%s: weight shape mismatch" % name)
    _req(block_tables.numel() >= batch * max_num_block, "%s: block_tables too short" % name)
    return dt


def indexer_scores(rt: Runtime, q: torch.Tensor, k_cache: torch.Tensor, weight: torch.Tensor, scores: torch.Tensor,
                   query_start_loc: torch.Tensor, lens: torch.Tensor, cached_lens: torch.Tensor,
                   block_tables: torch.Tensor, n_heads: int, head_dim: int, block_size: int, batch: int,
                   max_num_block: int) -> None:
    """DSA indexer scores over the cached keys (xlite/_C.pyi:1946-1983): row t of `scores`
    [total_query_len, max_num_block * block_size] gets sum_h weight[t, head_dim + h] * (q[t, h] . k[j]) for
    every position j of its sequence."""
    dt = _indexer_check("indexer_scores", q, k_cache, weight, query_start_loc, lens, cached_lens, block_tables,
                        n_heads, head_dim, batch, max_num_block)
    _dev("scores", scores)
    if scores.dtype != q.dtype:
        raise RuntimeError("indexer_scores: scores dtype %s unsupported!" % scores.dtype)
    T = q.shape[0]
    _req(scores.numel() == T * max_num_block * block_size, "indexer_scores: scores shape mismatch")
    _lib.check(rt._lib.xlite_hip_indexer_scores(
        rt.stream(), _ptr(q), _ptr(k_cache), _ptr(weight), _ptr(scores), _ptr(query_start_loc), _ptr(lens),
        _ptr(cached_lens), _ptr(block_tables), T, n_heads, head_dim, block_size, batch, max_num_block, dt))
    rt.finish()


def indexer_topk(rt: Runtime, q: torch.Tensor, k_cache: torch.Tensor, weight: torch.Tensor, indices: torch.Tensor,
                 topk_indices: torch.Tensor, query_start_loc: torch.Tensor, lens: torch.Tensor,
                 cached_lens: torch.Tensor, block_tables: torch.Tensor, n_heads: int, head_dim: int, block_size: int,
                 batch: int, max_num_block: int, top_k: int) -> None:
    """Fused indexer scores + top-k selection (xlite/_C.pyi:1985-2040): the first
    min(top_k, cached + query length) entries of every row of `topk_indices` [total_query_len, top_k] are
    written; the score rows live in the runtime's scratch pool."""
    dt = _indexer_check("indexer_topk", q, k_cache, weight, query_start_loc, lens, cached_lens, block_tables,
                        n_heads, head_dim, batch, max_num_block)
    _dev("indices", indices, torch.int32)
    _dev("topk_indices", topk_indices, torch.int32)
    if top_k > 2048:
        raise RuntimeError("indexer_topk: topK should be less than or equal to 2048")
    T = q.shape[0]
    _req(indices.numel() >= max_num_block * block_size, "indexer_topk: indices too short")
    _req(topk_indices.numel() == T * top_k, "indexer_topk: topk_indices shape mismatch")
    need = rt._lib.xlite_hip_indexer_topk_workspace_bytes(T, block_size, max_num_block)
    ws = rt.workspace(need)
    _lib.check(rt._lib.xlite_hip_indexer_topk(
        rt.stream(), _ptr(q), _ptr(k_cache), _ptr(weight), _ptr(indices), _ptr(topk_indices), _ptr(query_start_loc),
        _ptr(lens), _ptr(cached_lens), _ptr(block_tables), T, n_heads, head_dim, block_size, batch, max_num_block,
        top_k, dt, _ptr(ws), ws.numel() * ws.element_size()))
    rt.finish()


def _freqs_f32(freqs: torch.Tensor, rope_dim: int) -> torch.Tensor:
    """complex64 [max_pos, rope_dim/2] is read as interleaved fp32 (cos, sin), as the reference does."""
    _req(freqs.is_cuda and freqs.is_contiguous(), "freqs: contiguous GPU tensor expected")
    f = torch.view_as_real(freqs) if freqs.is_complex() else freqs
    _req(f.dtype == torch.float32, "freqs: complex64 / float32 expected")
    _req(f.numel() % rope_dim == 0, "freqs: row must hold rope_dim floats")
    return f


def rope_complex(rt: Runtime, n_local_heads: int, step_dim: int, rope_dim: int, input_with_r: torch.Tensor,
                 freqs: torch.Tensor, position: torch.Tensor, output: torch.Tensor) -> None:
    _dev("input_with_r", input_with_r)
    _dev("output", output)
    _dev("position", position, torch.int64)
    dt = _act_dtype("rope_complex", input_with_r, output)
    f = _freqs_f32(freqs, rope_dim)
    T = input_with_r.shape[0]
    _req(input_with_r.numel() == T * n_local_heads * step_dim, "rope_complex: input shape mismatch")
    _req(output.numel() == T * n_local_heads * rope_dim, "rope_complex: output shape mismatch")
    _req(position.numel() >= T, "rope_complex: position too short")
    _lib.check(rt._lib.xlite_hip_rope_complex(rt.stream(), T, n_local_heads, step_dim, rope_dim,
                                              _ptr(input_with_r), _ptr(f), _ptr(position), _ptr(output), dt))
    rt.finish()


def rope_complex_and_cache(rt: Runtime, n_local_heads: int, step_dim: int, rope_dim: int, offset: int, vdim: int,
                           input_with_r: torch.Tensor, freqs: torch.Tensor, position: torch.Tensor,
                           output: Optional[torch.Tensor] = None, out_step_dim: int = 0, out_offset: int = 0,
                           block_size: int = 0, cache: Optional[torch.Tensor] = None,
                           slot_mapping: Optional[torch.Tensor] = None) -> None:
    """The general interleaved-pair rope (no Python binding in the reference; XliteOpRopeComplex and
    XliteOpRopeComplexAndCache, xlite/csrc/op.cpp:1106-1150): the rope_dim columns from `offset` of every head,
    to `output` (which may be the input) or, with a cache, the vdim columns from `offset` to cache[slot]."""
    _dev("input_with_r", input_with_r)
    _dev("position", position, torch.int64)
    dt = _act_dtype("rope_complex_and_cache", input_with_r)
    f = _freqs_f32(freqs, rope_dim)
    T = input_with_r.shape[0]
    _req(input_with_r.numel() == T * n_local_heads * step_dim, "rope_complex_and_cache: input shape mismatch")
    _req(position.numel() >= T, "rope_complex_and_cache: position too short")
    if cache is not None:
        _dev("cache", cache, input_with_r.dtype)
        _dev("slot_mapping", slot_mapping, torch.int32)
        _req(block_size > 0 and cache.numel() % (block_size * vdim) == 0, "rope_complex_and_cache: cache shape mismatch")
        _req(slot_mapping.numel() >= T, "rope_complex_and_cache: slot_mapping too short")
    else:
        _dev("output", output, input_with_r.dtype)
        _req(output.numel() == T * n_local_heads * out_step_dim, "rope_complex_and_cache: output shape mismatch")
    _lib.check(rt._lib.xlite_hip_rope_complex_and_cache(
        rt.stream(), T, n_local_heads, step_dim, rope_dim, offset, vdim, _ptr(input_with_r), _ptr(output), out_step_dim,
        out_offset, _ptr(f), _ptr(position), block_size if cache is not None else 0, _ptr(cache), _ptr(slot_mapping), dt))
    rt.finish()


def layernorm(rt: Runtime, in_: torch.Tensor, norm: torch.Tensor, norm_bias: torch.Tensor, out: torch.Tensor,
              norm_eps: float, norm_dim: int) -> None:
    """LayerNorm over the first norm_dim columns of every row (xlite/csrc/_C.cpp:1122-1133)."""
    for n, t in (("in_", in_), ("norm", norm), ("norm_bias", norm_bias), ("out", out)):
        _dev(n, t)
    dt = _act_dtype("layernorm", in_, norm, norm_bias, out)
    _req(in_.dim() == 2 and out.dim() == 2 and in_.shape[0] == out.shape[0], "layernorm: [rows, columns] tensors expected")
    _req(norm.numel() >= norm_dim and norm_bias.numel() >= norm_dim, "layernorm: weight / bias shorter than norm_dim")
    _lib.check(rt._lib.xlite_hip_layernorm(rt.stream(), _ptr(in_), _ptr(norm), _ptr(norm_bias), _ptr(out), in_.shape[0],
                                           in_.shape[1], out.shape[1], norm_dim, float(norm_eps), dt))
    rt.finish()


def muls(rt: Runtime, input: torch.Tensor, scale: float, output: torch.Tensor, calc_offset: int = 0,
         calc_num: int = 0xFFFFFFFF) -> None:
    """output = input * scale (xlite/csrc/_C.cpp:1660-1667); `calc_offset` / `calc_num` restrict it to a column
    range of every row, the form the model runner calls (xlite/csrc/model.cpp:316)."""
    _dev("input", input)
    _dev("output", output)
    dt = _act_dtype("muls", input, output)
    _req(input.shape == output.shape, "muls: shape mismatch")
    rows = input.shape[0] if input.dim() >= 2 else 1
    row_len = input.numel() // max(rows, 1)
    _lib.check(rt._lib.xlite_hip_muls(rt.stream(), _ptr(input), _ptr(output), rows, row_len, calc_offset,
                                      min(calc_num, 0xFFFFFFFF), float(scale), dt))
    rt.finish()


def mla_prepare(rt: Runtime, attn_qkvc: torch.Tensor, q_norm: torch.Tensor, q_norm_bias: torch.Tensor,
                attn_norm_qc: torch.Tensor, kv_norm: torch.Tensor, kv_norm_bias: torch.Tensor,
                attn_norm_kvc: torch.Tensor, freqs: torch.Tensor, position: torch.Tensor, q_lora_rank: int,
                kv_lora_rank: int, rope_head_dim: int, block_size: int, k_cache: torch.Tensor,
                pe_cache: torch.Tensor, slot_mapping: torch.Tensor, norm_eps: float) -> None:
    for n, t in (("attn_qkvc", attn_qkvc), ("q_norm", q_norm), ("q_norm_bias", q_norm_bias),
                 ("attn_norm_qc", attn_norm_qc), ("kv_norm", kv_norm), ("kv_norm_bias", kv_norm_bias),
                 ("attn_norm_kvc", attn_norm_kvc)):
        _dev(n, t)
    _dev("position", position, torch.int64)
    dt = _act_dtype("mla_prepare", attn_qkvc, q_norm, q_norm_bias, attn_norm_qc, kv_norm, kv_norm_bias,
                    attn_norm_kvc)
    f = _freqs_f32(freqs, rope_head_dim)
    T = attn_qkvc.shape[0]
    _req(attn_qkvc.numel() == T * (q_lora_rank + kv_lora_rank + rope_head_dim), "mla_prepare: attn_qkvc shape mismatch")
    _req(attn_norm_qc.numel() == T * q_lora_rank and attn_norm_kvc.numel() == T * kv_lora_rank,
         "mla_prepare: output shape mismatch")
    if block_size:
        _dev("k_cache", k_cache, attn_qkvc.dtype)
        _dev("pe_cache", pe_cache, attn_qkvc.dtype)
        _dev("slot_mapping", slot_mapping, torch.int32)
        _req(slot_mapping.numel() >= T, "mla_prepare: slot_mapping too short")
    _lib.check(rt._lib.xlite_hip_mla_prepare(
        rt.stream(), _ptr(attn_qkvc), _ptr(q_norm), _ptr(q_norm_bias), _ptr(attn_norm_qc), _ptr(kv_norm),
        _ptr(kv_norm_bias), _ptr(attn_norm_kvc), _ptr(f), _ptr(position), T, q_lora_rank, kv_lora_rank,
        rope_head_dim, block_size, _ptr(k_cache) if block_size else None, _ptr(pe_cache) if block_size else None,
        _ptr(slot_mapping) if block_size else None, float(norm_eps), dt))
    rt.finish()


def get_tile_size_of_cached_kv(cached_lens: List[int], query_lens: List[int], head_num_in_group: int,
                               n_kv_heads: int, block_size: int, aic_num: int) -> int:
    """Host-only; same integer results as the reference tuner (xlite/csrc/auto_tuner.cpp:163-210)."""
    lib = _lib.load()
    n = len(query_lens)
    if len(cached_lens) != n:
        raise RuntimeError("get_tile_size_of_cached_kv: cached_lens and query_lens differ in length")
    arr = ctypes.c_uint32 * max(n, 1)
    rc = lib.xlite_hip_get_tile_size_of_cached_kv(arr(*cached_lens), arr(*query_lens), n, head_num_in_group,
                                                  n_kv_heads, block_size, aic_num)
    if rc < 0:
        _lib.check(rc)
    return rc


def quantize_kv(rt: Runtime, x: torch.Tensor, kv_dtype: torch.dtype = torch.int8):
    """x [..., head_dim] (fp16/bf16) -> (tensor of `kv_dtype` - int8 or float8_e4m3fn - of the same shape, fp32
    scales [...]). Not part of the reference API (its caches are never quantised)."""
    _dev("x", x)
    dt = _act_dtype("quantize_kv", x)
    _req(kv_dtype in _KV_DT, "quantize_kv: kv_dtype must be int8 or float8_e4m3fn")
    d = x.shape[-1]
    rows = x.numel() // d
    q = torch.empty(x.shape, dtype=kv_dtype, device=x.device)
    s = torch.empty(x.shape[:-1], dtype=torch.float32, device=x.device)
    _lib.check(rt._lib.xlite_hip_quantize_kv(rt.stream(), _ptr(x), _ptr(q), _ptr(s), rows, d, dt, _KV_DT[kv_dtype]))
    rt.finish()
    return q, s


def quantize_kv_int8(rt: Runtime, x: torch.Tensor):
    return quantize_kv(rt, x, torch.int8)
