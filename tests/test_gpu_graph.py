"""The operators under HIP graph capture: a decode step (rope_and_cache + attention) and an MLA decode call are
captured once and replayed several times on changed inputs, with eager work and synchronisations between the
replays; every replay must give the bits of the eager call on the same inputs. (The library enqueues kernels
only: no allocation, no memset, no synchronisation; the scratch pool is grown before the capture.)"""
import pytest
import torch

from gvirt_amd import workloads as W

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def test_decode_step_and_mla_under_graph_capture(rt):
    from gvirt_amd._C import attention, mla_attention, rope_and_cache
    blocking = rt.blocking
    rt.blocking = False
    try:
        s = W.LLAMA3_8B
        ctx = [700, 3000, 129, 2048, 64, 1500, 4096, 33]
        w = W.gqa_decode(s, ctx, 51, device=DEV)
        r = W.rope_inputs(s, w, 52)
        m = W.mla_decode(W.MlaShape(), [900, 2500, 77, 4000], 53, device=DEV)
        ms = m["shape"]

        def step():
            rope_and_cache(rt, r["inout"], w["k_cache"], w["v_cache"], r["position"], r["cosin"], r["slot_mapping"],
                           s.n_heads, s.n_kv_heads, s.head_dim, s.head_dim, s.block_size, True)
            attention(rt, r["inout"], w["k_cache"], w["v_cache"], w["output"], w["query_start_loc"],
                      w["lens"], w["cached_lens"], w["block_tables"], s.n_heads, s.n_kv_heads, s.head_dim, s.block_size,
                      w["batch"], w["max_num_block"])
            mla_attention(rt, m["q_absorb"], m["qr"], m["k_cache"], m["pe_cache"], m["o_absorb"], m["query_start_loc"], m["lens"],
                          m["cached_lens"], m["block_tables"], ms.n_heads, ms.rope_head_dim, ms.kv_lora_rank, ms.block_size,
                          m["batch"], m["max_num_blocks"], ms.scale)

        q_in = r["inout"]
        q0, qa0 = q_in.clone(), m["q_absorb"].clone()
        step()                                    # eager warm-up: kernel attributes set, scratch pool grown
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        side = torch.cuda.Stream()
        with torch.cuda.stream(side):
            q_in.copy_(q0)
            with torch.cuda.graph(graph, stream=side):
                step()
        torch.cuda.synchronize()
        for rep in range(4):
            # new inputs for this replay, eager reference first
            q_new = (q0.float() * (1.0 + 0.25 * rep)).to(q0.dtype)
            qa_new = (qa0.float() * (1.0 - 0.1 * rep)).to(qa0.dtype)
            q_in.copy_(q_new); m["q_absorb"].copy_(qa_new)
            step()
            torch.cuda.synchronize()
            want_a, want_m, want_q = w["output"].clone(), m["o_absorb"].clone(), q_in.clone()
            w["output"].zero_(); m["o_absorb"].zero_()
            q_in.copy_(q_new); m["q_absorb"].copy_(qa_new)
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(w["output"], want_a), "attention, replay %d" % rep
            assert torch.equal(m["o_absorb"], want_m), "mla, replay %d" % rep
            assert torch.equal(q_in, want_q), "rope_and_cache, replay %d" % rep
    finally:
        rt.blocking = blocking
