"""Host calls from several threads: the library's dispatch lock makes them take turns, and launches
that share the default stream still see the shared scratch areas in submission order."""

import threading

import pytest
import torch

import oracle
from pypto_amd import workloads
from pypto_amd.runtime import ffn_block, paged_attention, rms_norm, validate_golden

pytestmark = pytest.mark.gpu


def test_two_threads_run_different_programs_concurrently(worker):
    att = workloads.paged_attention_inputs(batch=5, num_heads=16, kv_head_num=4, block_size=64,
                                           context_lens=[900, 64, 333, 1, 2048], ctx_range=(1, 2048), seed=8)
    att_ref = oracle.paged_attention_golden(att.query, att.key_cache, att.value_cache, att.block_table,
                                            att.context_lens, att.config)
    f = workloads.ffn_inputs(tokens=200, hidden=512, intermediate=1408, seed=9)
    ffn_ref = oracle.ffn_block(f.x, f.gamma, f.w_gate, f.w_up, f.w_down, f.eps)
    g = torch.Generator().manual_seed(1)
    x = torch.randn((64, 4096), generator=g).to(torch.bfloat16)
    gamma = 1 + 0.02 * torch.randn((1, 4096), generator=g)
    norm_ref = oracle.rms_norm(x, gamma, 1e-6, out_dtype=torch.bfloat16)

    errors = []
    start = threading.Barrier(3)

    def loop(program, make_args, out_of, ref, tol):
        try:
            with worker.register(program) as h:
                start.wait()
                for _ in range(12):
                    args = make_args()
                    h(*args)
                    validate_golden({"out": out_of(args).float()}, {"out": ref.float()}, **tol)
        except Exception as e:  # noqa: BLE001 - reported by the main thread
            errors.append(e)

    def att_args():
        return (att.query, att.key_cache, att.value_cache, att.block_table, att.context_lens,
                torch.full_like(att.out, float("nan")), att.config)

    def ffn_args():
        return (f.x, f.gamma, f.w_gate, f.w_up, f.w_down, torch.full_like(f.out, float("nan")), f.eps)

    def norm_args():
        return (x, gamma, torch.zeros_like(x), 1e-6)

    threads = [
        threading.Thread(target=loop, args=(paged_attention, att_args, lambda a: a[5], att_ref, dict(rtol=2e-2, atol=1e-2))),
        threading.Thread(target=loop, args=(ffn_block, ffn_args, lambda a: a[5], ffn_ref, dict(rtol=2e-2, atol=1e-2))),
        threading.Thread(target=loop, args=(rms_norm, norm_args, lambda a: a[2], norm_ref, dict(rtol=8e-3, atol=8e-3))),
    ]
    for t in threads:
        t.start()
    for t in threads:
        t.join(timeout=110)
    assert not any(t.is_alive() for t in threads), "a thread did not finish"
    assert not errors, errors[0]
