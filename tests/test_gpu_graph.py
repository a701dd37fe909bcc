"""GPU: the library's launches can be captured into a HIP graph and replayed.

A serving loop captures one decode step and replays it while the device-side lengths, block
table and activations change underneath.  That works only if a call does nothing but launch
kernels once its workspaces have their size: no allocation, no memset node, no host round
trip.  Every replay is checked against the same call made eagerly on copies of the inputs.
"""

import pytest
import torch

from pypto_amd import workloads
from pypto_amd.runtime import decoder_layer_decode, ffn_block, paged_attention

pytestmark = pytest.mark.gpu


def _cuda(args, keep_host=()):
    return [a.cuda() if isinstance(a, torch.Tensor) and i not in keep_host else a for i, a in enumerate(args)]


def _capture(worker, program, args, stream):
    """Warm-up call (sizes the workspaces), then the same call recorded into a graph."""
    with torch.cuda.stream(stream):
        with worker.register(program) as h:
            h(*args, stream=stream.cuda_stream)
        stream.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            with worker.register(program) as h:
                h(*args, stream=stream.cuda_stream)
    return graph


@pytest.mark.parametrize("batch", [6, 40])
def test_decoder_layer_replays_follow_growing_sequences(worker, batch):
    """Batch 6 takes the skinny projections, batch 40 the tiled GEMMs whose k-split slabs feed the
    RoPE and RMSNorm kernels directly (a scratch area of their own)."""
    if batch == 6:
        ctxs = [100, 1, 250, 33, 60, 129]  # four more tokens stay inside each last block
    else:
        g0 = torch.Generator().manual_seed(21)
        ctxs = (torch.randint(0, 5, (batch,), generator=g0) * 64 + torch.randint(1, 59, (batch,), generator=g0)).tolist()
    inp = workloads.decoder_layer_inputs(batch=batch, hidden=1024, num_heads=8, kv_head_num=2, head_dim=128,
                                         intermediate=2816, block_size=64, context_lens=ctxs, seed=11)
    args = _cuda(inp.args())
    hidden, seq_lens, key_cache, value_cache, out = args[0], args[1], args[3], args[4], args[19]
    assert out.shape == hidden.shape
    stream = torch.cuda.Stream()
    # eager twin on its own copies of everything the step writes
    twin = list(args)
    for i in (0, 1, 3, 4, 19):
        twin[i] = args[i].clone()
    graph = _capture(worker, decoder_layer_decode, args, stream)
    # the warm-up and the capture's own (unexecuted) call left the caches one step ahead of the twin
    with worker.register(decoder_layer_decode) as h:
        h(*twin)
    worker.sync()
    g = torch.Generator(device="cuda").manual_seed(5)
    for step in range(4):
        # next decode step: one more token per sequence, new activations
        new_hidden = torch.randn(hidden.shape, generator=g, device="cuda").to(hidden.dtype)
        for a in (args, twin):
            a[0].copy_(new_hidden)
            a[1].add_(1)
        torch.cuda.synchronize()
        graph.replay()
        with worker.register(decoder_layer_decode) as h:
            h(*twin)
        torch.cuda.synchronize()
        assert torch.isfinite(out.float()).all()
        assert torch.equal(out, twin[19]), f"replay {step} differs from the eager step"
        assert torch.equal(key_cache, twin[3]) and torch.equal(value_cache, twin[4])
    assert int(seq_lens[0]) == ctxs[0] + 4


def test_attention_and_ffn_replays(worker):
    att = workloads.paged_attention_inputs(batch=4, num_heads=16, kv_head_num=4, head_dim=128, block_size=64,
                                           context_lens=[300, 40, 1, 680], ctx_range=(1, 1024), seed=3)
    a_args = _cuda(att.args(), keep_host=(6,))
    ffn = workloads.ffn_inputs(tokens=200, hidden=1024, intermediate=2816, seed=4)
    f_args = _cuda((ffn.x, ffn.gamma, ffn.w_gate, ffn.w_up, ffn.w_down, ffn.out, ffn.eps))
    stream = torch.cuda.Stream()
    # The FFN call after the attention capture needs a larger scratch buffer than the one the
    # attention launches were recorded with: the outgrown buffer must stay allocated.
    ga = _capture(worker, paged_attention, a_args, stream)
    gf = _capture(worker, ffn_block, f_args, stream)
    for step in range(3):
        a_args[4].add_(5)                       # longer contexts, still inside each sequence's last block
        f_args[0].mul_(0.5)
        a_args[5].fill_(float("nan"))
        f_args[5].fill_(float("nan"))
        torch.cuda.synchronize()
        ga.replay()
        gf.replay()
        torch.cuda.synchronize()
        got_a, got_f = a_args[5].clone(), f_args[5].clone()
        with worker.register(paged_attention) as h:
            h(*a_args)
        with worker.register(ffn_block) as h:
            h(*f_args)
        worker.sync()
        assert torch.equal(got_a, a_args[5]), f"attention replay {step}"
        assert torch.equal(got_f, f_args[5]), f"ffn replay {step}"
