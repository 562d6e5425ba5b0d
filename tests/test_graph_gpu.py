"""The entry points launch kernels and nothing else (no allocation, no memset, no synchronization), so a forward and
a tri_attn_bwd_noalloc call can be recorded into a HIP graph and replayed. Every replay runs on new input values
written into the captured tensors, with eager calls and synchronizations in between, and must reproduce the eager
result of the same inputs bit for bit."""
import ctypes
import math

import pytest
import torch

from trident_amd import _lib, operation

pytestmark = pytest.mark.gpu


def _fresh(shape, dtype, device, seed):
    g = torch.Generator().manual_seed(seed)
    return [torch.randn(*shape, generator=g).to(dtype).to(device) for _ in range(4)]


def _step(lib, tensors, causal, p, backward_entry, delta):
    q, k, v, d_o, o, lse, dq, dk, dv = tensors
    args = operation._make_args(q, k, v, o, lse, None, p, causal, 1.0 / math.sqrt(q.shape[-1]), 77 if p > 0 else 0, 3,
                                d_o, dq, dk, dv, None, delta)
    ref = ctypes.byref(args)
    _lib.check(lib.tri_attn_fwd(ref))
    _lib.check(getattr(lib, backward_entry)(ref))


@pytest.mark.parametrize("dtype,shape,causal,p", [
    (torch.bfloat16, (2, 4, 512, 128), True, 0.0),    # persistent forward, phased dQ with delta, phased dK/dV
    (torch.float16, (1, 3, 256, 64), False, 0.2),     # dropout
    (torch.float32, (2, 2, 200, 32), True, 0.0),      # 32-row-tile kernels (fp32 matrix instruction), ragged length
])
def test_forward_and_backward_replay_from_a_graph(dtype, shape, causal, p, device):
    lib = _lib.lib()
    B, H, S, D = shape

    def buffers():
        q, k, v, d_o = _fresh(shape, dtype, device, 1)
        return [q, k, v, d_o, torch.empty_like(q), torch.empty(B, H, S, device=device, dtype=torch.float32),
                torch.empty_like(q), torch.empty_like(q), torch.empty_like(q)]

    held = buffers()    # the tensors the graph is recorded on
    eager = buffers()
    delta = torch.empty(B, H, S, device=device, dtype=torch.float32)
    # once outside the capture: the library asks for the CU count and its scratch address on first use
    _step(lib, held, causal, p, "tri_attn_bwd_noalloc", None)
    torch.cuda.synchronize()

    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):   # (the argument structure takes torch's current stream: the capturing one)
        _step(lib, held, causal, p, "tri_attn_bwd_noalloc", None)

    for replay in range(3):
        new = _fresh(shape, dtype, device, 100 + replay)
        for dst_h, dst_e, src in zip(held[:4], eager[:4], new):
            dst_h.copy_(src)
            dst_e.copy_(src)
        for t in held[4:] + eager[4:]:
            t.fill_(float("nan"))
        graph.replay()
        _step(lib, eager, causal, p, "tri_attn_bwd", delta)
        torch.cuda.synchronize()
        for name, a, b in zip(("O", "LSE", "dQ", "dK", "dV"), held[4:], eager[4:]):
            assert not torch.isnan(a.float()).any(), f"{name}, replay {replay}"
            assert torch.equal(a, b), f"{name} differs in replay {replay}"
