"""tri_attn_bwd_noalloc (the backward whose delta buffer lives inside the library) against tri_attn_bwd,
through the C ABI: identical kernels on identical inputs, so dQ, dK and dV must agree bit for bit. Two
calls in a row, the second on a smaller problem, because every call on a GPU reuses the same buffer."""
import ctypes
import math

import pytest
import torch

from trident_amd import _lib, operation

pytestmark = pytest.mark.gpu


def _problem(device, B, H, S, D, dtype, causal, p, seed):
    g = torch.Generator().manual_seed(seed)
    q, k, v, d_o = [torch.randn(B, H, S, D, generator=g).to(dtype).to(device) for _ in range(4)]
    o = torch.empty_like(q)
    lse = torch.empty(B, H, S, device=device, dtype=torch.float32)
    return q, k, v, d_o, o, lse, causal, p


def _backward(lib, entry, prob, with_delta):
    q, k, v, d_o, o, lse, causal, p = prob
    D = q.shape[-1]
    dq, dk, dv = [torch.full_like(q, float("nan")) for _ in range(3)]
    delta = torch.empty_like(lse) if with_delta else None
    args = operation._make_args(q, k, v, o, lse, None, p, causal, 1.0 / math.sqrt(D), 4242 if p > 0 else 0, 1,
                                d_o, dq, dk, dv, None, delta)
    ref = ctypes.byref(args)
    _lib.check(lib.tri_attn_fwd(ref))
    _lib.check(getattr(lib, entry)(ref))
    torch.cuda.synchronize()
    return dq, dk, dv


@pytest.mark.parametrize("dtype,D,causal,p", [(torch.bfloat16, 128, True, 0.0), (torch.float16, 64, False, 0.25),
                                              (torch.float32, 32, True, 0.0)])
def test_noalloc_backward_matches_backward(dtype, D, causal, p, device):
    lib = _lib.lib()
    # the second problem is smaller than the first: it finds the first call's delta values in the buffer
    for (B, H, S) in [(2, 3, 512), (1, 2, 256 if dtype != torch.float32 else 100)]:
        prob = _problem(device, B, H, S, D, dtype, causal, p, 900 + S + D)
        want = _backward(lib, "tri_attn_bwd", prob, True)
        got = _backward(lib, "tri_attn_bwd_noalloc", prob, False)   # args.delta stays NULL
        for name, a, b in zip(("dQ", "dK", "dV"), got, want):
            assert not torch.isnan(a.float()).any(), name
            assert torch.equal(a, b), f"{name} differs at B={B} H={H} S={S} D={D}"


def test_noalloc_rejects_sizes_beyond_its_buffer(device):
    lib = _lib.lib()
    args = _lib.TriAttnArgs()
    args.struct_size = ctypes.sizeof(args)
    args.dtype = 2
    args.B, args.H, args.S, args.D = 1, 64, (_lib.NOALLOC_MAX_ROWS // 64) + 128, 64
    assert lib.tri_attn_bwd_noalloc(ctypes.byref(args)) == _lib.ESCRATCH
    assert b"NOALLOC_MAX_ROWS" in lib.tri_attn_strerror(_lib.ESCRATCH)
