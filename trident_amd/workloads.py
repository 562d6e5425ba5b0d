"""Seeded synthetic inputs of the five benchmark configurations.

Tensors are drawn on the CPU in fp32 from ``torch.Generator().manual_seed(seed)`` and then cast,
so a CPU checker and the GPU see identical bits.
"""
import dataclasses
import math

import torch


@dataclasses.dataclass(frozen=True)
class Workload:
    name: str
    dtype: torch.dtype
    B: int
    H: int
    S: int
    D: int
    is_causal: bool = False
    masked: bool = False       # additive fp32 mask [B,1,S,S], keys >= len_b set to -inf
    dense_mask: bool = False   # (with masked) N(0, 0.25) in every entry instead: no block of it is all zero or all -inf
    dropout_p: float = 0.0
    sigma_qkv: float = 1.0
    backward: bool = True
    seed: int = 0
    dropout_seed: int = 0x5EED

    @property
    def scale(self):
        return 1.0 / math.sqrt(self.D)

    def flops(self, backward=False):
        f = 4.0 * self.B * self.H * self.S * self.S * self.D
        if backward:
            f *= 3.5  # 14 B H S^2 D for forward + backward
        return f * (0.5 if self.is_causal else 1.0)


WORKLOADS = {
    "C1": Workload("C1", torch.float32, 2, 4, 64, 32, backward=False, seed=1001),
    "C2": Workload("C2", torch.float16, 4, 16, 1024, 64, backward=False, seed=1002),
    "C3": Workload("C3", torch.bfloat16, 2, 16, 4096, 128, is_causal=True, seed=1003),
    "C4": Workload("C4", torch.bfloat16, 8, 12, 2048, 64, masked=True, seed=1004),
    "C5": Workload("C5", torch.bfloat16, 1, 32, 16384, 128, is_causal=True, dropout_p=0.1, sigma_qkv=0.5, seed=1005),
}

# Beyond the five benchmark configurations: C3's shape in fp32 (the kernels on the fp32 matrix instruction at a real
# size), 16-bit problems with head sizes 32 and 16, and C4's shape at D = 128 with a dense fp32 mask shared by the heads.
EXTRA_WORKLOADS = {
    "F3": Workload("F3", torch.float32, 2, 16, 4096, 128, is_causal=True, seed=1103),
    "H32": Workload("H32", torch.bfloat16, 8, 16, 2048, 32, is_causal=True, seed=1132),
    "H16": Workload("H16", torch.bfloat16, 8, 16, 2048, 16, is_causal=True, seed=1116),
    "M128": Workload("M128", torch.bfloat16, 8, 12, 2048, 128, masked=True, dense_mask=True, seed=1128),
}


def length_mask(B, S, generator):
    """fp32 additive mask [B,1,S,S]: per batch a length in [S/2, S]; keys >= length are -inf."""
    lengths = torch.randint(S // 2, S + 1, (B,), generator=generator)
    cols = torch.arange(S)
    mask = torch.zeros(B, 1, S, S, dtype=torch.float32)
    for b in range(B):
        mask[b, 0, :, cols >= lengths[b]] = float("-inf")
    return mask, lengths


def make_inputs(w: Workload, B=None, H=None, S=None):
    """(q, k, v, d_o, mask) on the CPU in w.dtype (mask fp32 or None). B/H/S override the
    configured sizes for reduced-size parity runs."""
    B = w.B if B is None else B
    H = w.H if H is None else H
    S = w.S if S is None else S
    g = torch.Generator().manual_seed(w.seed)
    shape = (B, H, S, w.D)
    q = (torch.randn(shape, generator=g) * w.sigma_qkv).to(w.dtype)
    k = (torch.randn(shape, generator=g) * w.sigma_qkv).to(w.dtype)
    v = (torch.randn(shape, generator=g) * w.sigma_qkv).to(w.dtype)
    d_o = torch.randn(shape, generator=g).to(w.dtype)
    mask = None
    if w.masked:
        mask = 0.5 * torch.randn(B, 1, S, S, generator=g) if w.dense_mask else length_mask(B, S, g)[0]
    return q, k, v, d_o, mask
