"""Library-wide switches, same names as the reference (trident/config.py:16-17).

``use_autotune`` is kept for source compatibility and has no effect: tile shapes are fixed at
compile time per (dtype, head size, variant). ``use_trace`` wraps the operation and each kernel
launch in roctx ranges (the reference uses NVTX ranges, trident/util/util.py:93-100).

``dropout_seed``: None draws a fresh 63-bit Philox seed from torch's default CPU generator for
every forward call with dropout (so ``torch.manual_seed`` makes runs repeatable; the reference
draws a non-deterministic one, trident/operation/attention.py:125). An ``int`` or a
``(seed, offset)`` pair fixes the stream: the seed is used as given and the offset advances by
one per forward call.
"""
use_autotune = True
use_trace = False
dropout_seed = None
