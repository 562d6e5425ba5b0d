"""Library-wide switches, same names as the reference (trident/config.py:16-17).

``use_autotune`` is kept for source compatibility and has no effect: tile shapes are fixed at
compile time per (dtype, head size, variant). ``use_trace`` wraps the operation and each kernel
launch in roctx ranges (the reference uses NVTX ranges, trident/util/util.py:93-100).

``dropout_seed``: None draws a fresh 63-bit Philox seed from torch's default CPU generator for
every forward call with dropout (so ``torch.manual_seed`` makes runs repeatable; the reference
draws a non-deterministic one, trident/operation/attention.py:125). An ``int`` or a
``(seed, offset)`` pair fixes the stream: the seed is used as given and the offset advances by
one per forward call.

``reference_limits``: True keeps the reference's argument rules for attention (sequence length and head size
powers of two, boolean masks rejected with its error text, trident/operation/attention.py:31-45). False lifts
the two that the kernels here do not need: any sequence length is accepted, and a boolean mask is taken the way
torch.nn.functional.scaled_dot_product_attention takes it (True = the key takes part; it becomes an additive
0 / -inf mask and has no gradient).

``cache_mask_classes``: True keeps the classification of an additive mask's 64 x 64 blocks (all zero / all -inf / mixed,
one pass over the mask) per mask tensor, so that the backward call and later calls with the same unmodified tensor reuse
it. torch's version counter invalidates an entry; a write it does not see (``mask.data``, a raw pointer, a graph replay
into the mask's memory) does not: set this to False then (every call classifies again), or call
``trident_amd.operation.forget_mask_classes()`` after such a write.
"""
use_autotune = True
use_trace = False
dropout_seed = None
reference_limits = True
cache_mask_classes = True
