/* tri_rowops.h — C ABI of the attention path's sibling operations in libtrident_attn.so: row softmax,
 * masked row softmax and dropout for one MI355X (gfx950). All three are HBM-bound streaming kernels.
 *
 * They replace these Triton launches of the reference:
 *   kernel.Softmax.forward / backward_delta / backward
 *       trident/kernel/softmax.py:34-121, 180-238, 123-178; launched at trident/operation/softmax.py:57-65, 81-107
 *   kernel.MaskedSoftmax.forward / backward_delta / backward
 *       trident/kernel/masked_softmax.py:25-199; launched at trident/operation/masked_softmax.py:57-67, 83-113
 *   kernel.Dropout.forward / backward
 *       trident/kernel/dropout.py:35-133; launched at trident/operation/dropout.py:59-61, 74-76
 *
 * Conventions (shared with tri_attn.h): device pointers owned by the caller, nothing is allocated or
 * synchronised, work is enqueued on `stream`, 0 / negative TRI_ATTN_E* / positive hipError_t is returned.
 *
 * Row operations see a matrix of y_size rows and x_size columns through element strides (y_stride, x_stride),
 * ONE stride pair for every tensor of the call, as the reference's kernels do (trident/kernel/softmax.py:41-44):
 * softmax runs along x. The reference reaches dim = 0 of a 2-D tensor by exchanging the roles of the two
 * strides (trident/util/util.py:65-76); so does the wrapper here.
 *   softmax:        out[y,x] = exp(in[y,x] - max_x) / sum_x exp(in[y,x] - max_x), statistics in fp32
 *   masked softmax: the same with in[y,x] = -inf wherever mask[y,x] > 2.220446049250313e-16
 *                   (trident/kernel/masked_softmax.py:76; mask has its own dtype, the input's strides)
 *   backward:       delta[y] = sum_x grad_out[y,x] * out[y,x];  grad_in[y,x] = out[y,x] * (grad_out[y,x] - delta[y])
 *                   (the reference's two launches backward_delta + backward are one launch here; delta is fp32
 *                   and never leaves the chip)
 * Dropout sees a flat array of n elements: out[i] = keep(i) ? in[i] * 256 / (256 - thr8) : 0 with
 *   thr8 = clamp(rint(p * 256), 0, 256), keep(i) = u8(i) >= thr8,
 *   u8(i) = byte (i & 3) of word ((i >> 2) & 3) of Philox4x32-10(ctr = (lo32(i >> 4), hi32(i >> 4), 0x44524F50, offset),
 *                                                               key = (lo32(seed), hi32(seed)))
 * and grad_in[i] = keep(i) ? grad_out[i] * 256 / (256 - thr8) : 0 with the SAME (seed, offset, p).
 * This is the standard dropout gradient on a documented counter-based stream (same generator and 8-bit
 * threshold as the attention dropout in tri_attn.h). The reference draws tl.rand(seed, i) > p with a
 * non-deterministic seed, and its backward multiplies by (1 - p) and keeps the gradient where out > 0
 * (trident/kernel/dropout.py:70-71, 128-129); neither is pinned by its tests (p in {0, 1} only, where all of
 * these agree) and neither is copied.
 */
#ifndef TRI_ROWOPS_H
#define TRI_ROWOPS_H

#include <stdint.h>

#include "tri_attn.h"

#ifdef __cplusplus
extern "C" {
#endif

enum {  /* mask_dtype beyond TRI_ATTN_F32 / F16 / BF16 */
    TRI_ROW_MASK_I64 = 3,
    TRI_ROW_MASK_I32 = 4,
    TRI_ROW_MASK_U8 = 5   /* uint8 or bool */
};

typedef struct TriRowArgs {
    uint32_t struct_size;      /* = sizeof(TriRowArgs) */
    int32_t dtype;             /* TRI_ATTN_F32 / F16 / BF16: input, output, grad_output, grad_input */
    int64_t y_size, x_size;    /* rows, row length (dropout: n = y_size * x_size contiguous elements) */
    int64_t y_stride, x_stride;/* element strides, shared by all tensors of the call (dropout ignores them) */
    const void* input;         /* input_ptr (forward) */
    void* output;              /* output_ptr: written by forward, read by softmax backward */
    const void* mask;          /* mask_ptr or NULL */
    int32_t mask_dtype;
    float p;                   /* dropout probability */
    const void* grad_output;   /* grad_output_ptr (backward) */
    void* grad_input;          /* grad_input_ptr (backward) */
    uint64_t seed;             /* dropout: Philox key */
    uint64_t offset;           /* dropout: Philox counter word 3 (low 32 bits used) */
    void* stream;              /* hipStream_t */
} TriRowArgs;

/* kernel.Softmax.forward and, with args->mask set, kernel.MaskedSoftmax.forward. Reads input[, mask]; writes output. */
int tri_softmax_fwd(const TriRowArgs* args);

/* kernel.Softmax.backward_delta + kernel.Softmax.backward (and the MaskedSoftmax pair, which computes the same
 * thing: masked positions have output 0). Reads output, grad_output; writes grad_input. */
int tri_softmax_bwd(const TriRowArgs* args);

/* kernel.Dropout.forward. Reads input; writes output. */
int tri_dropout_fwd(const TriRowArgs* args);

/* kernel.Dropout.backward. Reads grad_output; writes grad_input (regenerates the keep decisions from seed, offset, p). */
int tri_dropout_bwd(const TriRowArgs* args);

#ifdef __cplusplus
}
#endif
#endif /* TRI_ROWOPS_H */
