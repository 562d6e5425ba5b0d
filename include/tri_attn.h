/* tri_attn.h — C ABI of libtrident_attn.so: scaled-dot-product attention forward and backward
 * for one MI355X (gfx950).
 *
 * This library replaces the three Triton launches of the reference's attention operation:
 *   kernel.Attention.forward       launched at trident/operation/attention.py:109-131
 *   kernel.Softmax.backward_delta  launched at trident/operation/attention.py:161-163
 *   kernel.Attention.backward      launched at trident/operation/attention.py:170-199
 * (kernel argument lists: trident/kernel/attention.py:33-56 and :169-197,
 *  trident/kernel/softmax.py:184-193).
 *
 * Conventions
 *   - Every pointer is a device pointer owned by the caller; the library never allocates or
 *     frees memory and never synchronises the device. Work is enqueued on `stream`
 *     (a hipStream_t; NULL = the default stream) and the buffers must stay alive until the
 *     stream has passed the call.
 *   - Tensors are [B, H, S, D] with element strides given for all four dimensions.
 *     The innermost (D) stride of q, k, v, o, d_o, dq, dk, dv must be 1.
 *   - lse and delta are dense fp32 [B, H, S]. lse holds log2(sum_j exp(s_ij)) with
 *     s = q k^T * softmax_scale + mask, i.e. natural-log LSE times log2(e)
 *     (the same log2-domain statistic the reference saves, trident/kernel/attention.py:164,
 *     but always fp32). For fp16/bf16 problems the 16-bit matrix-core kernels sum the probabilities as rounded to
 *     that type (the values that multiply V), so lse is accurate to half an ulp of the type times log2(e)
 *     (2.8e-3 for bf16, 3.5e-4 for fp16), not to fp32 precision; the backward calls expect this very lse.
 *     (fp32 problems keep fp32 products and sums throughout; 16-bit problems on the 32-row-tile kernels sum the
 *     probabilities in fp32 before rounding them for the product with V, so their lse has fp32 accuracy.)
 *   - mask is additive, dtype mask_dtype, logical shape [B, H, S, S] with element strides;
 *     a stride of 0 broadcasts that dimension; the innermost mask stride must be 1.
 *     mask and is_causal are mutually exclusive (trident/operation/attention.py:41-43).
 *   - A query row whose keys are ALL masked (-inf) behaves as in softmax: its output row and lse are NaN / -inf,
 *     and in the backward its probabilities are NaN, which makes its dQ row and all of that head's dK and dV
 *     NaN (what the reference's kernel and torch's attention give as well).
 *   - Causal rule: key j is visible to query i iff i >= j (trident/kernel/attention.py:131-134).
 *   - Dropout acts on the probabilities: P is multiplied by keep/(1 - thr8/256) where
 *     thr8 = clamp(rint(dropout_p * 256), 0, 256) and keep comes from Philox4x32-10:
 *       key = (seed & 0xffffffff, seed >> 32); ctr = (j >> 2, i >> 2, b*H + h, offset);
 *       u8 = (r[i & 3] >> (8 * (j & 3))) & 0xff; keep = u8 >= thr8.
 *     The backward calls must be given the same seed, offset and dropout_p as the forward.
 *   - All entry points return 0 on success, a negative TRI_ATTN_E* code for an argument
 *     error, or a positive hipError_t if a launch failed. They are re-entrant; the only
 *     state the library keeps is, per GPU, its compute-unit count (asked once, sizes the persistent
 *     launches) and the address of tri_attn_bwd_noalloc's buffer.
 */
#ifndef TRI_ATTN_H
#define TRI_ATTN_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define TRI_ATTN_ABI_VERSION 3

enum {
    TRI_ATTN_F32 = 0,
    TRI_ATTN_F16 = 1,
    TRI_ATTN_BF16 = 2
};

enum {
    TRI_ATTN_OK = 0,
    TRI_ATTN_ENULL = -1,      /* a required pointer is NULL */
    TRI_ATTN_ESHAPE = -2,     /* B,H,S,D out of range or D not in {16,32,64,128} */
    TRI_ATTN_EDTYPE = -3,     /* unknown dtype / mask_dtype */
    TRI_ATTN_ESTRIDE = -4,    /* innermost stride is not 1, or a stride is negative */
    TRI_ATTN_EMASKCAUSAL = -5,/* both mask and is_causal set */
    TRI_ATTN_EDROPOUT = -6,   /* dropout_p outside [0,1] */
    TRI_ATTN_ESIZE = -7,      /* struct_size does not match this ABI version */
    TRI_ATTN_EALIGN = -8,     /* a pointer or stride breaks the 16-byte alignment the kernels need */
    TRI_ATTN_ENOFUSE = -9,    /* tri_attn_bwd_dq_delta only: no fused kernel serves this problem, nothing was launched */
    TRI_ATTN_ESCRATCH = -10   /* tri_attn_bwd_noalloc only: B*H*S exceeds TRI_ATTN_NOALLOC_MAX_ROWS, nothing was launched */
};

typedef struct TriAttnArgs {
    uint32_t struct_size;      /* = sizeof(TriAttnArgs) */
    int32_t dtype;             /* TRI_ATTN_F32 / F16 / BF16: element type of q,k,v,o,d_o,dq,dk,dv */
    int32_t B, H, S, D;        /* y_size = S, x_size = D in the reference's naming */
    int32_t is_causal;
    int32_t mask_dtype;        /* element type of mask and dmask */
    float softmax_scale;
    float dropout_p;
    uint64_t seed;             /* Philox key */
    uint64_t offset;           /* Philox counter word 3 (low 32 bits used) */

    const void* q;             /* query  (query_ptr) */
    const void* k;             /* key    (key_ptr) */
    const void* v;             /* value  (value_ptr) */
    void* o;                   /* output (output_ptr); input to the backward calls */
    float* lse;                /* log2sum_ptr, fp32 [B,H,S]; written by fwd, read by bwd */
    const void* mask;          /* mask_ptr or NULL */
    const void* d_o;           /* grad_output_ptr */
    void* dq;                  /* grad_query_ptr (need not be zeroed) */
    void* dk;                  /* grad_key_ptr */
    void* dv;                  /* grad_value_ptr */
    void* dmask;               /* grad_mask_ptr or NULL: logical [B,H,S,S] through dmask_stride, in mask_dtype. A stride of 0
                                  sums the gradient over that dimension (a broadcast mask): the buffer must then be fp32 and
                                  zero-filled by the caller, and the kernels add to it atomically (order of summation not fixed) */
    float* delta;              /* delta_ptr, fp32 [B,H,S]: written by bwd_delta, read by dkdv/dq */

    int64_t q_stride[4];
    int64_t k_stride[4];
    int64_t v_stride[4];
    int64_t o_stride[4];
    int64_t do_stride[4];
    int64_t dq_stride[4];
    int64_t dk_stride[4];
    int64_t dv_stride[4];
    int64_t mask_stride[4];
    int64_t dmask_stride[4];

    void* stream;              /* hipStream_t */

    uint8_t* mask_classes;     /* NULL, or the classes of the mask's 64 x 64 blocks, filled by tri_attn_classify_mask and then
                                  read by tri_attn_fwd / tri_attn_bwd*: dense [MB][MH][RB][S/64] bytes with MB = B (1 if
                                  mask_stride[0] == 0), MH = H (1 if mask_stride[1] == 0), RB = S/64 (1 if mask_stride[2] == 0);
                                  0 = every entry of the block is 0, 1 = every entry is -inf, 2 = anything else.
                                  Only used where S is a multiple of 128. */
} TriAttnArgs;

/* ABI version of the loaded library (TRI_ATTN_ABI_VERSION it was built with). */
int tri_attn_version(void);

/* Text for a status code returned by any entry point below. */
const char* tri_attn_strerror(int status);

/* Replaces kernel.Attention.forward (trident/kernel/attention.py:33-165; launch at
 * trident/operation/attention.py:109-131). Reads q,k,v[,mask]; writes o and lse. */
int tri_attn_fwd(const TriAttnArgs* args);

/* Replaces kernel.Softmax.backward_delta as attention uses it (trident/kernel/softmax.py:184-238;
 * launch at trident/operation/attention.py:161-163). Reads o, d_o; writes delta = rowsum(d_o * o). */
int tri_attn_bwd_delta(const TriAttnArgs* args);

/* First half of kernel.Attention.backward (trident/kernel/attention.py:169-339; launch at
 * trident/operation/attention.py:170-199): dK and dV, one workgroup per key tile.
 * Reads q,k,v,d_o,lse,delta[,mask]; writes dk, dv. */
int tri_attn_bwd_dkdv(const TriAttnArgs* args);

/* Second half of kernel.Attention.backward: dQ (and dMask when args->dmask is set), one
 * workgroup per query tile, so every dQ tile is written once and needs no zero fill
 * (the reference accumulates into a zeroed dQ, trident/kernel/attention.py:321-323).
 * Reads q,k,v,d_o,lse,delta[,mask]; writes dq[, dmask]. */
int tri_attn_bwd_dq(const TriAttnArgs* args);

/* bwd_delta and bwd_dq in one launch, for the problems whose dQ kernel can compute delta from the dO
 * rows it loads anyway (the 16-bit matrix-core kernels without a mask: fp16/bf16, D in {16,32,64,128}, 16-byte
 * aligned rows of o): reads q,k,v,o,d_o,lse; writes delta and dq. tri_attn_bwd_dkdv, which reads delta, has to
 * follow it. Returns TRI_ATTN_ENOFUSE without launching anything where it does not apply (then call
 * tri_attn_bwd_delta, tri_attn_bwd_dkdv, tri_attn_bwd_dq). The reference has the two launches only
 * (trident/operation/attention.py:161-199); tri_attn_bwd picks between the two sequences itself. */
int tri_attn_bwd_dq_delta(const TriAttnArgs* args);

/* The whole backward (trident/operation/attention.py:137-202): the results of bwd_delta, bwd_dkdv and
 * bwd_dq called in that order, written to delta, dk, dv, dq[, dmask]. The library may launch fewer
 * kernels and in another order: without a mask, for sequence lengths that are multiples of 256 (and
 * without dropout at D = 128) the dQ kernel computes delta on its way and runs before dK/dV. */
int tri_attn_bwd(const TriAttnArgs* args);

/* tri_attn_bwd for callers that cannot allocate device memory (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc). It has no counterpart in the reference, whose backward allocates
 * delta itself (trident/operation/attention.py:155). Same results as tri_attn_bwd on the same arguments,
 * except that args->delta is ignored (it may be NULL): delta lives in a buffer inside the library,
 * TRI_ATTN_NOALLOC_MAX_ROWS fp32 values (4 MiB) that every GPU the library runs on holds until the process
 * ends. B*H*S above that limit returns TRI_ATTN_ESCRATCH and launches nothing. The call allocates and frees
 * nothing. All calls on one GPU share that GPU's buffer: calls that may overlap on one GPU (different streams
 * or threads) race on it and must be serialised by the caller; calls on one stream are ordered. */
#define TRI_ATTN_NOALLOC_MAX_ROWS (1 << 20)
int tri_attn_bwd_noalloc(const TriAttnArgs* args);

/* Classifies the 64 x 64 blocks of args->mask into args->mask_classes (see there; caller-allocated, size
 * tri_attn_mask_classes_size(args) bytes). It has no counterpart in the reference, whose kernel adds every mask
 * tile as it comes (trident/kernel/attention.py:135-138). With the classes at hand the kernels skip key tiles
 * that are masked out altogether and do not read mask tiles that are all zero (a key-padding or length mask is
 * made of such tiles but for one column of blocks). A tile whose mask is all zero then takes the arithmetic of a tile
 * without a mask (the scale folded into one fused multiply-add per score instead of a product, a sum and a
 * difference): results agree with those computed without classes to the last fp32 rounding of a score's exponent, i.e.
 * to within an ulp of the 16-bit outputs, not bit for bit. Reads mask; writes mask_classes.
 * Returns TRI_ATTN_ENOFUSE (nothing launched) where the classes would not be used: S not a multiple of 128. */
int tri_attn_classify_mask(const TriAttnArgs* args);
/* Bytes of mask_classes for these arguments (MB * MH * RB * S/64), 0 where tri_attn_classify_mask does not apply, or a
 * negative TRI_ATTN_E* code. */
int64_t tri_attn_mask_classes_size(const TriAttnArgs* args);

/* Which kernel family a call would run, without launching anything (no counterpart in the reference): pass 0 =
 * tri_attn_fwd, 1 = tri_attn_bwd_dkdv, 2 = tri_attn_bwd_dq on these arguments. Returns 1 for the 16-bit matrix-core
 * (MFMA) kernels (fp16/bf16, D in {16,32,64,128}, 16-byte aligned rows; any S without a mask, S a multiple of 128 with
 * one); 2 for the 32-row-tile matrix-core kernels (everything else whose pointers and strides are multiples of
 * four elements: fp32 problems on the fp32 matrix instruction with fp32 products and sums; fp16/bf16 problems with
 * masked lengths that are no multiple of 128 on the 16-bit 32x32x8 instruction);
 * 0 for the general vector-ALU kernels (views that are not aligned so); or a negative TRI_ATTN_E* code. */
int tri_attn_uses_matrix_cores(const TriAttnArgs* args, int pass);

/* Debug / parity helper with no counterpart in the reference (its dropout stream is unpinned):
 * writes the dropout keep decisions (1 = kept) for head index bh, rows [row0,row0+rows),
 * cols [col0,col0+cols) into keep[rows*cols] (device, uint8) using exactly the device code
 * the attention kernels use. */
int tri_attn_dropout_mask(uint64_t seed, uint64_t offset, float dropout_p, uint32_t bh,
                          int32_t row0, int32_t rows, int32_t col0, int32_t cols,
                          uint8_t* keep, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* TRI_ATTN_H */
