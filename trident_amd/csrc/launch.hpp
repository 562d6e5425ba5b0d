// Host-side launch entry points shared between the translation units of libtrident_attn.so.
#pragma once
#include <hip/hip_runtime.h>

#include "common.hpp"

namespace tri {

enum GenericKernel { kGenericFwd = 0, kGenericDelta = 1, kGenericDkdv = 2, kGenericDq = 3 };

// generic.hip: any shape / dtype, vector-ALU fp32 arithmetic.
int launch_generic_any(int which, int dtype, const KParams& p, hipStream_t stream);

// mfma_*.hip: fp16/bf16, D in {64,128}, 16-byte aligned rows; any S without a mask, S a multiple of 128 with one.
enum MfmaKernel { kMfmaFwd = 0, kMfmaDkdv = 1, kMfmaDq = 2 };
bool mfma_supported(int which, int dtype, const KParams& p);
int launch_mfma_fwd(int dtype, const KParams& p, hipStream_t stream);
// with_delta: the dQ pass also computes and stores delta (only where mfma_dq_fuses_delta() says so; the
// dK/dV pass must then follow it)
int launch_mfma_dq(int dtype, const KParams& p, hipStream_t stream, bool with_delta = false);
bool mfma_dq_fuses_delta(const KParams& p);
int launch_mfma_dkdv(int dtype, const KParams& p, hipStream_t stream);
int launch_delta(int dtype, const KParams& p, hipStream_t stream);

// mfma32.hip: the fp32 matrix instruction. fp32 / fp16 / bf16 storage, D in {16,32,64,128}, any S, any mask, rows
// aligned to four elements. `which` is a MfmaKernel.
bool mfma32_supported(int which, int dtype, const KParams& p);
int launch_mfma32(int which, int dtype, const KParams& p, hipStream_t stream);
// Classes of the mask's 64 x 64 blocks (0 all zero, 1 all -inf, 2 mixed) into `out`, laid out as p.mcs says.
int launch_classify_mask(const KParams& p, uint8_t* out, hipStream_t stream);
enum MaskClass { kMaskZero = 0, kMaskNegInf = 1, kMaskMixed = 2 };
// Number of workgroups for a kernel whose workgroups are persistent (one per CU, each walking several of
// the `items`): min(items, CUs of the current device).
int persistent_grid(int items);

}  // namespace tri
