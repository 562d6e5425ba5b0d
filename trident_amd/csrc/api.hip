// C ABI of libtrident_attn.so: argument checks, kernel selection, launches.
#include <math.h>
#include <string.h>

#include <atomic>

#include "common.hpp"
#include "launch.hpp"

// Backward scratch of tri_attn_bwd_noalloc (see below): file scope, one copy per GPU. In host code this name is
// only a stand-in for hipGetSymbolAddress; kernels get the device address as an argument.
static __device__ __align__(256) float scratch[TRI_ATTN_NOALLOC_MAX_ROWS];

namespace tri {
namespace {

bool valid_d(int d) { return d == 16 || d == 32 || d == 64 || d == 128; }

int check_strides(const int64_t* s) {
    if (s[3] != 1) return TRI_ATTN_ESTRIDE;
    for (int i = 0; i < 3; ++i)
        if (s[i] < 0) return TRI_ATTN_ESTRIDE;
    return TRI_ATTN_OK;
}

void copy3(int64_t* dst, const int64_t* src) {
    dst[0] = src[0];
    dst[1] = src[1];
    dst[2] = src[2];
}

// Common validation + translation. `need` bits: 1 = forward tensors, 2 = backward tensors.
int make_params(const TriAttnArgs* a, int need, KParams* p) {
    if (a == nullptr) return TRI_ATTN_ENULL;
    if (a->struct_size != sizeof(TriAttnArgs)) return TRI_ATTN_ESIZE;
    if (a->dtype < TRI_ATTN_F32 || a->dtype > TRI_ATTN_BF16) return TRI_ATTN_EDTYPE;
    if (a->B <= 0 || a->H <= 0 || a->S <= 0 || !valid_d(a->D)) return TRI_ATTN_ESHAPE;
    if (static_cast<int64_t>(a->B) * a->H > 2147483647LL / 64) return TRI_ATTN_ESHAPE;
    if (!(a->dropout_p >= 0.f && a->dropout_p <= 1.f)) return TRI_ATTN_EDROPOUT;
    if (a->mask != nullptr && a->is_causal) return TRI_ATTN_EMASKCAUSAL;
    if (a->mask != nullptr || a->dmask != nullptr) {
        if (a->mask_dtype < TRI_ATTN_F32 || a->mask_dtype > TRI_ATTN_BF16) return TRI_ATTN_EDTYPE;
    }
    memset(p, 0, sizeof(*p));
    int rc;
    if (need & 1) {
        if (!a->q || !a->k || !a->v || !a->o || !a->lse) return TRI_ATTN_ENULL;
        if ((rc = check_strides(a->q_stride)) || (rc = check_strides(a->k_stride)) ||
            (rc = check_strides(a->v_stride)) || (rc = check_strides(a->o_stride)))
            return rc;
    }
    if (need & 2) {
        if (!a->o || !a->d_o || !a->delta) return TRI_ATTN_ENULL;
        if ((rc = check_strides(a->o_stride)) || (rc = check_strides(a->do_stride))) return rc;
    }
    if (need & 4) {
        if (!a->q || !a->k || !a->v || !a->lse || !a->d_o || !a->delta || !a->dk || !a->dv) return TRI_ATTN_ENULL;
        if ((rc = check_strides(a->q_stride)) || (rc = check_strides(a->k_stride)) ||
            (rc = check_strides(a->v_stride)) || (rc = check_strides(a->do_stride)) ||
            (rc = check_strides(a->dk_stride)) || (rc = check_strides(a->dv_stride)))
            return rc;
    }
    if (need & 8) {
        if (!a->q || !a->k || !a->v || !a->lse || !a->d_o || !a->delta || !a->dq) return TRI_ATTN_ENULL;
        if ((rc = check_strides(a->q_stride)) || (rc = check_strides(a->k_stride)) ||
            (rc = check_strides(a->v_stride)) || (rc = check_strides(a->do_stride)) ||
            (rc = check_strides(a->dq_stride)))
            return rc;
        if (a->dmask != nullptr) {
            if (a->mask == nullptr) return TRI_ATTN_ENULL;
            if ((rc = check_strides(a->dmask_stride))) return rc;
        }
    }
    if (a->mask != nullptr && (rc = check_strides(a->mask_stride))) return rc;

    p->q = a->q;
    p->k = a->k;
    p->v = a->v;
    p->o = a->o;
    p->lse = a->lse;
    p->mask = a->mask;
    p->d_o = a->d_o;
    p->dq = a->dq;
    p->dk = a->dk;
    p->dv = a->dv;
    p->dmask = (need & 8) ? a->dmask : nullptr;
    p->delta = a->delta;
    copy3(p->qs, a->q_stride);
    copy3(p->ks, a->k_stride);
    copy3(p->vs, a->v_stride);
    copy3(p->os, a->o_stride);
    copy3(p->dos, a->do_stride);
    copy3(p->dqs, a->dq_stride);
    copy3(p->dks, a->dk_stride);
    copy3(p->dvs, a->dv_stride);
    copy3(p->ms, a->mask_stride);
    copy3(p->dms, a->dmask_stride);
    if (p->dmask != nullptr) {
        // a stride of 0 over a dimension that has more than one entry: the gradient is summed over it
        p->dmask_acc = (a->B > 1 && a->dmask_stride[0] == 0) || (a->H > 1 && a->dmask_stride[1] == 0) ||
                       (a->S > 1 && a->dmask_stride[2] == 0);
        if (p->dmask_acc && a->mask_dtype != TRI_ATTN_F32) return TRI_ATTN_EDTYPE;
    }
    if (a->mask != nullptr && a->S % 128 == 0) {
        // layout of the block classes (64 x 64 blocks), broadcast like the mask itself
        const int64_t cb = a->S / 64, rb = a->mask_stride[2] == 0 ? 1 : cb, mh = a->mask_stride[1] == 0 ? 1 : a->H;
        p->mcs[2] = rb == 1 ? 0 : cb;
        p->mcs[1] = mh == 1 ? 0 : rb * cb;
        p->mcs[0] = a->mask_stride[0] == 0 ? 0 : mh * rb * cb;
        p->mcls = a->mask_classes;
    }
    p->B = a->B;
    p->H = a->H;
    p->S = a->S;
    p->D = a->D;
    p->causal = a->is_causal ? 1 : 0;
    p->mask_dtype = a->mask_dtype;
    p->scale = a->softmax_scale;
    p->scale_log2 = a->softmax_scale * kLog2e;
    p->inv_scale = a->softmax_scale != 0.f ? 1.f / a->softmax_scale : 0.f;
    p->seed_lo = static_cast<uint32_t>(a->seed);
    p->seed_hi = static_cast<uint32_t>(a->seed >> 32);
    p->offset = static_cast<uint32_t>(a->offset);
    int thr = static_cast<int>(rintf(a->dropout_p * 256.f));
    thr = thr < 0 ? 0 : (thr > 256 ? 256 : thr);
    p->thr8 = thr;
    p->zscale = thr >= 256 ? 0.f : 256.f / static_cast<float>(256 - thr);
    return TRI_ATTN_OK;
}

__global__ void dropout_mask_kernel(KParams p, uint32_t bh, int row0, int rows, int col0, int cols, uint8_t* keep) {
    const int64_t n = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (n >= static_cast<int64_t>(rows) * cols) return;
    const int i = row0 + static_cast<int>(n / cols);
    const int j = col0 + static_cast<int>(n % cols);
    keep[n] = dropout_keep(p, bh, i, j) ? 1 : 0;
}

// ---- tri_attn_bwd_noalloc: the backward's delta buffer inside the library
// delta (fp32 [B,H,S]) is the one piece of device memory the backward needs beyond its inputs and outputs: the
// dQ kernel (or the delta pre-pass) writes it, the dK/dV kernel reads it. For callers that cannot allocate it
// lives here, once per GPU, for the life of the process.
constexpr int64_t kScratchRows = TRI_ATTN_NOALLOC_MAX_ROWS;
constexpr int kMaxDevices = 64;
std::atomic<float*> scratch_ptr[kMaxDevices];  // device address of `scratch` on each GPU (the name above is a host-side stand-in)

// Address of this GPU's copy of `scratch`, asked once per device with that device current.
int scratch_for_current_device(float** out) {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return static_cast<int>(e);
    if (dev < 0 || dev >= kMaxDevices) return TRI_ATTN_ESHAPE;
    float* ptr = scratch_ptr[dev].load(std::memory_order_acquire);
    if (ptr == nullptr) {
        e = hipGetSymbolAddress(reinterpret_cast<void**>(&ptr), HIP_SYMBOL(scratch));
        if (e != hipSuccess) return static_cast<int>(e);
        if (ptr == nullptr) return static_cast<int>(hipErrorInvalidSymbol);
        scratch_ptr[dev].store(ptr, std::memory_order_release);
    }
    *out = ptr;
    return TRI_ATTN_OK;
}

}  // namespace
}  // namespace tri

using namespace tri;

extern "C" {

int tri_attn_version(void) { return TRI_ATTN_ABI_VERSION; }

const char* tri_attn_strerror(int status) {
    switch (status) {
        case TRI_ATTN_OK: return "success";
        case TRI_ATTN_ENULL: return "a required pointer is NULL";
        case TRI_ATTN_ESHAPE: return "unsupported shape: B,H,S must be positive and D one of 16, 32, 64, 128";
        case TRI_ATTN_EDTYPE: return "unknown dtype";
        case TRI_ATTN_ESTRIDE: return "innermost stride must be 1 and strides must not be negative";
        case TRI_ATTN_EMASKCAUSAL: return "both mask and is_causal are set";
        case TRI_ATTN_EDROPOUT: return "dropout_p must lie in [0, 1]";
        case TRI_ATTN_ESIZE: return "TriAttnArgs.struct_size does not match this library";
        case TRI_ATTN_EALIGN: return "pointer or stride alignment not supported";
        case TRI_ATTN_ENOFUSE: return "no fused dQ + delta kernel for this problem (nothing launched)";
        case TRI_ATTN_ESCRATCH: return "tri_attn_bwd_noalloc: B*H*S exceeds TRI_ATTN_NOALLOC_MAX_ROWS (nothing launched)";
        default: break;
    }
    if (status > 0) return hipGetErrorString(static_cast<hipError_t>(status));
    return "unknown status";
}

int tri_attn_fwd(const TriAttnArgs* args) {
    KParams p;
    int rc = make_params(args, 1, &p);
    if (rc) return rc;
    hipStream_t st = static_cast<hipStream_t>(args->stream);
    if (mfma_supported(kMfmaFwd, args->dtype, p)) return launch_mfma_fwd(args->dtype, p, st);
    if (mfma32_supported(kMfmaFwd, args->dtype, p)) return launch_mfma32(kMfmaFwd, args->dtype, p, st);
    return launch_generic_any(kGenericFwd, args->dtype, p, st);
}

int tri_attn_bwd_delta(const TriAttnArgs* args) {
    KParams p;
    int rc = make_params(args, 2, &p);
    if (rc) return rc;
    return launch_delta(args->dtype, p, static_cast<hipStream_t>(args->stream));
}

int tri_attn_bwd_dkdv(const TriAttnArgs* args) {
    KParams p;
    int rc = make_params(args, 4, &p);
    if (rc) return rc;
    hipStream_t st = static_cast<hipStream_t>(args->stream);
    if (mfma_supported(kMfmaDkdv, args->dtype, p)) return launch_mfma_dkdv(args->dtype, p, st);
    if (mfma32_supported(kMfmaDkdv, args->dtype, p)) return launch_mfma32(kMfmaDkdv, args->dtype, p, st);
    return launch_generic_any(kGenericDkdv, args->dtype, p, st);
}

int tri_attn_bwd_dq(const TriAttnArgs* args) {
    KParams p;
    int rc = make_params(args, 8, &p);
    if (rc) return rc;
    hipStream_t st = static_cast<hipStream_t>(args->stream);
    if (mfma_supported(kMfmaDq, args->dtype, p)) return launch_mfma_dq(args->dtype, p, st);
    if (mfma32_supported(kMfmaDq, args->dtype, p)) return launch_mfma32(kMfmaDq, args->dtype, p, st);
    return launch_generic_any(kGenericDq, args->dtype, p, st);
}

int tri_attn_bwd_dq_delta(const TriAttnArgs* args) {
    KParams p;
    int rc = make_params(args, 2 | 8, &p);
    if (rc) return rc;
    if (!(mfma_supported(kMfmaDq, args->dtype, p) && mfma_dq_fuses_delta(p))) return TRI_ATTN_ENOFUSE;
    return launch_mfma_dq(args->dtype, p, static_cast<hipStream_t>(args->stream), true);
}

int tri_attn_bwd(const TriAttnArgs* args) {
    // (every argument is checked before the first launch: a call that fails leaves nothing half written)
    {
        KParams all;
        const int bad = make_params(args, 2 | 4 | 8, &all);
        if (bad) return bad;
    }
    // Where the dQ kernel can compute delta on the way (it loads the dO rows anyway), the pre-pass is
    // dropped and dQ runs first: dK/dV reads the delta it stored.
    int rc = tri_attn_bwd_dq_delta(args);
    if (rc == TRI_ATTN_OK) return tri_attn_bwd_dkdv(args);
    if (rc != TRI_ATTN_ENOFUSE) return rc;
    rc = tri_attn_bwd_delta(args);
    if (rc) return rc;
    rc = tri_attn_bwd_dkdv(args);
    if (rc) return rc;
    return tri_attn_bwd_dq(args);
}

int tri_attn_bwd_noalloc(const TriAttnArgs* args) {
    if (args == nullptr) return TRI_ATTN_ENULL;
    if (args->struct_size != sizeof(TriAttnArgs)) return TRI_ATTN_ESIZE;
    if (args->B <= 0 || args->H <= 0 || args->S <= 0) return TRI_ATTN_ESHAPE;
    if (static_cast<int64_t>(args->B) * args->H * args->S > kScratchRows) return TRI_ATTN_ESCRATCH;
    TriAttnArgs a = *args;  // (host copy of a plain struct)
    const int rc = scratch_for_current_device(&a.delta);
    if (rc) return rc;
    // every row of delta that dK/dV reads is written first by this call's dQ kernel or delta pre-pass:
    // nothing of the previous call's contents needs clearing
    return tri_attn_bwd(&a);
}

int64_t tri_attn_mask_classes_size(const TriAttnArgs* args) {
    if (args == nullptr) return TRI_ATTN_ENULL;
    if (args->struct_size != sizeof(TriAttnArgs)) return TRI_ATTN_ESIZE;
    if (args->B <= 0 || args->H <= 0 || args->S <= 0) return TRI_ATTN_ESHAPE;
    if (args->mask == nullptr || args->S % 128 != 0) return 0;
    const int64_t cb = args->S / 64, rb = args->mask_stride[2] == 0 ? 1 : cb;
    return (args->mask_stride[0] == 0 ? 1 : args->B) * (args->mask_stride[1] == 0 ? 1 : args->H) * rb * cb;
}

int tri_attn_classify_mask(const TriAttnArgs* args) {
    if (args == nullptr) return TRI_ATTN_ENULL;
    if (args->struct_size != sizeof(TriAttnArgs)) return TRI_ATTN_ESIZE;
    if (args->B <= 0 || args->H <= 0 || args->S <= 0) return TRI_ATTN_ESHAPE;
    if (args->mask == nullptr || args->mask_classes == nullptr) return TRI_ATTN_ENULL;
    if (args->mask_dtype < TRI_ATTN_F32 || args->mask_dtype > TRI_ATTN_BF16) return TRI_ATTN_EDTYPE;
    int rc = check_strides(args->mask_stride);
    if (rc) return rc;
    if (args->S % 128 != 0) return TRI_ATTN_ENOFUSE;
    KParams p;
    memset(&p, 0, sizeof(p));
    p.mask = args->mask;
    p.mask_dtype = args->mask_dtype;
    copy3(p.ms, args->mask_stride);
    p.B = args->B;
    p.H = args->H;
    p.S = args->S;
    const int64_t cb = args->S / 64, rb = args->mask_stride[2] == 0 ? 1 : cb, mh = args->mask_stride[1] == 0 ? 1 : args->H;
    p.mcs[2] = rb == 1 ? 0 : cb;
    p.mcs[1] = mh == 1 ? 0 : rb * cb;
    p.mcs[0] = args->mask_stride[0] == 0 ? 0 : mh * rb * cb;
    return launch_classify_mask(p, args->mask_classes, static_cast<hipStream_t>(args->stream));
}

int tri_attn_uses_matrix_cores(const TriAttnArgs* args, int pass) {
    if (pass < 0 || pass > 2) return TRI_ATTN_ESHAPE;
    KParams p;
    const int rc = make_params(args, pass == 0 ? 1 : (pass == 1 ? 4 : 8), &p);
    if (rc) return rc;
    const int which = pass == 0 ? kMfmaFwd : (pass == 1 ? kMfmaDkdv : kMfmaDq);
    if (mfma_supported(which, args->dtype, p)) return 1;
    return mfma32_supported(which, args->dtype, p) ? 2 : 0;
}

int tri_attn_dropout_mask(uint64_t seed, uint64_t offset, float dropout_p, uint32_t bh, int32_t row0, int32_t rows,
                          int32_t col0, int32_t cols, uint8_t* keep, void* stream) {
    if (keep == nullptr) return TRI_ATTN_ENULL;
    if (rows <= 0 || cols <= 0 || row0 < 0 || col0 < 0) return TRI_ATTN_ESHAPE;
    if (!(dropout_p >= 0.f && dropout_p <= 1.f)) return TRI_ATTN_EDROPOUT;
    KParams p;
    memset(&p, 0, sizeof(p));
    p.seed_lo = static_cast<uint32_t>(seed);
    p.seed_hi = static_cast<uint32_t>(seed >> 32);
    p.offset = static_cast<uint32_t>(offset);
    int thr = static_cast<int>(rintf(dropout_p * 256.f));
    p.thr8 = thr < 0 ? 0 : (thr > 256 ? 256 : thr);
    const int64_t n = static_cast<int64_t>(rows) * cols;
    hipLaunchKernelGGL(dropout_mask_kernel, dim3(static_cast<unsigned>((n + 255) / 256)), dim3(256), 0,
                       static_cast<hipStream_t>(stream), p, bh, row0, rows, col0, cols, keep);
    return static_cast<int>(hipGetLastError());
}

}  // extern "C"
