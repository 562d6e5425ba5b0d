// Shared device helpers for the attention kernels (gfx950 only).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "tri_attn.h"

namespace tri {

constexpr float kLog2e = 1.4426950408889634f;  // trident/language/constant.py:17-20

typedef _Float16 f16_t;
typedef __bf16 bf16_t;

// Kernel-side view of TriAttnArgs: batch/head/row strides only (innermost stride is 1),
// scale folded into the log2 domain, dropout threshold resolved.
struct KParams {
    const void* q;
    const void* k;
    const void* v;
    void* o;
    float* lse;
    const void* mask;
    const void* d_o;
    void* dq;
    void* dk;
    void* dv;
    void* dmask;
    float* delta;
    const uint8_t* mcls;   // classes of the mask's 64 x 64 blocks or nullptr
    int64_t qs[3], ks[3], vs[3], os[3], dos[3], dqs[3], dks[3], dvs[3], ms[3], dms[3];
    int64_t mcs[3];        // strides of mcls (bytes) over batch, head, row block; the column-block stride is 1
    int B, H, S, D;
    int causal;
    int mask_dtype;
    float scale;       // softmax_scale
    float scale_log2;  // softmax_scale * log2(e)
    float inv_scale;   // 1 / softmax_scale (0 where the scale is 0)
    uint32_t seed_lo, seed_hi, offset;
    int dmask_acc;     // dmask is summed over a broadcast dimension (stride 0): fp32 buffer, atomic adds
    int thr8;          // 0 = no dropout; keep iff u8 >= thr8
    float zscale;      // 256 / (256 - thr8), 0 when thr8 == 256
};

template <typename T>
__device__ __forceinline__ float to_f32(T x) {
    return static_cast<float>(x);
}
template <typename T>
__device__ __forceinline__ T from_f32(float x) {
    return static_cast<T>(x);
}

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ float fast_log2(float x) { return __builtin_amdgcn_logf(x); }

__device__ __forceinline__ float load_mask_elem(const void* base, int dtype, int64_t off) {
    if (dtype == TRI_ATTN_F32) return static_cast<const float*>(base)[off];
    if (dtype == TRI_ATTN_F16) return to_f32(static_cast<const f16_t*>(base)[off]);
    return to_f32(static_cast<const bf16_t*>(base)[off]);
}
__device__ __forceinline__ void store_mask_elem(void* base, int dtype, int64_t off, float x) {
    if (dtype == TRI_ATTN_F32) static_cast<float*>(base)[off] = x;
    else if (dtype == TRI_ATTN_F16) static_cast<f16_t*>(base)[off] = from_f32<f16_t>(x);
    else static_cast<bf16_t*>(base)[off] = from_f32<bf16_t>(x);
}

// Philox4x32-10 (Random123 constants; the generator behind tl.rand used at
// trident/kernel/attention.py:159).
struct Philox4 {
    uint32_t w[4];
};
__device__ __forceinline__ Philox4 philox4x32_10(uint32_t c0, uint32_t c1, uint32_t c2, uint32_t c3,
                                                 uint32_t k0, uint32_t k1) {
#pragma unroll
    for (int r = 0; r < 10; ++r) {
        const uint64_t p0 = static_cast<uint64_t>(0xD2511F53u) * c0;
        const uint64_t p1 = static_cast<uint64_t>(0xCD9E8D57u) * c2;
        const uint32_t n0 = static_cast<uint32_t>(p1 >> 32) ^ c1 ^ k0;
        const uint32_t n2 = static_cast<uint32_t>(p0 >> 32) ^ c3 ^ k1;
        c1 = static_cast<uint32_t>(p1);
        c3 = static_cast<uint32_t>(p0);
        c0 = n0;
        c2 = n2;
        k0 += 0x9E3779B9u;
        k1 += 0xBB67AE85u;
    }
    Philox4 out;
    out.w[0] = c0;
    out.w[1] = c1;
    out.w[2] = c2;
    out.w[3] = c3;
    return out;
}

// The 16 dropout bytes of the 4x4 block (rows 4*ib.., cols 4*jb..) of head bh:
// word r = row within the block, byte c = column within the block.
__device__ __forceinline__ Philox4 dropout_block(const KParams& p, uint32_t bh, uint32_t ib, uint32_t jb) {
    return philox4x32_10(jb, ib, bh, p.offset, p.seed_lo, p.seed_hi);
}
__device__ __forceinline__ bool dropout_keep(const KParams& p, uint32_t bh, uint32_t i, uint32_t j) {
    const Philox4 r = dropout_block(p, bh, i >> 2, j >> 2);
    const uint32_t s = i & 3;
    const uint32_t word = s == 0 ? r.w[0] : (s == 1 ? r.w[1] : (s == 2 ? r.w[2] : r.w[3]));
    const int u8 = static_cast<int>((word >> (8 * (j & 3))) & 0xffu);
    return u8 >= p.thr8;
}

}  // namespace tri
