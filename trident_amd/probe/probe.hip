// Calibration kernels (libtri_probe.so, include/tri_probe.h; not part of the operator's library): what the matrix pipe
// of this GPU sustains on random operands, alone and with its A operands streamed from LDS. They have no counterpart in
// the reference; bench.py --ceiling times them next
// to a large bf16 GEMM and the attention kernels, so that an attention kernel's distance from the published
// MFMA peak can be split into "cycles not spent in MFMAs" and "clock below 2.4 GHz under this load".
#include "mfma_common.hpp"
#include "tri_probe.h"

namespace tri {
namespace {

constexpr int kProbeThreads = 512;      // 8 waves per workgroup, two per SIMD
constexpr int kProbeLdsBytes = 128 * 1024;  // a wave's reads of one loop trip span 64 KiB from a base that moves per trip

// MODE 0: operands in registers (8 A and 8 B fragments per wave, all pairings over 8 loop trips)
// MODE 1: every MFMA takes its A fragment from LDS (one ds_read_b128 per MFMA, as the attention kernels do)
// MODE 2: every A fragment read from LDS feeds two MFMAs (two B fragments, two accumulators)
// MODE 3: the fp32 instruction (v_mfma_f32_32x32x2_f32), operands in registers: 64 steps of 4096 flops per loop trip
template <int MODE>
__global__ __launch_bounds__(kProbeThreads) void probe_kernel(const u32x4* __restrict__ operands, float* out, int iters) {
    __shared__ __attribute__((aligned(1024))) char smem[MODE == 0 || MODE == 3 ? 16 : kProbeLdsBytes];
    const int tid = threadIdx.x, lane = tid & 63;
    u32x4 a[8], b[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        a[i] = operands[i * kProbeThreads + tid];
        b[i] = operands[(8 + i) * kProbeThreads + tid];
    }
    if constexpr (MODE == 1 || MODE == 2) {
        for (int i = tid; i < kProbeLdsBytes / 16; i += kProbeThreads)
            *reinterpret_cast<u32x4*>(smem + i * 16) = operands[i % (16 * kProbeThreads)];
        __syncthreads();
    }
    f32x16 c[4] = {zero16(), zero16(), zero16(), zero16()};
    // the LDS modes keep a ring of 8 fragments in flight across loop trips (the base moves per trip, so no read
    // can be hoisted out of the loop)
    auto base_of = [&](int it) { return smem + (((it + (tid >> 6) * 8) & 63) << 10) + lane * 16; };
    u32x4 ring[8];
    if constexpr (MODE == 1 || MODE == 2) {
#pragma unroll
        for (int r = 0; r < 8; ++r) ring[r] = lds_read16(base_of(0), r * 1024);
    }
    for (int it = 0; it < iters; ++it) {
        if constexpr (MODE == 0) {
#pragma unroll
            for (int r = 0; r < 8; ++r)
#pragma unroll
                for (int j = 0; j < 8; ++j) c[j & 3] = Mma<bf16_t>::run(a[j], b[(j + r) & 7], c[j & 3]);
        } else if constexpr (MODE == 3) {
            // (a pair of bf16 values read as one fp32 number: the upper one with some more mantissa bits)
#pragma unroll
            for (int r = 0; r < 8; ++r)
#pragma unroll
                for (int j = 0; j < 8; ++j)
                    c[j & 3] = __builtin_amdgcn_mfma_f32_32x32x2f32(__builtin_bit_cast(float, a[j].x),
                                                                     __builtin_bit_cast(float, b[(j + r) & 7].x), c[j & 3], 0, 0, 0);
        } else {
            constexpr int kReads = MODE == 1 ? 64 : 32;
            const char* base = base_of(it);
            const char* next = base_of(it + 1);
#pragma unroll
            for (int j = 0; j < kReads; ++j) {
                const u32x4 f = ring[j & 7];
                if constexpr (MODE == 1) {
                    c[j & 3] = Mma<bf16_t>::run(f, b[j & 7], c[j & 3]);
                } else {
                    c[(2 * j) & 3] = Mma<bf16_t>::run(f, b[j & 7], c[(2 * j) & 3]);
                    c[(2 * j + 1) & 3] = Mma<bf16_t>::run(f, b[(j + 3) & 7], c[(2 * j + 1) & 3]);
                }
                ring[j & 7] = j + 8 < kReads ? lds_read16(base, (j + 8) * 1024) : lds_read16(next, (j + 8 - kReads) * 1024);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
    }
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < 16; ++i) s += (c[0][i] + c[1][i]) + (c[2][i] + c[3][i]);
    out[static_cast<int64_t>(blockIdx.x) * kProbeThreads + tid] = s;
}

// Do vector-ALU instructions of one wave run in the shadow of another wave's MFMAs on the same SIMD? Waves 0-3 of a
// workgroup (one per SIMD) run MFMAs (MATRIX 0: v_mfma_f32_32x32x16_bf16, 1: v_mfma_f32_32x32x2_f32; 16 per loop trip
// on 4 accumulators), waves 4-7 run vector work on 32 independent values per lane (VALU 0: one fma each; 1: one exp2 each;
// 2: fma, max, exp2 each - a softmax's mix). `who` selects which group works: 1 matrix only, 2 vector only, 3 both; 4 = waves 0-3 do both kinds of work themselves (two values'
// vector work after each matrix step) and waves 4-7 nothing.
template <int MATRIX, int VALU>
__global__ __launch_bounds__(kProbeThreads) void coexec_kernel(const u32x4* __restrict__ operands, float* out, int iters, int who) {
    const int tid = threadIdx.x, group = tid >> 8;
    float acc = 0.f;
    if (who != 4 && (who & 1) && group == 0) {
        f32x16 c[4] = {zero16(), zero16(), zero16(), zero16()};
        const u32x4 a = operands[tid], b = operands[kProbeThreads + tid];
        for (int it = 0; it < iters; ++it) {
#pragma unroll
            for (int j = 0; j < 16; ++j) {
                if constexpr (MATRIX == 0) c[j & 3] = Mma<bf16_t>::run(a, b, c[j & 3]);
                else c[j & 3] = __builtin_amdgcn_mfma_f32_32x32x2f32(__builtin_bit_cast(float, a.x), __builtin_bit_cast(float, b.x), c[j & 3], 0, 0, 0);
            }
        }
#pragma unroll
        for (int i = 0; i < 16; ++i) acc += (c[0][i] + c[1][i]) + (c[2][i] + c[3][i]);
    }
    if (who == 4 && group == 0) {  // both kinds of work in the SAME wave: each matrix step followed by two values' vector work
        f32x16 c[4] = {zero16(), zero16(), zero16(), zero16()};
        const u32x4 a = operands[tid], b = operands[kProbeThreads + tid];
        float x[32];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const u32x4 v = operands[2 * kProbeThreads + i * kProbeThreads + tid];
            x[4 * i + 0] = __builtin_bit_cast(float, v.x) * 1e-3f;
            x[4 * i + 1] = __builtin_bit_cast(float, v.y) * 1e-3f;
            x[4 * i + 2] = __builtin_bit_cast(float, v.z) * 1e-3f;
            x[4 * i + 3] = __builtin_bit_cast(float, v.w) * 1e-3f;
        }
        for (int it = 0; it < iters; ++it) {
#pragma unroll
            for (int j = 0; j < 16; ++j) {
                if constexpr (MATRIX == 0) c[j & 3] = Mma<bf16_t>::run(a, b, c[j & 3]);
                else c[j & 3] = __builtin_amdgcn_mfma_f32_32x32x2f32(__builtin_bit_cast(float, a.x), __builtin_bit_cast(float, b.x), c[j & 3], 0, 0, 0);
#pragma unroll
                for (int i = 2 * j; i < 2 * j + 2; ++i) {
                    if constexpr (VALU == 0) x[i] = fmaf(x[i], 0.999f, 0.001f);
                    else if constexpr (VALU == 1) x[i] = fast_exp2(x[i] * 0.5f);
                    else x[i] = fast_exp2(fmaxf(fmaf(x[i], 0.999f, 0.001f), 0.25f) - 1.f);
                }
            }
        }
#pragma unroll
        for (int i = 0; i < 16; ++i) acc += (c[0][i] + c[1][i]) + (c[2][i] + c[3][i]);
#pragma unroll
        for (int i = 0; i < 32; ++i) acc += x[i];
    }
    if (who != 4 && (who & 2) && group == 1) {
        float x[32];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const u32x4 v = operands[2 * kProbeThreads + i * kProbeThreads + tid];
            x[4 * i + 0] = __builtin_bit_cast(float, v.x) * 1e-3f;
            x[4 * i + 1] = __builtin_bit_cast(float, v.y) * 1e-3f;
            x[4 * i + 2] = __builtin_bit_cast(float, v.z) * 1e-3f;
            x[4 * i + 3] = __builtin_bit_cast(float, v.w) * 1e-3f;
        }
        for (int it = 0; it < iters; ++it) {
#pragma unroll
            for (int i = 0; i < 32; ++i) {
                if constexpr (VALU == 0) x[i] = fmaf(x[i], 0.999f, 0.001f);
                else if constexpr (VALU == 1) x[i] = fast_exp2(x[i] * 0.5f);
                else x[i] = fast_exp2(fmaxf(fmaf(x[i], 0.999f, 0.001f), 0.25f) - 1.f);
            }
        }
#pragma unroll
        for (int i = 0; i < 32; ++i) acc += x[i];
    }
    out[static_cast<int64_t>(blockIdx.x) * kProbeThreads + tid] = acc;
}

}  // namespace
}  // namespace tri

using namespace tri;

extern "C" int tri_probe_coexec(int matrix, int valu, int who, int workgroups, int iters, const void* operands,
                                     float* out, void* stream) {
    if (operands == nullptr || out == nullptr) return TRI_ATTN_ENULL;
    if (workgroups <= 0 || iters <= 0 || matrix < 0 || matrix > 1 || valu < 0 || valu > 2 || who < 1 || who > 4) return TRI_ATTN_ESHAPE;
    const dim3 grid(workgroups), block(kProbeThreads);
    hipStream_t st = static_cast<hipStream_t>(stream);
    const u32x4* ops = static_cast<const u32x4*>(operands);
    auto launch = [&](auto kern) { hipLaunchKernelGGL(kern, grid, block, 0, st, ops, out, iters, who); };
    if (matrix == 0 && valu == 0) launch(coexec_kernel<0, 0>);
    else if (matrix == 0 && valu == 1) launch(coexec_kernel<0, 1>);
    else if (matrix == 0) launch(coexec_kernel<0, 2>);
    else if (valu == 0) launch(coexec_kernel<1, 0>);
    else if (valu == 1) launch(coexec_kernel<1, 1>);
    else launch(coexec_kernel<1, 2>);
    return static_cast<int>(hipGetLastError());
}

extern "C" int tri_probe_mfma(int mode, int workgroups, int iters, const void* operands, float* out, void* stream) {
    if (operands == nullptr || out == nullptr) return TRI_ATTN_ENULL;
    if (workgroups <= 0 || iters <= 0 || mode < 0 || mode > 3) return TRI_ATTN_ESHAPE;
    const dim3 grid(workgroups), block(kProbeThreads);
    hipStream_t st = static_cast<hipStream_t>(stream);
    const u32x4* ops = static_cast<const u32x4*>(operands);
    if (mode == 0) hipLaunchKernelGGL(probe_kernel<0>, grid, block, 0, st, ops, out, iters);
    else if (mode == 1) hipLaunchKernelGGL(probe_kernel<1>, grid, block, 0, st, ops, out, iters);
    else if (mode == 2) hipLaunchKernelGGL(probe_kernel<2>, grid, block, 0, st, ops, out, iters);
    else hipLaunchKernelGGL(probe_kernel<3>, grid, block, 0, st, ops, out, iters);
    return static_cast<int>(hipGetLastError());
}
