// Row softmax, masked row softmax and dropout: the HBM-bound sibling operations of the attention path
// (C ABI in include/tri_rowops.h). Statistics are kept in fp32 in the log2 domain, as in the attention kernels.
#include <math.h>
#include <string.h>

#include <type_traits>

#include "common.hpp"
#include "tri_rowops.h"

namespace tri {
namespace {

constexpr float kMaskEps = 2.220446049250313e-16f;  // trident/language/constant.py:17-20 (eps)
constexpr uint32_t kDropoutStream = 0x44524F50u;    // counter word 2 of the stand-alone dropout ("DROP")

struct RowParams {
    const void* input;
    void* output;
    const void* mask;
    const void* grad_output;
    void* grad_input;
    int64_t y_size, x_size, y_stride, x_stride;
    int mask_dtype;
    uint32_t seed_lo, seed_hi, offset;
    int thr8;
    float zscale;
};

// M = element type of the mask (void: no mask). A position is masked where its mask value exceeds eps
// (trident/kernel/masked_softmax.py:76), i.e. is positive for the integer types.
template <typename M>
__device__ __forceinline__ bool mask_hit(const void* base, int64_t off) {
    if constexpr (std::is_same<M, void>::value) return false;
    else if constexpr (std::is_integral<M>::value) return static_cast<const M*>(base)[off] > 0;
    else return to_f32(static_cast<const M*>(base)[off]) > kMaskEps;
}

// (max, sum) pairs of a softmax in the log2 domain and their merge (the reference's language.combine_softmax,
// trident/language/combine.py:30-33); a -inf maximum stands for "nothing seen yet".
struct Stat {
    float m, l;
};
__device__ __forceinline__ float safe(float m) { return m == -INFINITY ? 0.f : m; }
__device__ __forceinline__ Stat merge(Stat a, Stat b) {
    const float m = fmaxf(a.m, b.m), ms = safe(m);
    return Stat{m, a.l * fast_exp2(a.m - ms) + b.l * fast_exp2(b.m - ms)};
}
__device__ __forceinline__ Stat wave_merge(Stat s) {
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) s = merge(s, Stat{__shfl_xor(s.m, d), __shfl_xor(s.l, d)});
    return s;
}
__device__ __forceinline__ float wave_sum(float x) {
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) x += __shfl_xor(x, d);
    return x;
}

template <typename T, int V>
struct alignas(sizeof(T) * V) Vec {
    T e[V];
};

// ------------------------------------------------------------------ rows with unit stride along x
// G threads share a row (a wave for short rows, the whole workgroup for long ones), V elements per load (16 bytes
// when the row geometry allows it). A row of up to G * V * kHeld elements is read once, all loads in flight together,
// and stays in registers between the statistics and the output; a longer row takes two sweeps, the second of which
// finds the row in the L2 it was just read through. Either way the HBM traffic is one read and one write.
constexpr int kHeld = 4;  // 16-byte pieces of a row a thread keeps

template <typename T, int V, int G, typename M>
__global__ __launch_bounds__(256) void softmax_fwd_rows_kernel(const RowParams p) {
    __shared__ Stat part[4];
    constexpr int kRowsPerGroup = 256 / G;
    const int t = threadIdx.x % G;
    const int64_t row = static_cast<int64_t>(blockIdx.x) * kRowsPerGroup + threadIdx.x / G;
    const bool live = row < p.y_size;  // (G == 256: always)
    const int64_t base = (live ? row : 0) * p.y_stride;
    const T* in = static_cast<const T*>(p.input) + base;
    T* out = static_cast<T*>(p.output) + base;
    using VT = Vec<T, V>;
    const bool resident = p.x_size <= static_cast<int64_t>(G) * V * kHeld;
    VT held[kHeld];
    if (live && resident) {
#pragma unroll
        for (int k = 0; k < kHeld; ++k) {
            const int64_t i = (static_cast<int64_t>(k) * G + t) * V;
            if (i < p.x_size) held[k] = *reinterpret_cast<const VT*>(in + i);
        }
    }
    // x[e] in the log2 domain, masked positions at -inf
    auto scores = [&](const VT& v, int64_t i, float (&x)[V]) {
#pragma unroll
        for (int e = 0; e < V; ++e) {
            x[e] = to_f32(v.e[e]) * kLog2e;
            if (mask_hit<M>(p.mask, base + i + e)) x[e] = -INFINITY;
        }
    };
    Stat s{-INFINITY, 0.f};
    auto absorb = [&](const VT& v, int64_t i) {
        float x[V];
        scores(v, i, x);
        float cm = -INFINITY;
#pragma unroll
        for (int e = 0; e < V; ++e) cm = fmaxf(cm, x[e]);
        const float m_new = fmaxf(s.m, cm), ms = safe(m_new);
        float acc = s.l * fast_exp2(s.m - ms);
#pragma unroll
        for (int e = 0; e < V; ++e) acc += fast_exp2(x[e] - ms);
        s = Stat{m_new, acc};
    };
    if (live) {
        if (resident) {
#pragma unroll
            for (int k = 0; k < kHeld; ++k) {
                const int64_t i = (static_cast<int64_t>(k) * G + t) * V;
                if (i < p.x_size) absorb(held[k], i);
            }
        } else {
            for (int64_t i = static_cast<int64_t>(t) * V; i < p.x_size; i += G * V) absorb(*reinterpret_cast<const VT*>(in + i), i);
        }
    }
    s = wave_merge(s);
    if constexpr (G == 256) {
        if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = s;
        __syncthreads();
        s = merge(merge(part[0], part[1]), merge(part[2], part[3]));
    }
    if (!live) return;
    const float ms = safe(s.m), inv = 1.f / s.l;  // a fully masked row: 0 * inf = NaN, as softmax gives
    auto emit = [&](const VT& v, int64_t i) {
        float x[V];
        scores(v, i, x);
        VT o;
#pragma unroll
        for (int e = 0; e < V; ++e) o.e[e] = from_f32<T>(fast_exp2(x[e] - ms) * inv);
        *reinterpret_cast<VT*>(out + i) = o;
    };
    if (resident) {
#pragma unroll
        for (int k = 0; k < kHeld; ++k) {
            const int64_t i = (static_cast<int64_t>(k) * G + t) * V;
            if (i < p.x_size) emit(held[k], i);
        }
    } else {
        for (int64_t i = static_cast<int64_t>(t) * V; i < p.x_size; i += G * V) emit(*reinterpret_cast<const VT*>(in + i), i);
    }
}

template <typename T, int V, int G>
__global__ __launch_bounds__(256) void softmax_bwd_rows_kernel(const RowParams p) {
    __shared__ float part[4];
    constexpr int kRowsPerGroup = 256 / G;
    const int t = threadIdx.x % G;
    const int64_t row = static_cast<int64_t>(blockIdx.x) * kRowsPerGroup + threadIdx.x / G;
    const bool live = row < p.y_size;
    const int64_t base = (live ? row : 0) * p.y_stride;
    const T* o = static_cast<const T*>(p.output) + base;
    const T* g = static_cast<const T*>(p.grad_output) + base;
    T* gi = static_cast<T*>(p.grad_input) + base;
    using VT = Vec<T, V>;
    const bool resident = p.x_size <= static_cast<int64_t>(G) * V * kHeld;
    VT held_o[kHeld], held_g[kHeld];
    if (live && resident) {
#pragma unroll
        for (int k = 0; k < kHeld; ++k) {
            const int64_t i = (static_cast<int64_t>(k) * G + t) * V;
            if (i < p.x_size) {
                held_o[k] = *reinterpret_cast<const VT*>(o + i);
                held_g[k] = *reinterpret_cast<const VT*>(g + i);
            }
        }
    }
    float delta = 0.f;
    auto absorb = [&](const VT& ov, const VT& gv) {
#pragma unroll
        for (int e = 0; e < V; ++e) delta = fmaf(to_f32(ov.e[e]), to_f32(gv.e[e]), delta);
    };
    if (live) {
        if (resident) {
#pragma unroll
            for (int k = 0; k < kHeld; ++k)
                if ((static_cast<int64_t>(k) * G + t) * V < p.x_size) absorb(held_o[k], held_g[k]);
        } else {
            for (int64_t i = static_cast<int64_t>(t) * V; i < p.x_size; i += G * V)
                absorb(*reinterpret_cast<const VT*>(o + i), *reinterpret_cast<const VT*>(g + i));
        }
    }
    delta = wave_sum(delta);
    if constexpr (G == 256) {
        if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = delta;
        __syncthreads();
        delta = (part[0] + part[1]) + (part[2] + part[3]);
    }
    if (!live) return;
    auto emit = [&](const VT& ov, const VT& gv, int64_t i) {
        VT r;
#pragma unroll
        for (int e = 0; e < V; ++e) r.e[e] = from_f32<T>(to_f32(ov.e[e]) * (to_f32(gv.e[e]) - delta));
        *reinterpret_cast<VT*>(gi + i) = r;
    };
    if (resident) {
#pragma unroll
        for (int k = 0; k < kHeld; ++k) {
            const int64_t i = (static_cast<int64_t>(k) * G + t) * V;
            if (i < p.x_size) emit(held_o[k], held_g[k], i);
        }
    } else {
        for (int64_t i = static_cast<int64_t>(t) * V; i < p.x_size; i += G * V)
            emit(*reinterpret_cast<const VT*>(o + i), *reinterpret_cast<const VT*>(g + i), i);
    }
}

// ------------------------------------------------------------------ any strides: one thread per row
// Serves softmax along dim 0 of a row-major matrix (y_stride == 1: neighbouring threads then read neighbouring
// addresses) and every other layout.
template <typename T, typename M>
__global__ __launch_bounds__(256) void softmax_fwd_cols_kernel(const RowParams p) {
    const int64_t row = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
    if (row >= p.y_size) return;
    const int64_t base = row * p.y_stride;
    const T* in = static_cast<const T*>(p.input);
    T* out = static_cast<T*>(p.output);
    Stat s{-INFINITY, 0.f};
    for (int64_t i = 0; i < p.x_size; ++i) {
        const int64_t off = base + i * p.x_stride;
        float x = to_f32(in[off]) * kLog2e;
        if (mask_hit<M>(p.mask, off)) x = -INFINITY;
        s = merge(s, Stat{x, 1.f});
    }
    const float ms = safe(s.m), inv = 1.f / s.l;
    for (int64_t i = 0; i < p.x_size; ++i) {
        const int64_t off = base + i * p.x_stride;
        float x = to_f32(in[off]) * kLog2e;
        if (mask_hit<M>(p.mask, off)) x = -INFINITY;
        out[off] = from_f32<T>(fast_exp2(x - ms) * inv);
    }
}

template <typename T>
__global__ __launch_bounds__(256) void softmax_bwd_cols_kernel(const RowParams p) {
    const int64_t row = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
    if (row >= p.y_size) return;
    const int64_t base = row * p.y_stride;
    const T* o = static_cast<const T*>(p.output);
    const T* g = static_cast<const T*>(p.grad_output);
    T* gi = static_cast<T*>(p.grad_input);
    float delta = 0.f;
    for (int64_t i = 0; i < p.x_size; ++i) delta = fmaf(to_f32(o[base + i * p.x_stride]), to_f32(g[base + i * p.x_stride]), delta);
    for (int64_t i = 0; i < p.x_size; ++i) {
        const int64_t off = base + i * p.x_stride;
        gi[off] = from_f32<T>(to_f32(o[off]) * (to_f32(g[off]) - delta));
    }
}

// ------------------------------------------------------------------ dropout
// A thread makes one Philox call = the 16 decisions of elements 16 t .. 16 t + 15; BACKWARD reads grad_output instead
// of input. A wave's 1024 elements are read and written 16 bytes per lane with consecutive lanes on consecutive
// addresses (whole cache lines per instruction), so a lane's piece belongs to another lane's Philox block: every lane
// leaves its four words in LDS and picks up the words of its pieces from there. Blocks that are ragged or unaligned
// fall back to a thread working through its own 16 elements.
__device__ __forceinline__ uint32_t drop_byte(const Philox4& r, int e) { return (r.w[e >> 2] >> (8 * (e & 3))) & 0xffu; }

template <typename T>
__global__ __launch_bounds__(256) void dropout_kernel(const RowParams p, const T* __restrict__ src, T* __restrict__ dst, int64_t n) {
    __shared__ __attribute__((aligned(16))) uint32_t words[256 * 4];
    const int64_t blk = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
    const int lane = threadIdx.x & 63;
    uint32_t* wave_words = words + (threadIdx.x - lane) * 4;
    const int64_t wave_i0 = (blk - lane) * 16;  // first element of this wave's 1024
    const Philox4 r = philox4x32_10(static_cast<uint32_t>(blk), static_cast<uint32_t>(blk >> 32), kDropoutStream, p.offset,
                                    p.seed_lo, p.seed_hi);
    *reinterpret_cast<uint4*>(wave_words + lane * 4) = uint4{r.w[0], r.w[1], r.w[2], r.w[3]};
    __syncthreads();
    if (wave_i0 >= n) return;
    constexpr int V = 16 / sizeof(T);  // elements of a 16-byte piece
    constexpr int W = V / 4;           // Philox words of a piece
    constexpr int PPB = 16 / V;        // pieces per Philox block
    using VT = Vec<T, V>;
    const bool whole = wave_i0 + 1024 <= n && (reinterpret_cast<uintptr_t>(src) & 15) == 0 && (reinterpret_cast<uintptr_t>(dst) & 15) == 0;
    if (whole) {  // (the same for every lane of the wave)
#pragma unroll
        for (int c = 0; c < PPB; ++c) {
            const int piece = c * 64 + lane;  // of the wave's 64 PPB pieces: words piece * W .. + W - 1 of the wave
            uint32_t w[W];
#pragma unroll
            for (int k = 0; k < W; ++k) w[k] = wave_words[piece * W + k];
            const VT v = *reinterpret_cast<const VT*>(src + wave_i0 + static_cast<int64_t>(piece) * V);
            VT o;
#pragma unroll
            for (int e = 0; e < V; ++e) {
                const bool keep = static_cast<int>((w[e >> 2] >> (8 * (e & 3))) & 0xffu) >= p.thr8;
                o.e[e] = from_f32<T>(keep ? to_f32(v.e[e]) * p.zscale : 0.f);
            }
            *reinterpret_cast<VT*>(dst + wave_i0 + static_cast<int64_t>(piece) * V) = o;
        }
    } else {
        const int64_t i0 = blk * 16;
        for (int e = 0; e < 16 && i0 + e < n; ++e) {
            const bool keep = static_cast<int>(drop_byte(r, e)) >= p.thr8;
            dst[i0 + e] = from_f32<T>(keep ? to_f32(src[i0 + e]) * p.zscale : 0.f);
        }
    }
}

// ------------------------------------------------------------------ host side
int make_row_params(const TriRowArgs* a, bool backward, bool dropout, RowParams* p) {
    if (a == nullptr) return TRI_ATTN_ENULL;
    if (a->struct_size != sizeof(TriRowArgs)) return TRI_ATTN_ESIZE;
    if (a->dtype < TRI_ATTN_F32 || a->dtype > TRI_ATTN_BF16) return TRI_ATTN_EDTYPE;
    if (a->y_size <= 0 || a->x_size <= 0) return TRI_ATTN_ESHAPE;
    if (!dropout && (a->y_stride < 0 || a->x_stride < 0)) return TRI_ATTN_ESTRIDE;
    if (a->mask != nullptr && (a->mask_dtype < TRI_ATTN_F32 || a->mask_dtype > TRI_ROW_MASK_U8)) return TRI_ATTN_EDTYPE;
    if (dropout && !(a->p >= 0.f && a->p <= 1.f)) return TRI_ATTN_EDROPOUT;
    if (backward) {
        if (!a->grad_output || !a->grad_input || (!dropout && !a->output)) return TRI_ATTN_ENULL;
    } else if (!a->input || !a->output) {
        return TRI_ATTN_ENULL;
    }
    memset(p, 0, sizeof(*p));
    p->input = a->input;
    p->output = a->output;
    p->mask = a->mask;
    p->grad_output = a->grad_output;
    p->grad_input = a->grad_input;
    p->y_size = a->y_size;
    p->x_size = a->x_size;
    p->y_stride = a->y_stride;
    p->x_stride = a->x_stride;
    p->mask_dtype = a->mask_dtype;
    p->seed_lo = static_cast<uint32_t>(a->seed);
    p->seed_hi = static_cast<uint32_t>(a->seed >> 32);
    p->offset = static_cast<uint32_t>(a->offset);
    int thr = static_cast<int>(rintf(a->p * 256.f));
    thr = thr < 0 ? 0 : (thr > 256 ? 256 : thr);
    p->thr8 = thr;
    p->zscale = thr >= 256 ? 0.f : 256.f / static_cast<float>(256 - thr);
    return TRI_ATTN_OK;
}

bool aligned16(const void* ptr) { return ptr == nullptr || (reinterpret_cast<uintptr_t>(ptr) & 15) == 0; }

template <typename T, typename M>
int launch_softmax_fwd(const RowParams& p, hipStream_t st) {
    constexpr int kV = 16 / sizeof(T);
    const dim3 block(256);
    if (p.x_stride != 1 && p.x_size != 1) {
        hipLaunchKernelGGL((softmax_fwd_cols_kernel<T, M>), dim3(static_cast<unsigned>((p.y_size + 255) / 256)), block, 0, st, p);
        return static_cast<int>(hipGetLastError());
    }
    // 16-byte accesses when every row starts on a 16-byte boundary and holds whole vectors
    const bool vec = p.x_size % kV == 0 && p.y_stride % kV == 0 && aligned16(p.input) && aligned16(p.output);
    const bool wide = p.x_size > 2048;  // the whole workgroup on one row, else a wave per row
    const dim3 grid(static_cast<unsigned>(wide ? p.y_size : (p.y_size + 3) / 4));
    if (vec && wide) hipLaunchKernelGGL((softmax_fwd_rows_kernel<T, kV, 256, M>), grid, block, 0, st, p);
    else if (vec) hipLaunchKernelGGL((softmax_fwd_rows_kernel<T, kV, 64, M>), grid, block, 0, st, p);
    else if (wide) hipLaunchKernelGGL((softmax_fwd_rows_kernel<T, 1, 256, M>), grid, block, 0, st, p);
    else hipLaunchKernelGGL((softmax_fwd_rows_kernel<T, 1, 64, M>), grid, block, 0, st, p);
    return static_cast<int>(hipGetLastError());
}

template <typename T>
int launch_softmax_bwd(const RowParams& p, hipStream_t st) {
    constexpr int kV = 16 / sizeof(T);
    const dim3 block(256);
    if (p.x_stride != 1 && p.x_size != 1) {
        hipLaunchKernelGGL((softmax_bwd_cols_kernel<T>), dim3(static_cast<unsigned>((p.y_size + 255) / 256)), block, 0, st, p);
        return static_cast<int>(hipGetLastError());
    }
    const bool vec = p.x_size % kV == 0 && p.y_stride % kV == 0 && aligned16(p.output) && aligned16(p.grad_output) && aligned16(p.grad_input);
    const bool wide = p.x_size > 2048;
    const dim3 grid(static_cast<unsigned>(wide ? p.y_size : (p.y_size + 3) / 4));
    if (vec && wide) hipLaunchKernelGGL((softmax_bwd_rows_kernel<T, kV, 256>), grid, block, 0, st, p);
    else if (vec) hipLaunchKernelGGL((softmax_bwd_rows_kernel<T, kV, 64>), grid, block, 0, st, p);
    else if (wide) hipLaunchKernelGGL((softmax_bwd_rows_kernel<T, 1, 256>), grid, block, 0, st, p);
    else hipLaunchKernelGGL((softmax_bwd_rows_kernel<T, 1, 64>), grid, block, 0, st, p);
    return static_cast<int>(hipGetLastError());
}

template <typename T>
int launch_softmax(const RowParams& p, bool backward, hipStream_t st) {
    if (p.y_size > 2147483647LL) return TRI_ATTN_ESHAPE;
    if (backward) return launch_softmax_bwd<T>(p, st);
    if (p.mask == nullptr) return launch_softmax_fwd<T, void>(p, st);
    switch (p.mask_dtype) {
        case TRI_ATTN_F32: return launch_softmax_fwd<T, float>(p, st);
        case TRI_ATTN_F16: return launch_softmax_fwd<T, f16_t>(p, st);
        case TRI_ATTN_BF16: return launch_softmax_fwd<T, bf16_t>(p, st);
        case TRI_ROW_MASK_I64: return launch_softmax_fwd<T, int64_t>(p, st);
        case TRI_ROW_MASK_I32: return launch_softmax_fwd<T, int32_t>(p, st);
        default: return launch_softmax_fwd<T, uint8_t>(p, st);
    }
}

int launch_softmax_any(int dtype, const RowParams& p, bool backward, hipStream_t st) {
    switch (dtype) {
        case TRI_ATTN_F32: return launch_softmax<float>(p, backward, st);
        case TRI_ATTN_F16: return launch_softmax<f16_t>(p, backward, st);
        default: return launch_softmax<bf16_t>(p, backward, st);
    }
}

template <typename T>
int launch_dropout(const RowParams& p, bool backward, hipStream_t st) {
    const int64_t n = p.y_size * p.x_size;
    const int64_t threads = (n + 15) / 16, groups = (threads + 255) / 256;
    if (groups > 2147483647LL) return TRI_ATTN_ESHAPE;
    const T* src = static_cast<const T*>(backward ? p.grad_output : p.input);
    T* dst = static_cast<T*>(backward ? p.grad_input : p.output);
    hipLaunchKernelGGL((dropout_kernel<T>), dim3(static_cast<unsigned>(groups)), dim3(256), 0, st, p, src, dst, n);
    return static_cast<int>(hipGetLastError());
}

int launch_dropout_any(int dtype, const RowParams& p, bool backward, hipStream_t st) {
    switch (dtype) {
        case TRI_ATTN_F32: return launch_dropout<float>(p, backward, st);
        case TRI_ATTN_F16: return launch_dropout<f16_t>(p, backward, st);
        default: return launch_dropout<bf16_t>(p, backward, st);
    }
}

}  // namespace
}  // namespace tri

using namespace tri;

extern "C" {

int tri_softmax_fwd(const TriRowArgs* args) {
    RowParams p;
    const int rc = make_row_params(args, false, false, &p);
    if (rc) return rc;
    return launch_softmax_any(args->dtype, p, false, static_cast<hipStream_t>(args->stream));
}

int tri_softmax_bwd(const TriRowArgs* args) {
    RowParams p;
    const int rc = make_row_params(args, true, false, &p);
    if (rc) return rc;
    p.mask = nullptr;  // masked positions have output 0: the gradient needs no mask
    return launch_softmax_any(args->dtype, p, true, static_cast<hipStream_t>(args->stream));
}

int tri_dropout_fwd(const TriRowArgs* args) {
    RowParams p;
    const int rc = make_row_params(args, false, true, &p);
    if (rc) return rc;
    return launch_dropout_any(args->dtype, p, false, static_cast<hipStream_t>(args->stream));
}

int tri_dropout_bwd(const TriRowArgs* args) {
    RowParams p;
    const int rc = make_row_params(args, true, true, &p);
    if (rc) return rc;
    return launch_dropout_any(args->dtype, p, true, static_cast<hipStream_t>(args->stream));
}

}  // extern "C"
