// Shape-generic attention kernels: any S >= 1, D in {16,32,64,128}, fp32/fp16/bf16 storage,
// fp32 arithmetic on the vector ALU, element-wise loads and stores. They take what neither matrix-core family
// does: views whose rows are not aligned to four elements (mfma32.hip serves every aligned problem the
// 16-bit MFMA kernels leave, fp32 inputs among them), and the delta pre-pass of such problems.
//
// Work split: a workgroup of 256 threads owns 64 rows (query rows for forward and dQ, key
// rows for dK/dV); each row is shared by 4 adjacent lanes that each hold D/4 of the head
// dimension, interleaved in 16-byte chunks so that LDS reads of the four lanes fall into
// different banks. The other operand streams through LDS in fp32 tiles of 32 rows.
#include "common.hpp"
#include "launch.hpp"

namespace tri {
namespace {

constexpr int kRows = 64;   // rows per workgroup
constexpr int kTile = 32;   // streamed rows per LDS tile

template <int D>
struct Slice {
    static constexpr int DP = D / 4;  // elements per lane
    // local element e -> head-dim index
    __device__ static __forceinline__ int dim(int part, int e) { return ((part + 4 * (e >> 2)) << 2) + (e & 3); }
};

template <typename T, int D>
__device__ __forceinline__ void load_slice(const T* row, int part, float (&dst)[D / 4]) {
#pragma unroll
    for (int e = 0; e < D / 4; ++e) dst[e] = to_f32(row[Slice<D>::dim(part, e)]);
}

template <int D>
__device__ __forceinline__ float dot_slice(const float (&a)[D / 4], const float* lds_row, int part) {
    float acc = 0.f;
#pragma unroll
    for (int m = 0; m < D / 16; ++m) {
        const float4 kv = reinterpret_cast<const float4*>(lds_row)[part + 4 * m];
        acc = fmaf(a[4 * m + 0], kv.x, acc);
        acc = fmaf(a[4 * m + 1], kv.y, acc);
        acc = fmaf(a[4 * m + 2], kv.z, acc);
        acc = fmaf(a[4 * m + 3], kv.w, acc);
    }
    return acc;
}

template <int D>
__device__ __forceinline__ void axpy_slice(float (&acc)[D / 4], float w, const float* lds_row, int part) {
#pragma unroll
    for (int m = 0; m < D / 16; ++m) {
        const float4 vv = reinterpret_cast<const float4*>(lds_row)[part + 4 * m];
        acc[4 * m + 0] = fmaf(w, vv.x, acc[4 * m + 0]);
        acc[4 * m + 1] = fmaf(w, vv.y, acc[4 * m + 1]);
        acc[4 * m + 2] = fmaf(w, vv.z, acc[4 * m + 2]);
        acc[4 * m + 3] = fmaf(w, vv.w, acc[4 * m + 3]);
    }
}

__device__ __forceinline__ float quad_sum(float x) {
    x += __shfl_xor(x, 1);
    x += __shfl_xor(x, 2);
    return x;
}

// Cooperative load of `kTile` rows [row0, row0+kTile) of a [S][D] matrix into fp32 LDS; rows
// past S are zero filled.
template <typename T, int D>
__device__ __forceinline__ void stage_tile(const T* base, int64_t row_stride, int row0, int S, float* dst) {
    for (int idx = threadIdx.x; idx < kTile * D; idx += 256) {
        const int r = idx / D, d = idx % D;
        const int row = row0 + r;
        dst[idx] = row < S ? to_f32(base[row * row_stride + d]) : 0.f;
    }
}

template <typename T, int D>
__global__ __launch_bounds__(256) void generic_fwd_kernel(const KParams p) {
    constexpr int DP = D / 4;
    __shared__ __attribute__((aligned(16))) float sK[kTile * D];
    __shared__ __attribute__((aligned(16))) float sV[kTile * D];

    const int part = threadIdx.x & 3;
    const int r = threadIdx.x >> 2;
    // one workgroup per (head, 64-row tile), head-major in grid.x (grid.y stops at 65 535)
    const int tiles = (p.S + kRows - 1) / kRows;
    const int bh = blockIdx.x / tiles;
    const int b = bh / p.H, h = bh % p.H;
    const int row0 = (blockIdx.x % tiles) * kRows;
    const int row = row0 + r;
    const bool row_ok = row < p.S;
    const int row_c = row_ok ? row : p.S - 1;

    const T* qrow = static_cast<const T*>(p.q) + b * p.qs[0] + h * p.qs[1] + row_c * p.qs[2];
    const T* kbase = static_cast<const T*>(p.k) + b * p.ks[0] + h * p.ks[1];
    const T* vbase = static_cast<const T*>(p.v) + b * p.vs[0] + h * p.vs[1];
    const int64_t mrow = p.mask ? b * p.ms[0] + h * p.ms[1] + row_c * p.ms[2] : 0;

    float q[DP], o[DP];
    load_slice<T, D>(qrow, part, q);
#pragma unroll
    for (int e = 0; e < DP; ++e) o[e] = 0.f;
    float m = -INFINITY, l = 0.f;

    const int n_end = p.causal ? min(p.S, row0 + kRows) : p.S;
    for (int t0 = 0; t0 < n_end; t0 += kTile) {
        __syncthreads();
        stage_tile<T, D>(kbase, p.ks[2], t0, p.S, sK);
        stage_tile<T, D>(vbase, p.vs[2], t0, p.S, sV);
        __syncthreads();
#pragma unroll 1
        for (int kb = 0; kb < kTile; kb += 8) {
            float s[8];
            float mx = -INFINITY;
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                const int j = t0 + kb + u;
                float x = quad_sum(dot_slice<D>(q, sK + (kb + u) * D, part)) * p.scale_log2;
                if (p.mask && j < p.S) x = fmaf(load_mask_elem(p.mask, p.mask_dtype, mrow + j), kLog2e, x);
                const bool visible = j < p.S && (!p.causal || j <= row);
                s[u] = visible ? x : -INFINITY;
                mx = fmaxf(mx, s[u]);
            }
            const float m_new = fmaxf(m, mx);
            const float m_use = m_new == -INFINITY ? 0.f : m_new;
            const float alpha = fast_exp2(m - m_use);
            l *= alpha;
#pragma unroll
            for (int e = 0; e < DP; ++e) o[e] *= alpha;
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                float pr = fast_exp2(s[u] - m_use);
                l += pr;
                if (p.thr8 > 0) {
                    const int j = t0 + kb + u;
                    pr = dropout_keep(p, bh, row, j) ? pr * p.zscale : 0.f;
                }
                axpy_slice<D>(o, pr, sV + (kb + u) * D, part);
            }
            m = m_new;
        }
    }
    if (!row_ok) return;
    const float inv = 1.f / l;
    T* orow = static_cast<T*>(p.o) + b * p.os[0] + h * p.os[1] + row * p.os[2];
#pragma unroll
    for (int e = 0; e < DP; ++e) orow[Slice<D>::dim(part, e)] = from_f32<T>(o[e] * inv);
    if (part == 0) p.lse[(static_cast<int64_t>(bh)) * p.S + row] = m + fast_log2(l);
}

// dQ (and dMask): a workgroup owns 64 query rows and streams all visible keys.
template <typename T, int D>
__global__ __launch_bounds__(256) void generic_dq_kernel(const KParams p) {
    constexpr int DP = D / 4;
    __shared__ __attribute__((aligned(16))) float sK[kTile * D];
    __shared__ __attribute__((aligned(16))) float sV[kTile * D];

    const int part = threadIdx.x & 3;
    const int r = threadIdx.x >> 2;
    // one workgroup per (head, 64-row tile), head-major in grid.x (grid.y stops at 65 535)
    const int tiles = (p.S + kRows - 1) / kRows;
    const int bh = blockIdx.x / tiles;
    const int b = bh / p.H, h = bh % p.H;
    const int row0 = (blockIdx.x % tiles) * kRows;
    const int row = row0 + r;
    const bool row_ok = row < p.S;
    const int row_c = row_ok ? row : p.S - 1;

    const T* qrow = static_cast<const T*>(p.q) + b * p.qs[0] + h * p.qs[1] + row_c * p.qs[2];
    const T* dorow = static_cast<const T*>(p.d_o) + b * p.dos[0] + h * p.dos[1] + row_c * p.dos[2];
    const T* kbase = static_cast<const T*>(p.k) + b * p.ks[0] + h * p.ks[1];
    const T* vbase = static_cast<const T*>(p.v) + b * p.vs[0] + h * p.vs[1];
    const int64_t mrow = p.mask ? b * p.ms[0] + h * p.ms[1] + row_c * p.ms[2] : 0;
    const int64_t dmrow = p.dmask ? b * p.dms[0] + h * p.dms[1] + row_c * p.dms[2] : 0;

    float q[DP], g[DP], acc[DP];
    load_slice<T, D>(qrow, part, q);
    load_slice<T, D>(dorow, part, g);
#pragma unroll
    for (int e = 0; e < DP; ++e) acc[e] = 0.f;
    const float lse = p.lse[static_cast<int64_t>(bh) * p.S + row_c];
    const float dlt = p.delta[static_cast<int64_t>(bh) * p.S + row_c];

    const int n_end = p.causal ? min(p.S, row0 + kRows) : p.S;
    for (int t0 = 0; t0 < n_end; t0 += kTile) {
        __syncthreads();
        stage_tile<T, D>(kbase, p.ks[2], t0, p.S, sK);
        stage_tile<T, D>(vbase, p.vs[2], t0, p.S, sV);
        __syncthreads();
#pragma unroll 2
        for (int u = 0; u < kTile; ++u) {
            const int j = t0 + u;
            float x = quad_sum(dot_slice<D>(q, sK + u * D, part)) * p.scale_log2;
            float dp = quad_sum(dot_slice<D>(g, sV + u * D, part));
            if (p.mask && j < p.S) x = fmaf(load_mask_elem(p.mask, p.mask_dtype, mrow + j), kLog2e, x);
            const bool visible = j < p.S && (!p.causal || j <= row);
            const float pr = visible ? fast_exp2(x - lse) : 0.f;
            if (p.thr8 > 0) dp = dropout_keep(p, bh, row, j) ? dp * p.zscale : 0.f;
            const float ds = pr * (dp - dlt);
            axpy_slice<D>(acc, ds, sK + u * D, part);
            if (p.dmask && row_ok && j < p.S && part == (u & 3)) {
                if (p.dmask_acc) unsafeAtomicAdd(static_cast<float*>(p.dmask) + dmrow + j, ds);
                else store_mask_elem(p.dmask, p.mask_dtype, dmrow + j, ds);
            }
        }
    }
    if (!row_ok) return;
    T* dqrow = static_cast<T*>(p.dq) + b * p.dqs[0] + h * p.dqs[1] + row * p.dqs[2];
#pragma unroll
    for (int e = 0; e < DP; ++e) dqrow[Slice<D>::dim(part, e)] = from_f32<T>(acc[e] * p.scale);
}

// dK and dV: a workgroup owns 64 key rows and streams the query rows that can see them.
template <typename T, int D>
__global__ __launch_bounds__(256) void generic_dkdv_kernel(const KParams p) {
    constexpr int DP = D / 4;
    __shared__ __attribute__((aligned(16))) float sQ[kTile * D];
    __shared__ __attribute__((aligned(16))) float sG[kTile * D];
    __shared__ float sLse[kTile];
    __shared__ float sDelta[kTile];

    const int part = threadIdx.x & 3;
    const int r = threadIdx.x >> 2;
    // one workgroup per (head, 64-row tile), head-major in grid.x (grid.y stops at 65 535)
    const int tiles = (p.S + kRows - 1) / kRows;
    const int bh = blockIdx.x / tiles;
    const int b = bh / p.H, h = bh % p.H;
    const int col0 = (blockIdx.x % tiles) * kRows;
    const int col = col0 + r;
    const bool col_ok = col < p.S;
    const int col_c = col_ok ? col : p.S - 1;

    const T* krow = static_cast<const T*>(p.k) + b * p.ks[0] + h * p.ks[1] + col_c * p.ks[2];
    const T* vrow = static_cast<const T*>(p.v) + b * p.vs[0] + h * p.vs[1] + col_c * p.vs[2];
    const T* qbase = static_cast<const T*>(p.q) + b * p.qs[0] + h * p.qs[1];
    const T* gbase = static_cast<const T*>(p.d_o) + b * p.dos[0] + h * p.dos[1];
    const int64_t mbase = p.mask ? b * p.ms[0] + h * p.ms[1] + col_c : 0;

    float k[DP], v[DP], dk[DP], dv[DP];
    load_slice<T, D>(krow, part, k);
    load_slice<T, D>(vrow, part, v);
#pragma unroll
    for (int e = 0; e < DP; ++e) dk[e] = dv[e] = 0.f;

    const int i_begin = p.causal ? (col0 / kTile) * kTile : 0;
    for (int t0 = i_begin; t0 < p.S; t0 += kTile) {
        __syncthreads();
        stage_tile<T, D>(qbase, p.qs[2], t0, p.S, sQ);
        stage_tile<T, D>(gbase, p.dos[2], t0, p.S, sG);
        if (threadIdx.x < kTile) {
            const int i = t0 + threadIdx.x;
            sLse[threadIdx.x] = i < p.S ? p.lse[static_cast<int64_t>(bh) * p.S + i] : 0.f;
            sDelta[threadIdx.x] = i < p.S ? p.delta[static_cast<int64_t>(bh) * p.S + i] : 0.f;
        }
        __syncthreads();
#pragma unroll 2
        for (int u = 0; u < kTile; ++u) {
            const int i = t0 + u;
            float x = quad_sum(dot_slice<D>(k, sQ + u * D, part)) * p.scale_log2;
            float dp = quad_sum(dot_slice<D>(v, sG + u * D, part));
            if (p.mask && i < p.S) x = fmaf(load_mask_elem(p.mask, p.mask_dtype, mbase + i * p.ms[2]), kLog2e, x);
            const bool visible = i < p.S && col_ok && (!p.causal || col <= i);
            float pr = visible ? fast_exp2(x - sLse[u]) : 0.f;
            if (p.thr8 > 0) {
                const bool keep = dropout_keep(p, bh, i, col);
                dp = keep ? dp * p.zscale : 0.f;
                const float ds = pr * (dp - sDelta[u]);
                pr = keep ? pr * p.zscale : 0.f;
                axpy_slice<D>(dk, ds, sQ + u * D, part);
            } else {
                const float ds = pr * (dp - sDelta[u]);
                axpy_slice<D>(dk, ds, sQ + u * D, part);
            }
            axpy_slice<D>(dv, pr, sG + u * D, part);
        }
    }
    if (!col_ok) return;
    T* dkrow = static_cast<T*>(p.dk) + b * p.dks[0] + h * p.dks[1] + col * p.dks[2];
    T* dvrow = static_cast<T*>(p.dv) + b * p.dvs[0] + h * p.dvs[1] + col * p.dvs[2];
#pragma unroll
    for (int e = 0; e < DP; ++e) {
        dkrow[Slice<D>::dim(part, e)] = from_f32<T>(dk[e] * p.scale);
        dvrow[Slice<D>::dim(part, e)] = from_f32<T>(dv[e]);
    }
}

// delta[bh, i] = sum_d dO[i,d] * O[i,d]; 4 lanes per row, fp32 accumulation
// (the reference accumulates and stores it in the input dtype, trident/kernel/softmax.py:223-238).
template <typename T, int D>
__global__ __launch_bounds__(256) void generic_delta_kernel(const KParams p) {
    const int part = threadIdx.x & 3;
    const int64_t row_lin = static_cast<int64_t>(blockIdx.x) * 64 + (threadIdx.x >> 2);
    const int64_t total = static_cast<int64_t>(p.B) * p.H * p.S;
    const int64_t rl = row_lin < total ? row_lin : total - 1;
    const int row = static_cast<int>(rl % p.S);
    const int bh = static_cast<int>(rl / p.S);
    const int b = bh / p.H, h = bh % p.H;
    const T* orow = static_cast<const T*>(p.o) + b * p.os[0] + h * p.os[1] + row * p.os[2];
    const T* grow = static_cast<const T*>(p.d_o) + b * p.dos[0] + h * p.dos[1] + row * p.dos[2];
    float acc = 0.f;
#pragma unroll
    for (int e = 0; e < D / 4; ++e) {
        const int d = Slice<D>::dim(part, e);
        acc = fmaf(to_f32(orow[d]), to_f32(grow[d]), acc);
    }
    acc = quad_sum(acc);
    if (part == 0 && row_lin < total) p.delta[rl] = acc;
}

template <typename T, int D>
int launch_generic(int which, const KParams& p, hipStream_t stream) {
    const dim3 block(256);
    const int64_t groups = static_cast<int64_t>((p.S + kRows - 1) / kRows) * p.B * p.H;
    if (groups > 2147483647LL) return TRI_ATTN_ESHAPE;
    const dim3 grid(static_cast<unsigned>(groups));
    switch (which) {
        case kGenericFwd:
            hipLaunchKernelGGL((generic_fwd_kernel<T, D>), grid, block, 0, stream, p);
            break;
        case kGenericDelta: {
            const int64_t total = static_cast<int64_t>(p.B) * p.H * p.S;
            hipLaunchKernelGGL((generic_delta_kernel<T, D>), dim3(static_cast<unsigned>((total + 63) / 64)), block, 0,
                               stream, p);
            break;
        }
        case kGenericDkdv:
            hipLaunchKernelGGL((generic_dkdv_kernel<T, D>), grid, block, 0, stream, p);
            break;
        case kGenericDq:
            hipLaunchKernelGGL((generic_dq_kernel<T, D>), grid, block, 0, stream, p);
            break;
        default:
            return TRI_ATTN_ESHAPE;
    }
    return static_cast<int>(hipGetLastError());
}

template <typename T>
int launch_generic_d(int which, const KParams& p, hipStream_t stream) {
    switch (p.D) {
        case 16: return launch_generic<T, 16>(which, p, stream);
        case 32: return launch_generic<T, 32>(which, p, stream);
        case 64: return launch_generic<T, 64>(which, p, stream);
        case 128: return launch_generic<T, 128>(which, p, stream);
        default: return TRI_ATTN_ESHAPE;
    }
}

}  // namespace

int launch_generic_any(int which, int dtype, const KParams& p, hipStream_t stream) {
    switch (dtype) {
        case TRI_ATTN_F32: return launch_generic_d<float>(which, p, stream);
        case TRI_ATTN_F16: return launch_generic_d<f16_t>(which, p, stream);
        case TRI_ATTN_BF16: return launch_generic_d<bf16_t>(which, p, stream);
        default: return TRI_ATTN_EDTYPE;
    }
}

}  // namespace tri
