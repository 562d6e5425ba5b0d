// Attention on 32-row tiles, four waves to a workgroup: fp32 inputs (on the fp32 matrix instruction,
// v_mfma_f32_32x32x2_f32), and every 16-bit problem the 16-bit kernels proper do not take (masked lengths that are not
// multiples of 128, rows aligned to four elements only; on v_mfma_f32_32x32x8_{f16,bf16_1k}). Any S >= 1, D in {16, 32, 64, 128},
// fp32 / fp16 / bf16 storage, additive mask of any dtype and broadcast, causal mask, dropout.
// With fp32 data products and sums are fp32 throughout (the instruction multiplies fp32 exactly), so results agree with
// the vector-ALU kernels of generic.hip to rounding; those remain for views whose rows are not 4-element aligned. With
// 16-bit data the inputs enter the matrix pipe as they are and P and dS rounded to their type, sums stay fp32.
//
// One 32x32x2 step takes 64 cycles of the matrix pipe for a single 4-byte operand per lane and side, so with fp32 data neither LDS
// bandwidth nor the vector ALU is anywhere near a limit here: the kernels keep it simple. 256 threads = 4 waves; a
// wave owns 32 rows (queries in forward and dQ, keys in dK/dV) whose operands stay in registers, the other side
// streams through LDS as fp32 tiles of 32 rows (row stride D + 4 floats: the 16-byte reads of 32 lanes then spread
// over all banks), converted on the way in, each tile fetched into registers while the previous one is computed on.
//
// Operand layouts (lane = 32 h + l32): A[i = l32][k = h], B[k = h][j = l32], C[i = c_row(r, h)][j = l32] for register r.
// The order in which a product's k index is walked is free as long as both operands agree, so
//   * S^T = K Q^T takes K from LDS 16 bytes at a time (dims 8 j + 4 h + 0..3 = four steps) against Q registers in
//     that order, and leaves lane (h, l32) with query l32 and keys c_row(r, h);
//   * O^T += V^T P^T walks the keys in exactly that order, step r using keys {c_row(r, 0), c_row(r, 1)}: the
//     probabilities are B operands as they stand, no exchange between lanes.
// Four consecutive steps (one 16-byte piece) are the unit the kernels are written in (quad_t below).
#include <type_traits>

#include "common.hpp"
#include "launch.hpp"
#include "mfma_common.hpp"

namespace tri {
namespace {

constexpr int kRowsPerGroup = 128;  // 4 waves x 32 rows
constexpr int kTile32 = 32;         // streamed rows per LDS tile

__device__ __forceinline__ f32x16 mma32(float a, float b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0);
}

// Four consecutive steps of a product's k index as one operand per side. fp32 data keeps the four values and takes
// four 32x32x2 steps. 16-bit data packs them and takes ONE step of the 16-bit 32x32x8 instruction, whose k index is
// 4 h + e for value e of half h: the same walk, at eight times the rate; probabilities and dS are then rounded to the
// 16-bit type on their way into the matrix pipe, exactly as in the 16-bit kernels proper.
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
template <typename T>
using quad_t = std::conditional_t<sizeof(T) == 4, float4, uint2>;
template <typename T>
__device__ __forceinline__ quad_t<T> quad(float4 v) {
    if constexpr (sizeof(T) == 4) return v;
    else return uint2{Mma<T>::pack2(v.x, v.y), Mma<T>::pack2(v.z, v.w)};
}
template <typename T>
__device__ __forceinline__ quad_t<T> quad(float a, float b, float c, float d) {
    return quad<T>(float4{a, b, c, d});
}
template <typename T>
__device__ __forceinline__ f32x16 mma_quad(quad_t<T> a, quad_t<T> b, f32x16 c) {
    if constexpr (sizeof(T) == 4) {
        c = mma32(a.x, b.x, c);
        c = mma32(a.y, b.y, c);
        c = mma32(a.z, b.z, c);
        return mma32(a.w, b.w, c);
    } else if constexpr (std::is_same_v<T, f16_t>) {
        return __builtin_amdgcn_mfma_f32_32x32x8f16(__builtin_bit_cast(f16x4, a), __builtin_bit_cast(f16x4, b), c, 0, 0, 0);
    } else {
        return __builtin_amdgcn_mfma_f32_32x32x8bf16_1k(__builtin_bit_cast(s16x4, a), __builtin_bit_cast(s16x4, b), c, 0, 0, 0);
    }
}
// two independent products side by side (fp32: their steps alternate, so that no step waits for the one before it)
template <typename T>
__device__ __forceinline__ void mma_quad2(quad_t<T> a0, quad_t<T> b0, f32x16& c0, quad_t<T> a1, quad_t<T> b1, f32x16& c1) {
    if constexpr (sizeof(T) == 4) {
        c0 = mma32(a0.x, b0.x, c0);
        c1 = mma32(a1.x, b1.x, c1);
        c0 = mma32(a0.y, b0.y, c0);
        c1 = mma32(a1.y, b1.y, c1);
        c0 = mma32(a0.z, b0.z, c0);
        c1 = mma32(a1.z, b1.z, c1);
        c0 = mma32(a0.w, b0.w, c0);
        c1 = mma32(a1.w, b1.w, c1);
    } else {
        c0 = mma_quad<T>(a0, b0, c0);
        c1 = mma_quad<T>(a1, b1, c1);
    }
}

// four consecutive elements as fp32
__device__ __forceinline__ float4 load4(const float* ptr) { return *reinterpret_cast<const float4*>(ptr); }
__device__ __forceinline__ float4 load4(const f16_t* ptr) {
    typedef _Float16 h4 __attribute__((ext_vector_type(4)));
    const h4 v = *reinterpret_cast<const h4*>(ptr);
    return float4{static_cast<float>(v[0]), static_cast<float>(v[1]), static_cast<float>(v[2]), static_cast<float>(v[3])};
}
__device__ __forceinline__ float4 load4(const bf16_t* ptr) {
    const uint2 w = *reinterpret_cast<const uint2*>(ptr);
    return float4{__builtin_bit_cast(float, w.x << 16), __builtin_bit_cast(float, w.x & 0xffff0000u),
                  __builtin_bit_cast(float, w.y << 16), __builtin_bit_cast(float, w.y & 0xffff0000u)};
}
__device__ __forceinline__ void store4(float* ptr, float4 v) { *reinterpret_cast<float4*>(ptr) = v; }
__device__ __forceinline__ void store4(f16_t* ptr, float4 v) {
    typedef _Float16 h4 __attribute__((ext_vector_type(4)));
    const h4 o = {static_cast<f16_t>(v.x), static_cast<f16_t>(v.y), static_cast<f16_t>(v.z), static_cast<f16_t>(v.w)};
    *reinterpret_cast<h4*>(ptr) = o;
}
__device__ __forceinline__ void store4(bf16_t* ptr, float4 v) {
    const uint32_t lo = Mma<bf16_t>::pack2(v.x, v.y), hi = Mma<bf16_t>::pack2(v.z, v.w);
    *reinterpret_cast<uint2*>(ptr) = uint2{lo, hi};
}

// A 32-row tile of a [S][D] matrix on its way into LDS: fetch() reads this thread's share into registers (rows past
// S as zeros), commit() writes it to the tile (row stride D + 4 floats).
template <typename T, int D>
struct Stage32 {
    static constexpr int LD = D + 4;
    static constexpr int CH = D / 4;                      // 4-element pieces per row
    static constexpr int N = (kTile32 * CH + 255) / 256;  // pieces per thread
    float4 r[N];
    __device__ __forceinline__ void fetch(const T* base, int64_t row_stride, int row0, int S) {
#pragma unroll
        for (int i = 0; i < N; ++i) {
            const int c = threadIdx.x + 256 * i;
            const int row = row0 + c / CH;
            const bool ok = (kTile32 * CH % 256 == 0 || c < kTile32 * CH) && row < S;
            r[i] = ok ? load4(base + row * row_stride + 4 * (c % CH)) : float4{0.f, 0.f, 0.f, 0.f};
        }
    }
    __device__ __forceinline__ void commit(float* tile) const {
#pragma unroll
        for (int i = 0; i < N; ++i) {
            const int c = threadIdx.x + 256 * i;
            if (kTile32 * CH % 256 == 0 || c < kTile32 * CH) store4(tile + (c / CH) * LD + 4 * (c % CH), r[i]);
        }
    }
};

__device__ __forceinline__ uint32_t pick_word(const Philox4& r, int s) {
    return s == 0 ? r.w[0] : (s == 1 ? r.w[1] : (s == 2 ? r.w[2] : r.w[3]));
}

// ------------------------------------------------------------------------------------------------ forward
template <typename T, int D>
__global__ __launch_bounds__(256, 2) void mfma32_fwd_kernel(const KParams p) {
    constexpr int LD = D + 4;
    constexpr int DB = D >= 32 ? D / 32 : 1;  // 32-wide blocks of the head dimension (D = 16: one, half empty)
    constexpr int KJ = D / 8;
    __shared__ __attribute__((aligned(16))) float sK[kTile32 * LD];
    __shared__ __attribute__((aligned(16))) float sV[kTile32 * LD];

    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int lane = threadIdx.x & 63, l32 = lane & 31, h = lane >> 5;
    int bh, qt;
    map_block(blockIdx.x, p.B * p.H, (p.S + kRowsPerGroup - 1) / kRowsPerGroup, p.causal ? kHeavyLast : kUniformTiles, &bh, &qt);
    const int b = bh / p.H, hd = bh % p.H;
    const int q0 = qt * kRowsPerGroup, wrow0 = q0 + 32 * wave, qrow = wrow0 + l32;
    const bool row_ok = qrow < p.S;
    const int qrow_c = row_ok ? qrow : p.S - 1;

    const T* kbase = static_cast<const T*>(p.k) + b * p.ks[0] + hd * p.ks[1];
    const T* vbase = static_cast<const T*>(p.v) + b * p.vs[0] + hd * p.vs[1];
    const int64_t mrow = p.mask ? b * p.ms[0] + hd * p.ms[1] + qrow_c * p.ms[2] : 0;

    // this lane's share of its query row: dims 8 j + 4 h + 0..3
    quad_t<T> qf[KJ];
    {
        const T* qptr = static_cast<const T*>(p.q) + b * p.qs[0] + hd * p.qs[1] + qrow_c * p.qs[2];
#pragma unroll
        for (int j = 0; j < KJ; ++j) qf[j] = quad<T>(load4(qptr + 8 * j + 4 * h));
    }
    f32x16 oacc[DB];
#pragma unroll
    for (int db = 0; db < DB; ++db) oacc[db] = zero16();
    float m = -INFINITY, l = 0.f;

    const int n_keys = p.causal ? min(p.S, q0 + kRowsPerGroup) : p.S;  // keys some row of the workgroup sees
    const int n_tiles = (n_keys + kTile32 - 1) / kTile32;
    Stage32<T, D> kst, vst;
    kst.fetch(kbase, p.ks[2], 0, p.S);
    vst.fetch(vbase, p.vs[2], 0, p.S);
    kst.commit(sK);
    vst.commit(sV);
    for (int t = 0; t < n_tiles; ++t) {
        const int k0 = t * kTile32;
        if (t + 1 < n_tiles) {
            kst.fetch(kbase, p.ks[2], k0 + kTile32, p.S);
            vst.fetch(vbase, p.vs[2], k0 + kTile32, p.S);
        }
        __syncthreads();
        if (!(p.causal && k0 > wrow0 + 31)) {  // (a tile wholly above this wave's rows has nothing for it)
            f32x16 s = zero16();
#pragma unroll
            for (int j = 0; j < KJ; ++j) {
                const float4 kf = *reinterpret_cast<const float4*>(sK + l32 * LD + 8 * j + 4 * h);
                s = mma_quad<T>(quad<T>(kf), qf[j], s);
            }
            // this lane has query qrow and keys k0 + c_row(i, h). One branch per tile picks the work its elements need:
            // with a mask, scaled scores plus mask values (log2 domain); without one the raw scores, whose scale goes
            // into the exponent's multiply-add; and only a tile that crosses the diagonal or the end of the sequence
            // tests its elements for visibility (a branch or a test per element costs more than the arithmetic).
            const bool edge = k0 + kTile32 > p.S || (p.causal && k0 + kTile32 - 1 > wrow0);
            float x[16];
            float xs = p.scale_log2;  // what x is still to be multiplied by
            if (p.mask) {
                xs = 1.f;
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    const int key = k0 + c_row(i, h);
                    float v = s[i] * p.scale_log2;
                    if (key < p.S) v = fmaf(load_mask_elem(p.mask, p.mask_dtype, mrow + key), kLog2e, v);
                    x[i] = key < p.S && (!p.causal || key <= qrow) ? v : -INFINITY;
                }
            } else if (edge) {
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    const int key = k0 + c_row(i, h);
                    const bool visible = key < p.S && (!p.causal || key <= qrow);
                    x[i] = visible ? s[i] : -INFINITY;
                }
            } else {
#pragma unroll
                for (int i = 0; i < 16; ++i) x[i] = s[i];
            }
            float mx = x[0];
#pragma unroll
            for (int i = 1; i < 16; ++i) mx = fmaxf(mx, x[i]);
            mx = max_xor32(mx) * xs;
            const float m_new = fmaxf(m, mx);
            if (__builtin_amdgcn_ballot_w64(m_new > m) != 0) {  // some row's maximum moved (else every factor is 1)
                const float alpha = fast_exp2(m - (m_new == -INFINITY ? 0.f : m_new));
                m = m_new;
                l *= alpha;  // (each lane sums its own 16 keys of a tile; the two halves meet at the end)
#pragma unroll
                for (int db = 0; db < DB; ++db)
#pragma unroll
                    for (int i = 0; i < 16; ++i) oacc[db][i] *= alpha;
            }
            const float m_use = m == -INFINITY ? 0.f : m;
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                x[i] = fast_exp2(fmaf(x[i], xs, -m_use));
                l += x[i];
            }
            if (p.thr8 > 0) {
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    // keys k0 + 8 g + 4 h + 0..3 of row qrow: one word of one generator block
                    const Philox4 r = dropout_block(p, bh, qrow >> 2, (k0 + 8 * g + 4 * h) >> 2);
                    const uint32_t word = pick_word(r, qrow & 3);
#pragma unroll
                    for (int bb = 0; bb < 4; ++bb) {
                        const bool keep = static_cast<int>((word >> (8 * bb)) & 0xffu) >= p.thr8;
                        x[4 * g + bb] = keep ? x[4 * g + bb] * p.zscale : 0.f;
                    }
                }
            }
#pragma unroll
            for (int g = 0; g < 4; ++g) {  // keys c_row(4 g + e, h) = 8 g + 4 h + e
                const float* vrow = sV + (8 * g + 4 * h) * LD + l32;
                const quad_t<T> pq = quad<T>(x[4 * g], x[4 * g + 1], x[4 * g + 2], x[4 * g + 3]);
#pragma unroll
                for (int db = 0; db < DB; ++db) {
                    const bool in = D >= 32 || l32 < D;
                    const float* v0 = vrow + 32 * db;
                    const quad_t<T> a = in ? quad<T>(v0[0], v0[LD], v0[2 * LD], v0[3 * LD]) : quad<T>(0.f, 0.f, 0.f, 0.f);
                    oacc[db] = mma_quad<T>(a, pq, oacc[db]);
                }
            }
        }
        __syncthreads();
        if (t + 1 < n_tiles) {
            kst.commit(sK);
            vst.commit(sV);
        }
    }
    l = sum_xor32(l);
    const float inv = 1.f / l;
    if (row_ok) {
        // O^T accumulators: register 4 g + e of block db is dim 32 db + 8 g + 4 h + e of this lane's query
        T* orow = static_cast<T*>(p.o) + b * p.os[0] + hd * p.os[1] + static_cast<int64_t>(qrow) * p.os[2];
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int d = 32 * db + 8 * g + 4 * h;
                if (D >= 32 || d < D)
                    store4(orow + d, float4{oacc[db][4 * g + 0] * inv, oacc[db][4 * g + 1] * inv, oacc[db][4 * g + 2] * inv,
                                            oacc[db][4 * g + 3] * inv});
            }
        if (h == 0) p.lse[static_cast<int64_t>(bh) * p.S + qrow] = m + fast_log2(l);
    }
}

// ------------------------------------------------------------------------------------------------ dQ (and dMask)
// Same data flow as the forward kernel: S^T = K Q^T and dP^T = V dO^T against the wave's Q and dO rows in registers,
// P and dS on the vector ALU (this lane: its query, 16 keys), dQ^T += K^T dS^T walking the keys in accumulator order.
template <typename T, int D>
__global__ __launch_bounds__(256, D == 128 ? 1 : 2) void mfma32_dq_kernel(const KParams p) {
    constexpr int LD = D + 4;
    constexpr int DB = D >= 32 ? D / 32 : 1;
    constexpr int KJ = D / 8;
    __shared__ __attribute__((aligned(16))) float sK[kTile32 * LD];
    __shared__ __attribute__((aligned(16))) float sV[kTile32 * LD];

    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int lane = threadIdx.x & 63, l32 = lane & 31, h = lane >> 5;
    int bh, qt;
    map_block(blockIdx.x, p.B * p.H, (p.S + kRowsPerGroup - 1) / kRowsPerGroup, p.causal ? kHeavyLast : kUniformTiles, &bh, &qt);
    const int b = bh / p.H, hd = bh % p.H;
    const int q0 = qt * kRowsPerGroup, wrow0 = q0 + 32 * wave, qrow = wrow0 + l32;
    const bool row_ok = qrow < p.S;
    const int qrow_c = row_ok ? qrow : p.S - 1;

    const T* kbase = static_cast<const T*>(p.k) + b * p.ks[0] + hd * p.ks[1];
    const T* vbase = static_cast<const T*>(p.v) + b * p.vs[0] + hd * p.vs[1];
    const int64_t mrow = p.mask ? b * p.ms[0] + hd * p.ms[1] + qrow_c * p.ms[2] : 0;
    const int64_t dmrow = p.dmask ? b * p.dms[0] + hd * p.dms[1] + qrow_c * p.dms[2] : 0;

    quad_t<T> qf[KJ], gf[KJ];
    {
        const T* qptr = static_cast<const T*>(p.q) + b * p.qs[0] + hd * p.qs[1] + qrow_c * p.qs[2];
        const T* gptr = static_cast<const T*>(p.d_o) + b * p.dos[0] + hd * p.dos[1] + qrow_c * p.dos[2];
#pragma unroll
        for (int j = 0; j < KJ; ++j) {
            qf[j] = quad<T>(load4(qptr + 8 * j + 4 * h));
            gf[j] = quad<T>(load4(gptr + 8 * j + 4 * h));
        }
    }
    const float lse = p.lse[static_cast<int64_t>(bh) * p.S + qrow_c];
    const float dlt = p.delta[static_cast<int64_t>(bh) * p.S + qrow_c];
    f32x16 acc[DB];
#pragma unroll
    for (int db = 0; db < DB; ++db) acc[db] = zero16();

    const int n_keys = p.causal ? min(p.S, q0 + kRowsPerGroup) : p.S;
    const int n_tiles = (n_keys + kTile32 - 1) / kTile32;
    Stage32<T, D> kst, vst;
    kst.fetch(kbase, p.ks[2], 0, p.S);
    vst.fetch(vbase, p.vs[2], 0, p.S);
    kst.commit(sK);
    vst.commit(sV);
    for (int t = 0; t < n_tiles; ++t) {
        const int k0 = t * kTile32;
        if (t + 1 < n_tiles) {
            kst.fetch(kbase, p.ks[2], k0 + kTile32, p.S);
            vst.fetch(vbase, p.vs[2], k0 + kTile32, p.S);
        }
        __syncthreads();
        if (!(p.causal && k0 > wrow0 + 31)) {
            f32x16 s = zero16(), dp = zero16();
#pragma unroll
            for (int j = 0; j < KJ; ++j) {
                const float4 kf = *reinterpret_cast<const float4*>(sK + l32 * LD + 8 * j + 4 * h);
                const float4 vf = *reinterpret_cast<const float4*>(sV + l32 * LD + 8 * j + 4 * h);
                mma_quad2<T>(quad<T>(kf), qf[j], s, quad<T>(vf), gf[j], dp);
            }
            // (one branch per tile decides about the mask: a branch per element costs more than the arithmetic it guards)
            float ds[16];
            if (p.mask) {
                float mk[16];
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    const int key = k0 + c_row(i, h);
                    mk[i] = key < p.S ? load_mask_elem(p.mask, p.mask_dtype, mrow + key) * kLog2e : 0.f;
                }
#pragma unroll
                for (int i = 0; i < 16; ++i) ds[i] = fast_exp2(fmaf(s[i], p.scale_log2, mk[i]) - lse);
            } else {
#pragma unroll
                for (int i = 0; i < 16; ++i) ds[i] = fast_exp2(fmaf(s[i], p.scale_log2, -lse));
            }
            if (k0 + kTile32 > p.S || (p.causal && k0 + kTile32 - 1 > wrow0)) {  // only such a tile has keys a row does not see
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    const int key = k0 + c_row(i, h);
                    const bool visible = key < p.S && (!p.causal || key <= qrow);
                    ds[i] = visible ? ds[i] : 0.f;
                }
            }
            if (p.thr8 > 0) {
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    const Philox4 r = dropout_block(p, bh, qrow >> 2, (k0 + 8 * g + 4 * h) >> 2);
                    const uint32_t word = pick_word(r, qrow & 3);
#pragma unroll
                    for (int bb = 0; bb < 4; ++bb) {
                        const bool keep = static_cast<int>((word >> (8 * bb)) & 0xffu) >= p.thr8;
                        dp[4 * g + bb] = keep ? dp[4 * g + bb] * p.zscale : 0.f;
                    }
                }
            }
#pragma unroll
            for (int i = 0; i < 16; ++i) ds[i] *= dp[i] - dlt;
            if (p.dmask && row_ok) {
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    const int key = k0 + c_row(i, h);
                    if (key < p.S) {
                        if (p.dmask_acc) unsafeAtomicAdd(static_cast<float*>(p.dmask) + dmrow + key, ds[i]);
                        else store_mask_elem(p.dmask, p.mask_dtype, dmrow + key, ds[i]);
                    }
                }
            }
#pragma unroll
            for (int g = 0; g < 4; ++g) {  // keys c_row(4 g + e, h) = 8 g + 4 h + e
                const float* krow = sK + (8 * g + 4 * h) * LD + l32;
                const quad_t<T> dq4 = quad<T>(ds[4 * g], ds[4 * g + 1], ds[4 * g + 2], ds[4 * g + 3]);
#pragma unroll
                for (int db = 0; db < DB; ++db) {
                    const bool in = D >= 32 || l32 < D;
                    const float* k0p = krow + 32 * db;
                    const quad_t<T> a = in ? quad<T>(k0p[0], k0p[LD], k0p[2 * LD], k0p[3 * LD]) : quad<T>(0.f, 0.f, 0.f, 0.f);
                    acc[db] = mma_quad<T>(a, dq4, acc[db]);
                }
            }
        }
        __syncthreads();
        if (t + 1 < n_tiles) {
            kst.commit(sK);
            vst.commit(sV);
        }
    }
    if (row_ok) {
        T* dqrow = static_cast<T*>(p.dq) + b * p.dqs[0] + hd * p.dqs[1] + static_cast<int64_t>(qrow) * p.dqs[2];
        const float sc = p.scale;
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int d = 32 * db + 8 * g + 4 * h;
                if (D >= 32 || d < D)
                    store4(dqrow + d, float4{acc[db][4 * g + 0] * sc, acc[db][4 * g + 1] * sc, acc[db][4 * g + 2] * sc,
                                             acc[db][4 * g + 3] * sc});
            }
    }
}

// ------------------------------------------------------------------------------------------------ dK, dV
// Roles exchanged: a wave owns 32 keys (K and V rows in registers, as B operands), Q and dO stream through LDS in
// 32-row tiles with their lse and delta. S = Q K^T and dP = dO V^T leave lane (h, l32) with key l32 and rows
// c_row(r, h); dV^T += dO^T P and dK^T += Q^T dS walk the rows in that order.
template <typename T, int D>
__global__ __launch_bounds__(256, D >= 64 ? 1 : 2) void mfma32_dkdv_kernel(const KParams p) {
    constexpr int LD = D + 4;
    constexpr int DB = D >= 32 ? D / 32 : 1;
    constexpr int KJ = D / 8;
    __shared__ __attribute__((aligned(16))) float sQ[kTile32 * LD];
    __shared__ __attribute__((aligned(16))) float sG[kTile32 * LD];
    __shared__ __attribute__((aligned(16))) float sLse[kTile32];
    __shared__ __attribute__((aligned(16))) float sDelta[kTile32];

    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int lane = threadIdx.x & 63, l32 = lane & 31, h = lane >> 5;
    int bh, kt;
    map_block(blockIdx.x, p.B * p.H, (p.S + kRowsPerGroup - 1) / kRowsPerGroup, p.causal ? kHeavyFirst : kUniformTiles, &bh, &kt);
    const int b = bh / p.H, hd = bh % p.H;
    const int g0 = kt * kRowsPerGroup, wkey0 = g0 + 32 * wave, key = wkey0 + l32;
    const bool key_ok = key < p.S;
    const int key_c = key_ok ? key : p.S - 1;

    const T* qbase = static_cast<const T*>(p.q) + b * p.qs[0] + hd * p.qs[1];
    const T* gbase = static_cast<const T*>(p.d_o) + b * p.dos[0] + hd * p.dos[1];
    const float* lse_base = p.lse + static_cast<int64_t>(bh) * p.S;
    const float* delta_base = p.delta + static_cast<int64_t>(bh) * p.S;
    const int64_t mcol = p.mask ? b * p.ms[0] + hd * p.ms[1] + key_c : 0;

    quad_t<T> kf[KJ], vf[KJ];
    {
        const T* kptr = static_cast<const T*>(p.k) + b * p.ks[0] + hd * p.ks[1] + key_c * p.ks[2];
        const T* vptr = static_cast<const T*>(p.v) + b * p.vs[0] + hd * p.vs[1] + key_c * p.vs[2];
#pragma unroll
        for (int j = 0; j < KJ; ++j) {
            kf[j] = quad<T>(load4(kptr + 8 * j + 4 * h));
            vf[j] = quad<T>(load4(vptr + 8 * j + 4 * h));
        }
    }
    f32x16 dk[DB], dv[DB];
#pragma unroll
    for (int db = 0; db < DB; ++db) {
        dk[db] = zero16();
        dv[db] = zero16();
    }

    const int r_begin = p.causal ? g0 : 0;  // rows above the workgroup's first key see none of its keys
    const int n_tiles = (p.S - r_begin + kTile32 - 1) / kTile32;
    Stage32<T, D> qst, gst;
    float aux = 0.f;  // threads 0-31: lse of a row of the tile, threads 32-63: its delta
    auto fetch_tile = [&](int r0) {
        qst.fetch(qbase, p.qs[2], r0, p.S);
        gst.fetch(gbase, p.dos[2], r0, p.S);
        if (threadIdx.x < 64) {
            const int row = r0 + l32;
            aux = row < p.S ? (h == 0 ? lse_base : delta_base)[row] : 0.f;
        }
    };
    auto commit_tile = [&]() {
        qst.commit(sQ);
        gst.commit(sG);
        if (threadIdx.x < 64) (h == 0 ? sLse : sDelta)[l32] = aux;
    };
    fetch_tile(r_begin);
    commit_tile();
    for (int t = 0; t < n_tiles; ++t) {
        const int r0 = r_begin + t * kTile32;
        if (t + 1 < n_tiles) fetch_tile(r0 + kTile32);
        __syncthreads();
        if (!(p.causal && r0 + 31 < wkey0)) {  // (rows wholly above this wave's keys see none of them)
            f32x16 s = zero16(), dp = zero16();
#pragma unroll
            for (int j = 0; j < KJ; ++j) {
                const float4 qa = *reinterpret_cast<const float4*>(sQ + l32 * LD + 8 * j + 4 * h);
                const float4 ga = *reinterpret_cast<const float4*>(sG + l32 * LD + 8 * j + 4 * h);
                mma_quad2<T>(quad<T>(qa), kf[j], s, quad<T>(ga), vf[j], dp);
            }
            // this lane: its key, rows r0 + c_row(i, h)
            float pr[16], ds[16];
            if (p.mask) {  // (one branch per tile, not one per element)
                float mk[16];
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    const int row = r0 + c_row(i, h);
                    mk[i] = row < p.S ? load_mask_elem(p.mask, p.mask_dtype, mcol + row * p.ms[2]) * kLog2e : 0.f;
                }
#pragma unroll
                for (int i = 0; i < 16; ++i) pr[i] = fast_exp2(fmaf(s[i], p.scale_log2, mk[i]) - sLse[c_row(i, h)]);
            } else {
#pragma unroll
                for (int i = 0; i < 16; ++i) pr[i] = fast_exp2(fmaf(s[i], p.scale_log2, -sLse[c_row(i, h)]));
            }
            // only a tile at the end of the sequence (rows or keys) or on the diagonal has elements that do not exist
            if (r0 + kTile32 > p.S || wkey0 + 32 > p.S || (p.causal && r0 < wkey0 + 31)) {
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    const int row = r0 + c_row(i, h);
                    const bool visible = row < p.S && key_ok && (!p.causal || key <= row);
                    pr[i] = visible ? pr[i] : 0.f;
                }
            }
            if (p.thr8 > 0) {
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    // rows r0 + 8 g + 4 h + 0..3 of this key: one byte of each word of one generator block
                    const Philox4 r = dropout_block(p, bh, (r0 + 8 * g + 4 * h) >> 2, key >> 2);
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const bool keep = static_cast<int>((r.w[e] >> (8 * (key & 3))) & 0xffu) >= p.thr8;
                        const int i = 4 * g + e;
                        ds[i] = pr[i] * ((keep ? dp[i] * p.zscale : 0.f) - sDelta[c_row(i, h)]);
                        pr[i] = keep ? pr[i] * p.zscale : 0.f;
                    }
                }
            } else {
#pragma unroll
                for (int i = 0; i < 16; ++i) ds[i] = pr[i] * (dp[i] - sDelta[c_row(i, h)]);
            }
#pragma unroll
            for (int g = 0; g < 4; ++g) {  // rows c_row(4 g + e, h) = 8 g + 4 h + e
                const float* grow = sG + (8 * g + 4 * h) * LD + l32;
                const float* qrow = sQ + (8 * g + 4 * h) * LD + l32;
                const quad_t<T> p4 = quad<T>(pr[4 * g], pr[4 * g + 1], pr[4 * g + 2], pr[4 * g + 3]);
                const quad_t<T> s4 = quad<T>(ds[4 * g], ds[4 * g + 1], ds[4 * g + 2], ds[4 * g + 3]);
#pragma unroll
                for (int db = 0; db < DB; ++db) {
                    const bool in = D >= 32 || l32 < D;
                    const float *g0p = grow + 32 * db, *q0p = qrow + 32 * db;
                    const quad_t<T> zero = quad<T>(0.f, 0.f, 0.f, 0.f);
                    mma_quad2<T>(in ? quad<T>(g0p[0], g0p[LD], g0p[2 * LD], g0p[3 * LD]) : zero, p4, dv[db],
                                 in ? quad<T>(q0p[0], q0p[LD], q0p[2 * LD], q0p[3 * LD]) : zero, s4, dk[db]);
                }
            }
        }
        __syncthreads();
        if (t + 1 < n_tiles) commit_tile();
    }
    if (key_ok) {
        T* dkrow = static_cast<T*>(p.dk) + b * p.dks[0] + hd * p.dks[1] + static_cast<int64_t>(key) * p.dks[2];
        T* dvrow = static_cast<T*>(p.dv) + b * p.dvs[0] + hd * p.dvs[1] + static_cast<int64_t>(key) * p.dvs[2];
        const float sc = p.scale;
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int d = 32 * db + 8 * g + 4 * h;
                if (D >= 32 || d < D) {
                    store4(dkrow + d, float4{dk[db][4 * g + 0] * sc, dk[db][4 * g + 1] * sc, dk[db][4 * g + 2] * sc,
                                             dk[db][4 * g + 3] * sc});
                    store4(dvrow + d, float4{dv[db][4 * g + 0], dv[db][4 * g + 1], dv[db][4 * g + 2], dv[db][4 * g + 3]});
                }
            }
    }
}

// dK, dV at D = 128: the kernel above would need K and V rows (128 registers) beside dK^T and dV^T (128 more) in one
// wave. Here a workgroup owns 64 keys whose K and V rows sit in LDS for the whole run (B operands are read from there,
// 16 bytes per four steps, like the A operands), and the two waves of a key block share its query rows: wave (kb, rh)
// takes the 32-row tiles 2 u + rh, both accumulate the full head dimension, and at the end the rh = 1 wave hands its
// accumulators to its partner through LDS.
template <typename T, int D>
__global__ __launch_bounds__(256, 1) void mfma32_dkdv_split_kernel(const KParams p) {
    constexpr int LD = D + 4;
    constexpr int DB = D / 32;
    constexpr int KJ = D / 8;
    constexpr int kKeys = 64;
    static_assert(D >= 64, "accumulators of two waves must fit into the row tiles' LDS");
    __shared__ __attribute__((aligned(16))) float sK[kKeys * LD];
    __shared__ __attribute__((aligned(16))) float sV[kKeys * LD];
    __shared__ __attribute__((aligned(16))) float sQ[2 * kTile32 * LD];  // tiles 2 u and 2 u + 1
    __shared__ __attribute__((aligned(16))) float sG[2 * kTile32 * LD];
    __shared__ __attribute__((aligned(16))) float sLse[2 * kTile32];
    __shared__ __attribute__((aligned(16))) float sDelta[2 * kTile32];

    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int kb = wave & 1, rh = wave >> 1;
    const int lane = threadIdx.x & 63, l32 = lane & 31, h = lane >> 5;
    int bh, kt;
    map_block(blockIdx.x, p.B * p.H, (p.S + kKeys - 1) / kKeys, p.causal ? kHeavyFirst : kUniformTiles, &bh, &kt);
    const int b = bh / p.H, hd = bh % p.H;
    const int g0 = kt * kKeys, wkey0 = g0 + 32 * kb, key = wkey0 + l32;
    const bool key_ok = key < p.S;
    const int key_c = key_ok ? key : p.S - 1;

    const T* qbase = static_cast<const T*>(p.q) + b * p.qs[0] + hd * p.qs[1];
    const T* gbase = static_cast<const T*>(p.d_o) + b * p.dos[0] + hd * p.dos[1];
    const float* lse_base = p.lse + static_cast<int64_t>(bh) * p.S;
    const float* delta_base = p.delta + static_cast<int64_t>(bh) * p.S;
    const int64_t mcol = p.mask ? b * p.ms[0] + hd * p.ms[1] + key_c : 0;

    // two 32-row tiles per fetch (Stage32 twice: rows r0 .. r0 + 31 and r0 + 32 .. r0 + 63)
    Stage32<T, D> st[2][2];
    float aux = 0.f;  // threads 0-63: lse of a row of the two tiles, threads 64-127: its delta
    auto fetch_rows = [&](int r0) {
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            st[u][0].fetch(qbase, p.qs[2], r0 + kTile32 * u, p.S);
            st[u][1].fetch(gbase, p.dos[2], r0 + kTile32 * u, p.S);
        }
        if (threadIdx.x < 128) {
            const int row = r0 + (threadIdx.x & 63);
            aux = row < p.S ? (threadIdx.x < 64 ? lse_base : delta_base)[row] : 0.f;
        }
    };
    auto commit_rows = [&]() {
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            st[u][0].commit(sQ + u * kTile32 * LD);
            st[u][1].commit(sG + u * kTile32 * LD);
        }
        if (threadIdx.x < 128) (threadIdx.x < 64 ? sLse : sDelta)[threadIdx.x & 63] = aux;
    };
    {
        // the workgroup's K and V rows (rows past S as zeros), through the same staging registers
        const T* kbase = static_cast<const T*>(p.k) + b * p.ks[0] + hd * p.ks[1];
        const T* vbase = static_cast<const T*>(p.v) + b * p.vs[0] + hd * p.vs[1];
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            st[u][0].fetch(kbase, p.ks[2], g0 + kTile32 * u, p.S);
            st[u][1].fetch(vbase, p.vs[2], g0 + kTile32 * u, p.S);
        }
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            st[u][0].commit(sK + u * kTile32 * LD);
            st[u][1].commit(sV + u * kTile32 * LD);
        }
    }
    f32x16 dk[DB], dv[DB];
#pragma unroll
    for (int db = 0; db < DB; ++db) {
        dk[db] = zero16();
        dv[db] = zero16();
    }
    const int r_begin = p.causal ? g0 : 0;
    const int n_steps = (p.S - r_begin + 2 * kTile32 - 1) / (2 * kTile32);
    fetch_rows(r_begin);
    commit_rows();
    const float* myK = sK + (32 * kb + l32) * LD + 4 * h;
    const float* myV = sV + (32 * kb + l32) * LD + 4 * h;
    const float* tQ = sQ + rh * kTile32 * LD;
    const float* tG = sG + rh * kTile32 * LD;
    for (int u = 0; u < n_steps; ++u) {
        const int r0 = r_begin + (2 * u + rh) * kTile32;  // this wave's tile
        if (u + 1 < n_steps) fetch_rows(r_begin + (2 * u + 2) * kTile32);
        __syncthreads();
        if (r0 < p.S && !(p.causal && r0 + 31 < wkey0)) {
            f32x16 s = zero16(), dp = zero16();
#pragma unroll
            for (int j = 0; j < KJ; ++j) {
                const float4 qa = *reinterpret_cast<const float4*>(tQ + l32 * LD + 8 * j + 4 * h);
                const float4 ga = *reinterpret_cast<const float4*>(tG + l32 * LD + 8 * j + 4 * h);
                const float4 kf = *reinterpret_cast<const float4*>(myK + 8 * j);
                const float4 vf = *reinterpret_cast<const float4*>(myV + 8 * j);
                mma_quad2<T>(quad<T>(qa), quad<T>(kf), s, quad<T>(ga), quad<T>(vf), dp);
            }
            float pr[16], ds[16];
            if (p.mask) {  // (one branch per tile, not one per element)
                float mk[16];
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    const int row = r0 + c_row(i, h);
                    mk[i] = row < p.S ? load_mask_elem(p.mask, p.mask_dtype, mcol + row * p.ms[2]) * kLog2e : 0.f;
                }
#pragma unroll
                for (int i = 0; i < 16; ++i) pr[i] = fast_exp2(fmaf(s[i], p.scale_log2, mk[i]) - sLse[kTile32 * rh + c_row(i, h)]);
            } else {
#pragma unroll
                for (int i = 0; i < 16; ++i) pr[i] = fast_exp2(fmaf(s[i], p.scale_log2, -sLse[kTile32 * rh + c_row(i, h)]));
            }
            if (r0 + kTile32 > p.S || wkey0 + 32 > p.S || (p.causal && r0 < wkey0 + 31)) {  // (as in the kernel above)
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    const int row = r0 + c_row(i, h);
                    const bool visible = row < p.S && key_ok && (!p.causal || key <= row);
                    pr[i] = visible ? pr[i] : 0.f;
                }
            }
            if (p.thr8 > 0) {
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    const Philox4 r = dropout_block(p, bh, (r0 + 8 * g + 4 * h) >> 2, key >> 2);
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const bool keep = static_cast<int>((r.w[e] >> (8 * (key & 3))) & 0xffu) >= p.thr8;
                        const int i = 4 * g + e;
                        ds[i] = pr[i] * ((keep ? dp[i] * p.zscale : 0.f) - sDelta[kTile32 * rh + c_row(i, h)]);
                        pr[i] = keep ? pr[i] * p.zscale : 0.f;
                    }
                }
            } else {
#pragma unroll
                for (int i = 0; i < 16; ++i) ds[i] = pr[i] * (dp[i] - sDelta[kTile32 * rh + c_row(i, h)]);
            }
#pragma unroll
            for (int g = 0; g < 4; ++g) {  // rows c_row(4 g + e, h) = 8 g + 4 h + e
                const float* grow = tG + (8 * g + 4 * h) * LD + l32;
                const float* qrow = tQ + (8 * g + 4 * h) * LD + l32;
                const quad_t<T> p4 = quad<T>(pr[4 * g], pr[4 * g + 1], pr[4 * g + 2], pr[4 * g + 3]);
                const quad_t<T> s4 = quad<T>(ds[4 * g], ds[4 * g + 1], ds[4 * g + 2], ds[4 * g + 3]);
#pragma unroll
                for (int db = 0; db < DB; ++db) {
                    const float *g0p = grow + 32 * db, *q0p = qrow + 32 * db;
                    mma_quad2<T>(quad<T>(g0p[0], g0p[LD], g0p[2 * LD], g0p[3 * LD]), p4, dv[db],
                                 quad<T>(q0p[0], q0p[LD], q0p[2 * LD], q0p[3 * LD]), s4, dk[db]);
                }
            }
        }
        __syncthreads();
        if (u + 1 < n_steps) commit_rows();
    }
    // the rh = 1 waves pass their sums to their partners: 2 DB blocks of 16 registers per lane, laid out so that a
    // lane's 16-byte pieces are contiguous over the lanes
    __syncthreads();
    {
        float* xch = (kb == 0 ? sQ : sG);  // 2 DB * 16 * 64 floats = 32 KiB at D = 128: inside one pair of row tiles
        static_assert(2 * DB * 16 * 64 <= 2 * kTile32 * LD, "exchange area");
        if (rh == 1) {
#pragma unroll
            for (int db = 0; db < DB; ++db)
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    store4(xch + ((2 * db + 0) * 4 + g) * 256 + lane * 4,
                           float4{dk[db][4 * g + 0], dk[db][4 * g + 1], dk[db][4 * g + 2], dk[db][4 * g + 3]});
                    store4(xch + ((2 * db + 1) * 4 + g) * 256 + lane * 4,
                           float4{dv[db][4 * g + 0], dv[db][4 * g + 1], dv[db][4 * g + 2], dv[db][4 * g + 3]});
                }
        }
        __syncthreads();
        if (rh == 0 && key_ok) {
            T* dkrow = static_cast<T*>(p.dk) + b * p.dks[0] + hd * p.dks[1] + static_cast<int64_t>(key) * p.dks[2];
            T* dvrow = static_cast<T*>(p.dv) + b * p.dvs[0] + hd * p.dvs[1] + static_cast<int64_t>(key) * p.dvs[2];
            const float sc = p.scale;
#pragma unroll
            for (int db = 0; db < DB; ++db)
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    const int d = 32 * db + 8 * g + 4 * h;
                    const float4 ok = *reinterpret_cast<const float4*>(xch + ((2 * db + 0) * 4 + g) * 256 + lane * 4);
                    const float4 ov = *reinterpret_cast<const float4*>(xch + ((2 * db + 1) * 4 + g) * 256 + lane * 4);
                    store4(dkrow + d, float4{(dk[db][4 * g + 0] + ok.x) * sc, (dk[db][4 * g + 1] + ok.y) * sc,
                                             (dk[db][4 * g + 2] + ok.z) * sc, (dk[db][4 * g + 3] + ok.w) * sc});
                    store4(dvrow + d, float4{dv[db][4 * g + 0] + ov.x, dv[db][4 * g + 1] + ov.y, dv[db][4 * g + 2] + ov.z,
                                             dv[db][4 * g + 3] + ov.w});
                }
        }
    }
}

template <typename T, int D>
int launch32(int which, const KParams& p, hipStream_t stream) {
    const int64_t groups = static_cast<int64_t>((p.S + kRowsPerGroup - 1) / kRowsPerGroup) * p.B * p.H;
    if (groups > 2147483647LL) return TRI_ATTN_ESHAPE;
    const dim3 grid(static_cast<unsigned>(groups)), block(256);
    switch (which) {
        case kMfmaFwd:
            hipLaunchKernelGGL((mfma32_fwd_kernel<T, D>), grid, block, 0, stream, p);
            break;
        case kMfmaDq:
            hipLaunchKernelGGL((mfma32_dq_kernel<T, D>), grid, block, 0, stream, p);
            break;
        case kMfmaDkdv:
            if constexpr (D == 128) {
                const int64_t groups64 = static_cast<int64_t>((p.S + 63) / 64) * p.B * p.H;
                if (groups64 > 2147483647LL) return TRI_ATTN_ESHAPE;
                hipLaunchKernelGGL((mfma32_dkdv_split_kernel<T, D>), dim3(static_cast<unsigned>(groups64)), block, 0, stream, p);
            } else {
                hipLaunchKernelGGL((mfma32_dkdv_kernel<T, D>), grid, block, 0, stream, p);
            }
            break;
        default:
            return TRI_ATTN_ESHAPE;
    }
    return static_cast<int>(hipGetLastError());
}

template <typename T>
int launch32_d(int which, const KParams& p, hipStream_t stream) {
    switch (p.D) {
        case 16: return launch32<T, 16>(which, p, stream);
        case 32: return launch32<T, 32>(which, p, stream);
        case 64: return launch32<T, 64>(which, p, stream);
        case 128: return launch32<T, 128>(which, p, stream);
        default: return TRI_ATTN_ESHAPE;
    }
}

bool rows4(const void* ptr, const int64_t* s, int elem_bytes) {
    return reinterpret_cast<uintptr_t>(ptr) % (4 * elem_bytes) == 0 && s[0] % 4 == 0 && s[1] % 4 == 0 && s[2] % 4 == 0;
}

}  // namespace

bool mfma32_supported(int which, int dtype, const KParams& p) {
    if (dtype < TRI_ATTN_F32 || dtype > TRI_ATTN_BF16) return false;
    if (p.D != 16 && p.D != 32 && p.D != 64 && p.D != 128) return false;
    if (!(p.scale > 0.f)) return false;  // the forward takes row maxima before scaling
    const int eb = dtype == TRI_ATTN_F32 ? 4 : 2;
    // rows are read and written four elements at a time
    if (!rows4(p.q, p.qs, eb) || !rows4(p.k, p.ks, eb) || !rows4(p.v, p.vs, eb)) return false;
    switch (which) {
        case kMfmaFwd: return rows4(p.o, p.os, eb);
        case kMfmaDq: return rows4(p.d_o, p.dos, eb) && rows4(p.dq, p.dqs, eb);
        case kMfmaDkdv: return rows4(p.d_o, p.dos, eb) && rows4(p.dk, p.dks, eb) && rows4(p.dv, p.dvs, eb);
        default: return false;
    }
}

int launch_mfma32(int which, int dtype, const KParams& p, hipStream_t stream) {
    switch (dtype) {
        case TRI_ATTN_F32: return launch32_d<float>(which, p, stream);
        case TRI_ATTN_F16: return launch32_d<f16_t>(which, p, stream);
        case TRI_ATTN_BF16: return launch32_d<bf16_t>(which, p, stream);
        default: return TRI_ATTN_EDTYPE;
    }
}

}  // namespace tri
