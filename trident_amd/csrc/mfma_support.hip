// Which calls the matrix-core kernels take, and the delta pre-pass.
#include <atomic>

#include "launch.hpp"
#include "mfma_common.hpp"

namespace tri {
namespace {

bool aligned16(const void* ptr) { return (reinterpret_cast<uintptr_t>(ptr) & 15) == 0; }
bool strides8(const int64_t* s) { return (s[0] % 8) == 0 && (s[1] % 8) == 0 && (s[2] % 8) == 0; }

// delta[bh, i] = sum_d dO[i,d] * O[i,d] (trident/kernel/softmax.py:184-238 as attention uses it).
// Pure streaming: 16-byte loads, D/8 lanes per row, fp32 accumulation, one fp32 store per row.
template <typename T, int D>
__global__ __launch_bounds__(256) void delta_kernel(const KParams p) {
    constexpr int kLanes = D / 8;           // lanes per row: 16 (D=128), 8 (D=64), 4 (D=32) or 2 (D=16)
    constexpr int kRowsPerBlock = 256 / kLanes;
    const int sub = threadIdx.x % kLanes;
    const int64_t row_lin = static_cast<int64_t>(blockIdx.x) * kRowsPerBlock + threadIdx.x / kLanes;
    const int64_t total = static_cast<int64_t>(p.B) * p.H * p.S;
    if (row_lin >= total) return;  // whole lane groups leave together: total is a multiple of 128
    const int row = static_cast<int>(row_lin % p.S);
    const int bh = static_cast<int>(row_lin / p.S);
    const int b = bh / p.H, h = bh % p.H;
    const T* orow = static_cast<const T*>(p.o) + b * p.os[0] + h * p.os[1] + static_cast<int64_t>(row) * p.os[2];
    const T* grow = static_cast<const T*>(p.d_o) + b * p.dos[0] + h * p.dos[1] + static_cast<int64_t>(row) * p.dos[2];
    const u32x4 ov = *reinterpret_cast<const u32x4*>(orow + sub * 8);
    const u32x4 gv = *reinterpret_cast<const u32x4*>(grow + sub * 8);
    float acc = 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        acc = fmaf(Mma<T>::lo(ov[i]), Mma<T>::lo(gv[i]), acc);
        acc = fmaf(Mma<T>::hi(ov[i]), Mma<T>::hi(gv[i]), acc);
    }
#pragma unroll
    for (int s = 1; s < kLanes; s <<= 1) acc += __shfl_xor(acc, s);
    if (sub == 0) p.delta[row_lin] = acc;
}

template <typename T, int D>
int launch_delta_t(const KParams& p, hipStream_t stream) {
    constexpr int kRowsPerBlock = 256 / (D / 8);
    const int64_t total = static_cast<int64_t>(p.B) * p.H * p.S;
    hipLaunchKernelGGL((delta_kernel<T, D>), dim3(static_cast<unsigned>((total + kRowsPerBlock - 1) / kRowsPerBlock)),
                       dim3(256), 0, stream, p);
    return static_cast<int>(hipGetLastError());
}

// Classes of the mask's 64 x 64 blocks. A wave takes 64 rows x 64 lanes x 16 bytes (256 fp32 or 512 16-bit keys):
// every lane folds its 16 bytes of each row into two flags (something non-zero, something other than -inf), the
// lanes of a block combine them, and one lane per block writes the class byte. Reads every mask element once.
template <typename M>
__global__ __launch_bounds__(256) void classify_mask_kernel(const KParams p, uint8_t* out, int strips, int64_t waves_total) {
    constexpr int kPerLane = 16 / sizeof(M);          // keys per lane
    constexpr int kLanesPerBlock = 64 / kPerLane;     // lanes that cover one 64-key block
    const int lane = threadIdx.x & 63;
    const int64_t w = static_cast<int64_t>(blockIdx.x) * 4 + (threadIdx.x >> 6);
    if (w >= waves_total) return;
    const int cb = p.S / 64;
    const int rbn = p.mcs[2] == 0 ? 1 : cb, mhn = p.mcs[1] == 0 ? 1 : p.H;
    const int strip = static_cast<int>(w % strips);
    const int rb = static_cast<int>((w / strips) % rbn);
    const int mh = static_cast<int>((w / strips / rbn) % mhn);
    const int mb = static_cast<int>(w / strips / rbn / mhn);
    const int key0 = (strip * 64 + lane) * kPerLane;
    const bool live = key0 < p.S;
    const M* src = static_cast<const M*>(p.mask) + mb * p.ms[0] + mh * p.ms[1] + static_cast<int64_t>(rb) * 64 * p.ms[2] + (live ? key0 : 0);
    bool nonzero = false, finite = false;
    for (int r = 0; r < 64; ++r) {
        const u32x4 v = *reinterpret_cast<const u32x4*>(src + r * p.ms[2]);
        const M* e = reinterpret_cast<const M*>(&v);
#pragma unroll
        for (int i = 0; i < kPerLane; ++i) {
            const float x = static_cast<float>(e[i]);
            nonzero |= !(x == 0.f);
            finite |= !(x == -INFINITY);
        }
    }
    int flags = (nonzero ? 1 : 0) | (finite ? 2 : 0);
#pragma unroll
    for (int d = 1; d < kLanesPerBlock; d <<= 1) flags |= __shfl_xor(flags, d);
    if (live && lane % kLanesPerBlock == 0) {
        const int cls = flags == 2 ? kMaskZero : (flags == 1 ? kMaskNegInf : kMaskMixed);  // (only finite, all of it zero) / (only -inf)
        out[mb * p.mcs[0] + mh * p.mcs[1] + rb * p.mcs[2] + key0 / 64] = static_cast<uint8_t>(cls);
    }
}

}  // namespace

int launch_classify_mask(const KParams& p, uint8_t* out, hipStream_t stream) {
    const int per_lane = p.mask_dtype == TRI_ATTN_F32 ? 4 : 8;
    if (!aligned16(p.mask) || (p.ms[0] % per_lane) || (p.ms[1] % per_lane) || (p.ms[2] % per_lane)) return TRI_ATTN_EALIGN;
    const int strips = (p.S + 64 * per_lane - 1) / (64 * per_lane);
    const int cb = p.S / 64, rbn = p.mcs[2] == 0 ? 1 : cb, mhn = p.mcs[1] == 0 ? 1 : p.H, mbn = p.mcs[0] == 0 ? 1 : p.B;
    const int64_t waves = static_cast<int64_t>(mbn) * mhn * rbn * strips;
    const dim3 grid(static_cast<unsigned>((waves + 3) / 4)), block(256);
    if (p.mask_dtype == TRI_ATTN_F32) hipLaunchKernelGGL((classify_mask_kernel<float>), grid, block, 0, stream, p, out, strips, waves);
    else if (p.mask_dtype == TRI_ATTN_F16) hipLaunchKernelGGL((classify_mask_kernel<f16_t>), grid, block, 0, stream, p, out, strips, waves);
    else hipLaunchKernelGGL((classify_mask_kernel<bf16_t>), grid, block, 0, stream, p, out, strips, waves);
    return static_cast<int>(hipGetLastError());
}

// 64 rows of a tile must be reachable with an unsigned 32-bit byte offset (2-byte elements)
static bool tile_offsets_fit(const int64_t* strides) { return strides[2] >= 0 && strides[2] < (int64_t{1} << 24); }

bool mfma_supported(int which, int dtype, const KParams& p) {
    if (dtype != TRI_ATTN_F16 && dtype != TRI_ATTN_BF16) return false;
    if (p.D != 16 && p.D != 32 && p.D != 64 && p.D != 128) return false;
    // lengths that are not multiples of 128 run the 4-wave kernels with boundary handling; those read no mask
    if (p.S % 128 != 0 && p.mask != nullptr) return false;
    if (!(p.scale > 0.f)) return false;  // the kernels take row maxima before scaling
    if (!aligned16(p.q) || !aligned16(p.k) || !aligned16(p.v)) return false;
    if (!strides8(p.qs) || !strides8(p.ks) || !strides8(p.vs)) return false;
    if (p.mask != nullptr) {
        if (p.mask_dtype != TRI_ATTN_F32 && p.mask_dtype != dtype) return false;
        if (!aligned16(p.mask)) return false;
        // mask rows are fetched 16 bytes at a time (D = 64, through LDS) or 8 / 16 bytes at a time (D = 128)
        const int64_t quantum = p.mask_dtype == TRI_ATTN_F32 ? 4 : 8;
        if ((p.ms[0] % quantum) || (p.ms[1] % quantum) || (p.ms[2] % quantum)) return false;
        if (p.ms[2] < 0 || p.ms[2] >= (int64_t{1} << 24)) return false;  // 32-bit offsets inside a mask block
    }
    switch (which) {
        case kMfmaFwd:
            // K and V tiles are fetched by LDS-direct loads with 32-bit per-lane byte offsets
            if (!tile_offsets_fit(p.ks) || !tile_offsets_fit(p.vs)) return false;
            return aligned16(p.o) && strides8(p.os);
        case kMfmaDkdv:
            // the streamed tiles are addressed with 32-bit byte offsets from a per-tile base
            if (!tile_offsets_fit(p.qs) || !tile_offsets_fit(p.dos) || !tile_offsets_fit(p.ks) || !tile_offsets_fit(p.vs)) return false;
            return aligned16(p.d_o) && strides8(p.dos) && aligned16(p.dk) && strides8(p.dks) && aligned16(p.dv) &&
                   strides8(p.dvs);
        case kMfmaDq:
            // (K, V tiles; the phased kernel also stages its Q, dO and O rows that way)
            if (!tile_offsets_fit(p.ks) || !tile_offsets_fit(p.vs) || !tile_offsets_fit(p.qs) || !tile_offsets_fit(p.dos)) return false;
            // the mask gradient leaves in 16-byte (fp32) or 8-byte (16-bit) pieces of four keys
            if (p.dmask != nullptr && (!aligned16(p.dmask) || (p.dms[0] % 4) || (p.dms[1] % 4) || (p.dms[2] % 4))) return false;
            return aligned16(p.d_o) && strides8(p.dos) && aligned16(p.dq) && strides8(p.dqs);
        default:
            return false;
    }
}

// Without a mask the dQ kernels compute delta themselves, from the dO rows they load anyway and the O rows (16-byte
// aligned like the others): the phased kernel through LDS (32-bit row offsets), the others with per-lane loads.
bool mfma_dq_fuses_delta(const KParams& p) {
    if (p.mask != nullptr) return false;
    if (!aligned16(p.o) || !strides8(p.os)) return false;
    const bool phased = p.D >= 64 && p.S % 256 == 0 && (p.D == 64 || p.thr8 <= 0 || p.causal);  // (as the launcher decides)
    return !phased || tile_offsets_fit(p.os);
}

int persistent_grid(int items) {
    static std::atomic<int> cus[64];  // per device ordinal; 0 = not asked yet (every thread would store the same value)
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return items;
    int n = cus[dev].load(std::memory_order_relaxed);
    if (n == 0) {
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) return items;
        cus[dev].store(n, std::memory_order_relaxed);
    }
    return items < n ? items : n;
}

int launch_delta(int dtype, const KParams& p, hipStream_t stream) {
    const bool vec = (dtype == TRI_ATTN_F16 || dtype == TRI_ATTN_BF16) && (p.D == 16 || p.D == 32 || p.D == 64 || p.D == 128) &&
                     aligned16(p.o) && aligned16(p.d_o) && strides8(p.os) && strides8(p.dos) &&
                     (static_cast<int64_t>(p.B) * p.H * p.S) % 128 == 0;
    if (!vec) return launch_generic_any(kGenericDelta, dtype, p, stream);
    if (dtype == TRI_ATTN_BF16)
        return p.D == 128 ? launch_delta_t<bf16_t, 128>(p, stream) : p.D == 64 ? launch_delta_t<bf16_t, 64>(p, stream)
             : p.D == 32 ? launch_delta_t<bf16_t, 32>(p, stream) : launch_delta_t<bf16_t, 16>(p, stream);
    return p.D == 128 ? launch_delta_t<f16_t, 128>(p, stream) : p.D == 64 ? launch_delta_t<f16_t, 64>(p, stream)
         : p.D == 32 ? launch_delta_t<f16_t, 32>(p, stream) : launch_delta_t<f16_t, 16>(p, stream);
}

}  // namespace tri
