// Forward attention on the matrix cores: online-softmax flash kernel for fp16/bf16,
// D in {64,128}, S a multiple of 128 (replaces trident/kernel/attention.py:33-165).
//
// A workgroup of NW waves owns 32*NW query rows, one wave 32 of them. Q stays in registers as
// the B operand of S^T = K Q^T; K and V tiles of 64 keys live row-major (swizzled) in a four-stage
// LDS ring filled by LDS-direct loads two tiles ahead: no staging registers, no address or
// permute arithmetic on the vector ALU, whose issue slots the softmax needs. K is read as row
// fragments, V^T through transposed LDS reads of the same row-major tile. S^T and O^T = V^T P^T
// accumulate in fp32; P goes from the S^T accumulators to the B operand of the second MFMA in
// registers. The row statistics live one per lane; the two lane halves of a row are combined
// with one cross-lane exchange per tile.
//
// With 8 waves there are two per SIMD. All of them run the same schedule: running the second wave
// of a SIMD half a tile out of phase (its P V one tile late) was measured 7 % slower, in the kernel
// and in a register-only model of its instruction mix alike.
#include "launch.hpp"
#include "mfma_common.hpp"

namespace tri {
namespace {

constexpr int kBN = 64;      // keys per tile
constexpr int kStages = 4;   // LDS ring depth
constexpr float kTau = 8.f;  // lazy-rescale threshold, log2 domain

enum MaskKind { kNoMask = 0, kMaskF32 = 1, kMaskT = 2 };

template <typename T, int D, int NW, bool CAUSAL, int MASK, bool DROPOUT>
__global__ __launch_bounds__(NW * 64, 2) void mfma_fwd_kernel(const KParams p) {
    using Tile = SwzTile<D>;
    constexpr int kBM = 32 * NW;
    constexpr int kKBytes = Tile::kBytes;
    constexpr int kStageBytes = 2 * Tile::kBytes;  // K tile, V tile
    constexpr int kBlocksPerWave = 2 * Tile::kBlocks / NW;  // LDS-direct loads per wave and tile
    constexpr int KK = D / 16;  // K-steps of S^T
    constexpr int DB = D / 32;  // 32-row blocks of O^T
    constexpr int kSteps = 2 * KK, kAhead = 4;
    constexpr int kPvSteps = 4 * DB, kPvAhead = 4;
    // An fp32 mask block of a wave (32 rows x 64 keys) goes through a private 8 KiB LDS region when
    // it fits (D = 64): lanes own rows, so direct loads would touch 32 cache lines per instruction,
    // while LDS-direct loads fetch whole 256-byte rows and the swizzled tile is read back without
    // bank conflicts. The region has the geometry of a 32-row SwzTile<128> (256-byte rows).
    constexpr bool kMaskViaLds = MASK == kMaskF32 && D == 64;
    using MaskTile = SwzTile<128>;
    constexpr int kMaskBytes = 32 * MaskTile::kRowBytes;
    __shared__ __attribute__((aligned(1024))) char smem[kStages * kStageBytes + (kMaskViaLds ? NW * kMaskBytes : 0)];

    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lane = tid & 63, l32 = lane & 31, h = lane >> 5;
    int bh, qt;
    map_block_for<MASK>(p, blockIdx.x, p.S / kBM, CAUSAL ? kHeavyLast : kUniformTiles, &bh, &qt);
    const int b = bh / p.H, hd = bh % p.H;
    const int q0 = qt * kBM;
    const int wrow0 = q0 + 32 * wave;  // first query row of this wave
    const int qrow = wrow0 + l32;

    const char* qbase = static_cast<const char*>(p.q) + (b * p.qs[0] + hd * p.qs[1]) * 2;
    const char* kbase = static_cast<const char*>(p.k) + (b * p.ks[0] + hd * p.ks[1]) * 2;
    const char* vbase = static_cast<const char*>(p.v) + (b * p.vs[0] + hd * p.vs[1]) * 2;
    const int64_t krow_bytes = p.ks[2] * 2, vrow_bytes = p.vs[2] * 2;

    u32x4 qf[KK];
#pragma unroll
    for (int kk = 0; kk < KK; ++kk)
        qf[kk] = *reinterpret_cast<const u32x4*>(qbase + qrow * p.qs[2] * 2 + (2 * kk + h) * 16);

    f32x16 oacc[DB];
#pragma unroll
    for (int db = 0; db < DB; ++db) oacc[db] = zero16();
    float m = -INFINITY, l = 0.f;  // reference exponent (log2 domain, scaled) and this lane's partial sum

    const int n_tiles = CAUSAL ? (q0 + kBM) / kBN : p.S / kBN;            // tiles the workgroup streams
    const int my_tiles = CAUSAL ? (wrow0 + 31) / kBN + 1 : n_tiles;       // tiles this wave has visible keys in
    const float c = p.scale_log2;

    char* mask_lds = smem + kStages * kStageBytes + wave * kMaskBytes;
    auto issue_mask = [&](int t) {  // mask block of tile t -> this wave's region (8 LDS-direct loads)
        if constexpr (kMaskViaLds) {
            const char* src = static_cast<const char*>(p.mask) +
                              (b * p.ms[0] + hd * p.ms[1] + static_cast<int64_t>(wrow0) * p.ms[2] + t * kBN) * 4;
            int l = lane;
            asm volatile("" : "+v"(l));  // offsets recomputed per tile rather than kept in registers
#pragma unroll
            for (int blk = 0; blk < kMaskBytes / 1024; ++blk)
                lds_direct_load16(src, static_cast<uint32_t>(MaskTile::src_off(blk, l, p.ms[2] * 4)), mask_lds + blk * 1024);
        }
    };
    issue_mask(0);

    auto issue_tile = [&](int t) {  // K and V rows of tile t -> ring slot t % kStages
        char* stage = smem + (t % kStages) * kStageBytes;
        int l = lane;
        asm volatile("" : "+v"(l));  // offsets recomputed per tile rather than kept in registers
#pragma unroll
        for (int i = 0; i < kBlocksPerWave; ++i) {
            const int blk = wave * kBlocksPerWave + i;  // 0 .. 2*kBlocks-1 over the K tile then the V tile
            const bool is_v = blk >= Tile::kBlocks;
            const char* tile_src = is_v ? vbase + static_cast<int64_t>(t) * kBN * vrow_bytes
                                        : kbase + static_cast<int64_t>(t) * kBN * krow_bytes;
            const uint32_t off = static_cast<uint32_t>(Tile::src_off(is_v ? blk - Tile::kBlocks : blk, l, is_v ? vrow_bytes : krow_bytes));
            lds_direct_load16(tile_src, off, stage + blk * 1024);
        }
    };
    issue_tile(0);
    if (n_tiles > 1) issue_tile(1);
    if (n_tiles > 2) issue_tile(2);
    // (the Q fragments were requested before the tiles, so both latencies overlap)
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) settle(qf[kk]);

    const int row_off0 = Tile::off(l32, h);
    const int tr_off0 = Tile::tr_off(0, 0, lane), tr_off1 = Tile::tr_off(0, 1, lane);
    // fragment s of the S^T operand (key block s / KK, K-step s % KK) and of the O^T operand
    // (K-step s / DB = 16 keys, column block s % DB)
    auto k_frag = [&](const char* sK, int s) { return lds_read16(sK, (row_off0 ^ ((s % KK) << 5)) + 32 * (s / KK) * Tile::kRowBytes); };
    auto v_frag = [&](const char* sV, int s) { return Tile::tr_frag(sV, tr_off0 ^ ((s % DB) << 6), tr_off1 ^ ((s % DB) << 6), s / DB); };

    for (int j = 0; j < n_tiles; ++j) {
        // tile j has landed (up to two younger tiles may still be in flight) and is visible to all
        // waves; every wave is done with tile j-1, whose slot takes the load of tile j+3
        {
            const int younger = min(2, n_tiles - 1 - j);
            if (younger == 2) TRI_WAIT_VMCNT(2 * kBlocksPerWave);
            else if (younger == 1) TRI_WAIT_VMCNT(kBlocksPerWave);
            else TRI_WAIT_VMCNT(0);
        }
        lds_barrier();
        if (j + 3 < n_tiles) issue_tile(j + 3);
        const char* sK = smem + (j % kStages) * kStageBytes;
        const char* sV = sK + kKBytes;
        const int t0 = j * kBN;

        const bool active = j < my_tiles;
        float x[32];  // scores of this lane: x[16*kb + i] is key t0 + 32*kb + c_row(i,h)
        float mk[MASK != kNoMask ? 32 : 1];
        if (active) {
            // additive mask for this lane's row: issued before the MFMAs, used after them
            if constexpr (kMaskViaLds) {
                // the block was requested a tile ago; only the loads of tile j+3 are younger (block 0
                // precedes every tile load, and tile 0 has landed)
                if (j > 0) {
                    if (j + 3 < n_tiles) TRI_WAIT_VMCNT(kBlocksPerWave);
                    else TRI_WAIT_VMCNT(0);
                }
#pragma unroll
                for (int g = 0; g < 8; ++g) {
                    const f32x4 v = *reinterpret_cast<const f32x4*>(mask_lds + MaskTile::off(l32, 8 * (g >> 2) + 2 * (g & 3) + h));
                    mk[4 * g + 0] = v.x; mk[4 * g + 1] = v.y; mk[4 * g + 2] = v.z; mk[4 * g + 3] = v.w;
                }
            } else if constexpr (MASK != kNoMask) {
                const int64_t mrow = b * p.ms[0] + hd * p.ms[1] + static_cast<int64_t>(qrow) * p.ms[2] + t0;
#pragma unroll
                for (int g = 0; g < 8; ++g) {
                    const int key0 = 32 * (g >> 2) + 8 * (g & 3) + 4 * h;
                    if constexpr (MASK == kMaskF32) {
                        const f32x4 v = *reinterpret_cast<const f32x4*>(static_cast<const float*>(p.mask) + mrow + key0);
                        mk[4 * g + 0] = v.x; mk[4 * g + 1] = v.y; mk[4 * g + 2] = v.z; mk[4 * g + 3] = v.w;
                    } else {
                        const u32x2 v = *reinterpret_cast<const u32x2*>(static_cast<const T*>(p.mask) + mrow + key0);
                        mk[4 * g + 0] = Mma<T>::lo(v.x); mk[4 * g + 1] = Mma<T>::hi(v.x);
                        mk[4 * g + 2] = Mma<T>::lo(v.y); mk[4 * g + 3] = Mma<T>::hi(v.y);
                    }
                }
            }
            // S^T = K Q^T with the A fragments requested kAhead MFMAs before their use
            u32x4 ring[kAhead];
#pragma unroll
            for (int s = 0; s < kAhead; ++s)
                ring[s] = k_frag(sK, s);
            __builtin_amdgcn_sched_barrier(0);
            f32x16 st[2] = {zero16(), zero16()};
#pragma unroll
            for (int s = 0; s < kSteps; ++s) {
                st[s / KK] = Mma<T>::run(ring[s % kAhead], qf[s % KK], st[s / KK]);
                if (s + kAhead < kSteps) {
                    const int n = s + kAhead;
                    ring[s % kAhead] = k_frag(sK, n);
                }
                __builtin_amdgcn_sched_barrier(0);
            }
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                x[i] = st[0][i];
                x[16 + i] = st[1][i];
            }
        }

        if constexpr (kMaskViaLds) {
            // this tile's mask values are in registers: the region can take the next block
            if (active && j + 1 < my_tiles) {
                asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                issue_mask(j + 1);
            }
        }

        if (active) {
            // scores in the log2 domain; without a mask the scale is folded into the exponent
            if constexpr (MASK != kNoMask) {
#pragma unroll
                for (int e = 0; e < 32; ++e) x[e] = fmaf(mk[e], kLog2e, x[e] * c);
            }
            if (CAUSAL && t0 + kBN - 1 > wrow0) {
#pragma unroll
                for (int e = 0; e < 32; ++e) {
                    const int key = t0 + 32 * (e >> 4) + c_row(e & 15, h);
                    x[e] = key <= qrow ? x[e] : -INFINITY;
                }
            }
            float mx = x[0];
#pragma unroll
            for (int e = 1; e < 32; ++e) mx = fmaxf(mx, x[e]);
            mx = fmaxf(mx, xor32(mx));
            if constexpr (MASK == kNoMask) mx *= c;
            // Lazy rescaling: m is the reference exponent of l and of the O accumulators, not
            // necessarily the running maximum. It is only moved (and O rescaled) when some row of
            // the wave outgrew it by more than 2^kTau; until then probabilities may exceed 1 by
            // that factor, which fp32 sums and 16-bit P hold without loss.
            if (__builtin_amdgcn_ballot_w64(mx > m + kTau) != 0) {
                const float m_new = fmaxf(m, mx);
                const float alpha = fast_exp2(m - (m_new == -INFINITY ? 0.f : m_new));
                l *= alpha;
                m = m_new;
#pragma unroll
                for (int db = 0; db < DB; ++db)
#pragma unroll
                    for (int i = 0; i < 16; ++i) oacc[db][i] *= alpha;
            }
            const float m_use = m == -INFINITY ? 0.f : m;
#pragma unroll
            for (int e = 0; e < 32; ++e) {
                if constexpr (MASK == kNoMask) x[e] = fast_exp2(fmaf(x[e], c, -m_use));
                else x[e] = fast_exp2(x[e] - m_use);
            }
            float psum = 0.f;
            if constexpr (DROPOUT) {
#pragma unroll
                for (int e = 0; e < 32; ++e) psum += x[e];
#pragma unroll
                for (int kb = 0; kb < 2; ++kb) {
                    // group g of key block kb: keys t0 + 32 kb + 8 g + 4 h .. +3; this lane generates g = lane % 4
                    const Philox4 mine = dropout_block(p, bh, qrow >> 2, (t0 + 32 * kb + 8 * (lane & 3) + 4 * h) >> 2);
                    uint32_t w[4];
                    quad_row_words(mine, lane, w);
#pragma unroll
                    for (int g = 0; g < 4; ++g)
#pragma unroll
                        for (int bb = 0; bb < 4; ++bb) {
                            const bool keep = static_cast<int>((w[g] >> (8 * bb)) & 0xffu) >= p.thr8;
                            x[16 * kb + 4 * g + bb] = keep ? x[16 * kb + 4 * g + bb] * p.zscale : 0.f;
                        }
                }
            }
            // P as B operands; without dropout the row sum is taken from the rounded P that is
            // actually multiplied with V, two values per instruction
            u32x4 pb[4];
#pragma unroll
            for (int ks = 0; ks < 4; ++ks) {
                pb[ks] = pack8<T>(&x[8 * ks]);
                if constexpr (!DROPOUT) {
                    psum = Mma<T>::add_pair(pb[ks].x, psum);
                    psum = Mma<T>::add_pair(pb[ks].y, psum);
                    psum = Mma<T>::add_pair(pb[ks].z, psum);
                    psum = Mma<T>::add_pair(pb[ks].w, psum);
                }
            }
            l += psum;
            // O^T += V^T P^T
            {
                u32x4 vring[kPvAhead];
#pragma unroll
                for (int s = 0; s < kPvAhead; ++s)
                    vring[s] = v_frag(sV, s);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int s = 0; s < kPvSteps; ++s) {
                    oacc[s % DB] = Mma<T>::run(vring[s % kPvAhead], pb[s / DB], oacc[s % DB]);
                    if (s + kPvAhead < kPvSteps) {
                        const int n = s + kPvAhead;
                        vring[s % kPvAhead] = v_frag(sV, n);
                    }
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
        }
    }

    l += xor32(l);
    const float inv = 1.f / l;
    // every wave is out of the loop: the ring can serve as the waves' private transposition patches
    lds_barrier();
    {
        using Store = RowBlockStore<T, DB>;
        static_assert(NW * Store::kPatchBytes <= kStages * kStageBytes, "patches must fit into the ring");
        char* o0 = static_cast<char*>(p.o) + (b * p.os[0] + hd * p.os[1] + static_cast<int64_t>(wrow0) * p.os[2]) * 2;
        Store::run(oacc, [inv](float x) { return x * inv; }, smem + wave * Store::kPatchBytes, o0, p.os[2] * 2, lane);
    }
    if (h == 0) p.lse[static_cast<int64_t>(bh) * p.S + qrow] = m + fast_log2(l);
}

template <typename T, int D, int NW, bool CAUSAL, int MASK>
int launch_fwd_dropout(const KParams& p, hipStream_t stream) {
    const dim3 grid(p.B * p.H * (p.S / (32 * NW))), block(64 * NW);
    if (p.thr8 > 0) hipLaunchKernelGGL((mfma_fwd_kernel<T, D, NW, CAUSAL, MASK, true>), grid, block, 0, stream, p);
    else hipLaunchKernelGGL((mfma_fwd_kernel<T, D, NW, CAUSAL, MASK, false>), grid, block, 0, stream, p);
    return static_cast<int>(hipGetLastError());
}

template <typename T, int D, int NW>
int launch_fwd_variant(int dtype, const KParams& p, hipStream_t stream) {
    if (p.causal) return launch_fwd_dropout<T, D, NW, true, kNoMask>(p, stream);
    if (p.mask == nullptr) return launch_fwd_dropout<T, D, NW, false, kNoMask>(p, stream);
    if (p.mask_dtype == TRI_ATTN_F32) return launch_fwd_dropout<T, D, NW, false, kMaskF32>(p, stream);
    if (p.mask_dtype == dtype) return launch_fwd_dropout<T, D, NW, false, kMaskT>(p, stream);
    return TRI_ATTN_EDTYPE;
}

template <typename T, int D>
int launch_fwd_waves(int dtype, const KParams& p, hipStream_t stream) {
    // 8 waves (256 query rows) when the sequence allows it: two waves per SIMD out of phase
    if (p.S % 256 == 0) return launch_fwd_variant<T, D, 8>(dtype, p, stream);
    return launch_fwd_variant<T, D, 4>(dtype, p, stream);
}

}  // namespace

int launch_mfma_fwd(int dtype, const KParams& p, hipStream_t stream) {
    if (dtype == TRI_ATTN_BF16)
        return p.D == 128 ? launch_fwd_waves<bf16_t, 128>(dtype, p, stream) : launch_fwd_waves<bf16_t, 64>(dtype, p, stream);
    return p.D == 128 ? launch_fwd_waves<f16_t, 128>(dtype, p, stream) : launch_fwd_waves<f16_t, 64>(dtype, p, stream);
}

}  // namespace tri
