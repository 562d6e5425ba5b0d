// Backward attention on the matrix cores for fp16/bf16, D in {16,32,64,128}, S a multiple of 128
// (replaces trident/kernel/attention.py:169-339, split in two passes so that no gradient
// tile is ever accumulated in global memory):
//
//   dQ pass    one workgroup per 256 (128) query rows (a wave owns 32), streaming key tiles of 64:
//              S^T = K Q^T, dP^T = V dO^T, dS^T = P^T * (dP^T - delta), dQ^T += K^T dS^T
//   dK/dV pass one workgroup per 256 (128) keys (a wave, or for D = 128 a pair of waves, owns 32),
//              streaming query tiles of 64: S = Q K^T, dP = dO V^T, dV^T += dO^T P, dK^T += Q^T dS
//
// In both, the lane index is the row that owns the accumulators (query row resp. key), the
// stationary operands (Q,dO resp. K,V) stay in registers as MFMA B operands, and P / dS go
// from the accumulators of one MFMA to the B operand of the next without leaving registers.
#include <type_traits>

#include "launch.hpp"
#include "mfma_common.hpp"

namespace tri {
namespace {

constexpr int kBM = 128;  // stationary rows per workgroup
constexpr int kBN = 64;   // streamed rows per tile

enum MaskKind { kNoMask = 0, kMaskF32 = 1, kMaskT = 2 };

template <typename T, int MASK>
__device__ __forceinline__ float mask_at(const void* mask, int64_t off) {
    if constexpr (MASK == kMaskF32) return static_cast<const float*>(mask)[off];
    else return static_cast<float>(static_cast<const T*>(mask)[off]);
}

// ------------------------------------------------------------------------------------ dQ
// A workgroup of NW waves owns 32*NW query rows, one wave 32 of them with its Q and dO rows in
// registers (B operands) and dQ^T in fp32 accumulators; two waves per SIMD. K and V stream as
// 64-key swizzled LDS tiles in a ring of 4, filled by LDS-direct loads three tiles ahead (no
// staging registers, no ds_write). Per 32-key block: S^T = K Q^T and dP^T = V dO^T from row
// fragments, dS^T = P^T (dP^T - delta) on the vector ALU, dQ^T += K^T dS^T with K^T read through
// transposed LDS reads of the same K tile.
// RAGGED (4 waves, no mask): S is not a multiple of 128. Rows and keys at or beyond S do not exist: loads clamp
// their row index to S - 1, keys >= S get probability 0, rows >= S are not stored.
// DMASK (with a mask): the kernel also writes the mask gradient dS (trident/kernel/attention.py:332-335), each lane four
// consecutive keys of its row at a time; where the mask is broadcast over a dimension (dmask stride 0) the values are
// added to the caller's zero-filled fp32 buffer with atomic adds instead.
// DELTA (no mask): the kernel also computes delta = rowsum(dO * O) of its rows from the dO rows it loads anyway, instead
// of reading it, and stores it for the dK/dV pass, which then runs after this one (tri_attn_bwd_dq_delta).
template <typename T, int D, int NW, bool CAUSAL, int MASK, bool DROPOUT, bool RAGGED = false, bool DMASK = false, bool DELTA = false>
__global__ __launch_bounds__(NW * 64, 2) void mfma_dq_kernel(const KParams p) {
    static_assert(!RAGGED || (NW == 4 && MASK == 0), "ragged lengths: 4 waves, no mask");
    static_assert(!DMASK || MASK != 0, "a mask gradient needs a mask");
    static_assert(!DELTA || MASK == 0, "delta on the way: the variants without a mask");
    using Tile = SwzTile<D>;
    constexpr int kRows = 32 * NW;
    constexpr int kStages = 4;
    constexpr int kStageBytes = 2 * Tile::kBytes;  // K tile, V tile
    constexpr int KK = D / 16;
    constexpr int DB = D >= 32 ? D / 32 : 1;  // (D = 16: one block of gradient columns, the upper 16 are not stored)
    constexpr int kBlocksPerWave = 2 * Tile::kBlocks / NW;  // LDS-direct loads per wave and tile
    static_assert(2 * Tile::kBlocks % NW == 0, "tile blocks must divide among the waves");
    // A mask block of a wave (32 rows x 64 keys) goes through a private LDS region (8 KiB fp32, 4 KiB for a mask of
    // the operand type) when it fits (D = 64): lanes own rows, so direct loads would touch 32 cache lines per
    // instruction, while LDS-direct loads fetch whole rows. Geometry of a 32-row SwzTile<128> / SwzTile<64>.
    constexpr bool kMaskViaLds = MASK != kNoMask && D <= 64;  // (at D = 128 the 4 KiB regions of a 16-bit mask would fit, but the kernel then spills)
    constexpr int kMaskElt = MASK == kMaskF32 ? 4 : 2;
    using MaskTile = std::conditional_t<MASK == kMaskF32, SwzTile<128>, SwzTile<64>>;
    constexpr int kMaskBytes = 32 * MaskTile::kRowBytes;
    constexpr int kMaskLoads = kMaskBytes / 1024;
    __shared__ __attribute__((aligned(1024))) char smem[kStages * kStageBytes + (kMaskViaLds ? NW * kMaskBytes : 0)];

    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lane = tid & 63, l32 = lane & 31, h = lane >> 5;
    int bh, qt;
    map_block_for<MASK>(p, blockIdx.x, (p.S + kRows - 1) / kRows, CAUSAL ? kHeavyLast : kUniformTiles, &bh, &qt);
    const int b = bh / p.H, hd = bh % p.H;
    const int q0 = qt * kRows;
    const int wrow0 = q0 + 32 * wave;
    const int qrow = wrow0 + l32;
    const int qrow_ld = RAGGED ? min(qrow, p.S - 1) : qrow;  // (a row that does not exist reads the last one)

    const char* qrowp = static_cast<const char*>(p.q) + (b * p.qs[0] + hd * p.qs[1] + static_cast<int64_t>(qrow_ld) * p.qs[2]) * 2;
    const char* gorowp = static_cast<const char*>(p.d_o) + (b * p.dos[0] + hd * p.dos[1] + static_cast<int64_t>(qrow_ld) * p.dos[2]) * 2;
    const char* kbase = static_cast<const char*>(p.k) + (b * p.ks[0] + hd * p.ks[1]) * 2;
    const char* vbase = static_cast<const char*>(p.v) + (b * p.vs[0] + hd * p.vs[1]) * 2;
    const int64_t krow_bytes = p.ks[2] * 2, vrow_bytes = p.vs[2] * 2;

    u32x4 qf[KK], gf[KK];
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) {
        qf[kk] = *reinterpret_cast<const u32x4*>(qrowp + (2 * kk + h) * 16);
        gf[kk] = *reinterpret_cast<const u32x4*>(gorowp + (2 * kk + h) * 16);
    }
    float lse = p.lse[static_cast<int64_t>(bh) * p.S + qrow_ld];
    float dlt = 0.f;
    u32x4 of[DELTA ? KK : 1];
    if constexpr (DELTA) {
        // this lane holds half of its dO row (the other half is in lane ^ 32) and fetches the same half of the O row
        const char* orowp = static_cast<const char*>(p.o) + (b * p.os[0] + hd * p.os[1] + static_cast<int64_t>(qrow_ld) * p.os[2]) * 2;
#pragma unroll
        for (int kk = 0; kk < KK; ++kk) of[kk] = *reinterpret_cast<const u32x4*>(orowp + (2 * kk + h) * 16);
    } else {
        dlt = p.delta[static_cast<int64_t>(bh) * p.S + qrow_ld];
    }
    const float c = p.scale_log2;
    [[maybe_unused]] const float inv_scale = p.inv_scale;  // (a mask value joins its score before the scale: s + mask / scale)
    // Without dropout (and where the registers allow) the subtraction in dS = P (dP - delta) is left to the matrix pipe:
    // the dP^T accumulators start from delta and take the product with the dO rows negated, which gives delta - dP^T;
    // dS^T then comes out negated and the sign goes into the scale of the final store.
    constexpr bool kDeltaInAcc = !DROPOUT && !DMASK && D <= 64;

    f32x16 acc[DB];
#pragma unroll
    for (int db = 0; db < DB; ++db) acc[db] = zero16();

    const int num_key_tiles = (p.S + kBN - 1) / kBN;
    int n_tiles = CAUSAL ? min((q0 + kRows) / kBN, num_key_tiles) : num_key_tiles;  // tiles the workgroup streams
    int my_tiles = CAUSAL ? min((wrow0 + 31) / kBN + 1, n_tiles) : n_tiles;         // tiles with keys visible to this wave
    // With the classes of the mask's blocks at hand: key tiles behind the last one that is not masked out altogether
    // are not streamed, and tiles whose mask is all zero over the workgroup's rows are not read.
    uint64_t zero_tiles = 0;
    if constexpr (MASK != kNoMask) {
        if (p.mcls != nullptr && n_tiles <= 64) {
            const TileClasses tc = tile_classes(p.mcls + b * p.mcs[0] + hd * p.mcs[1] + (q0 / 64) * p.mcs[2], 1, n_tiles,
                                                kRows / 64, p.mcs[2], lane);
            zero_tiles = tc.zero;
            // (a mask gradient written in place covers every tile: the tiles behind the last active one get their
            // zeros from the loop; an accumulated one adds into a buffer the caller has zero-filled)
            if (!DMASK || p.dmask_acc) {
                n_tiles = tc.active ? 64 - __builtin_clzll(tc.active) : 1;
                my_tiles = n_tiles;
            }
        }
    }
    auto mask_is_zero = [&](int t) { return MASK != kNoMask && ((zero_tiles >> t) & 1) != 0; };

    int src_off[kBlocksPerWave];
#pragma unroll
    for (int i = 0; i < kBlocksPerWave; ++i) {
        const int blk = wave * kBlocksPerWave + i;  // 0 .. 2*kBlocks-1 over the K tile then the V tile
        const bool is_v = blk >= Tile::kBlocks;
        src_off[i] = static_cast<int>(Tile::src_off(is_v ? blk - Tile::kBlocks : blk, lane, is_v ? vrow_bytes : krow_bytes));
    }
    auto issue_tile = [&](int t) {
        char* stage = smem + (t % kStages) * kStageBytes;
#pragma unroll
        for (int i = 0; i < kBlocksPerWave; ++i) {
            const int blk = wave * kBlocksPerWave + i;
            const bool is_v = blk >= Tile::kBlocks;
            const char* tile_src = is_v ? vbase + static_cast<int64_t>(t) * kBN * vrow_bytes
                                        : kbase + static_cast<int64_t>(t) * kBN * krow_bytes;
            if (RAGGED && (t + 1) * kBN > p.S)  // the sequence ends inside this tile
                lds_direct_load16(tile_src, Tile::src_off_clamped(is_v ? blk - Tile::kBlocks : blk, lane, is_v ? vrow_bytes : krow_bytes,
                                                                  p.S - 1 - t * kBN), stage + blk * 1024);
            else
                lds_direct_load16(tile_src, src_off[i], stage + blk * 1024);
        }
    };
    char* mask_lds = smem + kStages * kStageBytes + wave * kMaskBytes;
    auto issue_mask = [&](int t) {  // mask block of tile t -> this wave's region, unless it is all zero
        if constexpr (kMaskViaLds) {
            if (mask_is_zero(t)) return;
            const char* src = static_cast<const char*>(p.mask) +
                              (b * p.ms[0] + hd * p.ms[1] + static_cast<int64_t>(wrow0) * p.ms[2] + t * kBN) * kMaskElt;
            int l = lane;
            asm volatile("" : "+v"(l));  // offsets recomputed per tile rather than kept in registers
#pragma unroll
            for (int blk = 0; blk < kMaskLoads; ++blk)
                lds_direct_load16(src, static_cast<uint32_t>(MaskTile::src_off(blk, l, p.ms[2] * kMaskElt)), mask_lds + blk * 1024);
        }
    };
    // issue order: mask 0, tiles 0 1 2, then per tile j: mask j+1, tile j+3
    issue_mask(0);
    issue_tile(0);
    if (1 < n_tiles) issue_tile(1);
    if (2 < n_tiles) issue_tile(2);
    // (the row fragments were requested before the tiles, so both latencies overlap)
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) {
        settle(qf[kk]);
        settle(gf[kk]);
    }
    settle(lse);
    if constexpr (DELTA) {
        float part = 0.f;
#pragma unroll
        for (int kk = 0; kk < KK; ++kk) {
            settle(of[kk]);
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                part = fmaf(Mma<T>::lo(of[kk][i]), Mma<T>::lo(gf[kk][i]), part);
                part = fmaf(Mma<T>::hi(of[kk][i]), Mma<T>::hi(gf[kk][i]), part);
            }
        }
        dlt = sum_xor32(part);
        if (h == 0 && (!RAGGED || qrow < p.S)) p.delta[static_cast<int64_t>(bh) * p.S + qrow] = dlt;
    } else {
        settle(dlt);
    }
    f32x16 dlt16;
    if constexpr (kDeltaInAcc) {
#pragma unroll
        for (int kk = 0; kk < KK; ++kk)
#pragma unroll
            for (int i = 0; i < 4; ++i) gf[kk][i] ^= 0x80008000u;
#pragma unroll
        for (int i = 0; i < 16; ++i) dlt16[i] = dlt;
        asm volatile("" : "+v"(dlt16));  // (kept in registers: as a splat it would be made anew for every block)
    }

    const int row_off0 = Tile::off(l32, h);
    const int tr_off0 = Tile::tr_off(0, 0, lane), tr_off1 = Tile::tr_off(0, 1, lane);

    for (int j = 0; j < n_tiles; ++j) {
        // tile j has landed (up to two younger tiles may still be in flight) and is visible to all
        // waves; every wave is done with tile j-1, whose slot takes the load of tile j+3
        {
            // with a staged mask, block j must have landed too: only tile j+2 was issued after it
            // (tiles 1 and 2 for j = 0)
            // (a block that is all zero was never requested: then the two youngest tiles are what may be in flight)
            const int younger = kMaskViaLds && j > 0 && !mask_is_zero(j) ? min(1, max(0, n_tiles - 2 - j)) : min(2, n_tiles - 1 - j);
            if (younger == 2) TRI_WAIT_VMCNT(2 * kBlocksPerWave);
            else if (younger == 1) TRI_WAIT_VMCNT(kBlocksPerWave);
            else TRI_WAIT_VMCNT(0);
        }
        lds_barrier();
        float mk2[kMaskViaLds ? 32 : 1];
        if constexpr (kMaskViaLds) {
            // (a mask excludes the causal variant, so every wave works on every tile)
            if (!mask_is_zero(j)) {  // (a tile whose mask is all zero takes the arithmetic of a tile without a mask)
#pragma unroll
                for (int g = 0; g < 8; ++g) {  // keys 8 g + 4 h .. + 3 of this lane's row
                    if constexpr (MASK == kMaskF32) {
                        const f32x4 v = *reinterpret_cast<const f32x4*>(mask_lds + MaskTile::off(l32, 2 * g + h));
                        mk2[4 * g + 0] = v.x; mk2[4 * g + 1] = v.y; mk2[4 * g + 2] = v.z; mk2[4 * g + 3] = v.w;
                    } else {
                        const u32x2 v = *reinterpret_cast<const u32x2*>(mask_lds + MaskTile::off(l32, g) + 8 * h);
                        mk2[4 * g + 0] = Mma<T>::lo(v.x); mk2[4 * g + 1] = Mma<T>::hi(v.x);
                        mk2[4 * g + 2] = Mma<T>::lo(v.y); mk2[4 * g + 3] = Mma<T>::hi(v.y);
                    }
                }
                asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // region read before it is refilled
            }
            if (j + 1 < n_tiles) issue_mask(j + 1);
        }
        if (j + 3 < n_tiles) issue_tile(j + 3);
        if (j >= my_tiles) continue;

        const char* sK = smem + (j % kStages) * kStageBytes;
        const char* sV = sK + Tile::kBytes;
        const int t0 = j * kBN;
        const bool diag = CAUSAL && t0 + kBN - 1 > wrow0;
#pragma unroll
        for (int kb = 0; kb < 2; ++kb) {
            float mk[MASK != kNoMask ? 16 : 1];
            // (at D = 128 the registers do not hold a second form of the arithmetic: a tile whose mask is all zero adds zeros)
            const bool masked = MASK != kNoMask && (D == 128 || !mask_is_zero(j));
            if constexpr (kMaskViaLds) {
                if (masked) {
#pragma unroll
                    for (int i = 0; i < 16; ++i) mk[i] = mk2[16 * kb + i];
                }
            } else if constexpr (MASK != kNoMask) {
                if (mask_is_zero(j)) {
#pragma unroll
                    for (int i = 0; i < 16; ++i) mk[i] = 0.f;
                } else {
                    const int64_t mrow = b * p.ms[0] + hd * p.ms[1] + static_cast<int64_t>(qrow) * p.ms[2] + t0 + 32 * kb;
#pragma unroll
                    for (int i = 0; i < 16; ++i) mk[i] = mask_at<T, MASK>(p.mask, mrow + c_row(i, h));
                }
            }
            u32x4 fr[KK];
#pragma unroll
            for (int kk = 0; kk < KK; ++kk) fr[kk] = lds_read16(sK, (row_off0 ^ (kk << 5)) + 32 * kb * Tile::kRowBytes);
            __builtin_amdgcn_sched_barrier(0);
            f32x16 st = zero16(), dpt = zero16();
            if constexpr (kDeltaInAcc) dpt = dlt16;
#pragma unroll
            for (int kk = 0; kk < KK; ++kk) {
                st = Mma<T>::run(fr[kk], qf[kk], st);
                fr[kk] = lds_read16(sV, (row_off0 ^ (kk << 5)) + 32 * kb * Tile::kRowBytes);
                __builtin_amdgcn_sched_barrier(0);
            }
#pragma unroll
            for (int kk = 0; kk < KK; ++kk) dpt = Mma<T>::run(fr[kk], gf[kk], dpt);
            // first transposed K fragments of this block: they arrive during the vector-ALU part
            u32x4 tf[2 * DB];
#pragma unroll
            for (int i = 0; i < 2 * DB; ++i)
                tf[i] = Tile::tr_frag(sK, tr_off0 ^ ((i % DB) << 6), tr_off1 ^ ((i % DB) << 6), 2 * kb + i / DB);
            __builtin_amdgcn_sched_barrier(0);
            if (diag && t0 + 32 * kb + 31 > wrow0) {  // a block that crosses the diagonal: scores above it drop out
                asm volatile("");                     // (a real branch: the other blocks skip the comparisons)
#pragma unroll
                for (int i = 0; i < 16; ++i) st[i] = t0 + 32 * kb + c_row(i, h) <= qrow ? st[i] : -INFINITY;
            }
            if (RAGGED && !CAUSAL && t0 + 32 * kb + 32 > p.S) {  // keys that do not exist
#pragma unroll
                for (int i = 0; i < 16; ++i) st[i] = t0 + 32 * kb + c_row(i, h) < p.S ? st[i] : -INFINITY;
            }
            float ds[16];
            if (masked) {
#pragma unroll
                for (int i = 0; i < 16; ++i) ds[i] = fast_exp2(fmaf(fmaf(mk[i], inv_scale, st[i]), c, -lse));  // (s + mask / scale, then the scale)
            } else {
#pragma unroll
                for (int i = 0; i < 16; ++i) ds[i] = fast_exp2(fmaf(st[i], c, -lse));
            }
            if constexpr (DROPOUT) {
                const Philox4 mine = dropout_block(p, bh, qrow >> 2, (t0 + 32 * kb + 8 * (lane & 3) + 4 * h) >> 2);
                uint32_t w[4];
                quad_row_words(mine, lane, w);
#pragma unroll
                for (int g = 0; g < 4; ++g)
#pragma unroll
                    for (int bb = 0; bb < 4; ++bb) {
                        const bool keep = static_cast<int>((w[g] >> (8 * bb)) & 0xffu) >= p.thr8;
                        dpt[4 * g + bb] = keep ? dpt[4 * g + bb] * p.zscale : 0.f;
                    }
            }
#pragma unroll
            for (int i = 0; i < 16; ++i) ds[i] *= kDeltaInAcc ? dpt[i] : dpt[i] - dlt;
            if constexpr (DMASK) {
                const int64_t at = b * p.dms[0] + hd * p.dms[1] + static_cast<int64_t>(qrow) * p.dms[2] + t0 + 32 * kb + 4 * h;
                if (p.dmask_acc) {
                    float* dst = static_cast<float*>(p.dmask) + at;
#pragma unroll
                    for (int i = 0; i < 16; ++i) unsafeAtomicAdd(dst + 8 * (i >> 2) + (i & 3), ds[i]);
                } else if constexpr (MASK == kMaskF32) {
#pragma unroll
                    for (int g = 0; g < 4; ++g)
                        *reinterpret_cast<f32x4*>(static_cast<float*>(p.dmask) + at + 8 * g) = f32x4{ds[4 * g], ds[4 * g + 1], ds[4 * g + 2], ds[4 * g + 3]};
                } else {
#pragma unroll
                    for (int g = 0; g < 4; ++g)
                        *reinterpret_cast<u32x2*>(static_cast<T*>(p.dmask) + at + 8 * g) =
                            u32x2{Mma<T>::pack2(ds[4 * g], ds[4 * g + 1]), Mma<T>::pack2(ds[4 * g + 2], ds[4 * g + 3])};
                }
            }
            u32x4 bop[2];
            bop[0] = pack8<T>(&ds[0]);
            bop[1] = pack8<T>(&ds[8]);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int i = 0; i < 2 * DB; ++i) acc[i % DB] = Mma<T>::run(tf[i], bop[i / DB], acc[i % DB]);
        }
    }

    // every wave is out of the loop: the ring can serve as the waves' private transposition patches
    lds_barrier();
    {
        using Store = RowBlockStore<T, DB, D < 32 ? D : 32 * DB>;
        static_assert(NW * Store::kPatchBytes <= kStages * kStageBytes, "patches must fit into the ring");
        char* out0 = static_cast<char*>(p.dq) + (b * p.dqs[0] + hd * p.dqs[1] + static_cast<int64_t>(wrow0) * p.dqs[2]) * 2;
        const float sc = kDeltaInAcc ? -p.scale : p.scale;
        Store::run(acc, [sc](float x) { return x * sc; }, smem + wave * Store::kPatchBytes, out0, p.dqs[2] * 2, lane,
                   RAGGED ? p.S - wrow0 : 32);
    }
}

// ------------------------------------------------------------------ dQ, phased (8 waves, no mask)
// Same data flow and tile ring as above, restructured so that the two waves of a SIMD (w and w+4)
// never do the same kind of work at once. Per 64-key tile a wave runs a vector phase (P and dS of the
// tile from its S^T and dP^T, packed as B operands) and a matrix phase (dQ^T += K^T dS^T of this
// tile, then S^T and dP^T of the next one: 6 D / 16 MFMAs through one ring of LDS fragments), with a
// workgroup barrier after each; waves 4-7 run one phase behind waves 0-3. Tile loads are issued at
// the top of the vector phase (two tiles ahead in waves 0-3, three in waves 4-7, which start their
// phase later) and awaited before its barrier.
// With DELTA the kernel also computes delta = rowsum(dO * O) of its rows (instead of reading it) and stores
// it for the dK/dV pass, which then has to run after this one: the separate pre-pass over O and dO
// (trident/kernel/softmax.py:180-238) disappears into the prologue that loads the dO rows anyway.
template <typename T, int D, bool CAUSAL, bool DROPOUT, bool DELTA>
__global__ __launch_bounds__(512, 2) void mfma_dq_phased_kernel(const KParams p) {
    using Tile = SwzTile<D>;
    constexpr int NW = 8;
    constexpr int kRows = 32 * NW;
    constexpr int kStages = 4;
    constexpr int kStageBytes = 2 * Tile::kBytes;  // K tile, V tile
    constexpr int KK = D / 16;
    constexpr int DB = D / 32;
    constexpr int kBlocksPerWave = 2 * Tile::kBlocks / NW;
    constexpr int kPerOperand = Tile::kBlocks / NW;
    constexpr int kRowStep = NW * Tile::kRowsPerBlock;
    static_assert(kRowStep % 16 == 0 && 2 * kPerOperand == kBlocksPerWave, "block assignment");
    constexpr int kDqSteps = 4 * DB;           // MFMAs of dQ^T per tile
    constexpr int kSteps = kDqSteps + 4 * KK;  // + S^T and dP^T of the next tile
    constexpr int kRing = D == 128 ? 4 : 6;  // (registers: with dropout the Philox state, without it the delta accumulators)
    static_assert(kRing <= kDqSteps, "the vector phase requests dQ fragments only");
    // The workgroup's Q and dO rows reach the registers through LDS as well: lanes own rows, so direct loads
    // touch 32 cache lines per instruction, while LDS-direct loads fetch whole rows. Each wave stages its
    // own 32 rows behind ring stage 0, which takes tile 0 meanwhile; tiles 1 and 2 follow once every wave
    // has its rows. The O rows (for delta) take the place of the Q rows in a second round (LDS has no room
    // for a third operand at once; fetching them by direct loads during the first round measured 1 %
    // slower). What remains of a workgroup's start is the latency of its first loads (about 6 000 cycles
    // for a single plain load).
    constexpr int kWaveRowBytes = 32 * Tile::kRowBytes;  // a wave's rows of one operand
    constexpr int kRowLoads = kWaveRowBytes / 1024;      // LDS-direct loads per wave and operand
    __shared__ __attribute__((aligned(1024))) char smem[kStageBytes + 2 * NW * kWaveRowBytes];
    static_assert(kStageBytes + 2 * NW * kWaveRowBytes >= kStages * kStageBytes, "the ring lies inside");

    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lane = tid & 63, l32 = lane & 31, h = lane >> 5;
    int bh, qt;
    map_block(blockIdx.x, p.B * p.H, p.S / kRows, CAUSAL ? kHeavyLast : kUniformTiles, &bh, &qt);
    const int b = bh / p.H, hd = bh % p.H;
    const int q0 = qt * kRows;
    const int wrow0 = q0 + 32 * wave;
    const int qrow = wrow0 + l32;

    const char* qrows = static_cast<const char*>(p.q) + (b * p.qs[0] + hd * p.qs[1] + static_cast<int64_t>(wrow0) * p.qs[2]) * 2;
    const char* gorows = static_cast<const char*>(p.d_o) + (b * p.dos[0] + hd * p.dos[1] + static_cast<int64_t>(wrow0) * p.dos[2]) * 2;
    const char* kbase = static_cast<const char*>(p.k) + (b * p.ks[0] + hd * p.ks[1]) * 2;
    const char* vbase = static_cast<const char*>(p.v) + (b * p.vs[0] + hd * p.vs[1]) * 2;
    const int64_t krow_bytes = p.ks[2] * 2, vrow_bytes = p.vs[2] * 2;

    float lse = p.lse[static_cast<int64_t>(bh) * p.S + qrow];
    float dlt = 0.f;
    if constexpr (!DELTA) dlt = p.delta[static_cast<int64_t>(bh) * p.S + qrow];
    char* q_stage = smem + kStageBytes + wave * kWaveRowBytes;
    char* g_stage = q_stage + NW * kWaveRowBytes;
#pragma unroll
    for (int blk = 0; blk < kRowLoads; ++blk)
        lds_direct_load16(qrows, static_cast<uint32_t>(Tile::src_off(blk, lane, p.qs[2] * 2)), q_stage + blk * 1024);
#pragma unroll
    for (int blk = 0; blk < kRowLoads; ++blk)
        lds_direct_load16(gorows, static_cast<uint32_t>(Tile::src_off(blk, lane, p.dos[2] * 2)), g_stage + blk * 1024);
    const float c = p.scale_log2;
    [[maybe_unused]] const float inv_scale = p.inv_scale;  // (a mask value joins its score before the scale: s + mask / scale)

    f32x16 acc[DB];
#pragma unroll
    for (int db = 0; db < DB; ++db) acc[db] = zero16();

    const int n_tiles = CAUSAL ? (q0 + kRows) / kBN : p.S / kBN;     // tiles the workgroup streams
    const int my_tiles = CAUSAL ? (wrow0 + 31) / kBN + 1 : n_tiles;  // tiles with keys visible to this wave

    // A wave fetches blocks wave, wave + NW, ... of the K tile and of the V tile: their rows are a
    // multiple of 16 apart, so one per-lane source offset serves all of them.
    const uint32_t koff = static_cast<uint32_t>(Tile::src_off(wave, lane, krow_bytes));
    const uint32_t voff = static_cast<uint32_t>(Tile::src_off(wave, lane, vrow_bytes));
    auto issue_tile = [&](int t) {
        char* stage = smem + (t % kStages) * kStageBytes + wave * 1024;
#pragma unroll
        for (int i = 0; i < kPerOperand; ++i)
            lds_direct_load16(kbase + (static_cast<int64_t>(t) * kBN + i * kRowStep) * krow_bytes, koff, stage + i * NW * 1024);
#pragma unroll
        for (int i = 0; i < kPerOperand; ++i)
            lds_direct_load16(vbase + (static_cast<int64_t>(t) * kBN + i * kRowStep) * vrow_bytes, voff,
                              stage + Tile::kBytes + i * NW * 1024);
    };
    const int group = wave >> 2;
    const int dist = 2 + group;
    const int n_first = min(dist, n_tiles);
    issue_tile(0);

    const int row_off0 = Tile::off(l32, h);
    TRI_WAIT_VMCNT(kBlocksPerWave);  // this wave's Q and dO rows have landed (tile 0 may be on its way)
    asm volatile("" ::: "memory");
    u32x4 qf[KK], gf[KK];
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) {
        qf[kk] = lds_read16(q_stage, row_off0 ^ (kk << 5));
        gf[kk] = lds_read16(g_stage, row_off0 ^ (kk << 5));
    }
    if constexpr (DELTA) {
        // the O rows follow into the place of the Q rows; this lane holds half of its row (the other half is
        // in lane ^ 32)
        const char* orows = static_cast<const char*>(p.o) + (b * p.os[0] + hd * p.os[1] + static_cast<int64_t>(wrow0) * p.os[2]) * 2;
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // the Q rows are in registers
#pragma unroll
        for (int blk = 0; blk < kRowLoads; ++blk)
            lds_direct_load16(orows, static_cast<uint32_t>(Tile::src_off(blk, lane, p.os[2] * 2)), q_stage + blk * 1024);
        TRI_WAIT_VMCNT(0);
        asm volatile("" ::: "memory");
        float part = 0.f;
#pragma unroll
        for (int kk = 0; kk < KK; ++kk) {
            const u32x4 of = lds_read16(q_stage, row_off0 ^ (kk << 5));
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                part = fmaf(Mma<T>::lo(of[i]), Mma<T>::lo(gf[kk][i]), part);
                part = fmaf(Mma<T>::hi(of[i]), Mma<T>::hi(gf[kk][i]), part);
            }
        }
        dlt = sum_xor32(part);
        if (h == 0) p.delta[static_cast<int64_t>(bh) * p.S + qrow] = dlt;
    }

    // Without dropout the subtraction in dS = P (dP - delta) is left to the matrix pipe: the dP^T accumulators start from
    // delta and take the product with the dO rows negated (delta - dP^T); dS^T comes out negated and the sign goes into
    // the scale of the final store.
    constexpr bool kDeltaInAcc = !DROPOUT;
    f32x16 dlt16;
    if constexpr (kDeltaInAcc) {
#pragma unroll
        for (int kk = 0; kk < KK; ++kk)
#pragma unroll
            for (int i = 0; i < 4; ++i) gf[kk][i] ^= 0x80008000u;
#pragma unroll
        for (int i = 0; i < 16; ++i) dlt16[i] = dlt;
        asm volatile("" : "+v"(dlt16));  // (kept in registers: as a splat it would be made anew for every tile)
    }
    const int tr_off0 = Tile::tr_off(0, 0, lane), tr_off1 = Tile::tr_off(0, 1, lane);

    // fragment n of the matrix phase of tile t: n < kDqSteps: K^T of tile t (column block n % DB, K-step
    // n / DB); then the K rows (key block 0, 1) and the V rows (key block 0, 1) of tile t + 1
    auto frag = [&](int t, int n) {
        if (n < kDqSteps) {
            const char* sK = smem + ((t + kStages) % kStages) * kStageBytes;
            return Tile::tr_frag(sK, tr_off0 ^ ((n % DB) << 6), tr_off1 ^ ((n % DB) << 6), n / DB);
        }
        const int m = n - kDqSteps;
        const char* sT = smem + ((t + 1) % kStages) * kStageBytes + (m < 2 * KK ? 0 : Tile::kBytes);
        return lds_read16(sT, (row_off0 ^ ((m % KK) << 5)) + 32 * ((m / KK) & 1) * Tile::kRowBytes);
    };
    f32x16 st[2], dpt[2];  // S^T and dP^T of the current tile (two key blocks)
    u32x4 bop[4];          // dS^T of the current tile as B operands
    u32x4 ring[kRing];
    auto matrix_phase = [&](auto with_dq, int t, bool with_scores = true) {
        constexpr int first = decltype(with_dq)::value ? 0 : kDqSteps;
        f32x16 s_new[2] = {zero16(), zero16()}, dp_new[2] = {zero16(), zero16()};
        if constexpr (kDeltaInAcc) {
            dp_new[0] = dlt16;
            dp_new[1] = dlt16;
        }
#pragma unroll
        for (int n = first; n < kSteps; ++n) {
            if (n >= kDqSteps && !with_scores) break;
            const int slot = (n - first) % kRing;
            const int m = n - kDqSteps;
            if (n < kDqSteps) acc[n % DB] = Mma<T>::run(ring[slot], bop[n / DB], acc[n % DB]);
            else if (m < 2 * KK) s_new[m / KK] = Mma<T>::run(ring[slot], qf[m % KK], s_new[m / KK]);
            else dp_new[(m / KK) & 1] = Mma<T>::run(ring[slot], gf[m % KK], dp_new[(m / KK) & 1]);
            if (n + kRing < kSteps) ring[slot] = frag(t, n + kRing);
            __builtin_amdgcn_sched_barrier(0);
        }
        st[0] = s_new[0]; st[1] = s_new[1];
        dpt[0] = dp_new[0]; dpt[1] = dp_new[1];
    };
    using Yes = std::integral_constant<bool, true>;
    using No = std::integral_constant<bool, false>;
    auto wait_tile = [&](bool newest_in_flight) {
        if (newest_in_flight) TRI_WAIT_VMCNT(kBlocksPerWave);
        else TRI_WAIT_VMCNT(0);
    };

    // tile 0 has landed and is visible to all waves, and every wave has its rows in registers: the staging
    // area returns to the ring
    TRI_WAIT_VMCNT(0);
    settle(lse);
    if constexpr (!DELTA) settle(dlt);
    lds_barrier();
    if (n_first > 1) issue_tile(1);
    if (n_first > 2) issue_tile(2);
    if (group == 1) {
        // group 1 starts one phase late; group 0 reads tile 1 in its first matrix phase
        if (n_first == 3) TRI_WAIT_VMCNT(kBlocksPerWave);
        else TRI_WAIT_VMCNT(0);
        lds_barrier();
    }
    {
#pragma unroll
        for (int r = 0; r < kRing; ++r) ring[r] = frag(-1, kDqSteps + r);
        __builtin_amdgcn_sched_barrier(0);
        matrix_phase(No{}, -1);
    }

    for (int t = 0; t < my_tiles; ++t) {
        const bool issued = t + dist < n_tiles;
        if (issued) issue_tile(t + dist);
        // ---- vector phase: P and dS of the tile (only 32-key blocks that cross the diagonal pay for the
        // causal comparison)
        auto softmax_backward = [&](auto on_diagonal, int kb) {
            const int key0 = t * kBN + 32 * kb;
            float ds[16];
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                float pr = fast_exp2(fmaf(st[kb][i], c, -lse));
                if constexpr (decltype(on_diagonal)::value) pr = key0 + c_row(i, h) <= qrow ? pr : 0.f;
                ds[i] = pr;
            }
            f32x16 dpv = dpt[kb];
            if constexpr (DROPOUT) {
                const Philox4 mine = dropout_block(p, bh, qrow >> 2, (key0 + 8 * (lane & 3) + 4 * h) >> 2);
                uint32_t w[4];
                quad_row_words(mine, lane, w);
#pragma unroll
                for (int g = 0; g < 4; ++g)
#pragma unroll
                    for (int bb = 0; bb < 4; ++bb) {
                        const bool keep = static_cast<int>((w[g] >> (8 * bb)) & 0xffu) >= p.thr8;
                        dpv[4 * g + bb] = keep ? dpv[4 * g + bb] * p.zscale : 0.f;
                    }
            }
#pragma unroll
            for (int i = 0; i < 16; ++i) ds[i] *= kDeltaInAcc ? dpv[i] : dpv[i] - dlt;
            bop[2 * kb + 0] = pack8<T>(&ds[0]);
            bop[2 * kb + 1] = pack8<T>(&ds[8]);
        };
#pragma unroll
        for (int kb = 0; kb < 2; ++kb) {
            if (CAUSAL && t * kBN + 32 * kb + 31 > wrow0) softmax_backward(Yes{}, kb);
            else softmax_backward(No{}, kb);
        }
        // the first fragments of the matrix phase (K^T of this tile, visible since the previous barrier)
#pragma unroll
        for (int r = 0; r < kRing; ++r) ring[r] = frag(t, r);
        // tile t + dist - 1 has landed (the newest one may still be in flight); after the barrier it is
        // visible to every wave, and the partner group changes phase
        wait_tile(issued);
        __builtin_amdgcn_sched_barrier(0);
        asm volatile("s_barrier" ::: "memory");
        __builtin_amdgcn_sched_barrier(0);
        // ---- matrix phase (a wave's last tile has no successor to score; the dropout variant runs the S^T /
        // dP^T steps all the same, on whatever the next slot holds: leaving them out costs it registers it does
        // not have, and the result is never used)
        __builtin_amdgcn_s_setprio(2);
        matrix_phase(Yes{}, t, DROPOUT || t + 1 < my_tiles);
        __builtin_amdgcn_s_setprio(0);
        __builtin_amdgcn_sched_barrier(0);
        lds_barrier();
        __builtin_amdgcn_sched_barrier(0);
    }
    // afterwards a wave only keeps fetching its share of the remaining tiles and meeting the barriers
    for (int t = my_tiles; t < n_tiles; ++t) {
        const bool issued = t + dist < n_tiles;
        if (issued) issue_tile(t + dist);
        wait_tile(issued);
        lds_barrier();
        lds_barrier();
    }
    if (group == 0) lds_barrier();  // group 1 is still in its last matrix phase

    // every wave is out of the loop: the ring can serve as the waves' private transposition patches
    lds_barrier();
    {
        using Store = RowBlockStore<T, DB>;
        static_assert(NW * Store::kPatchBytes <= kStages * kStageBytes, "patches must fit into the ring");
        char* out0 = static_cast<char*>(p.dq) + (b * p.dqs[0] + hd * p.dqs[1] + static_cast<int64_t>(wrow0) * p.dqs[2]) * 2;
        const float sc = kDeltaInAcc ? -p.scale : p.scale;
        // the lane index taken afresh: the epilogue's per-lane offsets are then computed here instead of being
        // kept (or, with every register in use, spilled) across the loop
        int elane = threadIdx.x & 63;
        asm volatile("" : "+v"(elane));
        Store::run(acc, [sc](float x) { return x * sc; }, smem + wave * Store::kPatchBytes, out0, p.dqs[2] * 2, elane);
    }
}

// ------------------------------------------------------------------ dK, dV (8 waves)
// Same data flow as the dQ kernel with the roles of queries and keys exchanged: a workgroup of
// NW waves owns 32*NW keys, one wave 32 of them with its K and V rows in registers (B operands)
// and dK^T, dV^T in fp32 accumulators; two waves per SIMD. Q and dO stream as 64-row swizzled LDS
// tiles (plus their lse and delta) in a ring of 4 filled by LDS-direct loads three tiles ahead.
// Per 32-row query block: S = Q K^T and dP = dO V^T from row fragments, P and dS on the vector
// ALU, dV^T += dO^T P and dK^T += Q^T dS with the transposed LDS reads of the same tiles.
// RAGGED (4 waves, no mask; also serves D = 128, one workgroup per CU): S is not a multiple of 128. Loads clamp their
// row index to S - 1, query rows >= S get probability 0 (they would otherwise add the last row once more), keys >= S
// are not stored.
template <typename T, int D, int NW, bool CAUSAL, int MASK, bool DROPOUT, bool RAGGED = false>
__global__ __launch_bounds__(NW * 64, RAGGED ? 1 : 2) void mfma_dkdv_wide_kernel(const KParams p) {
    static_assert(!RAGGED || (NW == 4 && MASK == 0), "ragged lengths: 4 waves, no mask");
    using Tile = SwzTile<D>;
    constexpr int kKeys = 32 * NW;
    constexpr int kStages = 4;
    constexpr int kStageBytes = 2 * Tile::kBytes + 2 * kBN * 4;  // Q tile, dO tile, lse, delta
    constexpr int KK = D / 16;
    constexpr int DB = D >= 32 ? D / 32 : 1;  // (D = 16: one block of gradient columns, the upper 16 are not stored)
    constexpr int kBlocksPerWave = 2 * Tile::kBlocks / NW;
    constexpr int kLoadsPerTile = kBlocksPerWave + 1;            // + lse or delta: exact for every wave
    static_assert(2 * Tile::kBlocks % NW == 0, "tile blocks must divide among the waves");
    // A mask block of a wave (64 rows x its 32 keys) goes through a private LDS region (8 KiB fp32, 4 KiB for a mask
    // of the operand type) when it fits (D = 64). Plain loads would be tracked by the compiler, whose waits for them
    // also drain the LDS-direct tile loads issued in between (the counter completes in order), which makes the
    // tile prefetch synchronous. Geometry of a 64-row SwzTile<64> / SwzTile<32> (128- or 64-byte rows = 32 keys).
    constexpr bool kMaskViaLds = MASK != kNoMask && D <= 64;
    constexpr int kMaskElt = MASK == kMaskF32 ? 4 : 2;
    using MaskTile = std::conditional_t<MASK == kMaskF32, SwzTile<64>, SwzTile<32>>;
    constexpr int kMaskLoads = MaskTile::kBlocks;
    __shared__ __attribute__((aligned(1024))) char smem[kStages * kStageBytes + (kMaskViaLds ? NW * MaskTile::kBytes : 0)];

    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lane = tid & 63, l32 = lane & 31, h = lane >> 5;
    int bh, kt;
    map_block_for<MASK>(p, blockIdx.x, (p.S + kKeys - 1) / kKeys, CAUSAL ? kHeavyFirst : kUniformTiles, &bh, &kt);
    const int b = bh / p.H, hd = bh % p.H;
    const int k0 = kt * kKeys;
    const int wkey0 = k0 + 32 * wave;
    const int key = wkey0 + l32;
    const int key_ld = RAGGED ? min(key, p.S - 1) : key;  // (a key that does not exist reads the last one)

    const char* kbase = static_cast<const char*>(p.k) + (b * p.ks[0] + hd * p.ks[1]) * 2;
    const char* vbase = static_cast<const char*>(p.v) + (b * p.vs[0] + hd * p.vs[1]) * 2;
    const char* qbase = static_cast<const char*>(p.q) + (b * p.qs[0] + hd * p.qs[1]) * 2;
    const char* gbase = static_cast<const char*>(p.d_o) + (b * p.dos[0] + hd * p.dos[1]) * 2;
    const int64_t qrow_bytes = p.qs[2] * 2, grow_bytes = p.dos[2] * 2;
    const float* lse_base = p.lse + static_cast<int64_t>(bh) * p.S;
    const float* delta_base = p.delta + static_cast<int64_t>(bh) * p.S;

    u32x4 kf[KK], vf[KK];
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) {
        kf[kk] = *reinterpret_cast<const u32x4*>(kbase + static_cast<int64_t>(key_ld) * p.ks[2] * 2 + (2 * kk + h) * 16);
        vf[kk] = *reinterpret_cast<const u32x4*>(vbase + static_cast<int64_t>(key_ld) * p.vs[2] * 2 + (2 * kk + h) * 16);
    }
    const float c = p.scale_log2;
    [[maybe_unused]] const float inv_scale = p.inv_scale;  // (a mask value joins its score before the scale: s + mask / scale)
    // Without dropout the subtraction in dS = P (dP - delta) is left to the matrix pipe: the dP accumulators start from
    // the rows' delta values (as they come from the tile: the accumulator's layout) and take the product with the V
    // fragments negated, which gives delta - dP; dS then comes out negated and the sign goes into dK's final scale.
    constexpr bool kDeltaInAcc = !DROPOUT;

    f32x16 dk[DB], dv[DB];
#pragma unroll
    for (int db = 0; db < DB; ++db) {
        dk[db] = zero16();
        dv[db] = zero16();
    }

    int src_off[kBlocksPerWave];
#pragma unroll
    for (int i = 0; i < kBlocksPerWave; ++i) {
        const int blk = wave * kBlocksPerWave + i;
        const bool is_g = blk >= Tile::kBlocks;
        src_off[i] = static_cast<int>(Tile::src_off(is_g ? blk - Tile::kBlocks : blk, lane, is_g ? grow_bytes : qrow_bytes));
    }
    int t_begin = CAUSAL ? k0 / kBN : 0;                        // first tile with rows that see the workgroup's keys
    const int my_begin = CAUSAL ? wkey0 / kBN : 0;              // first tile with rows that see this wave's keys
    int n_tiles = (p.S + kBN - 1) / kBN;
    // With the classes of the mask's blocks at hand: row tiles before the first and behind the last one that is not
    // masked out altogether over the workgroup's keys are not streamed (keys beyond every length: nothing at all, the
    // gradients are zero), and tiles whose mask is all zero over the workgroup's keys are not read.
    uint64_t zero_tiles = 0;
    if constexpr (MASK != kNoMask) {
        if (p.mcls != nullptr && n_tiles <= 64) {
            const TileClasses tc = tile_classes(p.mcls + b * p.mcs[0] + hd * p.mcs[1] + k0 / 64, p.mcs[2], n_tiles, kKeys / 64, 1, lane);
            zero_tiles = tc.zero;
            if (tc.active) {
                t_begin = __builtin_ctzll(tc.active);
                n_tiles = 64 - __builtin_clzll(tc.active);
            } else {
                n_tiles = 0;
            }
        }
    }
    auto mask_is_zero = [&](int t) { return MASK != kNoMask && ((zero_tiles >> t) & 1) != 0; };
    auto issue_tile = [&](int t) {
        char* stage = smem + (t % kStages) * kStageBytes;
        const bool partial = RAGGED && (t + 1) * kBN > p.S;  // the sequence ends inside this tile
        const int last = p.S - 1 - t * kBN;
#pragma unroll
        for (int i = 0; i < kBlocksPerWave; ++i) {
            const int blk = wave * kBlocksPerWave + i;
            const bool is_g = blk >= Tile::kBlocks;
            const char* tile_src = is_g ? gbase + static_cast<int64_t>(t) * kBN * grow_bytes
                                        : qbase + static_cast<int64_t>(t) * kBN * qrow_bytes;
            char* dst = stage + (is_g ? Tile::kBytes + (blk - Tile::kBlocks) * 1024 : blk * 1024);
            if (partial)
                lds_direct_load16(tile_src, Tile::src_off_clamped(is_g ? blk - Tile::kBlocks : blk, lane, is_g ? grow_bytes : qrow_bytes, last), dst);
            else
                lds_direct_load16(tile_src, src_off[i], dst);
        }
        // every wave issues exactly one more load, so that the vmcnt bookkeeping is the same in all of
        // them: even waves fetch the 64 lse values, odd waves the 64 delta values (duplicates land
        // on the same bytes)
        const int aux = (partial ? min(lane, last) : lane) * 4;
        if (wave & 1) lds_direct_load4(delta_base + t * kBN, aux, stage + 2 * Tile::kBytes + kBN * 4);
        else lds_direct_load4(lse_base + t * kBN, aux, stage + 2 * Tile::kBytes);
    };
    char* mask_lds = smem + kStages * kStageBytes + wave * MaskTile::kBytes;
    auto issue_mask = [&](int t) {  // rows of tile t x this wave's keys -> the wave's region, unless the tile is all zero
        if constexpr (kMaskViaLds) {
            if (mask_is_zero(t)) return;
            const char* src = static_cast<const char*>(p.mask) +
                              (b * p.ms[0] + hd * p.ms[1] + static_cast<int64_t>(t) * kBN * p.ms[2] + wkey0) * kMaskElt;
            int l = lane;
            asm volatile("" : "+v"(l));  // offsets recomputed per tile rather than kept in registers
#pragma unroll
            for (int blk = 0; blk < kMaskLoads; ++blk)
                lds_direct_load16(src, static_cast<uint32_t>(MaskTile::src_off(blk, l, p.ms[2] * kMaskElt)), mask_lds + blk * 1024);
        }
    };
    // issue order: mask block of the first tile, three tiles, then per tile j: mask j+1, tile j+3
    if (t_begin < n_tiles) {
        issue_mask(t_begin);
        issue_tile(t_begin);
    }
    if (t_begin + 1 < n_tiles) issue_tile(t_begin + 1);
    if (t_begin + 2 < n_tiles) issue_tile(t_begin + 2);
    // (the K and V fragments were requested before the tiles, so both latencies overlap)
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) {
        settle(kf[kk]);
        settle(vf[kk]);
        if constexpr (kDeltaInAcc) {
#pragma unroll
            for (int i = 0; i < 4; ++i) vf[kk][i] ^= 0x80008000u;
        }
    }

    const int row_off0 = Tile::off(l32, h);
    const int tr_off0 = Tile::tr_off(0, 0, lane), tr_off1 = Tile::tr_off(0, 1, lane);

    for (int j = t_begin; j < n_tiles; ++j) {
        {
            // with a staged mask, block j must have landed too: only tile j+2 was issued after it
            // (two tiles after the first block)
            // (a block that is all zero was never requested: then the two youngest tiles are what may be in flight)
            const int younger = kMaskViaLds && j > t_begin && !mask_is_zero(j) ? min(1, max(0, n_tiles - 2 - j)) : min(2, n_tiles - 1 - j);
            if (younger == 2) TRI_WAIT_VMCNT(2 * kLoadsPerTile);
            else if (younger == 1) TRI_WAIT_VMCNT(kLoadsPerTile);
            else TRI_WAIT_VMCNT(0);
        }
        lds_barrier();
        float mk2[kMaskViaLds ? 32 : 1];
        if constexpr (kMaskViaLds) {
            // (a mask excludes the causal variant, so every wave works on every tile)
            if (!mask_is_zero(j)) {  // (a tile whose mask is all zero takes the arithmetic of a tile without a mask)
#pragma unroll
                for (int i = 0; i < 32; ++i) {  // row 32 (i / 16) + c_row(i % 16, h), this lane's key
                    const int row = 32 * (i >> 4) + c_row(i & 15, h);
                    if constexpr (MASK == kMaskF32)
                        mk2[i] = *reinterpret_cast<const float*>(mask_lds + MaskTile::off(row, l32 >> 2) + (l32 & 3) * 4);
                    else
                        mk2[i] = to_f32(*reinterpret_cast<const T*>(mask_lds + MaskTile::off(row, l32 >> 3) + (l32 & 7) * 2));
                }
                asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // region read before it is refilled
            }
            if (j + 1 < n_tiles) issue_mask(j + 1);
        }
        if (j + 3 < n_tiles) issue_tile(j + 3);
        if (j < my_begin) continue;

        const char* sQ = smem + (j % kStages) * kStageBytes;
        const char* sG = sQ + Tile::kBytes;
        const float* sLse = reinterpret_cast<const float*>(sG + Tile::kBytes);
        const float* sDelta = sLse + kBN;
        const int r0 = j * kBN;
        const bool diag = CAUSAL && r0 < wkey0 + 31;  // some row of the tile is above some key of the wave
#pragma unroll 1
        for (int qb = 0; qb < 2; ++qb) {
            const int rb = r0 + 32 * qb;
            if (CAUSAL && rb + 31 < wkey0) continue;  // whole block above the wave's keys
            float mk[MASK != kNoMask ? 16 : 1];
            const bool masked = MASK != kNoMask && !mask_is_zero(j);
            if constexpr (kMaskViaLds) {
                if (masked) {
#pragma unroll
                    for (int i = 0; i < 16; ++i) mk[i] = qb ? mk2[16 + i] : mk2[i];  // static indices keep it in registers
                }
            } else if constexpr (MASK != kNoMask) {
                if (masked) {
                    const int64_t mbase = b * p.ms[0] + hd * p.ms[1] + key;
#pragma unroll
                    for (int i = 0; i < 16; ++i)
                        mk[i] = mask_at<T, MASK>(p.mask, mbase + static_cast<int64_t>(rb + c_row(i, h)) * p.ms[2]);
                }
            }
            const int qoff = 32 * qb * Tile::kRowBytes;
            u32x4 fr[KK];
#pragma unroll
            for (int kk = 0; kk < KK; ++kk) fr[kk] = lds_read16(sQ, (row_off0 ^ (kk << 5)) + qoff);
            __builtin_amdgcn_sched_barrier(0);
            f32x16 s = zero16(), dp = zero16();
            if constexpr (kDeltaInAcc) {
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    const f32x4 d4 = *reinterpret_cast<const f32x4*>(sDelta + 32 * qb + 8 * g + 4 * h);
                    dp[4 * g + 0] = d4.x; dp[4 * g + 1] = d4.y; dp[4 * g + 2] = d4.z; dp[4 * g + 3] = d4.w;
                }
            }
#pragma unroll
            for (int kk = 0; kk < KK; ++kk) {
                s = Mma<T>::run(fr[kk], kf[kk], s);
                fr[kk] = lds_read16(sG, (row_off0 ^ (kk << 5)) + qoff);
                __builtin_amdgcn_sched_barrier(0);
            }
#pragma unroll
            for (int kk = 0; kk < KK; ++kk) dp = Mma<T>::run(fr[kk], vf[kk], dp);
            __builtin_amdgcn_sched_barrier(0);
            if (diag && rb < wkey0 + 31) {  // a block that crosses the diagonal: scores above it drop out
                asm volatile("");           // (a real branch: the other blocks skip the comparisons)
#pragma unroll
                for (int i = 0; i < 16; ++i) s[i] = key <= rb + c_row(i, h) ? s[i] : -INFINITY;
            }
            if (RAGGED && rb + 32 > p.S) {  // query rows that do not exist contribute nothing
#pragma unroll
                for (int i = 0; i < 16; ++i) s[i] = rb + c_row(i, h) < p.S ? s[i] : -INFINITY;
            }
            u32x4 pb[2], sb[2];
            {
                float pr[16], ds[16];
                // the probabilities first: with the mask's values, or as in a tile without a mask where they are all zero
                float pexp[16];
                if (masked) {
#pragma unroll
                    for (int g = 0; g < 4; ++g) {
                        const f32x4 l4 = *reinterpret_cast<const f32x4*>(sLse + 32 * qb + 8 * g + 4 * h);
#pragma unroll
                        for (int bb = 0; bb < 4; ++bb) pexp[4 * g + bb] = fast_exp2(fmaf(fmaf(mk[4 * g + bb], inv_scale, s[4 * g + bb]), c, -l4[bb]));
                    }
                } else {
#pragma unroll
                    for (int g = 0; g < 4; ++g) {
                        const f32x4 l4 = *reinterpret_cast<const f32x4*>(sLse + 32 * qb + 8 * g + 4 * h);
#pragma unroll
                        for (int bb = 0; bb < 4; ++bb) pexp[4 * g + bb] = fast_exp2(fmaf(s[4 * g + bb], c, -l4[bb]));
                    }
                }
                Philox4 mine;  // the block of rows rb + 8 (lane % 4) + 4 h .. +3: this lane's share of the quad's four
                if constexpr (DROPOUT) mine = dropout_block(p, bh, (rb + 8 * (lane & 3) + 4 * h) >> 2, key >> 2);
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    f32x4 d4 = {0.f, 0.f, 0.f, 0.f};
                    if constexpr (!kDeltaInAcc) d4 = *reinterpret_cast<const f32x4*>(sDelta + 32 * qb + 8 * g + 4 * h);
                    uint32_t dw[4];
                    if constexpr (DROPOUT) {
                        const Philox4 r = quad_bcast_from(g, mine);  // lane g of the quad generated rows rb + 8 g + 4 h .. +3
#pragma unroll
                        for (int bb = 0; bb < 4; ++bb) dw[bb] = (r.w[bb] >> (8 * (key & 3))) & 0xffu;
                    }
#pragma unroll
                    for (int bb = 0; bb < 4; ++bb) {
                        const int i = 4 * g + bb;
                        const float pv = pexp[i];
                        float dpv = dp[i];
                        if constexpr (DROPOUT) {
                            const bool keep = static_cast<int>(dw[bb]) >= p.thr8;
                            dpv = keep ? dpv * p.zscale : 0.f;
                            pr[i] = keep ? pv * p.zscale : 0.f;
                        } else {
                            pr[i] = pv;
                        }
                        ds[i] = kDeltaInAcc ? pv * dpv : pv * (dpv - d4[bb]);
                    }
                }
#pragma unroll
                for (int g = 0; g < 2; ++g) {
                    pb[g] = pack8<T>(&pr[8 * g]);
                    sb[g] = pack8<T>(&ds[8 * g]);
                }
            }
            __builtin_amdgcn_sched_barrier(0);
            // dV^T += dO^T P, then dK^T += Q^T dS; DB transposed fragments in flight
#pragma unroll
            for (int g = 0; g < 2; ++g) {
                u32x4 tf[DB];
#pragma unroll
                for (int db = 0; db < DB; ++db) tf[db] = Tile::tr_frag(sG, tr_off0 ^ (db << 6), tr_off1 ^ (db << 6), 2 * qb + g);
#pragma unroll
                for (int db = 0; db < DB; ++db) {
                    dv[db] = Mma<T>::run(tf[db], pb[g], dv[db]);
                    tf[db] = Tile::tr_frag(sQ, tr_off0 ^ (db << 6), tr_off1 ^ (db << 6), 2 * qb + g);
                }
#pragma unroll
                for (int db = 0; db < DB; ++db) dk[db] = Mma<T>::run(tf[db], sb[g], dk[db]);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
    }

    // every wave is out of the loop: the ring can serve as the waves' private transposition patches
    lds_barrier();
    {
        using Store = RowBlockStore<T, DB, D < 32 ? D : 32 * DB>;
        static_assert(NW * Store::kPatchBytes <= kStages * kStageBytes, "patches must fit into the ring");
        char* patch = smem + wave * Store::kPatchBytes;
        char* dk0 = static_cast<char*>(p.dk) + (b * p.dks[0] + hd * p.dks[1] + static_cast<int64_t>(wkey0) * p.dks[2]) * 2;
        char* dv0 = static_cast<char*>(p.dv) + (b * p.dvs[0] + hd * p.dvs[1] + static_cast<int64_t>(wkey0) * p.dvs[2]) * 2;
        const float sc = kDeltaInAcc ? -p.scale : p.scale;
        const int keys_here = RAGGED ? p.S - wkey0 : 32;
        Store::run(dk, [sc](float x) { return x * sc; }, patch, dk0, p.dks[2] * 2, lane, keys_here);
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // patch read before it is rewritten
        Store::run(dv, [](float x) { return x; }, patch, dv0, p.dvs[2] * 2, lane, keys_here);
    }
}

// ------------------------------------------------------------------ dK, dV (paired waves)
// For D = 128 the K and V rows plus both gradient accumulators of a 32-key block need 192
// registers, which rules out two waves per SIMD. Here two waves share a key block instead: a
// workgroup of 8 waves owns 128 keys; waves w and w+4 both hold the K and V rows of key block w%4.
// Per 64-row tile of Q and dO (swizzled LDS ring filled by LDS-direct loads, as in the dQ kernel)
//   score step:        member m of a pair computes S, dP, P and dS of query block m (16 MFMA +
//                      softmax) and leaves P and dS, already packed as B operands, in an LDS slot;
//   accumulation step: each member accumulates, for BOTH query blocks, the half of the head
//                      dimension it owns: dV^T[2m..2m+1] += dO^T P, dK^T[2m..2m+1] += Q^T dS (16 MFMA).
// No MFMA is executed twice, and a wave keeps only 128 persistent registers.
template <typename T, int D, bool CAUSAL, int MASK, bool DROPOUT>
__global__ __launch_bounds__(512, 2) void mfma_dkdv_pair_kernel(const KParams p) {
    using Tile = SwzTile<D>;
    constexpr int NW = 8;
    constexpr int kKeys = 128;
    constexpr int kStages = 3;
    constexpr int kStageBytes = 2 * Tile::kBytes + 2 * kBN * 4;  // Q tile, dO tile, lse, delta
    constexpr int kXchBytes = NW * 4 * 1024;                     // per wave: P[2], dS[2] fragments
    constexpr int KK = D / 16;
    constexpr int DB = D / 32;
    constexpr int DH = DB / 2;                                   // column blocks a pair member accumulates
    constexpr int kBlocksPerWave = 2 * Tile::kBlocks / NW;
    constexpr int kLoadsPerTile = kBlocksPerWave + 1;            // + lse or delta: exact for every wave
    __shared__ __attribute__((aligned(1024))) char smem[kStages * kStageBytes + kXchBytes];
    char* xch = smem + kStages * kStageBytes;

    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int kb = wave & 3, member = wave >> 2;
    const int lane = tid & 63, l32 = lane & 31, h = lane >> 5;
    int bh, kt;
    map_block_for<MASK>(p, blockIdx.x, p.S / kKeys, CAUSAL ? kHeavyFirst : kUniformTiles, &bh, &kt);
    const int b = bh / p.H, hd = bh % p.H;
    const int k0 = kt * kKeys;
    const int wkey0 = k0 + 32 * kb;
    const int key = wkey0 + l32;

    const char* kbase = static_cast<const char*>(p.k) + (b * p.ks[0] + hd * p.ks[1]) * 2;
    const char* vbase = static_cast<const char*>(p.v) + (b * p.vs[0] + hd * p.vs[1]) * 2;
    const char* qbase = static_cast<const char*>(p.q) + (b * p.qs[0] + hd * p.qs[1]) * 2;
    const char* gbase = static_cast<const char*>(p.d_o) + (b * p.dos[0] + hd * p.dos[1]) * 2;
    const int64_t qrow_bytes = p.qs[2] * 2, grow_bytes = p.dos[2] * 2;
    const float* lse_base = p.lse + static_cast<int64_t>(bh) * p.S;
    const float* delta_base = p.delta + static_cast<int64_t>(bh) * p.S;

    const float c = p.scale_log2;
    [[maybe_unused]] const float inv_scale = p.inv_scale;  // (a mask value joins its score before the scale: s + mask / scale)

    f32x16 dk[DH], dv[DH];
#pragma unroll
    for (int d = 0; d < DH; ++d) {
        dk[d] = zero16();
        dv[d] = zero16();
    }

    int src_off[kBlocksPerWave];
#pragma unroll
    for (int i = 0; i < kBlocksPerWave; ++i) {
        const int blk = wave * kBlocksPerWave + i;
        const bool is_g = blk >= Tile::kBlocks;
        src_off[i] = static_cast<int>(Tile::src_off(is_g ? blk - Tile::kBlocks : blk, lane, is_g ? grow_bytes : qrow_bytes));
    }
    const int t_begin = CAUSAL ? k0 / kBN : 0;
    const int n_tiles = p.S / kBN;
    auto issue_tile = [&](int t) {
        char* stage = smem + ((t - t_begin) % kStages) * kStageBytes;  // slots count from the first tile
#pragma unroll
        for (int i = 0; i < kBlocksPerWave; ++i) {
            const int blk = wave * kBlocksPerWave + i;
            const bool is_g = blk >= Tile::kBlocks;
            const char* tile_src = is_g ? gbase + static_cast<int64_t>(t) * kBN * grow_bytes
                                        : qbase + static_cast<int64_t>(t) * kBN * qrow_bytes;
            char* dst = stage + (is_g ? Tile::kBytes + (blk - Tile::kBlocks) * 1024 : blk * 1024);
            lds_direct_load16(tile_src, src_off[i], dst);
        }
        // every wave issues exactly one more load, so that the vmcnt bookkeeping is the same in all of
        // them: even waves fetch the 64 lse values, odd waves the 64 delta values (duplicates land
        // on the same bytes)
        if (wave & 1) lds_direct_load4(delta_base + t * kBN, lane * 4, stage + 2 * Tile::kBytes + kBN * 4);
        else lds_direct_load4(lse_base + t * kBN, lane * 4, stage + 2 * Tile::kBytes);
    };
    // The K and V rows of the workgroup (128 keys = two 64-row tiles each) also arrive through LDS:
    // lanes own keys, so loading the fragments straight into registers would touch 32 cache lines
    // per instruction (measured: 4.5 us of a 95 us workgroup), while LDS-direct loads fetch whole rows.
    // They land in the third ring slot plus the exchange slots, which nobody uses before the loop.
    char* kv_lds = smem + 2 * kStageBytes;
    static_assert(kStageBytes + kXchBytes >= 4 * Tile::kBytes, "K and V must fit behind the first two ring slots");
    static_assert(4 * Tile::kBlocks % NW == 0, "K/V blocks must divide among the waves");
    constexpr int kKvLoads = 4 * Tile::kBlocks / NW;
    {
        const int64_t krow_bytes = p.ks[2] * 2, vrow_bytes = p.vs[2] * 2;
#pragma unroll
        for (int i = 0; i < kKvLoads; ++i) {
            const int blk = wave * kKvLoads + i;           // 0 .. 4*kBlocks-1: K tile 0, K tile 1, V tile 0, V tile 1
            const int tile = blk / Tile::kBlocks, b16 = blk % Tile::kBlocks;
            const bool is_v = tile >= 2;
            const int64_t rb = is_v ? vrow_bytes : krow_bytes;
            const char* src = (is_v ? vbase : kbase) + (k0 + 64 * (tile & 1)) * rb;
            lds_direct_load16(src, static_cast<uint32_t>(Tile::src_off(b16, lane, rb)), kv_lds + blk * 1024);
        }
    }
    issue_tile(t_begin);
    if (t_begin + 1 < n_tiles) issue_tile(t_begin + 1);

    const int row_off0 = Tile::off(l32, h);
    const int tr_off0 = Tile::tr_off(0, 0, lane), tr_off1 = Tile::tr_off(0, 1, lane);
    // K and V have landed (the Q/dO tiles issued after them may still be in flight)
    if (t_begin + 1 < n_tiles) TRI_WAIT_VMCNT(2 * kLoadsPerTile);
    else TRI_WAIT_VMCNT(kLoadsPerTile);
    lds_barrier();
    u32x4 kf[KK], vf[KK];
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) {
        const int off = (row_off0 ^ (kk << 5)) + 32 * (kb & 1) * Tile::kRowBytes;
        kf[kk] = lds_read16(kv_lds + (kb >> 1) * Tile::kBytes, off);
        vf[kk] = lds_read16(kv_lds + (2 + (kb >> 1)) * Tile::kBytes, off);
    }
    lds_barrier();  // every wave has its fragments: the region is free for the exchange slots and tile 2
    char* my_xch = xch + wave * 4096 + lane * 16;
    const char* peer_xch = xch + (wave ^ 4) * 4096 + lane * 16;

    // The two members of a pair sit on the same SIMD and run half a tile apart, so that one is in
    // its score phase (softmax arithmetic) while the other is in its accumulation phase (MFMA only).
    // Half-step hs: member 0 scores tile hs/2 on even steps, member 1 on odd steps; a wave publishes
    // its P and dS at the start of its next accumulation step, so a slot is never rewritten before
    // the barrier after the partner's read. Member 1 accumulates tile t on step 2t+2, member 0 on
    // step 2t+3; by then it has scored tile t+1, so it takes its own P and dS of tile t back from
    // its slot just before it overwrites them.
    const int n_local = n_tiles - t_begin;
    u32x4 cur_p[2], cur_s[2];
#pragma unroll
    for (int g = 0; g < 2; ++g) {
        cur_p[g] = cur_s[g] = u32x4{0, 0, 0, 0};
        *reinterpret_cast<u32x4*>(my_xch + g * 1024) = cur_p[g];
        *reinterpret_cast<u32x4*>(my_xch + (2 + g) * 1024) = cur_s[g];
    }

    // even half-step 2*lt: tile lt must have landed; tile lt+1 is the only other one that can be in
    // flight. After the barrier every wave is done with tile lt-2, whose slot tile lt+1 takes.
    auto open_even_step = [&](int lt) {
        if (lt == 0 && n_local > 1) TRI_WAIT_VMCNT(kLoadsPerTile);
        else TRI_WAIT_VMCNT(0);
        lds_barrier();
    };
    // (after the barrier every wave is done with tile lt-2, whose slot tile lt+1 takes; a member issues
    // its share of the loads at the start of its accumulation step, the part of a tile in which it
    // would otherwise only wait: a load instruction holds the wave until the memory pipeline takes it)
    auto issue_next = [&](int lt) {
        if (lt >= 1 && lt + 1 < n_local) issue_tile(t_begin + lt + 1);
    };
    // A step is split once more, so that the matrix pipe and the vector ALU of the SIMD are both busy:
    //   first part:  the scoring member runs its 16 MFMAs (S and dP); the accumulating member exchanges
    //                P and dS through the LDS slots and requests its first fragments;
    //   second part: the scoring member does the softmax arithmetic; the accumulating member runs its
    //                16 MFMAs.
    // (Both members issuing MFMAs at once, and the arithmetic afterwards with an idle matrix pipe, cost
    // more than twice the time.) part_barrier() separates the parts; it does not wait for LDS reads in
    // flight, which the second part consumes.
    auto part_barrier = [&]() {
        __builtin_amdgcn_sched_barrier(0);
        asm volatile("s_barrier" ::: "memory");
        __builtin_amdgcn_sched_barrier(0);
    };
    // The state a step carries from its first part to its second. Every variable is assigned in every
    // first part (zeros on the idle paths), so that none of them stays live around the loop.
    f32x16 sc_s, sc_dp;                      // scores
    f32x4 sc_lse[4];                         // lse of this lane's 16 rows
    // (fetching delta ahead like lse, and deeper fragment rings, were measured: no gain)
    constexpr bool kRoomy = false;
    f32x4 sc_dlt[kRoomy ? 4 : 1];            // delta of the same rows
    float sc_mk[MASK != kNoMask ? 16 : 1];   // mask values of the same rows at this lane's key
    const uint32_t mask_lane_off = MASK == kMaskF32 ? static_cast<uint32_t>((4 * h * p.ms[2] + key) * 4) : 0u;
    u32x4 own_p[2], own_s[2], pp[2], ps[2];  // B operands of the accumulation
    constexpr int kAccSteps = 8 * DH, kAccRing = 4;
    u32x4 tf[kAccRing];                      // first transposed fragments of the accumulation
    // score step, first part: S and dP of query block `member` of local tile lt against this pair's keys
    auto score_mfma = [&](int lt) {
        const int j = t_begin + lt;
        const int rb = j * kBN + 32 * member;
        const char* sQ = smem + ((lt < n_local ? lt : 0) % kStages) * kStageBytes;
        const char* sG = sQ + Tile::kBytes;
        const float* sLse = reinterpret_cast<const float*>(sG + Tile::kBytes);
        if (lt < n_local && (!CAUSAL || rb + 31 >= wkey0)) {
            if constexpr (MASK != kNoMask) {
                // requested before anything else of the step and used in its second part: the loads' latency, which
                // used to stand in front of every block's arithmetic, passes behind the MFMAs and the barrier between
                // the parts (a row of the block is 128 contiguous bytes across the lanes of a half wave). Requesting
                // them a whole accumulation step earlier measured no better.
                if constexpr (MASK == kMaskF32) {
                    // (row rb + 8 g + 4 h + bb: a uniform 64-bit base per (g, bb), scalar arithmetic, plus one 32-bit
                    // offset per lane that does not change over the kernel: the row stride is below 2^24 elements.
                    // The 16-bit loads take the plain form: with this one they measured 2.4 times slower.)
                    const char* ubase = static_cast<const char*>(p.mask) + (b * p.ms[0] + hd * p.ms[1] + static_cast<int64_t>(rb) * p.ms[2]) * 4;
#pragma unroll
                    for (int i = 0; i < 16; ++i)
                        sc_mk[i] = *reinterpret_cast<const float*>(ubase + static_cast<int64_t>(8 * (i >> 2) + (i & 3)) * p.ms[2] * 4 + mask_lane_off);
                } else {
                    const int64_t mbase = b * p.ms[0] + hd * p.ms[1] + key;
#pragma unroll
                    for (int i = 0; i < 16; ++i)
                        sc_mk[i] = mask_at<T, MASK>(p.mask, mbase + static_cast<int64_t>(rb + c_row(i, h)) * p.ms[2]);
                }
            }
            const int qoff = 32 * member * Tile::kRowBytes;
            // row fragments of Q, then of dO, through a ring of kRing reads in flight
            constexpr int kRing = 4;
            auto row_frag = [&](int n) {
                return lds_read16(n < KK ? sQ : sG, (row_off0 ^ ((n % KK) << 5)) + qoff);
            };
            u32x4 fr[kRing];
#pragma unroll
            for (int n = 0; n < kRing; ++n) fr[n] = row_frag(n);
            __builtin_amdgcn_sched_barrier(0);
            __builtin_amdgcn_s_setprio(2);
            f32x16 s = zero16(), dp = zero16();
#pragma unroll
            for (int n = 0; n < 2 * KK; ++n) {
                if (n < KK) s = Mma<T>::run(fr[n % kRing], kf[n], s);
                else dp = Mma<T>::run(fr[n % kRing], vf[n - KK], dp);
                if (n + kRing < 2 * KK) fr[n % kRing] = row_frag(n + kRing);
                __builtin_amdgcn_sched_barrier(0);
            }
            __builtin_amdgcn_s_setprio(0);
            sc_s = s;
            sc_dp = dp;
        } else {
            sc_s = zero16();
            sc_dp = zero16();
        }
        // requested now, used in the second part (harmless where the step is idle)
#pragma unroll
        for (int g = 0; g < 4; ++g) sc_lse[g] = *reinterpret_cast<const f32x4*>(sLse + 32 * member + 8 * g + 4 * h);
        if constexpr (kRoomy) {
#pragma unroll
            for (int g = 0; g < 4; ++g) sc_dlt[g] = *reinterpret_cast<const f32x4*>(sLse + kBN + 32 * member + 8 * g + 4 * h);
        }
    };
    // score step, second part: P and dS from the scores, packed as B operands
    auto score_valu = [&](int lt) {
        const int j = t_begin + lt;
        const int rb = j * kBN + 32 * member;
        if (lt < n_local && (!CAUSAL || rb + 31 >= wkey0)) {
            const char* sQ = smem + (lt % kStages) * kStageBytes;
            const char* sG = sQ + Tile::kBytes;
            const float* sDelta = reinterpret_cast<const float*>(sG + Tile::kBytes) + kBN;
            f32x16 s = sc_s;
            const f32x16 dp = sc_dp;
            if (CAUSAL && rb < wkey0 + 31) {  // a block that crosses the diagonal: scores above it drop out
                asm volatile("");             // (a real branch: the other blocks skip the comparisons)
#pragma unroll
                for (int i = 0; i < 16; ++i) s[i] = key <= rb + c_row(i, h) ? s[i] : -INFINITY;
            }
            float mk[MASK != kNoMask ? 16 : 1];
            if constexpr (MASK != kNoMask) {
#pragma unroll
                for (int i = 0; i < 16; ++i) mk[i] = sc_mk[i];
            }
            Philox4 mine;  // the block of rows rb + 8 (lane % 4) + 4 h .. +3: this lane's share of the quad's four
            if constexpr (DROPOUT) mine = dropout_block(p, bh, (rb + 8 * (lane & 3) + 4 * h) >> 2, key >> 2);
#pragma unroll
            for (int gg = 0; gg < 2; ++gg) {  // eight rows at a time, packed as soon as they are done
                float pr[8], ds[8];
                f32x4 dlt4[2];
#pragma unroll
                for (int g2 = 0; g2 < 2; ++g2) {
                    if constexpr (kRoomy) dlt4[g2] = sc_dlt[2 * gg + g2];
                    else dlt4[g2] = *reinterpret_cast<const f32x4*>(sDelta + 32 * member + 8 * (2 * gg + g2) + 4 * h);
                }
#pragma unroll
                for (int g2 = 0; g2 < 2; ++g2) {
                    const int g = 2 * gg + g2;
                    f32x4 l4 = sc_lse[g];
                    const f32x4 d4 = dlt4[g2];
                    uint32_t dw[4];
                    if constexpr (DROPOUT) {
                        const Philox4 r = quad_bcast_from(g, mine);  // lane g of the quad generated rows rb + 8 g + 4 h .. +3
#pragma unroll
                        for (int bb = 0; bb < 4; ++bb) dw[bb] = (r.w[bb] >> (8 * (key & 3))) & 0xffu;
                    }
#pragma unroll
                    for (int bb = 0; bb < 4; ++bb) {
                        const int i = 4 * g + bb;
                        float pv;
                        if constexpr (MASK != kNoMask) pv = fast_exp2(fmaf(fmaf(mk[i], inv_scale, s[i]), c, -l4[bb]));
                        else pv = fast_exp2(fmaf(s[i], c, -l4[bb]));
                        float dpv = dp[i];
                        if constexpr (DROPOUT) {
                            const bool keep = static_cast<int>(dw[bb]) >= p.thr8;
                            dpv = keep ? dpv * p.zscale : 0.f;
                            pr[4 * g2 + bb] = keep ? pv * p.zscale : 0.f;
                        } else {
                            pr[4 * g2 + bb] = pv;
                        }
                        ds[4 * g2 + bb] = pv * (dpv - d4[bb]);
                    }
                }
                cur_p[gg] = pack8<T>(pr);
                cur_s[gg] = pack8<T>(ds);
                __builtin_amdgcn_sched_barrier(0);
            }
        } else {
#pragma unroll
            for (int g = 0; g < 2; ++g) cur_p[g] = cur_s[g] = u32x4{0, 0, 0, 0};
        }
    };
    // accumulation step, first part: publish the latest scores, fetch the partner's and the first
    // transposed fragments. Second part: add local tile lt to this member's half of the head dimension
    // for both query blocks: 8 DH MFMAs in the order (query block, K-step, dV^T or dK^T, column block),
    // their A operands through one ring of fragments.
    auto acc_frag = [&](int lt, int n) {
        const char* sQ = smem + (lt % kStages) * kStageBytes;
        const char* sG = sQ + Tile::kBytes;
        const int d = n % DH, which = (n / DH) % 2, g = (n / (2 * DH)) % 2, qb = n / (4 * DH);
        const int db = DH * member + d;
        return Tile::tr_frag(which ? sQ : sG, tr_off0 ^ (db << 6), tr_off1 ^ (db << 6), 2 * qb + g);
    };
    auto acc_on = [&](int lt) {
        return lt >= 0 && lt < n_local && (!CAUSAL || (t_begin + lt) * kBN + kBN - 1 >= wkey0);
    };
    auto acc_prep = [&](int lt) {
#pragma unroll
        for (int g = 0; g < 2; ++g) {
            if (member == 0) {  // LDS operations of one wave complete in order: read, then overwrite
                own_p[g] = *reinterpret_cast<const u32x4*>(my_xch + g * 1024);
                own_s[g] = *reinterpret_cast<const u32x4*>(my_xch + (2 + g) * 1024);
            } else {
                own_p[g] = cur_p[g];
                own_s[g] = cur_s[g];
            }
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int g = 0; g < 2; ++g) {
            *reinterpret_cast<u32x4*>(my_xch + g * 1024) = cur_p[g];
            *reinterpret_cast<u32x4*>(my_xch + (2 + g) * 1024) = cur_s[g];
        }
        // (unconditional reads: harmless where the step is idle)
#pragma unroll
        for (int g = 0; g < 2; ++g) {  // the partner's P and dS
            pp[g] = *reinterpret_cast<const u32x4*>(peer_xch + g * 1024);
            ps[g] = *reinterpret_cast<const u32x4*>(peer_xch + (2 + g) * 1024);
        }
        const int lt_safe = lt >= 0 && lt < n_local ? lt : 0;
#pragma unroll
        for (int n = 0; n < kAccRing; ++n) tf[n] = acc_frag(lt_safe, n);
    };
    auto acc_mfma = [&](int lt) {
        if (acc_on(lt)) {
            __builtin_amdgcn_s_setprio(2);
#pragma unroll
            for (int n = 0; n < kAccSteps; ++n) {
                const int d = n % DH, which = (n / DH) % 2, g = (n / (2 * DH)) % 2, qb = n / (4 * DH);
                if (which == 0) dv[d] = Mma<T>::run(tf[n % kAccRing], qb == member ? own_p[g] : pp[g], dv[d]);
                else dk[d] = Mma<T>::run(tf[n % kAccRing], qb == member ? own_s[g] : ps[g], dk[d]);
                if (n + kAccRing < kAccSteps) tf[n % kAccRing] = acc_frag(lt, n + kAccRing);
                __builtin_amdgcn_sched_barrier(0);
            }
            __builtin_amdgcn_s_setprio(0);
        }
    };

    if (member == 0) {
#pragma unroll 1
        for (int lt = 0; lt <= n_local; ++lt) {
            open_even_step(lt);
            score_mfma(lt);
            part_barrier();
            score_valu(lt);
            lds_barrier();
            issue_next(lt);  // in the part where this member only waits for the partner's MFMAs
            acc_prep(lt - 1);
            part_barrier();
            acc_mfma(lt - 1);
        }
    } else {
#pragma unroll 1
        for (int lt = 0; lt <= n_local; ++lt) {
            open_even_step(lt);
            issue_next(lt);
            acc_prep(lt - 1);
            part_barrier();
            acc_mfma(lt - 1);
            lds_barrier();
            score_mfma(lt);
            part_barrier();
            score_valu(lt);
        }
    }

    // every wave is out of the loop: the ring can serve as the waves' private transposition patches
    lds_barrier();
    {
        using Store = RowBlockStore<T, DH>;
        static_assert(NW * Store::kPatchBytes <= kStages * kStageBytes, "patches must fit into the ring");
        char* patch = smem + wave * Store::kPatchBytes;
        const int64_t row = wkey0;  // first key of this pair; this member writes columns 32*DH*member ..
        char* dk0 = static_cast<char*>(p.dk) + (b * p.dks[0] + hd * p.dks[1] + row * p.dks[2] + 32 * DH * member) * 2;
        char* dv0 = static_cast<char*>(p.dv) + (b * p.dvs[0] + hd * p.dvs[1] + row * p.dvs[2] + 32 * DH * member) * 2;
        const float sc = p.scale;
        // (the lane index taken afresh: the epilogue's per-lane offsets are computed here, not kept across the loop)
        int elane = threadIdx.x & 63;
        asm volatile("" : "+v"(elane));
        Store::run(dk, [sc](float x) { return x * sc; }, patch, dk0, p.dks[2] * 2, elane);
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // patch read before it is rewritten
        Store::run(dv, [](float x) { return x; }, patch, dv0, p.dvs[2] * 2, elane);
    }
}

// ------------------------------------------------------------------ dK, dV (paired waves, phased; no mask)
// The pairing of the kernel above (waves w and w+4 share key block w%4, each accumulates half of the
// head dimension) with the phase structure of the forward kernel. Q and dO stream as 32-row blocks
// (plus their lse and delta) through a ring of 7 slots; even blocks are scored by member 0, odd
// blocks by member 1, and both members accumulate every block. A member alternates
//   vector phase:  P and dS of its block from S' and dP' (softmax backward), published in its LDS slot;
//                  the partner's latest block is fetched from the partner's slot;
//   matrix phase:  dV^T, dK^T += the partner's latest block and its own (16 MFMAs), then S' = S - lse / c
//                  and dP' = dP - delta of its next block (18 MFMAs), through one ring of LDS fragments;
// with a workgroup barrier after each phase, member 1 one phase behind member 0: a SIMD always has one
// wave on the matrix pipe and one on the vector ALU. Block r is first read in phase r-1 and last in
// phase r+2; in phase ph every wave issues its share of block ph+4 and, before the barrier, waits for
// its share of block ph+2.
// With DROPOUT only -lse / c is folded into the accumulators: dS = P (Z dP - delta) needs delta beside the dropped dP,
// so the vector phase reads its 16 row values from the block's slot, and draws the keep decisions of its block (one
// Philox call per lane, shared inside the quad).
// With KEYMASK (kMaskF32 / kMaskT; never with the causal mask): an additive mask that is the same for every query row
// (row stride 0: a key-padding mask). Lanes own keys here, so the whole mask is one value per lane, read once, and goes
// into the exponent for free (the multiply by the scale becomes a fused multiply-add).
template <typename T, int D, bool CAUSAL, bool DROPOUT = false, int KEYMASK = kNoMask>
__global__ __launch_bounds__(512, 2) void mfma_dkdv_phased_kernel(const KParams p) {
    static_assert(KEYMASK == kNoMask || !CAUSAL, "a mask excludes the causal variant");
    using Tile = SwzTile<D>;
    constexpr int NW = 8;
    constexpr int kKeys = 128;
    constexpr int kBR = 32;                                  // rows per streamed block
    constexpr int kSlots = 7;
    constexpr int kHalfBytes = kBR * Tile::kRowBytes;        // one operand of a block
    constexpr int kSlotBytes = 2 * kHalfBytes + 512;         // Q rows, dO rows, lse, delta (256 B each)
    constexpr int kXchBytes = NW * 4096;                     // per wave: P[2], dS[2] fragments
    constexpr int KK = D / 16;
    constexpr int DB = D / 32;
    constexpr int DH = DB / 2;                               // column blocks a pair member accumulates
    constexpr int kLoads = 5;                                // loads per requesting wave and block
    static_assert(kHalfBytes == NW * 1024, "two Q loads and two dO loads per requesting wave and block");
    constexpr int kAccSteps = 4 * DH;                        // MFMAs that add one block
    constexpr int kSteps = 2 * kAccSteps + 2 * KK;           // matrix phase
    constexpr int kRing = 4;
    __shared__ __attribute__((aligned(1024))) char smem[kSlots * kSlotBytes + kXchBytes];
    char* xch = smem + kSlots * kSlotBytes;

    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int kb = wave & 3, member = wave >> 2;
    const int lane = tid & 63, l32 = lane & 31, h = lane >> 5;
    int bh, kt;
    map_block(blockIdx.x, p.B * p.H, p.S / kKeys, CAUSAL ? kHeavyFirst : kUniformTiles, &bh, &kt);
    const int b = bh / p.H, hd = bh % p.H;
    const int k0 = kt * kKeys;
    const int wkey0 = k0 + 32 * kb;
    const int key = wkey0 + l32;

    const char* kbase = static_cast<const char*>(p.k) + (b * p.ks[0] + hd * p.ks[1]) * 2;
    const char* vbase = static_cast<const char*>(p.v) + (b * p.vs[0] + hd * p.vs[1]) * 2;
    const char* qbase = static_cast<const char*>(p.q) + (b * p.qs[0] + hd * p.qs[1]) * 2;
    const char* gbase = static_cast<const char*>(p.d_o) + (b * p.dos[0] + hd * p.dos[1]) * 2;
    const int64_t qrow_bytes = p.qs[2] * 2, grow_bytes = p.dos[2] * 2;
    const float* lse_base = p.lse + static_cast<int64_t>(bh) * p.S;
    const float* delta_base = p.delta + static_cast<int64_t>(bh) * p.S;
    const float c = p.scale_log2;
    [[maybe_unused]] const float inv_scale = p.inv_scale;  // (a mask value joins its score before the scale: s + mask / scale)
    float key_bias = 0.f;  // mask value of this lane's key, log2 domain
    if constexpr (KEYMASK != kNoMask) key_bias = mask_at<T, KEYMASK>(p.mask, b * p.ms[0] + hd * p.ms[1] + key) * kLog2e;

    f32x16 dk[DH], dv[DH];
#pragma unroll
    for (int d = 0; d < DH; ++d) {
        dk[d] = zero16();
        dv[d] = zero16();
    }

    const int row_first = CAUSAL ? k0 : 0;          // first streamed row (block 0)
    const int n_blocks = (p.S - row_first) / kBR;   // >= 4, even
    // A block is requested by the four waves of ONE member, the one that is in its vector phase when the request is
    // due (member 0 the even blocks, member 1 the odd ones): a vector-memory instruction holds its wave until the
    // memory pipeline has taken it, which the matrix phase cannot afford. Wave kb of the member fetches the 1 KiB
    // pieces kb and kb + 4 of the Q rows and of the dO rows (rows 16 apart share the swizzle, so one per-lane offset
    // serves both) and the block's 32 lse (kb even) or delta (kb odd) values; lanes 32-63 repeat those. The source
    // pointers and the ring slot advance by two blocks per call.
    const uint32_t qoff = static_cast<uint32_t>(Tile::src_off(kb, lane, qrow_bytes));
    const uint32_t goff = static_cast<uint32_t>(Tile::src_off(kb, lane, grow_bytes));
    int next_block = member, next_slot = member;
    const char* next_q = qbase + (row_first + member * kBR) * qrow_bytes;
    const char* next_g = gbase + (row_first + member * kBR) * grow_bytes;
    const float* next_aux = ((kb & 1) ? delta_base : lse_base) + row_first + member * kBR;
    const int aux_lds = 2 * kHalfBytes + ((kb & 1) ? 256 : 0);
    auto issue_block = [&]() {  // this wave's share of its member's next block, if it exists
        if (next_block < n_blocks) {
            char* slot = smem + next_slot * kSlotBytes;
            lds_direct_load16(next_q, qoff, slot + kb * 1024);
            lds_direct_load16(next_g, goff, slot + kHalfBytes + kb * 1024);
            lds_direct_load16(next_q + 16 * qrow_bytes, qoff, slot + (kb + 4) * 1024);
            lds_direct_load16(next_g + 16 * grow_bytes, goff, slot + kHalfBytes + (kb + 4) * 1024);
            lds_direct_load4(next_aux, (lane & 31) * 4, slot + aux_lds);
        }
        next_block += 2;
        next_slot = next_slot >= kSlots - 2 ? next_slot + 2 - kSlots : next_slot + 2;
        next_q += 2 * kBR * qrow_bytes;
        next_g += 2 * kBR * grow_bytes;
        next_aux += 2 * kBR;
    };
    // before the barrier that ends vector phase ph of a member: its block ph+2 has landed, its block ph+4 may be in flight
    auto wait_blocks = [&](int ph) {
        if (ph + 4 < n_blocks) TRI_WAIT_VMCNT(kLoads);
        else TRI_WAIT_VMCNT(0);
    };

    // The K and V rows of the workgroup (128 keys = two 64-row tiles each) arrive through LDS too (lanes
    // own keys, so direct loads would touch 32 cache lines per instruction); they land behind the first
    // four ring slots, which take blocks 0-3 meanwhile.
    char* kv_lds = smem + 4 * kSlotBytes;
    static_assert(3 * kSlotBytes + kXchBytes >= 4 * Tile::kBytes, "K and V must fit behind the first four slots");
    constexpr int kKvLoads = 4 * Tile::kBlocks / NW;
    {
        const int64_t krow_bytes = p.ks[2] * 2, vrow_bytes = p.vs[2] * 2;
#pragma unroll
        for (int i = 0; i < kKvLoads; ++i) {
            const int blk = wave * kKvLoads + i;           // 0 .. 4*kBlocks-1: K tile 0, K tile 1, V tile 0, V tile 1
            const int tile = blk / Tile::kBlocks, b16 = blk % Tile::kBlocks;
            const bool is_v = tile >= 2;
            const int64_t rb = is_v ? vrow_bytes : krow_bytes;
            const char* src = (is_v ? vbase : kbase) + (k0 + 64 * (tile & 1)) * rb;
            lds_direct_load16(src, static_cast<uint32_t>(Tile::src_off(b16, lane, rb)), kv_lds + blk * 1024);
        }
    }
    issue_block();  // blocks 0 and 2 (member 0), 1 and 3 (member 1)
    issue_block();

    int row_off0 = Tile::off(l32, h);
    int tr_off0 = Tile::tr_off(0, 0, lane), tr_off1 = Tile::tr_off(0, 1, lane);
    // Taken afresh at the head of each member's loop: with every register in use, values computed once up here and
    // needed by only one of the two loops would otherwise be spilled around the other.
    auto refresh_lane_offsets = [&]() {
        int l = lane;
        asm volatile("" : "+v"(l));
        row_off0 = Tile::off(l & 31, l >> 5);
        tr_off0 = Tile::tr_off(0, 0, l);
        tr_off1 = Tile::tr_off(0, 1, l);
    };
    TRI_WAIT_VMCNT(2 * kLoads);  // K and V have landed
    lds_barrier();
    u32x4 kf[KK], vf[KK];
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) {
        const int off = (row_off0 ^ (kk << 5)) + 32 * (kb & 1) * Tile::kRowBytes;
        kf[kk] = lds_read16(kv_lds + (kb >> 1) * Tile::kBytes, off);
        vf[kk] = lds_read16(kv_lds + (2 + (kb >> 1)) * Tile::kBytes, off);
    }
    lds_barrier();  // every wave has its fragments: the region is free for the exchange slots and later blocks
    char* my_xch = xch + wave * 4096 + lane * 16;
    const char* peer_xch = xch + (wave ^ 4) * 4096 + lane * 16;
    u32x4 cur_p[2], cur_s[2];   // P and dS of this member's current block
    u32x4 par_p[2], par_s[2];   // the partner's latest block
#pragma unroll
    for (int g = 0; g < 2; ++g) {
        cur_p[g] = cur_s[g] = par_p[g] = par_s[g] = u32x4{0, 0, 0, 0};
        *reinterpret_cast<u32x4*>(my_xch + g * 1024) = cur_p[g];
        *reinterpret_cast<u32x4*>(my_xch + (2 + g) * 1024) = cur_s[g];
    }
    TRI_WAIT_VMCNT(kLoads);  // blocks 0 and 1 have landed
    lds_barrier();

    // whether this pair has anything in block r (under the causal mask: rows at or below its first key)
    auto block_on = [&](int r) { return r >= 0 && r < n_blocks && (!CAUSAL || r >= kb); };

    constexpr float kFoldUnit = 256.f;  // the constant the split terms multiply (keeps f16 terms in range)
    const float neg_inv_c = -1.f / c;
    f32x16 sc_s, sc_dp;  // S - lse / c and dP - delta of this member's next block
    u32x4 ring[kRing];
    // Ring slots are named by their byte offset in LDS and stepped from block to block (a slot index taken modulo 7
    // for every block a phase touches costs a dozen scalar instructions each time).
    constexpr int kRingBytes = kSlots * kSlotBytes;
    auto slot_step = [&](int so, int d) {
        int t = so + d * kSlotBytes;
        t = t >= kRingBytes ? t - kRingBytes : t;
        return t < 0 ? t + kRingBytes : t;
    };
    // fragment n of a matrix phase that adds the blocks in slots sa and sb and scores the block in slot ss
    auto frag = [&](int sa, int sb, int ss, int n) {
        if (n < 2 * kAccSteps) {
            const char* slot = smem + (n < kAccSteps ? sa : sb);
            const int m = n % kAccSteps;
            const int d = m % DH, which = (m / DH) % 2, g = m / (2 * DH);
            const int db = DH * member + d;
            return Tile::tr_frag(slot + (which ? 0 : kHalfBytes), tr_off0 ^ (db << 6), tr_off1 ^ (db << 6), g);
        }
        const int m = n - 2 * kAccSteps;
        return lds_read16(smem + ss + (m < KK ? 0 : kHalfBytes), row_off0 ^ ((m % KK) << 5));
    };
    auto matrix_phase = [&](auto with_acc, int sa, int sb, int ss, bool own_on = true, bool score_on = true) {
        constexpr int first = decltype(with_acc)::value ? 0 : 2 * kAccSteps;
        f32x16 s = zero16(), dp = zero16();
        // One more MFMA each puts -lse / c and -delta under S and dP (a row's value split into three 16-bit
        // terms against a column of constants), so that the vector phase needs neither value: P = exp2(c S'),
        // dS = P dP'. Each lane asks for its row's two values at the start of the phase.
        float row_lse = 0.f, row_delta = 0.f;
#pragma unroll
        for (int n = first; n < kSteps; ++n) {
            const int slot = (n - first) % kRing;
            if ((n == kAccSteps && !own_on && !score_on) || (n == 2 * kAccSteps && !score_on)) break;
            if (n == first) {
                const float* sLse = reinterpret_cast<const float*>(smem + ss + 2 * kHalfBytes);
                row_lse = sLse[l32];
                if constexpr (!DROPOUT) row_delta = sLse[64 + l32];
            }
            if (n == 2 * kAccSteps) {
                const u32x4 zero4 = {0, 0, 0, 0};
                const u32x4 al = split3<T>(row_lse * neg_inv_c * (1.f / kFoldUnit));
                const u32x4 ad = split3<T>(row_delta * (-1.f / kFoldUnit));
                const uint32_t u2 = Mma<T>::pack2(kFoldUnit, kFoldUnit), u1 = Mma<T>::pack2(kFoldUnit, 0.f);
                const u32x4 units = h == 0 ? u32x4{u2, u1, 0, 0} : zero4;
                s = Mma<T>::run(h == 0 ? al : zero4, units, s);
                if constexpr (!DROPOUT) dp = Mma<T>::run(h == 0 ? ad : zero4, units, dp);
            }
            if (n < 2 * kAccSteps) {
                const int m = n % kAccSteps;
                const int d = m % DH, which = (m / DH) % 2, g = m / (2 * DH);
                const bool own = n >= kAccSteps;
                if (which == 0) dv[d] = Mma<T>::run(ring[slot], own ? cur_p[g] : par_p[g], dv[d]);
                else dk[d] = Mma<T>::run(ring[slot], own ? cur_s[g] : par_s[g], dk[d]);
            } else {
                const int m = n - 2 * kAccSteps;
                if (m < KK) s = Mma<T>::run(ring[slot], kf[m], s);
                else dp = Mma<T>::run(ring[slot], vf[m - KK], dp);
            }
            if (n + kRing < kSteps) ring[slot] = frag(sa, sb, ss, n + kRing);
            __builtin_amdgcn_sched_barrier(0);
        }
        sc_s = s;
        sc_dp = dp;
    };
    using Yes = std::integral_constant<bool, true>;
    using No = std::integral_constant<bool, false>;

    // P = exp2(c S') and dS = P dP' of the block whose first row is rb, eight rows at a time, packed as soon as
    // they are done; only the block on the diagonal pays for the causal comparison (scores above it become -inf)
    auto softmax_backward = [&](bool on_diagonal, int rb, int so) {
        if (on_diagonal) {
            // a real branch, taken for one block per workgroup; the row base goes through a scalar register the
            // compiler cannot see through, so that the 16 comparisons are made here and not kept as lane masks
            // across the whole loop
            int rbo = rb;
            asm volatile("" : "+s"(rbo));
#pragma unroll
            for (int i = 0; i < 16; ++i) sc_s[i] = key <= rbo + c_row(i, h) ? sc_s[i] : -INFINITY;
        }
        const f32x16 s = sc_s, dp = sc_dp;
        const float* sDelta = reinterpret_cast<const float*>(smem + so + 2 * kHalfBytes) + 64;
        Philox4 mine;  // the block of rows rb + 8 (lane % 4) + 4 h .. +3: this lane's share of the quad's four
        if constexpr (DROPOUT) mine = dropout_block(p, bh, (rb + 8 * (lane & 3) + 4 * h) >> 2, key >> 2);
#pragma unroll
        for (int gg = 0; gg < 2; ++gg) {
            float pr[8], ds[8];
#pragma unroll
            for (int g2 = 0; g2 < 2; ++g2) {
                const int g = 2 * gg + g2;
                f32x4 d4 = {0.f, 0.f, 0.f, 0.f};
                uint32_t dw[4] = {0, 0, 0, 0};
                if constexpr (DROPOUT) {
                    d4 = *reinterpret_cast<const f32x4*>(sDelta + 8 * g + 4 * h);
                    const Philox4 rr = quad_bcast_from(g, mine);  // lane g of the quad generated rows rb + 8 g + 4 h .. +3
#pragma unroll
                    for (int bb = 0; bb < 4; ++bb) dw[bb] = (rr.w[bb] >> (8 * (key & 3))) & 0xffu;
                }
#pragma unroll
                for (int bb = 0; bb < 4; ++bb) {
                    const int i = 4 * g + bb, j = 4 * g2 + bb;
                    const float pv = KEYMASK != kNoMask ? fast_exp2(fmaf(s[i], c, key_bias)) : fast_exp2(s[i] * c);
                    if constexpr (DROPOUT) {
                        const bool keep = static_cast<int>(dw[bb]) >= p.thr8;
                        pr[j] = keep ? pv * p.zscale : 0.f;
                        ds[j] = pv * ((keep ? dp[i] * p.zscale : 0.f) - d4[bb]);
                    } else {
                        pr[j] = pv;
                        ds[j] = pv * dp[i];
                    }
                }
            }
            cur_p[gg] = pack8<T>(pr);
            cur_s[gg] = pack8<T>(ds);
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    // vector phase for block r (this member's): P and dS from sc_s, sc_dp
    auto vector_phase = [&](int r, int so) {
        if (block_on(r)) {
            const int rb = row_first + r * kBR;
            softmax_backward(CAUSAL && r == kb, rb, so);
        } else {
            // (the zeros are made inside this branch, where the compiler cannot lift them in front of the test above:
            // lifted, they are sixteen moves in every phase of the loop. The one variant that has no two registers to
            // spare for that keeps the plain assignment.)
            constexpr bool kPlainZeros = std::is_same<T, f16_t>::value && CAUSAL && !DROPOUT;
#pragma unroll
            for (int g = 0; g < 2; ++g) {
                if constexpr (kPlainZeros) {
                    cur_p[g] = cur_s[g] = u32x4{0, 0, 0, 0};
                } else {
                    uint32_t z[8];
#pragma unroll
                    for (int i = 0; i < 8; ++i) asm volatile("v_mov_b32 %0, 0" : "=v"(z[i]));
                    cur_p[g] = u32x4{z[0], z[1], z[2], z[3]};
                    cur_s[g] = u32x4{z[4], z[5], z[6], z[7]};
                }
            }
        }
    };
    // the second half of a vector phase in global phase ph, for a member whose block is r: publish, fetch
    // the partner's block r-1, request the first fragments of the matrix phase, meet the barrier
    // (so: the slot of block r; block r - 1 sits one slot before it, block r + 2 two after; at the ends of the range the
    // neighbour that does not exist is replaced by one that does, its P and dS are zero)
    auto close_vector_phase = [&](int ph, int r, int so) {
#pragma unroll
        for (int g = 0; g < 2; ++g) {
            *reinterpret_cast<u32x4*>(my_xch + g * 1024) = cur_p[g];
            *reinterpret_cast<u32x4*>(my_xch + (2 + g) * 1024) = cur_s[g];
        }
        issue_block();
        asm volatile("" ::: "memory");  // the reads below are issued after the writes above
#pragma unroll
        for (int g = 0; g < 2; ++g) {
            par_p[g] = *reinterpret_cast<const u32x4*>(peer_xch + g * 1024);
            par_s[g] = *reinterpret_cast<const u32x4*>(peer_xch + (2 + g) * 1024);
        }
        const int before = slot_step(so, -1);
        const int sa = r > 0 ? before : so, sb = r < n_blocks ? so : before;
#pragma unroll
        for (int n = 0; n < kRing; ++n) ring[n] = frag(sa, sb, slot_step(so, 2), n);
        // LDS operations of a wave complete in order: once at most the 4 + 2 kRing reads above are
        // outstanding, the slot is published
        static_assert(4 + 2 * kRing <= 15, "lgkmcnt range");
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_waitcnt(0xC07F | ((4 + 2 * kRing) << 8));
        wait_blocks(ph);
        __builtin_amdgcn_sched_barrier(0);
        asm volatile("s_barrier" ::: "memory");  // (the reads above stay in flight)
        __builtin_amdgcn_sched_barrier(0);
    };
    auto run_matrix_phase = [&](int r, int so) {
        // (the last rounds have no own block to add and no block r + 2 to score: those steps are left out, except
        // with dropout, where the shorter instruction stream would cost registers the variant does not have)
        __builtin_amdgcn_s_setprio(2);
        const int before = slot_step(so, -1);
        matrix_phase(Yes{}, r > 0 ? before : so, r < n_blocks ? so : before, slot_step(so, 2), DROPOUT || r < n_blocks,
                     DROPOUT || r + 2 < n_blocks);
        __builtin_amdgcn_s_setprio(0);
        __builtin_amdgcn_sched_barrier(0);
        lds_barrier();
        __builtin_amdgcn_sched_barrier(0);
    };

    // before phase 0: S and dP of each member's first block (member 0: block 0, member 1: block 1)
    {
#pragma unroll
        for (int n = 0; n < kRing; ++n) ring[n] = frag(0, 0, member * kSlotBytes, 2 * kAccSteps + n);
        __builtin_amdgcn_sched_barrier(0);
        matrix_phase(No{}, 0, 0, member * kSlotBytes);
        lds_barrier();
    }
    const int n_iter = n_blocks / 2;
    if (member == 0) {
        refresh_lane_offsets();
        int so = 0;  // slot of block r
#pragma unroll 1
        for (int t = 0; t <= n_iter; ++t) {   // the last round only adds member 1's last block
            const int r = 2 * t;
            vector_phase(r, so);
            close_vector_phase(2 * t, r, so);
            run_matrix_phase(r, so);
            so = slot_step(so, 2);
        }
    } else {
        refresh_lane_offsets();
        lds_barrier();  // (phase 0: member 0 alone)
        int so = kSlotBytes;  // slot of block r
#pragma unroll 1
        for (int t = 0; t < n_iter; ++t) {
            const int r = 2 * t + 1;
            vector_phase(r, so);
            close_vector_phase(2 * t + 1, r, so);
            run_matrix_phase(r, so);
            so = slot_step(so, 2);
        }
        lds_barrier();  // (the last phase: member 0 alone)
    }

    // every wave is out of the loop: the ring can serve as the waves' private transposition patches
    lds_barrier();
    {
        using Store = RowBlockStore<T, DH>;
        static_assert(NW * Store::kPatchBytes <= kSlots * kSlotBytes, "patches must fit into the ring");
        char* patch = smem + wave * Store::kPatchBytes;
        const int64_t row = wkey0;  // first key of this pair; this member writes columns 32*DH*member ..
        char* dk0 = static_cast<char*>(p.dk) + (b * p.dks[0] + hd * p.dks[1] + row * p.dks[2] + 32 * DH * member) * 2;
        char* dv0 = static_cast<char*>(p.dv) + (b * p.dvs[0] + hd * p.dvs[1] + row * p.dvs[2] + 32 * DH * member) * 2;
        const float sc = p.scale;
        // (the lane index taken afresh: the epilogue's per-lane offsets are computed here, not kept across the loop)
        int elane = threadIdx.x & 63;
        asm volatile("" : "+v"(elane));
        Store::run(dk, [sc](float x) { return x * sc; }, patch, dk0, p.dks[2] * 2, elane);
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // patch read before it is rewritten
        Store::run(dv, [](float x) { return x; }, patch, dv0, p.dvs[2] * 2, elane);
    }
}

// ---------------------------------------------------------------------------------- launch
template <typename T, int D, int NW, bool CAUSAL, int MASK>
int launch_dq_waves(const KParams& p, hipStream_t stream, bool with_delta = false) {
    const dim3 grid(p.B * p.H * (p.S / (32 * NW))), block(64 * NW);
    if constexpr (NW == 8 && D == 128 && MASK != kNoMask) {
        // with a mask gradient or dropout on top of a mask the 8-wave kernel does not fit its registers at D = 128 and
        // would spill to scratch memory (whose reloads are vector-memory loads that drain the tile prefetch): those
        // problems take 128-row workgroups, which fit
        if (p.dmask != nullptr || p.thr8 > 0) return launch_dq_waves<T, D, 4, CAUSAL, MASK>(p, stream, with_delta);
        hipLaunchKernelGGL((mfma_dq_kernel<T, D, NW, CAUSAL, MASK, false>), grid, block, 0, stream, p);
    } else {
        if constexpr (MASK != kNoMask) {
            if (p.dmask != nullptr) {
                if (p.thr8 > 0) hipLaunchKernelGGL((mfma_dq_kernel<T, D, NW, CAUSAL, MASK, true, false, true>), grid, block, 0, stream, p);
                else hipLaunchKernelGGL((mfma_dq_kernel<T, D, NW, CAUSAL, MASK, false, false, true>), grid, block, 0, stream, p);
                return static_cast<int>(hipGetLastError());
            }
        }
        if constexpr (MASK == kNoMask) {
            if (with_delta) {
                if (p.thr8 > 0) hipLaunchKernelGGL((mfma_dq_kernel<T, D, NW, CAUSAL, MASK, true, false, false, true>), grid, block, 0, stream, p);
                else hipLaunchKernelGGL((mfma_dq_kernel<T, D, NW, CAUSAL, MASK, false, false, false, true>), grid, block, 0, stream, p);
                return static_cast<int>(hipGetLastError());
            }
        }
        if (p.thr8 > 0) hipLaunchKernelGGL((mfma_dq_kernel<T, D, NW, CAUSAL, MASK, true>), grid, block, 0, stream, p);
        else hipLaunchKernelGGL((mfma_dq_kernel<T, D, NW, CAUSAL, MASK, false>), grid, block, 0, stream, p);
    }
    return static_cast<int>(hipGetLastError());
}

// whether the phased dQ kernel serves this problem (no mask, 256-row workgroups, D >= 64; with dropout at D = 128 it
// fits its registers only under the causal mask and with a fragment ring of 4). At D = 32 the kernel above needs 96
// registers, two of its workgroups share a CU, and that measured 27 % faster than the phased pairs.
template <int D, int MASK>
bool dq_is_phased(const KParams& p) {
    return MASK == kNoMask && D >= 64 && p.S % 256 == 0 && (D == 64 || p.thr8 <= 0 || p.causal);
}

template <typename T, int D, bool CAUSAL, int MASK>
int launch_dq_dropout(const KParams& p, hipStream_t stream, bool with_delta) {
    if constexpr (MASK == kNoMask && D >= 64) {
        if (dq_is_phased<D, MASK>(p)) {
            const dim3 grid(p.B * p.H * (p.S / 256)), block(512);
            if constexpr (D == 64 || CAUSAL) {
                if (p.thr8 > 0) {
                    if (with_delta) hipLaunchKernelGGL((mfma_dq_phased_kernel<T, D, CAUSAL, true, true>), grid, block, 0, stream, p);
                    else hipLaunchKernelGGL((mfma_dq_phased_kernel<T, D, CAUSAL, true, false>), grid, block, 0, stream, p);
                    return static_cast<int>(hipGetLastError());
                }
            }
            if (with_delta) hipLaunchKernelGGL((mfma_dq_phased_kernel<T, D, CAUSAL, false, true>), grid, block, 0, stream, p);
            else hipLaunchKernelGGL((mfma_dq_phased_kernel<T, D, CAUSAL, false, false>), grid, block, 0, stream, p);
            return static_cast<int>(hipGetLastError());
        }
    }
    if (with_delta && MASK != kNoMask) return TRI_ATTN_ESHAPE;  // (callers ask mfma_dq_fuses_delta first)
    // 8 waves (256 query rows) when the sequence allows it, else 4 waves (128 rows)
    if constexpr (D > 16) {  // (a D = 16 tile has four blocks in all: four waves)
        if (p.S % 256 == 0) return launch_dq_waves<T, D, 8, CAUSAL, MASK>(p, stream, with_delta);
    }
    if (p.S % 128 == 0) return launch_dq_waves<T, D, 4, CAUSAL, MASK>(p, stream, with_delta);
    if constexpr (MASK == kNoMask) {  // any other length: 128-row workgroups with boundary handling
        const dim3 grid(p.B * p.H * ((p.S + 127) / 128)), block(256);
        if (with_delta) {
            if (p.thr8 > 0) hipLaunchKernelGGL((mfma_dq_kernel<T, D, 4, CAUSAL, kNoMask, true, true, false, true>), grid, block, 0, stream, p);
            else hipLaunchKernelGGL((mfma_dq_kernel<T, D, 4, CAUSAL, kNoMask, false, true, false, true>), grid, block, 0, stream, p);
        } else if (p.thr8 > 0) hipLaunchKernelGGL((mfma_dq_kernel<T, D, 4, CAUSAL, kNoMask, true, true>), grid, block, 0, stream, p);
        else hipLaunchKernelGGL((mfma_dq_kernel<T, D, 4, CAUSAL, kNoMask, false, true>), grid, block, 0, stream, p);
        return static_cast<int>(hipGetLastError());
    }
    return TRI_ATTN_ESHAPE;  // (mfma_supported keeps masked problems of such lengths away)
}

template <typename T, int D, int NW, bool CAUSAL, int MASK>
int launch_dkdv_waves(const KParams& p, hipStream_t stream) {
    const dim3 grid(p.B * p.H * (p.S / (32 * NW))), block(64 * NW);
    if (p.thr8 > 0) hipLaunchKernelGGL((mfma_dkdv_wide_kernel<T, D, NW, CAUSAL, MASK, true>), grid, block, 0, stream, p);
    else hipLaunchKernelGGL((mfma_dkdv_wide_kernel<T, D, NW, CAUSAL, MASK, false>), grid, block, 0, stream, p);
    return static_cast<int>(hipGetLastError());
}

template <typename T, int D, bool CAUSAL, int MASK>
int launch_dkdv_dropout(const KParams& p, hipStream_t stream) {
    if (p.S % 128 != 0) {
        // any length (no mask): 128-key workgroups of the 32-keys-per-wave kernel with boundary handling, for both
        // head sizes (at D = 128 with the whole register file, one workgroup per CU)
        if constexpr (MASK == kNoMask) {
            const dim3 grid(p.B * p.H * ((p.S + 127) / 128)), block(256);
            if (p.thr8 > 0) hipLaunchKernelGGL((mfma_dkdv_wide_kernel<T, D, 4, CAUSAL, kNoMask, true, true>), grid, block, 0, stream, p);
            else hipLaunchKernelGGL((mfma_dkdv_wide_kernel<T, D, 4, CAUSAL, kNoMask, false, true>), grid, block, 0, stream, p);
            return static_cast<int>(hipGetLastError());
        }
        return TRI_ATTN_ESHAPE;  // (mfma_supported keeps masked problems of such lengths away)
    }
    if constexpr (D <= 64) {
        // the two-waves-per-SIMD kernel fits its registers: 8 waves (256 keys) when the sequence
        // allows it, else 4 waves (128 keys)
        if constexpr (D > 16) {
            if (p.S % 256 == 0) return launch_dkdv_waves<T, D, 8, CAUSAL, MASK>(p, stream);
        }
        return launch_dkdv_waves<T, D, 4, CAUSAL, MASK>(p, stream);
    } else {
        // D = 128: K, V and both gradient accumulators of a 32-key block take 192 registers, too many
        // for two waves per SIMD, so two waves are paired on each key block of a 128-key workgroup
        const dim3 grid(p.B * p.H * (p.S / kBM)), block(512);
        if constexpr (MASK == kNoMask) {
            if (p.thr8 <= 0) hipLaunchKernelGGL((mfma_dkdv_phased_kernel<T, D, CAUSAL, false>), grid, block, 0, stream, p);
            else hipLaunchKernelGGL((mfma_dkdv_phased_kernel<T, D, CAUSAL, true>), grid, block, 0, stream, p);
            return static_cast<int>(hipGetLastError());
        }
        if constexpr (MASK != kNoMask && !CAUSAL) {
            // a mask that is the same for every query row (a key-padding mask) is one value per key: the phased kernel
            if (p.ms[2] == 0) {
                if (p.thr8 <= 0) hipLaunchKernelGGL((mfma_dkdv_phased_kernel<T, D, false, false, MASK>), grid, block, 0, stream, p);
                else hipLaunchKernelGGL((mfma_dkdv_phased_kernel<T, D, false, true, MASK>), grid, block, 0, stream, p);
                return static_cast<int>(hipGetLastError());
            }
        }
        if (p.thr8 > 0) hipLaunchKernelGGL((mfma_dkdv_pair_kernel<T, D, CAUSAL, MASK, true>), grid, block, 0, stream, p);
        else hipLaunchKernelGGL((mfma_dkdv_pair_kernel<T, D, CAUSAL, MASK, false>), grid, block, 0, stream, p);
        return static_cast<int>(hipGetLastError());
    }
}

template <int WHICH, typename T, int D, bool CAUSAL, int MASK>
int launch_bwd_dropout(const KParams& p, hipStream_t stream, bool with_delta) {
    if constexpr (WHICH == kMfmaDq) {
        return launch_dq_dropout<T, D, CAUSAL, MASK>(p, stream, with_delta);
    } else {
        return launch_dkdv_dropout<T, D, CAUSAL, MASK>(p, stream);
    }
}

template <int WHICH, typename T, int D>
int launch_bwd_variant(int dtype, const KParams& p, hipStream_t stream, bool with_delta) {
    if (p.causal) return launch_bwd_dropout<WHICH, T, D, true, kNoMask>(p, stream, with_delta);
    if (p.mask == nullptr) return launch_bwd_dropout<WHICH, T, D, false, kNoMask>(p, stream, with_delta);
    if (p.mask_dtype == TRI_ATTN_F32) return launch_bwd_dropout<WHICH, T, D, false, kMaskF32>(p, stream, with_delta);
    if (p.mask_dtype == dtype) return launch_bwd_dropout<WHICH, T, D, false, kMaskT>(p, stream, with_delta);
    return TRI_ATTN_EDTYPE;
}

template <int WHICH, typename T>
int launch_bwd_head(int dtype, const KParams& p, hipStream_t stream, bool with_delta) {
    if (p.D == 128) return launch_bwd_variant<WHICH, T, 128>(dtype, p, stream, with_delta);
    if (p.D == 64) return launch_bwd_variant<WHICH, T, 64>(dtype, p, stream, with_delta);
    if (p.D == 32) return launch_bwd_variant<WHICH, T, 32>(dtype, p, stream, with_delta);
    return launch_bwd_variant<WHICH, T, 16>(dtype, p, stream, with_delta);
}

template <int WHICH>
int launch_bwd(int dtype, const KParams& p, hipStream_t stream, bool with_delta) {
    return dtype == TRI_ATTN_BF16 ? launch_bwd_head<WHICH, bf16_t>(dtype, p, stream, with_delta)
                                  : launch_bwd_head<WHICH, f16_t>(dtype, p, stream, with_delta);
}

}  // namespace

int launch_mfma_dq(int dtype, const KParams& p, hipStream_t stream, bool with_delta) {
    return launch_bwd<kMfmaDq>(dtype, p, stream, with_delta);
}
int launch_mfma_dkdv(int dtype, const KParams& p, hipStream_t stream) { return launch_bwd<kMfmaDkdv>(dtype, p, stream, false); }

}  // namespace tri
