// Forward attention on the matrix cores: online-softmax flash kernel for fp16/bf16,
// D in {16,32,64,128}; any S without a mask, multiples of 128 with one (replaces trident/kernel/attention.py:33-165).
//
// A workgroup of NW waves owns 32*NW query rows, one wave 32 of them. Q stays in registers as
// the B operand of S^T = K Q^T; K and V tiles of 64 keys live row-major (swizzled) in a four-stage
// LDS ring filled by LDS-direct loads two or three tiles ahead: no staging registers, no address or
// permute arithmetic on the vector ALU, whose issue slots the softmax needs. K is read as row
// fragments, V^T through transposed LDS reads of the same row-major tile. S^T and O^T = V^T P^T
// accumulate in fp32; P goes from the S^T accumulators to the B operand of the second MFMA in
// registers. The row statistics live one per lane; the two lane halves of a row are combined
// with one cross-lane exchange per tile.
//
// With 8 waves there are two per SIMD (waves w and w+4), and they run in opposite phases: a tile is
// a softmax phase (vector ALU: maximum, exponentials, conversion, the loads of a later tile) and a
// matrix phase (P V of this tile, then S^T of the next one), with a workgroup barrier after each;
// waves 4-7 run one phase behind waves 0-3. The matrix pipe then always has a wave feeding it
// while the other wave of the SIMD occupies the vector ALU, instead of both waves doing the same
// thing at once (MFMA and vector instructions share the SIMD's issue port, and a dependent vector
// instruction waits out the ALU latency unless the other wave fills the gap). The softmax
// denominator is accumulated by the matrix pipe too (an all-ones A operand), and without dropout
// half of the exponentials are taken in the matrix phase, between the MFMAs, to balance the two.
#include <type_traits>

#include "launch.hpp"
#include "mfma_common.hpp"

namespace tri {
namespace {

constexpr int kBN = 64;      // keys per tile
constexpr float kTau = 8.f;  // lazy-rescale threshold, log2 domain

enum MaskKind { kNoMask = 0, kMaskF32 = 1, kMaskT = 2 };

// RAGGED (4 waves, no mask): S is not a multiple of 128. Query rows and keys at or beyond S do not exist: row and
// tile loads clamp their row index to S - 1, the scores of keys >= S are set to -inf, and rows >= S are not stored.
template <typename T, int D, int NW, bool CAUSAL, int MASK, bool DROPOUT, bool RAGGED = false>
__global__ __launch_bounds__(NW * 64, 2) void mfma_fwd_kernel(const KParams p) {
    static_assert(!RAGGED || (NW == 4 && MASK == 0), "ragged lengths: 4 waves, no mask");
    using Tile = SwzTile<D>;
    // An fp32 mask at D = 128 (8 waves, no dropout) needs 64 KiB of LDS for its staging regions. The ring then has
    // three slots per operand and the K tiles run one tile ahead of the V tiles: K of tile t is last read one matrix
    // phase before V of tile t, so with K(j + dist) and V(j + dist - 1) requested together every tile keeps the lead
    // it has in the ring of four, and both fit three slots.
    constexpr bool kLeadK = D == 128 && MASK == 1 && NW == 8 && !DROPOUT;
    constexpr int kStages = kLeadK ? 3 : 4;  // LDS ring depth
    constexpr int kLag = kLeadK ? 1 : 0;     // how many tiles the V requests trail the K requests
    constexpr int kBM = 32 * NW;
    constexpr int kKBytes = Tile::kBytes;
    constexpr int kStageBytes = 2 * Tile::kBytes;  // K tile, V tile
    // The ring holds the K tiles first and the V tiles behind them (slot st: K at st * kKBytes, V at kVRing + st * kKBytes):
    // every slot of an operand then lies within the 64 KiB an LDS instruction's immediate offset reaches from the lane's
    // fragment address, and with the tile loop unrolled over the slots no fragment read needs address arithmetic.
    constexpr int kVRing = kStages * Tile::kBytes;
    constexpr int kBlocksPerWave = 2 * Tile::kBlocks / NW;  // LDS-direct loads per wave and tile
    static_assert(kBlocksPerWave >= 1, "every wave fetches a piece of every tile");
    constexpr int KK = D / 16;  // K-steps of S^T
    constexpr int DB = D >= 32 ? D / 32 : 1;  // 32-row blocks of O^T (D = 16: one block whose upper 16 rows are not stored)
    constexpr int kSteps = 2 * KK;    // MFMAs of S^T per tile
    constexpr int kPvSteps = 4 * DB;  // MFMAs of O^T per tile
    // operand fragments in flight (a mask and dropout together at D = 128 leave room for four only)
    // (at D = 32 the O^T product has four steps, and the softmax phase may request fragments of tile j only: tile j + 1
    // becomes visible with the barrier behind it)
    constexpr int kRing = (D <= 32 || (D == 128 && MASK != kNoMask && DROPOUT)) ? 4 : 6;
    static_assert(kRing <= kPvSteps, "the softmax phase requests fragments of the O^T product only");
    // A mask block of a wave (32 rows x 64 keys) goes through a private LDS region (8 KiB for an fp32 mask, 4 KiB
    // for one of the operand type) when it fits (D = 64): lanes own rows, so direct loads would touch 32 cache
    // lines per instruction, while LDS-direct loads fetch whole rows (256 or 128 bytes) and the swizzled tile is
    // read back 16 or 8 bytes at a time. The region has the geometry of a 32-row SwzTile<128> / SwzTile<64>.
    constexpr bool kMaskViaLds = MASK != kNoMask && (D <= 64 || (NW == 8 && !DROPOUT));  // (D = 128: 4 KiB regions fit, 8 KiB ones do not; with dropout the registers for the staged values are not there)
    constexpr int kMaskElt = MASK == kMaskF32 ? 4 : 2;
    using MaskTile = std::conditional_t<MASK == kMaskF32, SwzTile<128>, SwzTile<64>>;
    constexpr int kMaskBytes = 32 * MaskTile::kRowBytes;
    // Without an additive mask the 8-wave kernel is persistent: one workgroup per CU walks several (head, row
    // tile) items, and requests the Q rows and the first tiles of its next item before it stores the current
    // one, so that a new item's memory latency (6 000-9 000 cycles from a workgroup's entry to its first rows)
    // passes behind the epilogue. The epilogue's transposition patches then must not lie in ring stages 0-2.
    constexpr bool kPersistent = NW == 8 && MASK == kNoMask;
    constexpr int kStoreBlocks = DB >= 2 ? 2 : 1;
    using Store = RowBlockStore<T, kStoreBlocks, D < 32 ? D : 32 * kStoreBlocks>;  // the epilogue stores 64 columns at a time (32 at D = 32, 16 at D = 16)
    constexpr int kPatchOff = kPersistent ? kVRing + 3 * Tile::kBytes : 0;  // (behind the V tile of slot 2)
    constexpr int kRingBytes = kStages * kStageBytes;
    constexpr int kPatchEnd = kPatchOff + NW * Store::kPatchBytes;
    constexpr int kSmemBytes = (kPatchEnd > kRingBytes ? kPatchEnd : kRingBytes) + (kMaskViaLds ? NW * kMaskBytes : 0);
    __shared__ __attribute__((aligned(1024))) char smem[kSmemBytes];

    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lane = tid & 63, l32 = lane & 31, h = lane >> 5;
    // the current item (head bh, row tile qt) and what follows from it
    constexpr int kOrder = CAUSAL ? kHeavyLast : kUniformTiles;
    int round = 0;
    int bh, qt;
    const int num_row_tiles = (p.S + kBM - 1) / kBM;
    const int num_key_tiles = (p.S + kBN - 1) / kBN;
    if constexpr (kPersistent) map_item(blockIdx.x, gridDim.x, 0, p.B * p.H, num_row_tiles, kOrder, &bh, &qt);
    else map_block_for<MASK>(p, blockIdx.x, num_row_tiles, kOrder, &bh, &qt);
    int b, hd, wrow0, qrow, n_tiles, my_tiles;
    const char *kbase, *vbase;
    const int64_t krow_bytes = p.ks[2] * 2, vrow_bytes = p.vs[2] * 2;
    u32x4 qf[KK];
    auto set_item = [&]() {  // (also requests the item's Q rows)
        b = bh / p.H;
        hd = bh % p.H;
        const int q0 = qt * kBM;
        wrow0 = q0 + 32 * wave;  // first query row of this wave
        qrow = wrow0 + l32;
        const int qrow_ld = RAGGED ? min(qrow, p.S - 1) : qrow;  // (a row that does not exist reads the last one)
        const char* qbase = static_cast<const char*>(p.q) + (b * p.qs[0] + hd * p.qs[1]) * 2;
        kbase = static_cast<const char*>(p.k) + (b * p.ks[0] + hd * p.ks[1]) * 2;
        vbase = static_cast<const char*>(p.v) + (b * p.vs[0] + hd * p.vs[1]) * 2;
#pragma unroll
        for (int kk = 0; kk < KK; ++kk)
            qf[kk] = *reinterpret_cast<const u32x4*>(qbase + qrow_ld * p.qs[2] * 2 + (2 * kk + h) * 16);
        n_tiles = CAUSAL ? min((q0 + kBM) / kBN, num_key_tiles) : num_key_tiles;  // tiles the workgroup streams
        my_tiles = CAUSAL ? min((wrow0 + 31) / kBN + 1, n_tiles) : n_tiles;       // tiles this wave has visible keys in
    };
    set_item();
    // With the classes of the mask's blocks at hand (tri_attn_classify_mask): key tiles behind the last one that is not
    // masked out altogether are not streamed at all, and tiles whose mask is all zero over the workgroup's rows are not
    // read (a key-padding or length mask is all zero but for one column of blocks).
    uint64_t zero_tiles = 0;
    if constexpr (MASK != kNoMask) {
        if (p.mcls != nullptr && n_tiles <= 64) {
            const TileClasses tc = tile_classes(p.mcls + b * p.mcs[0] + hd * p.mcs[1] + (qt * kBM / 64) * p.mcs[2], 1, n_tiles,
                                                kBM / 64, p.mcs[2], lane);
            zero_tiles = tc.zero;
            n_tiles = tc.active ? 64 - __builtin_clzll(tc.active) : 1;  // (fully masked rows still run one tile: NaN like softmax)
            my_tiles = n_tiles;
        }
    }
    auto mask_is_zero = [&](int t) { return MASK != kNoMask && ((zero_tiles >> t) & 1) != 0; };

    f32x16 oacc[DB];
    float m, l;  // reference exponent (log2 domain, scaled) and this lane's partial sum
    float m_use;  // m, or 0 while no key has been seen (m = -inf): what the exponents are taken against; follows m
    const float c = p.scale_log2;
    const float inv_scale = p.inv_scale;  // (a mask value joins its score before the scale: s + mask / scale)

    char* mask_lds = smem + kStages * kStageBytes + wave * kMaskBytes;
    auto issue_mask = [&](int t) {  // mask block of tile t -> this wave's region (8 LDS-direct loads), unless it is all zero
        if constexpr (kMaskViaLds) {
            if (mask_is_zero(t)) return;
            const char* src = static_cast<const char*>(p.mask) +
                              (b * p.ms[0] + hd * p.ms[1] + static_cast<int64_t>(wrow0) * p.ms[2] + t * kBN) * kMaskElt;
            int l = lane;
            asm volatile("" : "+v"(l));  // offsets recomputed per tile rather than kept in registers
#pragma unroll
            for (int blk = 0; blk < kMaskBytes / 1024; ++blk)
                lds_direct_load16(src, static_cast<uint32_t>(MaskTile::src_off(blk, l, p.ms[2] * kMaskElt)), mask_lds + blk * 1024);
        }
    };
    issue_mask(0);

    // A wave fetches blocks wave, wave + NW, ... of the K tile and of the V tile: their rows are a
    // multiple of 16 apart, so one per-lane source offset (row within the block, swizzled chunk)
    // serves all of them and the rest of the address is scalar arithmetic.
    // (D = 16 with 4 waves: a tile has two blocks per operand, waves 0-1 fetch the K tile's and waves 2-3 the V tile's)
    constexpr bool kSplitOperands = Tile::kBlocks < NW;
    constexpr int kPerOperand = kSplitOperands ? 1 : Tile::kBlocks / NW;
    constexpr int kRowStep = NW * Tile::kRowsPerBlock;
    static_assert(kRowStep % 16 == 0 && (kSplitOperands ? kBlocksPerWave == 1 && 2 * Tile::kBlocks == NW && !kLeadK
                                                        : 2 * kPerOperand == kBlocksPerWave), "block assignment");
    const int my_block = kSplitOperands ? wave % Tile::kBlocks : wave;
    const uint32_t koff = static_cast<uint32_t>(Tile::src_off(my_block, lane, krow_bytes));
    const uint32_t voff = static_cast<uint32_t>(Tile::src_off(my_block, lane, vrow_bytes));
    // load number idx (0 .. kBlocksPerWave-1) of this wave's share of the K tile t (the first kPerOperand) and of the V
    // tile t - kLag (the others) -> ring slot (tile % kStages) of the operand
    auto issue_load = [&](int tk, int idx) {
        const int t = idx < kPerOperand ? tk : tk - kLag;
        char* stage = smem + (t % kStages) * kKBytes + my_block * 1024;
        if constexpr (kSplitOperands) {  // (this wave's one load: a block of the K tile or of the V tile)
            const int last = p.S - 1 - t * kBN;
            const bool partial = RAGGED && (t + 1) * kBN > p.S;
            if (wave < Tile::kBlocks)
                lds_direct_load16(kbase + static_cast<int64_t>(t) * kBN * krow_bytes,
                                  partial ? Tile::src_off_clamped(my_block, lane, krow_bytes, last) : koff, stage);
            else
                lds_direct_load16(vbase + static_cast<int64_t>(t) * kBN * vrow_bytes,
                                  partial ? Tile::src_off_clamped(my_block, lane, vrow_bytes, last) : voff, stage + kVRing);
            return;
        }
        const int i = idx % kPerOperand;
        if (RAGGED && (t + 1) * kBN > p.S) {  // the sequence ends inside this tile: clamped rows, offsets from the tile's first row
            const int last = p.S - 1 - t * kBN;
            if (idx < kPerOperand)
                lds_direct_load16(kbase + static_cast<int64_t>(t) * kBN * krow_bytes,
                                  Tile::src_off_clamped(wave + i * NW, lane, krow_bytes, last), stage + i * NW * 1024);
            else
                lds_direct_load16(vbase + static_cast<int64_t>(t) * kBN * vrow_bytes,
                                  Tile::src_off_clamped(wave + i * NW, lane, vrow_bytes, last), stage + kVRing + i * NW * 1024);
        } else if (idx < kPerOperand)
            lds_direct_load16(kbase + (static_cast<int64_t>(t) * kBN + i * kRowStep) * krow_bytes, koff, stage + i * NW * 1024);
        else
            lds_direct_load16(vbase + (static_cast<int64_t>(t) * kBN + i * kRowStep) * vrow_bytes, voff, stage + kVRing + i * NW * 1024);
    };
    // The loads of a tile are issued in four slices spread over the softmax phase: a wave stalls on a
    // load until the memory pipeline accepts it, and sixteen loads arriving at once from the four
    // waves of a group queue up for hundreds of cycles.
    // (k_ok / v_ok: the K tile t / the V tile t - kLag exists)
    auto issue_slice = [&](int t, int part, bool k_ok = true, bool v_ok = true) {
#pragma unroll
        for (int idx = 0; idx < kBlocksPerWave; ++idx)
            if (idx % 4 == part && (idx < kPerOperand ? k_ok : v_ok)) issue_load(t, idx);
    };
    auto issue_tile = [&](int t, bool k_ok = true, bool v_ok = true) {
#pragma unroll
        for (int part = 0; part < 4; ++part) issue_slice(t, part, k_ok, v_ok);
    };
    // Ping-pong schedule (8 waves): waves w and w+4 share a SIMD. The loop alternates a softmax
    // phase (vector ALU only) and a matrix phase (P V of this tile, then S^T of the next), with a
    // barrier after each; the waves of group 1 run one phase behind those of group 0, so that a SIMD
    // always has one wave issuing MFMAs and one issuing vector instructions instead of both doing
    // the same thing at once. Group 0 may request tiles 2 ahead, group 1 (one phase later) 3 ahead.
    constexpr bool kPingPong = NW == 8;
    const int group = kPingPong ? wave >> 2 : 0;
    const int dist = 2 + group;
    // all but the youngest (mask block, tile requests: of both operands, of the V tile only, none) have landed
    auto wait_loads = [&](bool mask_block, bool tile, bool tile_v = false) {
        constexpr int kM = kMaskBytes / 1024, kB = kBlocksPerWave;
        if (mask_block && tile) TRI_WAIT_VMCNT(kM + kB);
        else if (mask_block && kLeadK && tile_v) TRI_WAIT_VMCNT(kM + kPerOperand);
        else if (mask_block) TRI_WAIT_VMCNT(kM);
        else if (tile) TRI_WAIT_VMCNT(kB);
        else if (kLeadK && tile_v) TRI_WAIT_VMCNT(kPerOperand);
        else TRI_WAIT_VMCNT(0);
    };
    int n_first;
    auto request_first_tiles = [&]() {  // (the Q rows were requested before, so both latencies overlap)
        n_first = min(dist, n_tiles);                    // K tiles 0 .. n_first - 1
        const int v_first = min(dist - kLag, n_tiles);   // V tiles 0 .. v_first - 1
#pragma unroll
        for (int t = 0; t < 3; ++t) {
            const bool k_ok = t < n_first, v_ok = t - kLag >= 0 && t - kLag < v_first;
            if (k_ok || v_ok) issue_tile(t, k_ok, v_ok);
        }
    };
    request_first_tiles();

    int row_off0 = Tile::off(l32, h);
    int tr_off0 = kVRing + Tile::tr_off(0, 0, lane), tr_off1 = kVRing + Tile::tr_off(0, 1, lane);  // (from the K ring's slot st)
    // fragment s of the S^T operand (key block s / KK, K-step s % KK) and of the O^T operand
    // (K-step s / DB = 16 keys, column block s % DB)
    auto k_frag = [&](const char* sK, int s) { return lds_read16(sK, (row_off0 ^ ((s % KK) << 5)) + 32 * (s / KK) * Tile::kRowBytes); };
    auto v_frag = [&](const char* sV, int s) { return Tile::tr_frag(sV, tr_off0 ^ ((s % DB) << 6), tr_off1 ^ ((s % DB) << 6), s / DB); };

    f32x16 sc[2];  // scores of this lane: sc[kb][i] is key t0 + 32*kb + c_row(i,h)
    float mk[MASK != kNoMask ? 32 : 1];

    // additive mask values of this lane's row for tile t, straight from memory
    auto load_mask = [&](int t) {
        if constexpr (MASK != kNoMask && !kMaskViaLds) {
            if (mask_is_zero(t)) return;  // (the tile then takes the arithmetic of a tile without a mask: mk is not read)
            const int64_t mrow = b * p.ms[0] + hd * p.ms[1] + static_cast<int64_t>(qrow) * p.ms[2] + t * kBN;
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
    };
    // mask block t from this wave's LDS region, then the request for block t+1
    auto take_mask_block = [&](int t, bool first, bool tile_in_flight, bool v_in_flight = false) {
        if constexpr (kMaskViaLds) {
            // block t was requested a matrix phase ago and only the newest tile load may be younger
            // (block 0 precedes tile 0, which has landed)
            if (!mask_is_zero(t)) {
                if (!first) wait_loads(false, tile_in_flight, v_in_flight);
#pragma unroll
                for (int g = 0; g < 8; ++g) {  // keys 32 (g / 4) + 8 (g % 4) + 4 h .. + 3 of this lane's row
                    if constexpr (MASK == kMaskF32) {
                        const f32x4 v = *reinterpret_cast<const f32x4*>(mask_lds + MaskTile::off(l32, 8 * (g >> 2) + 2 * (g & 3) + h));
                        mk[4 * g + 0] = v.x; mk[4 * g + 1] = v.y; mk[4 * g + 2] = v.z; mk[4 * g + 3] = v.w;
                    } else {
                        const u32x2 v = *reinterpret_cast<const u32x2*>(mask_lds + MaskTile::off(l32, 4 * (g >> 2) + (g & 3)) + 8 * h);
                        mk[4 * g + 0] = Mma<T>::lo(v.x); mk[4 * g + 1] = Mma<T>::hi(v.x);
                        mk[4 * g + 2] = Mma<T>::lo(v.y); mk[4 * g + 3] = Mma<T>::hi(v.y);
                    }
                }
            }
            // the values are in registers: the region can take the next block
            if (t + 1 < my_tiles && !mask_is_zero(t + 1)) {
                asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                issue_mask(t + 1);
            }
        }
    };
    // The matrix phase of tile j: O^T += V^T P^T (steps 0 .. kPvSteps-1, skipped when WITH_PV is
    // false) and then S^T = K Q^T of tile j+1 (when WITH_S). All A operands come through one ring of
    // fragments requested kRing MFMAs before their use, across the boundary between the two products;
    // the caller has requested the first kRing fragments.
    u32x4 ring[kRing];
    u32x4 pb[4];
    // Without dropout the softmax denominator is accumulated by the matrix pipe as well: an all-ones
    // A operand makes every row of the product the column sums of P^T, i.e. each lane holds (16
    // times) the sum over ALL keys of its query row, taken from the same rounded P that multiplies
    // V. With dropout the sum has to be taken before elements are dropped, on the vector ALU.
    // Without dropout the exponentials of the second key block (and their conversion) are deferred into
    // the matrix phase, one or two per MFMA of the first key block's P V steps: that phase has issue slots
    // to spare, the softmax phase is the one the partner waits for.
    constexpr bool kDefer = !DROPOUT;
    float xd[16];        // deferred exponents and then probabilities
    float m_def = 0.f;   // the reference exponent they are taken against
    const uint32_t one2 = Mma<T>::pack2(1.f, 1.f);
    u32x4 ones = {one2, one2, one2, one2};
    asm volatile("" : "+v"(ones));  // (kept in registers: as a constant it would be made anew from scalars in every tile)
    f32x16 lacc = zero16();
    // (st: the ring slot of tile j, a literal at every call)
    auto frag = [&](auto with_pv, int st, int s) __attribute__((always_inline)) {
        constexpr int pv = decltype(with_pv)::value ? kPvSteps : 0;
        return s < pv ? v_frag(smem + st * kKBytes, s) : k_frag(smem + ((st + 1) % kStages) * kKBytes, s - pv);
    };
    auto matrix_phase = [&](auto with_pv, auto with_s, int st, bool do_s = true) __attribute__((always_inline)) {
        constexpr int pv = decltype(with_pv)::value ? kPvSteps : 0;
        constexpr int total = pv + (decltype(with_s)::value ? kSteps : 0);
        if constexpr (decltype(with_s)::value) {
            sc[0] = zero16();
            sc[1] = zero16();
        }
#pragma unroll
        for (int s = 0; s < total; ++s) {
            if (s >= pv && !do_s) break;
            if (s < pv) {
                oacc[s % DB] = Mma<T>::run(ring[s % kRing], pb[s / DB], oacc[s % DB]);
                // row sums of P (every accumulator row gets the same sum over the 16 keys)
                if (!DROPOUT && s % DB == DB - 1) lacc = Mma<T>::run(ones, pb[s / DB], lacc);
            } else {
                const int s2 = s - pv;
                sc[s2 / KK] = Mma<T>::run(ring[s % kRing], qf[s2 % KK], sc[s2 / KK]);
            }
            if (s + kRing < total) {
                const int n = s + kRing;
                ring[s % kRing] = frag(with_pv, st, n);
            }
            if constexpr (kDefer && pv > 0) {
                // group 2 (B operand of K-step 2, first used at step 2 DB) during steps 0 .. 2 DB - 1,
                // group 3 (first used at step 3 DB) during steps 2 DB .. 3 DB - 1
                if (s < 3 * DB) {
                    const int g = s < 2 * DB ? 2 : 3;
                    const int w0 = g == 2 ? 0 : 2 * DB, n = g == 2 ? 2 * DB : DB;
                    const int ne = n > 2 ? n - 2 : 1;           // steps that take exponentials
                    const int pack_step = ne < n - 1 ? ne : n - 1;
                    const int ls = s - w0;
#pragma unroll
                    for (int e = 0; e < 8; ++e)
                        if (e * ne / 8 == ls) {
                            float& v = xd[8 * (g - 2) + e];
                            v = fast_exp2(fmaf(v, c, -m_def));
                        }
                    if (ls == pack_step) pb[g] = pack8<T>(&xd[8 * (g - 2)]);
                }
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    using Yes = std::integral_constant<bool, true>;
    using No = std::integral_constant<bool, false>;

    for (bool first_item = true;; first_item = false) {  // one pass per item
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) settle(qf[kk]);
#pragma unroll
    for (int db = 0; db < DB; ++db) oacc[db] = zero16();
    lacc = zero16();
    m = -INFINITY;
    m_use = 0.f;
    l = 0.f;
    // tile 0 has landed and is visible to all waves (a later item's requests are older than the stores of the
    // item before it: everything is awaited)
    if (!first_item || kLeadK) TRI_WAIT_VMCNT(0);  // (the K-leading ring requests in another order: it awaits everything)
    else if (n_first == 3) TRI_WAIT_VMCNT(2 * kBlocksPerWave);
    else if (n_first == 2) TRI_WAIT_VMCNT(kBlocksPerWave);
    else TRI_WAIT_VMCNT(0);
    lds_barrier();
    if (kPingPong && group == 1) {
        // group 1 starts one phase late; group 0 reads tile 1 in its first matrix phase
        if (first_item && n_first == 3 && !kLeadK) TRI_WAIT_VMCNT(kBlocksPerWave);
        else TRI_WAIT_VMCNT(0);
        lds_barrier();
    }
    {
        load_mask(0);
#pragma unroll
        for (int r = 0; r < (kRing < kSteps ? kRing : kSteps); ++r) ring[r] = frag(No{}, kStages - 1, r);
        __builtin_amdgcn_sched_barrier(0);
        matrix_phase(No{}, Yes{}, kStages - 1);
        take_mask_block(0, true, false);
    }

    // A wave computes on its first my_tiles tiles (all of them without a causal mask) and afterwards
    // only keeps fetching its share of the remaining tiles and meeting the barriers.
    // One step of the tile loop; st = j % kStages is a literal at each of the loop's four calls.
    auto tile_step = [&](const int j, const int st) __attribute__((always_inline)) {
        // slot of tile j+dist: every wave is done with the tile it held (two barriers ago at the latest)
        const bool issued = j + dist < n_tiles;            // the K tile requested in this step exists
        const bool issued_v = j + dist - kLag < n_tiles;   // ... its V tile (the same tile, or the one before it)
        if (issued_v) issue_slice(j + dist, 0, issued, issued_v);
        const int t0 = j * kBN;
        constexpr bool active = true;

        if (active) {
            float x[32];
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                x[i] = sc[0][i];
                x[16 + i] = sc[1][i];
            }
            // The scale (to the log2 domain) is folded into the exponent's multiply-add; a mask value is added before it,
            // divided by the scale: one multiply-add per score, none in a tile whose mask is all zero.
            if constexpr (MASK != kNoMask) {
                if (!mask_is_zero(j)) {
#pragma unroll
                    for (int e = 0; e < 32; ++e) x[e] = fmaf(mk[e], inv_scale, x[e]);
                }
            }
            if (CAUSAL && t0 + kBN - 1 > wrow0) {
#pragma unroll
                for (int e = 0; e < 32; ++e) {
                    const int key = t0 + 32 * (e >> 4) + c_row(e & 15, h);
                    x[e] = key <= qrow ? x[e] : -INFINITY;
                }
            }
            if (RAGGED && !CAUSAL && t0 + kBN > p.S) {  // keys that do not exist (under the causal mask no existing row sees them)
#pragma unroll
                for (int e = 0; e < 32; ++e) {
                    const int key = t0 + 32 * (e >> 4) + c_row(e & 15, h);
                    x[e] = key < p.S ? x[e] : -INFINITY;
                }
            }
            // two chains (a dependent maximum waits out the ALU latency) of three-operand maxima, written out: through
            // fmaxf the compiler first canonicalises the operands of each chain (a maximum of a value with itself)
            float mx = max3(x[0], x[1], x[2]), mx1 = max3(x[16], x[17], x[18]);
#pragma unroll
            for (int e = 3; e < 15; e += 2) {
                mx = max3(mx, x[e], x[e + 1]);
                mx1 = max3(mx1, x[16 + e], x[17 + e]);
            }
            mx = max_xor32(max3(mx, x[15], max3(mx1, x[31], x[31])));
            mx *= c;
            // Lazy rescaling: m is the reference exponent of l and of the O accumulators, not
            // necessarily the running maximum. It is only moved (and O rescaled) when some row of
            // the wave outgrew it by more than 2^kTau; until then probabilities may exceed 1 by
            // that factor, which fp32 sums and 16-bit P hold without loss.
            if (__builtin_amdgcn_ballot_w64(mx > m + kTau) != 0) {
                const float m_new = fmaxf(m, mx);
                m_use = m_new == -INFINITY ? 0.f : m_new;
                const float alpha = fast_exp2(m - m_use);
                l *= alpha;
                m = m_new;
#pragma unroll
                for (int db = 0; db < DB; ++db)
#pragma unroll
                    for (int i = 0; i < 16; ++i) oacc[db][i] *= alpha;
                if constexpr (!DROPOUT) {
#pragma unroll
                    for (int i = 0; i < 16; ++i) lacc[i] *= alpha;
                }
            }
            // exponentials in four groups of eight keys (one B operand each); the remaining loads of the
            // next tile and the first fragment reads of the matrix phase (tile j has been visible since
            // the previous barrier) are issued between the groups, so that none of them queues
            if (issued_v) issue_slice(j + dist, 1, issued, issued_v);
            constexpr int kNow = kDefer ? 2 : 4;  // groups whose exponentials are taken here
#pragma unroll
            for (int ks = 0; ks < kNow; ++ks) {
#pragma unroll
                for (int e = 8 * ks; e < 8 * ks + 8; ++e) {
                    x[e] = fast_exp2(fmaf(x[e], c, -m_use));
                }
                if constexpr (!DROPOUT) pb[ks] = pack8<T>(&x[8 * ks]);
                if (ks < 2 && issued_v) issue_slice(j + dist, 2 + ks, issued, issued_v);
                if (ks < 2) {
#pragma unroll
                    for (int r = kRing / 2 * ks; r < kRing / 2 * (ks + 1); ++r) ring[r] = frag(Yes{}, st, r);
                }
                __builtin_amdgcn_sched_barrier(0);
            }
            if constexpr (kDefer) {
#pragma unroll
                for (int e = 0; e < 16; ++e) xd[e] = x[16 + e];
                m_def = m_use;
            }
            if constexpr (DROPOUT) {
                // row sum before dropping, in fp32: four interleaved partial sums (a dependent add waits
                // out the ALU latency)
                float ps[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int e = 0; e < 32; ++e) ps[e & 3] += x[e];
                l += (ps[0] + ps[1]) + (ps[2] + ps[3]);
            }
            if constexpr (DROPOUT) {
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
                            x[16 * kb + 4 * g + bb] = keep ? x[16 * kb + 4 * g + bb] : 0.f;  // (the 1 / (1 - p) factor: at the end)
                        }
                }
            }
            if constexpr (DROPOUT) {
                // P as B operands
#pragma unroll
                for (int ks = 0; ks < 4; ++ks) pb[ks] = pack8<T>(&x[8 * ks]);
            }
        }
        static_assert(kRing % 2 == 0, "the softmax phase requests the first fragments in two halves");

        const bool with_s = j + 1 < my_tiles;
        // tile j+dist-1 has landed (the next mask block and the newest tile may still be in flight);
        // after the barrier it is visible to every wave, and the partner group changes phase. The
        // fragment reads stay in flight across the barrier: nothing overwrites their slot before the
        // barrier after next.
        wait_loads(kMaskViaLds && with_s && !mask_is_zero(j + 1), issued, issued_v);
        __builtin_amdgcn_sched_barrier(0);
        asm volatile("s_barrier" ::: "memory");
        __builtin_amdgcn_sched_barrier(0);

        if (active) {
            // (a wave's last tile has no successor to score and leaves the S^T steps out; with dropout it runs
            // them on whatever the next slot holds, the result is never used: the branch would cost registers
            // that variant does not have)
            if (with_s) load_mask(j + 1);
            // the few instructions of this phase go first, so that the matrix pipe never waits for an
            // issue slot behind the partner's vector work
            __builtin_amdgcn_s_setprio(2);
            matrix_phase(Yes{}, Yes{}, st, with_s || DROPOUT);
            __builtin_amdgcn_s_setprio(0);
            if (with_s) take_mask_block(j + 1, false, issued, issued_v);
        }
        if constexpr (kPingPong) {
            __builtin_amdgcn_sched_barrier(0);
            lds_barrier();
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    static_assert(kStages == 4 || kStages == 3, "the tile loop is unrolled over the ring's slots");
    // (a mask and dropout together at D = 128 have no registers to spare for four copies of the step: rolled, the slot
    // is a run-time value there and every fragment read adds it to its address)
    constexpr bool kUnrolled = !(D == 128 && MASK != kNoMask && DROPOUT);
    if constexpr (kUnrolled && kStages == 3) {
        for (int j = 0; j < my_tiles; j += 3) {
            tile_step(j, 0);
            if (j + 1 < my_tiles) tile_step(j + 1, 1);
            if (j + 2 < my_tiles) tile_step(j + 2, 2);
        }
    } else if constexpr (kUnrolled) {
        for (int j = 0; j < my_tiles; j += 4) {
            tile_step(j, 0);
            if (j + 1 < my_tiles) tile_step(j + 1, 1);
            if (j + 2 < my_tiles) tile_step(j + 2, 2);
            if (j + 3 < my_tiles) tile_step(j + 3, 3);
        }
    } else {
        for (int j = 0; j < my_tiles; ++j) tile_step(j, j % kStages);
    }
    for (int j = my_tiles; j < n_tiles; ++j) {
        const bool issued = j + dist < n_tiles, issued_v = j + dist - kLag < n_tiles;
        if (issued_v) issue_tile(j + dist, issued, issued_v);
        wait_loads(false, issued, issued_v);
        lds_barrier();
        if constexpr (kPingPong) lds_barrier();
    }
    if (kPingPong && group == 0) lds_barrier();  // group 1 is still in its last matrix phase

    l = DROPOUT ? sum_xor32(l) : lacc[0];
    const float inv = (DROPOUT ? p.zscale : 1.f) / l;
    // every wave is out of the loop: the ring is free (for the waves' private transposition patches, and for
    // the first tiles of the next item)
    lds_barrier();
    char* o0 = static_cast<char*>(p.o) + (b * p.os[0] + hd * p.os[1] + static_cast<int64_t>(wrow0) * p.os[2]) * 2;
    float* lse_out = p.lse + static_cast<int64_t>(bh) * p.S + qrow;
    bool more = false;
    if constexpr (kPersistent) {
        more = map_item(blockIdx.x, gridDim.x, ++round, p.B * p.H, p.S / kBM, kOrder, &bh, &qt);
        if (more) {
            set_item();
            request_first_tiles();
        }
    }
    {
        static_assert(DB % kStoreBlocks == 0, "whole stores");
        char* patch = smem + kPatchOff + wave * Store::kPatchBytes;
#pragma unroll
        for (int cb = 0; cb < DB / kStoreBlocks; ++cb) {
            if (cb) asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // patch read before it is rewritten
            const f32x16(&part)[kStoreBlocks] = *reinterpret_cast<const f32x16(*)[kStoreBlocks]>(&oacc[kStoreBlocks * cb]);
            Store::run(part, [inv](float x) { return x * inv; }, patch, o0 + cb * 128, p.os[2] * 2, lane,
                       RAGGED ? p.S - wrow0 : 32);
        }
    }
    if (h == 0 && (!RAGGED || qrow < p.S)) *lse_out = m + fast_log2(l);
    if (!more) break;
    }
}

template <typename T, int D, bool CAUSAL>
int launch_fwd_ragged(const KParams& p, hipStream_t stream) {
    const dim3 grid(p.B * p.H * ((p.S + 127) / 128)), block(256);
    if (p.thr8 > 0) hipLaunchKernelGGL((mfma_fwd_kernel<T, D, 4, CAUSAL, kNoMask, true, true>), grid, block, 0, stream, p);
    else hipLaunchKernelGGL((mfma_fwd_kernel<T, D, 4, CAUSAL, kNoMask, false, true>), grid, block, 0, stream, p);
    return static_cast<int>(hipGetLastError());
}

template <typename T, int D, int NW, bool CAUSAL, int MASK>
int launch_fwd_dropout(const KParams& p, hipStream_t stream) {
    const int items = p.B * p.H * (p.S / (32 * NW));
    // (the kernel's kPersistent: one workgroup per CU walks the items)
    const dim3 grid(NW == 8 && MASK == kNoMask ? persistent_grid(items) : items), block(64 * NW);
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
    // 8 waves (256 query rows) when the sequence allows it: two waves per SIMD out of phase. At D = 32 the vector ALU
    // is the busy unit and a workgroup's phases are short: four independent 4-wave workgroups per CU (the kernel then
    // fits 128 registers) measured 28 % faster than the 8-wave pairs.
    if constexpr (D > 32) {
        if (p.S % 256 == 0) return launch_fwd_variant<T, D, 8>(dtype, p, stream);
    }
    if (p.S % 128 == 0) return launch_fwd_variant<T, D, 4>(dtype, p, stream);
    // any other length (no mask: mfma_supported): 128-row workgroups with boundary handling
    return p.causal ? launch_fwd_ragged<T, D, true>(p, stream) : launch_fwd_ragged<T, D, false>(p, stream);
}

template <typename T>
int launch_fwd_head(int dtype, const KParams& p, hipStream_t stream) {
    if (p.D == 128) return launch_fwd_waves<T, 128>(dtype, p, stream);
    if (p.D == 64) return launch_fwd_waves<T, 64>(dtype, p, stream);
    if (p.D == 32) return launch_fwd_waves<T, 32>(dtype, p, stream);
    return launch_fwd_waves<T, 16>(dtype, p, stream);
}

}  // namespace

int launch_mfma_fwd(int dtype, const KParams& p, hipStream_t stream) {
    return dtype == TRI_ATTN_BF16 ? launch_fwd_head<bf16_t>(dtype, p, stream) : launch_fwd_head<f16_t>(dtype, p, stream);
}

}  // namespace tri
