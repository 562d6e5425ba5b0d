// Building blocks of the matrix-core (MFMA) attention kernels for gfx950.
//
// All three kernels (forward, dQ, dK/dV) use v_mfma_f32_32x32x16_{bf16,f16}:
//   A is 32(M) x 16(K): lane l holds row M = l % 32 and the 8 K-slots 8*(l/32) .. 8*(l/32)+7
//   B is 16(K) x 32(N): lane l holds column N = l % 32 and the same 8 K-slots
//   C/D is 32 x 32 fp32: lane l holds column N = l % 32 and, in register i (0..15),
//   row M = 8*(i/4) + 4*(l/32) + i%4.
// The kernels are written "transposed" (S^T = K Q^T, O^T = V^T P^T, ...) so that the lane
// index is always the row the softmax statistics belong to: row maxima, sums, the LSE and
// delta are per-lane scalars, and a C tile can be fed back as the B operand of the next
// MFMA without leaving registers: registers 8g .. 8g+7 of a C tile, converted to 16 bit,
// are the 8 K-slots of K-step g; slot t of lane-half h then stands for tile row
// 16g + 8*(t/4) + 4h + t%4, and the A operand of that MFMA must present its K dimension in
// exactly that slot order, which is what the transposed LDS reads of SwzTile below deliver.
#pragma once
#include "common.hpp"

namespace tri {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef bf16_t bf16x8 __attribute__((ext_vector_type(8)));
typedef f16_t f16x8 __attribute__((ext_vector_type(8)));
typedef bf16_t bf16x2 __attribute__((ext_vector_type(2)));
typedef f16_t f16x2 __attribute__((ext_vector_type(2)));

template <typename T>
struct Mma;
template <>
struct Mma<bf16_t> {
    static __device__ __forceinline__ f32x16 run(u32x4 a, u32x4 b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c,
                                                       0, 0, 0);
    }
    static __device__ __forceinline__ uint32_t pack2(float lo, float hi) {
        bf16x2 v = {static_cast<bf16_t>(lo), static_cast<bf16_t>(hi)};
        return __builtin_bit_cast(uint32_t, v);
    }
    static __device__ __forceinline__ float lo(uint32_t w) { return __uint_as_float(w << 16); }
    static __device__ __forceinline__ float hi(uint32_t w) { return __uint_as_float(w & 0xffff0000u); }
    // acc + lo(w) + hi(w) in one instruction (v_dot2c_f32_bf16 against (1, 1))
    static __device__ __forceinline__ float add_pair(uint32_t w, float acc) {
        const bf16x2 ones = {static_cast<bf16_t>(1.0f), static_cast<bf16_t>(1.0f)};
        return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, w), ones, acc, false);
    }
};
template <>
struct Mma<f16_t> {
    static __device__ __forceinline__ f32x16 run(u32x4 a, u32x4 b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0,
                                                      0, 0);
    }
    static __device__ __forceinline__ uint32_t pack2(float lo, float hi) {
        f16x2 v = {static_cast<f16_t>(lo), static_cast<f16_t>(hi)};
        return __builtin_bit_cast(uint32_t, v);
    }
    static __device__ __forceinline__ float lo(uint32_t w) {
        return static_cast<float>(__builtin_bit_cast(f16x2, w)[0]);
    }
    static __device__ __forceinline__ float hi(uint32_t w) {
        return static_cast<float>(__builtin_bit_cast(f16x2, w)[1]);
    }
    static __device__ __forceinline__ float add_pair(uint32_t w, float acc) {
        const f16x2 ones = {static_cast<f16_t>(1.0f), static_cast<f16_t>(1.0f)};
        return __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2, w), ones, acc, false);
    }
};

// 8 consecutive C registers -> one B operand (8 K-slots) in the 16-bit type.
template <typename T>
__device__ __forceinline__ u32x4 pack8(const float* x) {
    u32x4 r;
    r.x = Mma<T>::pack2(x[0], x[1]);
    r.y = Mma<T>::pack2(x[2], x[3]);
    r.z = Mma<T>::pack2(x[4], x[5]);
    r.w = Mma<T>::pack2(x[6], x[7]);
    return r;
}

// x as three 16-bit terms (K-slots 0-2 of an operand, the rest zero): their sum restores x to fp32 precision.
template <typename T>
__device__ __forceinline__ u32x4 split3(float x) {
    const float a = static_cast<float>(static_cast<T>(x));
    const float r1 = x - a;
    const float b = static_cast<float>(static_cast<T>(r1));
    u32x4 r;
    r.x = Mma<T>::pack2(a, b);
    r.y = Mma<T>::pack2(r1 - b, 0.f);
    r.z = r.w = 0;
    return r;
}

__device__ __forceinline__ f32x16 zero16() {
    f32x16 z;
#pragma unroll
    for (int i = 0; i < 16; ++i) z[i] = 0.f;
    return z;
}

// Row index inside a 32-row C tile of register i for lane-half h.
__device__ __forceinline__ int c_row(int i, int h) { return 8 * (i >> 2) + 4 * h + (i & 3); }

__device__ __forceinline__ float xor32(float x) { return __shfl_xor(x, 32); }
// max / sum of a value with the one in lane ^ 32, exchanged on the vector ALU (no LDS round trip):
// the swap leaves {x[l % 32], x[l % 32 + 32]} in the two registers of every lane. The instruction
// needs two wait states after a vector write of its operands.
__device__ __forceinline__ void swap32(float& a, float& b) { asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1" : "+v"(a), "+v"(b)); }
// v_max3_f32 as it stands (scores are never signalling NaNs; fmaxf would canonicalise its operands first)
__device__ __forceinline__ float max3(float a, float b, float c) {
    float r;
    asm("v_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
    return r;
}
__device__ __forceinline__ float max_xor32(float x) { float a = x, b = x; swap32(a, b); return max3(a, b, b); }
__device__ __forceinline__ float sum_xor32(float x) { float a = x, b = x; swap32(a, b); return a + b; }

// ---------------------------------------------------------------- LDS access
__device__ __forceinline__ u32x4 lds_read16(const char* smem, int off) {
    return *reinterpret_cast<const u32x4*>(smem + off);
}
__device__ __forceinline__ void lds_write8(char* smem, int off, u32x2 v) { *reinterpret_cast<u32x2*>(smem + off) = v; }

// ---------------------------------------------------------------- swizzled tiles filled by LDS-direct loads
// Row-major tile [64][D] of 16-bit elements without padding, filled straight from HBM with
// global_load_lds_dwordx4 (no registers, no ds_write): one wave instruction deposits 64 x 16
// bytes at consecutive LDS addresses, so a lane can only choose WHICH 16-byte chunk of its row it
// fetches, and the bank-conflict-free layout is an XOR swizzle of the chunk index with the row.
// Both operand forms are read from the same tile:
//   row fragment   A[M = tile row][K = column]: one ds_read_b128 (rows r..r+31, chunk 2kk+h)
//   transposed     A[M = column][K = tile row]: two ds_read_b64_tr_b16; in each 16-lane group
//                  lane i receives the element (column base + i) of 4 consecutive tile rows
//                  when lane j points at row (base + j/4), columns 4*(j%4) .. +3.
// The transposed form yields the K-slot order of the C registers (see the top of this file)
// without any permuted storage.
typedef short s16x4 __attribute__((ext_vector_type(4)));

// LDS-direct loads and the matching barrier, issued through inline assembly. The compiler's own
// intrinsic for these loads is correct but pessimistic: it cannot tell which LDS reads depend on
// a load in flight, so it drains the vector-memory counter before the next LDS read and before
// every __syncthreads(), which turns a prefetch several tiles deep into a synchronous copy.
// Kernels that use these helpers order the loads themselves: TRI_WAIT_VMCNT(n) for "all but the
// last n loads have landed", then lds_barrier() to make them (and ordinary LDS writes) visible
// to the other waves. `base` and `lds_dst` must be uniform across the wave (they travel in scalar
// registers); a lane reads at base + lane_off (unsigned 32-bit byte offset) and its 16 (4) bytes
// land at lds_dst + 16*l (4*l). M0 holds the LDS address and needs one wait state before the load.
// LDS byte address of a pointer into __shared__ memory: the shared aperture is 4 GiB aligned, so the
// low half of the generic address is the LDS offset (no address-space cast, hence no null check).
__device__ __forceinline__ uint32_t lds_address(const void* p) { return static_cast<uint32_t>(reinterpret_cast<uintptr_t>(p)); }
__device__ __forceinline__ void lds_direct_load16(const void* base, uint32_t lane_off, const void* lds_dst) {
    const uint32_t dst = __builtin_amdgcn_readfirstlane(lds_address(lds_dst));
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" : : "s"(dst), "v"(lane_off), "s"(base) : "memory", "m0");
}
__device__ __forceinline__ void lds_direct_load4(const void* base, uint32_t lane_off, const void* lds_dst) {
    const uint32_t dst = __builtin_amdgcn_readfirstlane(lds_address(lds_dst));
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, %2" : : "s"(dst), "v"(lane_off), "s"(base) : "memory", "m0");
}
// Makes the compiler wait HERE for a value that an earlier global load produces. Otherwise the
// wait lands at the first use, which may be inside a loop that keeps LDS-direct loads in flight;
// the compiler does not know about those and its wait would drain them on every iteration.
template <typename V>
__device__ __forceinline__ void settle(const V& v) { asm volatile("" : : "v"(v)); }
// Workgroup barrier that waits for this wave's LDS traffic only, not for loads still in flight.
__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" : : : "memory"); }

template <int D>
struct SwzTile {
    static constexpr int kRowBytes = D * 2;
    static constexpr int kChunks = D / 8;               // 16-byte chunks per row
    static constexpr int kBytes = 64 * kRowBytes;       // 16 KiB (D=128) or 8 KiB (D=64)
    static constexpr int kBlocks = kBytes / 1024;       // wave instructions per tile
    static constexpr int kRowsPerBlock = 1024 / kRowBytes;
    // chunk swizzle: 16 consecutive rows (b128 reads) and 4 consecutive rows x 32 bytes (tr reads)
    // land in distinct banks
    static __device__ __forceinline__ int swz(int r) {
        if constexpr (D == 128) return ((r & 7) << 1) | ((r >> 3) & 1);
        else if constexpr (D == 32) return (r >> 2) & 3;  // (64-byte rows, four chunks: four rows fill the 64 banks once)
        else if constexpr (D == 16) return (r >> 3) & 1;  // (32-byte rows, two chunks: eight rows fill the banks once)
        else return (((r >> 1) & 3) << 1) | ((r >> 3) & 1);
    }
    static __device__ __forceinline__ int off(int r, int c) { return r * kRowBytes + ((c ^ swz(r)) << 4); }

    // Per-lane source offset (bytes from the tile's first row) of block `blk` (0..kBlocks-1).
    static __device__ __forceinline__ int64_t src_off(int blk, int lane, int64_t row_stride_bytes) {
        const int row = blk * kRowsPerBlock + lane / kChunks;
        const int c = (lane % kChunks) ^ swz(row);
        return row * row_stride_bytes + c * 16;
    }
    // The same for a tile whose rows beyond `last_row` (tile-relative, >= 0) do not exist (the sequence ends inside
    // the tile): such lanes fetch the last existing row instead, same chunk, so nothing outside the tensor is read
    // and the tile holds harmless copies that the kernels mask out.
    static __device__ __forceinline__ uint32_t src_off_clamped(int blk, int lane, int64_t row_stride_bytes, int last_row) {
        const int row = blk * kRowsPerBlock + lane / kChunks;
        const int c = (lane % kChunks) ^ swz(row);
        return static_cast<uint32_t>((row < last_row ? row : last_row) * row_stride_bytes + c * 16);
    }
    // byte offset (within the tile) a lane passes to the transposed read of column block db
    // (32 columns), half = 0/1 (K-slots 0-3 / 4-7); add ks * 16 * kRowBytes for K-step ks
    static __device__ __forceinline__ int tr_off(int db, int half, int lane) {
        const int g = lane >> 4, lam = lane & 15;
        const int r = 8 * half + 4 * (g >> 1) + (lam >> 2);
        // (D = 16: a row has 16 columns; the lanes of the upper 16 repeat the lower ones, their products are not stored)
        const int col = 32 * db + (D > 16 ? 16 * (g & 1) : 0) + 4 * (lam & 3);
        return r * kRowBytes + (((col >> 3) ^ swz(r)) << 4) + ((lam & 1) << 3);
    }
    static __device__ __forceinline__ u32x4 tr_frag(const char* tile, int off_half0, int off_half1, int ks) {
        const s16x4 a = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
            (__attribute__((address_space(3))) s16x4*)(tile + off_half0 + ks * 16 * kRowBytes));
        const s16x4 b = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
            (__attribute__((address_space(3))) s16x4*)(tile + off_half1 + ks * 16 * kRowBytes));
        u32x2 lo = __builtin_bit_cast(u32x2, a), hi = __builtin_bit_cast(u32x2, b);
        return u32x4{lo.x, lo.y, hi.x, hi.y};
    }
};

// s_waitcnt vmcnt(n) with the other counters left alone (gfx9 encoding: vmcnt in bits 3:0 and 15:14)
#define TRI_WAIT_VMCNT(n) __builtin_amdgcn_s_waitcnt(0x0F70 | ((n) & 15) | (((n) >> 4) << 14))

// Workgroup -> (head, tile) mapping. Workgroups are dealt round-robin to the 8 XCDs, each with
// its own L2, so every XCD is given whole heads (head % 8 == XCD). With uniform tiles the XCD
// walks head after head, which keeps one head's K/V in its L2. With causal tiles (work grows or
// shrinks with the tile index) it instead walks tile by tile from the heaviest down, all of
// its heads abreast: a dispatcher that hands the next workgroup to the first free slot then pairs
// long and short workgroups (longest-processing-time order), and workgroups of one head that
// start together stream the same K/V tiles at the same time.
enum TileOrder { kUniformTiles = 0, kHeavyLast = 1, kHeavyFirst = 2 };
__device__ __forceinline__ void map_block(int bid, int num_heads, int num_tiles, int order, int* bh, int* tile) {
    int head, t;
    const bool heavy_last = order == kHeavyLast;
    if ((num_heads & 7) == 0) {
        const int xcd = bid & 7, slot = bid >> 3, heads_per_xcd = num_heads >> 3;
        if (order != kUniformTiles) {
            head = (slot % heads_per_xcd) * 8 + xcd;
            t = slot / heads_per_xcd;
        } else {
            head = (slot / num_tiles) * 8 + xcd;
            t = slot % num_tiles;
        }
    } else if (order != kUniformTiles) {
        head = bid % num_heads;
        t = bid / num_heads;
    } else {
        head = bid / num_tiles;
        t = bid % num_tiles;
    }
    *bh = head;
    *tile = heavy_last ? num_tiles - 1 - t : t;
}

// Mapping for a mask that is shared by the H heads of a batch (head stride 0). The mask, not K/V,
// is then the big stream (S*S*4 bytes per batch against 4*S*D per head), so the H workgroups that
// read the same mask tile get consecutive slots of ONE XCD: they run side by side, the first one
// pulls the tile from HBM and the others find it in that XCD's L2.
__device__ __forceinline__ void map_block_shared_mask(int bid, int batches, int heads, int num_tiles, int* bh, int* tile) {
    const int units = batches * num_tiles;  // one unit = the `heads` workgroups of a (batch, tile)
    int unit, head;
    if ((units & 7) == 0) {
        const int xcd = bid & 7, slot = bid >> 3;
        unit = (slot / heads) * 8 + xcd;
        head = slot % heads;
    } else {
        unit = bid / heads;
        head = bid % heads;
    }
    *bh = (unit / num_tiles) * heads + head;
    *tile = unit % num_tiles;
}

// Persistent workgroups: a launch of `grid` workgroups (one per CU) walks the head x tile items in rounds;
// workgroup `bid` takes one item per round and the function says whether round `round` still has one for it.
// The items of an XCD are those map_block gives its workgroups, in the same order (heaviest tiles first
// under a causal mask, head after head otherwise); odd rounds hand them out in reverse, so that a
// workgroup with a heavy item in one round gets a light one in the next and all finish together.
__device__ __forceinline__ bool map_item(int bid, int grid, int round, int num_heads, int num_tiles, int order,
                                         int* bh, int* tile) {
    const int items = num_heads * num_tiles;
    if ((num_heads & 7) == 0 && (grid & 7) == 0) {
        const int xcd = bid & 7, slot = bid >> 3, per_round = grid >> 3;
        const int j = round * per_round + ((round & 1) ? per_round - 1 - slot : slot);
        if (j >= (items >> 3)) return false;
        map_block(j * 8 + xcd, num_heads, num_tiles, order, bh, tile);
        return true;
    }
    const int j = round * grid + bid;
    if (j >= items) return false;
    map_block(j, num_heads, num_tiles, order, bh, tile);
    return true;
}

template <int MASK>
__device__ __forceinline__ void map_block_for(const KParams& p, int bid, int num_tiles, int order, int* bh, int* tile) {
    if (MASK != 0 && p.ms[1] == 0 && p.H > 1) map_block_shared_mask(bid, p.B, p.H, num_tiles, bh, tile);
    else map_block(bid, p.B * p.H, num_tiles, order, bh, tile);
}

// ---------------------------------------------------------------- mask block classes
// What the classes of the mask's 64 x 64 blocks (tri_attn_classify_mask; 0 all zero, 1 all -inf, 2 mixed) say about
// the tiles a workgroup streams: tile t (t < n <= 64) covers `across` blocks that lie `step` bytes apart, the first
// at first[t * tile_step]. Every lane looks at one tile; the answers are wave-uniform bit masks.
struct TileClasses {
    uint64_t zero;    // bit t: every entry of the mask over the workgroup's rows (keys) and tile t is 0: nothing to read
    uint64_t active;  // bit t: not every entry is -inf: the tile contributes
};
__device__ __forceinline__ TileClasses tile_classes(const uint8_t* first, int64_t tile_step, int n, int across, int64_t step, int lane) {
    bool all_zero = lane < n, all_ninf = true;
    if (lane < n) {
        for (int i = 0; i < across; ++i) {
            const int c = first[lane * tile_step + i * step];
            all_zero &= c == 0;
            all_ninf &= c == 1;
        }
    }
    TileClasses r;
    r.zero = __builtin_amdgcn_ballot_w64(all_zero);
    r.active = __builtin_amdgcn_ballot_w64(lane < n && !all_ninf);
    return r;
}

// ---------------------------------------------------------------- coalesced epilogue
// A wave holds NB transposed C tiles: lane = output row (l32, two lanes per row), 16 registers per
// tile = 4 groups of 4 consecutive columns. Stored straight from registers, every store instruction
// would touch 32 rows with 16 bytes each. Instead the wave writes its 32 x (32 NB) block of 16-bit
// values into a private LDS patch (row pitch padded by 16 bytes) and reads it back with 16 bytes per
// lane along the rows, so that a store instruction writes whole 64 NB-byte row segments.
// `patch` must be private to the wave and no longer in use by anyone (barrier before the call).
// `scale(i)` is applied per register; `row0` points at column 0 of the wave's first row.
// COLS < 32 NB: only the first COLS columns of the block exist and are stored (head size 16: one block, 16 columns).
template <typename T, int NB, int COLS = 32 * NB>
struct RowBlockStore {
    static constexpr int kRowBytes = 2 * COLS;
    static constexpr int kPitch = kRowBytes + 16;
    static constexpr int kPatchBytes = 32 * kPitch;
    static constexpr int kLanesPerRow = kRowBytes / 16;
    static constexpr int kRowsPerStore = 64 / kLanesPerRow;
    // `rows`: how many of the wave's 32 rows exist (the others are not stored).
    template <typename Scale>
    static __device__ __forceinline__ void run(const f32x16 (&acc)[NB], Scale scale, char* patch, char* row0,
                                               int64_t row_stride_bytes, int lane, int rows = 32) {
        const int l32 = lane & 31, h = lane >> 5;
#pragma unroll
        for (int nb = 0; nb < NB; ++nb)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                if (32 * nb + 8 * g >= COLS) continue;  // (columns that do not exist)
                u32x2 v;
                v.x = Mma<T>::pack2(scale(acc[nb][4 * g + 0]), scale(acc[nb][4 * g + 1]));
                v.y = Mma<T>::pack2(scale(acc[nb][4 * g + 2]), scale(acc[nb][4 * g + 3]));
                lds_write8(patch, l32 * kPitch + (32 * nb + 8 * g + 4 * h) * 2, v);
            }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // same wave wrote, same wave reads
        const int r = lane / kLanesPerRow, c = lane % kLanesPerRow;
#pragma unroll
        for (int i = 0; i < 32 / kRowsPerStore; ++i) {
            const int row = i * kRowsPerStore + r;
            const u32x4 v = lds_read16(patch, row * kPitch + c * 16);
            if (row < rows) *reinterpret_cast<u32x4*>(row0 + row * row_stride_bytes + c * 16) = v;
        }
    }
};

// ---------------------------------------------------------------- dropout bits shared inside a quad
// A Philox call yields the 16 keep-bytes of a 4x4 block of P. In the MFMA register layouts the four
// lanes of a quad (lanes 4n..4n+3) own four consecutive rows (forward, dQ) or four consecutive
// columns (dK/dV) of the same blocks, so each of them would generate every block itself. Instead
// lane q of the quad generates only the blocks of group q (mod 4) and the others fetch them with
// quad-broadcast DPP moves: a quarter of the Philox work for 4 moves per block.
template <int G>
__device__ __forceinline__ uint32_t quad_bcast(uint32_t v) {
    return static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(v), G * 0x55, 0xf, 0xf, true));
}
// The block lane G of the quad holds, for every lane of the quad.
template <int G>
__device__ __forceinline__ Philox4 quad_bcast(const Philox4& r) {
    Philox4 o;
#pragma unroll
    for (int k = 0; k < 4; ++k) o.w[k] = quad_bcast<G>(r.w[k]);
    return o;
}
// Same with the source lane as an argument (a constant once the caller's loop is unrolled).
__device__ __forceinline__ Philox4 quad_bcast_from(int g, const Philox4& r) {
    return g == 0 ? quad_bcast<0>(r) : (g == 1 ? quad_bcast<1>(r) : (g == 2 ? quad_bcast<2>(r) : quad_bcast<3>(r)));
}
// Row-owner form: this lane owns row i (i % 4 == lane % 4) and wants, for groups g = 0..3, the word
// (4 key bytes) of keys key0 + gstride*g .. +3. `mine` is the block this lane generated for group
// lane % 4, i.e. dropout_block(p, bh, i >> 2, (key0 + gstride * (lane % 4)) >> 2).
__device__ __forceinline__ void quad_row_words(const Philox4& mine, int lane, uint32_t (&w)[4]) {
    const int q = lane & 3;
    const Philox4 b0 = quad_bcast<0>(mine), b1 = quad_bcast<1>(mine), b2 = quad_bcast<2>(mine), b3 = quad_bcast<3>(mine);
    w[0] = q == 0 ? b0.w[0] : (q == 1 ? b0.w[1] : (q == 2 ? b0.w[2] : b0.w[3]));
    w[1] = q == 0 ? b1.w[0] : (q == 1 ? b1.w[1] : (q == 2 ? b1.w[2] : b1.w[3]));
    w[2] = q == 0 ? b2.w[0] : (q == 1 ? b2.w[1] : (q == 2 ? b2.w[2] : b2.w[3]));
    w[3] = q == 0 ? b3.w[0] : (q == 1 ? b3.w[1] : (q == 2 ? b3.w[2] : b3.w[3]));
}

}  // namespace tri
