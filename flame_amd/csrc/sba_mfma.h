// Building blocks of the 16-bit MFMA kernels (gfx950): LDS tile layout, global->LDS tile
// copies, MFMA operand fetches and the per-tile stick-breaking arithmetic.  Written for bf16,
// which the comments speak of; the same text compiles for float16 (see SBA_ELEM_F16 below).
//
// Geometry.  A workgroup is 4 waves; wave w owns 32 query rows.  A sweep step covers
// 64 keys.  All score tiles are computed TRANSPOSED, S^T = K * Q^T, with
// v_mfma_f32_32x32x16_bf16: in its 32x32 accumulator layout lane (n = lane%32,
// h = lane/32) holds column n (one query) and rows 8*(r/4) + 4*h + r%4, r = 0..15.
// The 64 keys of a step are assigned to the two 32-row tiles t = 0,1 so that
//     key_local = 32*h + 16*t + r
// i.e. each lane holds 32 CONSECUTIVE keys of one query in registers (idx = 16*t + r),
// lower half-wave the left 32 keys, upper half-wave the right 32.  The products along
// the key axis that stick-breaking needs are then in-register chains plus one
// cross-half exchange per step, and the packed bf16 weights are directly the B operand of
// the following MFMAs (O^T += V^T * P^T, dQ^T += K^T * dZ^T).
//
// LDS tiles hold 64 rows of D bf16.  Row order is "MFMA order": key_local
// 32*hh + 16*t + 4*g + i lives in row rho = 32*t + 8*g + 4*hh + i, so that the A-operand
// fetch of tile t reads rows 32*t + lane%32.  16-byte chunks of a row are XOR-swizzled
// (see swz()) so that every access pattern used here is bank-conflict free.
#pragma once
#include "sba_common.h"

// The 16-bit element type.  Everything below is compiled once per type: bf16 by default, float16 with
// -DSBA_ELEM_F16 (same sources, second object files).  Kernels, helpers and launchers of the two builds live in
// different inline namespaces, so both sets link into one library; code that includes this header once sees them
// as plain sba:: names.
#ifdef SBA_ELEM_F16
#define SBA_ELEM_NS f16
#else
#define SBA_ELEM_NS bf16
#endif

namespace sba {
inline namespace SBA_ELEM_NS {

#ifdef SBA_ELEM_F16
typedef _Float16 elem16;
#else
typedef __bf16 elem16;
#endif
typedef __attribute__((ext_vector_type(8))) elem16 h16x8;
typedef __attribute__((ext_vector_type(2))) elem16 h16x2;
// 16-bit scalars in global memory (rem, d_rem)
#ifdef SBA_ELEM_F16
struct Elem16 {
    __device__ static float load(const char* p, int64_t i) { return (float)((const _Float16*)p)[i]; }
    __device__ static void store(char* p, int64_t i, float v) { ((_Float16*)p)[i] = (_Float16)v; }
};
#else
typedef Elem<uint16_t> Elem16;
#endif
typedef __attribute__((ext_vector_type(2))) float f32x2;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) short s16x4;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;

constexpr int kThreads = 256;

// Row fragments multiplied by the logit scale once, ahead of the sweep (fp32 product, rounded
// back to bf16): the score MFMAs then deliver base-2 logits directly and the per-element
// multiplication disappears from every step.  Costs one more bf16 rounding of q (relative
// 2^-9 per element, the size of the rounding the inputs already carry).
template <int NF> __device__ inline void prescale_frags(h16x8 (&f)[NF], float s) {
#pragma unroll
    for (int ks = 0; ks < NF; ++ks)
#pragma unroll
        for (int i = 0; i < 8; i += 2) {
            const f32x2 v = {(float)f[ks][i] * s, (float)f[ks][i + 1] * s};
            const h16x2 b = __builtin_convertvector(v, h16x2);
            f[ks][i] = b[0]; f[ks][i + 1] = b[1];
        }
}

__device__ inline int mfma_row_of_key(int kl) {   // key_local -> LDS row
    return ((kl >> 4) & 1) * 32 + ((kl >> 2) & 3) * 8 + (kl >> 5) * 4 + (kl & 3);
}

// XOR swizzle of the 16-byte chunk index, a function of row bits 0..3 only.  It has to keep
// four access patterns conflict-free at once (verified with SQ_LDS_BANK_CONFLICT = 0):
//   row reads    ds_read_b128  : 16 lanes = 16 consecutive rows, same chunk (64 banks / cycle)
//   row writes   ds_write_b128 :  8 lanes =  8 consecutive rows, same chunk (32 banks / cycle)
//   tile stores  ds_write_b128 :  consecutive lanes fill one row
//   transposing reads ds_read_b64_tr_b16 : 4 consecutive rows x 64 bytes per half-wave
template <int D> __device__ inline int swz(int row);
template <> __device__ inline int swz<64>(int row) {   // 8 chunks per row, two rows per 64 banks
    int v = (row >> 1) & 7;
    return (((v & 1) << 2) | (v & 2) | ((v >> 2) & 1)) ^ (row & 1);
}
template <> __device__ inline int swz<128>(int row) {  // 16 chunks per row, one row per 64 banks
    const int r0 = row & 1, r1 = (row >> 1) & 1, r2 = (row >> 2) & 1, r3 = (row >> 3) & 1;
    return (r1 << 3) | (r0 << 2) | ((r1 ^ r3) << 1) | r2;
}

template <> __device__ inline int swz<256>(int row) {  // 32 chunks per row: a row is two passes over the 64 banks, the bank
    return swz<128>(row);                               // of a chunk is its index modulo 16 as at head_dim 128
}

template <int D> __device__ inline int tile_offset(int row, int chunk) {   // bytes
    return row * (D * 2) + ((chunk ^ swz<D>(row)) << 4);
}

// Lane-dependent byte offsets of the three fetch patterns, computed once per kernel.  The
// swizzle only looks at row bits 0..3, so moving a fetch by a multiple of 16 rows (another
// tile t, another 8-key group c, another 16-query group) adds a CONSTANT to the address:
// every fetch below is "one of these few registers + an immediate".
template <int D> struct LaneOffsets {
    int rows[D / 16];          // row fetch: row (lane%32), chunk 2*ks + h          [+ 32*t rows]
    int cols[2][D / 32];       // transposing fetch, MFMA-order tiles: [a][db]      [+ 32*(c>>1) + 16*(c&1) rows]
    int nat[2][D / 32];        // transposing fetch, natural-order tiles: [a][cb]   [+ row0 (multiple of 16) rows]
    __device__ inline void init(int lane) {
        const int h = lane >> 5, G1 = (lane >> 4) & 1, s = lane & 15;
#pragma unroll
        for (int ks = 0; ks < D / 16; ++ks) rows[ks] = tile_offset<D>(lane & 31, 2 * ks + h);
#pragma unroll
        for (int a = 0; a < 2; ++a)
#pragma unroll
            for (int b = 0; b < D / 32; ++b) {
                const int chunk = 4 * b + 2 * G1 + ((s & 3) >> 1);
                cols[a][b] = tile_offset<D>(8 * a + 4 * h + (s >> 2), chunk) + ((s & 1) << 3);
                nat[a][b] = tile_offset<D>(8 * h + 4 * a + (s >> 2), chunk) + ((s & 1) << 3);
            }
    }
    // Turns the offsets into absolute LDS addresses (each pinned in its register), for kernels that name their
    // tiles by TileAt: every fetch is then "one of these registers + an immediate", with no address arithmetic
    // in the loop.
    __device__ inline void rebase(const char* lds) {
        auto fix = [&](int& v) {
            uint32_t b = (uint32_t)(uintptr_t)lds + (uint32_t)v;
            asm("" : "+v"(b));
            v = (int)b;
        };
#pragma unroll
        for (int ks = 0; ks < D / 16; ++ks) fix(rows[ks]);
#pragma unroll
        for (int a = 0; a < 2; ++a)
#pragma unroll
            for (int b = 0; b < D / 32; ++b) { fix(cols[a][b]); fix(nat[a][b]); }
    }
};

// A tile at a COMPILE-TIME byte offset from the start of the kernel's LDS array (loops that run in one copy per
// tile buffer), used with rebased LaneOffsets.  With the tile's address in a scalar register instead, each fetch -
// or, with pinned sums, each offset register per step - costs a vector add with a scalar operand (1.8 ns).
struct TileAt { int off; };

// Wait for every outstanding global load and store of this wave.  The compiler's wait-count
// bookkeeping merges control-flow paths pessimistically: a register loaded before a loop, or
// on a path that skips the instruction consuming it, counts as "perhaps still in flight" in
// every iteration, and the first read (or reload) of it then waits for ALL memory traffic,
// the loop's own prefetches included.  An explicit wait in front of such a loop and at the
// end of each iteration (where everything has long arrived) keeps the loop body free of
// those waits.
__device__ inline void wait_global_memory() { __builtin_amdgcn_s_waitcnt(0x0F70); }   // vmcnt(0)

__device__ inline s16x4 lds_read_tr(const char* p) {
    return __builtin_amdgcn_ds_read_tr16_b64_v4i16(
        (__attribute__((address_space(3))) s16x4*)(uintptr_t)(uint32_t)(uintptr_t)p);
}
// LDS address of `tile + lane offset`, pinned in ONE vector register (the empty asm keeps the compiler from
// re-associating the sum into "(tile + constant) + lane offset", which costs a vector add with a scalar
// operand per fetch; not volatile, so equal sums of a step are merged): the constants of the fetches that
// follow go into the instructions' offset fields.
__device__ inline uint32_t lds_lane_base(const char* tile, int lane_off) {
    uint32_t b = (uint32_t)(uintptr_t)tile + (uint32_t)lane_off;
    asm("" : "+v"(b));
    return b;
}
__device__ inline s16x4 lds_read_tr_at(uint32_t base, int imm) {
    return __builtin_amdgcn_ds_read_tr16_b64_v4i16(
        (__attribute__((address_space(3))) s16x4*)((__attribute__((address_space(3))) char*)(uintptr_t)base + imm));
}

// The three operand fetches, from the precomputed lane offsets:
//   fetch_rows_o  row fetch: lane (m = lane%32, h = lane/32) gets 8 bf16 of row 32*t + m, columns
//                 16*ks + 8*h .. +7;
//   fetch_cols_o  transposing fetch from an MFMA-order tile: lane (m, h) gets column 32*db + m of
//                 the 8 keys key_local = 32*h + 8*c + j, j = 0..7.  Each ds_read_b64_tr_b16 makes 16
//                 lanes read a [4 rows x 16 columns] block (lane s: row s/4, columns 4*(s%4)..+3)
//                 and hands lane s column s of it;
//   fetch_nat_o   the same from a tile whose rows are in NATURAL order (Q, dO, and the weight
//                 tiles of the key-owner pass): lane (m, h) gets column 32*cb + m of rows
//                 row0 + 8*h + j, j = 0..7.
template <int D> __device__ inline h16x8 fetch_rows_o(const char* tile, const LaneOffsets<D>& o, int t, int ks) {
    return *(const h16x8*)(tile + o.rows[ks] + t * 32 * D * 2);
}
template <int D> __device__ inline h16x8 fetch_rows_o(TileAt tile, const LaneOffsets<D>& o, int t, int ks) {
    return *(const __attribute__((address_space(3))) h16x8*)((__attribute__((address_space(3))) char*)(uintptr_t)(uint32_t)o.rows[ks] + (tile.off + t * 32 * D * 2));
}
// kPinBase: the sum `tile + lane offset` is pinned in a register (lds_lane_base) and the fetch's constant goes into
// the offset field; one vector add per offset register and step instead of one per fetch, at the price of registers
// for the pinned sums of both tile buffers (measured: forward -7 % on small grids and -3 % at head_dim 128, dQ -2 %
// / -7 % at head_dim 64 / 128; the one-step forward at head_dim 64 would leave its four waves per SIMD).
template <int D, bool kPinBase = true>
__device__ inline h16x8 fetch_cols_o(const char* tile, const LaneOffsets<D>& o, int db, int c) {
    union { s16x4 v[2]; h16x8 b; } u;
    const int add = (32 * (c >> 1) + 16 * (c & 1)) * D * 2;
    if (kPinBase) {
        u.v[0] = lds_read_tr_at(lds_lane_base(tile, o.cols[0][db]), add);
        u.v[1] = lds_read_tr_at(lds_lane_base(tile, o.cols[1][db]), add);
    } else {
        u.v[0] = lds_read_tr(tile + o.cols[0][db] + add);
        u.v[1] = lds_read_tr(tile + o.cols[1][db] + add);
    }
    return u.b;
}
template <int D, bool kPinBase = true>
__device__ inline h16x8 fetch_cols_o(TileAt tile, const LaneOffsets<D>& o, int db, int c) {
    union { s16x4 v[2]; h16x8 b; } u;
    const int add = tile.off + (32 * (c >> 1) + 16 * (c & 1)) * D * 2;
    u.v[0] = lds_read_tr_at((uint32_t)o.cols[0][db], add);
    u.v[1] = lds_read_tr_at((uint32_t)o.cols[1][db], add);
    return u.b;
}
template <int D, bool kPinBase = false>
__device__ inline h16x8 fetch_nat_o(TileAt tile, const LaneOffsets<D>& o, int row0, int cb) {
    union { s16x4 v[2]; h16x8 b; } u;
    u.v[0] = lds_read_tr_at((uint32_t)o.nat[0][cb], tile.off + row0 * D * 2);
    u.v[1] = lds_read_tr_at((uint32_t)o.nat[1][cb], tile.off + row0 * D * 2);
    return u.b;
}
template <int D, bool kPinBase = false>
__device__ inline h16x8 fetch_nat_o(const char* tile, const LaneOffsets<D>& o, int row0, int cb) {
    union { s16x4 v[2]; h16x8 b; } u;
    if (kPinBase) {
        u.v[0] = lds_read_tr_at(lds_lane_base(tile, o.nat[0][cb]), row0 * D * 2);
        u.v[1] = lds_read_tr_at(lds_lane_base(tile, o.nat[1][cb]), row0 * D * 2);
    } else {
        u.v[0] = lds_read_tr(tile + o.nat[0][cb] + row0 * D * 2);
        u.v[1] = lds_read_tr(tile + o.nat[1][cb] + row0 * D * 2);
    }
    return u.b;
}
// fetch_rows_o with the pinned base (see fetch_cols_o): row 32*t + lane%32 of a tile in natural or MFMA order
template <int D> __device__ inline h16x8 fetch_rows_p(TileAt tile, const LaneOffsets<D>& o, int t, int ks) {
    return fetch_rows_o<D>(tile, o, t, ks);
}
template <int D> __device__ inline h16x8 fetch_rows_p(const char* tile, const LaneOffsets<D>& o, int t, int ks) {
    return *(const __attribute__((address_space(3))) h16x8*)((__attribute__((address_space(3))) char*)(uintptr_t)lds_lane_base(tile, o.rows[ks]) + t * 32 * D * 2);
}
// The same with the two lane offsets already picked (column block chosen at run time:
// indexing the offset table with a run-time value would push it into scratch memory).
template <int ROWD> __device__ inline h16x8 fetch_nat_2(const char* tile, int off0, int off1, int row0) {
    union { s16x4 v[2]; h16x8 b; } u;
    u.v[0] = lds_read_tr(tile + off0 + row0 * ROWD * 2);
    u.v[1] = lds_read_tr(tile + off1 + row0 * ROWD * 2);
    return u.b;
}
template <int D> __device__ inline int pick_nat(const LaneOffsets<D>& o, int a, int cb) {
    int v = o.nat[a][0];
#pragma unroll
    for (int b = 1; b < D / 32; ++b) v = (cb == b) ? o.nat[a][b] : v;
    return v;
}

// Global -> registers -> LDS copy of one 64-row tile (rows row0..row0+63 of a sequence),
// split so that the global loads of the next tile overlap the arithmetic on this one.
// A thread moves chunks (row kl, chunk c) and (row kl + 64/kPerThread * i, c): the address
// is a wave-uniform 64-bit base plus a 32-bit per-thread offset that never changes, so a
// step costs no vector address arithmetic.
template <int D> struct TileCopy {
    static constexpr int kChunks = 64 * D / 8;                 // 16-byte chunks per tile
    static constexpr int kPerThread = kChunks / kThreads;      // 2 (D=64) or 4 (D=128)
    static constexpr int kRowStep = 64 / kPerThread;           // rows between a thread's chunks
    u32x4 regs[kPerThread];

    __device__ inline void load(const TensorArg& t, int64_t base, int row0, int len) {
        const int tid = threadIdx.x & (kThreads - 1);      // 256 threads copy one tile
        const int kl = tid / (D / 8), c = tid % (D / 8);
        const char* tile_base = t.ptr + 2 * (base + (int64_t)row0 * t.st);          // uniform
        const uint32_t lane_off = 2u * (uint32_t)(kl * (int)t.st + c * 8);
        const uint32_t step_off = 2u * (uint32_t)(kRowStep * (int)t.st);
        if (row0 + 64 <= len) {                                // whole tile inside the sequence
#pragma unroll
            for (int r = 0; r < kPerThread; ++r)
                regs[r] = *(const u32x4*)(tile_base + (size_t)(lane_off + r * step_off));
        } else {
#pragma unroll
            for (int r = 0; r < kPerThread; ++r) {
                u32x4 v = {0u, 0u, 0u, 0u};
                if (row0 + kl + r * kRowStep < len) v = *(const u32x4*)(tile_base + (size_t)(lane_off + r * step_off));
                regs[r] = v;
            }
        }
    }
    __device__ inline void scale(float f) {      // every bf16 of the tile times f (fp32 product, rounded back)
#pragma unroll
        for (int r = 0; r < kPerThread; ++r) {
            h16x8 b[1] = {__builtin_bit_cast(h16x8, regs[r])};
            prescale_frags(b, f);
            regs[r] = __builtin_bit_cast(u32x4, b[0]);
        }
    }
    __device__ inline void store(char* tile) const {
        const int tid = threadIdx.x & (kThreads - 1);
        const int kl = tid / (D / 8), c = tid % (D / 8);
#pragma unroll
        for (int r = 0; r < kPerThread; ++r)
            *(u32x4*)(tile + tile_offset<D>(mfma_row_of_key(kl + r * kRowStep), c)) = regs[r];
    }
};

// Global -> LDS copy of one 64-row tile that bypasses the registers: every instruction moves
// 64 x 16 bytes into 1 KB of consecutive LDS, and the lane picks the global chunk that belongs
// at its LDS position (rows in MFMA order, chunks swizzled).  Four waves copy a tile; wave w4
// issues instructions w4, w4 + 4, ...  The per-lane byte offsets inside a tile never change, so
// a step costs no vector address arithmetic.  Rows past the end of the sequence are clamped to
// its last row instead of zero-filled: those keys are masked for every valid query.
// The copy instruction is written as inline assembly.  Issued through the compiler's builtin, the compiler knows that it
// writes LDS, cannot tell which part, and puts a wait for ALL vector-memory traffic in front of the next LDS access that
// it cannot prove apart from the copy's destination: the first transposing fetch of every step (the V operands of the
// forward, the K operands of the dQ pass, the Q / dO operands of the key-owner kernels) and every barrier that has a
// release fence - all of them in the middle of a step, where the tile requested at its top (for the NEXT step) need not
// have landed.  The kernels wait for their tiles themselves, at the end of the step (wait_global_memory() in front of
// the barrier that publishes them).  A kernel that copies this way must not also use the builtin (the compiler would
// not know that M0 has changed between two of its own copies).
// kLateRagged: the lane's row and chunk for the one ragged tile of a sequence are worked out where that tile is
// requested, from a copy of the lane index that the compiler cannot see through.  As loop invariants they are
// otherwise computed once at the top of the kernel and occupy registers through the whole sweep: in the
// register-lean dQ kernel that is the difference between four spilled registers and none.
// 64 lanes x 16 bytes from `base + off` (uniform base, 32-bit lane offset) to LDS bytes lds_addr .. lds_addr + 1023
__device__ inline void dma16(const char* base, uint32_t off, uint32_t lds_addr) {
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %0" : : "s"(base), "v"(off), "s"(lds_addr) : "memory");
}
__device__ inline uint32_t lds_address(const char* p) { return (uint32_t)(uintptr_t)p; }   // (low half of the flat address)

template <int D, bool kNatural = false, bool kLateRagged = false> struct TileDma {      // kNatural: rows kept in their order (query tiles)
    static constexpr int kPerWave = 64 * D * 2 / 1024 / 4;    // 2 (D=64) or 4 (D=128)
    uint32_t off[kPerWave];
    const char* origin;        // row 0 of the (sequence, head) slice: uniform
    int st, w4, lane;          // row stride in elements

    __device__ static inline void where(int inst, int lane, int& kl, int& c) {
        const int pos = inst * 64 + lane;                  // LDS chunk position
        const int r = pos / (D / 8), pc = pos % (D / 8);
        c = pc ^ swz<D>(r);
        kl = kNatural ? r : (((r >> 2) & 1) << 5) | (((r >> 5) & 1) << 4) | (((r >> 3) & 3) << 2) | (r & 3);
    }
    // Only the slice origin and the row stride are kept: holding on to the whole tensor
    // descriptor costs scalar registers that the loops do not have.
    __device__ inline void init(int lane_, int w4_, const TensorArg& t, int64_t base) {
        lane = lane_; w4 = w4_;
        origin = t.ptr + 2 * base;
        st = (int)t.st;
        // Scalar registers of their own: left as parts of the 16-register tuple that the kernel arguments were
        // loaded into, they keep the whole tuple alive, and a spilled tuple comes back sixteen lane reads at a
        // time in every iteration.
        int st_own;
        const char* origin_own;
        asm volatile("s_mov_b32 %0, %1" : "=s"(st_own) : "s"(st));
        asm volatile("s_mov_b64 %0, %1" : "=s"(origin_own) : "s"(origin));
        st = st_own;
        origin = origin_own;
#pragma unroll
        for (int i = 0; i < kPerWave; ++i) {
            int kl, c;
            where(w4 + 4 * i, lane, kl, c);
            off[i] = 2u * (uint32_t)(kl * st + c * 8);
        }
    }
    // a tile known to lie inside the sequence (every key tile of a sweep but the rightmost)
    __device__ inline void issue_full(int row0, char* tile) const {
        const char* tile_base = origin + (((uint64_t)(uint32_t)row0 * (uint32_t)st) << 1);
#pragma unroll
        for (int i = 0; i < kPerWave; ++i) dma16(tile_base, off[i], lds_address(tile + (w4 + 4 * i) * 1024));
    }
    __device__ inline void issue(int row0, int len, char* tile) const {
        // uniform; row0 and the stride are non-negative: the unsigned product is two scalar instructions, the
        // signed 64-bit one about ten
        const char* tile_base = origin + (((uint64_t)(uint32_t)row0 * (uint32_t)st) << 1);
        if (row0 + 64 <= len) {
#pragma unroll
            for (int i = 0; i < kPerWave; ++i) dma16(tile_base, off[i], lds_address(tile + (w4 + 4 * i) * 1024));
        } else {
            int lane_here = lane;
            if (kLateRagged) asm volatile("" : "+v"(lane_here));
#pragma unroll
            for (int i = 0; i < kPerWave; ++i) {
                int kl, c;
                where(w4 + 4 * i, lane_here, kl, c);
                kl = min(kl, len - 1 - row0);
                dma16(tile_base, 2u * (uint32_t)(kl * st + c * 8), lds_address(tile + (w4 + 4 * i) * 1024));
            }
        }
    }
};

// Epilogue of the key-owner kernels.  An accumulator tile (lane (n, h), register r -> row
// 8*(r/4) + 4*h + r%4, column n) written straight to global memory is 16 two-byte stores per
// lane that each touch 64 cache lines; going through a [rows][D] bf16 staging tile in LDS
// turns a 64-row block into two 16-byte, fully coalesced stores per thread.
template <int D>
__device__ inline void stage_acc_tile(char* staging, int row0, int col0, const f32x16& acc, float scale, int lane) {
    const int n = lane & 31, h = lane >> 5;
#pragma unroll
    for (int r = 0; r < 16; r += 2) {
        // registers r, r+1 are two consecutive rows of the same column: one packed conversion
        // (round to nearest even in hardware), two 2-byte stores
        const int row = row0 + 8 * (r >> 2) + 4 * h + (r & 3);
        const f32x2 v = {acc[r] * scale, acc[r + 1] * scale};
        const uint32_t w = __builtin_bit_cast(uint32_t, __builtin_convertvector(v, h16x2));
        *(uint16_t*)(staging + row * (D * 2) + (col0 + n) * 2) = (uint16_t)w;
        *(uint16_t*)(staging + (row + 1) * (D * 2) + (col0 + n) * 2) = (uint16_t)(w >> 16);
    }
}
// 64 staged rows -> rows row0.. of a [rows, D] tensor; `tid` of `n_threads` threads take part.
template <int D>
__device__ inline void store_staged_rows(const char* staging, const TensorArg& t, int64_t base, int row0, int len,
                                         int tid, int n_threads) {
    for (int c = tid; c < 64 * D / 8; c += n_threads) {
        const int row = c / (D / 8), cc = c % (D / 8);
        if (row0 + row < len)
            *(u32x4*)(t.ptr + 2 * (base + (int64_t)(row0 + row) * t.st + cc * 8)) = *(const u32x4*)(staging + row * (D * 2) + cc * 16);
    }
}

// B operand kept in registers for the whole sweep: row `row` of a [rows, D] tensor,
// columns 16*ks + 8*h .. +7 for every ks.  Rows >= len read as zero.  One address, one
// predicate; the ks fragments are at constant offsets from it.
template <int D>
__device__ inline void load_row_frags(h16x8 (&f)[D / 16], const TensorArg& t, int64_t base, int row,
                                      int len, int lane) {
    const int h = lane >> 5;
    const char* ptr = t.ptr + 2 * (base + (int64_t)row * t.st + 8 * h);
    if (row < len) {
#pragma unroll
        for (int ks = 0; ks < D / 16; ++ks) f[ks] = __builtin_bit_cast(h16x8, *(const u32x4*)(ptr + 32 * ks));
    } else {
#pragma unroll
        for (int ks = 0; ks < D / 16; ++ks) f[ks] = h16x8{0};
    }
}

__device__ inline h16x8 pack8(const float* p) {
    h16x8 r;
#pragma unroll
    for (int i = 0; i < 8; i += 2) {
        f32x2 v = {p[i], p[i + 1]};
        h16x2 b = __builtin_convertvector(v, h16x2);
        r[i] = b[0]; r[i + 1] = b[1];
    }
    return r;
}

__device__ inline f32x16 mfma(h16x8 a, h16x8 b, f32x16 c) {
#ifdef SBA_ELEM_F16
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
#else
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
#endif
}

// S^T tile pair for one wave, raw MFMA accumulators (no vector-ALU instruction touches
// them here, so the matrix cores run ahead of whatever vector work follows):
// raw[t][r] = (K Q^T)[key_local = 32h + 16t + r][query n].
template <int D, bool kBatch = (D == 128), class Tile>
__device__ inline void score_raw_o(f32x16 (&raw)[2], Tile ktile, const LaneOffsets<D>& o,
                                   const h16x8 (&qf)[D / 16]) {
    // tile 1 first: the product chain starts at its keys (the right half of the lane's 32), and
    // can begin while the MFMAs of tile 0 are still in flight
#pragma unroll
    for (int t = 1; t >= 0; --t) {
        // all operands of the tile are requested before its first MFMA: at head_dim 128 the kernels
        // run one or two waves per SIMD, and nothing else hides an LDS round trip per MFMA
        h16x8 a[D / 16];
#pragma unroll
        for (int ks = 0; ks < D / 16; ++ks) a[ks] = fetch_rows_o<D>(ktile, o, t, ks);
        if (kBatch) __builtin_amdgcn_sched_barrier(0);
        f32x16 acc = {0};
#pragma unroll
        for (int ks = 0; ks < D / 16; ++ks) acc = mfma(a[ks], qf[ks], acc);
        raw[t] = acc;
    }
}

// base-2 logits from the raw accumulators: x[16*t + r] = scale2 * raw[t][r].
__device__ inline void scale_scores(float (&x)[32], const f32x16 (&raw)[2], float scale2) {
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int r = 0; r < 16; ++r) x[16 * t + r] = raw[t][r] * scale2;
}

template <int D, bool kBatch = (D == 128), class Tile>
__device__ inline void score_tiles_o(float (&x)[32], Tile ktile, const LaneOffsets<D>& o,
                                     const h16x8 (&qf)[D / 16], float scale2) {
    f32x16 raw[2];
    score_raw_o<D, kBatch>(raw, ktile, o, qf);
    scale_scores(x, raw, scale2);
}

// Score tiles from pre-scaled fragments: x[16*t + r] = raw accumulator, no vector work.
template <int D, bool kBatch = (D == 128), class Tile>
__device__ inline void score_tiles_ps(float (&x)[32], Tile ktile, const LaneOffsets<D>& o,
                                      const h16x8 (&qf)[D / 16]) {
    f32x16 raw[2];
    score_raw_o<D, kBatch>(raw, ktile, o, qf);
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int r = 0; r < 16; ++r) x[16 * t + r] = raw[t][r];
}

// In-place: x[idx] (base-2 logits, idx = key offset inside this lane's 32 keys; invalid
// pairs already set to -inf) -> stick-breaking weights of this step, given the carry
// `R` = product of (1 - beta) over all keys right of the step.
//
// The chain runs right-to-left inside the lane's 32 keys on  W = prod (1 + e),  e = 2^x:
//     W' = fma(W, e, W),   L' = 1 / W'  (= product of 1 - beta so far),   a = L - L',
//     beta = 1 - W / W' = fma(-W, L', 1)
// i.e. exp, fma, rcp, sub (and one fma for beta) per key; forming u = 1 / (1 + e) and L' = L u
// costs one instruction more.  Masked keys (x = -inf, e = 0) leave W unchanged and get a = 0,
// beta = 0 exactly.  W may overflow to +inf: then L' = 0 and every weight left of that key is 0,
// as it should be (the true values are below 2^-128).  Two expressions meet inf * 0 after such an
// overflow, where the right value is 0: W' itself when a later e is exactly 0 (a logit below
// -126), and beta (-inf * 0).  Both values lie in [0, 1], and so do the finished weights: the
// instructions that produce them carry the hardware's clamp modifier, which costs nothing and
// turns NaN into 0 (the kernels run with the DX10 clamp mode on, the default); the carry is
// clamped once per step.  (With beta = 0 there, dz = g - beta * prefix = 0, which is right: all
// g left of an overflow are 0.)
// One exchange between the half-waves supplies the factor the lower (left) half is missing.
// Outputs: x[idx] = A (attention weight); beta[idx] when kNeedBeta; R updated to the carry
// for the next (left) step; *lane_carry = the carry entering this lane's 32 keys.
// The two lanes (n, 0) and (n, 1) that share a query exchange one value per step.  The hardware
// swaps the upper half of one register with the lower half of another in a single vector
// instruction (v_permlane32_swap): started from two copies of `v`, one register ends up holding
// the lower half-wave's value in every lane and the other the upper half-wave's.  No LDS round
// trip (ds_bpermute) in the middle of the dependent chain.
__device__ inline void half_values(float v, float& lower, float& upper) {
    typedef unsigned u32x2 __attribute__((ext_vector_type(2)));
    const u32x2 r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    lower = __uint_as_float(r[0]);
    upper = __uint_as_float(r[1]);
}

__device__ inline float clamp01(float v) { return __builtin_amdgcn_fmed3f(v, 0.0f, 1.0f); }

template <bool kNeedBeta, int N>
__device__ inline float product_chain(float (&x)[N], float (&beta)[kNeedBeta ? N : 1]) {
    float W = 1.0f, L = 1.0f;
#pragma unroll
    for (int idx = N - 1; idx >= 0; --idx) {
        const float e = __builtin_amdgcn_exp2f(x[idx]);
        const float Wn = __builtin_fmaf(W, e, W);
        const float Ln = __builtin_amdgcn_rcpf(Wn);
        x[idx] = L - Ln;
        if (kNeedBeta) beta[idx] = clamp01(__builtin_fmaf(-W, Ln, 1.0f));
        W = Wn;
        L = Ln;
    }
    return clamp01(L);
}
// The same chain with a hook: `between(seg)` runs after every four keys (seg = 0 .. N/4 - 1) and
// a scheduling fence keeps what it issues at that place.  The exp/rcp of the chain overlap MFMAs
// in flight (plain vector instructions do not), so a kernel hands the chain the MFMAs that do
// not depend on the weights, a few per segment.
template <bool kNeedBeta, int N, class Between>
__device__ inline float product_chain_with(float (&x)[N], float (&beta)[kNeedBeta ? N : 1], Between&& between) {
    float W = 1.0f, L = 1.0f;
#pragma unroll
    for (int idx = N - 1; idx >= 0; --idx) {
        const float e = __builtin_amdgcn_exp2f(x[idx]);
        const float Wn = __builtin_fmaf(W, e, W);
        const float Ln = __builtin_amdgcn_rcpf(Wn);
        x[idx] = L - Ln;
        if (kNeedBeta) beta[idx] = clamp01(__builtin_fmaf(-W, Ln, 1.0f));
        W = Wn;
        L = Ln;
        if ((idx & 3) == 0) {
            between((N - 1 - idx) >> 2);
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    return clamp01(L);
}
// The chain from a given carry.  F = product of (1 - beta) over all keys right of THIS LANE's N keys (both
// half-waves read their own from the forward's two carry tables).  Run on  W = (1/F) prod (1 + e),  the
// reciprocals are the finished running products and their differences the finished weights: no scaling
// pass over the weights afterwards.  F = 0 (a product that has left the fp32 range, or the zero carry
// given to rows past the end of a sequence) makes W infinite, every reciprocal 0 or NaN and - through the
// clamps - every weight and beta exactly 0, which is what such a row's values are to fp32 precision.
// Returns the carry leaving the lane's keys on their left.
template <bool kNeedBeta, int N, class Between>
__device__ inline float carried_chain_with(float (&x)[N], float (&beta)[kNeedBeta ? N : 1], float F, Between&& between) {
    float W = __builtin_amdgcn_rcpf(F), L = F;
#pragma unroll
    for (int idx = N - 1; idx >= 0; --idx) {
        const float e = __builtin_amdgcn_exp2f(x[idx]);
        const float Wn = __builtin_fmaf(W, e, W);
        const float Ln = __builtin_amdgcn_rcpf(Wn);
        x[idx] = clamp01(L - Ln);
        if (kNeedBeta) beta[idx] = clamp01(__builtin_fmaf(-W, Ln, 1.0f));
        W = Wn;
        L = Ln;
        if ((idx & 3) == 0) {
            between((N - 1 - idx) >> 2);
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    return clamp01(L);
}
template <int N> __device__ inline void scale_clamped(float (&x)[N], float f) {
#pragma unroll
    for (int idx = 0; idx < N; ++idx) x[idx] = clamp01(x[idx] * f);
}

// Forward weights with ONE reciprocal per lane and step instead of one per key.  With
// W_j = prod_{k >= j} (1 + e_k) inside the lane's 32 keys, the running products of 1 - beta are
// L_j = 1 / W_j, and L_{j+1} = L_j (1 + e_j): from the single reciprocal of the lane's total
// the chain is walked back UP with one fma per key, and the weight of key j is
//     a_j = L_{j+1} - L_j = L_j e_j                      (no cancellation for small e_j).
// Starting the walk from  carry / W_0  delivers finished weights, so per key: exp, fma (W),
// mul (a), fma (L).  The walk needs a finite, not too large W_0 in every lane of the wave
// (2^96 leaves the reciprocal far from the denormals).  Otherwise - logits so large that the
// product of 32 factors leaves the fp32 range - the function returns false with R untouched
// (x then holds e = 2^logit), and the caller does the step with the reciprocal-per-key chain,
// which handles overflow.  The answer is the same in all lanes of a wave.
// In: x[idx] base-2 logits (-inf for invisible pairs).  Out: pf[c] = the weights of keys
// 8c .. 8c+7 packed to bf16 (the B operand of P*V), R advanced.  kWeights = false: only R is
// advanced (the carry-only forward).
constexpr float kFastChainLimit = 0x1p96f;

template <bool kWeights>
__device__ inline bool forward_weights_fast(float (&x)[32], h16x8 (&pf)[4], float& R, int lane, float& lane_carry) {
    float W = 1.0f;
#pragma unroll
    for (int idx = 31; idx >= 0; --idx) {
        x[idx] = __builtin_amdgcn_exp2f(x[idx]);          // e
        W = __builtin_fmaf(W, x[idx], W);
    }
    if (__builtin_amdgcn_ballot_w64(!(W < kFastChainLimit)) != 0) return false;
    const float Linv = __builtin_amdgcn_rcpf(W);
    float Llo, Lup;
    half_values(Linv, Llo, Lup);
    lane_carry = (lane >= 32) ? R : R * Lup;                  // the carry entering this lane's 32 keys
    if (kWeights) {
        float Lt = lane_carry * Linv;                         // ... over W_0
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            float a[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const float e = x[8 * c + i];
                a[i] = Lt * e;
                Lt = __builtin_fmaf(Lt, e, Lt);
            }
            pf[c] = pack8(a);
        }
    }
    R = R * Llo * Lup;
    return true;
}

template <bool kNeedBeta>
__device__ inline void stick_weights(float (&x)[32], float (&beta)[kNeedBeta ? 32 : 1], float& R, int lane,
                                     float* lane_carry = nullptr) {
    const float L = product_chain<kNeedBeta, 32>(x, beta);
    float Llo, Lup;
    half_values(L, Llo, Lup);
    // upper half-wave holds the right 32 keys: its chain starts from R itself
    const float F = (lane >= 32) ? R : R * Lup;
    if (lane_carry) *lane_carry = F;      // the carry entering this lane's 32 keys
    scale_clamped<32>(x, F);
    R = R * Llo * Lup;
}

// stick_weights<true> with a hook between the eight segments of the chain (see product_chain_with).
template <class Between>
__device__ inline void stick_weights_hooked(float (&x)[32], float (&beta)[32], float& R, int lane, float* lane_carry,
                                            Between&& between) {
    const float L = product_chain_with<true, 32>(x, beta, between);
    float Llo, Lup;
    half_values(L, Llo, Lup);
    const float F = (lane >= 32) ? R : R * Lup;
    if (lane_carry) *lane_carry = F;
    scale_clamped<32>(x, F);
    R = R * Llo * Lup;
}

// stick_weights<true> with the dP MFMAs of the step (dp[16t + r] = (V dO^T)[key][query], see
// dp_tiles_o) issued between the segments of the chain, their operands fetched one segment ahead.
template <int D, class Tile>
__device__ inline void stick_weights_and_dp(float (&x)[32], float (&beta)[32], float (&dp)[32], float& R, int lane,
                                            float* lane_carry, Tile vtile, const LaneOffsets<D>& o,
                                            const h16x8 (&dof)[D / 16]) {
    constexpr int kPer = D / 64;               // MFMAs per segment: 2 tiles x D/16 slices over 8 segments
    f32x16 dacc[2];
    h16x8 nx[kPer];
    // MFMA m (0 .. D/8 - 1): tile t = m & 1, slice ks = m >> 1 (neighbours use different accumulators)
#pragma unroll
    for (int i = 0; i < kPer; ++i) nx[i] = fetch_rows_o<D>(vtile, o, i & 1, i >> 1);
    stick_weights_hooked(x, beta, R, lane, lane_carry, [&](int seg) {
        h16x8 cur[kPer];
#pragma unroll
        for (int i = 0; i < kPer; ++i) cur[i] = nx[i];
        if (seg < 7) {
#pragma unroll
            for (int i = 0; i < kPer; ++i) {
                const int m = kPer * (seg + 1) + i;
                nx[i] = fetch_rows_o<D>(vtile, o, m & 1, m >> 1);
            }
        }
#pragma unroll
        for (int i = 0; i < kPer; ++i) {
            const int m = kPer * seg + i, t = m & 1, ks = m >> 1;
            dacc[t] = mfma(cur[i], dof[ks], ks == 0 ? f32x16{0} : dacc[t]);
        }
    });
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int r = 0; r < 16; ++r) dp[16 * t + r] = dacc[t][r];
}

// The same from this lane's own carry F (carried_chain_with): finished weights, beta and dP; returns the carry
// leaving the lane's keys.
// kPaced: the wave lowers its issue priority as it moves through the chain (3 for the first two 4-key segments, then 2,
// 1, 0).  Two waves of a SIMD that run this chain side by side otherwise issue oldest first: the older one runs as if
// alone and then idles at the next barrier while the younger one finishes at the rate of a single wave.  With the
// priority tied to progress, whichever wave is behind goes first and both arrive together.
template <int D, bool kPaced = false, class Tile>
__device__ inline float carried_weights_and_dp(float (&x)[32], float (&beta)[32], float (&dp)[32], float F,
                                               Tile vtile, const LaneOffsets<D>& o, const h16x8 (&dof)[D / 16]) {
    constexpr int kPer = D / 64;
    f32x16 dacc[2];
    h16x8 nx[kPer];
#pragma unroll
    for (int i = 0; i < kPer; ++i) nx[i] = fetch_rows_o<D>(vtile, o, i & 1, i >> 1);
    if (kPaced) __builtin_amdgcn_s_setprio(3);
    const float Lend = carried_chain_with<true, 32>(x, beta, F, [&](int seg) {
        if (kPaced) {
            if (seg == 1) __builtin_amdgcn_s_setprio(2);
            else if (seg == 3) __builtin_amdgcn_s_setprio(1);
            else if (seg == 5) __builtin_amdgcn_s_setprio(0);
        }
        h16x8 cur[kPer];
#pragma unroll
        for (int i = 0; i < kPer; ++i) cur[i] = nx[i];
        if (seg < 7) {
#pragma unroll
            for (int i = 0; i < kPer; ++i) {
                const int m = kPer * (seg + 1) + i;
                nx[i] = fetch_rows_o<D>(vtile, o, m & 1, m >> 1);
            }
        }
#pragma unroll
        for (int i = 0; i < kPer; ++i) {
            const int m = kPer * seg + i, t = m & 1, ks = m >> 1;
            dacc[t] = mfma(cur[i], dof[ks], ks == 0 ? f32x16{0} : dacc[t]);
        }
    });
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int r = 0; r < 16; ++r) dp[16 * t + r] = dacc[t][r];
    return Lend;
}

// The same in two parts, for kernels in which another wave-group handles the neighbouring
// step and the carry is only known after an exchange:
//   part 1: x[idx] <- weights relative to the right edge of THIS lane's 32 keys; returns the
//           factor that completes them inside the step (1 for the upper half-wave, the upper
//           half's product for the lower) and, in `total`, the product over all 64 keys;
//   part 2: scale_clamped(x, carry * factor).
template <bool kNeedBeta>
__device__ inline float stick_weights_local(float (&x)[32], float (&beta)[kNeedBeta ? 32 : 1], float& total,
                                            int lane) {
    const float L = product_chain<kNeedBeta, 32>(x, beta);
    float Llo, Lup;
    half_values(L, Llo, Lup);
    total = Llo * Lup;
    return (lane >= 32) ? 1.0f : Lup;
}

// Sets the logits of invisible (query, key) pairs of a diagonal step to -inf.
__device__ inline void mask_step(float (&x)[32], int key_first, int qi, int strict) {
    // key_first = first key of this lane's 32; key j visible iff j + strict <= qi
    const int nvis = qi - strict - key_first + 1;      // visible keys among idx 0..31
#pragma unroll
    for (int idx = 0; idx < 32; ++idx)
        if (idx >= nvis) x[idx] = -INFINITY;
}

// Row fetch from a natural-order tile: 8 bf16 of row `row`, columns 16*ks + 8*h .. +7.
template <int ROWD> __device__ inline h16x8 fetch_row_nat(const char* tile, int row, int ks, int lane) {
    return *(const h16x8*)(tile + tile_offset<ROWD>(row, 2 * ks + (lane >> 5)));
}

// dP^T tile pair: dp[16*t + r] = (V dO^T)[key_local][query].  The gradient of `rem` is not
// subtracted here: with g = a * dP taken from the plain dP, the term it contributes to the logit
// gradient is  -beta_ik * d_rem_i * rem_i  (the weights of a row and its remainder sum to one),
// i.e. a constant d_rem_i * rem_i added to the running prefix of g -- which is how the prefix
// tables carry it (see the dQ kernels).  `init` is what the accumulators start from (zero).
template <int D, class Tile>
__device__ inline void dp_tiles_o(float (&dp)[32], Tile vtile, const LaneOffsets<D>& o,
                                  const h16x8 (&dof)[D / 16], float init = 0.f) {
#pragma unroll
    for (int t = 0; t < 2; ++t) {
        f32x16 acc;
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[r] = init;
#pragma unroll
        for (int ks = 0; ks < D / 16; ++ks) acc = mfma(fetch_rows_o<D>(vtile, o, t, ks), dof[ks], acc);
#pragma unroll
        for (int r = 0; r < 16; ++r) dp[16 * t + r] = acc[r];
    }
}

// Gradient of the logits for one step.  In: a[idx] attention weights, beta[idx],
// dp[idx] = dO.v, Gc = sum of g over all keys LEFT of this step (plus d_rem * rem).
// Out: dp[idx] <- dz = g - beta * prefix_sum(g);  Gc advanced past this step.
// The inclusive prefix runs left-to-right inside the lane's 32 keys; the upper (right)
// half-wave adds the lower half's total.  kLowReg trades one more add per element for
// not keeping the 32 prefix values alive (two passes: sum, then running prefix).
template <bool kLowReg>
__device__ inline void logit_grads(const float (&a)[32], const float (&beta)[32], float (&dp)[32], float& Gc,
                                   int lane, float* lane_prefix = nullptr) {
    float c = 0.f;
    if (kLowReg) {
#pragma unroll
        for (int idx = 0; idx < 32; ++idx) {
            dp[idx] = a[idx] * dp[idx];     // g
            c += dp[idx];
        }
        float clo, cup;
        half_values(c, clo, cup);
        float run = (lane >= 32) ? Gc + clo : Gc;
        if (lane_prefix) *lane_prefix = run;     // the prefix entering this lane's 32 keys
#pragma unroll
        for (int idx = 0; idx < 32; ++idx) {
            run += dp[idx];
            dp[idx] = __builtin_fmaf(-beta[idx], run, dp[idx]);
        }
        Gc = Gc + clo + cup;
    } else {
        float pre[32];
#pragma unroll
        for (int idx = 0; idx < 32; ++idx) {
            dp[idx] = a[idx] * dp[idx];     // g
            c += dp[idx];
            pre[idx] = c;
        }
        float clo, cup;
        half_values(c, clo, cup);
        const float F = (lane >= 32) ? Gc + clo : Gc;
        if (lane_prefix) *lane_prefix = F;       // the prefix entering this lane's 32 keys
#pragma unroll
        for (int idx = 0; idx < 32; ++idx) dp[idx] = __builtin_fmaf(-beta[idx], pre[idx] + F, dp[idx]);
        Gc = Gc + clo + cup;
    }
}

// The same when the prefix entering this lane's keys is known up front (from the tables of the dQ pass):
// one pass, no exchange.  Out: dp[idx] <- dz.
template <int N>
__device__ inline void logit_grads_from(const float (&a)[N], const float (&beta)[N], float (&dp)[N], float run) {
#pragma unroll
    for (int idx = 0; idx < N; ++idx) {
        const float g = a[idx] * dp[idx];
        run += g;
        dp[idx] = __builtin_fmaf(-beta[idx], run, g);
    }
}

// Register-lean form of the backward's per-step arithmetic for the row-owner kernel at head_dim
// 128, where registers decide between one and two waves per SIMD: two arrays of 32 instead of
// four.  Part 1 runs the reciprocal-per-key chain right-to-left and leaves, in place of the
// logits, beta, and in place of dP, g' = a' * dP with a' the weight relative to the right edge of
// the lane's 32 keys (the finished weight is F * a', F the carry entering the lane's keys, which
// only the exchange after the chain supplies).  Returns the lane's product of (1 - beta) (clamped,
// see product_chain) and in `gsum` the lane's sum of g'.  Part 2 walks left-to-right from the
// prefix `G` entering the lane's keys:  t = F g',  G += t,  dz = t - beta G,  packed as it goes.
// chain_beta_gprime from this lane's own carry F (see carried_chain_with): dp[idx] <- g = a * dP with the finished
// weight, gsum their sum; returns the carry leaving the lane's keys.
__device__ inline float carried_beta_g(float (&x)[32], float (&dp)[32], float F, float& gsum) {
    float W = __builtin_amdgcn_rcpf(F), L = F, c = 0.f;
#pragma unroll
    for (int idx = 31; idx >= 0; --idx) {
        const float e = __builtin_amdgcn_exp2f(x[idx]);
        const float Wn = __builtin_fmaf(W, e, W);
        const float Ln = __builtin_amdgcn_rcpf(Wn);
        x[idx] = clamp01(__builtin_fmaf(-W, Ln, 1.0f));       // beta
        dp[idx] = clamp01(L - Ln) * dp[idx];                  // g (the clamps map the NaN of an overflowed chain to 0)
        c += dp[idx];
        W = Wn;
        L = Ln;
    }
    gsum = c;
    return clamp01(L);
}
// dz from beta, g and the prefix G entering the lane's keys
// (The running sum must stay a plain add: fused with the product that made g - which the compiler does across
// function boundaries when allowed to - it would need the two factors of every g alive instead of g itself,
// 32 registers more than this kernel has.)
__device__ inline void walk_logit_grads_g(const float (&beta)[32], const float (&g)[32], float G, h16x8 (&zf)[4]) {
#pragma clang fp contract(off)
#pragma unroll
    for (int c = 0; c < 4; ++c) {
        float dz[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            G += g[8 * c + i];
            dz[i] = __builtin_fmaf(-beta[8 * c + i], G, g[8 * c + i]);
        }
        zf[c] = pack8(dz);
    }
}
__device__ inline float chain_beta_gprime(float (&x)[32], float (&dp)[32], float& gsum) {
    float W = 1.0f, L = 1.0f, c = 0.f;
#pragma unroll
    for (int idx = 31; idx >= 0; --idx) {
        const float e = __builtin_amdgcn_exp2f(x[idx]);
        const float Wn = __builtin_fmaf(W, e, W);
        const float Ln = __builtin_amdgcn_rcpf(Wn);
        x[idx] = clamp01(__builtin_fmaf(-W, Ln, 1.0f));       // beta
        dp[idx] = clamp01(L - Ln) * dp[idx];                  // g' (the clamps map the NaN of an overflowed chain to 0)
        c += dp[idx];
        W = Wn;
        L = Ln;
    }
    gsum = c;
    return clamp01(L);
}
// Out: zf[c] = dz of keys 8c .. 8c+7 packed to bf16 (the B operand of dQ^T += K^T dZ^T).
__device__ inline void walk_logit_grads(const float (&beta)[32], const float (&g)[32], float F, float G, h16x8 (&zf)[4]) {
#pragma unroll
    for (int c = 0; c < 4; ++c) {
        float dz[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const float t = F * g[8 * c + i];
            G += t;
            dz[i] = __builtin_fmaf(-beta[8 * c + i], G, t);
        }
        zf[c] = pack8(dz);
    }
}

// logit_grads in two parts (see stick_weights_local): part 1 forms g in place of dp and
// returns this lane's offset inside the step (0 for the lower half-wave, the lower half's
// sum for the upper) and, in `total`, the step's sum of g; part 2 applies the prefix.
__device__ inline float logit_grads_local(const float (&a)[32], float (&dp)[32], float& total, int lane) {
    float c = 0.f;
#pragma unroll
    for (int idx = 0; idx < 32; ++idx) {
        dp[idx] = a[idx] * dp[idx];     // g
        c += dp[idx];
    }
    float clo, cup;
    half_values(c, clo, cup);
    total = clo + cup;
    return (lane >= 32) ? clo : 0.0f;
}
__device__ inline void logit_grads_apply(const float (&beta)[32], float (&dp)[32], float start) {
    float run = start;
#pragma unroll
    for (int idx = 0; idx < 32; ++idx) {
        run += dp[idx];
        dp[idx] = __builtin_fmaf(-beta[idx], run, dp[idx]);
    }
}

}  // inline namespace SBA_ELEM_NS
}  // namespace sba
