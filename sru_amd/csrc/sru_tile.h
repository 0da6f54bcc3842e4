// Row tiles: how the 16-bit kernels of sru_split.h touch memory.
//
// Why. With one column per lane, a wavefront's step touches 64*K 16-bit elements of U: 384 or
// 512 bytes, and 128 bytes of every other stream. A wavefront can have 64 vector-memory
// operations outstanding at most, so with one small operation per stream and step the bytes in
// flight per wavefront are capped at a few KB and the instruction stream is full of memory
// operations.
//
// How. Memory is touched in whole rows, 16 bytes per lane: the elements that a wavefront's columns
// hold for TC consecutive steps form a tile of TC rows (one row = one step, contiguous in memory),
// and the wavefront moves a tile with tile_bytes / 1024 instructions of 1 KB each, whatever a
// column's share of a row is. A tile passes through LDS to change hands: it is written there in
// memory order (ds_write_b128) and read back column-wise by the lane that owns the column; outputs
// go the other way. A wavefront owns its LDS tiles alone (wavefronts of a workgroup share none), and
// LDS executes a wavefront's instructions in order, so no barrier is needed. The loads of the next
// chunks are in flight in registers (staging sets, each refilled right after it is drained to LDS).
#pragma once

#include "sru_scan.h"

namespace sru_amd {

typedef uint32_t piece_t __attribute__((ext_vector_type(4)));   // what one lane moves: 16 bytes
typedef piece_t __attribute__((may_alias)) piece_a;
typedef uint32_t __attribute__((may_alias)) u32_a;
typedef uint16_t __attribute__((may_alias)) u16_a;
struct __attribute__((may_alias, aligned(8))) u32x2_a { uint32_t x, y; };

// Compiler-level ordering point between the two sides of an LDS hand-over inside a wavefront.
__device__ __forceinline__ void lds_handover() {
    __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
    __builtin_amdgcn_wave_barrier();
}

// A tile of TC rows; a row holds N 16-bit elements for each of the wavefront's W columns
// (W = 64: one column per lane; W = 32: two lanes per column, sru_split.h).
template <int N, int TC, int W = kBlock>
struct RowTile {
    static constexpr int kRowBytes = W * N * 2;
    static constexpr int kBytes = TC * kRowBytes;
    static_assert(kBytes % (kBlock * 16) == 0, "a tile is a whole number of 1 KB instructions");
    static constexpr int kPieces = kBytes / (kBlock * 16);
    struct Regs { piece_t v[kPieces]; };
    // lane's piece i: which row of the tile it lies in, and where inside that row
    __device__ __forceinline__ static int row_of(int i, int lane) { return ((i * kBlock + lane) * 16) / kRowBytes; }
    __device__ __forceinline__ static int within(int i, int lane) { return ((i * kBlock + lane) * 16) % kRowBytes; }
    // byte offsets of the lane's pieces from the first byte of the tile's first row in memory;
    // rows beyond `rows` (a ragged last chunk) are clamped to the last valid one
    __device__ __forceinline__ static void offsets(int64_t (&off)[kPieces], int lane, int64_t row_stride_bytes,
                                                   int rows = TC) {
#pragma unroll
        for (int i = 0; i < kPieces; ++i)
            off[i] = (int64_t)min(row_of(i, lane), rows - 1) * row_stride_bytes + within(i, lane);
    }
    template <bool NT>
    __device__ __forceinline__ static void load(Regs &r, const char *tile0, const int64_t (&off)[kPieces]) {
#pragma unroll
        for (int i = 0; i < kPieces; ++i) {
            const piece_t *q = reinterpret_cast<const piece_t *>(tile0 + off[i]);
            r.v[i] = NT ? __builtin_nontemporal_load(q) : *q;
        }
    }
    // rows: only pieces lying in rows below it are written
    template <bool NT>
    __device__ __forceinline__ static void store(const Regs &r, char *tile0, const int64_t (&off)[kPieces], int lane,
                                                 int rows) {
#pragma unroll
        for (int i = 0; i < kPieces; ++i) {
            if (rows == TC || row_of(i, lane) < rows) {
                piece_t *q = reinterpret_cast<piece_t *>(tile0 + off[i]);
                if (NT) __builtin_nontemporal_store(r.v[i], q);
                else *q = r.v[i];
            }
        }
    }
    // LDS copy of the tile: rows PITCH bytes apart (PITCH = kRowBytes: dense, in memory order)
    template <int PITCH = kRowBytes>
    __device__ __forceinline__ static void to_lds(const Regs &r, unsigned char *lds, int lane) {
#pragma unroll
        for (int i = 0; i < kPieces; ++i)
            *reinterpret_cast<piece_a *>(lds + row_of(i, lane) * PITCH + within(i, lane)) = r.v[i];
    }
    template <int PITCH = kRowBytes>
    __device__ __forceinline__ static void from_lds(Regs &r, const unsigned char *lds, int lane) {
#pragma unroll
        for (int i = 0; i < kPieces; ++i)
            r.v[i] = *reinterpret_cast<const piece_a *>(lds + row_of(i, lane) * PITCH + within(i, lane));
    }
};

}  // namespace sru_amd
