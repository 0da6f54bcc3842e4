// Row-tile scan kernels for 16-bit streams: the forward and the checkpointed backward scan for
// shapes in which every wavefront lies inside one direction and one batch row (d a multiple of 64).
//
// Why. With one column per lane, a wavefront's step touches 64*K 16-bit elements of U: 384 or
// 512 bytes, and 128 bytes of every other stream. A wavefront can have 64 vector-memory
// operations outstanding at most, so with one small operation per stream and step the bytes in
// flight per wavefront are capped at a few KB, and shapes with few wavefronts (32 768 columns =
// 512 wavefronts) cannot cover the memory latency: they ran at 40 % of the bandwidth the same
// kernels reach with float streams, at the same number of operations.
//
// How. Memory is touched in whole rows, 16 bytes per lane: the 64 columns' elements of TC
// consecutive steps form a tile of TC rows (one row = one step, contiguous in memory), and the
// wavefront moves a tile with tile_bytes / 1024 instructions of 1 KB each, whatever a column's
// share of a row is. A tile passes through LDS to change hands: it is written there in memory
// order (ds_write_b128) and read back column-wise by the lane that owns the column; outputs go the
// other way. One wavefront per workgroup owns its LDS tiles alone, and LDS executes a wavefront's
// instructions in order, so no barrier is needed. The loads of NBUF chunks ahead are in flight in
// registers (NBUF staging sets, each refilled right after it is drained to LDS).
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

// Waits for every vector-memory operation issued so far (s_waitcnt vmcnt(0), gfx9 encoding).
// Placed once before a pipelined loop: whatever was loaded before the loop and is used inside it
// would otherwise make the compiler place a wait inside the loop whose count also drains the
// loads the loop keeps in flight on purpose.
__device__ __forceinline__ void wait_for_all_loads() { __builtin_amdgcn_s_waitcnt(0x0F70); }

// A tile of TC rows; a row holds N 16-bit elements for each of the wavefront's 64 columns.
template <int N, int TC>
struct RowTile {
    static constexpr int kRowBytes = kBlock * N * 2;
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
    __device__ __forceinline__ static void to_lds(const Regs &r, unsigned char *lds, int lane) {
#pragma unroll
        for (int i = 0; i < kPieces; ++i) reinterpret_cast<piece_a *>(lds)[i * kBlock + lane] = r.v[i];
    }
    __device__ __forceinline__ static void from_lds(Regs &r, const unsigned char *lds, int lane) {
#pragma unroll
        for (int i = 0; i < kPieces; ++i) r.v[i] = reinterpret_cast<const piece_a *>(lds)[i * kBlock + lane];
    }
    // column `lane`'s N elements of row `row`, as floats
    template <typename T>
    __device__ __forceinline__ static void read_column(const unsigned char *lds, int row, int lane, float (&out)[N]) {
        const unsigned char *rowp = lds + row * kRowBytes;
        if constexpr (N == 1) {
            out[0] = bits_to_float<T>(reinterpret_cast<const u16_a *>(rowp)[lane]);
        } else if constexpr (N == 4) {
            const u32x2_a d = reinterpret_cast<const u32x2_a *>(rowp)[lane];
            out[0] = bits_to_float<T>(d.x & 0xffffu);
            out[1] = bits_to_float<T>(d.x >> 16);
            out[2] = bits_to_float<T>(d.y & 0xffffu);
            out[3] = bits_to_float<T>(d.y >> 16);
        } else {
            static_assert(N == 3, "1, 3 or 4 elements per column");
            // 6 bytes starting at byte 6 * lane: the two dwords around them, shifted by half a
            // dword in odd lanes
            const int first = (3 * lane) >> 1;
            const uint32_t d0 = reinterpret_cast<const u32_a *>(rowp)[first];
            const uint32_t d1 = reinterpret_cast<const u32_a *>(rowp)[first + 1];
            const uint32_t sh = 16u * (uint32_t)(lane & 1);
            const uint32_t lo = __builtin_amdgcn_alignbit(d1, d0, sh), hi = d1 >> sh;
            out[0] = bits_to_float<T>(lo & 0xffffu);
            out[1] = bits_to_float<T>(lo >> 16);
            out[2] = bits_to_float<T>(hi & 0xffffu);
        }
    }
    template <typename T>
    __device__ __forceinline__ static void write_column(unsigned char *lds, int row, int lane, const float (&v)[N]) {
        unsigned char *rowp = lds + row * kRowBytes;
        if constexpr (N == 4) {
            u32x2_a d;
            d.x = pack_pair<T>(v[0], v[1]);
            d.y = pack_pair<T>(v[2], v[3]);
            reinterpret_cast<u32x2_a *>(rowp)[lane] = d;
        } else {
#pragma unroll
            for (int i = 0; i < N; ++i)
                reinterpret_cast<u16_a *>(rowp)[lane * N + i] = (uint16_t)float_to_bits<T>(v[i]);
        }
    }
};

// ================================================================= forward scan, row tiles
// MODE bits: kHasPad, kCkpt (state checkpoints; without it no state is kept), kTanh, kNtLoad, kNtStore.
template <typename T, int K, int SKIP, int MODE, int TC, int NBUF>
__global__ void __launch_bounds__(kBlock) forward_scan_rows(const FwdParams p) {
    static_assert(sizeof(T) == 2, "16-bit streams");
    static_assert(TC == kCkptInterval, "a chunk is one checkpoint interval");
    constexpr bool NTL = (MODE & kNtLoad) != 0, NTS = (MODE & kNtStore) != 0;
    constexpr bool HAS_PAD = (MODE & kHasPad) != 0, CKPT = (MODE & kCkpt) != 0, TANH = (MODE & kTanh) != 0;
    using TU = RowTile<K, TC>;
    using T1 = RowTile<1, TC>;
    __shared__ __attribute__((aligned(16))) unsigned char lds_u[TU::kBytes];
    __shared__ __attribute__((aligned(16))) unsigned char lds_x[SKIP == 1 ? T1::kBytes : 16];
    __shared__ __attribute__((aligned(16))) unsigned char lds_h[T1::kBytes];
    // Small per-lane values of a staging set (padding flags; the chunk's start state in the backward
    // kernel) change hands through LDS as well, although the same lane reads them back: that ends
    // the life of the loaded register at the hand-over, so the set's refill can reuse it (a value
    // kept in its register across the refill makes the compiler copy registers at the loop's end,
    // and every such copy waits for loads that were meant to stay in flight).
    __shared__ uint32_t lds_pad[kBlock];

    const int lane = threadIdx.x;
    const int64_t colu = (int64_t)blockIdx.x * kBlock;   // the wavefront's first column (ncols is a multiple of 64)
    const int64_t col = colu + lane;
    const int Dp = p.Dp;
    const int ju = (int)(colu % Dp);
    const int j = ju + lane;
    const bool flip = ju >= p.d;

    const float wc1 = static_cast<const float *>(p.wc)[j], wc2 = static_cast<const float *>(p.wc)[Dp + j];
    const float b1 = p.bias[j], b2 = p.bias[Dp + j];
    const float m = p.mask_c ? p.mask_c[col] : 1.0f;
    float cur = p.c0[col];
    const float sx = (SKIP == 1 && p.scale_x) ? *p.scale_x : 1.0f;

    const int64_t L = p.L;
    const int64_t ef = (flip ? (L - 1) : 0) * p.ncols + colu;   // element of walk step 0, column colu
    const int64_t es = flip ? -p.ncols : p.ncols;               // elements per walk step
    const int64_t pf = (flip ? (L - 1) : 0) * p.B + colu / Dp;
    const int64_t ps = flip ? -p.B : p.B;
    const char *ubase = static_cast<const char *>(p.u);
    const char *xbase = static_cast<const char *>(p.x);
    char *hbase = static_cast<char *>(p.h);

    const int64_t nfull = L / TC;
    const int tail = (int)(L - nfull * TC);

    struct Stage {
        typename TU::Regs u;
        typename T1::Regs x;
        uint32_t pad;   // lane l: the padding flag of the chunk's step l % TC
    };
    int64_t ou[TU::kPieces], o1[T1::kPieces];
    TU::offsets(ou, lane, es * (K * 2));
    T1::offsets(o1, lane, es * 2);

    // issues the loads of chunk ch (rows: its number of valid steps; off_*: piece offsets to match)
    auto load_chunk = [&](Stage &s, int64_t ch, const int64_t (&offu)[TU::kPieces], const int64_t (&off1)[T1::kPieces],
                          int rows) __attribute__((always_inline)) {
        const int64_t e0 = ef + ch * TC * es;
        TU::template load<NTL>(s.u, ubase + e0 * (K * 2), offu);
        if (SKIP == 1) T1::template load<NTL>(s.x, xbase + e0 * 2, off1);
        if (HAS_PAD) s.pad = p.pad[pf + (ch * TC + min(lane % TC, rows - 1)) * ps];
    };

    // the chunk's tiles are in LDS; runs its n steps and writes its outputs
    auto compute_chunk = [&](int64_t ch, int n) __attribute__((always_inline)) {
        const uint32_t padreg = HAS_PAD ? reinterpret_cast<const u32_a *>(lds_pad)[lane] : 0u;
#pragma unroll
        for (int i = 0; i < TC; ++i) {
            if (i < n) {
                const bool padded = HAS_PAD && __builtin_amdgcn_readlane((int)padreg, i) != 0;
                float uu[K], xx[1] = {0.f};
                TU::template read_column<T>(lds_u, i, lane, uu);
                if (SKIP == 1) T1::template read_column<T>(lds_x, i, lane, xx);
                const float u0 = uu[0];
                const float g1 = gate<T>(uu[1], wc1, cur, b1);
                const float g2 = gate<T>(uu[2], wc2, cur, b2);
                const float cn = (cur - u0) * g1 + u0;
                const float val = TANH ? tanh_fast(cn) : cn;
                float out;
                if constexpr (SKIP != 0) {
                    const float xv = (SKIP == 1) ? xx[0] * sx : uu[K - 1];
                    out = (val - xv) * m * g2 + xv;
                } else {
                    out = val * m * g2;
                }
                cur = padded ? cur : cn;
                const float hv[1] = {padded ? 0.0f : out};
                T1::template write_column<T>(lds_h, i, lane, hv);
            }
        }
        lds_handover();
        typename T1::Regs hr;
        T1::from_lds(hr, lds_h, lane);
        if (n == TC) T1::template store<NTS>(hr, hbase + (ef + ch * TC * es) * 2, o1, lane, TC);
        else {
            int64_t ot[T1::kPieces];
            T1::offsets(ot, lane, es * 2, n);
            T1::template store<NTS>(hr, hbase + (ef + ch * TC * es) * 2, ot, lane, n);
        }
        if (CKPT && n == TC) p.ckpt[ch * p.ncols + col] = cur;
        lds_handover();   // the next chunk's tiles may now replace this one's
    };

    auto stage_to_lds = [&](const Stage &s) __attribute__((always_inline)) {
        TU::to_lds(s.u, lds_u, lane);
        if (SKIP == 1) T1::to_lds(s.x, lds_x, lane);
        if (HAS_PAD) reinterpret_cast<u32_a *>(lds_pad)[lane] = s.pad;
        lds_handover();
    };

    Stage set[NBUF], last;
    // the ragged last chunk is requested first and waits in registers until the end of the walk
    if (tail > 0) {
        int64_t tu[TU::kPieces], t1[T1::kPieces];
        TU::offsets(tu, lane, es * (K * 2), tail);
        T1::offsets(t1, lane, es * 2, tail);
        load_chunk(last, nfull, tu, t1, tail);
    }
    if (nfull > 0) {
#pragma unroll
        for (int b = 0; b < NBUF; ++b) load_chunk(set[b], min((int64_t)b, nfull - 1), ou, o1, TC);
    }
    wait_for_all_loads();
    int64_t g = 0;   // first chunk of the current group of NBUF
    for (; g + NBUF <= nfull; g += NBUF) {
#pragma unroll
        for (int b = 0; b < NBUF; ++b) {
            stage_to_lds(set[b]);
            // refill: a chunk beyond the last full one is replaced by the last full one (loaded, never used)
            load_chunk(set[b], min(g + NBUF + b, nfull - 1), ou, o1, TC);
            compute_chunk(g + b, TC);
        }
    }
#pragma unroll
    for (int b = 0; b < NBUF - 1; ++b) {
        if (g + b < nfull) {
            stage_to_lds(set[b]);
            compute_chunk(g + b, TC);
        }
    }
    if (tail > 0) {
        stage_to_lds(last);
        compute_chunk(nfull, tail);
    }
    p.c_last[col] = cur;
}

// ================================================================= backward scan from checkpoints, row tiles
// As backward_scan_ckpt: per chunk, last to first, the forward recurrence is rebuilt from the
// chunk's checkpoint, then the backward recurrence runs over the same steps. The gradient tiles
// replace the input tiles in LDS in place (grad_u over U, grad_x over x) on their way out.
template <typename T, int K, int SKIP, int MODE, int TC, int NBUF>
__global__ void __launch_bounds__(kBlock) backward_scan_rows(const BwdParams p) {
    static_assert(sizeof(T) == 2, "16-bit streams");
    static_assert(TC == kCkptInterval, "a chunk is one checkpoint interval");
    constexpr bool NTL = (MODE & kNtLoad) != 0, NTS = (MODE & kNtStore) != 0;
    constexpr bool HAS_PAD = (MODE & kHasPad) != 0, TANH = (MODE & kTanh) != 0;
    using TU = RowTile<K, TC>;
    using T1 = RowTile<1, TC>;
    __shared__ __attribute__((aligned(16))) unsigned char lds_u[TU::kBytes];
    __shared__ __attribute__((aligned(16))) unsigned char lds_x[SKIP == 1 ? T1::kBytes : 16];
    __shared__ __attribute__((aligned(16))) unsigned char lds_gh[T1::kBytes];
    __shared__ uint32_t lds_pad[kBlock];   // see forward_scan_rows
    __shared__ float lds_cstart[kBlock];

    const int lane = threadIdx.x;
    const int64_t colu = (int64_t)blockIdx.x * kBlock;
    const int64_t col = colu + lane;
    const int Dp = p.Dp;
    const int ju = (int)(colu % Dp);
    const int j = ju + lane;
    const bool flip = ju >= p.d;

    const float wc1 = static_cast<const float *>(p.wc)[j], wc2 = static_cast<const float *>(p.wc)[Dp + j];
    const float b1 = p.bias[j], b2 = p.bias[Dp + j];
    const float m = p.mask_c ? p.mask_c[col] : 1.0f;
    float cur = p.glast[col];   // d loss / d state
    CompensatedSum sw1, sw2, sb1, sb2;
    const float sx = (SKIP == 1 && p.scale_x) ? *p.scale_x : 1.0f;

    const int64_t L = p.L;
    const int64_t ef = (flip ? (L - 1) : 0) * p.ncols + colu;
    const int64_t es = flip ? -p.ncols : p.ncols;
    const int64_t pf = (flip ? (L - 1) : 0) * p.B + colu / Dp;
    const int64_t ps = flip ? -p.B : p.B;
    const char *ubase = static_cast<const char *>(p.u);
    const char *xbase = static_cast<const char *>(p.x);
    const char *ghbase = static_cast<const char *>(p.gh);
    char *gubase = static_cast<char *>(p.gu);
    char *gxbase = static_cast<char *>(p.gx);

    const int64_t nfull = L / TC;
    const int tail = (int)(L - nfull * TC);

    struct Stage {
        typename TU::Regs u;
        typename T1::Regs x, gh;
        uint32_t pad;
        float cstart;   // state before the chunk's first step
    };
    int64_t ou[TU::kPieces], o1[T1::kPieces];
    TU::offsets(ou, lane, es * (K * 2));
    T1::offsets(o1, lane, es * 2);

    auto load_chunk = [&](Stage &s, int64_t ch, const int64_t (&offu)[TU::kPieces], const int64_t (&off1)[T1::kPieces],
                          int rows) __attribute__((always_inline)) {
        const int64_t e0 = ef + ch * TC * es;
        TU::template load<NTL>(s.u, ubase + e0 * (K * 2), offu);
        if (SKIP == 1) T1::template load<NTL>(s.x, xbase + e0 * 2, off1);
        T1::template load<NTL>(s.gh, ghbase + e0 * 2, off1);
        if (HAS_PAD) s.pad = p.pad[pf + (ch * TC + min(lane % TC, rows - 1)) * ps];
        // one load from a selected address, so that every chunk issues the same operations
        const float *from = (ch == 0) ? p.c0 + col : p.ckpt + (ch - 1) * p.ncols + col;
        s.cstart = *from;
    };

    auto stage_to_lds = [&](const Stage &s) __attribute__((always_inline)) {
        TU::to_lds(s.u, lds_u, lane);
        if (SKIP == 1) T1::to_lds(s.x, lds_x, lane);
        T1::to_lds(s.gh, lds_gh, lane);
        if (HAS_PAD) reinterpret_cast<u32_a *>(lds_pad)[lane] = s.pad;
        lds_cstart[lane] = s.cstart;
        lds_handover();
    };

    auto compute_chunk = [&](int64_t ch, int n) __attribute__((always_inline)) {
        const uint32_t padreg = HAS_PAD ? reinterpret_cast<const u32_a *>(lds_pad)[lane] : 0u;
        const float cstart = lds_cstart[lane];
        float st[TC + 1];            // st[i] = state before step i of the chunk
        float g1[TC], g2[TC], u0s[TC], xs[TC];
        float gw1 = 0.f, gw2 = 0.f, gb1 = 0.f, gb2 = 0.f;
        st[0] = cstart;
#pragma unroll
        for (int i = 0; i < TC; ++i) {
            if (i < n) {
                const bool padded = HAS_PAD && __builtin_amdgcn_readlane((int)padreg, i) != 0;
                float uu[K];
                TU::template read_column<T>(lds_u, i, lane, uu);
                const float cp = st[i];
                u0s[i] = uu[0];
                if (SKIP == 2) xs[i] = uu[K - 1];
                g1[i] = gate<T>(uu[1], wc1, cp, b1);
                g2[i] = gate<T>(uu[2], wc2, cp, b2);
                const float cn = (cp - u0s[i]) * g1[i] + u0s[i];
                st[i + 1] = padded ? cp : cn;
            }
        }
        lds_handover();   // every U row has been read: grad_u may take its place
#pragma unroll
        for (int i = TC - 1; i >= 0; --i) {
            if (i < n) {
                const bool padded = HAS_PAD && __builtin_amdgcn_readlane((int)padreg, i) != 0;
                float xx[1] = {0.f}, ghs[1];
                if (SKIP == 1) T1::template read_column<T>(lds_x, i, lane, xx);
                T1::template read_column<T>(lds_gh, i, lane, ghs);
                const float cp = st[i];
                const float val = TANH ? tanh_fast(st[i + 1]) : st[i + 1];
                const float dact = TANH ? (1.0f - val * val) : 1.0f;
                const float u0 = u0s[i];
                const float G1 = g1[i], G2 = g2[i];
                const float xv = (SKIP == 0) ? 0.0f : (SKIP == 1) ? xx[0] * sx : xs[i];
                const float gh = ghs[0];

                const float gg2 = gh * (val - xv) * m * (G2 * (1.0f - G2));
                const float gc = TANH ? gh * m * (G2 * dact) + cur : gh * m * G2 + cur;
                const float gg1 = gc * (cp - u0) * (G1 * (1.0f - G1));
                const float gskip = gh * (1.0f - G2 * m);
                const float ncur = gc * G1 + gg1 * wc1 + gg2 * wc2;

                float gu[K];
                gu[0] = padded ? 0.0f : gc * (1.0f - G1);
                gu[1] = padded ? 0.0f : gg1;
                gu[2] = padded ? 0.0f : gg2;
                if (K == 4) gu[K - 1] = padded ? 0.0f : gskip;
                gb1 += padded ? 0.0f : gg1;
                gw1 += padded ? 0.0f : gg1 * cp;
                gb2 += padded ? 0.0f : gg2;
                gw2 += padded ? 0.0f : gg2 * cp;
                cur = padded ? cur : ncur;
                TU::template write_column<T>(lds_u, i, lane, gu);
                if (SKIP == 1) {
                    const float gx[1] = {padded ? 0.0f : gskip * sx};
                    T1::template write_column<T>(lds_x, i, lane, gx);
                }
            }
        }
        sw1.add(gw1);
        sw2.add(gw2);
        sb1.add(gb1);
        sb2.add(gb2);
        lds_handover();
        const int64_t e0 = ef + ch * TC * es;
        typename TU::Regs gur;
        TU::from_lds(gur, lds_u, lane);
        typename T1::Regs gxr;
        if (SKIP == 1) T1::from_lds(gxr, lds_x, lane);
        if (n == TC) {
            TU::template store<NTS>(gur, gubase + e0 * (K * 2), ou, lane, TC);
            if (SKIP == 1) T1::template store<NTS>(gxr, gxbase + e0 * 2, o1, lane, TC);
        } else {
            int64_t tu[TU::kPieces], t1[T1::kPieces];
            TU::offsets(tu, lane, es * (K * 2), n);
            T1::offsets(t1, lane, es * 2, n);
            TU::template store<NTS>(gur, gubase + e0 * (K * 2), tu, lane, n);
            if (SKIP == 1) T1::template store<NTS>(gxr, gxbase + e0 * 2, t1, lane, n);
        }
        lds_handover();
    };

    Stage set[NBUF];
    // set b of a group holds chunk top - b; chunks below 0 are replaced by chunk 0 (loaded, never used)
    int64_t top = nfull - 1;
    if (nfull > 0) {
#pragma unroll
        for (int b = 0; b < NBUF; ++b) load_chunk(set[b], max(top - b, (int64_t)0), ou, o1, TC);
    }
    if (tail > 0) {   // the ragged chunk is the last of the walk: visited first
        Stage last;
        int64_t tu[TU::kPieces], t1[T1::kPieces];
        TU::offsets(tu, lane, es * (K * 2), tail);
        T1::offsets(t1, lane, es * 2, tail);
        load_chunk(last, nfull, tu, t1, tail);
        stage_to_lds(last);
        compute_chunk(nfull, tail);
    }
    wait_for_all_loads();
    for (; top - (NBUF - 1) >= 0; top -= NBUF) {
#pragma unroll
        for (int b = 0; b < NBUF; ++b) {
            stage_to_lds(set[b]);
            load_chunk(set[b], max(top - NBUF - b, (int64_t)0), ou, o1, TC);
            compute_chunk(top - b, TC);
        }
    }
#pragma unroll
    for (int b = 0; b < NBUF - 1; ++b) {
        if (top - b >= 0) {
            stage_to_lds(set[b]);
            compute_chunk(top - b, TC);
        }
    }

    p.ginit[col] = cur;
    p.partial[col] = sw1.value();
    p.partial[p.ncols + col] = sw2.value();
    p.partial[2 * p.ncols + col] = sb1.value();
    p.partial[3 * p.ncols + col] = sb2.value();
}

}  // namespace sru_amd
