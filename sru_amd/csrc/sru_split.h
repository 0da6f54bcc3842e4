// Lane-pair scan kernels for 16-bit streams and few columns: two lanes share one column.
//
// Why. A wavefront that is alone on its SIMD issues one instruction at a time, whatever its
// kind, so with at most one wavefront per SIMD the time of a step is the number of instructions
// in it (counters: a one-column-per-lane kernel on row tiles kept its wavefront issuing 78 % of the
// time and waiting 18 %). A shape
// with 32 768 columns fills only 512 of the 1 024 SIMDs at one column per lane. Here a wavefront
// owns 32 columns and the two gates of a column run side by side in a lane pair, which halves the
// dependent chain's share of the instruction stream and uses every SIMD:
//   even lane (role 0): forget gate, state update; in the backward pass everything that belongs
//                       to the state path (grad of the candidate stream and of gate 1, the carried
//                       state gradient);
//   odd lane (role 1):  reset gate and the output; in the backward pass the output path (grad of
//                       gate 2 and of the skip term).
// Both lanes run the same instructions on role-specific operands (per-lane constants and LDS
// addresses); what one role needs from the other crosses the pair with one DPP move. Memory is
// touched in row tiles (sru_tile.h): whole rows, 16 bytes per lane, handed over through LDS; U and x share one LDS tile with a common row pitch so that every per-step LDS
// address is a per-lane base plus a compile-time offset.
#pragma once

#include "sru_tile.h"

namespace sru_amd {

constexpr int kSplitCols = 32;    // columns per wavefront
constexpr int kSplitChunk = 16;   // steps per chunk: two checkpoint intervals
// Wavefronts per workgroup (independent of each other): four land on the four SIMDs of a compute
// unit, where single-wavefront workgroups leave some SIMDs with two wavefronts and others with none.
constexpr int kSplitWaves = 4;

// value of the other lane of the pair (quad_perm [1,0,3,2])
__device__ __forceinline__ float pair_swap(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1, 0xf, 0xf, true));
}
// value of the pair's even lane in both lanes (quad_perm [0,0,2,2])
__device__ __forceinline__ float pair_even(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xA0, 0xf, 0xf, true));
}

template <typename T>
__device__ __forceinline__ float lds_elem(const unsigned char *p) {
    return bits_to_float<T>(*reinterpret_cast<const u16_a *>(p));
}
template <typename T>
__device__ __forceinline__ void lds_put(unsigned char *p, float v) {
    *reinterpret_cast<u16_a *>(p) = (uint16_t)float_to_bits<T>(v);
}

// Geometry shared by both passes: the input tile in LDS holds, per step, the U row of the
// wavefront's 32 columns followed by its x row (when the skip term comes from x).
template <int K, int SKIP>
struct SplitTile {
    static constexpr int TC = kSplitChunk, W = kSplitCols;
    using TU = RowTile<K, TC, W>;
    using T1 = RowTile<1, TC, W>;
    static constexpr int kPitch = TU::kRowBytes + (SKIP == 1 ? T1::kRowBytes : 0);
    static constexpr int kBytes = TC * kPitch;
    // Byte offsets inside a row of the two elements a lane reads per step.
    //   role 0: A = u0 (candidate), B = u1 (forget-gate stream)
    //   role 1: A = the skip operand (x, or U[..., 3]; unused without a skip term), B = u2
    __device__ __forceinline__ static int elem_a(int c, int role) {
        if (role == 0) return c * K * 2;
        if (SKIP == 1) return TU::kRowBytes + c * 2;
        return c * K * 2 + (SKIP == 2 ? 6 : 0);
    }
    __device__ __forceinline__ static int elem_b(int c, int role) { return c * K * 2 + (role ? 4 : 2); }
};

// ================================================================= forward scan, lane pairs
// MODE bits: kHasPad, kCkpt (state checkpoints; without it no state is kept), kTanh, kNtLoad, kNtStore.
// (These kernels run with one or two wavefronts per SIMD by construction, so the register
// allocator is told not to save registers for an occupancy that will not happen: with its default
// target of four it serialised the LDS reads of a chunk through one register.)
template <typename T, int K, int SKIP, int MODE, int NBUF>
__global__ void __launch_bounds__(kBlock * kSplitWaves) __attribute__((amdgpu_waves_per_eu(1, 2)))
forward_scan_split(const FwdParams p) {
    static_assert(sizeof(T) == 2, "16-bit streams");
    constexpr bool NTL = (MODE & kNtLoad) != 0, NTS = (MODE & kNtStore) != 0;
    constexpr bool HAS_PAD = (MODE & kHasPad) != 0, CKPT = (MODE & kCkpt) != 0, TANH = (MODE & kTanh) != 0;
    using G = SplitTile<K, SKIP>;
    using TU = typename G::TU;
    using T1 = typename G::T1;
    constexpr int TC = G::TC, W = G::W, PITCH = G::kPitch;
    static_assert(TC == 2 * kCkptInterval, "a chunk is two checkpoint intervals");
    fetch_params_early(p);
    __shared__ __attribute__((aligned(16))) unsigned char all_in[kSplitWaves][G::kBytes];
    __shared__ __attribute__((aligned(16))) unsigned char all_h[kSplitWaves][2 * T1::kBytes];   // h tile, then role 0's dump tile
    __shared__ uint32_t all_pad[kSplitWaves][kBlock];
    // the wavefronts of a workgroup share nothing: each has its own tiles and its own 32 columns
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x / kBlock));
    unsigned char *lds_in = all_in[wave], *lds_h = all_h[wave];
    uint32_t *lds_pad = all_pad[wave];

    const int lane = threadIdx.x % kBlock;
    const int c = lane >> 1, role = lane & 1;
    const int64_t colu = ((int64_t)blockIdx.x * kSplitWaves + wave) * W;   // the wavefront's first column (ncols is a multiple of 32)
    if (colu >= p.ncols) return;
    const int64_t col = colu + c;
    const int Dp = p.Dp;
    const int ju = (int)(colu % Dp);
    const int j = ju + c;
    const bool flip = ju >= p.d;

    // the lane's gate: role 0 the forget gate, role 1 the reset gate (operands folded as in gate())
    const float knw = kNegLog2e * static_cast<const float *>(p.wc)[role * Dp + j];
    const float knb = kNegLog2e * p.bias[role * Dp + j];
    const float m = p.mask_c ? p.mask_c[col] : 1.0f;
    const float sa = (SKIP == 1 && role == 1 && p.scale_x) ? *p.scale_x : 1.0f;   // scale of operand A (x * scale_x)
    float cur = p.c0 ? p.c0[col] : 0.0f;   // no initial state given: zeros

    const int64_t L = p.L;
    const int64_t ef = (flip ? (L - 1) : 0) * p.ncols + colu;
    const int64_t es = flip ? -p.ncols : p.ncols;
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
    const unsigned char *ra = lds_in + G::elem_a(c, role), *rb = lds_in + G::elem_b(c, role);
    unsigned char *wh = lds_h + (role ? c * 2 : T1::kBytes + c * 2);   // role 0 has no output: dump tile

    auto load_chunk = [&](Stage &s, int64_t ch, const int64_t (&offu)[TU::kPieces], const int64_t (&off1)[T1::kPieces],
                          int rows) __attribute__((always_inline)) {
        const int64_t e0 = ef + ch * TC * es;
        TU::template load<NTL>(s.u, ubase + e0 * (K * 2), offu);
        if (SKIP == 1) T1::template load<NTL>(s.x, xbase + e0 * 2, off1);
        if (HAS_PAD) s.pad = p.pad[pf + (ch * TC + min(lane % TC, rows - 1)) * ps];
    };

    auto stage_to_lds = [&](const Stage &s) __attribute__((always_inline)) {
        TU::template to_lds<PITCH>(s.u, lds_in, lane);
        if (SKIP == 1) T1::template to_lds<PITCH>(s.x, lds_in + TU::kRowBytes, lane);
        if (HAS_PAD) reinterpret_cast<u32_a *>(lds_pad)[lane] = s.pad;
        lds_handover();
    };

    auto compute_chunk = [&](int64_t ch, int n) __attribute__((always_inline)) {
        const uint32_t padreg = HAS_PAD ? reinterpret_cast<const u32_a *>(lds_pad)[lane] : 0u;
        // every LDS read of the chunk is issued before the first step: left next to their uses the
        // reads stay behind the previous step's output write, and a lone wavefront then sits out
        // the LDS latency once per step
        float av[TC], bv[TC];
#pragma unroll
        for (int i = 0; i < TC; ++i) {
            if (i < n) {
                av[i] = lds_elem<T>(ra + i * PITCH);   // role 0: u0; role 1: the skip operand
                bv[i] = lds_elem<T>(rb + i * PITCH);   // role 0: u1; role 1: u2
            }
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int i = 0; i < TC; ++i) {
            if (i < n) {
                const bool padded = HAS_PAD && __builtin_amdgcn_readlane((int)padreg, i) != 0;
                const float a = av[i], b = bv[i];   // role 0: u0 as it is; role 1: the skip operand before scaling
                const float g = sigmoid_exp2<T>(__builtin_fmaf(knw, cur, __builtin_fmaf(kNegLog2e, b, knb)));
                const float cn = pair_even((cur - a) * g + a);      // role 0's result: the new state, to both lanes
                const float val = TANH ? tanh_fast(cn) : cn;
                // role 1's result: h = (val - skip) * m * g + skip = val - (val - skip) * (1 - m * g), skip = sa * a
                const float out = (SKIP != 0) ? __builtin_fmaf(-__builtin_fmaf(-sa, a, val), __builtin_fmaf(-m, g, 1.0f), val)
                                              : val * m * g;
                cur = padded ? cur : cn;
                lds_put<T>(wh + i * T1::kRowBytes, padded ? 0.0f : out);
                if (CKPT && (i + 1) % kCkptInterval == 0)   // (both lanes of a pair store the same value)
                    p.ckpt[(ch * (TC / kCkptInterval) + i / kCkptInterval) * p.ncols + col] = cur;
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
        lds_handover();
    };

    Stage set[NBUF], last;
    if (tail > 0) {   // the ragged last chunk is requested first and waits in registers
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
    int64_t g = 0;
    for (; g + NBUF <= nfull; g += NBUF) {
#pragma unroll
        for (int b = 0; b < NBUF; ++b) {
            stage_to_lds(set[b]);
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

// ================================================================= backward scan from checkpoints, lane pairs
// Per chunk, last to first: the forward recurrence is rebuilt from the chunk's checkpoint (each
// lane keeps its own gate, the states and its operand A), then the backward recurrence runs over
// the same steps. The gradient tiles replace the input tile in LDS in place on their way out.
template <typename T, int K, int SKIP, int MODE, int NBUF>
__global__ void __launch_bounds__(kBlock * kSplitWaves) __attribute__((amdgpu_waves_per_eu(1, 2)))
backward_scan_split(const BwdParams p) {
    static_assert(sizeof(T) == 2, "16-bit streams");
    constexpr bool NTL = (MODE & kNtLoad) != 0, NTS = (MODE & kNtStore) != 0;
    constexpr bool HAS_PAD = (MODE & kHasPad) != 0, TANH = (MODE & kTanh) != 0;
    using G = SplitTile<K, SKIP>;
    using TU = typename G::TU;
    using T1 = typename G::T1;
    constexpr int TC = G::TC, W = G::W, PITCH = G::kPitch;
    fetch_params_early(p);
    // (without a skip term role 1 has no A output: a second tile takes those writes)
    __shared__ __attribute__((aligned(16))) unsigned char all_in[kSplitWaves][G::kBytes * (SKIP == 0 ? 2 : 1)];
    __shared__ __attribute__((aligned(16))) unsigned char all_gh[kSplitWaves][T1::kBytes];
    __shared__ uint32_t all_pad[kSplitWaves][kBlock];
    __shared__ float all_cstart[kSplitWaves][kBlock];
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x / kBlock));
    unsigned char *lds_in = all_in[wave], *lds_gh = all_gh[wave];
    uint32_t *lds_pad = all_pad[wave];
    float *lds_cstart = all_cstart[wave];

    const int lane = threadIdx.x % kBlock;
    const int c = lane >> 1, role = lane & 1;
    const int64_t colu = ((int64_t)blockIdx.x * kSplitWaves + wave) * W;
    if (colu >= p.ncols) return;
    const int64_t col = colu + c;
    const int Dp = p.Dp;
    const int ju = (int)(colu % Dp);
    const int j = ju + c;
    const bool flip = ju >= p.d;

    const float w = static_cast<const float *>(p.wc)[role * Dp + j];   // the lane's own gate
    const float knw = kNegLog2e * w, knb = kNegLog2e * p.bias[role * Dp + j];
    const float m = p.mask_c ? p.mask_c[col] : 1.0f;
    const float sx = (SKIP == 1 && p.scale_x) ? *p.scale_x : 1.0f;
    // scale of operand A: role 1's skip operand is x * scale_x, U[..., 3], or nothing (times zero)
    const float sa = role ? (SKIP == 0 ? 0.0f : sx) : 1.0f;
    const float oa_a = role ? m * sx : 1.0f, oa_b = role ? sx : 1.0f;   // see out_a below (sx is 1 unless the skip term is x)
    float cur = p.glast ? p.glast[col] : 0.0f;   // d loss / d state (meaningful in role 0); not given: zeros
    CompensatedSum sw, sb;      // the lane's gate: sums of its weight_c and bias gradients

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
    constexpr int kRowsPerChunk = TC / kCkptInterval;

    struct Stage {
        typename TU::Regs u;
        typename T1::Regs x, gh;
        uint32_t pad;
        float cstart;     // the chunk's start state as loaded; `keep` is applied when the chunk's turn comes:
        uint32_t keep;    // touched right after its load, the value would have to arrive, and since a
                          // wavefront's loads return in issue order, so would every tile of the chunk
    };
    int64_t ou[TU::kPieces], o1[T1::kPieces];
    TU::offsets(ou, lane, es * (K * 2));
    T1::offsets(o1, lane, es * 2);
    const unsigned char *ra = lds_in + G::elem_a(c, role), *rb = lds_in + G::elem_b(c, role);
    const unsigned char *rg = lds_gh + c * 2;
    // outputs: role 0 writes grad_u[0], grad_u[1]; role 1 writes grad_u[2] and its skip gradient
    // (grad_x into the x part of the tile, grad_u[3] for four streams, nothing without a skip term)
    unsigned char *wa = lds_in + (role == 0 ? c * K * 2
                                  : SKIP == 1 ? TU::kRowBytes + c * 2
                                  : SKIP == 2 ? c * K * 2 + 6
                                              : G::kBytes + c * 2);
    unsigned char *wb = lds_in + c * K * 2 + (role ? 4 : 2);

    auto load_chunk = [&](Stage &s, int64_t ch, const int64_t (&offu)[TU::kPieces], const int64_t (&off1)[T1::kPieces],
                          int rows) __attribute__((always_inline)) {
        const int64_t e0 = ef + ch * TC * es;
        TU::template load<NTL>(s.u, ubase + e0 * (K * 2), offu);
        if (SKIP == 1) T1::template load<NTL>(s.x, xbase + e0 * 2, off1);
        T1::template load<NTL>(s.gh, ghbase + e0 * 2, off1);
        if (HAS_PAD) s.pad = p.pad[pf + (ch * TC + min(lane % TC, rows - 1)) * ps];
        // one load from a selected address, so that every chunk issues the same operations
        // (without an initial state chunk 0 starts from zero: its load reads checkpoint row 0 and the
        // value is dropped with a bit mask. The address stays a select: blended with bit masks like the
        // value, the loop body became one basic block and 4-5 % slower.)
        const float *from = (ch == 0) ? (p.c0 ? p.c0 + col : p.ckpt + col) : p.ckpt + (ch * kRowsPerChunk - 1) * p.ncols + col;
        s.keep = (ch == 0 && !p.c0) ? 0u : ~0u;
        s.cstart = *from;
    };

    auto stage_to_lds = [&](const Stage &s) __attribute__((always_inline)) {
        TU::template to_lds<PITCH>(s.u, lds_in, lane);
        if (SKIP == 1) T1::template to_lds<PITCH>(s.x, lds_in + TU::kRowBytes, lane);
        T1::to_lds(s.gh, lds_gh, lane);
        if (HAS_PAD) reinterpret_cast<u32_a *>(lds_pad)[lane] = s.pad;
        lds_cstart[lane] = __builtin_bit_cast(float, __builtin_bit_cast(uint32_t, s.cstart) & s.keep);
        lds_handover();
    };

    auto compute_chunk = [&](int64_t ch, int n) __attribute__((always_inline)) {
        const uint32_t padreg = HAS_PAD ? reinterpret_cast<const u32_a *>(lds_pad)[lane] : 0u;
        float st[TC + 1];          // st[i] = state before step i (both lanes)
        float gt[TC], av[TC];      // the lane's gate and its operand A (u0 | skip operand) per step
        float vv[TC];              // role 0: state before the step; role 1: activation of the state after it
        st[0] = lds_cstart[lane];
        float bv[TC], ghv[TC];     // every LDS read of the chunk first (see forward_scan_split)
#pragma unroll
        for (int i = 0; i < TC; ++i) {
            if (i < n) {
                av[i] = lds_elem<T>(ra + i * PITCH);
                bv[i] = lds_elem<T>(rb + i * PITCH);
                ghv[i] = lds_elem<T>(rg + i * T1::kRowBytes);
            }
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int i = 0; i < TC; ++i) {
            if (i < n) {
                const bool padded = HAS_PAD && __builtin_amdgcn_readlane((int)padreg, i) != 0;
                const float b = bv[i];
                const float cp = st[i];
                gt[i] = sigmoid_exp2<T>(__builtin_fmaf(knw, cp, __builtin_fmaf(kNegLog2e, b, knb)));
                const float cn = pair_even((cp - av[i]) * gt[i] + av[i]);   // (role 0's operand A is u0 as it is)
                st[i + 1] = padded ? cp : cn;
                vv[i] = role ? (TANH ? tanh_fast(cn) : cn) : cp;
            }
        }
        lds_handover();   // every input row has been read: the gradients may take their place
        float gws = 0.f, gbs = 0.f;
#pragma unroll
        for (int i = TC - 1; i >= 0; --i) {
            if (i < n) {
                const bool padded = HAS_PAD && __builtin_amdgcn_readlane((int)padreg, i) != 0;
                const float gh = ghv[i];
                const float gg_ = gt[i], omg = 1.0f - gg_;
                const float d = gg_ * omg;                        // derivative of the lane's gate
                // role 1: what the output path hands to the state gradient
                const float ghm = gh * m;
                const float dact = TANH ? (1.0f - vv[i] * vv[i]) : 1.0f;
                const float to_state = pair_swap(TANH ? ghm * (gg_ * dact) : ghm * gg_);
                const float gc = to_state + cur;                   // role 0: d loss / d (state after the step)
                // the lane's gate gradient: role 0 gc * (c_prev - u0) * g1', role 1 gh * m * (val - skip) * g2'
                // (operand A scaled here: role 0 c_prev - u0, role 1 val - x * scale_x)
                const float gate_grad = (role ? ghm : gc) * __builtin_fmaf(-sa, av[i], vv[i]) * d;
                const float through_w = gate_grad * w;             // its way back into the previous state
                const float ncur = gc * gg_ + (through_w + pair_swap(through_w));
                // outputs A: role 0 grad of the candidate stream, gc * (1 - g1); role 1 grad of the skip
                // operand, gh * (1 - g2 * m) * scale_x: one product of a selected factor and
                // oa_b - gate * oa_a with per-lane constants
                const float out_a = (role ? gh : gc) * __builtin_fmaf(-gg_, oa_a, oa_b);
                lds_put<T>(wa + i * PITCH, padded ? 0.0f : out_a);
                lds_put<T>(wb + i * PITCH, padded ? 0.0f : gate_grad);
                gbs += padded ? 0.0f : gate_grad;
                gws += padded ? 0.0f : gate_grad * st[i];
                cur = padded ? cur : ncur;
            }
        }
        sw.add(gws);
        sb.add(gbs);
        lds_handover();
        const int64_t e0 = ef + ch * TC * es;
        typename TU::Regs gur;
        TU::template from_lds<PITCH>(gur, lds_in, lane);
        typename T1::Regs gxr;
        if (SKIP == 1) T1::template from_lds<PITCH>(gxr, lds_in + TU::kRowBytes, lane);
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

    if (role == 0) p.ginit[col] = cur;
    p.partial[role * p.ncols + col] = sw.value();         // rows of partial: gwc1, gwc2, gbias1, gbias2
    p.partial[(2 + role) * p.ncols + col] = sb.value();
}

}  // namespace sru_amd
