// Device-side code of the SRU recurrence kernels for gfx950.
//
// Mapping. One lane owns COLS (1 or 2) adjacent columns; a column is one (batch b,
// direction, hidden j) triple, col = b*D' + dir*d + j, exactly the column order of the
// (L, B, D') tensors. A 64-lane wavefront therefore reads 64*COLS*k consecutive
// elements of U per step and 64*COLS consecutive elements of every other stream, each
// lane with one vector instruction per stream (float: dwordx3 / dwordx4; 16-bit
// elements with COLS = 2: the same dword-granular mix, which is why the 16-bit kernels
// pair columns).
//
// Latency hiding. The time loop is strictly serial per column (both gates see the
// previous state), so memory latency is hidden by depth, not by width. The fast kernels
// (forward_scan_chunked, backward_scan_ckpt) cut the walk into chunks of 8 steps held in two
// alternating register sets: the loads of the next chunk are issued in one burst before the
// arithmetic of the current one. The general kernels and the backward kernel that reads the
// state after every step (forward_scan, backward_scan) keep a ring of P future steps in
// registers instead: each iteration consumes the oldest slot and refills it with the step P
// ahead.
//
// Directions. Columns of the second direction walk time backwards. The loop variable
// is the walk step s (uniform over the wavefront); the time index is s or L-1-s per lane.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace sru_amd {

constexpr int kBlock = 64;  // lanes of a wavefront; a wavefront is the unit of work of every kernel
// Wavefronts per workgroup of the chunked kernels (nothing is shared between them). Neighbouring
// wavefronts own neighbouring columns; in one workgroup they start together on one compute unit and
// stay close in time, so their 256- and 768-byte row segments reach memory as longer runs.
// (Four at most, one per SIMD, leave every wavefront the whole register file; the float kernels
// without a weight_c stream fit eight, i.e. into 256 registers.)
template <typename T> constexpr int max_waves_per_group(int mode) {
    return (sizeof(T) == 4 && (mode & 512) == 0) ? 8 : 4;
}

struct half_bits { uint16_t v; };  // IEEE binary16 storage
struct bf16_bits { uint16_t v; };  // bfloat16 storage

// Arithmetic type of a stream element type: double streams are computed in double (gates, state,
// sums and every small tensor; the general kernels only), everything else in float.
template <typename T> struct Arith { using type = float; };
template <> struct Arith<double> { using type = double; };
template <typename T> using arith_t = typename Arith<T>::type;

// ---------------------------------------------------------------- 16-bit conversion
template <typename T> __device__ __forceinline__ float bits_to_float(uint32_t h);  // h < 65536
template <> __device__ __forceinline__ float bits_to_float<half_bits>(uint32_t h) {
    return (float)__builtin_bit_cast(_Float16, (uint16_t)h);
}
template <> __device__ __forceinline__ float bits_to_float<bf16_bits>(uint32_t h) {
    return __builtin_bit_cast(float, h << 16);
}
template <typename T> __device__ __forceinline__ uint32_t float_to_bits(float v);  // round to nearest even
template <> __device__ __forceinline__ uint32_t float_to_bits<half_bits>(float v) {
    return __builtin_bit_cast(uint16_t, (_Float16)v);
}
template <> __device__ __forceinline__ uint32_t float_to_bits<bf16_bits>(float v) {
    return __builtin_bit_cast(uint16_t, (__bf16)v);
}
// two floats -> one dword of two 16-bit elements (lo first), one packed conversion
typedef float float2v __attribute__((ext_vector_type(2)));
template <typename T> __device__ __forceinline__ uint32_t pack_pair(float lo, float hi);
template <> __device__ __forceinline__ uint32_t pack_pair<half_bits>(float lo, float hi) {
    typedef _Float16 half2v __attribute__((ext_vector_type(2)));
    return __builtin_bit_cast(uint32_t, __builtin_convertvector((float2v){lo, hi}, half2v));
}
template <> __device__ __forceinline__ uint32_t pack_pair<bf16_bits>(float lo, float hi) {
    typedef __bf16 bf2v __attribute__((ext_vector_type(2)));
    return __builtin_bit_cast(uint32_t, __builtin_convertvector((float2v){lo, hi}, bf2v));
}

// ---------------------------------------------------------------- groups of N consecutive elements
// A Group is what one lane moves per stream and step. It is loaded and stored whole, as
// one vector of 1-4 dwords (one memory instruction), and stays in that storage form
// inside the register ring (16-bit pairs stay packed in dwords).
constexpr int group_align(int bytes) {
    return bytes % 16 == 0 ? 16 : bytes % 8 == 0 ? 8 : bytes % 4 == 0 ? 4 : 2;
}

// W dwords moved as one unit. Up to four they are one vector value; the vector types are
// declared dword-aligned because a group starts wherever its column starts.
template <int W> struct WordVec { typedef uint32_t type __attribute__((ext_vector_type(W), aligned(4))); };
template <> struct WordVec<1> { typedef uint32_t type; };

template <int W, bool VEC = (W <= 4)> struct Words;
template <int W> struct Words<W, true> {
    typename WordVec<W>::type v;
    __device__ __forceinline__ uint32_t get(int i) const {
        if constexpr (W == 1) return v;
        else return v[i];
    }
    __device__ __forceinline__ void set(int i, uint32_t x) {
        if constexpr (W == 1) v = x;
        else v[i] = x;
    }
};
template <int W> struct Words<W, false> {  // 6 or 8 dwords: two vectors of 3 or 4
    static_assert(W == 6 || W == 8, "wide groups are two vectors");
    typename WordVec<W / 2>::type lo, hi;
    __device__ __forceinline__ uint32_t get(int i) const { return i < W / 2 ? lo[i] : hi[i - W / 2]; }
    __device__ __forceinline__ void set(int i, uint32_t x) {
        if (i < W / 2) lo[i] = x;
        else hi[i - W / 2] = x;
    }
};

// storage kind: 0 float, 1 even count of 16-bit elements, 2 odd count of 16-bit elements, 3 double
template <typename T, int N> constexpr int group_kind() {
    return sizeof(T) == 8 ? 3 : sizeof(T) == 4 ? 0 : (N % 2 == 0 ? 1 : 2);
}

template <typename T, int N, int KIND = group_kind<T, N>()> struct Group;

template <int N>
struct Group<float, N, 0> {
    static constexpr int kWords = N;
    Words<N> w;
    __device__ __forceinline__ float get(int i) const { return __builtin_bit_cast(float, w.get(i)); }
    __device__ __forceinline__ static Group make(const float (&v)[N]) {
        Group g;
#pragma unroll
        for (int i = 0; i < N; ++i) g.w.set(i, __builtin_bit_cast(uint32_t, v[i]));
        return g;
    }
};

// even count of 16-bit elements: dwords holding two each
template <typename T, int N>
struct Group<T, N, 1> {
    static constexpr int kWords = N / 2;
    Words<N / 2> w;
    __device__ __forceinline__ float get(int i) const {
        const uint32_t d = w.get(i / 2);
        return bits_to_float<T>((i & 1) ? (d >> 16) : (d & 0xffffu));
    }
    __device__ __forceinline__ static Group make(const float (&v)[N]) {
        Group g;
#pragma unroll
        for (int i = 0; i < N / 2; ++i) g.w.set(i, pack_pair<T>(v[2 * i], v[2 * i + 1]));
        return g;
    }
};

// odd count of 16-bit elements (one column per lane): element-wise
template <typename T, int N>
struct alignas(2) Group<T, N, 2> {
    static constexpr int kWords = 0;
    uint16_t h[N];
    __device__ __forceinline__ float get(int i) const { return bits_to_float<T>(h[i]); }
    __device__ __forceinline__ static Group make(const float (&v)[N]) {
        Group g;
#pragma unroll
        for (int i = 0; i < N; ++i) g.h[i] = (uint16_t)float_to_bits<T>(v[i]);
        return g;
    }
};

// doubles: two dwords each (1 to 4 elements: one vector, or two vectors of 3 or 4 dwords)
template <int N>
struct Group<double, N, 3> {
    static constexpr int kWords = 2 * N;
    Words<2 * N> w;
    __device__ __forceinline__ double get(int i) const {
        return __builtin_bit_cast(double, (uint64_t)w.get(2 * i) | ((uint64_t)w.get(2 * i + 1) << 32));
    }
    __device__ __forceinline__ static Group make(const double (&v)[N]) {
        Group g;
#pragma unroll
        for (int i = 0; i < N; ++i) {
            const uint64_t b = __builtin_bit_cast(uint64_t, v[i]);
            g.w.set(2 * i, (uint32_t)b);
            g.w.set(2 * i + 1, (uint32_t)(b >> 32));
        }
        return g;
    }
};

// NT: mark the access non-temporal (streamed once; do not keep the line in the caches);
// applies to groups that travel as one or two vectors of dwords.
template <typename T, int N, bool NT = false>
__device__ __forceinline__ Group<T, N> load_group(const T *p) {
    typedef Group<T, N> G;
    constexpr int W = G::kWords;
    if constexpr (W >= 1 && W <= 4) {
        typedef typename WordVec<W>::type vec_t;
        G g;
        if constexpr (NT) g.w.v = __builtin_nontemporal_load(reinterpret_cast<const vec_t *>(p));
        else g.w.v = *reinterpret_cast<const vec_t *>(p);
        return g;
    } else if constexpr (W == 6 || W == 8) {
        typedef typename WordVec<W / 2>::type vec_t;
        const char *q = reinterpret_cast<const char *>(p);
        G g;
        if constexpr (NT) {
            g.w.lo = __builtin_nontemporal_load(reinterpret_cast<const vec_t *>(q));
            g.w.hi = __builtin_nontemporal_load(reinterpret_cast<const vec_t *>(q + 2 * W));
        } else {
            g.w.lo = *reinterpret_cast<const vec_t *>(q);
            g.w.hi = *reinterpret_cast<const vec_t *>(q + 2 * W);
        }
        return g;
    } else {
        return *reinterpret_cast<const G *>(p);
    }
}
template <typename T, int N, bool NT = false>
__device__ __forceinline__ void store_group(T *p, const arith_t<T> (&v)[N]) {
    typedef Group<T, N> G;
    constexpr int W = G::kWords;
    const G g = G::make(v);
    if constexpr (W >= 1 && W <= 4) {
        typedef typename WordVec<W>::type vec_t;
        if constexpr (NT) __builtin_nontemporal_store(g.w.v, reinterpret_cast<vec_t *>(p));
        else *reinterpret_cast<vec_t *>(p) = g.w.v;
    } else if constexpr (W == 6 || W == 8) {
        typedef typename WordVec<W / 2>::type vec_t;
        char *q = reinterpret_cast<char *>(p);
        if constexpr (NT) {
            __builtin_nontemporal_store(g.w.lo, reinterpret_cast<vec_t *>(q));
            __builtin_nontemporal_store(g.w.hi, reinterpret_cast<vec_t *>(q + 2 * W));
        } else {
            *reinterpret_cast<vec_t *>(q) = g.w.lo;
            *reinterpret_cast<vec_t *>(q + 2 * W) = g.w.hi;
        }
    } else {
        *reinterpret_cast<G *>(p) = g;
    }
}

// ---------------------------------------------------------------- a lane's share of a stream
// What one lane moves per stream and step (N elements per column), and how it finds its
// own elements in it.
//   plain: the lane's COLS columns form one Group<T, COLS*N> at the lane's own element.
//   PAIR (16-bit elements, one column per lane): lanes 2i and 2i+1 own adjacent columns
//   whose N+N elements form one dword-granular group. Both lanes load that group (same
//   address: the hardware serves the pair with one fetch) and each picks its half; for a
//   store the even lane takes the odd lane's values through a DPP lane swap and writes the
//   group, the odd lane writes nothing. This keeps one column per lane (twice the
//   wavefronts of COLS = 2, which matters when columns are few) with the same dword-wide
//   memory instructions.
template <typename T, int N, int COLS, bool PAIR>
struct Stream {
    static_assert(!PAIR || (COLS == 1 && sizeof(T) == 2), "pairs are for 16-bit elements, one column per lane");
    static constexpr int kElems = (PAIR ? 2 : COLS) * N;
    using G = Group<T, kElems>;

    // row: pointer to the stream's elements of the wavefront's (or lane's) first column at this
    // step; lane: the lane's column offset from there; q: lane parity
    // (signed arithmetic: with per-lane row pointers lane is 0 and the odd lane of a pair
    // steps back to the even lane's column)
    template <bool NT>
    __device__ __forceinline__ static G load(const T *row, uint32_t lane, int q) {
        const int32_t first = (int32_t)lane - (PAIR ? q : 0);
        return load_group<T, kElems, NT>(row + first * N);
    }
    // all elements of the lane's columns as floats: out[c * N + i] = element i of column c
    __device__ __forceinline__ static void unpack(const G &g, int q, float (&out)[COLS * N]) {
        if constexpr (!PAIR) {
#pragma unroll
            for (int i = 0; i < COLS * N; ++i) out[i] = g.get(i);
        } else {
            // The pair's group holds the even lane's N elements, then the odd lane's. Whole-dword
            // selects and one funnel shift move the lane's own elements to the front (a select
            // between g.get(i) and g.get(N + i) would become a run-time vector index).
            const uint32_t sh = (N % 2) ? 16u * (uint32_t)q : 0u;  // odd N: the odd lane starts mid-dword
            constexpr int W = (N + 1) / 2;                         // dwords holding the lane's elements
            uint32_t own[W];
            if constexpr (N % 2 == 0) {
#pragma unroll
                for (int i = 0; i < W; ++i) own[i] = q ? g.w.get(W + i) : g.w.get(i);
            } else if constexpr (N == 1) {
                own[0] = g.w.get(0) >> sh;
            } else {
                static_assert(N == 3, "odd groups are 1 or 3 elements");
                const uint32_t a = q ? g.w.get(1) : g.w.get(0);
                const uint32_t b = q ? g.w.get(2) : g.w.get(1);
                own[0] = __builtin_amdgcn_alignbit(b, a, sh);
                own[1] = b >> sh;
            }
#pragma unroll
            for (int i = 0; i < N; ++i)
                out[i] = bits_to_float<T>((i & 1) ? (own[i / 2] >> 16) : (own[i / 2] & 0xffffu));
        }
    }
    template <bool NT>
    __device__ __forceinline__ static void store(T *row, uint32_t lane, int q, const float (&v)[COLS * N]) {
        if constexpr (PAIR) {
            float both[2 * N];
#pragma unroll
            for (int i = 0; i < N; ++i) {
                both[i] = v[i];
                // quad_perm [1,0,3,2]: the value of the neighbouring lane of the pair (every lane
                // of a quad is a valid source, so with bound_ctrl set no previous value of the
                // destination is needed and none has to be materialised)
                both[N + i] = __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(
                    0, __builtin_bit_cast(int, v[i]), 0xB1, 0xf, 0xf, true));
            }
            if (q == 0) store_group<T, kElems, NT>(row + (int32_t)lane * N, both);
        } else {
            store_group<T, kElems, NT>(row + (int32_t)lane * N, v);
        }
    }
};

// ---------------------------------------------------------------- gate arithmetic
// sigmoid through the hardware exp2 and reciprocal (1 ulp each). The reciprocal's ulp is the
// largest part of the error where the gate is close to 1, and the state carries it along the
// whole walk, so float streams refine it with one Newton step (two fused multiply-adds): the
// result is then within 1e-7 of the exact sigmoid over the whole real line. 16-bit streams
// round their outputs to 2^-9 and skip the step. Saturates cleanly to 0 (2^-126) and 1.
#ifndef SRU_AMD_REFINE_SIGMOID
#define SRU_AMD_REFINE_SIGMOID 1
#endif
constexpr float kNegLog2e = -1.4426950408889634f;

// 1 / (1 + 2^t): the sigmoid of v for t = -log2(e) * v
template <typename T>
__device__ __forceinline__ float sigmoid_exp2(float t) {
    if constexpr (sizeof(T) == 4 && SRU_AMD_REFINE_SIGMOID) {
        // the exponent is capped so that d stays finite (inf * 0 in the correction would be NaN);
        // at the cap the result is 2^-126
        const float d = 1.0f + __builtin_amdgcn_exp2f(fminf(t, 126.0f));
        const float r = __builtin_amdgcn_rcpf(d);
        return __builtin_fmaf(__builtin_fmaf(-d, r, 1.0f), r, r);
    } else {
        return __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(t));
    }
}

// A gate: sigmoid(u + w * c + b). For 16-bit streams the factor -log2(e) that turns exp into the
// hardware's exp2 is folded into the operands: -log2(e) * w and -log2(e) * b are loop invariants
// (per-column constants, hoisted by the compiler), and u enters through a multiply-add that does
// not wait for the state, so the chain that depends on the state c is one multiply-add, exp2,
// add, reciprocal. Float streams keep the sum in its own scale and multiply afterwards: the folded
// form rounds relative to the terms instead of to their (often much smaller) sum, which doubled the
// largest gradient error at the headline shape.
// Double streams: the double-precision exp of the device library (saturates to 0 and 1 through inf
// like the float forms).
template <typename T>
__device__ __forceinline__ arith_t<T> gate(arith_t<T> u, arith_t<T> w, arith_t<T> c, arith_t<T> b) {
    if constexpr (sizeof(T) == 8) return 1.0 / (1.0 + exp(-(u + w * c + b)));
    else if constexpr (sizeof(T) == 4) return sigmoid_exp2<T>(kNegLog2e * (u + w * c + b));
    else return sigmoid_exp2<T>(__builtin_fmaf(kNegLog2e * w, c, __builtin_fmaf(kNegLog2e, u, kNegLog2e * b)));
}

// tanh through the same two units: 1 - 2 / (1 + e^(2v)). Absolute error below 3e-7 over the
// whole real line (the cancellation near 0 costs relative, not absolute, accuracy); saturates
// cleanly to -1 and 1.
__device__ __forceinline__ float tanh_fast(float v) {
    return 1.0f - 2.0f * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(2.8853900817779268f * v));
}
template <typename T>
__device__ __forceinline__ arith_t<T> tanh_of(arith_t<T> v) {
    if constexpr (sizeof(T) == 8) return tanh(v);
    else return tanh_fast(v);
}

// ---------------------------------------------------------------- kernel parameters
// The small tensors (bias, initial state, masks, scale, last state, partial sums) are typed for the
// float kernels; with double streams they hold doubles and the general kernels read them through
// as_arith<double>().
template <typename A> __device__ __forceinline__ const A *as_arith(const float *q) { return reinterpret_cast<const A *>(q); }
template <typename A> __device__ __forceinline__ A *as_arith(float *q) { return reinterpret_cast<A *>(q); }

struct FwdParams {
    const void *u, *x, *wc;
    const float *bias, *c0, *mask_c;
    const uint8_t *pad;
    const float *scale_x;
    void *h, *c;
    float *c_last;
    float *ckpt;          // (L / kCkptInterval, B, D') float state checkpoints, or nullptr
    int64_t L, B, ncols;  // ncols = B * D'
    int32_t d, Dp;        // hidden per direction, D' = dirs * d
    int32_t act, custom;  // act: host-side kernel selection and the general kernels; custom: general kernels
    int32_t x_float;      // host-side kernel selection: x is float next to 16-bit streams
};

struct BwdParams {
    const void *u, *x, *wc;
    const float *bias, *c0, *mask_c;
    const uint8_t *pad;
    const float *scale_x;
    const void *c, *gh;
    const float *ckpt;    // state checkpoints written by the forward pass (checkpoint kernels)
    const float *glast;
    void *gu, *gx, *gwc_steps;  // gwc_steps: per-step weight_c gradient (custom only)
    float *ginit;
    float *partial;  // (4, ncols): per-column sums gwc1, gwc2, gbias1, gbias2
    int64_t L, B, ncols;
    int32_t d, Dp;
    int32_t act, custom;
    int32_t x_float;      // host-side kernel selection: x and grad_x are float next to 16-bit streams
};

// Every field of the parameter block is read at the top of a kernel. Left alone, the compiler
// fetches each field from the kernel-argument segment right before its first use, which makes the
// prologue a chain of dependent scalar-memory round trips (one per basic block that needs a new
// field); pinned here, the fields arrive with a few wide scalar loads behind one wait.
#define SRU_AMD_PIN(v) asm volatile("" ::"s"(v))
__device__ __forceinline__ void fetch_params_early(const FwdParams &p) {
    SRU_AMD_PIN(p.u); SRU_AMD_PIN(p.x); SRU_AMD_PIN(p.wc); SRU_AMD_PIN(p.bias); SRU_AMD_PIN(p.c0);
    SRU_AMD_PIN(p.mask_c); SRU_AMD_PIN(p.pad); SRU_AMD_PIN(p.scale_x); SRU_AMD_PIN(p.h); SRU_AMD_PIN(p.c);
    SRU_AMD_PIN(p.c_last); SRU_AMD_PIN(p.ckpt); SRU_AMD_PIN(p.L); SRU_AMD_PIN(p.B); SRU_AMD_PIN(p.ncols);
    SRU_AMD_PIN(p.d); SRU_AMD_PIN(p.Dp);
}
__device__ __forceinline__ void fetch_params_early(const BwdParams &p) {
    SRU_AMD_PIN(p.u); SRU_AMD_PIN(p.x); SRU_AMD_PIN(p.wc); SRU_AMD_PIN(p.bias); SRU_AMD_PIN(p.c0);
    SRU_AMD_PIN(p.mask_c); SRU_AMD_PIN(p.pad); SRU_AMD_PIN(p.scale_x); SRU_AMD_PIN(p.c); SRU_AMD_PIN(p.gh);
    SRU_AMD_PIN(p.ckpt); SRU_AMD_PIN(p.glast); SRU_AMD_PIN(p.gu); SRU_AMD_PIN(p.gx); SRU_AMD_PIN(p.gwc_steps);
    SRU_AMD_PIN(p.ginit); SRU_AMD_PIN(p.partial); SRU_AMD_PIN(p.L); SRU_AMD_PIN(p.B); SRU_AMD_PIN(p.ncols);
    SRU_AMD_PIN(p.d); SRU_AMD_PIN(p.Dp);
}

// The loop body must stay one straight line of code for the compiler to keep the ring
// in fixed registers and count outstanding loads (a uniform branch inside it makes the
// inserted waits drain the ring at every step). The fast kernels therefore take "is
// there a padding mask", "is the per-step state kept" and the activation as template
// bits; the general kernels read those and the rarely used per-step weight_c option
// from the parameter block.
constexpr int kHasPad = 1;   // MODE bit (fast kernels): mask_pad given
constexpr int kKeepC = 2;    // MODE bit (fast forward kernels): c is stored
constexpr int kGeneral = 4;  // MODE bit: run-time pad / keep_c / act / custom
constexpr int kNtLoad = 8;   // MODE bit: stream loads are non-temporal
constexpr int kNtStore = 16; // MODE bit: stream stores are non-temporal
constexpr int kCkpt = 32;    // MODE bit (fast forward kernels): store a state checkpoint per chunk
constexpr int kPair = 64;    // MODE bit (chunked fast kernels, 16-bit): lanes pair up for memory access
constexpr int kTanh = 256;   // MODE bit (fast kernels): the output uses tanh(c_t) instead of c_t
constexpr int kCustom = 512; // MODE bit (chunked fast kernels): weight_c is a stream, (L, B, D', 2) in T
constexpr int kUniform = 128;// MODE bit (chunked fast kernels): a wavefront lies inside one direction and
                             // one batch row (d is a multiple of 64 * COLS), so the time index, the row
                             // pointers and the padding flag are scalar: no per-lane address arithmetic

// Checkpointed state. Instead of the state after every step (4 bytes per cell written by
// the forward pass and read again by the backward pass), the forward pass can keep only
// the state after every kCkptInterval-th step of each column's walk, in float, whatever
// the stream type: row r of the checkpoint array is the state after walk step
// (r+1)*kCkptInterval - 1. The backward pass then rebuilds the states inside a chunk
// from its checkpoint while it holds the chunk's U in registers anyway.
constexpr int kCkptInterval = 8;

// Kahan-compensated accumulation of one chunk's (or ring round's) sum `part` into a running sum
// that lives over the whole walk: the running sums of the weight_c / bias gradients have
// L terms per column, and plain float accumulation of that many terms was the largest single
// contribution to their error. Four instructions per chunk and sum, not per cell.
template <typename A>
struct CompensatedSumOf {
    A sum = 0, comp = 0;
    __device__ __forceinline__ void add(A part) {
        const A y = part - comp;
        const A t = sum + y;
        comp = (t - sum) - y;
        sum = t;
    }
    __device__ __forceinline__ A value() const { return sum - comp; }
};
using CompensatedSum = CompensatedSumOf<float>;

// Waits for every vector-memory operation issued so far (s_waitcnt vmcnt(0), gfx9 encoding).
// Placed once before a pipelined loop: whatever was loaded before the loop and is used inside it
// would otherwise make the compiler place a wait inside the loop whose count also drains the
// loads the loop keeps in flight on purpose.
__device__ __forceinline__ void wait_for_all_loads() { __builtin_amdgcn_s_waitcnt(0x0F70); }

// ================================================================= forward scan
// T: stream element type. K: streams per column in U. SKIP: 0 none, 1 from x, 2 from
// U[..., 3]. COLS: columns per lane (2 needs an even d). P: ring depth.
template <typename T, int K, int SKIP, int MODE, int COLS, int P>
__global__ void __launch_bounds__(kBlock * 4) forward_scan(const FwdParams p) {
    using A = arith_t<T>;
    constexpr bool GENERAL = (MODE & kGeneral) != 0;
    static_assert(sizeof(T) != 8 || (GENERAL && COLS == 1), "double streams: the general kernels, one column per lane");
    constexpr bool NTL = (MODE & kNtLoad) != 0, NTS = (MODE & kNtStore) != 0;
    static_assert((MODE & (kCkpt | kPair | kUniform)) == 0, "those exist in the chunked kernels only");
    const int64_t col = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) * COLS;  // lane's first column
    if (col >= p.ncols) return;

    const int Dp = p.Dp;
    const int j = (int)(col % Dp);
    const int64_t b = col / Dp;
    const bool flip = j >= p.d;  // second direction; never true when dirs == 1 (d == D')
    const bool custom = GENERAL && p.custom;
    const bool use_tanh = GENERAL ? (p.act != 0) : ((MODE & kTanh) != 0);
    const bool has_pad = GENERAL ? (p.pad != nullptr) : ((MODE & kHasPad) != 0);
    const bool keep_c = GENERAL ? (p.c != nullptr) : ((MODE & kKeepC) != 0);

    A wc1[COLS], wc2[COLS], b1[COLS], b2[COLS], m[COLS], cur[COLS];
#pragma unroll
    for (int c = 0; c < COLS; ++c) {
        wc1[c] = custom ? A(0) : static_cast<const A *>(p.wc)[j + c];
        wc2[c] = custom ? A(0) : static_cast<const A *>(p.wc)[Dp + j + c];
        b1[c] = as_arith<A>(p.bias)[j + c];
        b2[c] = as_arith<A>(p.bias)[Dp + j + c];
        m[c] = p.mask_c ? as_arith<A>(p.mask_c)[col + c] : A(1);
        cur[c] = p.c0 ? as_arith<A>(p.c0)[col + c] : A(0);   // no initial state given: zeros
    }
    const A sx = (SKIP == 1 && p.scale_x) ? *as_arith<A>(p.scale_x) : A(1);

    const int64_t L = p.L;
    const int64_t e0 = (flip ? (L - 1) : 0) * p.ncols + col;  // element of the first walk step
    const int64_t es = flip ? -p.ncols : p.ncols;             // elements per walk step
    const T *up = static_cast<const T *>(p.u) + e0 * K;
    const T *xp = (SKIP == 1) ? static_cast<const T *>(p.x) + e0 : nullptr;
    const T *vp = custom ? static_cast<const T *>(p.wc) + e0 * 2 : nullptr;
    const uint8_t *pp = has_pad ? p.pad + (flip ? (L - 1) : 0) * p.B + b : nullptr;
    const int64_t ps = flip ? -p.B : p.B;
    T *hp = static_cast<T *>(p.h) + e0;
    T *cp = keep_c ? static_cast<T *>(p.c) + e0 : nullptr;
    struct Slot {
        Group<T, COLS * K> u;
        Group<T, COLS> x;
        Group<T, COLS * 2> w;
        uint32_t pad;
    };
    Slot ring[P];

    auto fetch = [&](Slot &s) {
        s.u = load_group<T, COLS * K, NTL>(up);
        up += es * K;
        if (SKIP == 1) {
            s.x = load_group<T, COLS, NTL>(xp);
            xp += es;
        }
        if (custom) {
            s.w = load_group<T, COLS * 2, NTL>(vp);
            vp += es * 2;
        }
        s.pad = 0;
        if (has_pad) {
            s.pad = *pp;
            pp += ps;
        }
    };

    auto consume = [&](const Slot &s) {
        const bool padded = s.pad != 0;
        A hv[COLS], cv[COLS];
#pragma unroll
        for (int c = 0; c < COLS; ++c) {
            const A u0 = s.u.get(c * K), u1 = s.u.get(c * K + 1), u2 = s.u.get(c * K + 2);
            const A w1 = custom ? s.w.get(2 * c) : wc1[c];
            const A w2 = custom ? s.w.get(2 * c + 1) : wc2[c];
            const A g1 = gate<T>(u1, w1, cur[c], b1[c]);
            const A g2 = gate<T>(u2, w2, cur[c], b2[c]);
            const A cn = (cur[c] - u0) * g1 + u0;
            const A val = use_tanh ? tanh_of<T>(cn) : cn;
            A out;
            if (SKIP != 0) {
                const A xv = (SKIP == 1) ? s.x.get(c) * sx : s.u.get(c * K + K - 1);
                out = (val - xv) * m[c] * g2 + xv;
            } else {
                out = val * m[c] * g2;
            }
            cur[c] = padded ? cur[c] : cn;   // a padded step keeps the state ...
            hv[c] = padded ? A(0) : out;     // ... and emits zero
            cv[c] = cur[c];
        }
        store_group<T, COLS, NTS>(hp, hv);
        hp += es;
        if (keep_c) {
            store_group<T, COLS, NTS>(cp, cv);
            cp += es;
        }
    };

#pragma unroll
    for (int i = 0; i < P; ++i)
        if (i < L) fetch(ring[i]);

    int64_t s0 = 0;
    for (; s0 + 2 * P <= L; s0 += P) {  // steady state: every consumed slot is refilled
#pragma unroll
        for (int i = 0; i < P; ++i) {
            consume(ring[i]);
            fetch(ring[i]);
            // Keep the steps in program order: left alone, the scheduler gathers all
            // loads of a round at its end, where none of them has time to land.
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    for (; s0 < L; s0 += P) {  // last one or two rounds
#pragma unroll
        for (int i = 0; i < P; ++i) {
            if (s0 + i < L) {
                const Slot s = ring[i];
                if (s0 + i + P < L) fetch(ring[i]);
                consume(s);
            }
        }
    }
#pragma unroll
    for (int c = 0; c < COLS; ++c) as_arith<A>(p.c_last)[col + c] = cur[c];
}

// Window of a wavefront's walk outside of which every step is padded, for wavefronts whose lanes
// share one batch row (kUniform): [lo, hi) in walk steps, lo = hi = 0 when the whole row is
// padding. Lane l looks at steps l, l + 64, ...; the flags of any mask are honoured inside the
// window, so only leading and trailing padding is skipped (right-padded batches: the tail of the
// forward direction's walk, the head of the reverse direction's).
struct LiveWindow { int64_t lo, hi; };
__device__ __forceinline__ LiveWindow live_window(const uint8_t *pad, int64_t pf, int64_t ps, int64_t L) {
    if (L >= (INT64_C(1) << 30)) return {0, L};
    int lo = (int)L, hi = 0;
#pragma unroll 8
    for (int s = (int)(threadIdx.x % kBlock); s < (int)L; s += kBlock) {
        const bool live = pad[pf + s * ps] == 0;
        lo = live ? min(lo, s) : lo;
        hi = live ? max(hi, s + 1) : hi;
    }
#pragma unroll
    for (int off = kBlock / 2; off > 0; off >>= 1) {
        lo = min(lo, __shfl_xor(lo, off, kBlock));
        hi = max(hi, __shfl_xor(hi, off, kBlock));
    }
    lo = __builtin_amdgcn_readfirstlane(lo);
    hi = __builtin_amdgcn_readfirstlane(hi);
    if (hi <= lo) return {0, 0};
    return {lo, hi};
}

// ================================================================= forward scan, chunked
// Same results as forward_scan. Instead of a ring refilled step by step, the walk is cut
// into chunks of TC steps held in two alternating register sets: the loads of chunk n+1
// are issued in one burst before the arithmetic of chunk n, so a wavefront waits for a
// chunk it requested a whole chunk-time earlier while the next one is already in flight.
// (Fast kernels only; TC equals the checkpoint interval. The two lambdas must be inlined at
// every call site: a chunk that is passed by reference to a real function lives in scratch
// memory instead of registers.)
// TX: element type of x (the skip term when SKIP == 1): T, or float next to 16-bit streams (under
// autocast the layer's input stays float while U comes out of the projection in 16 bits).
template <typename T, int K, int SKIP, int MODE, int COLS, int TC, typename TX = T>
__global__ void __launch_bounds__(kBlock * max_waves_per_group<T>(MODE)) forward_scan_chunked(const FwdParams p) {
    static_assert((MODE & kGeneral) == 0, "fast kernels only");
    static_assert(TC == kCkptInterval, "a chunk is one checkpoint interval");
    static_assert(sizeof(TX) == sizeof(T) || (sizeof(TX) == 4 && SKIP == 1), "a float x next to 16-bit streams");
    constexpr bool NTL = (MODE & kNtLoad) != 0, NTS = (MODE & kNtStore) != 0;
    constexpr bool HAS_PAD = (MODE & kHasPad) != 0, KEEP_C = (MODE & kKeepC) != 0;
    constexpr bool CKPT = (MODE & kCkpt) != 0, PAIR = (MODE & kPair) != 0, UNI = (MODE & kUniform) != 0;
    constexpr bool TANH = (MODE & kTanh) != 0, CUSTOM = (MODE & kCustom) != 0;
    // Wave-uniform kernels with a padding mask: all lanes of a wavefront share the flags, so one
    // load per chunk fetches them (lane l the flag of step l % TC) instead of one load per step,
    // which leaves more of the 64 outstanding memory operations a wavefront may have to the
    // streams: 4 % at L=4096 fp16 inference. Not with lane pairing: those shapes are short of
    // issue slots, and reading a flag back from its lane costs one instruction more per step.
    constexpr bool PAD_BY_LANE = HAS_PAD && UNI && !PAIR;
    constexpr int kPadRegs = PAD_BY_LANE ? 1 : TC;
    fetch_params_early(p);
    using SU = Stream<T, K, COLS, PAIR>;   // U: K elements per column
    using S1 = Stream<T, 1, COLS, PAIR>;   // h, c: one element per column
    using SX = Stream<TX, 1, COLS, PAIR && sizeof(TX) == 2>;   // x (a float x needs no lane pairing)
    using SV = Stream<T, 2, COLS, PAIR>;   // a per-step weight_c: two elements per column
    // the wavefront's index in the launch (scalar), and the lane's in the wavefront
    const uint32_t wg = blockIdx.x * (blockDim.x / kBlock) + (uint32_t)__builtin_amdgcn_readfirstlane((int)(threadIdx.x / kBlock));
    const uint32_t wlane = threadIdx.x % kBlock;
    const int64_t col = ((int64_t)wg * kBlock + wlane) * COLS;
    if (col >= p.ncols) return;
    const int q = PAIR ? (int)(wlane & 1) : 0;  // columns of a pair are col - q, col - q + 1

    // colu decides direction and batch row: the wavefront's first column when that is the same
    // for all its lanes (scalar), else the lane's own column
    const int64_t colu = UNI ? (int64_t)wg * (kBlock * COLS) : col;
    const uint32_t lane = (uint32_t)(col - colu);
    const int Dp = p.Dp;
    const int ju = (int)(colu % Dp);
    const int j = ju + (int)lane;
    const bool flip = ju >= p.d;

    float wc1[COLS], wc2[COLS], b1[COLS], b2[COLS], m[COLS], cur[COLS];
#pragma unroll
    for (int c = 0; c < COLS; ++c) {
        wc1[c] = CUSTOM ? 0.f : static_cast<const float *>(p.wc)[j + c];
        wc2[c] = CUSTOM ? 0.f : static_cast<const float *>(p.wc)[Dp + j + c];
        b1[c] = p.bias[j + c];
        b2[c] = p.bias[Dp + j + c];
        m[c] = p.mask_c ? p.mask_c[col + c] : 1.0f;
        cur[c] = p.c0 ? p.c0[col + c] : 0.0f;   // no initial state given: zeros
    }
    const float sx = (SKIP == 1 && p.scale_x) ? *p.scale_x : 1.0f;

    const int64_t L = p.L;
    const int64_t ef = (flip ? (L - 1) : 0) * p.ncols + colu;  // element of walk step 0 (column colu)
    const int64_t es = flip ? -p.ncols : p.ncols;
    // per-lane on purpose: with a scalar address the padding bytes would come through the
    // scalar data cache, whose loads cannot be pipelined behind the vector loads
    const int64_t pf = (flip ? (L - 1) : 0) * p.B + col / Dp;
    const int64_t ps = flip ? -p.B : p.B;
    const T *ubase = static_cast<const T *>(p.u);
    const TX *xbase = static_cast<const TX *>(p.x);
    T *hbase = static_cast<T *>(p.h);
    T *cbase = static_cast<T *>(p.c);
    const T *vbase = static_cast<const T *>(p.wc);   // CUSTOM only

    struct Chunk {
        typename SU::G u[TC];
        typename SX::G x[TC];
        typename SV::G w[CUSTOM ? TC : 1];
        uint32_t pad[kPadRegs];  // padding flags of the chunk, see load_chunk
    };

    auto load_chunk = [&](Chunk &k, int64_t ch, int n) __attribute__((always_inline)) {
        const int64_t s0 = ch * TC;
#pragma unroll
        for (int i = 0; i < TC; ++i) {
            if (i < n) {
                const int64_t e = ef + (s0 + i) * es;
                k.u[i] = SU::template load<NTL>(ubase + e * K, lane, q);
                if (SKIP == 1) k.x[i] = SX::template load<NTL>(xbase + e, lane, q);
                if constexpr (CUSTOM) k.w[i] = SV::template load<NTL>(vbase + e * 2, lane, q);
                if (!PAD_BY_LANE) k.pad[i] = HAS_PAD ? p.pad[pf + (s0 + i) * ps] : 0;
            }
        }
        // one load for the whole chunk: lane l fetches the flag of step l % TC (clamped to the
        // chunk's last valid step), compute_chunk reads step i's flag from lane i
        if (PAD_BY_LANE) k.pad[0] = p.pad[pf + (s0 + min((int)(wlane % TC), n - 1)) * ps];
    };

    auto compute_chunk = [&](const Chunk &k, int64_t ch, int n) __attribute__((always_inline)) {
        const int64_t s0 = ch * TC;
#pragma unroll
        for (int i = 0; i < TC; ++i) {
            if (i < n) {
                // a padded step keeps the state and emits zero, through bit masks: with selects on a flag
                // that is uniform over the wavefront the compiler branches around the arithmetic, which
                // cuts the chunk into one basic block per step and column and serialises the columns
                const uint32_t flag = PAD_BY_LANE ? (uint32_t)__builtin_amdgcn_readlane((int)k.pad[0], i) : k.pad[i];
                const uint32_t keep = 0u - (uint32_t)(flag != 0);   // all ones at a padded step
                float hv[COLS], cv[COLS], uu[COLS * K], xx[COLS] = {};
                SU::unpack(k.u[i], q, uu);
                if (SKIP == 1) SX::unpack(k.x[i], q, xx);
                float ww[COLS * 2] = {};
                if constexpr (CUSTOM) SV::unpack(k.w[i], q, ww);
#pragma unroll
                for (int c = 0; c < COLS; ++c) {
                    const float u0 = uu[c * K];
                    const float g1 = gate<T>(uu[c * K + 1], CUSTOM ? ww[2 * c] : wc1[c], cur[c], b1[c]);
                    const float g2 = gate<T>(uu[c * K + 2], CUSTOM ? ww[2 * c + 1] : wc2[c], cur[c], b2[c]);
                    const float cn = (cur[c] - u0) * g1 + u0;
                    const float val = TANH ? tanh_fast(cn) : cn;
                    float out;
                    if constexpr (SKIP != 0) {
                        const float xv = (SKIP == 1) ? xx[c] * sx : uu[c * K + K - 1];
                        out = (val - xv) * m[c] * g2 + xv;
                    } else {
                        out = val * m[c] * g2;
                    }
                    cur[c] = __builtin_bit_cast(float, (__builtin_bit_cast(uint32_t, cur[c]) & keep) | (__builtin_bit_cast(uint32_t, cn) & ~keep));
                    hv[c] = __builtin_bit_cast(float, __builtin_bit_cast(uint32_t, out) & ~keep);
                    cv[c] = cur[c];
                }
                const int64_t e = ef + (s0 + i) * es;
                S1::template store<NTS>(hbase + e, lane, q, hv);
                if (KEEP_C) S1::template store<NTS>(cbase + e, lane, q, cv);
            }
        }
        if (CKPT && n == TC) {
#pragma unroll
            for (int c = 0; c < COLS; ++c) p.ckpt[ch * p.ncols + col + c] = cur[c];
        }
    };

    // steps the window leaves out are known to be padded: no loads, the outputs a padded step gets
    auto fill = [&](int64_t from, int64_t to) __attribute__((always_inline)) {
        const float zero[COLS] = {};
        for (int64_t s = from; s < to; ++s) {
            const int64_t e = ef + s * es;
            S1::template store<NTS>(hbase + e, lane, q, zero);
            if (KEEP_C) S1::template store<NTS>(cbase + e, lane, q, cur);
            if (CKPT && s % TC == TC - 1) {
#pragma unroll
                for (int c = 0; c < COLS; ++c) p.ckpt[(s / TC) * p.ncols + col + c] = cur[c];
            }
        }
    };

    const int64_t nfull = L / TC;
    const int tail = (int)(L - nfull * TC);
    int64_t ch = 0, nend = nfull;   // full chunks [ch, nend) are walked
    bool with_tail = tail > 0;      // and the ragged last chunk
    if constexpr (HAS_PAD && UNI) {
        const LiveWindow w = live_window(p.pad, pf, ps, L);
        ch = w.lo / TC;
        const int64_t chunks = (w.hi + TC - 1) / TC;
        nend = chunks < nfull ? chunks : nfull;
        with_tail = with_tail && chunks > nfull;
        fill(0, ch * TC);
    }
    Chunk ka, kb;
    if (ch < nend) load_chunk(ka, ch, TC);
    // two chunks per iteration: every prefetch inside the loop is a real chunk
    while (ch + 2 < nend) {
        load_chunk(kb, ch + 1, TC);
        __builtin_amdgcn_sched_barrier(0);  // all loads of the next chunk first, then the arithmetic
        compute_chunk(ka, ch, TC);
        __builtin_amdgcn_sched_barrier(0);
        load_chunk(ka, ch + 2, TC);
        __builtin_amdgcn_sched_barrier(0);
        compute_chunk(kb, ch + 1, TC);
        __builtin_amdgcn_sched_barrier(0);
        ch += 2;
    }
    // one or two full chunks remain (ka holds chunk ch), then the ragged tail
    if (ch + 1 < nend) {
        load_chunk(kb, ch + 1, TC);
        compute_chunk(ka, ch, TC);
        if (with_tail) load_chunk(ka, nfull, tail);
        compute_chunk(kb, ch + 1, TC);
        if (with_tail) compute_chunk(ka, nfull, tail);
    } else if (ch < nend) {
        if (with_tail) load_chunk(kb, nfull, tail);
        compute_chunk(ka, ch, TC);
        if (with_tail) compute_chunk(kb, nfull, tail);
    } else if (with_tail) {
        load_chunk(kb, nfull, tail);
        compute_chunk(kb, nfull, tail);
    }
    if constexpr (HAS_PAD && UNI) fill(with_tail ? L : nend * TC, L);
#pragma unroll
    for (int c = 0; c < COLS; ++c) p.c_last[col + c] = cur[c];
}

// ================================================================= backward scan
// Walks each column's steps in reverse order, carrying d(loss)/d(state). The gates are
// recomputed from U and the stored previous state. Sums of the weight_c and bias
// gradients over time stay in registers and leave the kernel as per-column partials;
// reduce_partials() then adds them over the batch in a fixed order.
template <typename T, int K, int SKIP, int MODE, int COLS, int P>
__global__ void __launch_bounds__(kBlock * 4) backward_scan(const BwdParams p) {
    using A = arith_t<T>;
    constexpr bool GENERAL = (MODE & kGeneral) != 0;
    static_assert(sizeof(T) != 8 || (GENERAL && COLS == 1), "double streams: the general kernels, one column per lane");
    constexpr bool NTL = (MODE & kNtLoad) != 0, NTS = (MODE & kNtStore) != 0;
    const int64_t col = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) * COLS;
    if (col >= p.ncols) return;

    const int Dp = p.Dp;
    const int j = (int)(col % Dp);
    const int64_t b = col / Dp;
    const bool flip = j >= p.d;
    const bool custom = GENERAL && p.custom;
    const bool use_tanh = GENERAL ? (p.act != 0) : ((MODE & kTanh) != 0);
    const bool has_pad = GENERAL ? (p.pad != nullptr) : ((MODE & kHasPad) != 0);

    A wc1[COLS], wc2[COLS], b1[COLS], b2[COLS], m[COLS], c_init[COLS];
    A cur[COLS];  // d loss / d state
    A gw1[COLS], gw2[COLS], gb1[COLS], gb2[COLS];  // sums of the current ring round
    CompensatedSumOf<A> sw1[COLS], sw2[COLS], sb1[COLS], sb2[COLS];  // sums over the whole walk
    auto fold_round = [&]() {
#pragma unroll
        for (int c = 0; c < COLS; ++c) {
            sw1[c].add(gw1[c]);
            sw2[c].add(gw2[c]);
            sb1[c].add(gb1[c]);
            sb2[c].add(gb2[c]);
            gw1[c] = gw2[c] = gb1[c] = gb2[c] = A(0);
        }
    };
#pragma unroll
    for (int c = 0; c < COLS; ++c) {
        wc1[c] = custom ? A(0) : static_cast<const A *>(p.wc)[j + c];
        wc2[c] = custom ? A(0) : static_cast<const A *>(p.wc)[Dp + j + c];
        b1[c] = as_arith<A>(p.bias)[j + c];
        b2[c] = as_arith<A>(p.bias)[Dp + j + c];
        m[c] = p.mask_c ? as_arith<A>(p.mask_c)[col + c] : A(1);
        c_init[c] = p.c0 ? as_arith<A>(p.c0)[col + c] : A(0);          // no initial state given: zeros
        cur[c] = p.glast ? as_arith<A>(p.glast)[col + c] : A(0);      // no gradient of the last state given: zeros
        gw1[c] = gw2[c] = gb1[c] = gb2[c] = A(0);
    }
    const A sx = (SKIP == 1 && p.scale_x) ? *as_arith<A>(p.scale_x) : A(1);

    const int64_t L = p.L;
    // The backward walk starts where the forward walk ended.
    const int64_t t_start = flip ? 0 : (L - 1);
    const int64_t e0 = t_start * p.ncols + col;
    const int64_t es = flip ? p.ncols : -p.ncols;
    const T *up = static_cast<const T *>(p.u) + e0 * K;
    const T *xp = (SKIP == 1) ? static_cast<const T *>(p.x) + e0 : nullptr;
    const T *vp = custom ? static_cast<const T *>(p.wc) + e0 * 2 : nullptr;
    const T *ghp = static_cast<const T *>(p.gh) + e0;
    const T *cpp = static_cast<const T *>(p.c) + e0 + es;  // state before the step
    const uint8_t *pp = has_pad ? p.pad + t_start * p.B + b : nullptr;
    const int64_t ps = flip ? p.B : -p.B;
    T *gup = static_cast<T *>(p.gu) + e0 * K;
    T *gxp = (SKIP == 1) ? static_cast<T *>(p.gx) + e0 : nullptr;
    T *gvp = custom ? static_cast<T *>(p.gwc_steps) + e0 * 2 : nullptr;

    A cv[COLS];  // state after the step being visited
    {
        const Group<T, COLS> g = load_group<T, COLS>(static_cast<const T *>(p.c) + e0);
#pragma unroll
        for (int c = 0; c < COLS; ++c) cv[c] = g.get(c);
    }

    struct Slot {
        Group<T, COLS * K> u;
        Group<T, COLS> x;
        Group<T, COLS * 2> w;
        Group<T, COLS> gh;
        Group<T, COLS> cprev;  // state before the step, as stored by the forward pass
        bool first;            // the column's first forward step: the state before it is c_init
        uint32_t pad;
    };
    Slot ring[P];

    auto fetch = [&](Slot &s, bool first) {
        s.u = load_group<T, COLS * K, NTL>(up);
        up += es * K;
        if (SKIP == 1) {
            s.x = load_group<T, COLS, NTL>(xp);
            xp += es;
        }
        if (custom) {
            s.w = load_group<T, COLS * 2, NTL>(vp);
            vp += es * 2;
        }
        s.gh = load_group<T, COLS, NTL>(ghp);
        ghp += es;
        s.first = first;
        // every step issues the same loads, so that the loop body stays one block and the waits count
        // exactly: the column's first step, whose previous state is c_init and not part of the
        // stream, reads the state after the step instead (a valid address) and drops it
        s.cprev = load_group<T, COLS, NTL>(cpp - (es & -(int64_t)first));
        cpp += es;
        s.pad = 0;
        if (has_pad) {
            s.pad = *pp;
            pp += ps;
        }
    };

    auto consume = [&](const Slot &s) {
        const bool padded = s.pad != 0;
        A gu[COLS * K], gx[COLS], gv[COLS * 2];
#pragma unroll
        for (int c = 0; c < COLS; ++c) {
            const A w1 = custom ? s.w.get(2 * c) : wc1[c];
            const A w2 = custom ? s.w.get(2 * c + 1) : wc2[c];
            const A cp = s.first ? c_init[c] : s.cprev.get(c);
            const A u0 = s.u.get(c * K);
            const A g1 = gate<T>(s.u.get(c * K + 1), w1, cp, b1[c]);
            const A g2 = gate<T>(s.u.get(c * K + 2), w2, cp, b2[c]);
            const A val = use_tanh ? tanh_of<T>(cv[c]) : cv[c];
            const A dact = use_tanh ? (A(1) - val * val) : A(1);
            const A xv = (SKIP == 0) ? A(0) : (SKIP == 1) ? s.x.get(c) * sx : s.u.get(c * K + K - 1);
            const A gh = s.gh.get(c);

            const A gg2 = gh * (val - xv) * m[c] * (g2 * (A(1) - g2));
            const A gc = gh * m[c] * (g2 * dact) + cur[c];
            const A gg1 = gc * (cp - u0) * (g1 * (A(1) - g1));
            const A gskip = gh * (A(1) - g2 * m[c]);
            const A ncur = gc * g1 + gg1 * w1 + gg2 * w2;

            gu[c * K] = padded ? A(0) : gc * (A(1) - g1);
            gu[c * K + 1] = padded ? A(0) : gg1;
            gu[c * K + 2] = padded ? A(0) : gg2;
            if (K == 4) gu[c * K + K - 1] = (padded || SKIP != 2) ? A(0) : gskip;
            gx[c] = padded ? A(0) : gskip * sx;
            gv[2 * c] = padded ? A(0) : gg1 * cp;
            gv[2 * c + 1] = padded ? A(0) : gg2 * cp;
            gb1[c] += padded ? A(0) : gg1;
            gw1[c] += padded ? A(0) : gg1 * cp;
            gb2[c] += padded ? A(0) : gg2;
            gw2[c] += padded ? A(0) : gg2 * cp;
            cur[c] = padded ? cur[c] : ncur;
            cv[c] = cp;  // the state before this step is the state after the next one visited
        }
        store_group<T, COLS * K, NTS>(gup, gu);
        gup += es * K;
        if (SKIP == 1) {
            store_group<T, COLS, NTS>(gxp, gx);
            gxp += es;
        }
        if (custom) {
            store_group<T, COLS * 2, NTS>(gvp, gv);
            gvp += es * 2;
        }
    };

#pragma unroll
    for (int i = 0; i < P; ++i)
        if (i < L) fetch(ring[i], i == L - 1);

    wait_for_all_loads();   // the ring's first fill: the waits inside the loop then count what the loop itself issued
    int64_t s0 = 0;
    for (; s0 + 2 * P <= L; s0 += P) {
#pragma unroll
        for (int i = 0; i < P; ++i) {
            consume(ring[i]);
            fetch(ring[i], s0 + i + P == L - 1);
            __builtin_amdgcn_sched_barrier(0);  // see forward_scan
        }
        fold_round();
    }
    for (; s0 < L; s0 += P) {
#pragma unroll
        for (int i = 0; i < P; ++i) {
            if (s0 + i < L) {
                const Slot s = ring[i];
                if (s0 + i + P < L) fetch(ring[i], s0 + i + P == L - 1);
                consume(s);
            }
        }
        fold_round();
    }

#pragma unroll
    for (int c = 0; c < COLS; ++c) {
        as_arith<A>(p.ginit)[col + c] = cur[c];
        as_arith<A>(p.partial)[col + c] = sw1[c].value();
        as_arith<A>(p.partial)[p.ncols + col + c] = sw2[c].value();
        as_arith<A>(p.partial)[2 * p.ncols + col + c] = sb1[c].value();
        as_arith<A>(p.partial)[3 * p.ncols + col + c] = sb2[c].value();
    }
}

// ================================================================= backward scan from checkpoints
// Same results as backward_scan, but the per-step state is rebuilt instead of read: the
// walk is cut into chunks of TC steps, visited last to first. For a chunk the kernel
// holds U, x and grad_h of its TC steps in registers, runs the forward recurrence from
// the chunk's checkpoint (keeping both gates and the states), then the backward
// recurrence over the same registers. Loads of the next chunk are issued before the
// arithmetic of the current one. Per cell: reads U (k), x, grad_h and 4/TC bytes of
// checkpoint; writes grad_u (k), grad_x.
// TX: element type of x and grad_x, see forward_scan_chunked.
template <typename T, int K, int SKIP, int MODE, int COLS, int TC, typename TX = T>
__global__ void __launch_bounds__(kBlock * max_waves_per_group<T>(MODE)) backward_scan_ckpt(const BwdParams p) {
    static_assert((MODE & kGeneral) == 0, "fast kernels only");
    static_assert(sizeof(TX) == sizeof(T) || (sizeof(TX) == 4 && SKIP == 1), "a float x next to 16-bit streams");
    constexpr bool NTL = (MODE & kNtLoad) != 0, NTS = (MODE & kNtStore) != 0;
    constexpr bool HAS_PAD = (MODE & kHasPad) != 0, PAIR = (MODE & kPair) != 0, UNI = (MODE & kUniform) != 0;
    // (forward_scan_chunked fetches the flags of a chunk with one load; here, where every flag
    // is needed twice, that measured 0-3 % slower, so the flags stay one load per step)
    constexpr bool TANH = (MODE & kTanh) != 0, CUSTOM = (MODE & kCustom) != 0;
    using SU = Stream<T, K, COLS, PAIR>;   // U, grad_u: K elements per column
    using S1 = Stream<T, 1, COLS, PAIR>;   // grad_h: one element per column
    using SX = Stream<TX, 1, COLS, PAIR && sizeof(TX) == 2>;   // x, grad_x
    using SV = Stream<T, 2, COLS, PAIR>;   // a per-step weight_c and its gradient: two elements per column
    fetch_params_early(p);
    // the wavefront's index in the launch (scalar), and the lane's in the wavefront
    const uint32_t wg = blockIdx.x * (blockDim.x / kBlock) + (uint32_t)__builtin_amdgcn_readfirstlane((int)(threadIdx.x / kBlock));
    const uint32_t wlane = threadIdx.x % kBlock;
    const int64_t col = ((int64_t)wg * kBlock + wlane) * COLS;
    if (col >= p.ncols) return;
    const int q = PAIR ? (int)(wlane & 1) : 0;

    const int64_t colu = UNI ? (int64_t)wg * (kBlock * COLS) : col;  // see forward_scan_chunked
    const uint32_t lane = (uint32_t)(col - colu);
    const int Dp = p.Dp;
    const int ju = (int)(colu % Dp);
    const int j = ju + (int)lane;
    const bool flip = ju >= p.d;

    float wc1[COLS], wc2[COLS], b1[COLS], b2[COLS], m[COLS];
    float cur[COLS];  // d loss / d state
    CompensatedSum sw1[COLS], sw2[COLS], sb1[COLS], sb2[COLS];  // weight_c / bias gradient sums over the walk
#pragma unroll
    for (int c = 0; c < COLS; ++c) {
        wc1[c] = CUSTOM ? 0.f : static_cast<const float *>(p.wc)[j + c];
        wc2[c] = CUSTOM ? 0.f : static_cast<const float *>(p.wc)[Dp + j + c];
        b1[c] = p.bias[j + c];
        b2[c] = p.bias[Dp + j + c];
        m[c] = p.mask_c ? p.mask_c[col + c] : 1.0f;
        cur[c] = p.glast ? p.glast[col + c] : 0.0f;      // no gradient of the last state given: zeros
    }
    const float sx = (SKIP == 1 && p.scale_x) ? *p.scale_x : 1.0f;

    const int64_t L = p.L;
    // forward-walk step s of this column sits at element ef + s * es
    const int64_t ef = (flip ? (L - 1) : 0) * p.ncols + colu;
    const int64_t es = flip ? -p.ncols : p.ncols;
    // per-lane on purpose: with a scalar address the padding bytes would come through the
    // scalar data cache, whose loads cannot be pipelined behind the vector loads
    const int64_t pf = (flip ? (L - 1) : 0) * p.B + col / Dp;
    const int64_t ps = flip ? -p.B : p.B;
    const T *ubase = static_cast<const T *>(p.u);
    const TX *xbase = static_cast<const TX *>(p.x);
    const T *ghbase = static_cast<const T *>(p.gh);
    T *gubase = static_cast<T *>(p.gu);
    TX *gxbase = static_cast<TX *>(p.gx);
    const T *vbase = static_cast<const T *>(p.wc);   // CUSTOM only
    T *gvbase = static_cast<T *>(p.gwc_steps);

    struct Chunk {
        typename SU::G u[TC];
        typename SX::G x[TC];
        typename S1::G gh[TC];
        typename SV::G w[CUSTOM ? TC : 1];
        uint32_t pad[TC];    // padding flags of the chunk's steps
        float cstart[COLS];  // state before the chunk's first step, as loaded
        uint32_t keep;       // all ones, or zero when that state is zero whatever was loaded
    };

    // Where in a chunk's burst of requests the start state goes: first, except in the builds with a
    // padding mask (measured, kernel time: 32 768 float columns of 512 steps 125.6 us with the old
    // placement and early mask, 116.8 us last, 108.1 us first; the same columns with 128 padded steps
    // 33.8 / 31.0 / 33.3 us).
    // (The two-columns-per-lane builds with per-lane row arithmetic have no register to spare for
    // the mask: they apply it at once, as all builds did before, and request the state last.)
    constexpr bool kLateMask = COLS == 1 || UNI;
    constexpr bool kStartFirst = kLateMask && !HAS_PAD;
    auto load_cstart = [&](Chunk &k, int64_t ch) __attribute__((always_inline)) {
        // one load from a selected address (a select between a register and a loaded value made the
        // compiler keep the initial state in scratch memory and select between addresses itself)
        // (without an initial state the first chunk starts from zero; its load reads checkpoint row 0,
        // which always exists, and the value is dropped with a bit mask when the chunk's turn comes:
        // a select makes the compiler branch around the load, inside the pipelined loop, and a mask
        // applied here would touch the value right after its load, which waits for it and, since a
        // wavefront's loads return in issue order, for every load issued before it)
        const uint32_t keep = (ch == 0 && !p.c0) ? 0u : ~0u;
        k.keep = kLateMask ? keep : ~0u;
        // The address is one of two bases. As a select it becomes a scalar branch that cuts the loop
        // body in two, which the one-column-per-lane kernels like (measured 8 % faster at 512
        // wavefronts, level at 2 048) and the two-columns-per-lane kernels do not (6 % slower at
        // 1 024 wavefronts): those blend the bases with bit masks instead.
        const float *from;
        if constexpr (COLS == 2) {
            const uintptr_t use_c0 = (ch == 0 && p.c0) ? ~(uintptr_t)0 : (uintptr_t)0;
            const uintptr_t base = (reinterpret_cast<uintptr_t>(p.c0) & use_c0) |
                                   (reinterpret_cast<uintptr_t>(p.ckpt + (ch > 0 ? ch - 1 : 0) * p.ncols) & ~use_c0);
            from = reinterpret_cast<const float *>(base) + col;
        } else {
            from = (ch == 0 && p.c0) ? p.c0 + col : p.ckpt + (ch > 0 ? ch - 1 : 0) * p.ncols + col;
        }
#pragma unroll
        for (int c = 0; c < COLS; ++c)
            k.cstart[c] = kLateMask ? from[c] : __builtin_bit_cast(float, __builtin_bit_cast(uint32_t, from[c]) & keep);
    };

    // n: number of valid steps in the chunk (TC except for a ragged last chunk)
    auto load_chunk = [&](Chunk &k, int64_t ch, int n) __attribute__((always_inline)) {
        const int64_t s0 = ch * TC;
        if constexpr (kStartFirst) load_cstart(k, ch);
#pragma unroll
        for (int i = 0; i < TC; ++i) {
            if (i < n) {
                const int64_t e = ef + (s0 + i) * es;
                k.u[i] = SU::template load<NTL>(ubase + e * K, lane, q);
                if (SKIP == 1) k.x[i] = SX::template load<NTL>(xbase + e, lane, q);
                k.gh[i] = S1::template load<NTL>(ghbase + e, lane, q);
                if constexpr (CUSTOM) k.w[i] = SV::template load<NTL>(vbase + e * 2, lane, q);
                k.pad[i] = HAS_PAD ? p.pad[pf + (s0 + i) * ps] : 0;
            }
        }
        if constexpr (!kStartFirst) load_cstart(k, ch);
    };

    auto compute_chunk = [&](const Chunk &k, int64_t ch, int n) __attribute__((always_inline)) {
        const int64_t s0 = ch * TC;
        float st[TC + 1][COLS];  // st[i] = state before step i of the chunk
        float g1[TC][COLS], g2[TC][COLS];
        float u0s[TC][COLS], xs[TC][COLS];  // candidate stream and (k = 4) skip stream, decoded once
#pragma unroll
        for (int c = 0; c < COLS; ++c) st[0][c] = __builtin_bit_cast(float, __builtin_bit_cast(uint32_t, k.cstart[c]) & k.keep);
        float gw1[COLS] = {}, gw2[COLS] = {}, gb1[COLS] = {}, gb2[COLS] = {};  // this chunk's share of the sums
#pragma unroll
        for (int i = 0; i < TC; ++i) {
            if (i < n) {
                const bool padded = k.pad[i] != 0;
                float uu[COLS * K];
                SU::unpack(k.u[i], q, uu);
                float ww[COLS * 2] = {};
                if constexpr (CUSTOM) SV::unpack(k.w[i], q, ww);
#pragma unroll
                for (int c = 0; c < COLS; ++c) {
                    const float cp = st[i][c];
                    u0s[i][c] = uu[c * K];
                    if (SKIP == 2) xs[i][c] = uu[c * K + K - 1];
                    g1[i][c] = gate<T>(uu[c * K + 1], CUSTOM ? ww[2 * c] : wc1[c], cp, b1[c]);
                    g2[i][c] = gate<T>(uu[c * K + 2], CUSTOM ? ww[2 * c + 1] : wc2[c], cp, b2[c]);
                    const float cn = (cp - u0s[i][c]) * g1[i][c] + u0s[i][c];
                    st[i + 1][c] = padded ? cp : cn;
                }
            }
        }
#pragma unroll
        for (int i = TC - 1; i >= 0; --i) {
            if (i < n) {
                const bool padded = k.pad[i] != 0;
                float gu[COLS * K], gx[COLS], xx[COLS] = {}, ghs[COLS];
                if (SKIP == 1) SX::unpack(k.x[i], q, xx);
                S1::unpack(k.gh[i], q, ghs);
                float ww[COLS * 2] = {}, gv[COLS * 2];
                if constexpr (CUSTOM) SV::unpack(k.w[i], q, ww);
#pragma unroll
                for (int c = 0; c < COLS; ++c) {
                    const float cp = st[i][c];
                    const float val = TANH ? tanh_fast(st[i + 1][c]) : st[i + 1][c];
                    const float dact = TANH ? (1.0f - val * val) : 1.0f;
                    const float u0 = u0s[i][c];
                    const float G1 = g1[i][c], G2 = g2[i][c];
                    const float xv = (SKIP == 0) ? 0.0f : (SKIP == 1) ? xx[c] * sx : xs[i][c];
                    const float gh = ghs[c];

                    const float gg2 = gh * (val - xv) * m[c] * (G2 * (1.0f - G2));
                    const float gc = TANH ? gh * m[c] * (G2 * dact) + cur[c] : gh * m[c] * G2 + cur[c];
                    const float gg1 = gc * (cp - u0) * (G1 * (1.0f - G1));
                    const float gskip = gh * (1.0f - G2 * m[c]);
                    const float ncur = gc * G1 + gg1 * (CUSTOM ? ww[2 * c] : wc1[c]) + gg2 * (CUSTOM ? ww[2 * c + 1] : wc2[c]);
                    gv[2 * c] = padded ? 0.0f : gg1 * cp;
                    gv[2 * c + 1] = padded ? 0.0f : gg2 * cp;

                    gu[c * K] = padded ? 0.0f : gc * (1.0f - G1);
                    gu[c * K + 1] = padded ? 0.0f : gg1;
                    gu[c * K + 2] = padded ? 0.0f : gg2;
                    if (K == 4) gu[c * K + K - 1] = padded ? 0.0f : gskip;
                    gx[c] = padded ? 0.0f : gskip * sx;
                    gb1[c] += padded ? 0.0f : gg1;
                    gw1[c] += padded ? 0.0f : gg1 * cp;
                    gb2[c] += padded ? 0.0f : gg2;
                    gw2[c] += padded ? 0.0f : gg2 * cp;
                    cur[c] = padded ? cur[c] : ncur;
                }
                const int64_t e = ef + (s0 + i) * es;
                SU::template store<NTS>(gubase + e * K, lane, q, gu);
                if (SKIP == 1) SX::template store<NTS>(gxbase + e, lane, q, gx);
                if constexpr (CUSTOM) SV::template store<NTS>(gvbase + e * 2, lane, q, gv);
            }
        }
#pragma unroll
        for (int c = 0; c < COLS; ++c) {
            sw1[c].add(gw1[c]);
            sw2[c].add(gw2[c]);
            sb1[c].add(gb1[c]);
            sb2[c].add(gb2[c]);
        }
    };

    // steps the window leaves out are known to be padded: no loads, zero gradients
    auto fill = [&](int64_t from, int64_t to) __attribute__((always_inline)) {
        const float zu[COLS * K] = {}, z1[COLS] = {}, zv[COLS * 2] = {};
        for (int64_t s = from; s < to; ++s) {
            const int64_t e = ef + s * es;
            SU::template store<NTS>(gubase + e * K, lane, q, zu);
            if (SKIP == 1) SX::template store<NTS>(gxbase + e, lane, q, z1);
            if constexpr (CUSTOM) SV::template store<NTS>(gvbase + e * 2, lane, q, zv);
        }
    };

    const int64_t nfull = L / TC;
    const int tail = (int)(L - nfull * TC);
    int64_t first = 0, nend = nfull;   // full chunks [first, nend) are walked, last to first
    bool with_tail = tail > 0;         // and, before them, the ragged last chunk
    if constexpr (HAS_PAD && UNI) {
        const LiveWindow w = live_window(p.pad, pf, ps, L);
        first = w.lo / TC;
        const int64_t chunks = (w.hi + TC - 1) / TC;
        nend = chunks < nfull ? chunks : nfull;
        with_tail = with_tail && chunks > nfull;
        fill(with_tail ? L : nend * TC, L);
    }
    Chunk ka, kb;
    int64_t ch = nend - 1;             // next full chunk to compute
    if (ch >= first) load_chunk(ka, ch, TC);
    if (with_tail) {                   // the ragged chunk is the last of the walk: visited first
        load_chunk(kb, nfull, tail);
        compute_chunk(kb, nfull, tail);
    }
    // Two chunks per iteration (ka, kb alternate) so that no register copies are needed and
    // the loop body is a single block in which every prefetch is a real chunk.
    while (ch >= first + 2) {
        load_chunk(kb, ch - 1, TC);
        compute_chunk(ka, ch, TC);
        __builtin_amdgcn_sched_barrier(0);
        load_chunk(ka, ch - 2, TC);
        compute_chunk(kb, ch - 1, TC);
        __builtin_amdgcn_sched_barrier(0);
        ch -= 2;
    }
    if (ch == first + 1) {
        load_chunk(kb, first, TC);
        compute_chunk(ka, first + 1, TC);
        compute_chunk(kb, first, TC);
    } else if (ch == first) {
        compute_chunk(ka, first, TC);
    }
    if constexpr (HAS_PAD && UNI) fill(0, first * TC);

#pragma unroll
    for (int c = 0; c < COLS; ++c) {
        p.ginit[col + c] = cur[c];
        p.partial[col + c] = sw1[c].value();
        p.partial[p.ncols + col + c] = sw2[c].value();
        p.partial[2 * p.ncols + col + c] = sb1[c].value();
        p.partial[3 * p.ncols + col + c] = sb2[c].value();
    }
}

}  // namespace sru_amd
