// Device-side building blocks of the SRU recurrence kernels for gfx950.
//
// Mapping: one lane owns one column (batch b, direction, hidden j), col = b*D' + dir*d + j,
// exactly the column order of the (L, B, D') tensors, so a 64-lane wavefront reads
// 64*k consecutive elements of U per step and 64 consecutive elements of every other
// stream. The time loop is strictly serial per column (the gates see the previous state),
// so memory latency is hidden by depth, not by width: every lane keeps a ring of P
// future steps in registers; each iteration consumes the oldest slot and refills it
// with the step P ahead, so about P steps of loads are in flight per lane at all times.
//
// Columns of the second direction walk time backwards. The loop variable is the walk
// step s (uniform over the wavefront); the time index is s or L-1-s per lane.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace sru_amd {

constexpr int kBlock = 64;  // one wavefront per workgroup: finest dispatch granularity

struct half_bits { uint16_t v; };  // IEEE binary16 storage
struct bf16_bits { uint16_t v; };  // bfloat16 storage

// ---------------------------------------------------------------- element conversion
__device__ __forceinline__ float to_float(float v) { return v; }
__device__ __forceinline__ float to_float(half_bits v) {
    return (float)__builtin_bit_cast(_Float16, v.v);
}
__device__ __forceinline__ float to_float(bf16_bits v) {
    return __builtin_bit_cast(float, (uint32_t)v.v << 16);
}

template <typename T> __device__ __forceinline__ T from_float(float v);
template <> __device__ __forceinline__ float from_float<float>(float v) { return v; }
template <> __device__ __forceinline__ half_bits from_float<half_bits>(float v) {
    return half_bits{__builtin_bit_cast(uint16_t, (_Float16)v)};  // round to nearest even
}
template <> __device__ __forceinline__ bf16_bits from_float<bf16_bits>(float v) {
    uint32_t u = __builtin_bit_cast(uint32_t, v);
    if ((u & 0x7fffffffu) > 0x7f800000u) return bf16_bits{(uint16_t)((u >> 16) | 0x40u)};  // NaN
    u += 0x7fffu + ((u >> 16) & 1u);  // round to nearest even
    return bf16_bits{(uint16_t)(u >> 16)};
}

// ---------------------------------------------------------------- packed groups of N elements
// N consecutive elements moved by one instruction where the type allows it:
// float x3 -> dwordx3, float x4 -> dwordx4, 16-bit x2 -> dword, 16-bit x4 -> dwordx2.
template <typename T, int N> struct Pack;
template <> struct alignas(4) Pack<float, 2> { float e[2]; };
template <> struct alignas(4) Pack<float, 3> { float e[3]; };
template <> struct alignas(16) Pack<float, 4> { float e[4]; };
template <> struct alignas(4) Pack<half_bits, 2> { half_bits e[2]; };
template <> struct alignas(2) Pack<half_bits, 3> { half_bits e[3]; };
template <> struct alignas(8) Pack<half_bits, 4> { half_bits e[4]; };
template <> struct alignas(4) Pack<bf16_bits, 2> { bf16_bits e[2]; };
template <> struct alignas(2) Pack<bf16_bits, 3> { bf16_bits e[3]; };
template <> struct alignas(8) Pack<bf16_bits, 4> { bf16_bits e[4]; };

template <typename T, int N>
__device__ __forceinline__ void load_group(const T *p, float (&out)[N]) {
    const Pack<T, N> v = *reinterpret_cast<const Pack<T, N> *>(p);
#pragma unroll
    for (int i = 0; i < N; ++i) out[i] = to_float(v.e[i]);
}

template <typename T, int N>
__device__ __forceinline__ void store_group(T *p, const float (&in)[N]) {
    Pack<T, N> v;
#pragma unroll
    for (int i = 0; i < N; ++i) v.e[i] = from_float<T>(in[i]);
    *reinterpret_cast<Pack<T, N> *>(p) = v;
}

// ---------------------------------------------------------------- gate arithmetic
// sigmoid through the hardware exp2 and reciprocal (1 ulp each): absolute error of the
// result stays below 2e-7 over the whole real line; saturates cleanly to 0 and 1.
__device__ __forceinline__ float sigmoid(float v) {
    return __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.4426950408889634f * v));
}

// ---------------------------------------------------------------- kernel parameters
struct FwdParams {
    const void *u, *x, *wc;
    const float *bias, *c0, *mask_c;
    const uint8_t *pad;
    const float *scale_x;
    void *h, *c;
    float *c_last;
    int64_t L, B, ncols;  // ncols = B * D'
    int32_t d, Dp;        // hidden per direction, D' = dirs * d
    int32_t act, custom;  // only read by the general kernels
};

struct BwdParams {
    const void *u, *x, *wc;
    const float *bias, *c0, *mask_c;
    const uint8_t *pad;
    const float *scale_x;
    const void *c, *gh;
    const float *glast;
    void *gu, *gx, *gwc_steps;  // gwc_steps: per-step weight_c gradient (custom only)
    float *ginit;
    float *partial;  // (4, ncols): per-column sums gwc1, gwc2, gbias1, gbias2
    int64_t L, B, ncols;
    int32_t d, Dp;
    int32_t act, custom;
};

// ================================================================= forward scan
// T: stream element type. K: streams per column in U. SKIP: 0 none, 1 from x, 2 from
// U[..., 3]. MODE: see below. P: ring depth.
//
// The loop body must stay one straight line of code for the compiler to count the
// outstanding loads exactly (a uniform branch inside it makes the inserted waits drain
// the whole ring once per round). The fast kernels therefore take "is there a padding
// mask" and "is the per-step state kept" as template bits; the general kernels read
// those and the rarely used tanh / per-step weight_c options from the parameters.
constexpr int kGeneral = 4;  // MODE bit: run-time pad / keep_c / act / custom
constexpr int kHasPad = 1;   // MODE bit (fast kernels): mask_pad given
constexpr int kKeepC = 2;    // MODE bit (fast forward kernels): c is stored

template <typename T, int K, int SKIP, int MODE, int P>
__global__ void __launch_bounds__(kBlock) forward_scan(const FwdParams p) {
    constexpr bool GENERAL = (MODE & kGeneral) != 0;
    const int64_t col = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (col >= p.ncols) return;

    const int Dp = p.Dp;
    const int j = (int)(col % Dp);
    const int64_t b = col / Dp;
    const bool flip = j >= p.d;  // second direction; never true when dirs == 1 (d == D')
    const bool custom = GENERAL && p.custom;
    const bool use_tanh = GENERAL && p.act;

    float wc1 = 0.f, wc2 = 0.f;
    if (!custom) {
        wc1 = static_cast<const float *>(p.wc)[j];
        wc2 = static_cast<const float *>(p.wc)[Dp + j];
    }
    const float b1 = p.bias[j], b2 = p.bias[Dp + j];
    const float m = p.mask_c ? p.mask_c[col] : 1.0f;
    const float sx = (SKIP == 1 && p.scale_x) ? *p.scale_x : 1.0f;
    float cur = p.c0[col];

    const int64_t L = p.L;
    const int64_t e0 = (flip ? (L - 1) : 0) * p.ncols + col;  // element of the first walk step
    const int64_t es = flip ? -p.ncols : p.ncols;             // elements per walk step
    const T *up = static_cast<const T *>(p.u) + e0 * K;
    const T *xp = (SKIP == 1) ? static_cast<const T *>(p.x) + e0 : nullptr;
    const T *vp = custom ? static_cast<const T *>(p.wc) + e0 * 2 : nullptr;
    const bool has_pad = GENERAL ? (p.pad != nullptr) : ((MODE & kHasPad) != 0);
    const bool keep_c = GENERAL ? (p.c != nullptr) : ((MODE & kKeepC) != 0);
    const uint8_t *pp = has_pad ? p.pad + (flip ? (L - 1) : 0) * p.B + b : nullptr;
    const int64_t ps = flip ? -p.B : p.B;
    T *hp = static_cast<T *>(p.h) + e0;
    T *cp = keep_c ? static_cast<T *>(p.c) + e0 : nullptr;

    struct Slot {
        float u[K];
        float x;
        float w[2];
        uint32_t pad;
    };
    Slot ring[P];

    auto fetch = [&](Slot &s) {
        load_group<T, K>(up, s.u);
        up += es * K;
        if (SKIP == 1) {
            s.x = to_float(*xp);
            xp += es;
        }
        if (custom) {
            load_group<T, 2>(vp, s.w);
            vp += es * 2;
        }
        s.pad = 0;
        if (has_pad) {
            s.pad = *pp;
            pp += ps;
        }
    };

    auto consume = [&](const Slot &s) {
        const float w1 = custom ? s.w[0] : wc1;
        const float w2 = custom ? s.w[1] : wc2;
        const float g1 = sigmoid(s.u[1] + w1 * cur + b1);
        const float g2 = sigmoid(s.u[2] + w2 * cur + b2);
        const float cn = (cur - s.u[0]) * g1 + s.u[0];
        const float val = use_tanh ? tanhf(cn) : cn;
        float hv;
        if (SKIP != 0) {
            const float xv = (SKIP == 1) ? s.x * sx : s.u[K - 1];
            hv = (val - xv) * m * g2 + xv;
        } else {
            hv = val * m * g2;
        }
        const bool padded = s.pad != 0;
        cur = padded ? cur : cn;  // a padded step keeps the state ...
        *hp = from_float<T>(padded ? 0.0f : hv);  // ... and emits zero
        hp += es;
        if (keep_c) {
            *cp = from_float<T>(cur);
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
    p.c_last[col] = cur;
}

// ================================================================= backward scan
// Walks each column's steps in reverse order, carrying d(loss)/d(state). The gates are
// recomputed from U and the stored previous state. Sums of the weight_c and bias
// gradients over time stay in four registers per lane and leave the kernel as
// per-column partials; reduce_partials() then adds them over the batch in a fixed order.
template <typename T, int K, int SKIP, int MODE, int P>
__global__ void __launch_bounds__(kBlock) backward_scan(const BwdParams p) {
    constexpr bool GENERAL = (MODE & kGeneral) != 0;
    const int64_t col = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (col >= p.ncols) return;

    const int Dp = p.Dp;
    const int j = (int)(col % Dp);
    const int64_t b = col / Dp;
    const bool flip = j >= p.d;
    const bool custom = GENERAL && p.custom;
    const bool use_tanh = GENERAL && p.act;

    float wc1 = 0.f, wc2 = 0.f;
    if (!custom) {
        wc1 = static_cast<const float *>(p.wc)[j];
        wc2 = static_cast<const float *>(p.wc)[Dp + j];
    }
    const float b1 = p.bias[j], b2 = p.bias[Dp + j];
    const float m = p.mask_c ? p.mask_c[col] : 1.0f;
    const float sx = (SKIP == 1 && p.scale_x) ? *p.scale_x : 1.0f;
    const float c_init = p.c0[col];

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
    const bool has_pad = GENERAL ? (p.pad != nullptr) : ((MODE & kHasPad) != 0);
    const uint8_t *pp = has_pad ? p.pad + t_start * p.B + b : nullptr;
    const int64_t ps = flip ? p.B : -p.B;
    T *gup = static_cast<T *>(p.gu) + e0 * K;
    T *gxp = (SKIP == 1) ? static_cast<T *>(p.gx) + e0 : nullptr;
    T *gvp = custom ? static_cast<T *>(p.gwc_steps) + e0 * 2 : nullptr;

    float cur = p.glast[col];                                       // d loss / d state
    float cv = to_float(static_cast<const T *>(p.c)[e0]);           // state after the step
    float gw1 = 0.f, gw2 = 0.f, gb1 = 0.f, gb2 = 0.f;

    struct Slot {
        float u[K];
        float x;
        float w[2];
        float gh;
        float cprev;
        uint32_t pad;
    };
    Slot ring[P];

    // `last` = this is the column's first forward step: its previous state is c_init.
    auto fetch = [&](Slot &s, bool last) {
        load_group<T, K>(up, s.u);
        up += es * K;
        if (SKIP == 1) {
            s.x = to_float(*xp);
            xp += es;
        }
        if (custom) {
            load_group<T, 2>(vp, s.w);
            vp += es * 2;
        }
        s.gh = to_float(*ghp);
        ghp += es;
        s.cprev = c_init;
        if (!last) s.cprev = to_float(*cpp);
        cpp += es;
        s.pad = 0;
        if (has_pad) {
            s.pad = *pp;
            pp += ps;
        }
    };

    auto consume = [&](const Slot &s) {
        const float w1 = custom ? s.w[0] : wc1;
        const float w2 = custom ? s.w[1] : wc2;
        const float cp = s.cprev;
        const float u0 = s.u[0];
        const float g1 = sigmoid(s.u[1] + w1 * cp + b1);
        const float g2 = sigmoid(s.u[2] + w2 * cp + b2);
        const float val = use_tanh ? tanhf(cv) : cv;
        const float dact = use_tanh ? (1.0f - val * val) : 1.0f;
        const float xv = (SKIP == 0) ? 0.0f : (SKIP == 1) ? s.x * sx : s.u[K - 1];
        const float gh = s.gh;
        const bool padded = s.pad != 0;

        const float gg2 = gh * (val - xv) * m * (g2 * (1.0f - g2));
        const float gc = gh * m * (g2 * dact) + cur;
        const float gg1 = gc * (cp - u0) * (g1 * (1.0f - g1));
        const float gskip = gh * (1.0f - g2 * m);
        const float ncur = gc * g1 + gg1 * w1 + gg2 * w2;

        float gu[K];
        gu[0] = padded ? 0.0f : gc * (1.0f - g1);
        gu[1] = padded ? 0.0f : gg1;
        gu[2] = padded ? 0.0f : gg2;
        if (K == 4) gu[K - 1] = (padded || SKIP != 2) ? 0.0f : gskip;
        store_group<T, K>(gup, gu);
        gup += es * K;
        if (SKIP == 1) {
            *gxp = from_float<T>(padded ? 0.0f : gskip * sx);
            gxp += es;
        }
        if (custom) {
            const float gv[2] = {padded ? 0.0f : gg1 * cp, padded ? 0.0f : gg2 * cp};
            store_group<T, 2>(gvp, gv);
            gvp += es * 2;
        }
        gb1 += padded ? 0.0f : gg1;
        gw1 += padded ? 0.0f : gg1 * cp;
        gb2 += padded ? 0.0f : gg2;
        gw2 += padded ? 0.0f : gg2 * cp;
        cur = padded ? cur : ncur;
        cv = cp;  // the state before this step is the state after the next one visited
    };

#pragma unroll
    for (int i = 0; i < P; ++i)
        if (i < L) fetch(ring[i], i == L - 1);

    int64_t s0 = 0;
    for (; s0 + 2 * P <= L; s0 += P) {
#pragma unroll
        for (int i = 0; i < P; ++i) {
            consume(ring[i]);
            fetch(ring[i], s0 + i + P == L - 1);
            __builtin_amdgcn_sched_barrier(0);  // see forward_scan
        }
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
    }

    p.ginit[col] = cur;
    p.partial[col] = gw1;
    p.partial[p.ncols + col] = gw2;
    p.partial[2 * p.ncols + col] = gb1;
    p.partial[3 * p.ncols + col] = gb2;
}

// ================================================================= batch reduction
// partial (4, B, D') -> grad_wc (2, D'), grad_bias (2, D'). One workgroup per 64 hidden
// indices and per quantity; its 16 wavefronts take every 16th batch row each (loads of
// a wavefront are 256 contiguous bytes), accumulate in double and are combined through
// LDS in a fixed order, so the result does not depend on scheduling.
constexpr int kReduceSlices = 16;

__global__ void __launch_bounds__(64 * kReduceSlices)
reduce_partials(const float *partial, float *grad_wc, float *grad_bias, int64_t B, int32_t Dp) {
    __shared__ double acc[kReduceSlices][64];
    const int lane = threadIdx.x & 63;
    const int slice = threadIdx.x >> 6;
    const int j = blockIdx.x * 64 + lane;
    const int q = blockIdx.y;  // 0 gwc1, 1 gwc2, 2 gbias1, 3 gbias2
    double sum = 0.0;
    if (j < Dp) {
        const float *src = partial + ((int64_t)q * B) * Dp + j;
        int64_t b = slice;
        for (; b + 3 * kReduceSlices < B; b += 4 * kReduceSlices) {  // 4 loads in flight
            const float v0 = src[b * Dp], v1 = src[(b + kReduceSlices) * Dp];
            const float v2 = src[(b + 2 * kReduceSlices) * Dp], v3 = src[(b + 3 * kReduceSlices) * Dp];
            sum += (double)v0;
            sum += (double)v1;
            sum += (double)v2;
            sum += (double)v3;
        }
        for (; b < B; b += kReduceSlices) sum += (double)src[b * Dp];
    }
    acc[slice][lane] = sum;
    __syncthreads();
    if (slice == 0 && j < Dp) {
        double total = acc[0][lane];
#pragma unroll
        for (int s = 1; s < kReduceSlices; ++s) total += acc[s][lane];
        float *dst = (q < 2) ? grad_wc : grad_bias;
        if (dst) dst[(q & 1) * Dp + j] = (float)total;
    }
}

}  // namespace sru_amd
