// Kernel selection for one stream element type T. Included by scan_<type>_fwd.hip, scan_<type>_bwd.hip and
// scan_f64.hip only.
//
// Fast kernels exist for the three layouts the SRU layer produces without a per-step
// weight_c: (k=3, skip from x), (k=3, no skip term) and (k=4, skip from U[..., 3]); whether a
// padding mask is given, whether and how c is stored and the activation are compiled in.
// Everything else (per-step weight_c; k=4 without a skip term, which the layer never
// produces) runs the general kernels, one column per lane. Double streams run the general
// kernels for everything, computing in double.
//
// Every launcher returns the status of its own hipLaunchKernel call; nothing here reads or
// clears the runtime's sticky error state, which may hold an error of the embedding program.
#pragma once

#include <algorithm>

#include "sru_launch.h"
#include "sru_split.h"

namespace sru_amd {

// Columns per lane of the fast kernels, per element type: float streams move as dwordx3 /
// dwordx4 per column already; 16-bit streams need two columns per lane (or paired lanes)
// for dword-granular accesses.
template <typename T> struct Tune { static constexpr int kCols = sizeof(T) == 2 ? 2 : 1; };
constexpr int kRingDepth = 8;  // ring kernels (reference-style state, general modes)
// (double streams: a slot is twice as wide, so half the slots keep the ring in registers)
template <typename T> constexpr int general_ring_depth() { return sizeof(T) == 8 ? kRingDepth / 2 : kRingDepth; }
// Every large stream is touched exactly once per kernel, so loads and stores are marked
// non-temporal: measured at the headline shape with cache-cold operands, forward + backward
// 447 us -> 425 us (float), 230 us -> 214 us (bfloat16).
constexpr int kNt = kNtLoad | kNtStore;
// 16-bit streams with few columns: below this many lanes at two columns per lane (fewer than
// 1024 wavefronts) the kernels keep one column per lane and pair lanes for memory access.
#ifndef SRU_AMD_PAIR_BELOW   // (set by tuning builds only)
#define SRU_AMD_PAIR_BELOW 65536
#endif
constexpr int64_t kPairBelow = SRU_AMD_PAIR_BELOW;

// Lane-pair kernels (sru_split.h): 16-bit streams, d a multiple of 32, at most 1024 wavefronts of 32
// columns, every stream 16-byte aligned, state kept as checkpoints or not at all.
#ifndef SRU_AMD_SPLIT_NBUF   // (set by tuning builds only)
#define SRU_AMD_SPLIT_NBUF 2
#endif
constexpr int kSplitNbuf = SRU_AMD_SPLIT_NBUF;   // chunks (of 16 steps) in flight per wavefront
#ifndef SRU_AMD_SPLIT_MAX_WAVES   // (set by tuning builds only)
#define SRU_AMD_SPLIT_MAX_WAVES 1024
#endif
inline bool split_wanted(int64_t ncols, int32_t d) { return d % kSplitCols == 0 && ncols / kSplitCols <= SRU_AMD_SPLIT_MAX_WAVES; }

inline bool aligned_to(const void *p, size_t a) { return (reinterpret_cast<uintptr_t>(p) % a) == 0; }

// launch of a lane-pair kernel: wavefronts of 32 columns, kSplitWaves per workgroup
template <typename P>
inline hipError_t launch_split(void (*kernel)(P), hipStream_t st, const P &p) {
    void *args[] = {const_cast<P *>(&p)};
    const int64_t wavefronts = p.ncols / kSplitCols;
    return hipLaunchKernel(reinterpret_cast<const void *>(kernel), dim3((unsigned)((wavefronts + kSplitWaves - 1) / kSplitWaves)),
                           dim3(kBlock * kSplitWaves), args, 0, st);
}

// Wavefronts per workgroup for the chunked kernels: 8 or 4 (as the kernel allows) while the launch
// still has a workgroup for each of the 256 compute units, else 1. (Not 2: workgroups of two
// wavefronts measured up to 25 % slower than either neighbour.)
inline int waves_per_group(int64_t wavefronts, int most) {
    for (int n = most; n >= 4; n /= 2)
        if (wavefronts / n >= 256) return n;
    return 1;
}
// launch of a chunked kernel: `most` wavefronts per workgroup at most
template <typename P>
inline hipError_t launch_grouped(void (*kernel)(P), int64_t ncols, int cols, int most, hipStream_t st, const P &p) {
    const int64_t wavefronts = (ncols / cols + kBlock - 1) / kBlock;
    const int n = waves_per_group(wavefronts, most);
    void *args[] = {const_cast<P *>(&p)};
    return hipLaunchKernel(reinterpret_cast<const void *>(kernel), dim3((unsigned)((wavefronts + n - 1) / n)), dim3(kBlock * n),
                           args, 0, st);
}

// Two columns per lane need an even d (a pair must not straddle a direction or a batch
// row) and stream pointers aligned to the pair groups.
template <typename T, int K>
bool pair_ok(const sru_amd_shape &s, std::initializer_list<const void *> wide,
             std::initializer_list<const void *> narrow) {
    if (Tune<T>::kCols != 2 || (s.hidden % 2) != 0) return false;
    const size_t es = sizeof(T);
    for (const void *q : wide)
        if (q && !aligned_to(q, group_align((int)(2 * K * es)))) return false;
    for (const void *q : narrow)
        if (q && !aligned_to(q, group_align((int)(2 * es)))) return false;
    return true;
}

// true when every wavefront lies inside one direction and one batch row
inline bool wave_uniform(int32_t d, int cols) { return d % (kBlock * cols) == 0; }

// X: the template bits fixed so far (pairing, then uniformity, then activation); the run-time
// properties are turned into template bits one at a time.
// TX: element type of x / grad_x (T, or float next to 16-bit streams: those builds exist for the
// identity activation, checkpointed or no state, no per-step weight_c; callers start them at STAGE 1).
template <typename T, int K, int SKIP, int COLS, int X = 0, int STAGE = 0, typename TX = T>
hipError_t fast_forward(const FwdParams &p, hipStream_t st) {
    if constexpr (STAGE == 0 && (X & kCustom) != 0) {   // (a per-step weight_c with tanh runs the general kernels)
        return fast_forward<T, K, SKIP, COLS, X, 1, TX>(p, st);
    } else if constexpr (STAGE == 0) {
        return p.act ? fast_forward<T, K, SKIP, COLS, X | kTanh, 1, TX>(p, st) : fast_forward<T, K, SKIP, COLS, X, 1, TX>(p, st);
    } else if constexpr (STAGE == 1) {
        return wave_uniform(p.d, COLS) ? fast_forward<T, K, SKIP, COLS, X | kUniform, 2, TX>(p, st)
                                       : fast_forward<T, K, SKIP, COLS, X, 2, TX>(p, st);
    } else if constexpr (STAGE == 2) {
        return p.pad ? fast_forward<T, K, SKIP, COLS, X | kHasPad, 3, TX>(p, st) : fast_forward<T, K, SKIP, COLS, X, 3, TX>(p, st);
    } else {
        constexpr int TC = kCkptInterval;
        const int most = max_waves_per_group<T>(X);
        // what is kept for the backward pass: checkpoints, the state after every step, or nothing
        if (p.ckpt) return launch_grouped(forward_scan_chunked<T, K, SKIP, X | kNt | kCkpt, COLS, TC, TX>, p.ncols, COLS, most, st, p);
        // (with a per-step weight_c the state after every step is the general kernels'; with a float x
        // next to 16-bit streams it is refused before)
        if constexpr ((X & kCustom) == 0 && sizeof(TX) == sizeof(T)) {
            if (p.c) return launch_grouped(forward_scan_chunked<T, K, SKIP, X | kNt | kKeepC, COLS, TC>, p.ncols, COLS, most, st, p);
        }
        return launch_grouped(forward_scan_chunked<T, K, SKIP, X | kNt, COLS, TC, TX>, p.ncols, COLS, most, st, p);
    }
}

template <typename T, int K, int SKIP, int COLS, int X = 0, int STAGE = 0, typename TX = T>
hipError_t fast_backward(const BwdParams &p, hipStream_t st) {
    if constexpr (STAGE == 0 && (X & kCustom) != 0) {
        return fast_backward<T, K, SKIP, COLS, X, 1, TX>(p, st);
    } else if constexpr (STAGE == 0) {
        return p.act ? fast_backward<T, K, SKIP, COLS, X | kTanh, 1, TX>(p, st) : fast_backward<T, K, SKIP, COLS, X, 1, TX>(p, st);
    } else if constexpr (STAGE == 1) {
        return p.pad ? fast_backward<T, K, SKIP, COLS, X | kHasPad, 2, TX>(p, st) : fast_backward<T, K, SKIP, COLS, X, 2, TX>(p, st);
    } else {
        if constexpr ((X & (kPair | kCustom)) == 0 && sizeof(TX) == sizeof(T)) {   // (lane pairing, the weight_c stream and a float x exist in the chunked kernels only)
            // reference-style state: the ring kernel reads it step by step
            if (!p.ckpt) return launch_grouped(backward_scan<T, K, SKIP, X | kNt, COLS, kRingDepth>, p.ncols, COLS, 4, st, p);
        }
        constexpr int TC = kCkptInterval;
        const int most = max_waves_per_group<T>(X);
        if (wave_uniform(p.d, COLS))
            return launch_grouped(backward_scan_ckpt<T, K, SKIP, X | kNt | kUniform, COLS, TC, TX>, p.ncols, COLS, most, st, p);
        return launch_grouped(backward_scan_ckpt<T, K, SKIP, X | kNt, COLS, TC, TX>, p.ncols, COLS, most, st, p);
    }
}

template <typename T, int K, int SKIP, int X = 0, int STAGE = 0>
hipError_t split_forward(const FwdParams &p, hipStream_t st) {
    if constexpr (STAGE == 0) {
        return p.act ? split_forward<T, K, SKIP, X | kTanh, 1>(p, st) : split_forward<T, K, SKIP, X, 1>(p, st);
    } else if constexpr (STAGE == 1) {
        return p.pad ? split_forward<T, K, SKIP, X | kHasPad, 2>(p, st) : split_forward<T, K, SKIP, X, 2>(p, st);
    } else {
        if (p.ckpt) return launch_split(forward_scan_split<T, K, SKIP, X | kNt | kCkpt, kSplitNbuf>, st, p);
        return launch_split(forward_scan_split<T, K, SKIP, X | kNt, kSplitNbuf>, st, p);
    }
}

template <typename T, int K, int SKIP, int X = 0, int STAGE = 0>
hipError_t split_backward(const BwdParams &p, hipStream_t st) {
    if constexpr (STAGE == 0) {
        return p.act ? split_backward<T, K, SKIP, X | kTanh, 1>(p, st) : split_backward<T, K, SKIP, X, 1>(p, st);
    } else {
        if (p.pad) return launch_split(backward_scan_split<T, K, SKIP, X | kNt | kHasPad, kSplitNbuf>, st, p);
        return launch_split(backward_scan_split<T, K, SKIP, X | kNt, kSplitNbuf>, st, p);
    }
}

inline bool all_aligned_16(std::initializer_list<const void *> ptrs) {
    for (const void *q : ptrs)
        if (q && !aligned_to(q, 16)) return false;
    return true;
}

template <typename T, int K, int SKIP>
hipError_t general_forward(const FwdParams &p, hipStream_t st) {
    return launch_grouped(forward_scan<T, K, SKIP, kGeneral | kNt, 1, general_ring_depth<T>()>, p.ncols, 1, 4, st, p);
}
template <typename T, int K, int SKIP>
hipError_t general_backward(const BwdParams &p, hipStream_t st) {
    return launch_grouped(backward_scan<T, K, SKIP, kGeneral | kNt, 1, general_ring_depth<T>()>, p.ncols, 1, 4, st, p);
}

// 16-bit streams whose columns cannot be paired (odd d, or a stream pointer that is not aligned to a
// pair's group) run the general kernels, one column per lane with 2-byte accesses; the host side
// refuses checkpointed state for them.
template <typename T, int K, int SKIP>
hipError_t pick_forward(const sru_amd_shape &s, const FwdParams &p, hipStream_t st) {
    if constexpr (sizeof(T) == 2) {
        if constexpr (SKIP == 1) {
            if (p.x_float) {   // a float x next to 16-bit streams: chunked kernels only (the flag combinations were checked before)
                if (p.act || p.c || !pair_ok<T, K>(s, {p.u}, {p.h}) || !aligned_to(p.x, 4)) return hipErrorInvalidValue;
                if (p.ncols / 2 < kPairBelow) return fast_forward<T, K, SKIP, 1, kPair, 1, float>(p, st);
                return fast_forward<T, K, SKIP, 2, 0, 1, float>(p, st);
            }
        }
        if (!p.c && split_wanted(p.ncols, p.d) && all_aligned_16({p.u, p.x, p.h}))
            return split_forward<T, K, SKIP>(p, st);
        if (!pair_ok<T, K>(s, {p.u}, {p.x, p.h, p.c}))
            return p.ckpt ? hipErrorInvalidValue : general_forward<T, K, SKIP>(p, st);
        if (p.ncols / 2 < kPairBelow) return fast_forward<T, K, SKIP, 1, kPair>(p, st);
        return fast_forward<T, K, SKIP, 2>(p, st);
    } else {
        return fast_forward<T, K, SKIP, 1>(p, st);
    }
}

template <typename T, int K, int SKIP>
hipError_t pick_backward(const sru_amd_shape &s, const BwdParams &p, hipStream_t st) {
    if constexpr (sizeof(T) == 2) {
        if constexpr (SKIP == 1) {
            if (p.x_float) {
                if (p.act || !p.ckpt || !pair_ok<T, K>(s, {p.u, p.gu}, {p.gh}) || !aligned_to(p.x, 4) || !aligned_to(p.gx, 4))
                    return hipErrorInvalidValue;
                if (p.ncols / 2 < kPairBelow) return fast_backward<T, K, SKIP, 1, kPair, 1, float>(p, st);
                return fast_backward<T, K, SKIP, 2, 0, 1, float>(p, st);
            }
        }
        if (p.ckpt && split_wanted(p.ncols, p.d) && all_aligned_16({p.u, p.x, p.gh, p.gu, p.gx}))
            return split_backward<T, K, SKIP>(p, st);
        if (!pair_ok<T, K>(s, {p.u, p.gu}, {p.x, p.c, p.gh, p.gx}))   // p.c is null with checkpoints
            return p.ckpt ? hipErrorInvalidValue : general_backward<T, K, SKIP>(p, st);
        if (p.ckpt && p.ncols / 2 < kPairBelow) return fast_backward<T, K, SKIP, 1, kPair>(p, st);
        return fast_backward<T, K, SKIP, 2>(p, st);
    } else {
        return fast_backward<T, K, SKIP, 1>(p, st);
    }
}

// (k, skip_type) pairs that pass the shape check: (3,0) (3,1) (4,0) (4,2).
// A per-step weight_c runs the chunked kernels (with the weight_c stream compiled in) when the
// activation is the identity, the state is kept as checkpoints or not at all, and, for 16-bit
// streams, columns can be paired; everything else about it is the general kernels' business.
template <typename T, int K>
bool custom_chunked_ok(const sru_amd_shape &s, bool full_state, std::initializer_list<const void *> wide,
                       std::initializer_list<const void *> mid, std::initializer_list<const void *> narrow) {
    if (!s.is_custom || s.activation_type != 0 || full_state || (s.skip_type == 0 && s.k == 4)) return false;
    if (sizeof(T) == 4) return true;
    for (const void *q : mid)
        if (q && !aligned_to(q, 8)) return false;
    return pair_ok<T, K>(s, wide, narrow);
}

template <typename T, int K, int SKIP>
hipError_t custom_forward(const FwdParams &p, hipStream_t st) {
    return fast_forward<T, K, SKIP, Tune<T>::kCols, kCustom>(p, st);
}
template <typename T, int K, int SKIP>
hipError_t custom_backward(const BwdParams &p, hipStream_t st) {
    return fast_backward<T, K, SKIP, Tune<T>::kCols, kCustom>(p, st);
}

template <typename T>
hipError_t launch_forward(const sru_amd_shape &s, const FwdParams &p, hipStream_t st) {
    if constexpr (sizeof(T) != 8) {
        if (s.k == 3 ? custom_chunked_ok<T, 3>(s, p.c != nullptr, {p.u}, {p.wc}, {p.x, p.h})
                     : custom_chunked_ok<T, 4>(s, p.c != nullptr, {p.u}, {p.wc}, {p.x, p.h})) {
            if (s.k == 4) return custom_forward<T, 4, 2>(p, st);
            if (s.skip_type == 1) return custom_forward<T, 3, 1>(p, st);
            return custom_forward<T, 3, 0>(p, st);
        }
        const bool general = s.is_custom != 0 || (s.skip_type == 0 && s.k == 4);
        if (!general) {
            if (s.k == 4) return pick_forward<T, 4, 2>(s, p, st);
            if (s.skip_type == 1) return pick_forward<T, 3, 1>(s, p, st);
            return pick_forward<T, 3, 0>(s, p, st);
        }
    }
    if (s.k == 3 && s.skip_type == 1) return general_forward<T, 3, 1>(p, st);
    if (s.k == 3) return general_forward<T, 3, 0>(p, st);
    if (s.skip_type == 2) return general_forward<T, 4, 2>(p, st);
    return general_forward<T, 4, 0>(p, st);
}

template <typename T>
hipError_t launch_backward(const sru_amd_shape &s, const BwdParams &p, hipStream_t st) {
    if constexpr (sizeof(T) != 8) {
        if (s.k == 3 ? custom_chunked_ok<T, 3>(s, p.ckpt == nullptr, {p.u, p.gu}, {p.wc, p.gwc_steps}, {p.x, p.gh, p.gx})
                     : custom_chunked_ok<T, 4>(s, p.ckpt == nullptr, {p.u, p.gu}, {p.wc, p.gwc_steps}, {p.x, p.gh, p.gx})) {
            if (s.k == 4) return custom_backward<T, 4, 2>(p, st);
            if (s.skip_type == 1) return custom_backward<T, 3, 1>(p, st);
            return custom_backward<T, 3, 0>(p, st);
        }
        const bool general = s.is_custom != 0 || (s.skip_type == 0 && s.k == 4);
        if (!general) {
            if (s.k == 4) return pick_backward<T, 4, 2>(s, p, st);
            if (s.skip_type == 1) return pick_backward<T, 3, 1>(s, p, st);
            return pick_backward<T, 3, 0>(s, p, st);
        }
    }
    if (p.ckpt) return hipErrorInvalidValue;   // the general kernels read the state after every step (refused by the shape and alignment checks before)
    if (s.k == 3 && s.skip_type == 1) return general_backward<T, 3, 1>(p, st);
    if (s.k == 3) return general_backward<T, 3, 0>(p, st);
    if (s.skip_type == 2) return general_backward<T, 4, 2>(p, st);
    return general_backward<T, 4, 0>(p, st);
}

}  // namespace sru_amd
