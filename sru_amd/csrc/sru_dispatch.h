// Kernel selection for one stream element type T. Included by scan_<type>_fwd.hip and scan_<type>_bwd.hip only.
//
// Fast kernels exist for the three layouts the SRU layer produces without a per-step
// weight_c: (k=3, skip from x), (k=3, no skip term) and (k=4, skip from U[..., 3]); whether a
// padding mask is given, whether and how c is stored and the activation are compiled in.
// Everything else (per-step weight_c; k=4 without a skip term, which the layer never
// produces) runs the general kernels, one column per lane.
#pragma once

#include "sru_launch.h"

namespace sru_amd {

// Columns per lane and ring depths of the fast kernels, per element type (the macros let
// a tuning build override them from the compiler command line).
#ifndef SRU_AMD_F32_COLS
#define SRU_AMD_F32_COLS 1
#endif
#ifndef SRU_AMD_F32_FWD_DEPTH
#define SRU_AMD_F32_FWD_DEPTH 8
#endif
#ifndef SRU_AMD_F32_BWD_DEPTH
#define SRU_AMD_F32_BWD_DEPTH 8
#endif
#ifndef SRU_AMD_H16_FWD_DEPTH
#define SRU_AMD_H16_FWD_DEPTH 8
#endif
#ifndef SRU_AMD_H16_BWD_DEPTH
#define SRU_AMD_H16_BWD_DEPTH 8
#endif
// Every large stream is touched exactly once per kernel, so the fast kernels mark their
// loads and stores non-temporal: measured at the headline shape with cache-cold operands,
// forward + backward 447 us -> 425 us (float), 230 us -> 214 us (bfloat16).
#ifndef SRU_AMD_FWD_NT
#define SRU_AMD_FWD_NT (kNtLoad | kNtStore)   // bits for the fast forward kernels
#endif
#ifndef SRU_AMD_BWD_NT
#define SRU_AMD_BWD_NT (kNtLoad | kNtStore)   // the same for the fast backward kernels
#endif
constexpr int kFwdNt = SRU_AMD_FWD_NT, kBwdNt = SRU_AMD_BWD_NT;
// 16-bit streams with few columns: below this many lanes at two columns per lane (fewer than
// 1024 wavefronts) the kernels keep one column per lane and pair lanes for memory access.
#ifndef SRU_AMD_PAIR_BELOW
#define SRU_AMD_PAIR_BELOW 65536
#endif
// Fast forward kernels: forward_scan_chunked (1) or the ring kernel forward_scan (0). Chunked is
// level at 2048 wavefronts and 15-30 % faster where only 256-512 wavefronts exist.
#ifndef SRU_AMD_FWD_CHUNKED
#define SRU_AMD_FWD_CHUNKED 1
#endif
template <typename T> struct Tune;
template <> struct Tune<float> {
    static constexpr int kCols = SRU_AMD_F32_COLS, kFwdDepth = SRU_AMD_F32_FWD_DEPTH,
                         kBwdDepth = SRU_AMD_F32_BWD_DEPTH;
};
template <> struct Tune<half_bits> {
    static constexpr int kCols = 2, kFwdDepth = SRU_AMD_H16_FWD_DEPTH, kBwdDepth = SRU_AMD_H16_BWD_DEPTH;
};
template <> struct Tune<bf16_bits> {
    static constexpr int kCols = 2, kFwdDepth = SRU_AMD_H16_FWD_DEPTH, kBwdDepth = SRU_AMD_H16_BWD_DEPTH;
};
constexpr int kGeneralDepth = 8;

inline bool aligned_to(const void *p, size_t a) { return (reinterpret_cast<uintptr_t>(p) % a) == 0; }

inline dim3 grid_for(int64_t ncols, int cols) {
    const int64_t lanes = ncols / cols;
    return dim3((unsigned)((lanes + kBlock - 1) / kBlock));
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
#ifndef SRU_AMD_UNIFORM
#define SRU_AMD_UNIFORM 1   // 0: never use the scalar-addressing builds (tuning)
#endif
inline bool wave_uniform(int32_t d, int cols) { return SRU_AMD_UNIFORM && d % (kBlock * cols) == 0; }

template <typename T, int K, int SKIP, int COLS, int PAIR = 0, int UNI = -1, int ACT = -1>
void fast_forward(const FwdParams &p, hipStream_t st) {
    if constexpr (ACT < 0) {   // the activation is a template bit of the fast kernels
        if (p.act) return fast_forward<T, K, SKIP, COLS, PAIR, UNI, kTanh>(p, st);
        return fast_forward<T, K, SKIP, COLS, PAIR, UNI, 0>(p, st);
    }
#if SRU_AMD_FWD_CHUNKED
    if constexpr (UNI < 0) {   // pick the scalar-addressing build of the kernel when the shape allows
        if (wave_uniform(p.d, COLS)) return fast_forward<T, K, SKIP, COLS, PAIR, kUniform, ACT>(p, st);
        return fast_forward<T, K, SKIP, COLS, PAIR, 0, ACT>(p, st);
    }
#endif
    constexpr int X = PAIR | (UNI > 0 ? UNI : 0) | (ACT > 0 ? ACT : 0);
    constexpr int P = Tune<T>::kFwdDepth;
    const dim3 grid = grid_for(p.ncols, COLS), block(kBlock);
    // what is kept for the backward pass: nothing, the state after every step, or checkpoints
    const int keep = p.ckpt ? kCkpt : (p.c ? kKeepC : 0);
    const int mode = (p.pad ? kHasPad : 0) | keep;
#if SRU_AMD_FWD_CHUNKED
    constexpr int TC = kCkptInterval;
    switch (mode) {
    case 0: hipLaunchKernelGGL((forward_scan_chunked<T, K, SKIP, kFwdNt | X, COLS, TC>), grid, block, 0, st, p); return;
    case kHasPad: hipLaunchKernelGGL((forward_scan_chunked<T, K, SKIP, kHasPad | kFwdNt | X, COLS, TC>), grid, block, 0, st, p); return;
    case kKeepC: hipLaunchKernelGGL((forward_scan_chunked<T, K, SKIP, kKeepC | kFwdNt | X, COLS, TC>), grid, block, 0, st, p); return;
    case kHasPad | kKeepC: hipLaunchKernelGGL((forward_scan_chunked<T, K, SKIP, kHasPad | kKeepC | kFwdNt | X, COLS, TC>), grid, block, 0, st, p); return;
    case kCkpt: hipLaunchKernelGGL((forward_scan_chunked<T, K, SKIP, kCkpt | kFwdNt | X, COLS, TC>), grid, block, 0, st, p); return;
    default: hipLaunchKernelGGL((forward_scan_chunked<T, K, SKIP, kHasPad | kCkpt | kFwdNt | X, COLS, TC>), grid, block, 0, st, p); return;
    }
#else
    static_assert(PAIR == 0, "lane pairing exists in the chunked kernels only");
    switch (mode) {
    case 0: hipLaunchKernelGGL((forward_scan<T, K, SKIP, kFwdNt | (ACT > 0 ? ACT : 0), COLS, P>), grid, block, 0, st, p); break;
    case kHasPad: hipLaunchKernelGGL((forward_scan<T, K, SKIP, kHasPad | kFwdNt | (ACT > 0 ? ACT : 0), COLS, P>), grid, block, 0, st, p); break;
    case kKeepC: hipLaunchKernelGGL((forward_scan<T, K, SKIP, kKeepC | kFwdNt | (ACT > 0 ? ACT : 0), COLS, P>), grid, block, 0, st, p); break;
    case kHasPad | kKeepC: hipLaunchKernelGGL((forward_scan<T, K, SKIP, kHasPad | kKeepC | kFwdNt | (ACT > 0 ? ACT : 0), COLS, P>), grid, block, 0, st, p); break;
    case kCkpt: hipLaunchKernelGGL((forward_scan<T, K, SKIP, kCkpt | kFwdNt | (ACT > 0 ? ACT : 0), COLS, kCkptInterval>), grid, block, 0, st, p); break;
    default: hipLaunchKernelGGL((forward_scan<T, K, SKIP, kHasPad | kCkpt | kFwdNt | (ACT > 0 ? ACT : 0), COLS, kCkptInterval>), grid, block, 0, st, p); break;
    }
#endif
}

template <typename T, int K, int SKIP, int COLS, int PAIR = 0, int ACT = -1>
void fast_backward(const BwdParams &p, hipStream_t st) {
    if constexpr (ACT < 0) {
        if (p.act) return fast_backward<T, K, SKIP, COLS, PAIR, kTanh>(p, st);
        return fast_backward<T, K, SKIP, COLS, PAIR, 0>(p, st);
    }
    constexpr int A = ACT > 0 ? ACT : 0;
    constexpr int P = Tune<T>::kBwdDepth;
    constexpr int TC = kCkptInterval;
    const dim3 grid = grid_for(p.ncols, COLS), block(kBlock);
    if (p.ckpt) {
        const int mode = (p.pad ? 1 : 0) | (wave_uniform(p.d, COLS) ? 2 : 0);
        switch (mode) {
        case 0: hipLaunchKernelGGL((backward_scan_ckpt<T, K, SKIP, kBwdNt | PAIR | A, COLS, TC>), grid, block, 0, st, p); break;
        case 1: hipLaunchKernelGGL((backward_scan_ckpt<T, K, SKIP, kHasPad | kBwdNt | PAIR | A, COLS, TC>), grid, block, 0, st, p); break;
        case 2: hipLaunchKernelGGL((backward_scan_ckpt<T, K, SKIP, kBwdNt | PAIR | A | kUniform, COLS, TC>), grid, block, 0, st, p); break;
        default: hipLaunchKernelGGL((backward_scan_ckpt<T, K, SKIP, kHasPad | kBwdNt | PAIR | A | kUniform, COLS, TC>), grid, block, 0, st, p); break;
        }
    } else if (p.pad) {
        hipLaunchKernelGGL((backward_scan<T, K, SKIP, kHasPad | kBwdNt | A, COLS, P>), grid, block, 0, st, p);
    } else {
        hipLaunchKernelGGL((backward_scan<T, K, SKIP, kBwdNt | A, COLS, P>), grid, block, 0, st, p);
    }
}

template <typename T, int K, int SKIP>
void pick_forward(const sru_amd_shape &s, const FwdParams &p, hipStream_t st) {
    if constexpr (Tune<T>::kCols == 2) {
        if (pair_ok<T, K>(s, {p.u}, {p.x, p.h, p.c})) {
#if SRU_AMD_FWD_CHUNKED
            if constexpr (sizeof(T) == 2) {
                if (p.ncols / 2 < SRU_AMD_PAIR_BELOW) return fast_forward<T, K, SKIP, 1, kPair>(p, st);
            }
#endif
            return fast_forward<T, K, SKIP, 2>(p, st);
        }
    }
    fast_forward<T, K, SKIP, 1>(p, st);
}

template <typename T, int K, int SKIP>
void pick_backward(const sru_amd_shape &s, const BwdParams &p, hipStream_t st) {
    if constexpr (Tune<T>::kCols == 2) {
        if (pair_ok<T, K>(s, {p.u, p.gu}, {p.x, p.c, p.gh, p.gx})) {  // p.c is null with checkpoints
            if constexpr (sizeof(T) == 2) {
                if (p.ckpt && p.ncols / 2 < SRU_AMD_PAIR_BELOW) return fast_backward<T, K, SKIP, 1, kPair>(p, st);
            }
            return fast_backward<T, K, SKIP, 2>(p, st);
        }
    }
    fast_backward<T, K, SKIP, 1>(p, st);
}

// (k, skip_type) pairs that pass the shape check: (3,0) (3,1) (4,0) (4,2).
template <typename T>
void launch_forward(const sru_amd_shape &s, const FwdParams &p, hipStream_t st) {
    const bool general = s.is_custom != 0 || (s.skip_type == 0 && s.k == 4);
    const dim3 grid = grid_for(p.ncols, 1), block(kBlock);
    constexpr int P = kGeneralDepth;
    if (!general) {
        if (s.k == 4) pick_forward<T, 4, 2>(s, p, st);
        else if (s.skip_type == 1) pick_forward<T, 3, 1>(s, p, st);
        else pick_forward<T, 3, 0>(s, p, st);
    } else if (s.k == 3 && s.skip_type == 1) {
        hipLaunchKernelGGL((forward_scan<T, 3, 1, kGeneral | kFwdNt, 1, P>), grid, block, 0, st, p);
    } else if (s.k == 3) {
        hipLaunchKernelGGL((forward_scan<T, 3, 0, kGeneral | kFwdNt, 1, P>), grid, block, 0, st, p);
    } else if (s.skip_type == 2) {
        hipLaunchKernelGGL((forward_scan<T, 4, 2, kGeneral | kFwdNt, 1, P>), grid, block, 0, st, p);
    } else {
        hipLaunchKernelGGL((forward_scan<T, 4, 0, kGeneral | kFwdNt, 1, P>), grid, block, 0, st, p);
    }
}

template <typename T>
void launch_backward(const sru_amd_shape &s, const BwdParams &p, hipStream_t st) {
    const bool general = s.is_custom != 0 || (s.skip_type == 0 && s.k == 4);
    const dim3 grid = grid_for(p.ncols, 1), block(kBlock);
    constexpr int P = kGeneralDepth;
    if (!general) {
        if (s.k == 4) pick_backward<T, 4, 2>(s, p, st);
        else if (s.skip_type == 1) pick_backward<T, 3, 1>(s, p, st);
        else pick_backward<T, 3, 0>(s, p, st);
    } else if (s.k == 3 && s.skip_type == 1) {
        hipLaunchKernelGGL((backward_scan<T, 3, 1, kGeneral | kBwdNt, 1, P>), grid, block, 0, st, p);
    } else if (s.k == 3) {
        hipLaunchKernelGGL((backward_scan<T, 3, 0, kGeneral | kBwdNt, 1, P>), grid, block, 0, st, p);
    } else if (s.skip_type == 2) {
        hipLaunchKernelGGL((backward_scan<T, 4, 2, kGeneral | kBwdNt, 1, P>), grid, block, 0, st, p);
    } else {
        hipLaunchKernelGGL((backward_scan<T, 4, 0, kGeneral | kBwdNt, 1, P>), grid, block, 0, st, p);
    }
}

}  // namespace sru_amd
