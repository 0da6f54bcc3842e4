// Layer normalisation next to the recurrence: the reference normalises a layer's input before the
// projection (sru/modules.py:250-253) or its output after the recurrence (:278-279) with
// torch.nn.LayerNorm over the feature dimension (created at :155-162, eps 1e-5, affine).
// These kernels read the tensor once in the dtype it has and write the normalised rows in the dtype
// the consumer wants (the 16-bit operand of the projection under autocast), which replaces the
// chain "cast to float, normalise, cast to 16 bits" that autocast builds around torch's kernel.
//
// Mapping: one workgroup per row at a time (a row = the D features of one (t, b) position), 1 to 8
// wavefronts of which every lane holds 8 consecutive features, so rows of float move as two
// 16-byte vectors per lane, 16-bit rows as one; workgroups walk rows with a stride of the grid and
// load the next row while they reduce the current one. Statistics are float: mean first, then the
// variance of the centred values (wavefront reductions combined through LDS in wavefront order).
// The backward kernel runs at most one workgroup per compute unit: 16 wavefronts that form several
// row groups, each working like a workgroup of the forward kernel on rows of its own. Every lane
// keeps its share of the weight / bias gradient sums in registers over the rows its group visits;
// at the end the groups add their shares through LDS in group order and the workgroup leaves one
// partial row (at most 256 in all, 4 MB at 2 048 features); reduce_rows() then adds the workgroups
// in index order, in double, in one launch: bit-reproducible.
#include "sru_amd.h"

#include <hip/hip_runtime.h>

#include "sru_scan.h"

namespace {

using namespace sru_amd;

constexpr int kLanes = 64;
constexpr int kPer = 8;                       // features per lane and pass
constexpr int kPass = kLanes * kPer;          // features per pass of a wavefront

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

template <typename T> __device__ __forceinline__ void load8(const T *p, float (&v)[kPer]);
template <> __device__ __forceinline__ void load8<float>(const float *p, float (&v)[kPer]) {
    const f32x4 a = *reinterpret_cast<const f32x4 *>(p), b = *reinterpret_cast<const f32x4 *>(p + 4);
#pragma unroll
    for (int i = 0; i < 4; ++i) { v[i] = a[i]; v[4 + i] = b[i]; }
}
template <typename T> __device__ __forceinline__ void load8(const T *p, float (&v)[kPer]) {
    const u32x4 a = *reinterpret_cast<const u32x4 *>(p);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        v[2 * i] = bits_to_float<T>(a[i] & 0xffffu);
        v[2 * i + 1] = bits_to_float<T>(a[i] >> 16);
    }
}
template <typename T> __device__ __forceinline__ void store8(T *p, const float (&v)[kPer]);
template <> __device__ __forceinline__ void store8<float>(float *p, const float (&v)[kPer]) {
    f32x4 a, b;
#pragma unroll
    for (int i = 0; i < 4; ++i) { a[i] = v[i]; b[i] = v[4 + i]; }
    *reinterpret_cast<f32x4 *>(p) = a;
    *reinterpret_cast<f32x4 *>(p + 4) = b;
}
template <typename T> __device__ __forceinline__ void store8(T *p, const float (&v)[kPer]) {
    u32x4 a;
#pragma unroll
    for (int i = 0; i < 4; ++i) a[i] = pack_pair<T>(v[2 * i], v[2 * i + 1]);
    *reinterpret_cast<u32x4 *>(p) = a;
}

// A lane's 8 features of one row as they come from memory: loaded without a condition (the
// callers clamp the address), so that the load can stay in flight across a loop trip, and turned
// into floats only when the row's turn comes.
template <typename T> struct Raw {
    u32x4 a;
    __device__ __forceinline__ void load(const T *p) { a = *reinterpret_cast<const u32x4 *>(p); }
    __device__ __forceinline__ void unpack(float (&v)[kPer]) const {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            v[2 * i] = bits_to_float<T>(a[i] & 0xffffu);
            v[2 * i + 1] = bits_to_float<T>(a[i] >> 16);
        }
    }
};
template <> struct Raw<float> {
    f32x4 a, b;
    __device__ __forceinline__ void load(const float *p) {
        a = *reinterpret_cast<const f32x4 *>(p);
        b = *reinterpret_cast<const f32x4 *>(p + 4);
    }
    __device__ __forceinline__ void unpack(float (&v)[kPer]) const {
#pragma unroll
        for (int i = 0; i < 4; ++i) { v[i] = a[i]; v[4 + i] = b[i]; }
    }
};

// v of another lane, chosen by a data-parallel-primitive control word; lanes outside row_mask get 0
template <int CTRL, int ROW_MASK = 0xF>
__device__ __forceinline__ float dpp(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, ROW_MASK, 0xF, false));
}

// Sum over the wavefront, the same value in every lane: pairs, quads, then the four quads of each
// row of 16 lanes by rotation, then row 0 into row 1 and row 2 into row 3, rows 0-1 into rows 2-3,
// and the last lane's total to all.
__device__ __forceinline__ float wave_sum(float v) {
    v += dpp<0xB1>(v);         // quad_perm [1,0,3,2]
    v += dpp<0x4E>(v);         // quad_perm [2,3,0,1]
    v += dpp<0x124>(v);        // row_ror 4
    v += dpp<0x128>(v);        // row_ror 8
    v += dpp<0x142, 0xA>(v);   // row_bcast 15 into rows 1 and 3
    v += dpp<0x143, 0xC>(v);   // row_bcast 31 into rows 2 and 3
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));
}

// Rows a workgroup handles per trip: their loads are in flight together and their sums share a barrier.
constexpr int kRowsPer = 2;

// Sums over the WAVES wavefronts that share a row (a whole workgroup, or one row group of it; the
// barrier is the workgroup's) of N values at once, the wavefronts' shares added in wavefront order. `red` holds N * WAVES floats and must not be
// rewritten before every thread has read it (the callers alternate two arrays so that the next
// barrier provides that).
template <int WAVES, int N>
__device__ __forceinline__ void block_sums(float (&v)[N], float *red) {
#pragma unroll
    for (int n = 0; n < N; ++n) v[n] = wave_sum(v[n]);
    if constexpr (WAVES > 1) {
        if ((threadIdx.x & (kLanes - 1)) == 0) {
#pragma unroll
            for (int n = 0; n < N; ++n) red[n * WAVES + ((threadIdx.x >> 6) % WAVES)] = v[n];
        }
        __syncthreads();
#pragma unroll
        for (int n = 0; n < N; ++n) {
            v[n] = red[n * WAVES];
#pragma unroll
            for (int w = 1; w < WAVES; ++w) v[n] += red[n * WAVES + w];
        }
    }
}

// y = (x - mean) * rstd * gamma + beta per row; mean and rstd (float, one per row) are kept for
// the backward pass. A workgroup of WAVES wavefronts owns kRowsPer consecutive rows at a time, every
// lane 8 consecutive features of each (D <= 512 * WAVES), and walks the row groups with a stride of
// the grid; the next group's loads are issued before the current group's reductions.
template <typename TI, typename TO, int WAVES>
__global__ void __launch_bounds__(kLanes * WAVES)
layer_norm_forward(const TI *x, const float *gamma, const float *beta, TO *y, float *mean, float *rstd,
                   int64_t rows, int32_t D, float eps) {
    constexpr int R = kRowsPer;
    __shared__ float red_a[R * WAVES], red_b[R * WAVES];
    const int e = threadIdx.x * kPer;
    const bool active = e < D;
    float g[kPer] = {}, b[kPer] = {};
    if (active) {
        load8<float>(gamma + e, g);
        load8<float>(beta + e, b);
    }
    const float inv_d = 1.0f / (float)D;
    const TI *mine = x + (active ? e : 0);   // lanes past the row's end re-read its start and drop it
    const int64_t last = rows - 1;
    Raw<TI> next[R];
    int64_t row = (int64_t)blockIdx.x * R;
#pragma unroll
    for (int r = 0; r < R; ++r) next[r].load(mine + (row + r < last ? row + r : last) * D);
    for (; row < rows; row += (int64_t)gridDim.x * R) {
        float v[R][kPer], s[R], q[R];
#pragma unroll
        for (int r = 0; r < R; ++r) next[r].unpack(v[r]);
        const int64_t after = row + (int64_t)gridDim.x * R;
#pragma unroll
        for (int r = 0; r < R; ++r) next[r].load(mine + (after + r < last ? after + r : last) * D);
#pragma unroll
        for (int r = 0; r < R; ++r) {
            s[r] = 0.f;
#pragma unroll
            for (int i = 0; i < kPer; ++i) {
                v[r][i] = active ? v[r][i] : 0.f;
                s[r] += v[r][i];
            }
        }
        block_sums<WAVES, R>(s, red_a);
#pragma unroll
        for (int r = 0; r < R; ++r) {
            s[r] *= inv_d;
            q[r] = 0.f;
            if (active) {
#pragma unroll
                for (int i = 0; i < kPer; ++i) {
                    v[r][i] -= s[r];
                    q[r] += v[r][i] * v[r][i];
                }
            }
        }
        block_sums<WAVES, R>(q, red_b);
#pragma unroll
        for (int r = 0; r < R; ++r) {
            if (row + r >= rows) break;
            const float rs = rsqrtf(q[r] * inv_d + eps);
            if (active) {
                float o[kPer];
#pragma unroll
                for (int i = 0; i < kPer; ++i) o[i] = v[r][i] * rs * g[i] + b[i];
                store8<TO>(y + (row + r) * D + e, o);
            }
            if (threadIdx.x == 0) {
                mean[row + r] = s[r];
                rstd[row + r] = rs;
            }
        }
    }
}

// dx = rstd * (g - mean(g) - xhat * mean(g * xhat)) with g = dy * gamma, xhat = (x - mean) * rstd;
// partial[block] = (sum over the block's rows of dy * xhat, sum of dy), each D floats.
// A workgroup is GROUPS row groups of WAVES wavefronts; a group owns kRowsPer consecutive rows per
// trip, every lane 8 consecutive features of each, and the groups of all workgroups walk the rows
// with a stride of the launch. Every feature belongs to one lane of each group, which adds its rows
// in the order it visits them; the groups' sums are added in group order at the end.
template <typename TI, typename TG, typename TD, int WAVES, int GROUPS>
__global__ void __launch_bounds__(kLanes * WAVES * GROUPS)
layer_norm_backward(const TI *x, const float *gamma, const float *mean, const float *rstd, const TG *dy, TD *dx,
                    float *partial, int64_t rows, int32_t D) {
    constexpr int R = kRowsPer;
    __shared__ float red[2][GROUPS][2 * R * WAVES];   // alternate by trip: one barrier per trip
    __shared__ float acc[2 * kPass * WAVES];            // the groups' weight / bias sums, added in group order
    const int grp = __builtin_amdgcn_readfirstlane((int)(threadIdx.x / (kLanes * WAVES)));
    const int e = (int)(threadIdx.x % (kLanes * WAVES)) * kPer;
    const bool active = e < D;
    float g[kPer] = {}, dg[kPer] = {}, db[kPer] = {};
    if (active) load8<float>(gamma + e, g);
    const float inv_d = 1.0f / (float)D;
    const int ec = active ? e : 0;   // lanes past the row's end re-read its start and drop it
    const TI *my_x = x + ec;
    const TG *my_dy = dy + ec;
    const int64_t last = rows - 1;
    const int64_t stride = (int64_t)gridDim.x * GROUPS * R;
    Raw<TI> nx[R];
    Raw<TG> nd[R];
    float nmu[R], nrs[R];
    // The rows of a trip and their statistics are requested a trip ahead, the statistics first: a
    // wavefront's loads return in the order they were issued, so a statistic fetched after the
    // next trip's rows would make the current trip wait for those rows as well (44.9 -> 41.8 us at
    // 16 384 x 2 048 in bfloat16). A group past the last row repeats the last row and drops it.
    auto fetch = [&](int64_t row0) __attribute__((always_inline)) {
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const int64_t at = row0 + r < last ? row0 + r : last;
            nmu[r] = mean[at];
            nrs[r] = rstd[at];
        }
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const int64_t at = (row0 + r < last ? row0 + r : last) * D;
            nx[r].load(my_x + at);
            nd[r].load(my_dy + at);
        }
    };
    // `first` is the first row of the workgroup's trip (the same for all its groups, so that every
    // wavefront makes the same number of trips and meets the others at the barriers)
    int64_t first = (int64_t)blockIdx.x * GROUPS * R;
    fetch(first + grp * R);
    int parity = 0;
    for (; first < rows; first += stride, parity ^= 1) {
        const int64_t row = first + grp * R;
        float xh[R][kPer], gy[R][kPer], sums[2 * R], rs[R], mus[R];
#pragma unroll
        for (int r = 0; r < R; ++r) {
            nx[r].unpack(xh[r]);
            nd[r].unpack(gy[r]);
            mus[r] = nmu[r];
            rs[r] = nrs[r];
        }
        fetch(row + stride);
        __builtin_amdgcn_sched_barrier(0);   // the requests of the next trip go out before this trip's arithmetic
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const bool live = row + r < rows;   // a row past the end repeats the last row and is dropped
            const float mu = mus[r];
            rs[r] = live ? rs[r] : 0.f;
            float s1 = 0.f, s2 = 0.f;
            if (live) {
#pragma unroll
                for (int i = 0; i < kPer; ++i) {
                    const float d = active ? gy[r][i] : 0.f;
                    xh[r][i] = (xh[r][i] - mu) * rs[r];
                    gy[r][i] = d * g[i];
                    s1 += gy[r][i];
                    s2 += gy[r][i] * xh[r][i];
                    dg[i] += d * xh[r][i];
                    db[i] += d;
                }
            }
            sums[2 * r] = s1;
            sums[2 * r + 1] = s2;
        }
        block_sums<WAVES, 2 * R>(sums, red[parity][grp]);
#pragma unroll
        for (int r = 0; r < R; ++r) {
            if (row + r >= rows || !active) continue;
            const float c1 = sums[2 * r] * inv_d, c2 = sums[2 * r + 1] * inv_d;
            float o[kPer];
#pragma unroll
            for (int i = 0; i < kPer; ++i) o[i] = rs[r] * (gy[r][i] - c1 - xh[r][i] * c2);
            store8<TD>(dx + (row + r) * D + e, o);
        }
    }
    // the groups' shares, added in group order
#pragma unroll
    for (int gi = 0; gi < GROUPS; ++gi) {
        if (grp == gi && active) {
#pragma unroll
            for (int i = 0; i < kPer; ++i) {
                acc[e + i] = (gi == 0 ? 0.f : acc[e + i]) + dg[i];
                acc[kPass * WAVES + e + i] = (gi == 0 ? 0.f : acc[kPass * WAVES + e + i]) + db[i];
            }
        }
        __syncthreads();
    }
    if (grp == 0 && active) {
        float *out = partial + (int64_t)blockIdx.x * 2 * D;
#pragma unroll
        for (int i = 0; i < kPer; ++i) {
            dg[i] = acc[e + i];
            db[i] = acc[kPass * WAVES + e + i];
        }
        store8<float>(out + e, dg);
        store8<float>(out + D + e, db);
    }
}

// out[e] = sum over the rows r of partial[r][e]. One workgroup per 64 columns; its 16 wavefronts
// take every 16th row each, accumulate in double and are combined through LDS in a fixed order.
constexpr int kRowSlices = 16;
__global__ void __launch_bounds__(kLanes * kRowSlices)
reduce_rows(const float *partial, float *out, int32_t nrows, int32_t width) {
    __shared__ double part[kRowSlices][kLanes];
    const int lane = threadIdx.x & (kLanes - 1), slice = threadIdx.x >> 6;
    const int e = blockIdx.x * kLanes + lane;
    double s = 0.0;
    if (e < width) {
        // the loads of a batch are issued together (addresses clamped, surplus values dropped), then added in row order
        constexpr int kBatch = 8;
        for (int r0 = slice; r0 < nrows; r0 += kRowSlices * kBatch) {
            float v[kBatch];
#pragma unroll
            for (int i = 0; i < kBatch; ++i) {
                const int r = r0 + i * kRowSlices;
                v[i] = partial[(int64_t)(r < nrows ? r : nrows - 1) * width + e];
            }
#pragma unroll
            for (int i = 0; i < kBatch; ++i) s += (r0 + i * kRowSlices < nrows) ? (double)v[i] : 0.0;
        }
    }
    part[slice][lane] = s;
    __syncthreads();
    if (slice == 0 && e < width) {
        double total = part[0][lane];
#pragma unroll
        for (int i = 1; i < kRowSlices; ++i) total += part[i][lane];
        out[e] = (float)total;
    }
}

// wavefronts per row: 8 features per lane
inline int norm_waves(int32_t D) {
    const int need = (D + kPass - 1) / kPass;
    return need <= 1 ? 1 : need <= 2 ? 2 : need <= 4 ? 4 : 8;
}

// Workgroups of a forward launch: each walks groups of kRowsPer rows with a stride of the grid.
int norm_blocks(int64_t rows) {
    const int64_t groups = (rows + kRowsPer - 1) / kRowsPer;
    return (int)(groups < 1024 ? groups : 1024);
}

// The backward kernel: 16 wavefronts per workgroup (16 / waves-per-row row groups) and at most one
// workgroup per compute unit for 16-bit rows, 8 wavefronts and at most two workgroups for float rows
// (measured at 16 384 x 2 048: bf16 44 us against 48 us with 8, float 84 us against 89 us with 16),
// so that the partial rows stay few; rows of more than 2 048 features (8 wavefronts per row) form
// one group per workgroup of 8.
inline int backward_waves(size_t x_elem_bytes, int waves) { return (x_elem_bytes == 4 || waves == 8) ? 8 : 16; }
int backward_blocks(int64_t rows, int32_t D, size_t x_elem_bytes) {
    const int waves = norm_waves(D), per = backward_waves(x_elem_bytes, waves), groups = per / waves;
    const int64_t per_block = (int64_t)groups * kRowsPer;
    const int64_t blocks = (rows + per_block - 1) / per_block;
    const int64_t most = 256 * (16 / per);
    return (int)(blocks < most ? blocks : most);
}

bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) % 16) == 0; }

int check_norm(int64_t rows, int64_t cols, int dt_a, int dt_b) {
    if (rows < 1 || cols < 1 || cols % kPer != 0 || cols > SRU_AMD_NORM_MAX_FEATURES || rows > (INT64_C(1) << 40))
        return SRU_AMD_ERR_BAD_SHAPE;
    for (int dt : {dt_a, dt_b})
        if (dt != SRU_AMD_F32 && dt != SRU_AMD_F16 && dt != SRU_AMD_BF16) return SRU_AMD_ERR_BAD_DTYPE;
    return SRU_AMD_OK;
}

template <typename TI, typename TO>
hipError_t launch_norm_forward(const void *x, const float *gamma, const float *beta, void *y, float *mean,
                               float *rstd, int64_t rows, int32_t D, float eps, hipStream_t st) {
    const TI *xi = static_cast<const TI *>(x);
    TO *yo = static_cast<TO *>(y);
    void *args[] = {&xi, &gamma, &beta, &yo, &mean, &rstd, &rows, &D, &eps};
    const int waves = norm_waves(D);
    const void *k = waves == 1   ? reinterpret_cast<const void *>(layer_norm_forward<TI, TO, 1>)
                    : waves == 2 ? reinterpret_cast<const void *>(layer_norm_forward<TI, TO, 2>)
                    : waves == 4 ? reinterpret_cast<const void *>(layer_norm_forward<TI, TO, 4>)
                                 : reinterpret_cast<const void *>(layer_norm_forward<TI, TO, 8>);
    return hipLaunchKernel(k, dim3(norm_blocks(rows)), dim3(kLanes * waves), args, 0, st);
}

template <typename TI, typename TG, typename TD>
hipError_t launch_norm_backward(const void *x, const float *gamma, const float *mean, const float *rstd,
                                const void *dy, void *dx, float *partial, int64_t rows, int32_t D, hipStream_t st) {
    const TI *xi = static_cast<const TI *>(x);
    const TG *gi = static_cast<const TG *>(dy);
    TD *di = static_cast<TD *>(dx);
    void *args[] = {&xi, &gamma, &mean, &rstd, &gi, &di, &partial, &rows, &D};
    const int waves = norm_waves(D);
    constexpr int PER = sizeof(TI) == 4 ? 8 : 16;   // backward_waves()
    const void *k = waves == 1   ? reinterpret_cast<const void *>(layer_norm_backward<TI, TG, TD, 1, PER>)
                    : waves == 2 ? reinterpret_cast<const void *>(layer_norm_backward<TI, TG, TD, 2, PER / 2>)
                    : waves == 4 ? reinterpret_cast<const void *>(layer_norm_backward<TI, TG, TD, 4, PER / 4>)
                                 : reinterpret_cast<const void *>(layer_norm_backward<TI, TG, TD, 8, 1>);
    return hipLaunchKernel(k, dim3(backward_blocks(rows, D, sizeof(TI))), dim3(kLanes * backward_waves(sizeof(TI), waves)),
                           args, 0, st);
}

// run F<A, B>(...) for the two runtime dtypes
template <typename A>
hipError_t forward_by_out(int dt_y, const void *x, const float *gamma, const float *beta, void *y, float *mean,
                          float *rstd, int64_t rows, int32_t D, float eps, hipStream_t st) {
    if (dt_y == SRU_AMD_F32) return launch_norm_forward<A, float>(x, gamma, beta, y, mean, rstd, rows, D, eps, st);
    if (dt_y == SRU_AMD_F16) return launch_norm_forward<A, half_bits>(x, gamma, beta, y, mean, rstd, rows, D, eps, st);
    return launch_norm_forward<A, bf16_bits>(x, gamma, beta, y, mean, rstd, rows, D, eps, st);
}

// the gradient of x has x's dtype
template <typename A>
hipError_t backward_by_grad(int dt_y, const void *x, const float *gamma, const float *mean, const float *rstd,
                            const void *dy, void *dx, float *partial, int64_t rows, int32_t D, hipStream_t st) {
    if (dt_y == SRU_AMD_F32) return launch_norm_backward<A, float, A>(x, gamma, mean, rstd, dy, dx, partial, rows, D, st);
    if (dt_y == SRU_AMD_F16) return launch_norm_backward<A, half_bits, A>(x, gamma, mean, rstd, dy, dx, partial, rows, D, st);
    return launch_norm_backward<A, bf16_bits, A>(x, gamma, mean, rstd, dy, dx, partial, rows, D, st);
}

}  // namespace

extern "C" {

int sru_amd_layer_norm_forward(int64_t rows, int64_t cols, const void *x, int x_dtype, const float *weight,
                               const float *bias, float eps, void *y, int y_dtype, float *mean, float *rstd,
                               void *stream) {
    if (const int rc = check_norm(rows, cols, x_dtype, y_dtype)) return rc;
    if (!x || !weight || !bias || !y || !mean || !rstd) return SRU_AMD_ERR_NULL_POINTER;
    if (!aligned16(x) || !aligned16(y) || !aligned16(weight) || !aligned16(bias)) return SRU_AMD_ERR_MISALIGNED;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const int32_t D = (int32_t)cols;
    const hipError_t err =
        x_dtype == SRU_AMD_F32   ? forward_by_out<float>(y_dtype, x, weight, bias, y, mean, rstd, rows, D, eps, st)
        : x_dtype == SRU_AMD_F16 ? forward_by_out<half_bits>(y_dtype, x, weight, bias, y, mean, rstd, rows, D, eps, st)
                                 : forward_by_out<bf16_bits>(y_dtype, x, weight, bias, y, mean, rstd, rows, D, eps, st);
    return err == hipSuccess ? SRU_AMD_OK : SRU_AMD_ERR_LAUNCH;
}

size_t sru_amd_layer_norm_backward_workspace_bytes(int64_t rows, int64_t cols) {
    if (check_norm(rows, cols, SRU_AMD_F32, SRU_AMD_F32) != SRU_AMD_OK) return 0;
    // one float row pair per workgroup of the backward kernel (the larger of the two launch shapes)
    return (size_t)backward_blocks(rows, (int32_t)cols, 4) * 2 * (size_t)cols * sizeof(float);
}

int sru_amd_layer_norm_backward(int64_t rows, int64_t cols, const void *x, int x_dtype, const float *weight,
                                const float *mean, const float *rstd, const void *grad_y, int y_dtype,
                                void *grad_x, float *grad_weight, float *grad_bias, void *workspace,
                                size_t workspace_bytes, void *stream) {
    if (const int rc = check_norm(rows, cols, x_dtype, y_dtype)) return rc;
    if (!x || !weight || !mean || !rstd || !grad_y || !grad_x || !grad_weight || !grad_bias)
        return SRU_AMD_ERR_NULL_POINTER;
    if (!aligned16(x) || !aligned16(grad_y) || !aligned16(grad_x) || !aligned16(weight)) return SRU_AMD_ERR_MISALIGNED;
    if (!workspace || !aligned16(workspace) || workspace_bytes < sru_amd_layer_norm_backward_workspace_bytes(rows, cols))
        return SRU_AMD_ERR_WORKSPACE;
    // the two sums must be contiguous for the single reduction launch: (grad_weight, grad_bias) = out[0:D], out[D:2D]
    if (grad_bias != grad_weight + cols) return SRU_AMD_ERR_MISALIGNED;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const int32_t D = (int32_t)cols;
    float *partial = static_cast<float *>(workspace);
    const hipError_t err =
        x_dtype == SRU_AMD_F32   ? backward_by_grad<float>(y_dtype, x, weight, mean, rstd, grad_y, grad_x, partial, rows, D, st)
        : x_dtype == SRU_AMD_F16 ? backward_by_grad<half_bits>(y_dtype, x, weight, mean, rstd, grad_y, grad_x, partial, rows, D, st)
                                 : backward_by_grad<bf16_bits>(y_dtype, x, weight, mean, rstd, grad_y, grad_x, partial, rows, D, st);
    if (err != hipSuccess) return SRU_AMD_ERR_LAUNCH;
    int32_t nrows = backward_blocks(rows, D, x_dtype == SRU_AMD_F32 ? 4 : 2), width = 2 * D;
    const float *src = partial;
    void *args[] = {&src, &grad_weight, &nrows, &width};
    return hipLaunchKernel(reinterpret_cast<const void *>(reduce_rows), dim3((width + kLanes - 1) / kLanes),
                           dim3(kLanes * kRowSlices), args, 0, st) == hipSuccess ? SRU_AMD_OK : SRU_AMD_ERR_LAUNCH;
}

}  // extern "C"
