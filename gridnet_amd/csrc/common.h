// Shared device helpers and host-side error plumbing for libgridnet_hip.so (gfx950 only).
#pragma once

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdio>

#include "../../include/gridnet_hip.h"

namespace gridnet {

constexpr int kWave = 64;        // CDNA wavefront width
constexpr int kMaxBackwardIters = 32;

// ---- host: thread-local error message -------------------------------------------------
char *error_buffer();
int fail(int status, const char *fmt, ...) __attribute__((format(printf, 2, 3)));
int check_launch(const char *what);

// ---- device: activations ---------------------------------------------------------------
// Values follow torch (gridnet/backend_torch.py:270-280): leaky slope 0.01; the derivative
// at exactly 0 is the negative-side one, as torch's backward formulas give.
template <typename T> __device__ __forceinline__ T exp_accurate(T v);
template <> __device__ __forceinline__ float exp_accurate<float>(float v) { return expf(v); }
template <> __device__ __forceinline__ double exp_accurate<double>(double v) { return exp(v); }

template <typename T> __device__ __forceinline__ T sigmoid_stable(T u) {
    // one exp of a non-positive argument: never overflows
    T e = exp_accurate<T>(u > T(0) ? -u : u);
    T s = e / (T(1) + e);          // sigmoid(-|u|)
    return u > T(0) ? T(1) - s : s;
}

template <int ACT, typename T> struct Act;

template <typename T> struct Act<GRIDNET_ACT_RELU, T> {
    static __device__ __forceinline__ T f(T u) { return u > T(0) ? u : T(0); }
    static __device__ __forceinline__ void fd(T u, T &f, T &d) {
        bool pos = u > T(0);
        f = pos ? u : T(0);
        d = pos ? T(1) : T(0);
    }
};
template <typename T> struct Act<GRIDNET_ACT_LEAKY_RELU, T> {
    static __device__ __forceinline__ T f(T u) { return u > T(0) ? u : T(0.01) * u; }
    static __device__ __forceinline__ void fd(T u, T &f, T &d) {
        bool pos = u > T(0);
        f = pos ? u : T(0.01) * u;
        d = pos ? T(1) : T(0.01);
    }
};
template <typename T> struct Act<GRIDNET_ACT_SILU, T> {
    static __device__ __forceinline__ T f(T u) { return u * sigmoid_stable(u); }
    static __device__ __forceinline__ void fd(T u, T &f, T &d) {
        T s = sigmoid_stable(u);
        f = u * s;
        d = s * (T(1) + u * (T(1) - s));
    }
};
template <typename T> struct Act<GRIDNET_ACT_TANH, T> {
    static __device__ __forceinline__ T f(T u) {
        // tanh(u) = sign(u) * (1 - e) / (1 + e), e = exp(-2|u|): accurate and overflow-free
        T a = u < T(0) ? -u : u;
        T e = exp_accurate<T>(T(-2) * a);
        T t = (T(1) - e) / (T(1) + e);
        return u < T(0) ? -t : t;
    }
    static __device__ __forceinline__ void fd(T u, T &f, T &d) {
        f = Act::f(u);
        d = T(1) - f * f;
    }
};

// ---- device: reductions ----------------------------------------------------------------
template <typename T> __device__ __forceinline__ T wave_sum(T v) {
#pragma unroll
    for (int off = kWave / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, kWave);
    return v;
}

// Sum over the whole workgroup; every thread gets the same bits (fixed combination order).
// `scratch` holds one T per wave.  Contains two barriers.
template <typename T> __device__ __forceinline__ T block_sum(T v, T *scratch, int tid, int nthreads) {
    v = wave_sum(v);
    const int nwaves = (nthreads + kWave - 1) / kWave;
    if (nwaves == 1) return v;
    __syncthreads();  // scratch may still be read by a previous call
    if ((tid & (kWave - 1)) == 0) scratch[tid / kWave] = v;
    __syncthreads();
    T total = scratch[0];
    for (int i = 1; i < nwaves; ++i) total += scratch[i];
    return total;
}

// Workgroup id -> (spatial block, batch chunk).  Workgroup ids are dealt to the 8 XCDs
// round-robin and every XCD has its own L2, so XCD x is given a CONTIGUOUS range of spatial
// blocks (raster order: neighbours along K, then N): neighbouring blocks share halo cells and
// whole cache lines of every K-row, and the chunks of one block share its 29 parameter planes.
// Handing neighbouring blocks to different XCDs makes each L2 fetch those lines again.
// The grid is padded to 8 * ceil(nblk / 8) * nchunk workgroups; returns false for the padding.
constexpr int kXcds = 8;
__host__ __device__ __forceinline__ int padded_grid(int nblk, int nchunk) {
    return kXcds * ((nblk + kXcds - 1) / kXcds) * nchunk;
}
__device__ __forceinline__ bool split_block_id(int wg, int nblk, int nchunk, int &blk, int &chunk) {
    const int per_xcd = (nblk + kXcds - 1) / kXcds;
    const int xcd = wg % kXcds, slot = wg / kXcds;
    blk = xcd * per_xcd + slot / nchunk;
    chunk = slot % nchunk;
    return slot / nchunk < per_xcd && blk < nblk;
}

}  // namespace gridnet
