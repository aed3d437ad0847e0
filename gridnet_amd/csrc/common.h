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

// The sigmoid inside silu, fp32, in eleven instructions where expf and an IEEE division take
// twenty-five (silu is the default activation of two of the reference's three training scripts,
// and in the row-wise kernels it was a fifth of the forward's time).  2^t comes from the
// hardware's exp2 (1 ulp) with the product t = -u log2(e) carried in two floats, so that the
// argument's rounding (|u| 2^-24 relative otherwise) does not reach the result; the reciprocal is
// the hardware's with one Newton step.  u is clamped to +-87, where 2^t stays a normal number:
// silu's own factor u restores infinities and NaN.  Not for a sigmoid that stands alone.
__device__ __forceinline__ float sigmoid_inside_silu(float u) {
    const float uc = __builtin_amdgcn_fmed3f(u, -87.f, 87.f);
    constexpr float c_hi = -1.44269502162933349609375f;  // -float(log2 e)
    constexpr float c_lo = -1.92596298909109e-08f;      // -(log2 e - float(log2 e))
    const float hi = uc * c_hi;
    const float lo = fmaf(uc, c_lo, fmaf(uc, c_hi, -hi));  // what the product's rounding dropped
    float e = __builtin_amdgcn_exp2f(hi);
    e = fmaf(e, lo * 0.693147180559945309f, e);  // 2^(hi + lo) = 2^hi (1 + lo ln 2 + O(lo^2)), |lo| < 2^-17
    const float d = 1.f + e;
    const float r = __builtin_amdgcn_rcpf(d);
    return fmaf(fmaf(-d, r, 1.f), r, r);
}
template <typename T> __device__ __forceinline__ T silu_sigmoid(T u) { return sigmoid_stable(u); }
template <> __device__ __forceinline__ float silu_sigmoid<float>(float u) { return sigmoid_inside_silu(u); }

template <int ACT, typename T> struct Act;

// max as one instruction (a compare and a select otherwise); max(u, 0) and, for a slope below
// one, max(u, slope * u) are relu and leaky_relu for every u, signed zeros and NaN included
__device__ __forceinline__ float max_of(float a, float b) { return __builtin_fmaxf(a, b); }
__device__ __forceinline__ double max_of(double a, double b) { return __builtin_fmax(a, b); }

template <typename T> struct Act<GRIDNET_ACT_RELU, T> {
    static __device__ __forceinline__ T f(T u) { return max_of(u, T(0)); }
    static __device__ __forceinline__ void fd(T u, T &f, T &d) {
        bool pos = u > T(0);
        f = pos ? u : T(0);
        d = pos ? T(1) : T(0);
    }
};
template <typename T> struct Act<GRIDNET_ACT_LEAKY_RELU, T> {
    static __device__ __forceinline__ T f(T u) { return max_of(u, T(0.01) * u); }
    static __device__ __forceinline__ void fd(T u, T &f, T &d) {
        bool pos = u > T(0);
        f = pos ? u : T(0.01) * u;
        d = pos ? T(1) : T(0.01);
    }
};
template <typename T> struct Act<GRIDNET_ACT_SILU, T> {
    static __device__ __forceinline__ T f(T u) { return u * silu_sigmoid(u); }
    static __device__ __forceinline__ void fd(T u, T &f, T &d) {
        T s = silu_sigmoid(u);
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

// ---- device: the last step of the LayerNorm backward's two sums --------------------------
// (s1_i, s2_i), `parts` pairs of sample b -> (sum s1 / n, sum s2 / n), by one workgroup of THREADS
// threads: doubles, a fixed order.  `red` is LDS, one pair per wave.  A kernel of its own in
// layernorm.hip; also run by spare workgroups of the kernel that adds up the gradient copies.
constexpr int kFinUnroll = 4;  // pairs a thread requests before it uses any
template <int THREADS>
__device__ __forceinline__ void finalize_sums_of_sample(const float *__restrict__ part, int parts, long n,
                                                        float *__restrict__ sums, int b,
                                                        double (*red)[2]) {
    const int tid = threadIdx.x;
    const float2 *ps = reinterpret_cast<const float2 *>(part) + (long)b * parts;
    double s1 = 0.0, s2 = 0.0;
    for (int i0 = tid; i0 < parts; i0 += THREADS * kFinUnroll) {
        float2 v[kFinUnroll];
#pragma unroll
        for (int k = 0; k < kFinUnroll; ++k) {
            const int i = i0 + k * THREADS;
            v[k] = i < parts ? ps[i] : make_float2(0.f, 0.f);
        }
#pragma unroll
        for (int k = 0; k < kFinUnroll; ++k) {
            s1 += (double)v[k].x;
            s2 += (double)v[k].y;
        }
    }
    s1 = wave_sum(s1);
    s2 = wave_sum(s2);
    if ((tid & (kWave - 1)) == 0) {
        red[tid / kWave][0] = s1;
        red[tid / kWave][1] = s2;
    }
    __syncthreads();
    if (tid == 0) {
        s1 = s2 = 0.0;
        for (int w = 0; w < THREADS / kWave; ++w) {
            s1 += red[w][0];
            s2 += red[w][1];
        }
        sums[2 * b] = (float)(s1 / (double)n);
        sums[2 * b + 1] = (float)(s2 / (double)n);
    }
}

// ---- device: gathering what a block's cells send to the window around it -----------------
// In the backward of a block-local update every cell c sends weight[t][c] * delta[c] to window
// entry c + offset(t), t = 9a+3b+c' <-> offset (a-1, b-1, c'-1).  Scattering that with LDS float
// atomics is slow (ds_add_f32: the fp32 kernels took 3x as long as with this gather), so the
// one-thread-per-cell fp32 kernels publish their 27 products in a table prod[27][bs^3] and every
// window entry e sums the ones aimed at it: tap t from cell e - offset(t), where that cell exists.
// ds_add_f64 keeps up, and an fp64 table would leave room for one workgroup per CU only (measured
// 1.7x slower than the scatter), so fp64 keeps the atomics.
template <typename T> constexpr bool kGatherTaps = sizeof(T) == 4;

template <int BS> struct TapGather {
    static constexpr int S = BS + 2, W = S * S * S, NT = BS * BS * BS;
    static constexpr int kEntries = (W + NT - 1) / NT;  // window entries per thread
    static constexpr int kLinBias = (BS + 1) * BS * BS;  // halo entries have cell indices < 0

    // Descriptor of window entry idx: per axis, which of the three offsets lead back into the
    // block (bits 0-2, 3-5, 6-8), and above them the biased linear cell index of the entry.
    static __device__ __forceinline__ unsigned describe(int idx) {
        const int wk = idx % S, wj = (idx / S) % S, wi = idx / (S * S);
        unsigned bits = 0;
#pragma unroll
        for (int o = 0; o < 3; ++o) {
            const int si = wi - (o - 1), sj = wj - (o - 1), sk = wk - (o - 1);  // source, window coords
            if (si >= 1 && si <= BS) bits |= 1u << o;
            if (sj >= 1 && sj <= BS) bits |= 8u << o;
            if (sk >= 1 && sk <= BS) bits |= 64u << o;
        }
        if (idx >= W) bits = 0;
        const int lin = ((wi - 1) * BS + (wj - 1)) * BS + (wk - 1);
        return bits | ((unsigned)(lin + kLinBias) << 9);
    }

    template <typename T>
    static __device__ __forceinline__ T collect(const T *prod, unsigned desc) {
        const int lin = (int)(desc >> 9) - kLinBias;
        T acc = T(0);
#pragma unroll
        for (int a = 0; a < 3; ++a)
#pragma unroll
            for (int b = 0; b < 3; ++b)
#pragma unroll
                for (int c = 0; c < 3; ++c) {
                    const unsigned bit = (1u << a) | (8u << b) | (64u << c);
                    const bool ok = (desc & bit) == bit;
                    const int src = lin - (((a - 1) * BS + (b - 1)) * BS + (c - 1));
                    const T p = prod[(a * 9 + b * 3 + c) * NT + (ok ? src : 0)];
                    acc += ok ? p : T(0);
                }
        return acc;
    }
};

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
// The workgroup that takes this one's place when a launch walks its blocks backwards: same XCD
// (what a block's workgroups left in that XCD's L2 in the launch before stays where it is looked
// for), the XCD's workgroups in reverse order.  `grid` is a padded_grid().
__device__ __forceinline__ int reversed_on_its_xcd(int wg, int grid) {
    return wg % kXcds + kXcds * (grid / kXcds - 1 - wg / kXcds);
}
__device__ __forceinline__ bool split_block_id(int wg, int nblk, int nchunk, int &blk, int &chunk) {
    const int per_xcd = (nblk + kXcds - 1) / kXcds;
    const int xcd = wg % kXcds, slot = wg / kXcds;
    blk = xcd * per_xcd + slot / nchunk;
    chunk = slot % nchunk;
    return slot / nchunk < per_xcd && blk < nblk;
}

}  // namespace gridnet
