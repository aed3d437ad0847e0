// Per-sample LayerNorm over all grid cells with elementwise affine, forward and backward.
//
// The callers of the grid update run torch.nn.LayerNorm((M,N,K)) after every outer step
// (gridnet/scripts/train_mnist.py:54,64; gridnet/scripts/train_imagenet.py:67,86), so one
// "sample" is a whole grid: n = M*N*K cells (262 144 at 64^3), far more than a workgroup
// holds.  Each sample is therefore cut into chunks of 4096 cells, one workgroup per chunk:
//
//   forward   ln_partial_stats : per chunk (mean, M2) with M2 centred on the chunk's own mean
//             ln_apply         : every workgroup merges its sample's chunk statistics in a
//                                fixed order (exact pairwise-combination formula, no
//                                E[x^2]-mean^2 cancellation) and normalises its chunk
//   backward  ln_bwd_partial   : per chunk sum(g) and sum(g*xhat), g = dy*gamma
//             ln_bwd_apply     : every workgroup merges the chunk sums into the per-sample
//                                means; one thread owns 4 adjacent cells for ALL samples, so
//                                dgamma and dbeta are reduced over the batch in registers,
//                                without atomics and in a fixed order
//             (ln_bwd_finalize : the per-sample means as a kernel of their own, for the
//                                callers that need them as a tensor)
//
// Every reduction has a fixed order, so results are bitwise reproducible.

#include "common.h"
#include "launch.h"
#include "plan.h"

namespace gridnet {

namespace {

constexpr int kLnThreads = 256;
constexpr int kLnPerThread = 16;
constexpr int kLnChunk = kLnThreads * kLnPerThread;  // cells per workgroup

template <typename T> struct alignas(4 * sizeof(T)) Vec4 { T v[4]; };

// Load this thread's 16 cells of a chunk; cells past `n` read as `fill` and are not counted.
// Layout: 4 rounds; in a round the 256 threads read 256 consecutive groups of 4 cells.
template <typename T, bool VEC>
__device__ __forceinline__ void load_chunk(const T *p, long start, long n, int tid, T (&r)[kLnPerThread]) {
#pragma unroll
    for (int round = 0; round < 4; ++round) {
        const long at = start + ((long)round * kLnThreads + tid) * 4;
        if (VEC) {
            if (at < n) {  // n % 4 == 0: the whole group is in range
                const Vec4<T> q = *reinterpret_cast<const Vec4<T> *>(p + at);
#pragma unroll
                for (int e = 0; e < 4; ++e) r[round * 4 + e] = q.v[e];
            } else {
#pragma unroll
                for (int e = 0; e < 4; ++e) r[round * 4 + e] = T(0);
            }
        } else {
#pragma unroll
            for (int e = 0; e < 4; ++e) r[round * 4 + e] = (at + e < n) ? p[at + e] : T(0);
        }
    }
}

template <typename T, bool VEC>
__device__ __forceinline__ void store_chunk(T *p, long start, long n, int tid, const T (&r)[kLnPerThread]) {
#pragma unroll
    for (int round = 0; round < 4; ++round) {
        const long at = start + ((long)round * kLnThreads + tid) * 4;
        if (VEC) {
            if (at < n) {
                Vec4<T> q;
#pragma unroll
                for (int e = 0; e < 4; ++e) q.v[e] = r[round * 4 + e];
                *reinterpret_cast<Vec4<T> *>(p + at) = q;
            }
        } else {
#pragma unroll
            for (int e = 0; e < 4; ++e)
                if (at + e < n) p[at + e] = r[round * 4 + e];
        }
    }
}

__device__ __forceinline__ bool cell_valid(long start, long n, int tid, int i) {
    return start + ((long)(i / 4) * kLnThreads + tid) * 4 + (i % 4) < n;
}

template <typename T, bool VEC>
__global__ __launch_bounds__(kLnThreads) void ln_partial_stats(const T *__restrict__ x,
                                                               T *__restrict__ partial, long n,
                                                               int nchunk) {
    __shared__ T red[kLnThreads / kWave];
    const int tid = threadIdx.x, chunk = blockIdx.x, b = blockIdx.y;
    const long start = (long)chunk * kLnChunk;
    const long count = min((long)kLnChunk, n - start);
    T r[kLnPerThread];
    load_chunk<T, VEC>(x + (long)b * n, start, n, tid, r);
    T s = T(0);
#pragma unroll
    for (int i = 0; i < kLnPerThread; ++i) s += r[i];  // out-of-range cells hold 0
    const T mean = block_sum(s, red, tid, kLnThreads) / T(count);
    T q = T(0);
#pragma unroll
    for (int i = 0; i < kLnPerThread; ++i) {
        const T d = r[i] - mean;
        q += cell_valid(start, n, tid, i) ? d * d : T(0);
    }
    const T m2 = block_sum(q, red, tid, kLnThreads);
    if (tid == 0) {
        partial[((long)b * nchunk + chunk) * 2 + 0] = mean;
        partial[((long)b * nchunk + chunk) * 2 + 1] = m2;
    }
}

template <typename T, bool VEC>
__global__ __launch_bounds__(kLnThreads) void ln_apply(const T *__restrict__ x,
                                                       const T *__restrict__ gamma,
                                                       const T *__restrict__ beta,
                                                       const T *__restrict__ partial,
                                                       T *__restrict__ y, T *__restrict__ mean_out,
                                                       T *__restrict__ rstd_out, long n, int nchunk,
                                                       T eps) {
    __shared__ T red[kLnThreads / kWave];
    const int tid = threadIdx.x, chunk = blockIdx.x, b = blockIdx.y;
    const T *ps = partial + (long)b * nchunk * 2;
    // merge the chunk statistics of this sample: mean = sum(c_i m_i)/n,
    // M2 = sum(M2_i + c_i (m_i - mean)^2)
    T s = T(0);
    for (int c = tid; c < nchunk; c += kLnThreads) {
        const long cnt = min((long)kLnChunk, n - (long)c * kLnChunk);
        s += T(cnt) * ps[c * 2];
    }
    const T mean = block_sum(s, red, tid, kLnThreads) / T(n);
    T q = T(0);
    for (int c = tid; c < nchunk; c += kLnThreads) {
        const long cnt = min((long)kLnChunk, n - (long)c * kLnChunk);
        const T d = ps[c * 2] - mean;
        q += ps[c * 2 + 1] + T(cnt) * d * d;
    }
    const T var = block_sum(q, red, tid, kLnThreads) / T(n);
    const T rstd = T(1) / sqrt(var + eps);
    if (chunk == 0 && tid == 0) {
        mean_out[b] = mean;
        rstd_out[b] = rstd;
    }
    const long start = (long)chunk * kLnChunk;
    T r[kLnPerThread], gm[kLnPerThread], bt[kLnPerThread];
    load_chunk<T, VEC>(x + (long)b * n, start, n, tid, r);
    load_chunk<T, VEC>(gamma, start, n, tid, gm);
    load_chunk<T, VEC>(beta, start, n, tid, bt);
#pragma unroll
    for (int i = 0; i < kLnPerThread; ++i) r[i] = (r[i] - mean) * rstd * gm[i] + bt[i];
    store_chunk<T, VEC>(y + (long)b * n, start, n, tid, r);
}

template <typename T, bool VEC>
__global__ __launch_bounds__(kLnThreads) void ln_bwd_partial(const T *__restrict__ dy,
                                                             const T *__restrict__ x,
                                                             const T *__restrict__ gamma,
                                                             const T *__restrict__ mean,
                                                             const T *__restrict__ rstd,
                                                             T *__restrict__ partial, long n,
                                                             int nchunk, int stat_stride) {
    __shared__ T red[kLnThreads / kWave];
    const int tid = threadIdx.x, chunk = blockIdx.x, b = blockIdx.y;
    const long start = (long)chunk * kLnChunk;
    const T mu = mean[b * stat_stride], rs = rstd[b * stat_stride];
    T g[kLnPerThread], xv[kLnPerThread], gm[kLnPerThread];
    load_chunk<T, VEC>(dy + (long)b * n, start, n, tid, g);
    load_chunk<T, VEC>(x + (long)b * n, start, n, tid, xv);
    load_chunk<T, VEC>(gamma, start, n, tid, gm);
    T s1 = T(0), s2 = T(0);
#pragma unroll
    for (int i = 0; i < kLnPerThread; ++i) {
        const T gi = g[i] * gm[i];  // out-of-range cells: dy = 0 -> no contribution
        s1 += gi;
        s2 += gi * ((xv[i] - mu) * rs);
    }
    s1 = block_sum(s1, red, tid, kLnThreads);
    s2 = block_sum(s2, red, tid, kLnThreads);
    if (tid == 0) {
        partial[((long)b * nchunk + chunk) * 2 + 0] = s1;
        partial[((long)b * nchunk + chunk) * 2 + 1] = s2;
    }
}

template <typename T>
__global__ __launch_bounds__(kLnThreads) void ln_bwd_finalize(const T *__restrict__ partial,
                                                              T *__restrict__ sample_means, long n,
                                                              int nchunk) {
    __shared__ T red[kLnThreads / kWave];
    const int tid = threadIdx.x, b = blockIdx.x;
    const T *ps = partial + (long)b * nchunk * 2;
    T s1 = T(0), s2 = T(0);
    for (int c = tid; c < nchunk; c += kLnThreads) {
        s1 += ps[c * 2];
        s2 += ps[c * 2 + 1];
    }
    s1 = block_sum(s1, red, tid, kLnThreads);
    s2 = block_sum(s2, red, tid, kLnThreads);
    if (tid == 0) {
        sample_means[b * 2 + 0] = s1 / T(n);
        sample_means[b * 2 + 1] = s2 / T(n);
    }
}

// The per-sample means of the two sums are formed here, by every workgroup for itself, from the
// chunk partials (8 lanes per sample, fixed order): B * nchunk pairs are little to read next to
// the B * 1024 * VEC cells a workgroup streams, and a kernel of its own for it costs more in
// launch and drain than it computes.  Samples are handled kLnSumBatch at a time.
constexpr int kLnSumBatch = kLnThreads / 8;

template <typename T, int VEC, bool ACCUM>
__global__ __launch_bounds__(kLnThreads) void ln_bwd_apply(
    const T *__restrict__ dy, const T *__restrict__ x, const T *__restrict__ gamma,
    const T *__restrict__ mean, const T *__restrict__ rstd, const T *__restrict__ partial,
    int nchunk, T *__restrict__ dx, T *__restrict__ dgamma, T *__restrict__ dbeta, int B, long n) {
    __shared__ T sample_means[kLnSumBatch * 2];
    const long at = ((long)blockIdx.x * kLnThreads + threadIdx.x) * VEC;
    const bool live = at < n;
    T gm[VEC], dg[VEC], dbt[VEC];
#pragma unroll
    for (int e = 0; e < VEC; ++e) {
        gm[e] = live ? gamma[at + e] : T(0);
        dg[e] = T(0);
        dbt[e] = T(0);
    }
    struct alignas(sizeof(T) * VEC) Pack { T v[VEC]; };
    for (int b0 = 0; b0 < B; b0 += kLnSumBatch) {
        {   // means of the next kLnSumBatch samples: lane group of 8 per sample
            const int sb = b0 + threadIdx.x / 8, part = threadIdx.x % 8;
            T s1 = T(0), s2 = T(0);
            if (sb < B)
                for (int c = part; c < nchunk; c += 8) {
                    s1 += partial[((long)sb * nchunk + c) * 2];
                    s2 += partial[((long)sb * nchunk + c) * 2 + 1];
                }
#pragma unroll
            for (int off = 4; off > 0; off >>= 1) {
                s1 += __shfl_xor(s1, off, 8);
                s2 += __shfl_xor(s2, off, 8);
            }
            __syncthreads();  // the previous batch's values are no longer read
            if (part == 0) {
                sample_means[(threadIdx.x / 8) * 2] = s1 / T(n);
                sample_means[(threadIdx.x / 8) * 2 + 1] = s2 / T(n);
            }
            __syncthreads();
        }
        if (!live) continue;
        const int bend = min(B, b0 + kLnSumBatch);
#pragma unroll 4
        for (int b = b0; b < bend; ++b) {
            const T mu = mean[b], rs = rstd[b];
            const T c1 = sample_means[(b - b0) * 2], c2 = sample_means[(b - b0) * 2 + 1];
            const Pack d = *reinterpret_cast<const Pack *>(dy + (long)b * n + at);
            const Pack xv = *reinterpret_cast<const Pack *>(x + (long)b * n + at);
            Pack o;
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                const T xh = (xv.v[e] - mu) * rs;
                dg[e] += d.v[e] * xh;
                dbt[e] += d.v[e];
                o.v[e] = rs * (d.v[e] * gm[e] - c1 - xh * c2);
            }
            *reinterpret_cast<Pack *>(dx + (long)b * n + at) = o;
        }
    }
    if (!live) return;
#pragma unroll
    for (int e = 0; e < VEC; ++e) {
        if (ACCUM) {
            dgamma[at + e] += dg[e];
            dbeta[at + e] += dbt[e];
        } else {
            dgamma[at + e] = dg[e];
            dbeta[at + e] = dbt[e];
        }
    }
}

// ---- pieces of the LayerNorm folded into the step kernels (fp32) ---------------------------
// The step kernels leave per-group partial results; these small kernels turn them into the
// per-sample numbers, in double and in a fixed order (one workgroup per sample).

// workgroup size: as few waves as request every pair in one round (fewer waves start sooner and
// leave a shorter last loop), up to the largest workgroup
inline int finalize_threads(int parts) {
    const int t = (parts + kFinUnroll - 1) / kFinUnroll;
    return t <= 256 ? 256 : t <= 512 ? 512 : 1024;
}

// (mean_i, M2_i) over `count` cells each -> (mean, rstd): mean = avg(mean_i),
// M2 = sum(M2_i + count (mean_i - mean)^2)  (exact pairwise-combination formula).
template <int THREADS>
__global__ __launch_bounds__(THREADS) void ln_finalize_stats(const float *__restrict__ part,
                                                                 int parts, int count,
                                                                 float *__restrict__ stats, double eps) {
    __shared__ double red[THREADS / kWave][3];
    const int tid = threadIdx.x, b = blockIdx.x;
    const float2 *ps = reinterpret_cast<const float2 *>(part) + (long)b * parts;
    double s = 0.0, q = 0.0, qm = 0.0;
    // one pass: sum(mean_i), sum(M2_i), sum(mean_i^2); means are O(1) and few thousand, so the
    // squares lose nothing in double
    for (int i0 = tid; i0 < parts; i0 += THREADS * kFinUnroll) {
        float2 v[kFinUnroll];
#pragma unroll
        for (int k = 0; k < kFinUnroll; ++k) {
            const int i = i0 + k * THREADS;
            v[k] = i < parts ? ps[i] : make_float2(0.f, 0.f);
        }
#pragma unroll
        for (int k = 0; k < kFinUnroll; ++k) {
            s += (double)v[k].x;
            q += (double)v[k].y;
            qm += (double)v[k].x * (double)v[k].x;
        }
    }
    // the three sums cross the workgroup together: one trip through LDS, one barrier
    s = wave_sum(s);
    q = wave_sum(q);
    qm = wave_sum(qm);
    if ((tid & (kWave - 1)) == 0) {
        red[tid / kWave][0] = s;
        red[tid / kWave][1] = q;
        red[tid / kWave][2] = qm;
    }
    __syncthreads();
    if (tid == 0) {
        s = q = qm = 0.0;
        for (int w = 0; w < THREADS / kWave; ++w) {
            s += red[w][0];
            q += red[w][1];
            qm += red[w][2];
        }
        const double mean = s / parts;
        // sum count (mean_i - mean)^2 = count (sum mean_i^2 - parts mean^2)
        const double var = (q + count * (qm - parts * mean * mean)) / ((double)parts * count);
        stats[2 * b] = (float)mean;
        stats[2 * b + 1] = (float)(1.0 / sqrt((var > 0.0 ? var : 0.0) + eps));
    }
}

// (s1_i, s2_i) -> (sum s1 / n, sum s2 / n)
template <int THREADS>
__global__ __launch_bounds__(THREADS) void ln_finalize_sums(const float *__restrict__ part,
                                                                int parts, long n,
                                                                float *__restrict__ sums) {
    __shared__ double red[THREADS / kWave][2];
    finalize_sums_of_sample<THREADS>(part, parts, n, sums, blockIdx.x, red);
}

// y = (x - mean) * rstd * gamma + beta with statistics that are already known
template <bool VEC>
__global__ __launch_bounds__(kLnThreads) void ln_apply_stats(const float *__restrict__ x,
                                                             const float *__restrict__ stats,
                                                             const float *__restrict__ gamma,
                                                             const float *__restrict__ beta,
                                                             float *__restrict__ y, long n) {
    const int tid = threadIdx.x, chunk = blockIdx.x, b = blockIdx.y;
    const float mean = stats[2 * b], rstd = stats[2 * b + 1];
    const long start = (long)chunk * kLnChunk;
    float r[kLnPerThread], gm[kLnPerThread], bt[kLnPerThread];
    load_chunk<float, VEC>(x + (long)b * n, start, n, tid, r);
    load_chunk<float, VEC>(gamma, start, n, tid, gm);
    load_chunk<float, VEC>(beta, start, n, tid, bt);
#pragma unroll
    for (int i = 0; i < kLnPerThread; ++i) r[i] = (r[i] - mean) * rstd * gm[i] + bt[i];
    store_chunk<float, VEC>(y + (long)b * n, start, n, tid, r);
}

inline int chunks_of(long n) { return (int)((n + kLnChunk - 1) / kLnChunk); }

template <typename T> bool aligned4(const void *p) { return ((uintptr_t)p % (4 * sizeof(T))) == 0; }

template <typename T> int forward_t(const LayerNormArgs &a, hipStream_t st) {
    const int nchunk = chunks_of(a.n);
    T *partial = (T *)a.workspace;
    const bool vec = a.n % 4 == 0 && aligned4<T>(a.x) && aligned4<T>(a.y) && aligned4<T>(a.gamma) &&
                     aligned4<T>(a.beta);
    dim3 grid(nchunk, a.B), block(kLnThreads);
    if (vec) {
        hipLaunchKernelGGL((ln_partial_stats<T, true>), grid, block, 0, st, (const T *)a.x, partial,
                           a.n, nchunk);
        hipLaunchKernelGGL((ln_apply<T, true>), grid, block, 0, st, (const T *)a.x,
                           (const T *)a.gamma, (const T *)a.beta, partial, (T *)a.y, (T *)a.mean,
                           (T *)a.rstd, a.n, nchunk, (T)a.eps);
    } else {
        hipLaunchKernelGGL((ln_partial_stats<T, false>), grid, block, 0, st, (const T *)a.x, partial,
                           a.n, nchunk);
        hipLaunchKernelGGL((ln_apply<T, false>), grid, block, 0, st, (const T *)a.x,
                           (const T *)a.gamma, (const T *)a.beta, partial, (T *)a.y, (T *)a.mean,
                           (T *)a.rstd, a.n, nchunk, (T)a.eps);
    }
    return check_launch("layernorm_forward");
}

template <typename T> int backward_t(const LayerNormArgs &a, hipStream_t st) {
    const int nchunk = chunks_of(a.n);
    T *partial = (T *)a.workspace;
    const bool vec = a.n % 4 == 0 && aligned4<T>(a.x) && aligned4<T>(a.dy) && aligned4<T>(a.gamma) &&
                     aligned4<T>(a.dx);
    const bool accum = (a.flags & GRIDNET_OVERWRITE_PARAMS) == 0;
    dim3 grid(nchunk, a.B), block(kLnThreads);
    if (vec)
        hipLaunchKernelGGL((ln_bwd_partial<T, true>), grid, block, 0, st, (const T *)a.dy,
                           (const T *)a.x, (const T *)a.gamma, (const T *)a.mean_in,
                           (const T *)a.rstd_in, partial, a.n, nchunk, 1);
    else
        hipLaunchKernelGGL((ln_bwd_partial<T, false>), grid, block, 0, st, (const T *)a.dy,
                           (const T *)a.x, (const T *)a.gamma, (const T *)a.mean_in,
                           (const T *)a.rstd_in, partial, a.n, nchunk, 1);
#define GRIDNET_LN_APPLY(V, ACC)                                                                   \
    hipLaunchKernelGGL((ln_bwd_apply<T, V, ACC>),                                                  \
                       dim3((unsigned)((a.n + (long)kLnThreads * V - 1) / ((long)kLnThreads * V))), \
                       block, 0, st, (const T *)a.dy, (const T *)a.x, (const T *)a.gamma,          \
                       (const T *)a.mean_in, (const T *)a.rstd_in, partial, nchunk, (T *)a.dx,     \
                       (T *)a.dgamma, (T *)a.dbeta, a.B, a.n)
    // A thread owns its cells for the whole batch, so the grid is n / (256 x cells per thread)
    // workgroups whatever the batch: with four cells per thread a 32^3 grid is 32 of them (100 us
    // at batch 256, 35 us with one cell per thread) and a 64^3 grid 256 (batch 128: 100 against
    // 66 us; batch 32: 20 us either way).  Below two workgroups per CU a thread takes one cell:
    // four times the workgroups, the same bits.
    const bool wide = vec && a.n / (4L * kLnThreads) >= 2L * plan_device_cus();
    if (wide) {
        if (accum) GRIDNET_LN_APPLY(4, true); else GRIDNET_LN_APPLY(4, false);
    } else {
        if (accum) GRIDNET_LN_APPLY(1, true); else GRIDNET_LN_APPLY(1, false);
    }
#undef GRIDNET_LN_APPLY
    return check_launch("layernorm_backward");
}

}  // namespace

int layernorm_finalize_stats(const float *part, int parts_per_sample, int count, float *stats, int B,
                             double eps, hipStream_t st) {
    switch (finalize_threads(parts_per_sample)) {
    case 256:
        hipLaunchKernelGGL(ln_finalize_stats<256>, dim3(B), dim3(256), 0, st, part, parts_per_sample, count,
                           stats, eps);
        break;
    case 512:
        hipLaunchKernelGGL(ln_finalize_stats<512>, dim3(B), dim3(512), 0, st, part, parts_per_sample, count,
                           stats, eps);
        break;
    default:
        hipLaunchKernelGGL(ln_finalize_stats<1024>, dim3(B), dim3(1024), 0, st, part, parts_per_sample, count,
                           stats, eps);
    }
    return check_launch("ln_finalize_stats");
}

int layernorm_finalize_sums(const float *part, int parts_per_sample, long n, float *sums, int B,
                            hipStream_t st) {
    switch (finalize_threads(parts_per_sample)) {
    case 256:
        hipLaunchKernelGGL(ln_finalize_sums<256>, dim3(B), dim3(256), 0, st, part, parts_per_sample, n, sums);
        break;
    case 512:
        hipLaunchKernelGGL(ln_finalize_sums<512>, dim3(B), dim3(512), 0, st, part, parts_per_sample, n, sums);
        break;
    default:
        hipLaunchKernelGGL(ln_finalize_sums<1024>, dim3(B), dim3(1024), 0, st, part, parts_per_sample, n, sums);
    }
    return check_launch("ln_finalize_sums");
}

int layernorm_apply_stats(const float *x, const float *stats, const float *gamma, const float *beta,
                          float *y, int B, long n, hipStream_t st) {
    const bool vec = n % 4 == 0 && aligned4<float>(x) && aligned4<float>(y) &&
                     aligned4<float>(gamma) && aligned4<float>(beta);
    dim3 grid(chunks_of(n), B), block(kLnThreads);
    if (vec) hipLaunchKernelGGL((ln_apply_stats<true>), grid, block, 0, st, x, stats, gamma, beta, y, n);
    else hipLaunchKernelGGL((ln_apply_stats<false>), grid, block, 0, st, x, stats, gamma, beta, y, n);
    return check_launch("ln_apply_stats");
}

int layernorm_backward_sums(const float *dy, const float *x, const float *stats, const float *gamma,
                            float *sums, int B, long n, float *partial, hipStream_t st) {
    const int nchunk = chunks_of(n);
    const bool vec = n % 4 == 0 && aligned4<float>(x) && aligned4<float>(dy) && aligned4<float>(gamma);
    dim3 grid(nchunk, B), block(kLnThreads);
    if (vec)
        hipLaunchKernelGGL((ln_bwd_partial<float, true>), grid, block, 0, st, dy, x, gamma, stats,
                           stats + 1, partial, n, nchunk, 2);
    else
        hipLaunchKernelGGL((ln_bwd_partial<float, false>), grid, block, 0, st, dy, x, gamma, stats,
                           stats + 1, partial, n, nchunk, 2);
    hipLaunchKernelGGL((ln_bwd_finalize<float>), dim3(B), block, 0, st, (const float *)partial, sums, n,
                       nchunk);
    return check_launch("layernorm_backward_sums");
}

size_t layernorm_workspace(int dtype, int B, long n) {
    const size_t elt = dtype == GRIDNET_F64 ? 8 : 4;
    return ((size_t)B * chunks_of(n) * 2 + (size_t)B * 2) * elt;
}

int layernorm_forward(const LayerNormArgs &a, hipStream_t st) {
    return a.dtype == GRIDNET_F64 ? forward_t<double>(a, st) : forward_t<float>(a, st);
}

int layernorm_backward(const LayerNormArgs &a, hipStream_t st) {
    return a.dtype == GRIDNET_F64 ? backward_t<double>(a, st) : backward_t<float>(a, st);
}

}  // namespace gridnet
