// Gated variant of the block-local update: x' = gate * x + (1 - gate) * act(pre) with
// pre = b[0] + sum_t W[t,0] x_nbr and gate = sigmoid(b[1] + sum_t W[t,1] x_nbr)
// (gridnet/backend_torch.py:145-267; the reference's kernels: src/gridnet_cuda_kernels.cu:452-734).
// Weight layout [27, 2, M, N, K], bias [2, M, N, K].  One thread per cell, fp32/fp64.
// Coverage path: same decomposition as the generic plain kernels (one workgroup per spatial
// block walks a chunk of the batch with both 27-tap weight sets in registers).

#include "common.h"
#include "launch.h"

namespace gridnet {

namespace {

template <int BS> struct GGeo {
    static constexpr int S = BS + 2, W = S * S * S, NT = BS * BS * BS;
};

template <typename T, int BS>
__device__ __forceinline__ void gated_load_window(T *win, const T *xs, int p0, int q0, int r0, int M,
                                                  int N, int K, int tid) {
    using G = GGeo<BS>;
    for (int idx = tid; idx < G::W; idx += G::NT) {
        const int wk = idx % G::S, wj = (idx / G::S) % G::S, wi = idx / (G::S * G::S);
        const int gi = p0 + wi - 1, gj = q0 + wj - 1, gk = r0 + wk - 1;
        T v = T(0);
        if (gi >= 0 && gi < M && gj >= 0 && gj < N && gk >= 0 && gk < K)
            v = xs[((long)gi * N + gj) * K + gk];
        win[idx] = v;
    }
}

template <typename T, int BS>
__device__ __forceinline__ void two_dots(const T *win, int base, const T (&wa)[27], const T (&wg)[27],
                                         T ba, T bg, T &pre, T &gpre) {
    using G = GGeo<BS>;
    pre = ba;
    gpre = bg;
#pragma unroll
    for (int a = 0; a < 3; ++a)
#pragma unroll
        for (int b = 0; b < 3; ++b)
#pragma unroll
            for (int c = 0; c < 3; ++c) {
                const T v = win[base + (a * G::S + b) * G::S + c];
                pre += wa[a * 9 + b * 3 + c] * v;
                gpre += wg[a * 9 + b * 3 + c] * v;
            }
}

template <typename T, int BS, int ACT>
__global__ __launch_bounds__(BS *BS *BS) void gated_fwd(const T *__restrict__ weight,
                                                        const T *__restrict__ bias,
                                                        const T *__restrict__ x, T *__restrict__ y,
                                                        int B, int M, int N, int K, int inner,
                                                        int nblk, int nchunk, int chunk_len) {
    using G = GGeo<BS>;
    __shared__ T win[G::W];
    const int tid = threadIdx.x;
    int blk, chunk;
    if (!split_block_id(blockIdx.x, nblk, nchunk, blk, chunk)) return;
    const int kb = K / BS, nb = N / BS;
    const int p0 = (blk / (kb * nb)) * BS, q0 = ((blk / kb) % nb) * BS, r0 = (blk % kb) * BS;
    const int ci = tid / (BS * BS), cj = (tid / BS) % BS, ck = tid % BS;
    const long cells = (long)M * N * K;
    const long gc = ((long)(p0 + ci) * N + (q0 + cj)) * K + (r0 + ck);
    const int base = (ci * G::S + cj) * G::S + ck;
    const int centre = base + (G::S + 1) * G::S + 1;
    T wa[27], wg[27];
#pragma unroll
    for (int t = 0; t < 27; ++t) {
        wa[t] = weight[(t * 2 + 0) * cells + gc];
        wg[t] = weight[(t * 2 + 1) * cells + gc];
    }
    const T ba = bias[gc], bg = bias[cells + gc];
    const int s_end = min(B, (chunk + 1) * chunk_len);
    for (int s = chunk * chunk_len; s < s_end; ++s) {
        gated_load_window<T, BS>(win, x + s * cells, p0, q0, r0, M, N, K, tid);
        __syncthreads();
        T cur = win[centre];
        for (int it = 0; it < inner; ++it) {
            T pre, gpre;
            two_dots<T, BS>(win, base, wa, wg, ba, bg, pre, gpre);
            const T gate = sigmoid_stable(gpre);
            cur = gate * cur + (T(1) - gate) * Act<ACT, T>::f(pre);
            __syncthreads();
            win[centre] = cur;
            __syncthreads();
        }
        y[s * cells + gc] = cur;
        __syncthreads();
    }
}

template <typename T, int BS, int ACT>
__global__ __launch_bounds__(BS *BS *BS) void gated_bwd(
    const T *__restrict__ weight, const T *__restrict__ bias, const T *__restrict__ x,
    const T *__restrict__ dy, T *__restrict__ dweight, T *__restrict__ dbias, T *__restrict__ dx,
    int B, int M, int N, int K, int inner, int nblk, int nchunk, int chunk_len, int param_mode) {
    using G = GGeo<BS>;
    __shared__ T win[G::W];   // window state x_i
    __shared__ T gwin[G::W];  // dL/d(window); the owned entry is rewritten every iteration
    // fp32: the cells' 27 products, gathered by the window entries instead of LDS float atomics
    using Gather = TapGather<BS>;
    __shared__ T prod[kGatherTaps<T> ? 27 * G::NT : 1];
    const int tid = threadIdx.x;
    int blk, chunk;
    if (!split_block_id(blockIdx.x, nblk, nchunk, blk, chunk)) return;
    unsigned entry[Gather::kEntries];  // the window entries this thread gathers for
#pragma unroll
    for (int e = 0; e < Gather::kEntries; ++e) entry[e] = Gather::describe(tid + e * G::NT);
    const int kb = K / BS, nb = N / BS;
    const int p0 = (blk / (kb * nb)) * BS, q0 = ((blk / kb) % nb) * BS, r0 = (blk % kb) * BS;
    const int ci = tid / (BS * BS), cj = (tid / BS) % BS, ck = tid % BS;
    const long cells = (long)M * N * K;
    const long gc = ((long)(p0 + ci) * N + (q0 + cj)) * K + (r0 + ck);
    const int base = (ci * G::S + cj) * G::S + ck;
    const int centre = base + (G::S + 1) * G::S + 1;
    T wa[27], wg[27], dwa[27], dwg[27];
#pragma unroll
    for (int t = 0; t < 27; ++t) {
        wa[t] = weight[(t * 2 + 0) * cells + gc];
        wg[t] = weight[(t * 2 + 1) * cells + gc];
        dwa[t] = dwg[t] = T(0);
    }
    const T ba = bias[gc], bg = bias[cells + gc];
    T dba = T(0), dbg = T(0);
    T hist[kMaxBackwardIters];
    const int s_end = min(B, (chunk + 1) * chunk_len);
    for (int s = chunk * chunk_len; s < s_end; ++s) {
        gated_load_window<T, BS>(win, x + s * cells, p0, q0, r0, M, N, K, tid);
        for (int idx = tid; idx < G::W; idx += G::NT) gwin[idx] = T(0);
        __syncthreads();
        T cur = win[centre];
        for (int it = 0; it < inner; ++it) {
            hist[it] = cur;
            T pre, gpre;
            two_dots<T, BS>(win, base, wa, wg, ba, bg, pre, gpre);
            const T gate = sigmoid_stable(gpre);
            cur = gate * cur + (T(1) - gate) * Act<ACT, T>::f(pre);
            __syncthreads();
            win[centre] = cur;
            __syncthreads();
        }
        T g = dy[s * cells + gc];  // dL/d(x_{i+1}) of the owned cell
        for (int it = inner - 1; it >= 0; --it) {
            win[centre] = hist[it];
            __syncthreads();
            T pre, gpre;
            two_dots<T, BS>(win, base, wa, wg, ba, bg, pre, gpre);
            const T gate = sigmoid_stable(gpre);
            T f, d;
            Act<ACT, T>::fd(pre, f, d);
            const T dpre = g * (T(1) - gate) * d;
            const T dgpre = g * (hist[it] - f) * gate * (T(1) - gate);
            dba += dpre;
            dbg += dgpre;
            // the owned cell's gradient restarts from the direct path gate * g; whatever the
            // neighbours (and this cell's own centre tap) add below accumulates on top
            gwin[centre] = gate * g;
            __syncthreads();
#pragma unroll
            for (int a = 0; a < 3; ++a)
#pragma unroll
                for (int b = 0; b < 3; ++b)
#pragma unroll
                    for (int c = 0; c < 3; ++c) {
                        const int o = base + (a * G::S + b) * G::S + c;
                        const int t = a * 9 + b * 3 + c;
                        const T v = win[o];
                        dwa[t] += v * dpre;
                        dwg[t] += v * dgpre;
                        const T sent = wa[t] * dpre + wg[t] * dgpre;
                        if (kGatherTaps<T>) prod[t * G::NT + tid] = sent;
                        else atomicAdd(&gwin[o], sent);
                    }
            __syncthreads();
            if (kGatherTaps<T>) {
#pragma unroll
                for (int e = 0; e < Gather::kEntries; ++e) {
                    const int idx = tid + e * G::NT;
                    const T acc = Gather::collect(prod, entry[e]);
                    if (idx < G::W) gwin[idx] += acc;
                }
                __syncthreads();
            }
            g = gwin[centre];
        }
        if (inner == 0) gwin[centre] = g;
        __syncthreads();
        T *dxs = dx + s * cells;
        for (int idx = tid; idx < G::W; idx += G::NT) {
            const int wk = idx % G::S, wj = (idx / G::S) % G::S, wi = idx / (G::S * G::S);
            const int gi = p0 + wi - 1, gj = q0 + wj - 1, gk = r0 + wk - 1;
            if (gi >= 0 && gi < M && gj >= 0 && gj < N && gk >= 0 && gk < K)
                unsafeAtomicAdd(&dxs[((long)gi * N + gj) * K + gk], gwin[idx]);
        }
        __syncthreads();
    }
    auto commit = [&](T *p, T v) {
        if (param_mode == kParamStore) *p = v;
        else if (param_mode == kParamAddExclusive) *p += v;
        else unsafeAtomicAdd(p, v);
    };
#pragma unroll
    for (int t = 0; t < 27; ++t) {
        commit(dweight + (t * 2 + 0) * cells + gc, dwa[t]);
        commit(dweight + (t * 2 + 1) * cells + gc, dwg[t]);
    }
    commit(dbias + gc, dba);
    commit(dbias + cells + gc, dbg);
}

template <typename T> __global__ void gated_fill_zero(T *p, long n) {
    long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    const long stride = (long)gridDim.x * blockDim.x;
    for (; i < n; i += stride) p[i] = T(0);
}

template <typename T> int zero(T *p, long n, hipStream_t st) {
    long blocks = (n + 255) / 256;
    if (blocks > 4096) blocks = 4096;
    hipLaunchKernelGGL(gated_fill_zero<T>, dim3((unsigned)blocks), dim3(256), 0, st, p, n);
    return check_launch("fill_zero");
}

template <typename T, int BS, int ACT> int run_act(const StepArgs &a, bool bwd, hipStream_t st) {
    const int nblk = (a.M / BS) * (a.N / BS) * (a.K / BS);
    int nchunk = (1024 + nblk - 1) / nblk;
    if (nchunk > a.B) nchunk = a.B;
    if (nchunk < 1) nchunk = 1;
    const int chunk_len = (a.B + nchunk - 1) / nchunk;
    nchunk = (a.B + chunk_len - 1) / chunk_len;
    dim3 grid(padded_grid(nblk, nchunk)), block(GGeo<BS>::NT);
    if (!bwd) {
        hipLaunchKernelGGL((gated_fwd<T, BS, ACT>), grid, block, 0, st, (const T *)a.weight,
                           (const T *)a.bias, (const T *)a.x, (T *)a.y, a.B, a.M, a.N, a.K, a.inner,
                           nblk, nchunk, chunk_len);
        return check_launch("gated_fwd");
    }
    const long cells = (long)a.M * a.N * a.K;
    const bool new_params = (a.flags & GRIDNET_OVERWRITE_PARAMS) != 0;
    if (a.flags & GRIDNET_OVERWRITE_DX)
        if (int rc = zero((T *)a.dx, (long)a.B * cells, st)) return rc;
    int mode = kParamAtomic;
    if (nchunk == 1) {
        mode = new_params ? kParamStore : kParamAddExclusive;
    } else if (new_params) {
        if (int rc = zero((T *)a.dweight, 54 * cells, st)) return rc;
        if (int rc = zero((T *)a.dbias, 2 * cells, st)) return rc;
    }
    hipLaunchKernelGGL((gated_bwd<T, BS, ACT>), grid, block, 0, st, (const T *)a.weight,
                       (const T *)a.bias, (const T *)a.x, (const T *)a.dy, (T *)a.dweight,
                       (T *)a.dbias, (T *)a.dx, a.B, a.M, a.N, a.K, a.inner, nblk, nchunk, chunk_len,
                       mode);
    return check_launch("gated_bwd");
}

template <typename T, int BS> int run_bs(const StepArgs &a, bool bwd, hipStream_t st) {
    switch (a.activation) {
        case GRIDNET_ACT_RELU: return run_act<T, BS, GRIDNET_ACT_RELU>(a, bwd, st);
        case GRIDNET_ACT_LEAKY_RELU: return run_act<T, BS, GRIDNET_ACT_LEAKY_RELU>(a, bwd, st);
        case GRIDNET_ACT_SILU: return run_act<T, BS, GRIDNET_ACT_SILU>(a, bwd, st);
        case GRIDNET_ACT_TANH: return run_act<T, BS, GRIDNET_ACT_TANH>(a, bwd, st);
    }
    return fail(GRIDNET_ERR_ACTIVATION, "unknown activation function: id %d", a.activation);
}

template <typename T> int run_t(const StepArgs &a, bool bwd, hipStream_t st) {
    return a.block_size == 8 ? run_bs<T, 8>(a, bwd, st) : run_bs<T, 4>(a, bwd, st);
}

}  // namespace

int gated_forward(const StepArgs &a, hipStream_t st) {
    return a.dtype == GRIDNET_F64 ? run_t<double>(a, false, st) : run_t<float>(a, false, st);
}
int gated_backward(const StepArgs &a, hipStream_t st) {
    return a.dtype == GRIDNET_F64 ? run_t<double>(a, true, st) : run_t<float>(a, true, st);
}

}  // namespace gridnet
