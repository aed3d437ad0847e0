// Generic block-local update kernels: one thread per cell, any dtype (fp32/fp64), any
// activation, optional per-window normalisation, up to 32 inner iterations in backward.
// This is the coverage path (fp64, and fp32 problems the tuned kernels decline); the tuned fp32
// kernels are separate (step_fast.hip).
//
// Work decomposition: one workgroup owns one spatial block (bs^3 threads) and walks a chunk
// of batch elements with the block's 27 weights, bias and scale held in registers, so the
// parameters are fetched once per chunk instead of once per batch element.
//
// Semantics follow gridnet/backend_torch.py:61-142 (forward) and autograd of it (backward);
// the reference evaluates the same recurrences in src/gridnet_cuda_kernels.cu:101-450.

#include "common.h"
#include "launch.h"

namespace gridnet {

namespace {

template <int BS> struct Geo {
    static constexpr int S = BS + 2;          // window side
    static constexpr int W = S * S * S;       // window entries
    static constexpr int NT = BS * BS * BS;   // threads = cells
};

// Copy the (bs+2)^3 window of batch element `xs` around block origin (p0,q0,r0) into LDS;
// entries outside the grid are zero (gridnet/backend_torch.py:63).
template <typename T, int BS>
__device__ __forceinline__ void load_window(T *win, const T *xs, int p0, int q0, int r0, int M,
                                            int N, int K, int tid) {
    using G = Geo<BS>;
    for (int idx = tid; idx < G::W; idx += G::NT) {
        const int wk = idx % G::S, wj = (idx / G::S) % G::S, wi = idx / (G::S * G::S);
        const int gi = p0 + wi - 1, gj = q0 + wj - 1, gk = r0 + wk - 1;
        T v = T(0);
        if (gi >= 0 && gi < M && gj >= 0 && gj < N && gk >= 0 && gk < K)
            v = xs[((long)gi * N + gj) * K + gk];
        win[idx] = v;
    }
}

// mean and 1/(std+eps) of the window, population std, two-pass for accuracy.
template <typename T, int BS>
__device__ __forceinline__ void window_stats(const T *win, T *red, int tid, T eps, T &mean, T &sd,
                                             T &inv) {
    using G = Geo<BS>;
    T s = T(0);
    for (int idx = tid; idx < G::W; idx += G::NT) s += win[idx];
    mean = block_sum(s, red, tid, G::NT) / T(G::W);
    T q = T(0);
    for (int idx = tid; idx < G::W; idx += G::NT) {
        T d = win[idx] - mean;
        q += d * d;
    }
    sd = sqrt(block_sum(q, red, tid, G::NT) / T(G::W));
    inv = T(1) / (sd + eps);
}

template <typename T, int BS, bool NORM>
__device__ __forceinline__ T pre_activation(const T *win, const T (&w)[27], T bias, int base,
                                            T mean, T inv) {
    using G = Geo<BS>;
    T u = bias;
#pragma unroll
    for (int a = 0; a < 3; ++a)
#pragma unroll
        for (int b = 0; b < 3; ++b)
#pragma unroll
            for (int c = 0; c < 3; ++c) {
                T v = win[base + (a * G::S + b) * G::S + c];
                if (NORM) v = (v - mean) * inv;
                u += w[a * 9 + b * 3 + c] * v;
            }
    return u;
}

template <typename T, int BS, int ACT, bool NORM>
__global__ __launch_bounds__(BS *BS *BS) void step_fwd_generic(
    const T *__restrict__ weight, const T *__restrict__ bias, const T *__restrict__ scale,
    const T *__restrict__ x, T *__restrict__ y, int B, int M, int N, int K, int inner, T eps,
    int nblk, int nchunk, int chunk_len) {
    using G = Geo<BS>;
    __shared__ T win[G::W];
    __shared__ T red[8];

    const int tid = threadIdx.x;
    int blk, chunk;
    if (!split_block_id(blockIdx.x, nblk, nchunk, blk, chunk)) return;  // grid padding
    const int kb = K / BS, nb = N / BS;
    const int p0 = (blk / (kb * nb)) * BS, q0 = ((blk / kb) % nb) * BS, r0 = (blk % kb) * BS;
    const int ci = tid / (BS * BS), cj = (tid / BS) % BS, ck = tid % BS;
    const long cells = (long)M * N * K;
    const long gc = ((long)(p0 + ci) * N + (q0 + cj)) * K + (r0 + ck);
    const int base = (ci * G::S + cj) * G::S + ck;           // window index of tap (0,0,0)
    const int centre = base + (G::S + 1) * G::S + 1;         // window index of the cell itself

    T w[27];
#pragma unroll
    for (int t = 0; t < 27; ++t) w[t] = weight[t * cells + gc];
    const T bv = bias[gc], rv = scale[gc];

    const int s_end = min(B, (chunk + 1) * chunk_len);
    for (int s = chunk * chunk_len; s < s_end; ++s) {
        load_window<T, BS>(win, x + s * cells, p0, q0, r0, M, N, K, tid);
        __syncthreads();
        T cur = win[centre];
        for (int it = 0; it < inner; ++it) {
            T mean = T(0), sd = T(0), inv = T(1);
            if (NORM) window_stats<T, BS>(win, red, tid, eps, mean, sd, inv);
            const T u = pre_activation<T, BS, NORM>(win, w, bv, base, mean, inv);
            cur += rv * Act<ACT, T>::f(u);
            __syncthreads();  // everyone has read the old state
            win[centre] = cur;
            __syncthreads();
        }
        y[s * cells + gc] = cur;
        __syncthreads();  // window is reloaded next
    }
}

// LDS of the backward kernel: three windows, the table of per-tap products and the reduction
// scratch.  Above 64 KB for fp64 at block size 8, hence dynamic.
extern __shared__ __align__(16) unsigned char generic_lds[];

template <typename T, int BS> constexpr size_t bwd_generic_lds() {
    return (3 * Geo<BS>::W + (kGatherTaps<T> ? 27 * Geo<BS>::NT : 0) + 8 + 3 * kMaxBackwardIters) *
           sizeof(T);
}

template <typename T, int BS, int ACT, bool NORM>
__global__ __launch_bounds__(BS *BS *BS) void step_bwd_generic(
    const T *__restrict__ weight, const T *__restrict__ bias, const T *__restrict__ scale,
    const T *__restrict__ x, const T *__restrict__ dy, T *__restrict__ dweight,
    T *__restrict__ dbias, T *__restrict__ dscale, T *__restrict__ dx, int B, int M, int N, int K,
    int inner, T eps, int nblk, int nchunk, int chunk_len, int param_mode) {
    using G = Geo<BS>;
    T *win = reinterpret_cast<T *>(generic_lds);  // state v_i of the window
    T *gwin = win + G::W;                         // dL/d(window), carried through the iterations
    T *dz = gwin + G::W;                          // dL/d(stencil input) of the current iteration
    T *prod = dz + G::W;                          // [27][cells]: weight * delta of every cell
    T *red = prod + (kGatherTaps<T> ? 27 * G::NT : 0);
    T *stat = red + 8;  // (mean, std, 1/(std+eps)) of the window before each inner iteration

    const int tid = threadIdx.x;
    int blk, chunk;
    if (!split_block_id(blockIdx.x, nblk, nchunk, blk, chunk)) return;  // grid padding
    const int kb = K / BS, nb = N / BS;
    const int p0 = (blk / (kb * nb)) * BS, q0 = ((blk / kb) % nb) * BS, r0 = (blk % kb) * BS;
    const int ci = tid / (BS * BS), cj = (tid / BS) % BS, ck = tid % BS;
    const long cells = (long)M * N * K;
    const long gc = ((long)(p0 + ci) * N + (q0 + cj)) * K + (r0 + ck);
    const int base = (ci * G::S + cj) * G::S + ck;
    const int centre = base + (G::S + 1) * G::S + 1;

    T w[27], dw[27];
#pragma unroll
    for (int t = 0; t < 27; ++t) {
        w[t] = weight[t * cells + gc];
        dw[t] = T(0);
    }
    const T bv = bias[gc], rv = scale[gc];
    T db = T(0), dr = T(0);
    T hist[kMaxBackwardIters];  // this cell's value before each inner iteration

    using Gather = TapGather<BS>;
    unsigned entry[Gather::kEntries];  // the window entries this thread gathers for
#pragma unroll
    for (int e = 0; e < Gather::kEntries; ++e) entry[e] = Gather::describe(tid + e * G::NT);

    const int s_end = min(B, (chunk + 1) * chunk_len);
    for (int s = chunk * chunk_len; s < s_end; ++s) {
        load_window<T, BS>(win, x + s * cells, p0, q0, r0, M, N, K, tid);
        for (int idx = tid; idx < G::W; idx += G::NT) gwin[idx] = T(0);
        __syncthreads();
        gwin[centre] = dy[s * cells + gc];
        if (inner == 0) __syncthreads();  // no loop barrier lies before the window is read below

        // forward recompute, remembering this cell's trajectory
        T cur = win[centre];
        for (int it = 0; it < inner; ++it) {
            hist[it] = cur;
            T mean = T(0), sd = T(0), inv = T(1);
            if (NORM) {
                window_stats<T, BS>(win, red, tid, eps, mean, sd, inv);
                if (tid == 0) {
                    stat[3 * it] = mean;
                    stat[3 * it + 1] = sd;
                    stat[3 * it + 2] = inv;
                }
            }
            const T u = pre_activation<T, BS, NORM>(win, w, bv, base, mean, inv);
            cur += rv * Act<ACT, T>::f(u);
            __syncthreads();
            win[centre] = cur;
            __syncthreads();
        }

        for (int it = inner - 1; it >= 0; --it) {
            win[centre] = hist[it];  // window back to state v_it (the halo never changed)
            if (!kGatherTaps<T>)
                for (int idx = tid; idx < G::W; idx += G::NT) dz[idx] = T(0);
            __syncthreads();
            T mean = T(0), sd = T(0), inv = T(1);
            if (NORM) {  // as the recompute found them: the window is back in that state
                mean = stat[3 * it];
                sd = stat[3 * it + 1];
                inv = stat[3 * it + 2];
            }
            const T u = pre_activation<T, BS, NORM>(win, w, bv, base, mean, inv);
            T f, d;
            Act<ACT, T>::fd(u, f, d);
            const T g = gwin[centre];
            dr += f * g;
            const T delta = d * g * rv;
            db += delta;
#pragma unroll
            for (int a = 0; a < 3; ++a)
#pragma unroll
                for (int b = 0; b < 3; ++b)
#pragma unroll
                    for (int c = 0; c < 3; ++c) {
                        const int t = a * 9 + b * 3 + c;
                        T v = win[base + (a * G::S + b) * G::S + c];
                        if (NORM) v = (v - mean) * inv;
                        dw[t] += v * delta;
                        if (kGatherTaps<T>) prod[t * G::NT + tid] = w[t] * delta;
                        else atomicAdd(&dz[base + (a * G::S + b) * G::S + c], w[t] * delta);
                    }
            __syncthreads();
#pragma unroll
            for (int e = 0; e < (kGatherTaps<T> ? Gather::kEntries : 0); ++e) {
                const int idx = tid + e * G::NT;
                const T acc = Gather::collect(prod, entry[e]);
                if (idx < G::W) dz[idx] = acc;
            }
            if (kGatherTaps<T>) __syncthreads();
            if (NORM) {
                // z = (v - mean) * inv over the whole window: push dz back through it
                T sdz = T(0), sproj = T(0);
                for (int idx = tid; idx < G::W; idx += G::NT) {
                    sdz += dz[idx];
                    sproj += dz[idx] * (win[idx] - mean);
                }
                const T mdz = block_sum(sdz, red, tid, G::NT) / T(G::W);
                const T proj = block_sum(sproj, red, tid, G::NT);
                const T tiny = T(1e-30);
                const T coef = proj * inv * inv / (T(G::W) * (sd > tiny ? sd : tiny));
                for (int idx = tid; idx < G::W; idx += G::NT)
                    gwin[idx] += inv * (dz[idx] - mdz) - coef * (win[idx] - mean);
            } else {
                for (int idx = tid; idx < G::W; idx += G::NT) gwin[idx] += dz[idx];
            }
            __syncthreads();
        }

        // the window of gradients lands on the input grid; halo entries belong to the
        // neighbouring blocks' cells, hence the atomics (dx was zeroed or holds a prior sum)
        T *dxs = dx + s * cells;
        for (int idx = tid; idx < G::W; idx += G::NT) {
            const int wk = idx % G::S, wj = (idx / G::S) % G::S, wi = idx / (G::S * G::S);
            const int gi = p0 + wi - 1, gj = q0 + wj - 1, gk = r0 + wk - 1;
            if (gi >= 0 && gi < M && gj >= 0 && gj < N && gk >= 0 && gk < K)
                unsafeAtomicAdd(&dxs[((long)gi * N + gj) * K + gk], gwin[idx]);
        }
        __syncthreads();
    }

    // parameter gradients, already summed over this chunk of the batch in registers
    if (param_mode == kParamStore) {
#pragma unroll
        for (int t = 0; t < 27; ++t) dweight[t * cells + gc] = dw[t];
        dbias[gc] = db;
        dscale[gc] = dr;
    } else if (param_mode == kParamAddExclusive) {
#pragma unroll
        for (int t = 0; t < 27; ++t) dweight[t * cells + gc] += dw[t];
        dbias[gc] += db;
        dscale[gc] += dr;
    } else {
#pragma unroll
        for (int t = 0; t < 27; ++t) unsafeAtomicAdd(&dweight[t * cells + gc], dw[t]);
        unsafeAtomicAdd(&dbias[gc], db);
        unsafeAtomicAdd(&dscale[gc], dr);
    }
}

template <typename T> __global__ void fill_zero_kernel(T *p, long n) {
    long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    const long stride = (long)gridDim.x * blockDim.x;
    for (; i < n; i += stride) p[i] = T(0);
}

template <typename T, int BS, int ACT>
int launch_fwd_norm(const StepArgs &a, int nblk, int nchunk, int chunk_len, hipStream_t st) {
    dim3 grid(padded_grid(nblk, nchunk)), block(Geo<BS>::NT);
    auto args = [&](auto kern) {
        hipLaunchKernelGGL(kern, grid, block, 0, st, (const T *)a.weight, (const T *)a.bias,
                           (const T *)a.scale, (const T *)a.x, (T *)a.y, a.B, a.M, a.N, a.K,
                           a.inner, (T)a.eps, nblk, nchunk, chunk_len);
    };
    if (a.normalize) args(step_fwd_generic<T, BS, ACT, true>);
    else args(step_fwd_generic<T, BS, ACT, false>);
    return check_launch("step_fwd_generic");
}

template <typename T, int BS, int ACT, bool NORM>
int launch_bwd_kernel(const StepArgs &a, int nblk, int nchunk, int chunk_len, int param_mode,
                      hipStream_t st) {
    dim3 grid(padded_grid(nblk, nchunk)), block(Geo<BS>::NT);
    auto kern = step_bwd_generic<T, BS, ACT, NORM>;
    constexpr size_t lds = bwd_generic_lds<T, BS>();
    static bool big_lds_enabled = false;  // per instantiation
    if (lds > 64 * 1024 && !big_lds_enabled) {
        hipError_t e = hipFuncSetAttribute((const void *)kern,
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess)
            return fail(GRIDNET_ERR_LAUNCH, "cannot enable %zu bytes of LDS: %s", lds,
                        hipGetErrorString(e));
        big_lds_enabled = true;
    }
    hipLaunchKernelGGL(kern, grid, block, lds, st, (const T *)a.weight, (const T *)a.bias,
                       (const T *)a.scale, (const T *)a.x, (const T *)a.dy, (T *)a.dweight,
                       (T *)a.dbias, (T *)a.dscale, (T *)a.dx, a.B, a.M, a.N, a.K, a.inner,
                       (T)a.eps, nblk, nchunk, chunk_len, param_mode);
    return check_launch("step_bwd_generic");
}

template <typename T, int BS, int ACT>
int launch_bwd_norm(const StepArgs &a, int nblk, int nchunk, int chunk_len, int param_mode,
                    hipStream_t st) {
    if (a.normalize)
        return launch_bwd_kernel<T, BS, ACT, true>(a, nblk, nchunk, chunk_len, param_mode, st);
    return launch_bwd_kernel<T, BS, ACT, false>(a, nblk, nchunk, chunk_len, param_mode, st);
}

template <typename T, int BS, bool BWD>
int dispatch_act(const StepArgs &a, int nblk, int nchunk, int chunk_len, int param_mode,
                 hipStream_t st) {
#define GRIDNET_CASE(ID)                                                                     \
    case ID:                                                                                 \
        if (BWD) return launch_bwd_norm<T, BS, ID>(a, nblk, nchunk, chunk_len, param_mode, st); \
        return launch_fwd_norm<T, BS, ID>(a, nblk, nchunk, chunk_len, st);
    switch (a.activation) {
        GRIDNET_CASE(GRIDNET_ACT_RELU)
        GRIDNET_CASE(GRIDNET_ACT_LEAKY_RELU)
        GRIDNET_CASE(GRIDNET_ACT_SILU)
        GRIDNET_CASE(GRIDNET_ACT_TANH)
    }
#undef GRIDNET_CASE
    return fail(GRIDNET_ERR_ACTIVATION, "unknown activation function: %d", a.activation);
}

// Enough workgroups to cover the chip a few times over, without splitting the batch more
// than needed (every chunk refetches the block's parameters).
int pick_chunks(int nblk, int B) {
    const int want = 256 * 4;
    int nchunk = (want + nblk - 1) / nblk;
    if (nchunk > B) nchunk = B;
    if (nchunk < 1) nchunk = 1;
    return nchunk;
}

template <typename T> int fill_zero(T *p, long n, hipStream_t st) {
    if (n <= 0) return GRIDNET_OK;
    long blocks = (n + 255) / 256;
    if (blocks > 4096) blocks = 4096;
    hipLaunchKernelGGL(fill_zero_kernel<T>, dim3((unsigned)blocks), dim3(256), 0, st, p, n);
    return check_launch("fill_zero");
}

template <typename T> int run_generic(const StepArgs &a, bool bwd, hipStream_t st) {
    const int bs = a.block_size;
    const int nblk = (a.M / bs) * (a.N / bs) * (a.K / bs);
    int nchunk = pick_chunks(nblk, a.B);
    const int chunk_len = (a.B + nchunk - 1) / nchunk;
    nchunk = (a.B + chunk_len - 1) / chunk_len;
    int param_mode = kParamAtomic;
    if (bwd) {
        const long cells = (long)a.M * a.N * a.K;
        const bool new_params = (a.flags & GRIDNET_OVERWRITE_PARAMS) != 0;
        if (a.flags & GRIDNET_OVERWRITE_DX) {  // dx is built with atomics: start from zero
            if (int rc = fill_zero((T *)a.dx, (long)a.B * cells, st)) return rc;
        }
        if (nchunk == 1) {
            param_mode = new_params ? kParamStore : kParamAddExclusive;
        } else if (new_params) {
            if (int rc = fill_zero((T *)a.dweight, 27 * cells, st)) return rc;
            if (int rc = fill_zero((T *)a.dbias, cells, st)) return rc;
            if (int rc = fill_zero((T *)a.dscale, cells, st)) return rc;
        }
    }
    if (bs == 8) {
        return bwd ? dispatch_act<T, 8, true>(a, nblk, nchunk, chunk_len, param_mode, st)
                   : dispatch_act<T, 8, false>(a, nblk, nchunk, chunk_len, param_mode, st);
    }
    return bwd ? dispatch_act<T, 4, true>(a, nblk, nchunk, chunk_len, param_mode, st)
               : dispatch_act<T, 4, false>(a, nblk, nchunk, chunk_len, param_mode, st);
}

}  // namespace

int step_forward_generic(const StepArgs &a, hipStream_t st) {
    return a.dtype == GRIDNET_F64 ? run_generic<double>(a, false, st)
                                  : run_generic<float>(a, false, st);
}

int step_backward_generic(const StepArgs &a, hipStream_t st) {
    return a.dtype == GRIDNET_F64 ? run_generic<double>(a, true, st)
                                  : run_generic<float>(a, true, st);
}

}  // namespace gridnet
