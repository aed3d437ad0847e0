// Tuned fp32 kernels for the gated variant of the block-local update,
//   x' = gate * x + (1 - gate) * act(pre),  pre  = b[0] + sum_t W[t,0] x_nbr,
//                                           gate = sigmoid(b[1] + sum_t W[t,1] x_nbr)
// (gridnet/backend_torch.py:145-267; the reference's kernels: src/gridnet_cuda_kernels.cu:452-734).
// Weight [27, 2, M, N, K], bias [2, M, N, K]; no scale, no normalisation.
//
// Same decomposition as the tuned kernels of the plain step (step_fast.hip, whose building
// blocks these share): a slot of threads advances one (block, batch element) pair with both
// weight sets in registers, the window in LDS, one barrier per inner iteration; a neighbour row
// read from LDS feeds both dot products.  Backward: each thread owns ONE cell (54 weights, their
// 54 mirrored neighbours' weights and 54 gradient accumulators fill the register file), the two
// deltas of an iteration go to two zero-haloed LDS windows and are gathered from there; what
// crosses a block boundary depends on the iterations only through D0 = sum_i delta0_i and
// D1 = sum_i delta1_i (the halo is frozen), which the kernel leaves for the cross-block kernel
// of the plain step run on two weight sets.  No atomics: where the batch of a block is split over
// workgroups every chunk commits into a copy of the gradient arrays of its own (see plan.h).

#include "common.h"
#include "fast_tiles.h"
#include "plan.h"
#include "launch.h"

namespace gridnet {

namespace {

constexpr int kGatedDepth = 4;  // neighbour rows requested ahead of the arithmetic

// pre[c], gp[c] = init + sum over the 27 taps, both weight sets fed from the same window rows
template <typename TL, int CPT>
__device__ __forceinline__ void stencil2(const float *win, int row00, const float (&wa)[27][CPT],
                                         const float (&wg)[27][CPT], const float (&ba)[CPT],
                                         const float (&bg)[CPT], float (&pre)[CPT], float (&gp)[CPT]) {
#pragma unroll
    for (int c = 0; c < CPT; ++c) {
        pre[c] = ba[c];
        gp[c] = bg[c];
    }
    for_each_row<TL, CPT, kGatedDepth>(win + row00, [&](int r, const float (&v)[CPT + 2]) {
#pragma unroll
        for (int cc = 0; cc < 3; ++cc)
#pragma unroll
            for (int c = 0; c < CPT; ++c) {
                pre[c] = fmaf(wa[r * 3 + cc][c], v[c + cc], pre[c]);
                gp[c] = fmaf(wg[r * 3 + cc][c], v[c + cc], gp[c]);
            }
    });
}

// ---- forward --------------------------------------------------------------------------------
template <int BS, int CPT, int NSLOT, int ACT>
__global__ __launch_bounds__((Tile<BS, CPT>::TPS * NSLOT)) __attribute__((amdgpu_waves_per_eu(3)))
void gated_fwd_fast(const float *__restrict__ weight, const float *__restrict__ bias,
                    const float *__restrict__ x, float *__restrict__ y, int B, int M, int N, int K,
                    int inner, int nblk, int nchunk, int chunk_len) {
    using TL = Tile<BS, CPT>;
    __shared__ __attribute__((aligned(16))) float lds[NSLOT * 2 * TL::WIN];  // two window copies per slot

    int blk, chunk;
    if (!split_block_id(blockIdx.x, nblk, nchunk, blk, chunk)) return;  // grid padding
    const Place<TL, CPT, NSLOT> pl(threadIdx.x, blk, N, K);
    const Fetch<TL> fx(pl.lane, pl.p0, pl.q0, pl.r0, M, N, K);
    float *win = lds + pl.slot * (2 * TL::WIN);
    const long cells = (long)M * N * K;

    float wa[27][CPT], wg[27][CPT], ba[CPT], bg[CPT];
#pragma unroll
    for (int t = 0; t < 27; ++t) {
        load_cells<CPT>(weight + (t * 2 + 0) * cells + pl.gc, wa[t]);
        load_cells<CPT>(weight + (t * 2 + 1) * cells + pl.gc, wg[t]);
    }
    load_cells<CPT>(bias + pl.gc, ba);
    load_cells<CPT>(bias + cells + pl.gc, bg);
    wait_global_loads();

    const int s0 = chunk * chunk_len, s1 = min(B, s0 + chunk_len);
    typename Fetch<TL>::Buf pre_win;
    if (s0 + pl.slot < s1) fx.fetch(x + (s0 + pl.slot) * cells, pre_win);
    // the result of an element is stored one element late, after the next window has been
    // committed: the wait for the prefetched window would otherwise also wait for that store
    float done[CPT];
    int done_s = -1;
    for (int sb = s0; sb < s1; sb += NSLOT) {
        const int s = sb + pl.slot;
        const bool active = s < s1;  // a slot past the end idles through the barriers
        if (active) fx.commit(win, pre_win);
        lds_barrier();
        if (done_s >= 0) store_cells<CPT>(y + done_s * cells + pl.gc, done);
        if (s + NSLOT < s1) fx.fetch(x + (s + NSLOT) * cells, pre_win);  // next element, in flight
        float cur[CPT];
        if (active) {
#pragma unroll
            for (int c = 0; c < CPT; ++c) cur[c] = win[pl.own + c];
        }
        for (int it = 0; it < inner; ++it) {
            if (active) {
                float pre[CPT], gp[CPT];
                stencil2<TL, CPT>(win + (it & 1) * TL::WIN, pl.row00, wa, wg, ba, bg, pre, gp);
#pragma unroll
                for (int c = 0; c < CPT; ++c) {
                    const float gate = sigmoid_stable(gp[c]);
                    const float a = Act<ACT, float>::f(pre[c]);
                    cur[c] = fmaf(gate, cur[c] - a, a);  // gate * x + (1 - gate) * act(pre)
                    win[((it + 1) & 1) * TL::WIN + pl.own + c] = cur[c];
                }
            }
            lds_barrier();
        }
        done_s = active ? s : -1;
#pragma unroll
        for (int c = 0; c < CPT; ++c) done[c] = cur[c];
        if (inner == 0) lds_barrier();  // `cur` was read from the window that is rewritten next
    }
    if (done_s >= 0) store_cells<CPT>(y + done_s * cells + pl.gc, done);
}

// ---- backward, first kernel (block-local part) ------------------------------------------------
// LDS per slot (floats): [x window x2 | delta0 window x2 | delta1 window x2 | history: inner
// slabs of 3 * TPS (x_i, pre_i, gate pre-activation_i of the owned cell)]
template <int BS> __host__ __device__ constexpr int gated_slot_floats(int inner) {
    return 6 * Tile<BS, 1>::WIN + inner * Tile<BS, 1>::TPS * 3;
}
// ... and at least one set of 27 weight planes of the block, which pass through LDS at set-up
template <int BS, int NSLOT> size_t gated_lds_bytes(int inner) {
    const size_t run = (size_t)NSLOT * gated_slot_floats<BS>(inner) * sizeof(float);
    const size_t setup = (size_t)27 * BS * BS * BS * sizeof(float);
    return run > setup ? run : setup;
}

template <int BS, int NSLOT, int ACT>
__global__ __launch_bounds__((Tile<BS, 1>::TPS * NSLOT)) __attribute__((amdgpu_waves_per_eu(2)))
void gated_bwd_fast(const float *__restrict__ weight, const float *__restrict__ bias,
                    const float *__restrict__ x, const float *__restrict__ dy,
                    float *__restrict__ dweight, float *__restrict__ dbias, float *__restrict__ dx,
                    float *__restrict__ dsum_out, int B, int M, int N, int K, int inner, int nblk,
                    int nchunk, int chunk_len, int param_mode, int dx_accumulate, long slab_stride) {
    using TL = Tile<BS, 1>;
    extern __shared__ __attribute__((aligned(16))) float lds[];
    const int slot_floats = gated_slot_floats<BS>(inner);

    int blk, chunk;
    if (!split_block_id(blockIdx.x, nblk, nchunk, blk, chunk)) return;  // grid padding
    if (slab_stride) {  // a split batch: every chunk commits into a copy of the gradient arrays of its own
        dweight += chunk * slab_stride;
        dbias += chunk * slab_stride;
    }
    const Place<TL, 1, NSLOT> pl(threadIdx.x, blk, N, K);
    const Fetch<TL> fx(pl.lane, pl.p0, pl.q0, pl.r0, M, N, K);
    float *win = lds + pl.slot * slot_floats;
    float *d0win = win + 2 * TL::WIN, *d1win = win + 4 * TL::WIN;
    float *hist = win + 6 * TL::WIN + pl.lane;  // + it * 3 * TPS: x_i; + TPS: pre_i; + 2 TPS: gate's
    // the x window copy that would receive x_inner (never needed) gets a zero in the block's
    // cells instead: the halo alone, for the weights of the taps that read it
    const float *xhalo = win + (inner & 1) * TL::WIN;
    const long cells = (long)M * N * K;

    // slot [t] of the mirrored arrays belongs to the weights of the neighbour at c + off_t where
    // that lies in this block, and to this cell's own weights of tap t where it does not
    auto in_block = [&](int t) {
        const int ni = pl.i + t / 9 - 1, nj = pl.j + (t / 3) % 3 - 1, nk = pl.kt + t % 3 - 1;
        return ni >= 0 && ni < BS && nj >= 0 && nj < BS && nk >= 0 && nk < BS;
    };
    // index into [27, 2, M, N, K] of the weight that slot t of set k stands for
    auto owner_of = [&](int t, int k) {
        if (in_block(t))
            return ((26 - t) * 2 + k) * cells + pl.gc + ((t / 9 - 1) * N + ((t / 3) % 3 - 1)) * K + (t % 3 - 1);
        return (t * 2 + k) * cells + pl.gc;
    };

    // ---- once per workgroup ----
    // wa, wg : this cell's weights (forward recompute)
    // va, vg : V[t] = W[26-t, c + off_t], what the neighbour at c + off_t multiplies this cell by
    // na, ng : gradient of that same neighbour weight (this thread is its only contributor);
    //          where the neighbour lies in another block, of this cell's own weight of tap t,
    //          which reads a frozen halo entry: x_halo * D, added once per element
    float wa[27][1], wg[27][1], va[27], vg[27], na[27], ng[27];
#pragma unroll
    for (int t = 0; t < 27; ++t) {
        wa[t][0] = weight[(t * 2 + 0) * cells + pl.gc];
        wg[t][0] = weight[(t * 2 + 1) * cells + pl.gc];
        na[t] = ng[t] = 0.f;
    }
    float ba[1], bg[1], dba = 0.f, dbg = 0.f;
    ba[0] = bias[pl.gc];
    bg[0] = bias[cells + pl.gc];
    {   // the mirrored weights are other threads' own weights: exchanged through LDS, one set
        // after the other (the windows are not in use yet)
        constexpr int NC = BS * BS * BS;
        float *wl = lds;  // [27][NC], by block-local cell (i, j, k)
        const int lin = (pl.i * BS + pl.j) * BS + pl.kt;
#pragma unroll
        for (int k = 0; k < 2; ++k) {
            if (pl.slot == 0) {
#pragma unroll
                for (int t = 0; t < 27; ++t) wl[t * NC + lin] = k ? wg[t][0] : wa[t][0];
            }
            lds_barrier();
#pragma unroll
            for (int t = 0; t < 27; ++t) {
                const float got = in_block(t) ? wl[(26 - t) * NC + lin + ((t / 9 - 1) * BS + ((t / 3) % 3 - 1)) * BS + (t % 3 - 1)]
                                              : 0.f;
                if (k) vg[t] = got;
                else va[t] = got;
            }
            lds_barrier();  // the next set, then the windows, reuse this memory
        }
    }
    // delta windows: the halo stays zero for the whole kernel
    for (int idx = pl.lane; idx < 4 * TL::WIN; idx += TL::TPS) d0win[idx] = 0.f;
    wait_global_loads();
    // add-in-place mode: the accumulators start from what the gradient buffers hold and are
    // stored at the end like in the overwrite mode
    if (param_mode == kParamAddExclusive && pl.slot == 0) {
#pragma unroll
        for (int t = 0; t < 27; ++t) {
            na[t] = dweight[owner_of(t, 0)];
            ng[t] = dweight[owner_of(t, 1)];
        }
        dba = dbias[pl.gc];
        dbg = dbias[cells + pl.gc];
    }

    const int s0 = chunk * chunk_len, s1 = min(B, s0 + chunk_len);
    typename Fetch<TL>::Buf pre_win;
    float g = 0.f, gnext = 0.f;
    auto fetch_element = [&](int s) {
        fx.fetch(x + s * cells, pre_win);
        gnext = dy[s * cells + pl.gc];
    };
    auto take_element = [&]() {
        g = gnext;
        fx.commit(win, pre_win);
    };
    if (s0 + pl.slot < s1) {
        fetch_element(s0 + pl.slot);
        take_element();
    }
    // results are stored one element late, away from the wait on the prefetched window
    float g_done = 0.f, d0_done = 0.f, d1_done = 0.f;
    int done_s = -1;
    auto finish_done = [&]() {
        if (done_s < 0) return;
        const long o = (long)done_s * cells + pl.gc;
        dsum_out[o] = d0_done;
        dsum_out[(long)B * cells + o] = d1_done;
        if (dx_accumulate) dx[o] += g_done;
        else dx[o] = g_done;
        done_s = -1;
    };
    for (int sb = s0; sb < s1; sb += NSLOT) {
        const int s = sb + pl.slot;
        const bool active = s < s1;  // a slot past the end idles through the barriers
        lds_barrier();               // this element's window
        finish_done();
        if (s + NSLOT < s1) fetch_element(s + NSLOT);
        float cur = 0.f;
        if (active) cur = win[pl.own];

        // ---- forward recompute, remembering x_i and both pre-activations of the owned cell ----
        for (int it = 0; it < inner; ++it) {
            if (active) {
                float pre[1], gp[1];
                stencil2<TL, 1>(win + (it & 1) * TL::WIN, pl.row00, wa, wg, ba, bg, pre, gp);
                float *h = hist + it * (3 * TL::TPS);
                h[0] = cur;
                h[TL::TPS] = pre[0];
                h[2 * TL::TPS] = gp[0];
                if (it + 1 < inner) {
                    const float gate = sigmoid_stable(gp[0]);
                    const float a = Act<ACT, float>::f(pre[0]);
                    cur = fmaf(gate, cur - a, a);
                    win[((it + 1) & 1) * TL::WIN + pl.own] = cur;
                } else {  // x_inner itself is never needed: that copy becomes the halo window
                    win[((it + 1) & 1) * TL::WIN + pl.own] = 0.f;
                }
            }
            if (it + 1 < inner) lds_barrier();
        }

        // ---- reverse sweep: delta window copies (it & 1) hold the deltas of iteration it ----
        float dsum0 = 0.f, dsum1 = 0.f;
        for (int it = inner - 1; it >= 0; --it) {
            float xi = 0.f, direct = 0.f;
            if (active) {
                const float *h = hist + it * (3 * TL::TPS);
                xi = h[0];
                const float pre = h[TL::TPS], gp = h[2 * TL::TPS];
                const float gate = sigmoid_stable(gp);
                float f, d;
                Act<ACT, float>::fd(pre, f, d);
                const float delta0 = g * (1.f - gate) * d;
                const float delta1 = g * (xi - f) * gate * (1.f - gate);
                dba += delta0;
                dbg += delta1;
                dsum0 += delta0;
                dsum1 += delta1;
                direct = gate * g;  // the path through gate * x
                d0win[(it & 1) * TL::WIN + pl.own] = delta0;
                d1win[(it & 1) * TL::WIN + pl.own] = delta1;
            }
            if (it == 0) {
                // D0, D1 are complete: the weights of the taps that read the halo.  Before this
                // iteration's barrier, so that nobody commits the next element's window while
                // the halo is read; behind a barrier of its own when the zeros of the halo
                // window were written in the iteration just before (inner == 1).
                if (inner == 1) lds_barrier();
                if (active)
                    for_each_row<TL, 1, kGatedDepth>(xhalo + pl.row00, [&](int r, const float (&xv)[3]) {
#pragma unroll
                        for (int cc = 0; cc < 3; ++cc) {
                            na[r * 3 + cc] = fmaf(xv[cc], dsum0, na[r * 3 + cc]);
                            ng[r * 3 + cc] = fmaf(xv[cc], dsum1, ng[r * 3 + cc]);
                        }
                    });
            }
            lds_barrier();
            if (active) {
                float acc = direct;
                const float *d0 = d0win + (it & 1) * TL::WIN + pl.row00;
                const float *d1 = d1win + (it & 1) * TL::WIN + pl.row00;
                for_each_row<TL, 1, kGatedDepth>(d0, [&](int r, const float (&dv)[3]) {
#pragma unroll
                    for (int cc = 0; cc < 3; ++cc) {
                        na[r * 3 + cc] = fmaf(xi, dv[cc], na[r * 3 + cc]);
                        acc = fmaf(va[r * 3 + cc], dv[cc], acc);
                    }
                });
                for_each_row<TL, 1, kGatedDepth>(d1, [&](int r, const float (&dv)[3]) {
#pragma unroll
                    for (int cc = 0; cc < 3; ++cc) {
                        ng[r * 3 + cc] = fmaf(xi, dv[cc], ng[r * 3 + cc]);
                        acc = fmaf(vg[r * 3 + cc], dv[cc], acc);
                    }
                });
                g = acc;
            }
        }

        if (inner == 0) lds_barrier();  // no barrier since the top: others may still read LDS
        done_s = active ? s : -1;
        g_done = g;
        d0_done = dsum0;
        d1_done = dsum1;
        // the x windows are free (the reverse sweep does not read them): commit the next one
        if (s + NSLOT < s1) take_element();
    }
    finish_done();

    // ---- parameter gradients: reduce across slots through LDS, then commit ----
    if (NSLOT > 1) {
        float *red = lds;  // NSLOT * TPS floats, reused value by value
        auto reduce = [&](float &val) {
            lds_barrier();
            red[pl.slot * TL::TPS + pl.lane] = val;
            lds_barrier();
            if (pl.slot == 0) {
#pragma unroll
                for (int q = 1; q < NSLOT; ++q) val += red[q * TL::TPS + pl.lane];
            }
        };
#pragma unroll
        for (int t = 0; t < 27; ++t) {
            reduce(na[t]);
            reduce(ng[t]);
        }
        reduce(dba);
        reduce(dbg);
        if (pl.slot != 0) return;
    }
    // plain stores in every mode: this workgroup is the only one that writes these entries of its
    // arrays (the caller's, or its chunk's copy of them), and the accumulating mode started from
    // the old contents
#pragma unroll
    for (int t = 0; t < 27; ++t) {
        dweight[owner_of(t, 0)] = na[t];
        dweight[owner_of(t, 1)] = ng[t];
    }
    dbias[pl.gc] = dba;
    dbias[cells + pl.gc] = dbg;
}

__global__ void gated_fast_fill_zero(float *p, long n) {
    long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    const long stride = (long)gridDim.x * blockDim.x;
    for (; i < n; i += stride) p[i] = 0.f;
}

int fill_zero(float *p, long n, hipStream_t st) {
    if (n <= 0) return GRIDNET_OK;
    long blocks = (n + 1023) / 1024;
    if (blocks > 8192) blocks = 8192;
    hipLaunchKernelGGL(gated_fast_fill_zero, dim3((unsigned)blocks), dim3(256), 0, st, p, n);
    return check_launch("fill_zero");
}

int device_cus() {
    static int cus = 0;
    if (cus == 0) {
        int dev = 0, n = 0;
        if (hipGetDevice(&dev) == hipSuccess &&
            hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && n > 0)
            cus = n;
        else
            cus = 256;
    }
    return cus;
}

// The batch is dealt to workgroups in chunks, a chunk is walked NSLOT elements at a time; when
// the blocks alone do not fill the chip the batch is split so that the grid is one full wave.
void plan_chunks(int B, int nblk, int nslot, int resident, bool whole, int &nchunk, int &chunk_len) {
    nchunk = whole ? 1 : resident / nblk;
    const int max_chunks = (B + nslot - 1) / nslot;
    if (nchunk > max_chunks) nchunk = max_chunks;
    if (nchunk < 1) nchunk = 1;
    chunk_len = (B + nchunk - 1) / nchunk;
    chunk_len = (chunk_len + nslot - 1) / nslot * nslot;
    nchunk = (B + chunk_len - 1) / chunk_len;
}

// the tuned shapes
constexpr int kFwdCpt = 2;                        // both block sizes: two cells (108 weights) per thread
constexpr int kFwdSlots8 = 1, kFwdSlots4 = 4;     // 256 threads; four 32-thread slots
constexpr int kBwdSlots8 = 1, kBwdSlots4 = 2;     // 512 threads; two 64-thread slots
constexpr size_t kMaxLds = 160 * 1024;

template <int BS, int NSLOT, int ACT> int launch_fwd(const StepArgs &a, hipStream_t st) {
    using TL = Tile<BS, kFwdCpt>;
    auto kern = gated_fwd_fast<BS, kFwdCpt, NSLOT, ACT>;
    static int per_cu = 0;
    if (per_cu == 0) {
        int n = 0;
        if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, kern, TL::TPS * NSLOT, 0) != hipSuccess || n < 1)
            n = 1;
        per_cu = n;
    }
    const int nblk = (a.M / BS) * (a.N / BS) * (a.K / BS);
    int nchunk, chunk_len;
    plan_chunks(a.B, nblk, NSLOT, per_cu * device_cus(), false, nchunk, chunk_len);
    hipLaunchKernelGGL(kern, dim3(padded_grid(nblk, nchunk)), dim3(TL::TPS * NSLOT), 0, st,
                       (const float *)a.weight, (const float *)a.bias, (const float *)a.x, (float *)a.y,
                       a.B, a.M, a.N, a.K, a.inner, nblk, nchunk, chunk_len);
    return check_launch("gated_fwd_fast");
}

template <int BS, int NSLOT, int ACT> int launch_bwd(const StepArgs &a, hipStream_t st) {
    using TL = Tile<BS, 1>;
    const long cells = (long)a.M * a.N * a.K;
    const size_t lds = gated_lds_bytes<BS, NSLOT>(a.inner);
    auto kern = gated_bwd_fast<BS, NSLOT, ACT>;
    static bool big_lds_enabled = false;             // per instantiation
    static int per_cu_cache[kMaxBackwardIters + 1];  // per instantiation, by inner iterations
    if (lds > 64 * 1024 && !big_lds_enabled) {
        hipError_t e = hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize,
                                           (int)kMaxLds);
        if (e != hipSuccess)
            return fail(GRIDNET_ERR_LAUNCH, "cannot enable %zu bytes of LDS: %s", lds, hipGetErrorString(e));
        big_lds_enabled = true;
    }
    int &per_cu = per_cu_cache[a.inner];
    if (per_cu == 0) {
        int n = 0;
        if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, kern, TL::TPS * NSLOT, lds) != hipSuccess || n < 1)
            n = 1;
        per_cu = n;
    }
    const int nblk = (a.M / BS) * (a.N / BS) * (a.K / BS);
    // one workgroup owns the whole batch of its block (plain stores for the parameter gradients)
    // as soon as the blocks alone give every CU a workgroup
    int nchunk, chunk_len;
    plan_chunks(a.B, nblk, NSLOT, per_cu * device_cus(), nblk >= device_cus(), nchunk, chunk_len);
    const bool new_params = (a.flags & GRIDNET_OVERWRITE_PARAMS) != 0;
    // A split batch: every chunk gets a copy of the gradient arrays in the scratch; with less
    // room than chunks the batch is split less (down to not at all).
    const long slab_floats = kGatedSlabPlanes * cells;
    if (nchunk > 1) {
        const int room = plan_split_room(plan_slab_capacity(a.slabs, a.slab_bytes, slab_floats), a.B, chunk_len);
        if (room < nchunk) plan_chunks(a.B, nblk, NSLOT, (room < 2 ? 1 : room) * nblk, room < 2, nchunk, chunk_len);
    }
    const bool split = nchunk > 1;
    const int param_mode = split || new_params ? kParamStore : kParamAddExclusive;
    float *slab = (float *)a.slabs;
    const int dx_accumulate = (a.flags & GRIDNET_OVERWRITE_DX) ? 0 : 1;
    hipLaunchKernelGGL(kern, dim3(padded_grid(nblk, nchunk)), dim3(TL::TPS * NSLOT), lds, st,
                       (const float *)a.weight, (const float *)a.bias, (const float *)a.x,
                       (const float *)a.dy, split ? slab : (float *)a.dweight,
                       split ? slab + 54 * cells : (float *)a.dbias, (float *)a.dx,
                       (float *)a.workspace, a.B, a.M, a.N, a.K, a.inner, nblk, nchunk, chunk_len,
                       param_mode, dx_accumulate, split ? slab_floats : 0L);
    if (int rc = check_launch("gated_bwd_fast")) return rc;
    if (split) {
        SlabTargets t{};
        t.dst[0] = (float *)a.dweight; t.end[0] = 54 * cells;
        t.dst[1] = (float *)a.dbias;   t.end[1] = 56 * cells;
        t.count = 2;
        if (int rc = plan_reduce_slabs(slab, nchunk, slab_floats, t, new_params ? 0 : 1, st)) return rc;
    }
    // same blocks, same batch chunks; the parameter gradients are complete, dx is not yet
    return gated_cross_launch(a, (const float *)a.workspace, nchunk, chunk_len, st);
}

template <bool BWD, int ACT> int dispatch_bs(const StepArgs &a, hipStream_t st) {
    if (a.block_size == 8) return BWD ? launch_bwd<8, kBwdSlots8, ACT>(a, st) : launch_fwd<8, kFwdSlots8, ACT>(a, st);
    return BWD ? launch_bwd<4, kBwdSlots4, ACT>(a, st) : launch_fwd<4, kFwdSlots4, ACT>(a, st);
}

template <bool BWD> int dispatch(const StepArgs &a, hipStream_t st) {
    switch (a.activation) {
        case GRIDNET_ACT_RELU: return dispatch_bs<BWD, GRIDNET_ACT_RELU>(a, st);
        case GRIDNET_ACT_LEAKY_RELU: return dispatch_bs<BWD, GRIDNET_ACT_LEAKY_RELU>(a, st);
        case GRIDNET_ACT_SILU: return dispatch_bs<BWD, GRIDNET_ACT_SILU>(a, st);
        case GRIDNET_ACT_TANH: return dispatch_bs<BWD, GRIDNET_ACT_TANH>(a, st);
    }
    return fail(GRIDNET_ERR_ACTIVATION, "unknown activation function: id %d", a.activation);
}

}  // namespace

bool gated_fast_supports(const StepArgs &a, bool backward) {
    if (a.dtype != GRIDNET_F32) return false;
    if (a.block_size != 4 && a.block_size != 8) return false;
    if (backward) {
        const size_t lds = a.block_size == 8 ? gated_lds_bytes<8, kBwdSlots8>(a.inner)
                                             : gated_lds_bytes<4, kBwdSlots4>(a.inner);
        if (lds > kMaxLds) return false;
    }
    return true;
}

size_t gated_fast_backward_workspace(const StepArgs &a) {
    // D0 and D1 of every cell, handed from gated_bwd_fast to the cross-block kernel
    return (size_t)2 * a.B * a.M * a.N * a.K * sizeof(float);
}

size_t gated_fast_slab_bytes(const StepArgs &a) {
    // the most chunks any plan of the backward kernel makes (see step_fast_slab_bytes)
    const long nblk = (long)(a.M / a.block_size) * (a.N / a.block_size) * (a.K / a.block_size);
    if (nblk >= device_cus()) return 0;
    const int nslot = a.block_size == 8 ? kBwdSlots8 : kBwdSlots4;
    long chunks = (long)(a.block_size == 8 ? 2 : 16) * device_cus() / nblk;
    const long most = (a.B + nslot - 1) / nslot;
    if (chunks > most) chunks = most;
    if (chunks < 2) return 0;
    return (size_t)chunks * kGatedSlabPlanes * a.M * a.N * a.K * sizeof(float);
}

int gated_forward_fast(const StepArgs &a, hipStream_t st) { return dispatch<false>(a, st); }
int gated_backward_fast(const StepArgs &a, hipStream_t st) { return dispatch<true>(a, st); }

}  // namespace gridnet
