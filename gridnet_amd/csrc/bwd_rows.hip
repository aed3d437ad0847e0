// The backward of a step with ONE inner iteration, dealt by whole K-rows: the first of two kernels.
//
// With a single inner iteration the step is a plain stencil over the whole grid (see fwd_rows.hip):
//   u[c] = b[c] + sum_t w[t, c] x[c + off_t],   y[c] = x[c] + r[c] act(u[c]).
// With g the gradient with respect to y and delta[c] = act'(u[c]) g[c] r[c]:
//   dx[c] = g[c] + sum_t w[26-t, c + off_t] delta[c + off_t]
//   dw[t, c] = sum over the batch of x[c + off_t] delta[c],  db[c] = sum delta[c],
//   dr[c] = sum act(u[c]) g[c].
// This kernel recomputes u, forms delta and the parameter gradients, and leaves delta of every cell
// (in the scratch tensor the block kernels leave D in) and the direct part of dx, g.  The sum
// over the neighbours' deltas is cross_rows' job (cross_rows.hip, with ALL taps instead of the
// ones that cross a block boundary).
//
// The two sums the backward of the LayerNorm in FRONT of the step needs, sum gamma dx and
// sum gamma dx xn (xn the normalised input before gamma and beta), are formed HERE, before dx
// exists, so that cross_rows need not read x again: with xh = gamma xn + beta the step's input,
//   sum_c gamma[c] dx[c]        = sum_c gamma[c] g[c] + delta[c] Wg[c],   Wg[c] = sum_t w[t, c] gamma[c + off_t]
//   sum_c dx[c] (xh[c] - beta[c]) = sum_c g[c] (xh[c] - beta[c]) + delta[c] (u[c] - b[c] - Wb[c]),
//                                                               Wb[c] = sum_t w[t, c] beta[c + off_t]
// (every delta[c] reaches the cells c + off_t with the weights w[t, c], and sum_t w[t, c] xh[c + off_t]
// is u[c] - b[c]); Wg and Wb are two numbers per cell, formed once per workgroup.  The residual
// loop keeps cross_rows' sums.
// The reference does all of this per block with shared-memory and global atomics
// (src/gridnet_cuda_kernels.cu:300-450); here nothing is scattered.
//
// A workgroup takes a tube of 4 x 4 whole grid rows; a thread owns TWO cells along K with their 54
// weights and 54 weight-gradient accumulators in registers for its share of the batch (a split
// batch commits into per-chunk copies of the gradient arrays, see plan.h).  The 6 x 6 rows of x in
// and around the tube wait in LDS, two stages alternating, one barrier per batch element; a row
// is read twice per element (once for u, once for the weight gradients, when delta is known)
// as 8-byte pieces with the cell before and after from the neighbouring lanes.
//
// LN / RES as in step_bwd_fast (LnFold): x is normalised while its rows are committed; dy passes
// the backward of the LayerNorm behind the step as it is loaded (dgamma, dbeta fall out); the
// residual loop adds G'' and stores G', and its direct part of dx is G' - G' = 0.

#include "common.h"
#include "fast_tiles.h"
#include "launch.h"
#include "plan.h"

namespace gridnet {

namespace {

constexpr int kTube = 4;                          // the tube is 4 x 4 grid rows
constexpr int kWinRows = (kTube + 2) * (kTube + 2);  // rows in and around it

template <int ACT, bool LN, bool RES>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2, 3)))
void bwd_rows(const float *__restrict__ weight, const float *__restrict__ bias, const float *__restrict__ scale,
              const float *__restrict__ x, const float *__restrict__ dy, float *__restrict__ dweight,
              float *__restrict__ dbias, float *__restrict__ dscale, float *__restrict__ dx,
              float *__restrict__ delta_out, int B, int M, int N, int K, int ntube, int nchunk, int chunk_len,
              int param_mode, int dx_accumulate, LnFold ln, long slab_stride) {
    static_assert(LN || !RES, "the residual form comes with the folded LayerNorm");
    // [2 stages][36 rows][K]; LN: then gamma and beta of the 36 rows
    extern __shared__ __attribute__((aligned(16))) float lds[];

    int tube, chunk;
    if (!split_block_id(blockIdx.x, ntube, nchunk, tube, chunk)) return;  // grid padding
    if (slab_stride) {  // a split batch: this chunk's copy of the gradient arrays
        const long off = chunk * slab_stride;
        dweight += off;
        dbias += off;
        dscale += off;
        if (LN) {
            ln.dgamma += off;
            ln.dbeta += off;
        }
    }
    const int kb = K / 2, nt = 16 * kb, tid = threadIdx.x;  // kb: threads along a row
    const int bk = tid % kb, r = tid / kb, ci = r / kTube, cj = r % kTube;
    const int nbj = N / kTube, p0 = (tube / nbj) * kTube, q0 = (tube % nbj) * kTube;
    const long cells = (long)M * N * K;
    const int grow = ((p0 + ci) * N + (q0 + cj)) * K + 2 * bk;  // this thread's two cells
    const bool ln_in = LN && ln.x_stats != nullptr;              // x is the raw output of the step before
    const bool through_ln = LN && (!RES || ln.y_raw != nullptr);  // dy passes a LayerNorm on load

    float w[27][2], nw[27][2], bv[2], rv[2], db[2] = {0.f, 0.f}, dr[2] = {0.f, 0.f};
    float gam[2] = {0.f, 0.f}, dgam[2] = {0.f, 0.f}, dbet[2] = {0.f, 0.f};
#pragma unroll
    for (int t = 0; t < 27; ++t) {
        load_cells<2>(weight + t * cells + grow, w[t]);
        nw[t][0] = nw[t][1] = 0.f;
    }
    load_cells<2>(bias + grow, bv);
    load_cells<2>(scale + grow, rv);
    if (LN) load_cells<2>(ln.gamma + grow, gam);
    // The taps that would leave the row along K read what the neighbouring lane sends, a piece of
    // another row: their weights are zeroed here, and their weight gradients at the end.
    const float keep_first = bk == 0 ? 0.f : 1.f, keep_last = bk == kb - 1 ? 0.f : 1.f;
#pragma unroll
    for (int pq = 0; pq < 9; ++pq) {
        w[pq * 3][0] *= keep_first;
        w[pq * 3 + 2][1] *= keep_last;
    }

    // ---- the window rows this thread moves, as 16-byte pieces: piece tid and, for the first
    // eighth of the threads, piece tid + nt (36 K / 4 pieces in all) ----
    const int kq = K / 4;
    int goff[2], loff[2];
    bool ok[2], have[2];
    float *gam_rows = lds + 2 * kWinRows * K, *bet_rows = gam_rows + kWinRows * K;
#pragma unroll
    for (int e = 0; e < 2; ++e) {
        const int id = tid + e * nt, row = id / kq, q = id % kq;
        const int wi = row / (kTube + 2), wj = row % (kTube + 2);
        const int gi = p0 + wi - 1, gj = q0 + wj - 1;
        have[e] = row < kWinRows;
        ok[e] = have[e] && gi >= 0 && gi < M && gj >= 0 && gj < N;
        // (anything valid when not used: the same piece of the thread's own row)
        goff[e] = (ok[e] ? (gi * N + gj) : ((p0 + ci) * N + (q0 + cj))) * K + 4 * q;
        loff[e] = (have[e] ? row : 0) * K + 4 * q;
        if (ln_in && have[e]) {  // gamma and beta of the piece, once per workgroup
            float gq[4], bq[4];
            load_cells<4>(ln.gamma + goff[e], gq);
            load_cells<4>(ln.beta + goff[e], bq);
#pragma unroll
            for (int c = 0; c < 4; ++c) {  // zeros outside the grid: no test per element then
                gq[c] = ok[e] ? gq[c] : 0.f;
                bq[c] = ok[e] ? bq[c] : 0.f;
            }
            store_cells<4>(gam_rows + loff[e], gq);
            store_cells<4>(bet_rows + loff[e], bq);
        }
    }
    const int own_row = (ci + 1) * (kTube + 2) + (cj + 1);
    wait_global_loads();
    // the LayerNorm sums of dx (see the head of the file): Wg and b + Wb of the thread's cells
    const bool sums_here = LN && !RES && ln_in && ln.x_part != nullptr;
    float bet[2] = {0.f, 0.f}, wgam[2] = {0.f, 0.f}, bwb[2] = {bv[0], bv[1]};
    if (LN && !RES) {
        if (sums_here) {  // the same for the whole workgroup
            load_cells<2>(ln.beta + grow, bet);
            __syncthreads();  // gamma and beta of the 36 rows are in LDS
            auto over_taps = [&](const float *rows36, float (&acc)[2]) {
#pragma unroll
                for (int pq = 0; pq < 9; ++pq) {
                    const int di = pq / 3 - 1, dj = pq % 3 - 1;
                    float mid[2], d[4];
                    load_cells<2>(rows36 + (own_row + di * (kTube + 2) + dj) * K + 2 * bk, mid);
                    d[0] = lane_before(mid[1]);
                    d[1] = mid[0];
                    d[2] = mid[1];
                    d[3] = lane_after(mid[0]);
#pragma unroll
                    for (int cc = 0; cc < 3; ++cc)
#pragma unroll
                        for (int c = 0; c < 2; ++c) acc[c] = fmaf(w[pq * 3 + cc][c], d[c + cc], acc[c]);
                }
            };
            over_taps(gam_rows, wgam);
            over_taps(bet_rows, bwb);
        }
    }
    const int s0 = chunk * chunk_len, s1 = min(B, s0 + chunk_len);
    float xbuf[2][4], gnext[2], ynext[2] = {0.f, 0.f}, gprev[2] = {0.f, 0.f}, dxold[2] = {0.f, 0.f};
    float xmean = 0.f, xrstd = 1.f, ny[4] = {0.f, 1.f, 0.f, 0.f};
    auto fetch = [&](int s) {
        const long at = (long)s * cells;
        load_cells<2>(dy + at + grow, gnext);
        if (through_ln) {
            if (RES) load_cells<2>(ln.y_raw + at + grow, ynext);  // the plain loop recomputes it
            ny[0] = load_ahead(ln.y_stats, 2 * s);
            ny[1] = load_ahead(ln.y_stats, 2 * s + 1);
            ny[2] = load_ahead(ln.y_sums, 2 * s);
            ny[3] = load_ahead(ln.y_sums, 2 * s + 1);
        }
        if (RES && through_ln) load_cells<2>(ln.g_prev + at + grow, gprev);
        if (dx_accumulate) load_cells<2>(dx + at + grow, dxold);
        if (ln_in) {
            xmean = load_ahead(ln.x_stats, 2 * s);
            xrstd = load_ahead(ln.x_stats, 2 * s + 1);
        }
#pragma unroll
        for (int e = 0; e < 2; ++e) load_cells<4>(x + at + goff[e], xbuf[e]);
    };
    if (s0 < s1) fetch(s0);
    for (int s = s0; s < s1; ++s) {
        float *stage = lds + ((s - s0) & 1) * kWinRows * K;
#pragma unroll
        for (int e = 0; e < 2; ++e) {
            if (!have[e]) break;
            float v[4];
            if (ln_in) {
                float gq[4], bq[4];
                load_cells<4>(gam_rows + loff[e], gq);
                load_cells<4>(bet_rows + loff[e], bq);
#pragma unroll
                for (int q = 0; q < 4; ++q) v[q] = fmaf((xbuf[e][q] - xmean) * xrstd, gq[q], bq[q]);
            } else {
#pragma unroll
                for (int q = 0; q < 4; ++q) v[q] = ok[e] ? xbuf[e][q] : 0.f;
            }
            store_cells<4>(stage + loff[e], v);
        }
        // the element's incoming gradient, through the backward of the LayerNorm behind the step
        // (the plain loop: further down, from the raw output recomputed there; what the prefetch of the
        // next element is about to overwrite is set aside)
        constexpr bool kLate = LN && !RES;
        float g[2], gin[2], gcur[2] = {gnext[0], gnext[1]}, nyc[4] = {ny[0], ny[1], ny[2], ny[3]};
#pragma unroll
        for (int c = 0; c < 2; ++c) {
            if (kLate) {
                g[c] = 0.f;
            } else if (through_ln) {
                const float yh = (ynext[c] - ny[0]) * ny[1];
                dgam[c] = fmaf(gnext[c], yh, dgam[c]);
                dbet[c] += gnext[c];
                g[c] = ny[1] * (gam[c] * gnext[c] - ny[2] - yh * ny[3]);
                if (RES) g[c] += gprev[c];
            } else {
                g[c] = gnext[c];
            }
            gin[c] = g[c];
        }
        float keep[2];  // what dx holds already (accumulate mode)
#pragma unroll
        for (int c = 0; c < 2; ++c) keep[c] = dxold[c];
        lds_barrier();  // the stage is complete (the first: gamma and beta too); the other one's readers are done
        fetch(min(s + 1, s1 - 1));
        auto rows = [&](auto &&use) {  // the nine rows around the thread's cells, in tap order
#pragma unroll
            for (int pq = 0; pq < 9; ++pq) {
                const int di = pq / 3 - 1, dj = pq % 3 - 1;
                float mid[2], d[4];
                load_cells<2>(stage + (own_row + di * (kTube + 2) + dj) * K + 2 * bk, mid);
                d[0] = lane_before(mid[1]);
                d[1] = mid[0];
                d[2] = mid[1];
                d[3] = lane_after(mid[0]);
                use(pq, d);
            }
        };
        float u[2] = {bv[0], bv[1]}, own[2] = {0.f, 0.f};
        rows([&](int pq, const float (&d)[4]) {
            if (pq == 4) {
                own[0] = d[1];
                own[1] = d[2];
            }
#pragma unroll
            for (int cc = 0; cc < 3; ++cc)
#pragma unroll
                for (int c = 0; c < 2; ++c) u[c] = fmaf(w[pq * 3 + cc][c], d[c + cc], u[c]);
        });
        float delta[2], out[2];
#pragma unroll
        for (int c = 0; c < 2; ++c) {
            float f, d;
            Act<ACT, float>::fd(u[c], f, d);
            if (kLate) {
                // the step's raw output as the forward formed it (fwd_rows.hip: the same multiply-adds in
                // the same order), instead of reading it back: a quarter of this kernel's reads
                const float yh = (fmaf(rv[c], f, own[c]) - nyc[0]) * nyc[1];
                dgam[c] = fmaf(gcur[c], yh, dgam[c]);
                dbet[c] += gcur[c];
                g[c] = nyc[1] * (gam[c] * gcur[c] - nyc[2] - yh * nyc[3]);
            }
            delta[c] = d * g[c] * rv[c];
            dr[c] = fmaf(f, g[c], dr[c]);
            db[c] += delta[c];
            // the direct part of dx (the residual loop's dn: G' - G' = 0)
            out[c] = (RES ? 0.f : g[c]) + (dx_accumulate ? keep[c] : 0.f);
        }
        const long o = (long)s * cells + grow;
        store_cells<2>(delta_out + o, delta);
        store_cells<2>(dx + o, out);
        if (RES && ln.g_out) store_cells<2>(ln.g_out + o, gin);
        if (LN && !RES) {
            if (sums_here) {
                float t1 = 0.f, t2 = 0.f;
#pragma unroll
                for (int c = 0; c < 2; ++c) {
                    t1 = fmaf(gam[c], out[c], fmaf(delta[c], wgam[c], t1));
                    t2 = fmaf(out[c], own[c] - bet[c], fmaf(delta[c], u[c] - bwb[c], t2));
                }
                const float w1 = slot_wave_sum<64>(t1), w2 = slot_wave_sum<64>(t2);
                if ((tid & 63) == 0) {
                    float *to = ln.x_part + (((long)s * ntube + tube) * (nt / 64) + tid / 64) * 2;
                    to[0] = w1;
                    to[1] = w2;
                }
            }
        }
        rows([&](int pq, const float (&d)[4]) {
#pragma unroll
            for (int cc = 0; cc < 3; ++cc)
#pragma unroll
                for (int c = 0; c < 2; ++c) nw[pq * 3 + cc][c] = fmaf(d[c + cc], delta[c], nw[pq * 3 + cc][c]);
        });
    }
    // ---- parameter gradients: plain stores of whole rows ----
#pragma unroll
    for (int pq = 0; pq < 9; ++pq) {
        nw[pq * 3][0] *= keep_first;
        nw[pq * 3 + 2][1] *= keep_last;
    }
    if (param_mode == kParamAddExclusive) {  // add-in-place mode: on top of what the buffers hold
        auto add_old = [&](const float *from, float (&v)[2]) {
            float old[2];
            load_cells<2>(from + grow, old);
            v[0] += old[0];
            v[1] += old[1];
        };
#pragma unroll
        for (int t = 0; t < 27; ++t) add_old(dweight + t * cells, nw[t]);
        add_old(dbias, db);
        add_old(dscale, dr);
        if (LN) {
            add_old(ln.dgamma, dgam);
            add_old(ln.dbeta, dbet);
        }
    }
#pragma unroll
    for (int t = 0; t < 27; ++t) store_cells<2>(dweight + t * cells + grow, nw[t]);
    store_cells<2>(dbias + grow, db);
    store_cells<2>(dscale + grow, dr);
    if (LN) {
        store_cells<2>(ln.dgamma + grow, dgam);
        store_cells<2>(ln.dbeta + grow, dbet);
    }
}

bool k_ok(int K) { return K == 16 || K == 32 || K == 64; }

template <int ACT, bool LN, bool RES> int launch(const StepArgs &a, hipStream_t st) {
    auto kern = bwd_rows<ACT, LN, RES>;
    const long cells = (long)a.M * a.N * a.K;
    const int nt = 8 * a.K, ntube = (a.M / kTube) * (a.N / kTube);
    const size_t lds = (size_t)(LN ? 4 : 2) * kWinRows * a.K * sizeof(float);
    static int per_cu_cache[3] = {0, 0, 0};  // per instantiation, by K
    int &per_cu = per_cu_cache[a.K == 16 ? 0 : a.K == 32 ? 1 : 2];
    if (per_cu == 0) {
        int n = 0;
        if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, kern, nt, lds) != hipSuccess || n < 1) n = 1;
        per_cu = n;
    }
    // chunks of the batch: enough workgroups to fill the chip, none shorter than eight elements,
    // and no more than there is room for copies of the gradient arrays
    int nchunk = per_cu * plan_device_cus() / ntube;
    if (nchunk > a.B / 8) nchunk = a.B / 8;
    const long slab_floats = kStepSlabPlanes * cells;
    const int room = plan_slab_capacity(a.slabs, a.slab_bytes, slab_floats);
    if (nchunk > room) nchunk = room;
    if (nchunk < 2) nchunk = 1;
    const int chunk_len = (a.B + nchunk - 1) / nchunk;
    nchunk = (a.B + chunk_len - 1) / chunk_len;
    const bool split = nchunk > 1;
    const bool new_params = (a.flags & GRIDNET_OVERWRITE_PARAMS) != 0;
    const int param_mode = split || new_params ? kParamStore : kParamAddExclusive;
    float *slab = (float *)a.slabs;
    LnFold ln = a.ln;
    if (split && LN) {
        ln.dgamma = slab + 29 * cells;
        ln.dbeta = slab + 30 * cells;
    }
    const int dx_accumulate = (a.flags & GRIDNET_OVERWRITE_DX) ? 0 : 1;
    hipLaunchKernelGGL(kern, dim3(padded_grid(ntube, nchunk)), dim3(nt), lds, st, (const float *)a.weight,
                       (const float *)a.bias, (const float *)a.scale, (const float *)a.x, (const float *)a.dy,
                       split ? slab : (float *)a.dweight, split ? slab + 27 * cells : (float *)a.dbias,
                       split ? slab + 28 * cells : (float *)a.dscale, (float *)a.dx, (float *)a.workspace, a.B, a.M,
                       a.N, a.K, ntube, nchunk, chunk_len, param_mode, dx_accumulate, ln, split ? slab_floats : 0L);
    if (int rc = check_launch("bwd_rows")) return rc;
    if (split) {
        SlabTargets t{};
        t.dst[0] = (float *)a.dweight; t.end[0] = 27 * cells;
        t.dst[1] = (float *)a.dbias;   t.end[1] = 28 * cells;
        t.dst[2] = (float *)a.dscale;  t.end[2] = 29 * cells;
        t.count = 3;
        if (LN) {
            t.dst[3] = a.ln.dgamma; t.end[3] = 30 * cells;
            t.dst[4] = a.ln.dbeta;  t.end[4] = 31 * cells;
            t.count = 5;
        }
        // the LayerNorm sums the kernel above left per wave are finished by spare workgroups of this one
        SumsJob job{nullptr, 0, 0, 0, nullptr};
        if (bwd_rows_leaves_sums(a)) job = SumsJob{a.ln.x_part, bwd_rows_pairs(a), a.B, cells, a.ln.x_sums};
        if (int rc = plan_reduce_slabs(slab, nchunk, slab_floats, t, new_params ? 0 : 1, st, job)) return rc;
    } else if (bwd_rows_leaves_sums(a)) {
        if (int rc = layernorm_finalize_sums(a.ln.x_part, bwd_rows_pairs(a), cells, a.ln.x_sums, a.B, st)) return rc;
    }
    // dx holds its direct part, the scratch tensor delta: the sum over the neighbours' deltas, all
    // 27 taps of it; the LayerNorm sums of the finished rows only where the kernel above left them out
    const bool sums_here = LN && !RES && a.ln.x_stats && a.ln.x_part;
    return cross_rows_full_launch(a, st, !sums_here);
}

template <int ACT> int dispatch(const StepArgs &a, hipStream_t st) {
    if (a.ln.gamma && a.ln.residual) return launch<ACT, true, true>(a, st);
    if (a.ln.gamma) return launch<ACT, true, false>(a, st);
    return launch<ACT, false, false>(a, st);
}

}  // namespace

bool bwd_rows_supports(const StepArgs &a) {
    return a.dtype == GRIDNET_F32 && a.inner == 1 && !a.normalize && (a.block_size == 4 || a.block_size == 8) &&
           k_ok(a.K) && a.M % 4 == 0 && a.N % 4 == 0 && cross_rows_supports(a);
}

bool bwd_rows_leaves_sums(const StepArgs &a) {
    return bwd_rows_supports(a) && a.ln.gamma && !a.ln.residual && a.ln.x_stats && a.ln.x_part && a.ln.x_sums;
}

int bwd_rows_pairs(const StepArgs &a) {
    if (a.ln.residual) return cross_rows_pairs(a);
    return (a.M / kTube) * (a.N / kTube) * (8 * a.K / 64);
}

// room for per-chunk copies of the gradient arrays that lets the batch be split as far as the
// kernel likes (three workgroups per CU, none with fewer than eight elements)
size_t bwd_rows_slab_bytes(const StepArgs &a) {
    const long ntube = (long)(a.M / kTube) * (a.N / kTube);
    long chunks = 3L * plan_device_cus() / ntube;
    if (chunks > a.B / 8) chunks = a.B / 8;
    if (chunks < 2) return 0;
    return (size_t)chunks * kStepSlabPlanes * a.M * a.N * a.K * sizeof(float);
}

int bwd_rows_launch(const StepArgs &a, hipStream_t st) {
    switch (a.activation) {
        case GRIDNET_ACT_RELU: return dispatch<GRIDNET_ACT_RELU>(a, st);
        case GRIDNET_ACT_LEAKY_RELU: return dispatch<GRIDNET_ACT_LEAKY_RELU>(a, st);
        case GRIDNET_ACT_SILU: return dispatch<GRIDNET_ACT_SILU>(a, st);
        case GRIDNET_ACT_TANH: return dispatch<GRIDNET_ACT_TANH>(a, st);
    }
    return fail(GRIDNET_ERR_ACTIVATION, "unknown activation function: id %d", a.activation);
}

}  // namespace gridnet
