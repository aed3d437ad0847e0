// The forward of a step with ONE inner iteration, dealt by whole K-rows.
//
// With a single inner iteration nothing is stale: every tap, inside the block or across a block
// boundary, reads the step's input (gridnet/backend_torch.py:61-106 with inner_iterations = 1;
// the halo copy equals the neighbours' values).  The step is then a plain 27-tap stencil with
// per-cell weights over the whole grid, zero outside it, and the block size does not enter:
//   y[c] = x[c] + r[c] act(b[c] + sum_t w[t, c] x[c + off_t]).
// The block kernels (step_fast.hip) pay per batch element for what serves many iterations there
// (a window commit, barriers between iterations, 32-byte pieces of rows); with one iteration
// that is most of their time.  Here a workgroup takes a tube of 4 x 4 whole grid rows, a thread
// owns 4 cells along K with their 108 weights in registers for its share of the batch, the
// 6 x 6 rows in and around the tube wait in LDS (two stages alternating, one barrier per batch
// element), and a thread reads one aligned 16-byte piece of each of nine rows, with the cell
// before and after it from the neighbouring lanes.  Memory is touched in whole rows.
//
// LN (the LayerNorm of the network body folded in, see LnFold): the rows are normalised as they
// are committed to LDS, gamma and beta of the tube's rows waiting in LDS beside them; every wave
// leaves (mean, M2) of its 256 results.  RES: the residual form of the loop, the result is the
// RAW input plus the update.

#include "common.h"
#include "fast_tiles.h"
#include "launch.h"
#include "plan.h"

namespace gridnet {

namespace {

constexpr int kRowsTube = 4;                                  // the tube is 4 x 4 grid rows
constexpr int kRowsWin = (kRowsTube + 2) * (kRowsTube + 2);  // rows in and around it
constexpr int kRowsRpt = (kRowsWin + 15) / 16;               // rows a thread moves

template <int ACT, bool LN, bool RES>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(RES ? 2 : 3, 3)))  // RES: four more values per thread
void fwd_rows(const float *__restrict__ weight, const float *__restrict__ bias, const float *__restrict__ scale,
              const float *__restrict__ x, float *__restrict__ y, int B, int M, int N, int K, int ntube,
              int nchunk, int chunk_len, LnFold ln) {
    static_assert(LN || !RES, "the residual form comes with the folded LayerNorm");
    // [2 stages][36 rows][K]; LN: then gamma and beta of the 36 rows
    extern __shared__ __attribute__((aligned(16))) float lds[];

    int tube, chunk;
    if (!split_block_id(ln.walk_reverse ? reversed_on_its_xcd(blockIdx.x, gridDim.x) : blockIdx.x, ntube, nchunk,
                        tube, chunk))
        return;  // grid padding
    const int kb = K / 4, nt = 16 * kb, tid = threadIdx.x;  // kb: threads along a row
    const int bk = tid % kb, r = tid / kb, ci = r / kRowsTube, cj = r % kRowsTube;
    const int nbj = N / kRowsTube, p0 = (tube / nbj) * kRowsTube, q0 = (tube % nbj) * kRowsTube;
    const long cells = (long)M * N * K;
    const int grow = ((p0 + ci) * N + (q0 + cj)) * K + 4 * bk;  // this thread's four cells
    const bool ln_in = LN && ln.x_stats != nullptr;  // x is the raw output of the step before

    float w[9][3][4], bv[4], rv[4];
#pragma unroll
    for (int pq = 0; pq < 9; ++pq)
#pragma unroll
        for (int cc = 0; cc < 3; ++cc) load_cells<4>(weight + (pq * 3 + cc) * cells + grow, w[pq][cc]);
    load_cells<4>(bias + grow, bv);
    load_cells<4>(scale + grow, rv);
    // the taps that would leave the row along K: their weights are zeroed instead of the value the
    // neighbouring lane (a piece of another row) sends
    const float keep_first = bk == 0 ? 0.f : 1.f, keep_last = bk == kb - 1 ? 0.f : 1.f;
#pragma unroll
    for (int pq = 0; pq < 9; ++pq) {
        w[pq][0][0] *= keep_first;
        w[pq][2][3] *= keep_last;
    }

    // ---- the rows this thread moves: rows r, r + 16 and (the first four r) r + 32 ----
    int goff[kRowsRpt], loff[kRowsRpt];
    bool ok[kRowsRpt];
    float *gam_rows = lds + 2 * kRowsWin * K, *bet_rows = gam_rows + kRowsWin * K;
#pragma unroll
    for (int e = 0; e < kRowsRpt; ++e) {
        const int row = r + 16 * e, wi = row / (kRowsTube + 2), wj = row % (kRowsTube + 2);
        const int gi = p0 + wi - 1, gj = q0 + wj - 1;
        ok[e] = row < kRowsWin && gi >= 0 && gi < M && gj >= 0 && gj < N;
        goff[e] = ok[e] ? (gi * N + gj) * K + 4 * bk : grow;  // anything valid when not used
        loff[e] = row * K + 4 * bk;
        if (ln_in && row < kRowsWin) {
            // gamma and beta of the row, once per workgroup; zeros for a row outside the grid, which
            // makes whatever is loaded in its place a zero without a test per element
            float gq[4], bq[4];
            load_cells<4>(ln.gamma + goff[e], gq);
            load_cells<4>(ln.beta + goff[e], bq);
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                gq[q] = ok[e] ? gq[q] : 0.f;
                bq[q] = ok[e] ? bq[q] : 0.f;
            }
            store_cells<4>(gam_rows + loff[e], gq);
            store_cells<4>(bet_rows + loff[e], bq);
        }
    }
    const bool has_last = r + 16 * (kRowsRpt - 1) < kRowsWin;
    const int own_row = (ci + 1) * (kRowsTube + 2) + (cj + 1);
    wait_global_loads();

    const int s0 = chunk * chunk_len, s1 = min(B, s0 + chunk_len);
    float xbuf[kRowsRpt][4], raw[4], xmean = 0.f, xrstd = 1.f;
    auto fetch = [&](int s) {
        const long at = (long)s * cells;
        if (RES) load_cells<4>(x + at + grow, raw);
        if (ln_in) {
            xmean = load_ahead(ln.x_stats, 2 * s);
            xrstd = load_ahead(ln.x_stats, 2 * s + 1);
        }
#pragma unroll
        for (int e = 0; e < kRowsRpt; ++e) load_cells<4>(x + at + goff[e], xbuf[e]);
    };
    if (s0 < s1) fetch(s0);
    for (int s = s0; s < s1; ++s) {
        float *stage = lds + ((s - s0) & 1) * kRowsWin * K;
#pragma unroll
        for (int e = 0; e < kRowsRpt; ++e) {
            if (e == kRowsRpt - 1 && !has_last) break;
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
        float base[4];
#pragma unroll
        for (int c = 0; c < 4; ++c) base[c] = RES ? raw[c] : 0.f;
        lds_barrier();  // the stage is complete (the first: gamma and beta too); the other one's readers are done
        fetch(min(s + 1, s1 - 1));
        // the requests leave now, with the whole stencil in front of the element that needs them
        // (left to itself the compiler sinks two of the three past it)
        __builtin_amdgcn_sched_barrier(0);
        float u[4], own[4];
#pragma unroll
        for (int c = 0; c < 4; ++c) u[c] = bv[c];
        // taps in the reference's order: rows (di, dj), along K inside a row
#pragma unroll
        for (int pq = 0; pq < 9; ++pq) {
            const int di = pq / 3 - 1, dj = pq % 3 - 1;
            float d[6], mid[4];
            load_cells<4>(stage + (own_row + di * (kRowsTube + 2) + dj) * K + 4 * bk, mid);
            d[0] = lane_before(mid[3]);
            d[5] = lane_after(mid[0]);
#pragma unroll
            for (int c = 0; c < 4; ++c) d[c + 1] = mid[c];
            if (pq == 4) {
#pragma unroll
                for (int c = 0; c < 4; ++c) own[c] = mid[c];
            }
#pragma unroll
            for (int cc = 0; cc < 3; ++cc)
#pragma unroll
                for (int c = 0; c < 4; ++c) u[c] = fmaf(w[pq][cc][c], d[c + cc], u[c]);
        }
        float out[4];
#pragma unroll
        for (int c = 0; c < 4; ++c) out[c] = fmaf(rv[c], Act<ACT, float>::f(u[c]), RES ? base[c] : own[c]);
        store_cells<4>(y + (long)s * cells + grow, out);
        if (LN && ln.y_part) {
            // statistics of the result for the LayerNorm that follows: one (mean, M2) pair per wave
            const float sum = (out[0] + out[1]) + (out[2] + out[3]);
            const float mean = row16_sum(sum) * (1.f / 64);
            float m2 = 0.f;
#pragma unroll
            for (int c = 0; c < 4; ++c) m2 = fmaf(out[c] - mean, out[c] - mean, m2);
            m2 = row16_sum(m2);
            float wave_mean, wave_m2;
            slot_wave_moments<64>(mean, m2, 64, wave_mean, wave_m2);
            if ((tid & 63) == 0) {
                const int nwave = nt / 64;
                float *to = ln.y_part + (((long)s * ntube + tube) * nwave + tid / 64) * 2;
                to[0] = wave_mean;
                to[1] = wave_m2;
            }
        }
    }
}

bool k_ok(int K) { return K == 16 || K == 32 || K == 64 || K == 128; }

template <int ACT, bool LN, bool RES> int launch(const StepArgs &a, hipStream_t st) {
    auto kern = fwd_rows<ACT, LN, RES>;
    const int nt = 4 * a.K, ntube = (a.M / kRowsTube) * (a.N / kRowsTube);
    const size_t lds = (size_t)(LN ? 4 : 2) * kRowsWin * a.K * sizeof(float);
    static bool big_lds_enabled = false;  // per instantiation
    if (lds > 64 * 1024 && !big_lds_enabled) {
        if (hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024) != hipSuccess) {
            (void)hipGetLastError();
            return fail(GRIDNET_ERR_LAUNCH, "fwd_rows: cannot enable %zu bytes of LDS", lds);
        }
        big_lds_enabled = true;
    }
    static int per_cu_cache[4] = {0, 0, 0, 0};  // per instantiation, by K
    int &per_cu = per_cu_cache[a.K == 16 ? 0 : a.K == 32 ? 1 : a.K == 64 ? 2 : 3];
    if (per_cu == 0) {
        int n = 0;
        if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, kern, nt, lds) != hipSuccess || n < 1) n = 1;
        per_cu = n;
    }
    // chunks of the batch: enough workgroups to fill the chip, but none that walks fewer than
    // eight elements for its one fetch of the weights (32^3 grid, batch 256: chunks of 11 beat
    // chunks of 16, 32 and 64 elements, 10.33 against 10.42, 11.9 and 14.3 ms per 64-step training
    // step: what limits the kernel is the trip to memory per element, and more workgroups hide it)
    int nchunk = per_cu * plan_device_cus() / ntube;
    if (nchunk > a.B / 8) nchunk = a.B / 8;
    if (nchunk < 1) nchunk = 1;
    const int chunk_len = (a.B + nchunk - 1) / nchunk;
    nchunk = (a.B + chunk_len - 1) / chunk_len;
    hipLaunchKernelGGL(kern, dim3(padded_grid(ntube, nchunk)), dim3(nt), lds, st, (const float *)a.weight,
                       (const float *)a.bias, (const float *)a.scale, (const float *)a.x, (float *)a.y, a.B, a.M,
                       a.N, a.K, ntube, nchunk, chunk_len, a.ln);
    return check_launch("fwd_rows");
}

template <int ACT> int dispatch(const StepArgs &a, hipStream_t st) {
    if (a.ln.gamma && a.ln.residual) return launch<ACT, true, true>(a, st);
    if (a.ln.gamma) return launch<ACT, true, false>(a, st);
    return launch<ACT, false, false>(a, st);
}

}  // namespace

bool fwd_rows_supports(const StepArgs &a) {
    return a.dtype == GRIDNET_F32 && a.inner == 1 && !a.normalize && (a.block_size == 4 || a.block_size == 8) &&
           k_ok(a.K) && a.M % 4 == 0 && a.N % 4 == 0;
}

// (mean, M2) pairs per sample that it leaves in a.ln.y_part, each over 256 cells
int fwd_rows_pairs(const StepArgs &a) { return (int)((long)a.M * a.N * a.K / 256); }

int fwd_rows_launch(const StepArgs &a, hipStream_t st) {
    switch (a.activation) {
        case GRIDNET_ACT_RELU: return dispatch<GRIDNET_ACT_RELU>(a, st);
        case GRIDNET_ACT_LEAKY_RELU: return dispatch<GRIDNET_ACT_LEAKY_RELU>(a, st);
        case GRIDNET_ACT_SILU: return dispatch<GRIDNET_ACT_SILU>(a, st);
        case GRIDNET_ACT_TANH: return dispatch<GRIDNET_ACT_TANH>(a, st);
    }
    return fail(GRIDNET_ERR_ACTIVATION, "unknown activation function: id %d", a.activation);
}

}  // namespace gridnet
