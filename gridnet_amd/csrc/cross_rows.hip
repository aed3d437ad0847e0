// The cross-block part of the backward, dealt by whole K-rows.
//
// step_bwd_fast leaves D = sum_i delta_i of every cell and the block-local part of dx.  What is
// still owed to a cell c is, over the taps t whose neighbour h = c + off_t lies in ANOTHER block,
//   dx[c] += W[26-t, h] * D[h]
// (the reference scatters these through its window atomics, src/gridnet_cuda_kernels.cu:424-449).
// A block's row along K is 16 or 32 bytes: a workgroup per block touches memory in pieces of that
// size that lie a whole grid row apart (and with 4^3 blocks 56 of a block's 64 cells have such
// taps).  Here a workgroup takes a TUBE instead: 16 whole grid rows, 4 x 4 x K cells with 4^3
// blocks (the K/4 blocks that share a block row and column), 2 x 8 x K with 8^3 blocks (a quarter
// of such a row of blocks).  A thread owns 4 cells along K (lanes run along K, so the rows of
// the tube are read and written as whole contiguous rows) and keeps the mirrored weights of all
// its (cell, tap) pairs in registers for its share of the batch, zero where the tap stays inside
// the block or leaves the grid: the arithmetic is the plain 27-tap stencil on D, uniform for all
// threads.  D of the rows in and around the tube waits in LDS, two stages alternating, one
// barrier per batch element; a thread reads 16-byte pieces of nine rows and gets the two cells
// beside a piece from the lanes next to it (a wave shift, no LDS access).
//
// LN as in step_bwd_cross (LnFold): with the LayerNorm of the network body folded in the finished
// rows also give the two per-sample sums of that LayerNorm's backward, one pair per wave.  (The
// residual form of the loop needs nothing here: step_bwd_fast takes G' off the cells' own part.)
// NORM (per-window normalisation, see step_bwd_fast): `dsum` holds D1, and a cell that lies in the
// halo of a neighbouring block a additionally receives R_a - x Q_a, with (Q, R) the two numbers
// per (element, block) that step_bwd_fast left in `qr`.  All threads of a tube have the same 3 x 3
// columns of blocks around them: their (Q, R) travel through LDS with the D rows.
// SETS = 2: the gated variant of the update (weight [27, 2, M, N, K]): two D tensors, one behind
// the other in `dsum`, each with its own set of mirrored weights; the cell receives the sum.

#include "common.h"
#include "fast_tiles.h"
#include "launch.h"
#include "plan.h"

namespace gridnet {

namespace {

// a tube is RI x RJ grid rows (16 of them), the D rows in and around it (RI + 2) x (RJ + 2)
template <int BS> struct Tube {
    static constexpr int RI = 16 / BS, RJ = BS, WJ = RJ + 2, ROWS = (RI + 2) * WJ;
    static constexpr int RPT = (ROWS + 15) / 16;  // D rows a thread moves
    static_assert(BS == 4 || BS == 8, "block sizes 4 and 8");
};

// FULL: ALL taps, not only those that leave the block: the second kernel of the backward of a step
// with one inner iteration (bwd_rows.hip), where `dsum` holds delta of every cell and dx the
// direct part of the gradient.
template <int BS, bool LN, bool NORM = false, int SETS = 1, bool FULL = false>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(SETS == 1 ? 3 : 2, SETS == 1 ? 3 : 2)))
void cross_rows(const float *__restrict__ weight, const float *__restrict__ x,
                const float *__restrict__ dsum, float *__restrict__ dx, int B, int M, int N, int K,
                int ntube, int nchunk, int chunk_len, LnFold ln, const float *__restrict__ qr) {
    using TB = Tube<BS>;
    static_assert(!(NORM && LN), "the folded LayerNorm comes without normalisation");
    static_assert(SETS == 1 || !(LN || NORM), "the gated update has no variants");
    // [2 stages][SETS][TB::ROWS][K]; NORM: then [2 stages][3 x 3 columns of blocks][K / BS + 2] (Q, R) pairs
    extern __shared__ __attribute__((aligned(16))) float lds[];

    int tube, chunk;
    if (!split_block_id(blockIdx.x, ntube, nchunk, tube, chunk)) return;  // grid padding
    const int kb = K / 4, nt = 16 * kb, tid = threadIdx.x;  // kb: threads along a row
    const int bk = tid % kb, r = tid / kb, ci = r / TB::RJ, cj = r % TB::RJ;
    const int nbj = N / TB::RJ, p0 = (tube / nbj) * TB::RI, q0 = (tube % nbj) * TB::RJ;
    // where the thread's row and its first cell lie inside their block
    const int bi = (p0 + ci) % BS, bj = cj, bk0 = (4 * bk) % BS;
    const long cells = (long)M * N * K;
    const int grow = ((p0 + ci) * N + (q0 + cj)) * K + 4 * bk;  // this thread's four cells
    const bool first = bk == 0, last = bk == kb - 1;

    // ---- mirrored weights of the pairs (cell, tap) that cross a block boundary ----
    float vx[SETS][9][3][4];
#pragma unroll
    for (int pq = 0; pq < 9; ++pq) {
        const int di = pq / 3 - 1, dj = pq % 3 - 1;
        const int gi = p0 + ci + di, gj = q0 + cj + dj;
        const bool side = bi + di < 0 || bi + di >= BS || bj + dj < 0 || bj + dj >= BS;
        const bool row_ok = gi >= 0 && gi < M && gj >= 0 && gj < N;
        // A tap's four weights W[26-t, h] for the thread's cells lie side by side along K, one
        // cell off its own four for dk = -1 / +1: one aligned 16-byte load per tap (every lane of
        // the row loads its own piece of the same plane and row) and the missing end from the lane
        // next door, instead of four scattered 4-byte loads.
        const int rowbase = row_ok ? (gi * N + gj) * K + 4 * bk : grow;
#pragma unroll
        for (int k = 0; k < SETS; ++k)
#pragma unroll
            for (int dk = -1; dk <= 1; ++dk) {
                const int t = (di + 1) * 9 + (dj + 1) * 3 + (dk + 1);
                float piece[4];
                load_cells<4>(weight + ((26 - t) * SETS + k) * cells + rowbase, piece);
                const float before = lane_before(piece[3]), after = lane_after(piece[0]);
#pragma unroll
                for (int ck = 0; ck < 4; ++ck) {
                    // a tap along K can only cross where it leaves the thread's four cells (known
                    // when compiling); taps that never cross are not held at all
                    if (!FULL && pq == 4 && !(ck + dk < 0 || ck + dk > 3)) continue;
                    const bool along = bk0 + ck + dk < 0 || bk0 + ck + dk >= BS;
                    const int gk = 4 * bk + ck + dk;
                    const bool use = (FULL || side || along) && row_ok && gk >= 0 && gk < K;
                    const float wv = ck + dk < 0 ? before : ck + dk > 3 ? after : piece[(ck + dk) & 3];
                    vx[k][pq][dk + 1][ck] = use ? wv : 0.f;
                }
            }
    }
    const bool ln_in = LN && ln.x_stats != nullptr;
    float gam[4] = {0.f, 0.f, 0.f, 0.f};
    if (ln_in) load_cells<4>(ln.gamma + grow, gam);

    // ---- the D rows this thread moves: rows r, r + 16, ... while there are any ----
    constexpr int RPT = TB::RPT;
    int goff[RPT], loff[RPT];
    bool ok[RPT];
#pragma unroll
    for (int e = 0; e < RPT; ++e) {
        const int row = r + 16 * e, wi = row / TB::WJ, wj = row % TB::WJ;
        const int gi = p0 + wi - 1, gj = q0 + wj - 1;
        ok[e] = row < TB::ROWS && gi >= 0 && gi < M && gj >= 0 && gj < N;
        goff[e] = ok[e] ? (gi * N + gj) * K + 4 * bk : grow;  // anything valid when not used
        loff[e] = row * K + 4 * bk;
    }
    const bool has_last = r + 16 * (RPT - 1) < TB::ROWS;
    const int own_row = (ci + 1) * TB::WJ + (cj + 1);

    // NORM: (Q, R) of the blocks in the 3 x 3 columns around the tube's own, a row of K / BS blocks
    // each with a zero pair at either end; thread n < 9 K / BS moves one pair per element
    const int nbk = K / BS, qrow = nbk + 2;
    float2 *qrs = reinterpret_cast<float2 *>(lds + 2 * SETS * TB::ROWS * K);  // [2][9][qrow]
    long qr_from = -1;
    int qr_to = 0;
    // which columns hold blocks that have this thread's row in their halo (beside its own), and
    // where its own block sits in a row of pairs
    const int ei = bi == 0 ? -1 : bi == BS - 1 ? 1 : 0, ej = bj == 0 ? -1 : bj == BS - 1 ? 1 : 0;
    const int kcol = 4 * bk / BS + 1;
    if (NORM) {
        const int nblk_j = N / BS, col_i = p0 / BS, col_j = q0 / BS;
        if (tid < 9 * nbk) {
            const int a = tid / (3 * nbk), b = (tid / nbk) % 3, kk = tid % nbk;
            const int gi = col_i + a - 1, gj = col_j + b - 1;
            qr_to = (a * 3 + b) * qrow + kk + 1;
            if (gi >= 0 && gi < M / BS && gj >= 0 && gj < nblk_j) qr_from = ((long)gi * nblk_j + gj) * nbk + kk;
        }
        if (tid < 36) {  // the zero pairs at the ends of the rows, both stages, once
            const int st = tid / 18, row = (tid % 18) / 2, end = tid & 1;
            qrs[(st * 9 + row) * qrow + (end ? qrow - 1 : 0)] = make_float2(0.f, 0.f);
        }
    }
    wait_global_loads();

    const int s0 = chunk * chunk_len, s1 = min(B, s0 + chunk_len);
    float dbuf[SETS][RPT][4], gx[4], xr[4], xmean = 0.f, xrstd = 1.f;
    float2 qbuf = make_float2(0.f, 0.f);
    const long nblk = (long)(M / BS) * (N / BS) * nbk;
    auto fetch = [&](int s) {
        const long at = (long)s * cells;
        load_cells<4>(dx + at + grow, gx);
        if (NORM) {
            load_cells<4>(x + at + grow, xr);
            // (every thread loads, a valid address always; the commit selects)
            qbuf = *reinterpret_cast<const float2 *>(qr + (s * nblk + (qr_from >= 0 ? qr_from : 0)) * 2);
        }
        if (ln_in) {
            load_cells<4>(x + at + grow, xr);
            xmean = load_ahead(ln.x_stats, 2 * s);
            xrstd = load_ahead(ln.x_stats, 2 * s + 1);
        }
#pragma unroll
        for (int k = 0; k < SETS; ++k)
#pragma unroll
            for (int e = 0; e < RPT; ++e) load_cells<4>(dsum + (long)k * B * cells + at + goff[e], dbuf[k][e]);
    };
    if (s0 < s1) fetch(s0);
    for (int s = s0; s < s1; ++s) {
        float *stage = lds + ((s - s0) & 1) * SETS * TB::ROWS * K;
#pragma unroll
        for (int k = 0; k < SETS; ++k)
#pragma unroll
            for (int e = 0; e < RPT; ++e) {
                if (e == RPT - 1 && !has_last) break;
                float v[4];
#pragma unroll
                for (int q = 0; q < 4; ++q) v[q] = ok[e] ? dbuf[k][e][q] : 0.f;
                store_cells<4>(stage + k * TB::ROWS * K + loff[e], v);
            }
        const float2 *qst = qrs + ((s - s0) & 1) * 9 * qrow;
        if (NORM && tid < 9 * nbk)
            qrs[((s - s0) & 1) * 9 * qrow + qr_to] = qr_from >= 0 ? qbuf : make_float2(0.f, 0.f);
        float g[4], xc[4];
        const float mean = xmean, rstd = xrstd;
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            g[c] = gx[c];
            xc[c] = (ln_in || NORM) ? xr[c] : 0.f;
        }
        lds_barrier();  // the stage is complete; the readers of the other one are done
        fetch(min(s + 1, s1 - 1));
        // fixed order per cell: rows (di, dj) in tap order, along K inside a row
#pragma unroll
        for (int k = 0; k < SETS; ++k)
#pragma unroll
        for (int pq = 0; pq < 9; ++pq) {
            const int di = pq / 3 - 1, dj = pq % 3 - 1;
            float d[6];
            float mid[4];
            load_cells<4>(stage + (k * TB::ROWS + own_row + di * TB::WJ + dj) * K + 4 * bk, mid);
            const float before = lane_before(mid[3]), after = lane_after(mid[0]);
            d[0] = first ? 0.f : before;
            d[5] = last ? 0.f : after;
#pragma unroll
            for (int c = 0; c < 4; ++c) d[c + 1] = mid[c];
#pragma unroll
            for (int dk = -1; dk <= 1; ++dk)
#pragma unroll
                for (int ck = 0; ck < 4; ++ck) {
                    if (!FULL && pq == 4 && !(ck + dk < 0 || ck + dk > 3)) continue;
                    g[ck] = fmaf(vx[k][pq][dk + 1][ck], d[ck + 1 + dk], g[ck]);
                }
        }
        if (NORM) {
            // blocks that have the cell in their halo, by their offset along K: the columns
            // (0, 0), (ei, 0), (0, ej), (ei, ej) as far as the row lies on that side of its block;
            // at offset 0 the block itself is left out, offsets -1 / +1 concern the cell at that
            // end of the block only
            float sq[3] = {0.f, 0.f, 0.f}, sr[3] = {0.f, 0.f, 0.f};
#pragma unroll
            for (int ia = 0; ia < 2; ++ia)
#pragma unroll
                for (int ib = 0; ib < 2; ++ib) {
                    const bool use = (ia == 0 || ei != 0) && (ib == 0 || ej != 0);
                    const float2 *row = qst + ((1 + ia * ei) * 3 + (1 + ib * ej)) * qrow + kcol;
#pragma unroll
                    for (int dk = 0; dk < 3; ++dk) {
                        if (dk == 1 && ia == 0 && ib == 0) continue;
                        const float2 v = row[dk - 1];
                        sq[dk] += use ? v.x : 0.f;
                        sr[dk] += use ? v.y : 0.f;
                    }
                }
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                g[c] += fmaf(-xc[c], sq[1], sr[1]);
                if (c == 0 && bk0 == 0) g[c] += fmaf(-xc[c], sq[0], sr[0]);
                if (c == 3 && bk0 + 3 == BS - 1) g[c] += fmaf(-xc[c], sq[2], sr[2]);
            }
        }
        store_cells<4>(dx + (long)s * cells + grow, g);
        if (ln_in) {
            float t1 = 0.f, t2 = 0.f;
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                const float a = gam[c] * g[c];
                t1 += a;
                t2 = fmaf(a, (xc[c] - mean) * rstd, t2);
            }
            const float w1 = slot_wave_sum<64>(t1), w2 = slot_wave_sum<64>(t2);
            if ((tid & 63) == 0) {
                const int nwave = nt / 64;
                float *to = ln.x_part + (((long)s * ntube + tube) * nwave + tid / 64) * 2;
                to[0] = w1;
                to[1] = w2;
            }
        }
    }
}

bool k_ok(int K) { return K == 16 || K == 32 || K == 64 || K == 128; }

template <int BS, bool LN, bool NORM = false, int SETS = 1, bool FULL = false>
int launch(const StepArgs &a, const float *dsum, hipStream_t st) {
    using TB = Tube<BS>;
    auto kern = cross_rows<BS, LN, NORM, SETS, FULL>;
    const int nt = 4 * a.K, ntube = (a.M / TB::RI) * (a.N / TB::RJ);
    const size_t lds = ((size_t)2 * SETS * TB::ROWS * a.K + (NORM ? 2 * 9 * (a.K / BS + 2) * 2 : 0)) * sizeof(float);
    static bool big_lds_enabled = false;  // per instantiation
    if (lds > 64 * 1024 && !big_lds_enabled) {
        if (hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024) != hipSuccess) {
            (void)hipGetLastError();
            return fail(GRIDNET_ERR_LAUNCH, "cross_rows: cannot enable %zu bytes of LDS", lds);
        }
        big_lds_enabled = true;
    }
    // NORM: (Q, R) per (element, block) behind the D tensor in the workspace
    const float *qr = NORM ? dsum + (size_t)a.B * a.M * a.N * a.K : nullptr;
    static int per_cu_cache[4] = {0, 0, 0, 0};  // per instantiation, by K
    int &per_cu = per_cu_cache[a.K == 16 ? 0 : a.K == 32 ? 1 : a.K == 64 ? 2 : 3];
    if (per_cu == 0) {
        int n = 0;
        if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, kern, nt, lds) != hipSuccess || n < 1) n = 1;
        per_cu = n;
    }
    // chunks of the batch: enough workgroups to fill the chip, but none that walks fewer than
    // eight elements for its one fetch of the weights
    int nchunk = per_cu * plan_device_cus() / ntube;
    if (nchunk > a.B / 8) nchunk = a.B / 8;
    if (nchunk < 1) nchunk = 1;
    const int chunk_len = (a.B + nchunk - 1) / nchunk;
    nchunk = (a.B + chunk_len - 1) / chunk_len;
    hipLaunchKernelGGL(kern, dim3(padded_grid(ntube, nchunk)), dim3(nt), lds, st, (const float *)a.weight,
                       (const float *)a.x, dsum, (float *)a.dx, a.B, a.M, a.N, a.K,
                       ntube, nchunk, chunk_len, a.ln, qr);
    return check_launch("cross_rows");
}

template <int BS> int dispatch(const StepArgs &a, hipStream_t st) {
    const float *dsum = (const float *)a.workspace;
    if (a.normalize) return launch<BS, false, true>(a, dsum, st);
    if (a.ln.gamma) return launch<BS, true>(a, dsum, st);
    return launch<BS, false>(a, dsum, st);
}

}  // namespace

bool cross_rows_supports(const StepArgs &a) {
    const int bs = a.block_size;
    return a.dtype == GRIDNET_F32 && (bs == 4 || bs == 8) && !(a.normalize && a.ln.gamma) && k_ok(a.K) &&
           a.M % bs == 0 && a.N % bs == 0;
}

// one pair per wave: 16 grid rows of K / 4 threads each per workgroup
int cross_rows_pairs(const StepArgs &a) { return (a.M * a.N / 16) * (4 * a.K / 64); }

int cross_rows_launch(const StepArgs &a, hipStream_t st) {
    return a.block_size == 8 ? dispatch<8>(a, st) : dispatch<4>(a, st);
}

// all 27 taps (the second kernel of bwd_rows.hip); the block size does not enter then
int cross_rows_full_launch(const StepArgs &a, hipStream_t st, bool ln_sums) {
    const float *dsum = (const float *)a.workspace;
    return a.ln.gamma && ln_sums ? launch<4, true, false, 1, true>(a, dsum, st)
                                 : launch<4, false, false, 1, true>(a, dsum, st);
}

// the gated update: weight [27, 2, M, N, K], D0 and D1 of every cell behind one another in `dsum`
bool cross_rows_gated_supports(const StepArgs &a) {
    const int bs = a.block_size;
    return a.dtype == GRIDNET_F32 && (bs == 4 || bs == 8) && k_ok(a.K) && a.M % bs == 0 && a.N % bs == 0;
}
int cross_rows_gated_launch(const StepArgs &a, const float *dsum, hipStream_t st) {
    return a.block_size == 8 ? launch<8, false, false, 2>(a, dsum, st) : launch<4, false, false, 2>(a, dsum, st);
}

}  // namespace gridnet
