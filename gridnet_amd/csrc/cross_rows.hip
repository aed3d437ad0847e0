// The cross-block part of the backward for 4^3 blocks, dealt by whole K-rows.
//
// step_bwd_fast leaves D = sum_i delta_i of every cell and the block-local part of dx.  What is
// still owed to a cell c is, over the taps t whose neighbour h = c + off_t lies in ANOTHER block,
//   dx[c] += W[26-t, h] * D[h]
// (the reference scatters these through its window atomics, src/gridnet_cuda_kernels.cu:424-449).
// With 4^3 blocks 56 of a block's 64 cells have such taps and a block's row along K is 16 bytes:
// a workgroup per block touches memory in 16-byte pieces that lie a whole grid row apart.  Here
// a workgroup takes a TUBE instead: the K/4 blocks that share (block row, block column), 4 x 4 x K
// cells.  A thread owns one block row of 4 cells (lanes run along K, so the 16 rows of the tube
// are read and written as whole contiguous rows) and keeps the mirrored weights of all its
// (cell, tap) pairs in registers for its share of the batch, zero where the tap stays inside the
// block or leaves the grid: the arithmetic is the plain 27-tap stencil on D, uniform for all
// threads.  D of the 6 x 6 rows around the tube waits in LDS, two stages alternating, one barrier
// per batch element; a thread reads 16-byte pieces of nine rows and gets the two cells beside a
// piece from the lanes next to it (a wave shift, no LDS access).
//
// LN / RES as in step_bwd_cross (LnFold): with the LayerNorm of the network body folded in the
// finished rows also give the two per-sample sums of that LayerNorm's backward, one pair per
// wave; the residual loop's G' is subtracted from the rows first.

#include "common.h"
#include "fast_tiles.h"
#include "launch.h"
#include "plan.h"

namespace gridnet {

namespace {

constexpr int kTubeRows = 36;  // 6 x 6 rows of D around (and in) a tube

// the lane before / after in the wave (the caller masks the ends of a row)
__device__ __forceinline__ float lane_before(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x138, 0xf, 0xf, false));
}
__device__ __forceinline__ float lane_after(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x130, 0xf, 0xf, false));
}

template <bool LN, bool RES>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2, 3)))
void cross_rows(const float *__restrict__ weight, const float *__restrict__ x,
                const float *__restrict__ dsum, float *__restrict__ dx, int B, int M, int N, int K,
                int ntube, int nchunk, int chunk_len, LnFold ln) {
    extern __shared__ __attribute__((aligned(16))) float lds[];  // [2 stages][36 rows][K]

    int tube, chunk;
    if (!split_block_id(blockIdx.x, ntube, nchunk, tube, chunk)) return;  // grid padding
    const int kb = K / 4, nt = 16 * kb, tid = threadIdx.x;
    const int bk = tid % kb, r = tid / kb, ci = r >> 2, cj = r & 3;
    const int nbj = N / 4, p0 = (tube / nbj) * 4, q0 = (tube % nbj) * 4;
    const long cells = (long)M * N * K;
    const int grow = ((p0 + ci) * N + (q0 + cj)) * K + 4 * bk;  // this thread's four cells
    const bool first = bk == 0, last = bk == kb - 1;

    // ---- mirrored weights of the pairs (cell, tap) that cross a block boundary ----
    float vx[9][3][4];
#pragma unroll
    for (int pq = 0; pq < 9; ++pq) {
        const int di = pq / 3 - 1, dj = pq % 3 - 1;
        const int gi = p0 + ci + di, gj = q0 + cj + dj;
        const bool side = ci + di < 0 || ci + di > 3 || cj + dj < 0 || cj + dj > 3;
        const bool row_ok = gi >= 0 && gi < M && gj >= 0 && gj < N;
#pragma unroll
        for (int dk = -1; dk <= 1; ++dk)
#pragma unroll
            for (int ck = 0; ck < 4; ++ck) {
                const bool along = ck + dk < 0 || ck + dk > 3;  // known when compiling
                if (pq == 4 && !along) continue;                // never crosses: not held at all
                const int gk = 4 * bk + ck + dk;
                const int t = (di + 1) * 9 + (dj + 1) * 3 + (dk + 1);
                const bool use = (side || along) && row_ok && gk >= 0 && gk < K;
                const long h = ((long)gi * N + gj) * K + gk;
                vx[pq][dk + 1][ck] = use ? weight[(26 - t) * cells + h] : 0.f;
            }
    }
    const bool ln_in = LN && ln.x_stats != nullptr;
    float gam[4] = {0.f, 0.f, 0.f, 0.f};
    if (ln_in) load_cells<4>(ln.gamma + grow, gam);

    // ---- the D rows this thread moves: rows r, r + 16 and (the first four r) r + 32 ----
    int goff[3], loff[3];
    bool ok[3];
#pragma unroll
    for (int e = 0; e < 3; ++e) {
        const int row = r + 16 * e, wi = row / 6, wj = row % 6;
        const int gi = p0 + wi - 1, gj = q0 + wj - 1;
        ok[e] = row < kTubeRows && gi >= 0 && gi < M && gj >= 0 && gj < N;
        goff[e] = ok[e] ? (gi * N + gj) * K + 4 * bk : grow;  // anything valid when not used
        loff[e] = row * K + 4 * bk;
    }
    const bool third = r < kTubeRows - 32;
    const int own_row = (ci + 1) * 6 + (cj + 1);
    wait_global_loads();

    const int s0 = chunk * chunk_len, s1 = min(B, s0 + chunk_len);
    float dbuf[3][4], gx[4], xr[4], gr[4], xmean = 0.f, xrstd = 1.f;
    auto fetch = [&](int s) {
        const long at = (long)s * cells;
        load_cells<4>(dx + at + grow, gx);
        if (RES) load_cells<4>(ln.g_rows + at + grow, gr);
        if (ln_in) {
            load_cells<4>(x + at + grow, xr);
            xmean = load_ahead(ln.x_stats, 2 * s);
            xrstd = load_ahead(ln.x_stats, 2 * s + 1);
        }
#pragma unroll
        for (int e = 0; e < 3; ++e) load_cells<4>(dsum + at + goff[e], dbuf[e]);
    };
    if (s0 < s1) fetch(s0);
    for (int s = s0; s < s1; ++s) {
        float *stage = lds + ((s - s0) & 1) * kTubeRows * K;
#pragma unroll
        for (int e = 0; e < 3; ++e) {
            if (e == 2 && !third) break;
            float v[4];
#pragma unroll
            for (int q = 0; q < 4; ++q) v[q] = ok[e] ? dbuf[e][q] : 0.f;
            store_cells<4>(stage + loff[e], v);
        }
        float g[4], xc[4], grc[4];
        const float mean = xmean, rstd = xrstd;
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            g[c] = gx[c];
            xc[c] = ln_in ? xr[c] : 0.f;
            grc[c] = RES ? gr[c] : 0.f;
        }
        lds_barrier();  // the stage is complete; the readers of the other one are done
        fetch(min(s + 1, s1 - 1));
        // fixed order per cell: rows (di, dj) in tap order, along K inside a row
#pragma unroll
        for (int pq = 0; pq < 9; ++pq) {
            const int di = pq / 3 - 1, dj = pq % 3 - 1;
            float d[6];
            float mid[4];
            load_cells<4>(stage + (own_row + di * 6 + dj) * K + 4 * bk, mid);
            const float before = lane_before(mid[3]), after = lane_after(mid[0]);
            d[0] = first ? 0.f : before;
            d[5] = last ? 0.f : after;
#pragma unroll
            for (int c = 0; c < 4; ++c) d[c + 1] = mid[c];
#pragma unroll
            for (int dk = -1; dk <= 1; ++dk)
#pragma unroll
                for (int ck = 0; ck < 4; ++ck) {
                    if (pq == 4 && !(ck + dk < 0 || ck + dk > 3)) continue;
                    g[ck] = fmaf(vx[pq][dk + 1][ck], d[ck + 1 + dk], g[ck]);
                }
        }
        if (RES) {
#pragma unroll
            for (int c = 0; c < 4; ++c) g[c] -= grc[c];
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

template <bool LN, bool RES> int launch(const StepArgs &a, hipStream_t st) {
    auto kern = cross_rows<LN, RES>;
    const int nt = 4 * a.K, ntube = (a.M / 4) * (a.N / 4);
    const size_t lds = (size_t)2 * kTubeRows * a.K * sizeof(float);
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
                       (const float *)a.x, (const float *)a.workspace, (float *)a.dx, a.B, a.M, a.N, a.K,
                       ntube, nchunk, chunk_len, a.ln);
    return check_launch("cross_rows");
}

}  // namespace

bool cross_rows_supports(const StepArgs &a) {
    return a.dtype == GRIDNET_F32 && a.block_size == 4 && !a.normalize && k_ok(a.K) && a.M % 4 == 0 &&
           a.N % 4 == 0;
}

int cross_rows_pairs(const StepArgs &a) { return (a.M / 4) * (a.N / 4) * (4 * a.K / 64); }

int cross_rows_launch(const StepArgs &a, hipStream_t st) {
    if (a.ln.gamma && a.ln.residual) return launch<true, true>(a, st);
    if (a.ln.gamma) return launch<true, false>(a, st);
    return launch<false, false>(a, st);
}

}  // namespace gridnet
