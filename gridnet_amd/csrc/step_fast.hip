// Tuned fp32 kernels for the block-local update.  Written for normalize=false (every
// configuration the reference's training scripts use: gridnet/scripts/train_mnist.py:51,
// train_imagenet.py:50); the NORM variants add the per-window normalisation of the reference's
// default on top (see step_fwd_fast and step_bwd_fast).
//
// Mapping.  A "slot" is the group of threads that advances ONE (spatial block, batch element)
// pair: bs*bs*(bs/CPT) threads, each owning CPT consecutive cells of a K-row together with
// their 27*CPT weights in registers.  A workgroup is NSLOT slots on the same spatial block,
// each walking its share of the batch elements the workgroup owns, so the 29 parameter planes
// of a block are fetched once per workgroup and reused for every batch element and every inner
// iteration.  The (bs+2)^3 window lives in LDS, rows padded to a multiple of 4 floats, so a
// thread reads the CPT+2 values it needs from each of its 9 neighbour rows with 64/128-bit LDS
// loads: (CPT+2)*9 loaded values feed 27*CPT FMAs.  Two copies of the window alternate between
// inner iterations (the frozen halo is written to both), which leaves one barrier per iteration.
// The next batch element's window is fetched into registers while the current one iterates.
//
// Backward, without any atomics (the reference scatters w*delta with shared-memory atomicAdd and
// adds windows to the grid with global atomicAdd, src/gridnet_cuda_kernels.cu:384-387, 424-449):
//   * per batch element the inner forward is recomputed, each thread keeping its own x_i and u_i
//     in a private LDS slab;
//   * the gradient of an owned cell stays in a register g.  In iteration i each thread writes
//     delta_i = act'(u_i) g r of its cells into a zero-haloed LDS window and then GATHERS
//     g += sum_t V[t] * delta_i[c + off_t], where V[t][c] = W[26-t, c + off_t] are the
//     neighbours' mirrored weights, loaded once per workgroup into registers (zero where the
//     neighbour lies in another block).  Same shape as the forward stencil, fixed order;
//   * the same delta rows give the weight gradients: x_i[c] * delta_i[c + off_t] is the gradient
//     of the NEIGHBOUR's mirrored weight W[26-t, c + off_t], and this thread is the only one that
//     ever contributes to it, so it accumulates in a register over iterations and batch elements
//     (the x window is not re-read in the reverse sweep);
//   * what depends on a (frozen) halo entry or on another block depends on the iterations only
//     through D = sum_i delta_i.  The gradient of a weight whose tap reads a halo entry is
//     x_halo * D: the first kernel adds it once per element.  What the cells of NEIGHBOURING
//     blocks receive needs the neighbours' D: the first kernel leaves D of every cell in a
//     scratch tensor and a second kernel works it out and completes dx, in a fixed order:
//     cross_rows (cross_rows.hip), dealt by whole grid rows, for rows of 16, 32, 64 or 128 cells;
//     step_bwd_cross, dealt by block face from the D window with its real halo, for the rest.
// Forward with 8^3 blocks: the same mapping over a window stored in two parts, so that every LDS
// access of the inner loop is aligned and free of bank conflicts (step_fwd_split).
// Parameter gradients leave the kernel once per workgroup: reduced across slots through LDS and,
// when one workgroup owns the whole batch of its block, written with plain stores.  Results are
// bitwise reproducible in that case.

#include "common.h"
#include "fast_tiles.h"
#include "plan.h"
#include "launch.h"

namespace gridnet {

namespace {

constexpr int kFwdDepth = 9;  // neighbour rows requested ahead of the arithmetic

// LN: the variant with the LayerNorm of the network body folded in (see LnFold); without it
// `ln` is ignored and the code is the plain step's.
// RES (with LN): the output is x + (result - LayerNorm(x)), the reference's outer_residual form
// (gridnet/scripts/train_imagenet.py:81-83); the statistics left for the next LayerNorm are
// those of that output.
// NORM: per-window normalisation (gridnet/backend_torch.py:126-129,
// src/gridnet_cuda_kernels.cu:164-170): before every inner iteration the whole (bs+2)^3 window,
// halo and zeros outside the grid included, is brought to mean 0 and divided by (std + eps); the
// stencil reads the normalised values, the residual adds to the raw ones.  With S = sum_t w_t x_t
// over the RAW window the pre-activation is b + (S - mean * sum_t w_t) / (std + eps), so the
// stencil itself is unchanged; the statistics come from sums the threads keep of their own
// cells (the halo never changes, its sums are taken once, when the window is committed).
template <int BS, int CPT, int NSLOT, int ACT, bool LN, bool RES = false, bool NORM = false>
__global__ __launch_bounds__((Tile<BS, CPT>::TPS * NSLOT))
__attribute__((amdgpu_waves_per_eu((NORM && CPT >= 4) ? 2 : 3)))  // NORM at 108 weights: no room at 168 registers
void step_fwd_fast(
    const float *__restrict__ weight, const float *__restrict__ bias,
    const float *__restrict__ scale, const float *__restrict__ x, float *__restrict__ y, int B, int M,
    int N, int K, int inner, int nblk, int nchunk, int chunk_len, LnFold ln, float norm_eps) {
    using TL = Tile<BS, CPT>;
    constexpr int GROUPS = TL::TPS / 16;  // 16-lane groups of a slot
    constexpr int NORM_FLOATS = NORM ? NSLOT * GROUPS * (4 + 2 * 2) : 0;
    // per slot two copies of the window; then, for the folded LayerNorm, the packed gamma/beta;
    // then, for NORM, per slot and 16-lane group the sums taken at commit and, twice (alternating
    // between inner iterations), the sums of the owned cells
    __shared__ __attribute__((aligned(16))) float
        lds[NSLOT * 2 * TL::WIN + (LN ? Fetch<TL>::AFFINE : 0) + NORM_FLOATS];
    static_assert(!(NORM && (LN || RES)), "the folded LayerNorm comes without normalisation");

    int blk, chunk;
    if (!split_block_id(ln.walk_reverse ? reversed_on_its_xcd(blockIdx.x, gridDim.x) : blockIdx.x, nblk, nchunk,
                        blk, chunk))
        return;  // grid padding
    const Place<TL, CPT, NSLOT> pl(threadIdx.x, blk, N, K);
    const Fetch<TL> fx(pl.lane, pl.p0, pl.q0, pl.r0, M, N, K);
    float *win = lds + pl.slot * (2 * TL::WIN);
    float *affine = lds + NSLOT * 2 * TL::WIN;
    const long cells = (long)M * N * K;
    const bool ln_in = LN && ln.x_stats != nullptr;  // x is the raw output of the step before

    float w[27][CPT], bv[CPT], rv[CPT];
#pragma unroll
    for (int t = 0; t < 27; ++t) load_cells<CPT>(weight + t * cells + pl.gc, w[t]);
    load_cells<CPT>(bias + pl.gc, bv);
    load_cells<CPT>(scale + pl.gc, rv);
    // NORM: sum of the 27 weights of every owned cell; the sums of this slot in LDS
    float wsum[CPT], zero[CPT];
    float *sums_at_commit = lds + NSLOT * 2 * TL::WIN + (LN ? Fetch<TL>::AFFINE : 0) + pl.slot * GROUPS * 8;
    float *own_sums = sums_at_commit + GROUPS * 4;  // [2][GROUPS][2]
    const int group = pl.lane / 16;
    constexpr float inv_count = 1.f / (TL::S * TL::S * TL::S);
    if (NORM) {
#pragma unroll
        for (int c = 0; c < CPT; ++c) {
            zero[c] = 0.f;
            wsum[c] = 0.f;
#pragma unroll
            for (int t = 0; t < 27; ++t) wsum[c] += w[t][c];
        }
    }
    typename Fetch<TL>::Buf pre;
    if (ln_in) {  // gamma and beta of the window, once per workgroup
        if (pl.slot == 0) {
            typename Fetch<TL>::Buf bet;
            fx.fetch(ln.gamma, pre);
            fx.fetch(ln.beta, bet);
            fx.pack_affine(affine, pre, bet);
        }
        lds_barrier();
    }
    wait_global_loads();

    const int s0 = chunk * chunk_len, s1 = min(B, s0 + chunk_len);
    float pre_mean = 0.f, pre_rstd = 1.f;  // LayerNorm statistics of the element in `pre`
    // NORM: the window is kept minus one of its own values (the block's first cell), see
    // Fetch::commit_sums; `shift` belongs to the element being iterated, `pre_shift` to `pre`
    float pre_shift = 0.f, shift = 0.f, done_shift = 0.f;
    const int first_cell = (pl.p0 * N + pl.q0) * K + pl.r0;
    auto fetch_element = [&](int s) {
        fx.fetch(x + s * cells, pre);
        if (ln_in) {
            pre_mean = load_ahead(ln.x_stats, 2 * s);
            pre_rstd = load_ahead(ln.x_stats, 2 * s + 1);
        }
        if (NORM) pre_shift = load_ahead(x + s * cells, first_cell);
    };
    if (s0 + pl.slot < s1) fetch_element(s0 + pl.slot);
    // The result of an element is stored one element late, after the next window has been
    // committed: the wait for the prefetched window would otherwise also wait for a store that
    // was issued an instant earlier (loads and stores share one in-order counter).
    float done[CPT];
    int done_s = -1;
    for (int sb = s0; sb < s1; sb += NSLOT) {
        const int s = sb + pl.slot;
        const bool active = s < s1;  // a slot past the end idles through the barriers
        if (active) {
            if (ln_in) fx.commit_ln(win, pre, affine, pre_mean, pre_rstd);
            else if (NORM) {
                float part[4];
                shift = pre_shift;
                fx.commit_sums(win, pre, shift, part);
#pragma unroll
                for (int q = 0; q < 4; ++q) part[q] = row16_sum(part[q]);
                if ((pl.lane & 15) == 0)
                    *reinterpret_cast<float4 *>(sums_at_commit + group * 4) =
                        make_float4(part[0], part[1], part[2], part[3]);
            } else fx.commit(win, pre);
        }
        slot_barrier<TL::TPS>();
        if (done_s >= 0) {
            if (NORM) {
#pragma unroll
                for (int c = 0; c < CPT; ++c) done[c] += done_shift;
            }
            store_cells<CPT>(y + done_s * cells + pl.gc, done);
        }
        if (s + NSLOT < s1) fetch_element(s + NSLOT);  // next element, in flight
        float cur[CPT], base[CPT], raw[CPT];
        float halo1 = 0.f, halo2 = 0.f, own1 = 0.f, own2 = 0.f;  // NORM: sums of the window
        if (active) {
#pragma unroll
            for (int c = 0; c < CPT; ++c) cur[c] = win[pl.own + c];
            if (RES) {
                load_cells<CPT>(x + s * cells + pl.gc, raw);
#pragma unroll
                for (int c = 0; c < CPT; ++c) base[c] = cur[c];
            }
            if (NORM) {
#pragma unroll
                for (int q = 0; q < GROUPS; ++q) {  // fixed order: every thread gets the same sums
                    const float4 p4 = *reinterpret_cast<const float4 *>(sums_at_commit + q * 4);
                    halo1 += p4.x; halo2 += p4.y; own1 += p4.z; own2 += p4.w;
                }
            }
        }
        for (int it = 0; it < inner; ++it) {
            if (active) {
                float u[CPT];
                if (NORM) {
                    if (it > 0) {
                        own1 = own2 = 0.f;
#pragma unroll
                        for (int q = 0; q < GROUPS; ++q) {
                            const float2 p2 = *reinterpret_cast<const float2 *>(
                                own_sums + ((it & 1) * GROUPS + q) * 2);
                            own1 += p2.x; own2 += p2.y;
                        }
                    }
                    const float mean = (halo1 + own1) * inv_count;
                    const float var = fmaxf(fmaf(-mean, mean, (halo2 + own2) * inv_count), 0.f);
                    const float inv = 1.f / (sqrtf(var) + norm_eps);
                    stencil<TL, CPT, kFwdDepth>(win + (it & 1) * TL::WIN, pl.row00, w, zero, u);
#pragma unroll
                    for (int c = 0; c < CPT; ++c) u[c] = fmaf(inv, fmaf(-mean, wsum[c], u[c]), bv[c]);
                } else {
                    stencil<TL, CPT, kFwdDepth>(win + (it & 1) * TL::WIN, pl.row00, w, bv, u);
                }
                float s1 = 0.f, s2 = 0.f;
#pragma unroll
                for (int c = 0; c < CPT; ++c) {
                    cur[c] = fmaf(rv[c], Act<ACT, float>::f(u[c]), cur[c]);
                    win[((it + 1) & 1) * TL::WIN + pl.own + c] = cur[c];
                    s1 += cur[c];
                    s2 = fmaf(cur[c], cur[c], s2);
                }
                if (NORM && it + 1 < inner) {  // the owned cells' part of the next statistics
                    s1 = row16_sum(s1);
                    s2 = row16_sum(s2);
                    if ((pl.lane & 15) == 0)
                        *reinterpret_cast<float2 *>(own_sums + (((it + 1) & 1) * GROUPS + group) * 2) =
                            make_float2(s1, s2);
                }
            }
            slot_barrier<TL::TPS>();
        }
        if (RES && active) {
#pragma unroll
            for (int c = 0; c < CPT; ++c) cur[c] = raw[c] + (cur[c] - base[c]);
        }
        if (LN && active && ln.y_part) {
            // statistics of the result for the LayerNorm that follows: every group of 16 lanes
            // leaves (mean, M2 about that mean) of its 16*CPT cells
            float sum = 0.f, m2 = 0.f;
#pragma unroll
            for (int c = 0; c < CPT; ++c) sum += cur[c];
            const float mean = row16_sum(sum) * (1.f / (16 * CPT));
#pragma unroll
            for (int c = 0; c < CPT; ++c) m2 = fmaf(cur[c] - mean, cur[c] - mean, m2);
            m2 = row16_sum(m2);
            // one pair per wave of the slot (per slot, for half-wave slots)
            constexpr int PARTS = TL::TPS >= 64 ? TL::TPS / 64 : 1;
            float wave_mean, wave_m2;
            slot_wave_moments<TL::TPS>(mean, m2, 16 * CPT, wave_mean, wave_m2);
            if ((pl.lane & (TL::TPS >= 64 ? 63 : 31)) == 0) {
                float *to = ln.y_part + (((long)s * nblk + blk) * PARTS + (TL::TPS >= 64 ? pl.lane / 64 : 0)) * 2;
                to[0] = wave_mean;
                to[1] = wave_m2;
            }
        }
        done_s = active ? s : -1;
        done_shift = shift;
#pragma unroll
        for (int c = 0; c < CPT; ++c) done[c] = cur[c];
        if (inner == 0) slot_barrier<TL::TPS>();  // `cur` was read from the window that is rewritten next
    }
    if (done_s >= 0) {
        if (NORM) {
#pragma unroll
            for (int c = 0; c < CPT; ++c) done[c] += done_shift;
        }
        store_cells<CPT>(y + done_s * cells + pl.gc, done);
    }
}

// ---- forward, 8^3 blocks: the split window ------------------------------------------------
// The LDS pipeline limits step_fwd_fast at this block size as much as the vector ALU does: a
// thread's 6-float row is a 128-bit plus a 64-bit read whose lanes collide on banks, and the
// results go back as unaligned 32-bit writes that use a quarter of the banks.  This kernel keeps
// the window in two parts instead:
//   * centre: the 8 block columns of every window row as 8 floats, the second four REVERSED
//     (columns 0 1 2 3 7 6 5 4).  A thread owns four cells of a row, holds them in the order
//     they are stored, and reads or writes them as one aligned, conflict-free 128-bit access;
//   * side: the two halo columns of every row, dense, one 32-bit read per row.
// The sixth value of a row, the cell next to the thread's four on the inner side, is the last
// register of the lane that owns the other half of the row (lane ^ 1): one DPP operand, no LDS.
// With the second half reversed both lanes of a pair see the same picture -- [side entry, own
// four cells outward-in, partner's cell] -- so the code is uniform; the lanes of the second
// half hold their weights mirrored along K to match.
struct SplitWin {
    static constexpr int S = 10, RS = 8, PS = S * RS;  // centre rows and planes (floats)
    static constexpr int CEN = S * PS;
    static constexpr int SP = 12, SS = S * SP;         // side rows of 10 at stride 12, per side
    static constexpr int COPY = CEN + 2 * SS;          // floats per window copy
};

// value of `v` in the lane that owns the other half of the row (lanes 2m and 2m+1 swap)
__device__ __forceinline__ float partner_lane(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0xB1, 0xf, 0xf, true));
}

// LN, RES: the variants with the LayerNorm of the network body folded in, as in step_fwd_fast.
// NORM: per-window normalisation, as in step_fwd_fast (running sums, unchanged stencil).
template <int ACT, bool LN, bool RES = false, bool NORM = false>
__global__ __launch_bounds__(128) __attribute__((amdgpu_waves_per_eu(NORM ? 2 : 3)))
void step_fwd_split(
    const float *__restrict__ weight, const float *__restrict__ bias,
    const float *__restrict__ scale, const float *__restrict__ x, float *__restrict__ y, int B, int M,
    int N, int K, int inner, int nblk, int nchunk, int chunk_len, LnFold ln, float norm_eps) {
    using TL = Tile<8, 4>;
    using SW = SplitWin;
    using FX = Fetch<TL>;
    static_assert(!(NORM && (LN || RES)), "the folded LayerNorm comes without normalisation");
    // two copies of the window; then, for the folded LayerNorm, gamma and beta laid out alike;
    // for NORM, per wave the four sums taken at commit and, twice, the two of the owned cells;
    // for RES, twice (alternating between elements) what the owned cells get back at the end:
    // their raw input minus what the stencil saw of it, laid out like the centre part
    __shared__ __attribute__((aligned(16))) float lds[(LN ? 4 : 2) * SW::COPY + (NORM ? 16 : 0) + (RES ? 2 * SW::CEN : 0)];
    float *gwin = lds + 2 * SW::COPY, *bwin = gwin + SW::COPY;
    float *back = lds + 4 * SW::COPY;  // RES (which comes with LN)
    float *sums_at_commit = lds + 2 * SW::COPY, *own_sums = sums_at_commit + 8;  // NORM: [2][4], [2][2][2]
    const int wave = threadIdx.x >> 6;
    const bool ln_in = LN && ln.x_stats != nullptr;  // x is the raw output of the step before

    int blk, chunk;
    if (!split_block_id(ln.walk_reverse ? reversed_on_its_xcd(blockIdx.x, gridDim.x) : blockIdx.x, nblk, nchunk,
                        blk, chunk))
        return;  // grid padding
    const Place<TL, 4, 1> pl(threadIdx.x, blk, N, K);
    const FX fx(pl.lane, pl.p0, pl.q0, pl.r0, M, N, K);
    const long cells = (long)M * N * K;
    const bool second = pl.kt != 0;  // this thread holds columns 7 6 5 4, in that order

    // where this thread's half rows go: the four cells into the centre part, the end entry
    // into the side part of its half
    int cen_at[FX::RPT], side_at[FX::RPT];
#pragma unroll
    for (int e = 0; e < FX::RPT; ++e) {
        const int id = pl.lane + e * TL::TPS;
        const int half = id & 1, row = id >> 1;
        const int wj = row % SW::S, wi = row / SW::S;
        cen_at[e] = wi * SW::PS + wj * SW::RS + half * 4;
        side_at[e] = SW::CEN + half * SW::SS + wi * SW::SP + wj;
    }
    // tap (a, b) of this thread's rows: centre vector and side entry
    const int cen00 = pl.i * SW::PS + pl.j * SW::RS + pl.kt * 4;
    const int side00 = SW::CEN + pl.kt * SW::SS + pl.i * SW::SP + pl.j;
    const int own = cen00 + SW::PS + SW::RS;

    // Parameters in register order.  First half: w[t][r] is tap t of column r.  Second half:
    // register r is column 7-r and a step of one register is a step of -1 along K, so the tap
    // with K-offset cc sits at register offset 2-cc.
    float w[27][4], bv[4], rv[4];
#pragma unroll
    for (int ab = 0; ab < 9; ++ab) {
        float wt[3][4];
#pragma unroll
        for (int cc = 0; cc < 3; ++cc) load_cells<4>(weight + (ab * 3 + cc) * cells + pl.gc, wt[cc]);
#pragma unroll
        for (int cc = 0; cc < 3; ++cc)
#pragma unroll
            for (int r = 0; r < 4; ++r) w[ab * 3 + cc][r] = second ? wt[2 - cc][3 - r] : wt[cc][r];
    }
    {
        float bt[4], rt[4];
        load_cells<4>(bias + pl.gc, bt);
        load_cells<4>(scale + pl.gc, rt);
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            bv[r] = second ? bt[3 - r] : bt[r];
            rv[r] = second ? rt[3 - r] : rt[r];
        }
    }
    float wsum[4];  // NORM: sum of the 27 weights of every owned cell
    if (NORM) {
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            wsum[r] = 0.f;
#pragma unroll
            for (int t = 0; t < 27; ++t) wsum[r] += w[t][r];
        }
    }
    // A fetched element goes into `copies` window copies at `to`; with `fold` the LayerNorm of
    // the producer is applied on the way: (v - mean) * rstd * gamma + beta, gamma and beta from
    // their own windows; entries outside the grid stay zero.
    float part[4];  // NORM: what the last commit added up
    // NORM: the window is kept minus one of its own values (the block's first cell), see
    // Fetch::commit_sums; `pre_shift` belongs to `pre`, `shift` to the element being iterated
    float pre_shift = 0.f, shift = 0.f, done_shift = 0.f;
    const int first_cell = (pl.p0 * N + pl.q0) * K + pl.r0;
    auto commit = [&](float *to, int copies, const typename FX::Buf &v, bool fold, float mean, float rstd,
                      float *give_back = nullptr) {
#pragma unroll
        for (int q = 0; q < 4; ++q) part[q] = 0.f;
#pragma unroll
        for (int e = 0; e < FX::RPT; ++e)
            if (fx.loff[e] >= 0) {
                float end = v[e][4], c[4];
#pragma unroll
                for (int r = 0; r < 4; ++r) c[r] = fx.hi[e] ? v[e][3 - r] : v[e][r];
                if (LN && fold) {
                    const float4 g4 = *reinterpret_cast<const float4 *>(gwin + cen_at[e]);
                    const float4 b4 = *reinterpret_cast<const float4 *>(bwin + cen_at[e]);
                    float n[4];
                    n[0] = fmaf((c[0] - mean) * rstd, g4.x, b4.x);
                    n[1] = fmaf((c[1] - mean) * rstd, g4.y, b4.y);
                    n[2] = fmaf((c[2] - mean) * rstd, g4.z, b4.z);
                    n[3] = fmaf((c[3] - mean) * rstd, g4.w, b4.w);
                    // RES: raw minus normalised, for whoever owns these cells (rows of the halo
                    // leave entries nobody reads)
                    if (RES && give_back)
                        *reinterpret_cast<float4 *>(give_back + cen_at[e]) =
                            make_float4(c[0] - n[0], c[1] - n[1], c[2] - n[2], c[3] - n[3]);
#pragma unroll
                    for (int r = 0; r < 4; ++r) c[r] = n[r];
                    end = fmaf((end - mean) * rstd, gwin[side_at[e]], bwin[side_at[e]]);
                }
                if (!(fx.ok[e] && fx.edge_ok[e])) end = 0.f;
#pragma unroll
                for (int r = 0; r < 4; ++r) c[r] = fx.ok[e] ? c[r] : 0.f;
                if (NORM) {  // minus the shift; (sum, sum of squares) of halo entries and block cells
                    end -= pre_shift;
#pragma unroll
                    for (int r = 0; r < 4; ++r) c[r] -= pre_shift;
                    const int row = (pl.lane + e * TL::TPS) >> 1, wj = row % SW::S, wi = row / SW::S;
                    const bool halo_row = wi == 0 || wi == SW::S - 1 || wj == 0 || wj == SW::S - 1;
                    const float s1 = (c[0] + c[1]) + (c[2] + c[3]);
                    const float s2 = fmaf(c[0], c[0], fmaf(c[1], c[1], fmaf(c[2], c[2], c[3] * c[3])));
                    part[0] += end + (halo_row ? s1 : 0.f);
                    part[1] += fmaf(end, end, halo_row ? s2 : 0.f);
                    part[2] += halo_row ? 0.f : s1;
                    part[3] += halo_row ? 0.f : s2;
                }
                for (int copy = 0; copy < copies; ++copy) {
                    *reinterpret_cast<float4 *>(to + copy * SW::COPY + cen_at[e]) =
                        make_float4(c[0], c[1], c[2], c[3]);
                    to[copy * SW::COPY + side_at[e]] = end;
                }
            }
    };
    typename FX::Buf pre;
    if (ln_in) {  // gamma and beta of the window, once per workgroup
        fx.fetch(ln.gamma, pre);
        commit(gwin, 1, pre, false, 0.f, 1.f);
        fx.fetch(ln.beta, pre);
        commit(bwin, 1, pre, false, 0.f, 1.f);
        lds_barrier();
    }
    auto store_result = [&](int s, const float (&cur)[4]) {
        float out[4];
#pragma unroll
        for (int c = 0; c < 4; ++c) out[c] = (second ? cur[3 - c] : cur[c]) + (NORM ? done_shift : 0.f);
        store_cells<4>(y + s * cells + pl.gc, out);
    };

    const int s0 = chunk * chunk_len, s1 = min(B, s0 + chunk_len);
    float pre_mean = 0.f, pre_rstd = 1.f;  // LayerNorm statistics of the element in `pre`
    auto fetch_element = [&](int s) {
        fx.fetch(x + s * cells, pre);
        if (ln_in) {
            pre_mean = load_ahead(ln.x_stats, 2 * s);
            pre_rstd = load_ahead(ln.x_stats, 2 * s + 1);
        }
        if (NORM) pre_shift = load_ahead(x + s * cells, first_cell);
    };
    if (s0 < s1) fetch_element(s0);
    // The result of an element is stored one element late, after the next window has been
    // committed (see step_fwd_fast).
    float done[4];
    int done_s = -1;
    // Turns pay when the grid is a single round of workgroups (the batch was split to fill the
    // chip: nchunk > 1).  With one workgroup per block and more blocks than the chip holds, a
    // workgroup that ends early is replaced at once, and the turns cost 1.5 % (128^3, batch 8).
    const bool turns = nchunk > 1;
    for (int s = s0; s < s1; ++s) {
        if (turns) take_turns(s);
        commit(lds, 2, pre, ln_in, pre_mean, pre_rstd, RES ? back + ((s - s0) & 1) * SW::CEN : nullptr);
        if (NORM) {
            shift = pre_shift;
#pragma unroll
            for (int q = 0; q < 4; ++q) part[q] = slot_wave_sum<64>(part[q]);
            if ((threadIdx.x & 63) == 0)
                *reinterpret_cast<float4 *>(sums_at_commit + wave * 4) =
                    make_float4(part[0], part[1], part[2], part[3]);
        }
        lds_barrier();
        if (done_s >= 0) store_result(done_s, done);
        if (s + 1 < s1) fetch_element(s + 1);  // next element, in flight
        float cur[4];
        {
            const float4 q = *reinterpret_cast<const float4 *>(lds + own);
            cur[0] = q.x; cur[1] = q.y; cur[2] = q.z; cur[3] = q.w;
        }
        float halo1 = 0.f, halo2 = 0.f, own1 = 0.f, own2 = 0.f;  // NORM: sums over the window
        if (NORM) {
            const float4 a4 = *reinterpret_cast<const float4 *>(sums_at_commit);
            const float4 b4 = *reinterpret_cast<const float4 *>(sums_at_commit + 4);
            halo1 = a4.x + b4.x; halo2 = a4.y + b4.y; own1 = a4.z + b4.z; own2 = a4.w + b4.w;
        }
        for (int it = 0; it < inner; ++it) {
            const float *from = lds + (it & 1) * SW::COPY;
            float u[4];
            float nmean = 0.f, ninv = 1.f;
            if (NORM) {
                if (it > 0) {
                    const float4 o4 = *reinterpret_cast<const float4 *>(own_sums + (it & 1) * 4);
                    own1 = o4.x + o4.z;
                    own2 = o4.y + o4.w;
                }
                nmean = (halo1 + own1) * (1.f / 1000);
                const float var = fmaxf(fmaf(-nmean, nmean, (halo2 + own2) * (1.f / 1000)), 0.f);
                ninv = 1.f / (sqrtf(var) + norm_eps);
            }
#pragma unroll
            for (int r = 0; r < 4; ++r) u[r] = NORM ? 0.f : bv[r];
#pragma unroll
            for (int a = 0; a < 3; ++a)
#pragma unroll
                for (int b = 0; b < 3; ++b) {
                    const float4 q =
                        *reinterpret_cast<const float4 *>(from + cen00 + a * SW::PS + b * SW::RS);
                    float v[6];
                    v[0] = from[side00 + a * SW::SP + b];
                    v[1] = q.x; v[2] = q.y; v[3] = q.z; v[4] = q.w;
                    v[5] = partner_lane(q.w);
#pragma unroll
                    for (int cc = 0; cc < 3; ++cc)
#pragma unroll
                        for (int r = 0; r < 4; ++r)
                            u[r] = fmaf(w[a * 9 + b * 3 + cc][r], v[r + cc], u[r]);
                }
            if (NORM) {
#pragma unroll
                for (int r = 0; r < 4; ++r) u[r] = fmaf(ninv, fmaf(-nmean, wsum[r], u[r]), bv[r]);
            }
#pragma unroll
            for (int r = 0; r < 4; ++r) cur[r] = fmaf(rv[r], Act<ACT, float>::f(u[r]), cur[r]);
            *reinterpret_cast<float4 *>(lds + ((it + 1) & 1) * SW::COPY + own) =
                make_float4(cur[0], cur[1], cur[2], cur[3]);
            if (NORM && it + 1 < inner) {  // the owned cells' part of the next statistics
                const float s1 = slot_wave_sum<64>((cur[0] + cur[1]) + (cur[2] + cur[3]));
                const float s2 = slot_wave_sum<64>(
                    fmaf(cur[0], cur[0], fmaf(cur[1], cur[1], fmaf(cur[2], cur[2], cur[3] * cur[3]))));
                if ((threadIdx.x & 63) == 0)
                    *reinterpret_cast<float2 *>(own_sums + ((it + 1) & 1) * 4 + wave * 2) = make_float2(s1, s2);
            }
            lds_barrier();
        }
        if (RES) {  // x + (result - n): the difference x - n was left at commit, in register order
            const float4 q = *reinterpret_cast<const float4 *>(back + ((s - s0) & 1) * SW::CEN + own);
            cur[0] += q.x; cur[1] += q.y; cur[2] += q.z; cur[3] += q.w;
        }
        if (LN && ln.y_part) {
            // statistics of the result for the LayerNorm that follows: every group of 16 lanes
            // leaves (mean, M2 about that mean) of its 64 cells
            float sum = 0.f, m2 = 0.f;
#pragma unroll
            for (int r = 0; r < 4; ++r) sum += cur[r];
            const float mean = row16_sum(sum) * (1.f / 64);
#pragma unroll
            for (int r = 0; r < 4; ++r) m2 = fmaf(cur[r] - mean, cur[r] - mean, m2);
            m2 = row16_sum(m2);
            float wave_mean, wave_m2;  // one pair per wave
            slot_wave_moments<128>(mean, m2, 64, wave_mean, wave_m2);
            if ((pl.lane & 63) == 0) {
                // the wave's number as a scalar: the address is uniform then, and no per-lane
                // pointer is carried (spilled) through the batch loop for this one store
                const int wv = __builtin_amdgcn_readfirstlane(pl.lane / 64);
                float *to = ln.y_part + (((long)s * nblk + blk) * 2 + wv) * 2;
                to[0] = wave_mean;
                to[1] = wave_m2;
            }
        }
        done_s = s;
        done_shift = shift;
#pragma unroll
        for (int r = 0; r < 4; ++r) done[r] = cur[r];
        if (inner == 0) lds_barrier();  // `cur` was read from the window that is rewritten next
    }
    if (done_s >= 0) store_result(done_s, done);
}

// ---- forward, 8^3 blocks, the chain's variant: two batch elements per pass -------------------
// step_fwd_split<ACT, LN = true> with every thread advancing TWO batch elements side by side:
// the same 108 weights in registers feed both, the two elements' dependent FMA chains and LDS
// round trips interleave (neither the LDS nor the vector ALU is saturated by one element per
// wave: what limits step_fwd_split is latency), a barrier serves two elements, and with fewer,
// larger workgroups the 29 parameter planes of a block are fetched twice per launch instead of
// three times (64^3 grid, batch 32).  Two waves per SIMD instead of three: the second element's
// state and prefetch need the registers.
template <int ACT>
__global__ __launch_bounds__(128) __attribute__((amdgpu_waves_per_eu(2)))
void step_fwd_pair(
    const float *__restrict__ weight, const float *__restrict__ bias,
    const float *__restrict__ scale, const float *__restrict__ x, float *__restrict__ y, int B, int M,
    int N, int K, int inner, int nblk, int nchunk, int chunk_len, LnFold ln) {
    using TL = Tile<8, 4>;
    using SW = SplitWin;
    using FX = Fetch<TL>;
    constexpr int E = 2;
    // per element two copies of the window; then gamma and beta laid out alike
    __shared__ __attribute__((aligned(16))) float lds[(2 * E + 2) * SW::COPY];
    float *gwin = lds + 2 * E * SW::COPY, *bwin = gwin + SW::COPY;
    const bool ln_in = ln.x_stats != nullptr;  // x is the raw output of the step before

    int blk, chunk;
    if (!split_block_id(ln.walk_reverse ? reversed_on_its_xcd(blockIdx.x, gridDim.x) : blockIdx.x, nblk, nchunk,
                        blk, chunk))
        return;  // grid padding
    const Place<TL, 4, 1> pl(threadIdx.x, blk, N, K);
    const FX fx(pl.lane, pl.p0, pl.q0, pl.r0, M, N, K);
    const long cells = (long)M * N * K;
    const bool second = pl.kt != 0;  // this thread holds columns 7 6 5 4, in that order

    int cen_at[FX::RPT], side_at[FX::RPT];
#pragma unroll
    for (int e = 0; e < FX::RPT; ++e) {
        const int id = pl.lane + e * TL::TPS;
        const int half = id & 1, row = id >> 1;
        const int wj = row % SW::S, wi = row / SW::S;
        cen_at[e] = wi * SW::PS + wj * SW::RS + half * 4;
        side_at[e] = SW::CEN + half * SW::SS + wi * SW::SP + wj;
    }
    const int cen00 = pl.i * SW::PS + pl.j * SW::RS + pl.kt * 4;
    const int side00 = SW::CEN + pl.kt * SW::SS + pl.i * SW::SP + pl.j;
    const int own = cen00 + SW::PS + SW::RS;

    // parameters in register order (see step_fwd_split)
    float w[27][4], bv[4], rv[4];
#pragma unroll
    for (int ab = 0; ab < 9; ++ab) {
        float wt[3][4];
#pragma unroll
        for (int cc = 0; cc < 3; ++cc) load_cells<4>(weight + (ab * 3 + cc) * cells + pl.gc, wt[cc]);
#pragma unroll
        for (int cc = 0; cc < 3; ++cc)
#pragma unroll
            for (int r = 0; r < 4; ++r) w[ab * 3 + cc][r] = second ? wt[2 - cc][3 - r] : wt[cc][r];
    }
    {
        float bt[4], rt[4];
        load_cells<4>(bias + pl.gc, bt);
        load_cells<4>(scale + pl.gc, rt);
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            bv[r] = second ? bt[3 - r] : bt[r];
            rv[r] = second ? rt[3 - r] : rt[r];
        }
    }
    auto commit = [&](float *to, int copies, const typename FX::Buf &v, bool fold, float mean, float rstd) {
#pragma unroll
        for (int e = 0; e < FX::RPT; ++e)
            if (fx.loff[e] >= 0) {
                float end = v[e][4], c[4];
#pragma unroll
                for (int r = 0; r < 4; ++r) c[r] = fx.hi[e] ? v[e][3 - r] : v[e][r];
                if (fold) {
                    const float4 g4 = *reinterpret_cast<const float4 *>(gwin + cen_at[e]);
                    const float4 b4 = *reinterpret_cast<const float4 *>(bwin + cen_at[e]);
                    c[0] = fmaf((c[0] - mean) * rstd, g4.x, b4.x);
                    c[1] = fmaf((c[1] - mean) * rstd, g4.y, b4.y);
                    c[2] = fmaf((c[2] - mean) * rstd, g4.z, b4.z);
                    c[3] = fmaf((c[3] - mean) * rstd, g4.w, b4.w);
                    end = fmaf((end - mean) * rstd, gwin[side_at[e]], bwin[side_at[e]]);
                }
                if (!(fx.ok[e] && fx.edge_ok[e])) end = 0.f;
#pragma unroll
                for (int r = 0; r < 4; ++r) c[r] = fx.ok[e] ? c[r] : 0.f;
                for (int copy = 0; copy < copies; ++copy) {
                    *reinterpret_cast<float4 *>(to + copy * SW::COPY + cen_at[e]) =
                        make_float4(c[0], c[1], c[2], c[3]);
                    to[copy * SW::COPY + side_at[e]] = end;
                }
            }
    };
    typename FX::Buf pre[E];
    if (ln_in) {  // gamma and beta of the window, once per workgroup
        fx.fetch(ln.gamma, pre[0]);
        commit(gwin, 1, pre[0], false, 0.f, 1.f);
        fx.fetch(ln.beta, pre[0]);
        commit(bwin, 1, pre[0], false, 0.f, 1.f);
        lds_barrier();
    }
    auto store_result = [&](int s, const float (&cur)[4]) {
        float out[4];
#pragma unroll
        for (int c = 0; c < 4; ++c) out[c] = second ? cur[3 - c] : cur[c];
        store_cells<4>(y + s * cells + pl.gc, out);
    };

    const int s0 = chunk * chunk_len, s1 = min(B, s0 + chunk_len);
    float pre_mean[E], pre_rstd[E];
    // Loads are unconditional: past the end of the chunk they repeat its last element, whose
    // copy nobody stores (with branches around them the compiler cannot count the loads in flight)
    auto fetch_pair = [&](int s) {
#pragma unroll
        for (int e = 0; e < E; ++e) {
            const int sc = min(s + e, s1 - 1);
            fx.fetch(x + sc * cells, pre[e]);
            pre_mean[e] = ln_in ? load_ahead(ln.x_stats, 2 * sc) : 0.f;
            pre_rstd[e] = ln_in ? load_ahead(ln.x_stats, 2 * sc + 1) : 1.f;
        }
    };
    if (s0 < s1) fetch_pair(s0);
    float done[E][4];
    int done_s = -1;
    const bool turns = nchunk > 1;
    for (int s = s0; s < s1; s += E) {
        if (turns) take_turns(s >> 1);
#pragma unroll
        for (int e = 0; e < E; ++e) commit(lds + e * 2 * SW::COPY, 2, pre[e], ln_in, pre_mean[e], pre_rstd[e]);
        lds_barrier();
        if (done_s >= 0) {
#pragma unroll
            for (int e = 0; e < E; ++e)
                if (done_s + e < s1) store_result(done_s + e, done[e]);
        }
        if (s + E < s1) fetch_pair(s + E);  // next pair, in flight
        float cur[E][4];
#pragma unroll
        for (int e = 0; e < E; ++e) {
            const float4 q = *reinterpret_cast<const float4 *>(lds + e * 2 * SW::COPY + own);
            cur[e][0] = q.x; cur[e][1] = q.y; cur[e][2] = q.z; cur[e][3] = q.w;
        }
        for (int it = 0; it < inner; ++it) {
            float u[E][4];
#pragma unroll
            for (int e = 0; e < E; ++e)
#pragma unroll
                for (int r = 0; r < 4; ++r) u[e][r] = bv[r];
#pragma unroll
            for (int a = 0; a < 3; ++a)
#pragma unroll
                for (int b = 0; b < 3; ++b) {
#pragma unroll
                    for (int e = 0; e < E; ++e) {
                        const float *from = lds + (e * 2 + (it & 1)) * SW::COPY;
                        const float4 q =
                            *reinterpret_cast<const float4 *>(from + cen00 + a * SW::PS + b * SW::RS);
                        float v[6];
                        v[0] = from[side00 + a * SW::SP + b];
                        v[1] = q.x; v[2] = q.y; v[3] = q.z; v[4] = q.w;
                        v[5] = partner_lane(q.w);
#pragma unroll
                        for (int cc = 0; cc < 3; ++cc)
#pragma unroll
                            for (int r = 0; r < 4; ++r)
                                u[e][r] = fmaf(w[a * 9 + b * 3 + cc][r], v[r + cc], u[e][r]);
                    }
                }
#pragma unroll
            for (int e = 0; e < E; ++e) {
#pragma unroll
                for (int r = 0; r < 4; ++r) cur[e][r] = fmaf(rv[r], Act<ACT, float>::f(u[e][r]), cur[e][r]);
                *reinterpret_cast<float4 *>(lds + (e * 2 + ((it + 1) & 1)) * SW::COPY + own) =
                    make_float4(cur[e][0], cur[e][1], cur[e][2], cur[e][3]);
            }
            lds_barrier();
        }
        if (ln.y_part) {
            // statistics of the results for the LayerNorm that follows: one (mean, M2) pair per wave
#pragma unroll
            for (int e = 0; e < E; ++e) {
                float sum = 0.f, m2 = 0.f;
#pragma unroll
                for (int r = 0; r < 4; ++r) sum += cur[e][r];
                const float mean = row16_sum(sum) * (1.f / 64);
#pragma unroll
                for (int r = 0; r < 4; ++r) m2 = fmaf(cur[e][r] - mean, cur[e][r] - mean, m2);
                m2 = row16_sum(m2);
                float wave_mean, wave_m2;
                slot_wave_moments<128>(mean, m2, 64, wave_mean, wave_m2);
                if ((pl.lane & 63) == 0 && s + e < s1) {
                    float *to = ln.y_part + (((long)(s + e) * nblk + blk) * 2 + pl.lane / 64) * 2;
                    to[0] = wave_mean;
                    to[1] = wave_m2;
                }
            }
        }
        done_s = s;
#pragma unroll
        for (int e = 0; e < E; ++e)
#pragma unroll
            for (int r = 0; r < 4; ++r) done[e][r] = cur[e][r];
    }
    if (done_s >= 0) {
#pragma unroll
        for (int e = 0; e < E; ++e)
            if (done_s + e < s1) store_result(done_s + e, done[e]);
    }
}

// ---- backward ------------------------------------------------------------------------------
constexpr int kBwdDepth = 4;  // neighbour rows requested ahead of the arithmetic

// LDS layout of the backward kernel (floats): per slot [x window x2 | delta window x2 |
// history: inner slabs of TPS*2*CPT].
template <int BS, int CPT> __host__ __device__ constexpr int bwd_slot_floats(int inner) {
    return 4 * Tile<BS, CPT>::WIN + inner * Tile<BS, CPT>::TPS * 2 * CPT;
}
// NORM, per slot behind all of the above: (mean, std, 1/(std+eps), -) of the window before
// every inner iteration, then the sums the waves of a slot exchange: 4 floats per wave taken
// at commit, 2 x 2 per wave for the owned cells (alternating between iterations), 2 per wave in
// the reverse sweep
template <int BS, int CPT> __host__ __device__ constexpr int bwd_norm_waves() {
    return Tile<BS, CPT>::TPS >= 64 ? Tile<BS, CPT>::TPS / 64 : 1;
}
// ... and three values per owned cell that live as long as the kernel but are touched once per
// iteration or element (sum of the cell's weights, sum of those whose taps read the halo, D2
// summed over the batch): in LDS, the register file has no room for them
template <int BS, int CPT> __host__ __device__ constexpr int bwd_norm_floats(int inner) {
    return 4 * inner + 12 * bwd_norm_waves<BS, CPT>() + 3 * CPT * Tile<BS, CPT>::TPS;
}
// ... and at least the 27 weight planes of the block, which pass through LDS once at set-up
template <int BS, int CPT, int NSLOT> size_t bwd_lds_bytes(int inner, bool ln = false, bool norm = false) {
    const size_t run = ((size_t)NSLOT * bwd_slot_floats<BS, CPT>(inner) +
                        (ln ? Fetch<Tile<BS, CPT>>::AFFINE : 0) +
                        (norm ? NSLOT * bwd_norm_floats<BS, CPT>(inner) : 0)) * sizeof(float);
    const size_t setup = (size_t)27 * BS * BS * BS * sizeof(float);
    return run > setup ? run : setup;
}

// RES (with LN): the outer_residual form of the loop, see LnFold.
// NORM: per-window normalisation (see step_fwd_fast).  With mean_i, std_i, inv_i = 1/(std_i+eps)
// of the window before iteration i, n_i = (x_i - mean_i) inv_i what the stencil reads, and
// dn_i[k] = sum of w_t[c] delta_i[c] over the (c, t) that read window entry k, the gradient that
// iteration i adds to window entry k is (N = (bs+2)^3 entries)
//   inv_i (dn_i[k] - A_i / N) - (x_i[k] - mean_i) C_i,   A_i = sum_k dn_i[k],
//   C_i = inv_i^2 / (N std_i) * sum_k dn_i[k] (x_i[k] - mean_i).
// Both sums run over the whole window.  The owned cells' part comes from the gather of the
// reverse sweep; the halo's part needs no halo entry of dn: summed over the halo,
// dn_i = sum_c delta_i[c] * (sum of c's weights whose taps read the halo) and
// dn_i x = sum_c delta_i[c] * (those weights times the halo values they read), and both
// brackets are fixed for the element (the halo is frozen).  What the HALO entries receive over
// all iterations is, for halo entry h,
//   sum over (c, t) reading h of w_t[c] D1[c]  -  x_h Q + R,
//   D1 = sum_i inv_i delta_i,  Q = sum_i C_i,  R = sum_i (mean_i C_i - inv_i A_i / N):
// the first term is what step_bwd_cross computes from the tensor this kernel leaves (D1 instead
// of D), Q and R are two numbers per (element, block) left in `qr_out` for it.  The weights of
// the taps that read the halo get x_h D1[c] - D2[c], D2 = sum_i mean_i inv_i delta_i (the halo
// pass adds the first term, the second is subtracted once at the end).
template <int BS, int CPT, int NSLOT, int ACT, bool LN, bool RES = false, bool NORM = false>
__global__ __launch_bounds__((Tile<BS, CPT>::TPS * NSLOT)) __attribute__((amdgpu_waves_per_eu(2)))
void step_bwd_fast(
    const float *__restrict__ weight, const float *__restrict__ bias,
    const float *__restrict__ scale, const float *__restrict__ x, const float *__restrict__ dy,
    float *__restrict__ dweight, float *__restrict__ dbias, float *__restrict__ dscale,
    float *__restrict__ dx, float *__restrict__ dsum_out, int B, int M, int N, int K, int inner,
    int nblk, int nchunk, int chunk_len, int param_mode, int dx_accumulate, LnFold ln,
    float norm_eps, float *__restrict__ qr_out, long slab_stride) {
    using TL = Tile<BS, CPT>;
    static_assert(!(NORM && (LN || RES)), "the folded LayerNorm comes without normalisation");
    extern __shared__ __attribute__((aligned(16))) float lds[];
    const int slot_floats = bwd_slot_floats<BS, CPT>(inner);
    // LN (the LayerNorm of the network body folded in, see LnFold): `dy` is the gradient with
    // respect to LayerNorm(y_raw) and is taken through that LayerNorm's backward as it is
    // loaded (dgamma, dbeta fall out on the way); x is normalised as it is loaded when it is
    // the raw output of the step before.
    const bool ln_in = LN && ln.x_stats != nullptr;

    int blk, chunk;
    if (!split_block_id(blockIdx.x, nblk, nchunk, blk, chunk)) return;  // grid padding
    if (slab_stride) {
        // the batch of this block is split over workgroups: every chunk commits into a copy of
        // the gradient arrays of its own (plain stores; the copies are added up afterwards)
        const long off = chunk * slab_stride;
        dweight += off;
        dbias += off;
        dscale += off;
        if (LN) {
            ln.dgamma += off;
            ln.dbeta += off;
        }
    }
    const Place<TL, CPT, NSLOT> pl(threadIdx.x, blk, N, K);
    const Fetch<TL> fx(pl.lane, pl.p0, pl.q0, pl.r0, M, N, K);
    float *win = lds + pl.slot * slot_floats;
    float *dwin = win + 2 * TL::WIN;
    float *hist = dwin + 2 * TL::WIN + pl.lane * CPT;  // + it*TPS*2*CPT (x_i), + TPS*CPT more (u_i)
    // The x window copy that would receive x_inner (never needed) gets zeros in the block's
    // cells instead: the x window's halo alone, for the weights of the taps that read it.
    const float *xhalo = win + (inner & 1) * TL::WIN;
    float *affine = lds + NSLOT * slot_floats;  // LN: gamma and beta of the window, packed
    const long cells = (long)M * N * K;
    // NORM: the slot's statistics per iteration and the sums its waves exchange
    constexpr int NW = bwd_norm_waves<BS, CPT>();
    const int norm_stride = bwd_norm_floats<BS, CPT>(inner);
    float *nstat = lds + NSLOT * slot_floats + pl.slot * norm_stride;
    float *ncommit = nstat + 4 * inner, *nown = ncommit + 4 * NW, *nrev = nown + 4 * NW;
    float *wsum_at = nrev + 4 * NW + pl.lane * CPT;  // this thread's: sum of a cell's weights
    float *wout_at = wsum_at + CPT * TL::TPS;         // of those whose taps read the halo
    float *d2acc_at = wout_at + CPT * TL::TPS;        // D2 summed over the batch elements
    const int wave_in_slot = TL::TPS >= 64 ? pl.lane / 64 : 0;
    constexpr float inv_count = 1.f / TL::NWIN;

    // nw[t][c] belongs to the weight of the neighbour at c + off_t where that lies in this block,
    // and to this cell's own weight of tap t where it does not (see below)
    auto in_block = [&](int t, int c) {
        const int ni = pl.i + t / 9 - 1, nj = pl.j + (t / 3) % 3 - 1, nk = pl.kt * CPT + c + t % 3 - 1;
        return ni >= 0 && ni < BS && nj >= 0 && nj < BS && nk >= 0 && nk < BS;
    };
    auto neighbour_weight = [&](int t, int c) {
        return (26 - t) * cells + pl.gc + c + ((t / 9 - 1) * N + ((t / 3) % 3 - 1)) * K + (t % 3 - 1);
    };
    auto owner_of = [&](int t, int c) {
        return in_block(t, c) ? neighbour_weight(t, c) : t * cells + pl.gc + c;
    };
    auto always = [](int, int) { return true; };

    // ---- once per workgroup: parameters and mirrored neighbour weights ----
    // w : this cell's weights (forward recompute)
    // v : V[t][c] = W[26-t, c + off_t], what the neighbour at c + off_t multiplies cell c by
    // nw: gradient of that same neighbour weight; it is the product of this cell's x and the
    //     neighbour's delta summed over iterations and batch, so this thread owns it completely.
    //     Where the neighbour lies in ANOTHER block the slot would stay empty (the delta halo is
    //     zero); it holds the gradient of this cell's own weight of tap t instead: that tap reads
    //     a halo entry, frozen over the iterations, so its gradient is x_halo[c + off_t] * D[c]
    //     with D = sum_i delta_i, added once per element from a window that holds the halo alone.
    float w[27][CPT], v[27][CPT], nw[27][CPT], bv[CPT], rv[CPT], db[CPT], dr[CPT];
#pragma unroll
    for (int t = 0; t < 27; ++t) {
        load_cells<CPT>(weight + t * cells + pl.gc, w[t]);
#pragma unroll
        for (int c = 0; c < CPT; ++c) nw[t][c] = 0.f;
    }
    load_cells<CPT>(bias + pl.gc, bv);
    load_cells<CPT>(scale + pl.gc, rv);
#pragma unroll
    for (int c = 0; c < CPT; ++c) db[c] = dr[c] = 0.f;
    float gam[CPT], dgam[CPT], dbet[CPT];
    if (LN) {
        load_cells<CPT>(ln.gamma + pl.gc, gam);
#pragma unroll
        for (int c = 0; c < CPT; ++c) dgam[c] = dbet[c] = 0.f;
    }
    {   // The mirrored neighbour weights are other threads' w: they are exchanged through LDS
        // (the windows are not in use yet) instead of read from global memory a second time --
        // every workgroup of the grid does this at the same moment, and twice the weight tensor
        // was what the set-up phase waited for.
        constexpr int NC = BS * BS * BS;
        float *wl = lds;  // [27][NC], by block-local cell (i, j, k)
        const int lin = (pl.i * BS + pl.j) * BS + pl.kt * CPT;
        if (pl.slot == 0) {
#pragma unroll
            for (int t = 0; t < 27; ++t) store_cells<CPT>(wl + t * NC + lin, w[t]);
        }
        lds_barrier();
#pragma unroll
        for (int t = 0; t < 27; ++t)
#pragma unroll
            for (int c = 0; c < CPT; ++c)
                v[t][c] = in_block(t, c) ? wl[(26 - t) * NC + lin + c + ((t / 9 - 1) * BS + ((t / 3) % 3 - 1)) * BS + (t % 3 - 1)]
                                         : 0.f;
        lds_barrier();  // the windows reuse this memory
    }
    // NORM: sum of a cell's 27 weights, and of those whose taps read the halo (only this thread
    // ever touches its three LDS entries per cell: no barrier needed for them)
    float zero[CPT];
    if (NORM) {
        float wsum[CPT], wout[CPT];
#pragma unroll
        for (int c = 0; c < CPT; ++c) {
            wsum[c] = wout[c] = zero[c] = 0.f;
#pragma unroll
            for (int t = 0; t < 27; ++t) {
                wsum[c] += w[t][c];
                wout[c] += in_block(t, c) ? 0.f : w[t][c];
            }
        }
        store_cells<CPT>(wsum_at, wsum);
        store_cells<CPT>(wout_at, wout);
        store_cells<CPT>(d2acc_at, zero);
    }
    typename Fetch<TL>::Buf pre;
    if (ln_in && pl.slot == 0) {  // gamma and beta of the window, once per workgroup
        typename Fetch<TL>::Buf bet;
        fx.fetch(ln.gamma, pre);
        fx.fetch(ln.beta, bet);
        fx.pack_affine(affine, pre, bet);
    }

    // delta windows: the halo stays zero for the whole kernel
    for (int idx = pl.lane; idx < 2 * TL::WIN; idx += TL::TPS) dwin[idx] = 0.f;
    wait_global_loads();
    // Add-in-place mode: slot 0's accumulators start from what the gradient buffers hold and
    // are stored at the end like in the overwrite mode.  Requested here, behind the set-up
    // wait, the old values arrive while the first element is recomputed.
    if (param_mode == kParamAddExclusive && pl.slot == 0) {
#pragma unroll
        for (int t = 0; t < 27; ++t)
#pragma unroll
            for (int c = 0; c < CPT; ++c) nw[t][c] = dweight[owner_of(t, c)];
#pragma unroll
        for (int c = 0; c < CPT; ++c) {
            db[c] = dbias[pl.gc + c];
            dr[c] = dscale[pl.gc + c];
        }
        if (LN) {
            load_cells<CPT>(ln.dgamma + pl.gc, dgam);
            load_cells<CPT>(ln.dbeta + pl.gc, dbet);
        }
    }

    const int s0 = chunk * chunk_len, s1 = min(B, s0 + chunk_len);
    // what is requested one element ahead: the x window, the incoming gradient of the owned
    // cells and, for LN, the raw output there and the per-sample numbers of both LayerNorms
    float g[CPT], gnext[CPT], ynext[CPT], nx_mean = 0.f, nx_rstd = 1.f, ny[4] = {0.f, 1.f, 0.f, 0.f};
    // RES: G'' of the owned cells (of the step after), G' as formed for the current element, and
    // the latter again for the element whose results are stored one element late
    float gprev[CPT], gin[CPT], gin_done[CPT];
    const bool through_ln = LN && (!RES || ln.y_raw != nullptr);  // dy passes a LayerNorm on load
    // NORM: the x window is kept minus one of its own values (the block's first cell), see
    // Fetch::commit_sums; everything downstream only sees differences of window entries, except
    // R, which is handed on for the unshifted x (R + shift * Q)
    float pre_shift = 0.f, shift = 0.f;
    const int first_cell = (pl.p0 * N + pl.q0) * K + pl.r0;
    auto fetch_element = [&](int s) {
        fx.fetch(x + s * cells, pre);
        load_cells<CPT>(dy + s * cells + pl.gc, gnext);
        if (RES && through_ln) load_cells<CPT>(ln.g_prev + s * cells + pl.gc, gprev);
        if (through_ln) {
            load_cells<CPT>(ln.y_raw + s * cells + pl.gc, ynext);
            ny[0] = load_ahead(ln.y_stats, 2 * s);
            ny[1] = load_ahead(ln.y_stats, 2 * s + 1);
            ny[2] = load_ahead(ln.y_sums, 2 * s);
            ny[3] = load_ahead(ln.y_sums, 2 * s + 1);
        }
        if (ln_in) {
            nx_mean = load_ahead(ln.x_stats, 2 * s);
            nx_rstd = load_ahead(ln.x_stats, 2 * s + 1);
        }
        if (NORM) pre_shift = load_ahead(x + s * cells, first_cell);
    };
    // the element just fetched becomes the current one: its gradient (through the LayerNorm
    // backward for LN) and its window
    auto take_element = [&]() {
#pragma unroll
        for (int c = 0; c < CPT; ++c) {
            if (through_ln) {
                const float yh = (ynext[c] - ny[0]) * ny[1];
                dgam[c] = fmaf(gnext[c], yh, dgam[c]);
                dbet[c] += gnext[c];
                g[c] = ny[1] * (gam[c] * gnext[c] - ny[2] - yh * ny[3]);
                if (RES) g[c] += gprev[c];
            } else {
                g[c] = gnext[c];
            }
            if (RES) gin[c] = g[c];
        }
        if (ln_in) fx.commit_ln(win, pre, affine, nx_mean, nx_rstd);
        else if (NORM) {
            float part[4];
            shift = pre_shift;
            fx.commit_sums(win, pre, shift, part);
#pragma unroll
            for (int q = 0; q < 4; ++q) part[q] = slot_wave_sum<TL::TPS>(part[q]);
            if ((pl.lane & 63 & (TL::TPS - 1)) == 0)
                *reinterpret_cast<float4 *>(ncommit + wave_in_slot * 4) =
                    make_float4(part[0], part[1], part[2], part[3]);
        } else fx.commit(win, pre);
    };
    if (ln_in) lds_barrier();  // gamma and beta windows
    if (s0 + pl.slot < s1) {
        fetch_element(s0 + pl.slot);
        take_element();
    }
    // Per element: commit its window, barrier, [stores of the PREVIOUS element], recompute,
    // reverse sweep, commit the next window.  The stores are issued one element late, away from
    // the wait on the prefetched window (loads and stores share one in-order counter).  Besides
    // the gradient of its own cells a thread leaves D = sum_i delta_i of them: what the cells
    // of neighbouring blocks and the weights of taps that read the frozen halo receive depends
    // on the iterations only through D, and a second kernel (step_bwd_cross) works it out.
    float g_done[CPT], d_done[CPT], q_done = 0.f, r_done = 0.f;
    int done_s = -1;
    auto finish_done = [&]() {
        if (done_s < 0) return;
        const long o = (long)done_s * cells + pl.gc;
        store_cells<CPT>(dsum_out + o, d_done);
        if (NORM && pl.lane == 0)
            *reinterpret_cast<float2 *>(qr_out + ((long)done_s * nblk + blk) * 2) = make_float2(q_done, r_done);
        if (dx_accumulate) add_cells<CPT>(dx + o, g_done);
        else store_cells<CPT>(dx + o, g_done);
        if (RES && ln.g_out) store_cells<CPT>(ln.g_out + o, gin_done);
        done_s = -1;
    };
    for (int sb = s0; sb < s1; sb += NSLOT) {
        const int s = sb + pl.slot;
        const bool active = s < s1;  // a slot past the end idles through the barriers
        take_turns(sb / NSLOT);
        slot_barrier<TL::TPS>();               // this element's window
        finish_done();
        if (s + NSLOT < s1) fetch_element(s + NSLOT);
        float cur[CPT];
        float halo1 = 0.f, halo2 = 0.f, own1 = 0.f, own2 = 0.f;  // NORM: sums over the window
        // NORM: statistics of the iteration at hand.  Every thread of the slot derives the same
        // numbers from the same sums; one of them files them in LDS for the reverse sweep, which
        // starts with those of the last iteration still in these registers (no barrier lies
        // between that iteration and the sweep).
        float mean = 0.f, sd = 1.f, inv = 1.f;
        if (active) {
#pragma unroll
            for (int c = 0; c < CPT; ++c) cur[c] = win[pl.own + c];
            if (NORM) {
#pragma unroll
                for (int q = 0; q < NW; ++q) {  // fixed order: every thread forms the same sums
                    const float4 p4 = *reinterpret_cast<const float4 *>(ncommit + q * 4);
                    halo1 += p4.x; halo2 += p4.y; own1 += p4.z; own2 += p4.w;
                }
            }
        }

        // ---- forward recompute, remembering x_i and u_i of the owned cells ----
        for (int it = 0; it < inner; ++it) {
            if (active) {
                float u[CPT];
                if (NORM) {
                    if (it > 0) {
                        own1 = own2 = 0.f;
#pragma unroll
                        for (int q = 0; q < NW; ++q) {
                            const float2 p2 = *reinterpret_cast<const float2 *>(nown + ((it & 1) * NW + q) * 2);
                            own1 += p2.x; own2 += p2.y;
                        }
                    }
                    mean = (halo1 + own1) * inv_count;
                    sd = sqrtf(fmaxf(fmaf(-mean, mean, (halo2 + own2) * inv_count), 0.f));
                    inv = 1.f / (sd + norm_eps);
                    if (pl.lane == 0) *reinterpret_cast<float4 *>(nstat + 4 * it) = make_float4(mean, sd, inv, 0.f);
                    stencil<TL, CPT, kBwdDepth>(win + (it & 1) * TL::WIN, pl.row00, w, zero, u);
                    float wsum[CPT];
                    load_cells<CPT>(wsum_at, wsum);
#pragma unroll
                    for (int c = 0; c < CPT; ++c) u[c] = fmaf(inv, fmaf(-mean, wsum[c], u[c]), bv[c]);
                } else {
                    stencil<TL, CPT, kBwdDepth>(win + (it & 1) * TL::WIN, pl.row00, w, bv, u);
                }
                float *h = hist + it * (TL::TPS * 2 * CPT);
                store_cells<CPT>(h, cur);
                store_cells<CPT>(h + TL::TPS * CPT, u);
                if (it + 1 < inner) {
                    float s1 = 0.f, s2 = 0.f;
#pragma unroll
                    for (int c = 0; c < CPT; ++c) {
                        cur[c] = fmaf(rv[c], Act<ACT, float>::f(u[c]), cur[c]);
                        win[((it + 1) & 1) * TL::WIN + pl.own + c] = cur[c];
                        s1 += cur[c];
                        s2 = fmaf(cur[c], cur[c], s2);
                    }
                    if (NORM) {  // the owned cells' part of the next iteration's statistics
                        s1 = slot_wave_sum<TL::TPS>(s1);
                        s2 = slot_wave_sum<TL::TPS>(s2);
                        if ((pl.lane & 63 & (TL::TPS - 1)) == 0)
                            *reinterpret_cast<float2 *>(nown + (((it + 1) & 1) * NW + wave_in_slot) * 2) =
                                make_float2(s1, s2);
                    }
                } else {  // x_inner itself is never needed: that copy becomes the halo window
#pragma unroll
                    for (int c = 0; c < CPT; ++c) win[((it + 1) & 1) * TL::WIN + pl.own + c] = 0.f;
                }
            }
            if (it + 1 < inner) slot_barrier<TL::TPS>();
        }

        // ---- reverse sweep: delta window copy (it & 1) holds delta_it ----
        // NORM: dsum is D1, d2 is D2; x_i of the owned cells as the stencil saw it (xn); delta of
        // the iteration; the halo brackets (wout is fixed, sout belongs to the element); Q and R
        float dsum[CPT], xi[CPT], xn[CPT], d2[CPT], dlt[CPT], sout[CPT], q_sum = 0.f, r_sum = 0.f;
#pragma unroll
        for (int c = 0; c < CPT; ++c) dsum[c] = d2[c] = sout[c] = 0.f;
        for (int it = inner - 1; it >= 0; --it) {
            if (active) {
                const float *h = hist + it * (TL::TPS * 2 * CPT);
                float u[CPT];
                load_cells<CPT>(h, xi);
                load_cells<CPT>(h + TL::TPS * CPT, u);
                if (NORM && it < inner - 1) {
                    const float4 st4 = *reinterpret_cast<const float4 *>(nstat + 4 * it);
                    mean = st4.x; sd = st4.y; inv = st4.z;
                }
#pragma unroll
                for (int c = 0; c < CPT; ++c) {
                    float f, d;
                    Act<ACT, float>::fd(u[c], f, d);
                    const float delta = d * g[c] * rv[c];
                    dr[c] = fmaf(f, g[c], dr[c]);
                    db[c] += delta;
                    if (NORM) {
                        dlt[c] = delta;
                        dsum[c] = fmaf(inv, delta, dsum[c]);
                        d2[c] = fmaf(mean * inv, delta, d2[c]);
                        xn[c] = (xi[c] - mean) * inv;
                    } else {
                        dsum[c] += delta;
                        xn[c] = xi[c];
                    }
                    dwin[(it & 1) * TL::WIN + pl.own + c] = delta;
                }
            }
            if (it == 0) {
                // D is complete: the weights of the taps that read the halo.  Before this
                // iteration's barrier, so that nobody commits the next element's window while
                // the halo is read; behind a barrier of its own when the zeros of the halo
                // window were written in the iteration just before (inner == 1).
                if (inner == 1) slot_barrier<TL::TPS>();
                if (active)
                    for_each_row<TL, CPT, kBwdDepth>(xhalo + pl.row00, [&](int r, const float (&xv)[CPT + 2]) {
#pragma unroll
                        for (int cc = 0; cc < 3; ++cc)
#pragma unroll
                            for (int c = 0; c < CPT; ++c)
                                nw[r * 3 + cc][c] = fmaf(xv[c + cc], dsum[c], nw[r * 3 + cc][c]);
                    });
            }
            slot_barrier<TL::TPS>();
            if (NORM && active && it == inner - 1) {
                // once per element: what the owned cells' taps into the halo see there (the
                // halo window holds zeros in the block's cells, so the other taps add nothing)
                stencil<TL, CPT, kBwdDepth>(xhalo, pl.row00, w, zero, sout);
            }
            float dn[CPT];  // NORM: gradient with respect to the normalised value of the owned cells
#pragma unroll
            for (int c = 0; c < CPT; ++c) dn[c] = 0.f;
            if (active) {
                const float *dwn = dwin + (it & 1) * TL::WIN + pl.row00;
                for_each_row<TL, CPT, kBwdDepth>(dwn, [&](int r, const float (&dv)[CPT + 2]) {
#pragma unroll
                    for (int cc = 0; cc < 3; ++cc)
#pragma unroll
                        for (int c = 0; c < CPT; ++c) {
                            nw[r * 3 + cc][c] = fmaf(xn[c], dv[c + cc], nw[r * 3 + cc][c]);
                            if (NORM) dn[c] = fmaf(v[r * 3 + cc][c], dv[c + cc], dn[c]);
                            else g[c] = fmaf(v[r * 3 + cc][c], dv[c + cc], g[c]);
                        }
                });
            }
            if (NORM) {
                // A = sum dn and sum dn * x over the whole window, the halo through its brackets
                float pa = 0.f, pb = 0.f;
                if (active) {
                    float wout[CPT];
                    load_cells<CPT>(wout_at, wout);
#pragma unroll
                    for (int c = 0; c < CPT; ++c) {
                        pa += fmaf(dlt[c], wout[c], dn[c]);
                        pb += fmaf(dlt[c], sout[c], dn[c] * xi[c]);
                    }
                    pa = slot_wave_sum<TL::TPS>(pa);
                    pb = slot_wave_sum<TL::TPS>(pb);
                }
                if (NW > 1) {
                    if (active && (pl.lane & 63) == 0)
                        *reinterpret_cast<float2 *>(nrev + wave_in_slot * 2) = make_float2(pa, pb);
                    lds_barrier();
                    if (active) {
                        pa = pb = 0.f;
#pragma unroll
                        for (int q = 0; q < NW; ++q) {
                            const float2 p2 = *reinterpret_cast<const float2 *>(nrev + q * 2);
                            pa += p2.x; pb += p2.y;
                        }
                    }
                }
                if (active) {
                    const float a_mean = pa * inv_count;
                    const float proj = fmaf(-mean, pa, pb);  // sum dn (x - mean)
                    const float coef = proj * inv * inv * inv_count / fmaxf(sd, 1e-30f);
#pragma unroll
                    for (int c = 0; c < CPT; ++c)
                        g[c] += fmaf(inv, dn[c] - a_mean, -(xi[c] - mean) * coef);
                    q_sum += coef;
                    r_sum += fmaf(mean, coef, -inv * a_mean);
                }
            }
        }

        if (inner == 0) slot_barrier<TL::TPS>();  // no barrier since the top: others may still read LDS
        done_s = active ? s : -1;
#pragma unroll
        for (int c = 0; c < CPT; ++c) {
            // RES: what leaves is dn = (gradient with respect to n) - G'; the cells' own part takes
            // the whole of G', the cross-block kernel adds the rest of the first term
            g_done[c] = RES ? g[c] - gin[c] : g[c];
            d_done[c] = dsum[c];
            if (RES) gin_done[c] = gin[c];
        }
        if (NORM && active) {
            float d2acc[CPT];
            load_cells<CPT>(d2acc_at, d2acc);
#pragma unroll
            for (int c = 0; c < CPT; ++c) d2acc[c] += d2[c];
            store_cells<CPT>(d2acc_at, d2acc);
        }
        if (NORM) {
            q_done = q_sum;
            r_done = fmaf(shift, q_sum, r_sum);
        }
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
        for (int t = 0; t < 27; ++t)
#pragma unroll
            for (int c = 0; c < CPT; ++c) reduce(nw[t][c]);
#pragma unroll
        for (int c = 0; c < CPT; ++c) {
            reduce(db[c]);
            reduce(dr[c]);
            if (LN) {
                reduce(dgam[c]);
                reduce(dbet[c]);
            }
        }
        if (NORM) {  // D2 of the other slots: their entries lie one slot's stride further each
            lds_barrier();
            if (pl.slot == 0) {
                float d2acc[CPT];
                load_cells<CPT>(d2acc_at, d2acc);
#pragma unroll
                for (int q = 1; q < NSLOT; ++q) {
                    float more[CPT];
                    load_cells<CPT>(d2acc_at + q * norm_stride, more);
#pragma unroll
                    for (int c = 0; c < CPT; ++c) d2acc[c] += more[c];
                }
                store_cells<CPT>(d2acc_at, d2acc);
            }
        }
        if (pl.slot != 0) return;
    }
    if (NORM) {  // the taps that read the halo: x_h D1 was added per element, D2 is still owed
        float d2acc[CPT];
        load_cells<CPT>(d2acc_at, d2acc);
#pragma unroll
        for (int t = 0; t < 27; ++t)
#pragma unroll
            for (int c = 0; c < CPT; ++c) nw[t][c] -= in_block(t, c) ? 0.f : d2acc[c];
    }
    commit_grads<27, CPT>(dweight, nw, param_mode, owner_of, always);
    float one[1][CPT];
    auto own_cell = [&](int, int c) { return pl.gc + c; };
#pragma unroll
    for (int c = 0; c < CPT; ++c) one[0][c] = db[c];
    commit_grads<1, CPT>(dbias, one, param_mode, own_cell, always);
#pragma unroll
    for (int c = 0; c < CPT; ++c) one[0][c] = dr[c];
    commit_grads<1, CPT>(dscale, one, param_mode, own_cell, always);
    if (LN) {
#pragma unroll
        for (int c = 0; c < CPT; ++c) one[0][c] = dgam[c];
        commit_grads<1, CPT>(ln.dgamma, one, param_mode, own_cell, always);
#pragma unroll
        for (int c = 0; c < CPT; ++c) one[0][c] = dbet[c];
        commit_grads<1, CPT>(ln.dbeta, one, param_mode, own_cell, always);
    }
}

// ---- backward, second kernel: everything that crosses a block boundary ----------------------
// The window halo is frozen during the inner iterations, so the gradient that the cells of
// NEIGHBOURING blocks receive depends on the iterations only through D = sum_i delta_i, which
// step_bwd_fast leaves in `dsum`.  For a cell c of the block and a tap t with h = c + off_t in
// another block:
//   dx[c] += W[26-t, h] * D[h]        (h's mirrored tap reads c)
// Only boundary cells have such taps, and a tap leaves the block through a face: the work is
// dealt by FACE.  A slot (one batch element of the block) is 6 faces of bs*bs threads; the
// thread of face cell c owns the 9 taps that leave through its face, minus those that also
// leave through a face of a lower axis (edges and corners; counted there).  So every
// (cell, tap) pair has exactly one thread, which keeps its mirrored weight in registers for the
// whole batch.  The D window of the element sits in LDS with its REAL halo (the neighbouring
// blocks' values, zero outside the grid), two stages alternating, fetched one round ahead.  Every thread leaves what it found
// for its cell in a small LDS slab; one round late (after the next barrier) the slot's row
// threads add the parts of each cell to dx in a fixed order; no atomics.
// A pass over one element is short (9 LDS reads, 9 FMAs per thread), and a block has few
// workgroups to hide latency behind: a slot therefore takes E elements per round, so that
// one barrier, one trip to LDS and one trip to memory serve E elements.
// LN (the LayerNorm of the network body folded in, see LnFold): when x is the raw output of the
// step before, dx as this kernel completes it is the gradient with respect to LayerNorm(x).  The
// row threads, which hold the finished rows, then also form the two per-sample sums that
// LayerNorm's backward needs, sum(gamma dx) and sum(gamma dx xhat), and leave them per 16 lanes;
// for that they load their row of x beside their row of dx.
// RES (with LN): the outer_residual form of the loop, see LnFold: what goes to dx (and into the
// sums) is dn = (the gradient with respect to n = LayerNorm(x)) - G', G' the gradient with respect
// to the step's output; step_bwd_fast has taken G' off the cells' own part, so nothing differs here.
// NORM (per-window normalisation, see step_bwd_fast): `dsum` holds D1, and a cell that lies in
// the halo of a neighbouring block a additionally receives R_a - x Q_a from it, Q and R being
// the two numbers per (element, block) that step_bwd_fast left in `qr`.  The row threads add
// that: they load their row of x, and the (Q, R) of the 26 neighbours of the block travel
// through LDS with the D windows.
// SETS = 2: the gated variant of the update (weight [27, 2, M, N, K]): two D tensors, one behind
// the other in `dsum`, each with its own set of mirrored weights; the cell receives the sum.
template <int BS, int NSLOT, int E, bool LN, bool RES = false, bool NORM = false, int SETS = 1>
__global__ __launch_bounds__((6 * BS * BS * NSLOT)) __attribute__((amdgpu_waves_per_eu(3)))
void step_bwd_cross(
    const float *__restrict__ weight, const float *__restrict__ x, const float *__restrict__ dsum,
    float *__restrict__ dx, int B, int M, int N, int K, int nblk, int nchunk, int chunk_len,
    LnFold ln, const float *__restrict__ qr) {
    using TL = Tile<BS, 1>;  // window geometry only
    constexpr int FS = BS * BS, TPS = 6 * FS;
    constexpr int PAIR = SETS * TL::WIN;           // the D window(s) of one element
    constexpr int STAGE = E * PAIR;                // the E elements of a round
    constexpr int QRS = NORM ? 2 * E * 27 * 2 : 0; // NORM: (Q, R) of the neighbours, two stages
    constexpr int SLOT = 2 * STAGE + 2 * E * TPS + QRS;  // two stages, two slabs
    __shared__ __attribute__((aligned(16))) float lds[NSLOT * SLOT];
    static_assert(!(NORM && (LN || RES)), "the folded LayerNorm comes without normalisation");

    int blk, chunk;
    if (!split_block_id(blockIdx.x, nblk, nchunk, blk, chunk)) return;  // grid padding
    const int slot = NSLOT == 1 ? 0 : threadIdx.x / TPS, lane = threadIdx.x - slot * TPS;
    const int kb = K / BS, nb = N / BS;
    const int p0 = (blk / (kb * nb)) * BS, q0 = ((blk / kb) % nb) * BS, r0 = (blk % kb) * BS;
    const FetchLines<TL, TPS> fx(lane, p0, q0, r0, M, N, K);
    float *stages = lds + slot * SLOT, *slabs = stages + 2 * STAGE;
    const long cells = (long)M * N * K;

    // ---- which cell, which taps ----
    const int face = lane / FS, axis = face >> 1, side = face & 1;
    const int u = (lane % FS) / BS, v = lane % BS, fix = side ? BS - 1 : 0;
    const int ci = axis == 0 ? fix : u;
    const int cj = axis == 0 ? u : axis == 1 ? fix : v;
    const int ck = axis == 2 ? fix : v;
    const int gcell = ((p0 + ci) * N + (q0 + cj)) * K + (r0 + ck);
    const int own = (ci + 1) * TL::PS + (cj + 1) * TL::RS + (ck + 1);
    const int out = side ? 1 : -1;  // the face's outward direction along its axis
    // The first bs*bs threads of the slot double as ROW threads: thread (ri, rj) adds what the
    // faces found for the bs cells of block row (ri, rj) to dx, whole rows at a time (a row is
    // one vector-cache line access to read and one to write; cell by cell it would be eight).
    const bool is_row = lane < FS;
    const int ri = lane / BS, rj = lane % BS;  // meaningful for row threads only
    const long grow = ((long)(p0 + ri) * N + (q0 + rj)) * K + r0;
    const bool ri_edge = ri == 0 || ri == BS - 1, rj_edge = rj == 0 || rj == BS - 1;

    const bool ln_in = LN && ln.x_stats != nullptr;
    // NORM: thread n < 27 fetches (Q, R) of the neighbouring block at offset
    // (n/9 - 1, (n/3)%3 - 1, n%3 - 1); blocks outside the grid (and the block itself) count as 0
    float *qrs = slabs + 2 * E * TPS;  // [2 stages][E][27][2]
    int qr_blk = -1;
    if (NORM && lane < 27 && lane != 13) {
        const int mb = M / BS;
        const int bi = blk / (kb * nb) + lane / 9 - 1, bj = (blk / kb) % nb + (lane / 3) % 3 - 1,
                  bk = blk % kb + lane % 3 - 1;
        if (bi >= 0 && bi < mb && bj >= 0 && bj < nb && bk >= 0 && bk < kb) qr_blk = (bi * nb + bj) * kb + bk;
    }
    float vx[SETS][9];
    float grw[BS];  // LN, row threads: gamma of their row
    if (ln_in && is_row) load_cells<BS>(ln.gamma + grow, grw);
    int hoff[9];
    bool mine[9];
#pragma unroll
    for (int pq = 0; pq < 9; ++pq) {
        const int dp = pq / 3 - 1, dq = pq % 3 - 1;  // steps along the two in-face axes
        const int di = axis == 0 ? out : dp;
        const int dj = axis == 0 ? dp : axis == 1 ? out : dq;
        const int dk = axis == 2 ? out : dq;
        const int t = (di + 1) * 9 + (dj + 1) * 3 + (dk + 1);
        // also leaving through a face of a lower axis: that face's thread has the pair
        const bool lower = (axis >= 1 && ((di < 0 && ci == 0) || (di > 0 && ci == BS - 1))) ||
                           (axis == 2 && ((dj < 0 && cj == 0) || (dj > 0 && cj == BS - 1)));
        const int gi = p0 + ci + di, gj = q0 + cj + dj, gk = r0 + ck + dk;
        const bool in_grid = gi >= 0 && gi < M && gj >= 0 && gj < N && gk >= 0 && gk < K;
        mine[pq] = !lower;
        hoff[pq] = own + di * TL::PS + dj * TL::RS + dk;
        const long hcell = gcell + (long)(di * N + dj) * K + dk;
#pragma unroll
        for (int k = 0; k < SETS; ++k)
            vx[k][pq] = (mine[pq] && in_grid) ? weight[((26 - t) * SETS + k) * cells + hcell] : 0.f;
    }
    wait_global_loads();

    const int s0 = chunk * chunk_len, s1 = min(B, s0 + chunk_len);
    using Buf = typename FetchLines<TL, TPS>::Buf;
    // element e of round r of this slot; past the end of the chunk it is not `real`
    auto sample = [&](int r, int e) { return s0 + (r * E + e) * NSLOT + slot; };
    Buf pd[E][SETS];
    float2 pq[E];  // NORM: (Q, R) of this thread's neighbour block
    // Loads and commits are unconditional (past the end of the chunk they repeat its last
    // element, which nobody then uses): with branches around them the compiler cannot count the
    // loads in flight and waits for ALL of them wherever it needs one.
    auto fetch_round = [&](int r) {
#pragma unroll
        for (int e = 0; e < E; ++e) {
            const int sc = min(sample(r, e), s1 - 1);
            const long at = (long)sc * cells;
#pragma unroll
            for (int k = 0; k < SETS; ++k) fx.fetch(dsum + (long)k * B * cells + at, pd[e][k]);
            if (NORM) {  // every thread loads (a valid address always), the commit selects
                const float *from = qr + ((long)sc * nblk + (qr_blk >= 0 ? qr_blk : blk)) * 2;
                pq[e] = make_float2(from[0], from[1]);
            }
        }
    };
    auto commit_round = [&](int st) {
#pragma unroll
        for (int e = 0; e < E; ++e) {
#pragma unroll
            for (int k = 0; k < SETS; ++k)
                fx.template commit<1>(stages + st * STAGE + e * PAIR + k * TL::WIN, pd[e][k]);
            if (NORM && lane < 27)
                *reinterpret_cast<float2 *>(qrs + ((st * E + e) * 27 + lane) * 2) =
                    qr_blk >= 0 ? pq[e] : make_float2(0.f, 0.f);
        }
    };
    float gx[E][BS];  // row threads: dx of their row so far (the own block's part)
    float xr[E][BS], xmean[E], xrstd[E];  // LN, row threads: their row of x and its statistics
    int r_prev = -1;
    // the round before: its parts are all in slab `st` by now (a barrier lies in between)
    auto finish_prev = [&](int st) {
        if (r_prev >= 0 && is_row) {
#pragma unroll
            for (int e = 0; e < E; ++e) {
                const int s = sample(r_prev, e);
                const float *slab = slabs + (st * E + e) * TPS;
                // fixed order per cell: k faces, then i face, then j face
                gx[e][0] += slab[4 * FS + ri * BS + rj];
                gx[e][BS - 1] += slab[5 * FS + ri * BS + rj];
                if (ri_edge) {
                    float part[BS];
                    load_cells<BS>(slab + (ri == 0 ? 0 : 1) * FS + rj * BS, part);
#pragma unroll
                    for (int c = 0; c < BS; ++c) gx[e][c] += part[c];
                }
                if (rj_edge) {
                    float part[BS];
                    load_cells<BS>(slab + (rj == 0 ? 2 : 3) * FS + ri * BS, part);
#pragma unroll
                    for (int c = 0; c < BS; ++c) gx[e][c] += part[c];
                }
                if (NORM) {
                    // neighbours that have this row in their halo, by their offset along K:
                    // (0, 0), (ei, 0), (0, ej), (ei, ej) with ei, ej the side of the block the
                    // row lies on, if any; along K only the row's end cells are concerned
                    const float *q27 = qrs + (st * E + e) * 27 * 2;
                    const int ei = ri == 0 ? -1 : ri == BS - 1 ? 1 : 0, ej = rj == 0 ? -1 : rj == BS - 1 ? 1 : 0;
                    float rq[3], rr[3];
#pragma unroll
                    for (int dk = 0; dk < 3; ++dk) {
                        float sq = 0.f, sr = 0.f;
                        auto add = [&](int a, int b) {
                            const float2 v2 = *reinterpret_cast<const float2 *>(q27 + (((a + 1) * 3 + (b + 1)) * 3 + dk) * 2);
                            sq += v2.x;
                            sr += v2.y;
                        };
                        if (dk != 1) add(0, 0);
                        if (ei != 0) add(ei, 0);
                        if (ej != 0) add(0, ej);
                        if (ei != 0 && ej != 0) add(ei, ej);
                        rq[dk] = sq;
                        rr[dk] = sr;
                    }
#pragma unroll
                    for (int c = 0; c < BS; ++c) gx[e][c] += fmaf(-xr[e][c], rq[1], rr[1]);
                    gx[e][0] += fmaf(-xr[e][0], rq[0], rr[0]);
                    gx[e][BS - 1] += fmaf(-xr[e][BS - 1], rq[2], rr[2]);
                }
                if (s < s1) store_cells<BS>(dx + (long)s * cells + grow, gx[e]);
                if (ln_in) {
                    float t1 = 0.f, t2 = 0.f;
#pragma unroll
                    for (int c = 0; c < BS; ++c) {
                        const float a = grw[c] * gx[e][c];
                        t1 += a;
                        t2 = fmaf(a, (xr[e][c] - xmean[e]) * xrstd[e], t2);
                    }
                    // one pair per (element, block): the row threads are 16 lanes (bs=4), or the
                    // whole first wave of the slot (bs=8)
                    static_assert(FS == 16 || (FS == 64 && TPS % 64 == 0), "row threads fill a row or a wave");
                    const float w1 = FS == 64 ? slot_wave_sum<64>(t1) : row16_sum(t1);
                    const float w2 = FS == 64 ? slot_wave_sum<64>(t2) : row16_sum(t2);
                    if (lane == 0 && s < s1) {
                        float *to = ln.x_part + ((long)s * nblk + blk) * 2;
                        to[0] = w1;
                        to[1] = w2;
                    }
                }
            }
        }
        r_prev = -1;
    };
    const int rounds = (s1 - s0 + E * NSLOT - 1) / (E * NSLOT);
    fetch_round(0);
    commit_round(0);
    for (int r = 0; r < rounds; ++r) {
        const int st = r & 1;
        lds_barrier();  // stage `st` and slab `st ^ 1` are complete; their old readers are done
        finish_prev(st ^ 1);
        if (is_row) {  // requested before the prefetch, so that they are awaited first
#pragma unroll
            for (int e = 0; e < E; ++e) {
                const int sc = min(sample(r, e), s1 - 1);
                load_cells<BS>(dx + (long)sc * cells + grow, gx[e]);
                if (NORM) load_cells<BS>(x + (long)sc * cells + grow, xr[e]);
                if (ln_in) {
                    load_cells<BS>(x + (long)sc * cells + grow, xr[e]);
                    xmean[e] = load_ahead(ln.x_stats, 2 * sc);
                    xrstd[e] = load_ahead(ln.x_stats, 2 * sc + 1);
                }
            }
        }
        fetch_round(r + 1);
#pragma unroll
        for (int e = 0; e < E; ++e) {
            float g = 0.f;
#pragma unroll
            for (int k = 0; k < SETS; ++k) {
                const float *dw = stages + st * STAGE + e * PAIR + k * TL::WIN;
                float dh[9];
#pragma unroll
                for (int pq = 0; pq < 9; ++pq) dh[pq] = dw[hoff[pq]];
#pragma unroll
                for (int pq = 0; pq < 9; ++pq) g = fmaf(vx[k][pq], dh[pq], g);
            }
            slabs[(st * E + e) * TPS + lane] = g;
        }
        r_prev = r;
        commit_round(st ^ 1);
    }
    lds_barrier();
    finish_prev((rounds - 1) & 1);
}

__global__ void fill_zero_f32(float *p, long n) {
    long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    const long stride = (long)gridDim.x * blockDim.x;
    for (; i < n; i += stride) p[i] = 0.f;
}

int fill_zero(float *p, long n, hipStream_t st) {
    if (n <= 0) return GRIDNET_OK;
    long blocks = (n + 1023) / 1024;
    if (blocks > 8192) blocks = 8192;
    hipLaunchKernelGGL(fill_zero_f32, dim3((unsigned)blocks), dim3(256), 0, st, p, n);
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

struct Plan {
    int nblk, nchunk, chunk_len;
};

// The batch is dealt to workgroups in chunks; a chunk is walked NSLOT elements at a time.
// `resident` = workgroups the chip holds at once: when the blocks alone do not fill it, the
// batch is split so that the grid is one full wave of workgroups.
Plan make_plan(const StepArgs &a, int nslot, int resident, bool whole_batch_per_wg) {
    Plan p;
    const int bs = a.block_size;
    p.nblk = (a.M / bs) * (a.N / bs) * (a.K / bs);
    int nchunk = whole_batch_per_wg ? 1 : resident / p.nblk;
    const int max_chunks = (a.B + nslot - 1) / nslot;
    if (nchunk > max_chunks) nchunk = max_chunks;
    if (nchunk < 1) nchunk = 1;
    p.chunk_len = (a.B + nchunk - 1) / nchunk;
    p.chunk_len = (p.chunk_len + nslot - 1) / nslot * nslot;
    p.nchunk = (a.B + p.chunk_len - 1) / p.chunk_len;
    return p;
}

template <int BS, int CPT, int NSLOT, int ACT, bool LN, bool RES = false, bool NORM = false>
int launch_fwd_ln(const StepArgs &a, hipStream_t st) {
    using TL = Tile<BS, CPT>;
    auto kern = step_fwd_fast<BS, CPT, NSLOT, ACT, LN, RES, NORM>;
    static int per_cu = 0;
    if (per_cu == 0) {
        int n = 0;
        if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, kern, TL::TPS * NSLOT, 0) != hipSuccess ||
            n < 1)
            n = 1;
        per_cu = n;
    }
    const Plan p = make_plan(a, NSLOT, per_cu * device_cus(), false);
    hipLaunchKernelGGL(kern, dim3(padded_grid(p.nblk, p.nchunk)), dim3(TL::TPS * NSLOT), 0, st,
                       (const float *)a.weight, (const float *)a.bias, (const float *)a.scale,
                       (const float *)a.x, (float *)a.y, a.B, a.M, a.N, a.K, a.inner, p.nblk, p.nchunk,
                       p.chunk_len, a.ln, (float)a.eps);
    return check_launch("step_fwd_fast");
}
template <int ACT, bool LN, bool RES = false, bool NORM = false>
int launch_fwd_split(const StepArgs &a, hipStream_t st) {
    auto kern = step_fwd_split<ACT, LN, RES, NORM>;
    static int per_cu = 0;
    if (per_cu == 0) {
        int n = 0;
        if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, kern, 128, 0) != hipSuccess || n < 1) n = 1;
        per_cu = n;
    }
    const Plan p = make_plan(a, 1, per_cu * device_cus(), false);
    hipLaunchKernelGGL(kern, dim3(padded_grid(p.nblk, p.nchunk)), dim3(128), 0, st,
                       (const float *)a.weight, (const float *)a.bias, (const float *)a.scale,
                       (const float *)a.x, (float *)a.y, a.B, a.M, a.N, a.K, a.inner, p.nblk, p.nchunk,
                       p.chunk_len, a.ln, (float)a.eps);
    return check_launch("step_fwd_split");
}
template <int ACT> int launch_fwd_pair(const StepArgs &a, hipStream_t st) {
    auto kern = step_fwd_pair<ACT>;
    static int per_cu = 0;
    if (per_cu == 0) {
        int n = 0;
        if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, kern, 128, 0) != hipSuccess || n < 1) n = 1;
        per_cu = n;
    }
    const Plan p = make_plan(a, 2, per_cu * device_cus(), false);
    hipLaunchKernelGGL(kern, dim3(padded_grid(p.nblk, p.nchunk)), dim3(128), 0, st,
                       (const float *)a.weight, (const float *)a.bias, (const float *)a.scale,
                       (const float *)a.x, (float *)a.y, a.B, a.M, a.N, a.K, a.inner, p.nblk, p.nchunk,
                       p.chunk_len, a.ln);
    return check_launch("step_fwd_pair");
}
template <int BS, int CPT, int NSLOT, int ACT> int launch_fwd(const StepArgs &a, hipStream_t st) {
    if (a.normalize) {
        if (BS == 8) return launch_fwd_split<ACT, false, false, true>(a, st);
        return launch_fwd_ln<BS, CPT, NSLOT, ACT, false, false, true>(a, st);
    }
    if (a.ln.gamma && a.ln.residual) {
        if (BS == 8) return launch_fwd_split<ACT, true, true>(a, st);
        return launch_fwd_ln<BS, CPT, NSLOT, ACT, true, true>(a, st);
    }
    // The chain's forward on SMALL grids (fewer blocks than a sixth of the workgroups the chip
    // holds, so that a workgroup of step_fwd_split gets four batch elements or fewer for one fetch
    // of its 29 parameter planes): two elements per pass.  Measured with 3 waves per SIMD for
    // step_fwd_split: 32^3 grid, batch 64: 0.279 -> 0.238 ms per 8-step chain; on larger grids the
    // lower occupancy of the pair kernel costs more than it brings (64^3 / batch 32: 66 -> 69 us
    // per step, 128^3 / batch 8: 2.61 -> 3.00 ms per 16-step chain).
    if (BS == 8 && a.ln.gamma && a.B >= 2 && a.inner >= 1) {
        const int nblk = (a.M / 8) * (a.N / 8) * (a.K / 8);
        const int chunks = 6 * device_cus() / nblk;  // what step_fwd_split's plan would use
        if (chunks >= 1 && (a.B + chunks - 1) / chunks <= 4) return launch_fwd_pair<ACT>(a, st);
    }
    if (BS == 8) return a.ln.gamma ? launch_fwd_split<ACT, true>(a, st) : launch_fwd_split<ACT, false>(a, st);
    if (a.ln.gamma) return launch_fwd_ln<BS, CPT, NSLOT, ACT, true>(a, st);
    return launch_fwd_ln<BS, CPT, NSLOT, ACT, false>(a, st);
}

constexpr size_t kMaxLds = 160 * 1024;

// the cross-block kernel's own shapes (it shares the main kernel's blocks and batch chunks)
constexpr int kCrossSlots8 = 1, kCrossElems8 = 2;  // bs=8: 384 threads, one wave per face
constexpr int kCrossSlots4 = 2, kCrossElems4 = 2;  // bs=4: two slots of 96 threads

template <int BS, int CPT, int NSLOT, int ACT, bool LN, bool RES = false, bool NORM = false>
int launch_bwd_ln(const StepArgs &a, hipStream_t st) {
    using TL = Tile<BS, CPT>;
    const long cells = (long)a.M * a.N * a.K;
    const size_t lds = bwd_lds_bytes<BS, CPT, NSLOT>(a.inner, LN, NORM);
    auto kern = step_bwd_fast<BS, CPT, NSLOT, ACT, LN, RES, NORM>;
    static bool big_lds_enabled = false;            // per instantiation
    static int per_cu_cache[kMaxBackwardIters + 1];  // per instantiation, by inner iterations
    if (lds > 64 * 1024 && !big_lds_enabled) {
        hipError_t e = hipFuncSetAttribute((const void *)kern,
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)kMaxLds);
        if (e != hipSuccess)
            return fail(GRIDNET_ERR_LAUNCH, "cannot enable %zu bytes of LDS: %s", lds,
                        hipGetErrorString(e));
        big_lds_enabled = true;
    }
    int &per_cu = per_cu_cache[a.inner];
    if (per_cu == 0) {
        int n = 0;
        if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, kern, TL::TPS * NSLOT, lds) != hipSuccess ||
            n < 1)
            n = 1;
        per_cu = n;
    }
    const int nblk = (a.M / BS) * (a.N / BS) * (a.K / BS);
    // one workgroup owns the whole batch of its block (no cross-workgroup reduction of the
    // parameter gradients) as soon as the blocks alone give every CU a workgroup
    const bool whole = nblk >= device_cus();
    Plan p = make_plan(a, NSLOT, per_cu * device_cus(), whole);
    const bool new_params = (a.flags & GRIDNET_OVERWRITE_PARAMS) != 0;
    // A split batch: every chunk gets a copy of the gradient arrays in the scratch; with less
    // room than chunks the batch is split less (down to not at all).
    const long slab_floats = kStepSlabPlanes * cells;
    if (p.nchunk > 1) {
        const int room = plan_split_room(plan_slab_capacity(a.slabs, a.slab_bytes, slab_floats), a.B, p.chunk_len);
        if (room < p.nchunk) p = make_plan(a, NSLOT, (room < 2 ? 1 : room) * nblk, room < 2);
    }
    const bool split = p.nchunk > 1;
    const int param_mode = split || new_params ? kParamStore : kParamAddExclusive;
    float *slab = (float *)a.slabs;
    LnFold ln = a.ln;
    if (split && LN) {
        ln.dgamma = slab + 29 * cells;
        ln.dbeta = slab + 30 * cells;
    }
    const int dx_accumulate = (a.flags & GRIDNET_OVERWRITE_DX) ? 0 : 1;
    // NORM: (Q, R) per (element, block), behind the D tensor in the workspace
    float *qr = NORM ? (float *)a.workspace + (size_t)a.B * cells : nullptr;
    hipLaunchKernelGGL(kern, dim3(padded_grid(p.nblk, p.nchunk)), dim3(TL::TPS * NSLOT), lds, st,
                       (const float *)a.weight, (const float *)a.bias, (const float *)a.scale,
                       (const float *)a.x, (const float *)a.dy, split ? slab : (float *)a.dweight,
                       split ? slab + 27 * cells : (float *)a.dbias,
                       split ? slab + 28 * cells : (float *)a.dscale, (float *)a.dx,
                       (float *)a.workspace, a.B, a.M, a.N, a.K, a.inner, p.nblk, p.nchunk, p.chunk_len,
                       param_mode, dx_accumulate, ln, (float)a.eps, qr, split ? slab_floats : 0L);
    if (int rc = check_launch("step_bwd_fast")) return rc;
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
        if (int rc = plan_reduce_slabs(slab, p.nchunk, slab_floats, t, new_params ? 0 : 1, st)) return rc;
    }
    // same blocks, same batch chunks; the parameter gradients are complete, dx is not yet
    constexpr int XSLOT = BS == 8 ? kCrossSlots8 : kCrossSlots4;
    constexpr int XE = BS == 8 ? kCrossElems8 : kCrossElems4;
    if (cross_rows_supports(a)) return cross_rows_launch(a, st);  // by whole K-rows
    hipLaunchKernelGGL((step_bwd_cross<BS, XSLOT, XE, LN, false, NORM>), dim3(padded_grid(p.nblk, p.nchunk)),
                       dim3(6 * BS * BS * XSLOT), 0, st, (const float *)a.weight,
                       (const float *)a.x, (const float *)a.workspace, (float *)a.dx, a.B, a.M, a.N,
                       a.K, p.nblk, p.nchunk, p.chunk_len, a.ln, (const float *)qr);
    if (int rc = check_launch("step_bwd_cross")) return rc;
    return GRIDNET_OK;
}
template <int BS, int CPT, int NSLOT, int ACT> int launch_bwd(const StepArgs &a, hipStream_t st) {
    if (a.normalize) return launch_bwd_ln<BS, CPT, NSLOT, ACT, false, false, true>(a, st);
    if (a.ln.gamma && a.ln.residual) return launch_bwd_ln<BS, CPT, NSLOT, ACT, true, true>(a, st);
    if (a.ln.gamma) return launch_bwd_ln<BS, CPT, NSLOT, ACT, true>(a, st);
    return launch_bwd_ln<BS, CPT, NSLOT, ACT, false>(a, st);
}

// ---- the tuned shapes ---------------------------------------------------------------------
constexpr int kFwdCpt8 = 4, kFwdSlots8 = 1;   // bs=8 forward: 128 threads, 4 cells each
constexpr int kBwdCpt8 = 2, kBwdSlots8 = 1;   // bs=8 backward: 256 threads, 2 cells each
constexpr int kFwdCpt4 = 2, kFwdSlots4 = 4;   // bs=4: 32-thread slots, 4 per workgroup
constexpr int kBwdCpt4 = 2, kBwdSlots4 = 2;   // bs=4 backward: two 32-thread slots, 2 cells per thread

template <bool BWD, int ACT> int dispatch_bs(const StepArgs &a, hipStream_t st) {
    if (a.block_size == 8) {
        if (BWD) return launch_bwd<8, kBwdCpt8, kBwdSlots8, ACT>(a, st);
        return launch_fwd<8, kFwdCpt8, kFwdSlots8, ACT>(a, st);
    }
    if (BWD) return launch_bwd<4, kBwdCpt4, kBwdSlots4, ACT>(a, st);
    return launch_fwd<4, kFwdCpt4, kFwdSlots4, ACT>(a, st);
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

// The cross-block kernel alone, completing a dx whose block-local part another kernel wrote
// (8^3 blocks; the LayerNorm fold as a.ln says; D in a.workspace).
int step_cross_launch(const StepArgs &a, int nchunk, int chunk_len, hipStream_t st) {
    if (cross_rows_supports(a)) return cross_rows_launch(a, st);
    const int nblk = (a.M / 8) * (a.N / 8) * (a.K / 8);
    hipLaunchKernelGGL((step_bwd_cross<8, kCrossSlots8, kCrossElems8, true>), dim3(padded_grid(nblk, nchunk)),
                       dim3(6 * 64 * kCrossSlots8), 0, st, (const float *)a.weight, (const float *)a.x,
                       (const float *)a.workspace, (float *)a.dx, a.B, a.M, a.N, a.K, nblk, nchunk,
                       chunk_len, a.ln, (const float *)nullptr);
    return check_launch("step_bwd_cross");
}

// The cross-block kernel for the gated update: D0 and D1 of every cell behind one another in
// `dsum`, weight [27, 2, M, N, K]; same blocks and batch chunks as the kernel that left them.
int gated_cross_launch(const StepArgs &a, const float *dsum, int nchunk, int chunk_len, hipStream_t st) {
    if (cross_rows_gated_supports(a)) return cross_rows_gated_launch(a, dsum, st);
    const int bs = a.block_size;
    const int nblk = (a.M / bs) * (a.N / bs) * (a.K / bs);
    const LnFold none{};
    if (bs == 8)
        hipLaunchKernelGGL((step_bwd_cross<8, kCrossSlots8, 1, false, false, false, 2>),
                           dim3(padded_grid(nblk, nchunk)), dim3(6 * 64 * kCrossSlots8), 0, st,
                           (const float *)a.weight, (const float *)a.x, dsum, (float *)a.dx, a.B, a.M,
                           a.N, a.K, nblk, nchunk, chunk_len, none, (const float *)nullptr);
    else
        hipLaunchKernelGGL((step_bwd_cross<4, kCrossSlots4, 1, false, false, false, 2>),
                           dim3(padded_grid(nblk, nchunk)), dim3(6 * 16 * kCrossSlots4), 0, st,
                           (const float *)a.weight, (const float *)a.x, dsum, (float *)a.dx, a.B, a.M,
                           a.N, a.K, nblk, nchunk, chunk_len, none, (const float *)nullptr);
    return check_launch("step_bwd_cross (gated)");
}

// one pair per wave of a slot, or per slot where a slot is half a wave
int step_fast_forward_parts(int block_size) {
    const int tps = block_size == 8 ? Tile<8, kFwdCpt8>::TPS : Tile<4, kFwdCpt4>::TPS;
    return tps >= 64 ? tps / 64 : 1;
}
int step_fast_forward_part_count(int block_size) {
    return block_size * block_size * block_size / step_fast_forward_parts(block_size);
}
// per block at most: the kernel dealt by block face leaves one pair per block, the row-wise one a
// pair per 256 cells (two per 8^3 block, a quarter per 4^3 block)
int step_fast_forward_pairs(const StepArgs &a) {
    if (fwd_rows_supports(a)) return fwd_rows_pairs(a);
    return (a.M / a.block_size) * (a.N / a.block_size) * (a.K / a.block_size) * step_fast_forward_parts(a.block_size);
}
int step_fast_forward_pair_count(const StepArgs &a) {
    return fwd_rows_supports(a) ? 256 : step_fast_forward_part_count(a.block_size);
}
int step_fast_backward_parts(int block_size) { return block_size == 8 ? 2 : 1; }
int step_fast_backward_pairs(const StepArgs &a) {
    if (bwd_rows_supports(a)) return bwd_rows_pairs(a);
    return step_fast_cross_pairs(a);
}
int step_fast_cross_pairs(const StepArgs &a) {
    if (cross_rows_supports(a)) return cross_rows_pairs(a);
    return (a.M / a.block_size) * (a.N / a.block_size) * (a.K / a.block_size);
}

bool step_fast_supports(const StepArgs &a, bool backward) {
    if (a.dtype != GRIDNET_F32) return false;
    if (a.normalize && a.ln.gamma) return false;  // the folded LayerNorm: plain step only
    if (a.block_size != 4 && a.block_size != 8) return false;
    if (backward) {
        const bool ln = a.ln.gamma != nullptr;
        const size_t lds = a.block_size == 8
                               ? bwd_lds_bytes<8, kBwdCpt8, kBwdSlots8>(a.inner, ln, a.normalize)
                               : bwd_lds_bytes<4, kBwdCpt4, kBwdSlots4>(a.inner, ln, a.normalize);
        if (lds > kMaxLds) return false;
    }
    return true;
}

size_t step_fast_backward_workspace(const StepArgs &a) {
    // D = sum_i delta_i of every cell, handed from step_bwd_fast to step_bwd_cross; with
    // normalize, two more numbers per (element, block)
    const size_t nblk = (size_t)(a.M / a.block_size) * (a.N / a.block_size) * (a.K / a.block_size);
    return ((size_t)a.B * a.M * a.N * a.K + (a.normalize ? (size_t)a.B * nblk * 2 : 0)) * sizeof(float);
}

size_t step_fast_slab_bytes(const StepArgs &a) {
    if (bwd_rows_supports(a)) return bwd_rows_slab_bytes(a);
    // the most chunks any plan of the backward kernels makes: resident workgroups (two per CU with
    // 8^3 blocks, bounded by 16 with 4^3) over the blocks, and never more than the batch gives
    const long nblk = (long)(a.M / a.block_size) * (a.N / a.block_size) * (a.K / a.block_size);
    if (nblk >= device_cus()) return 0;  // one workgroup owns the whole batch of its block
    const int nslot = a.block_size == 8 ? kBwdSlots8 : kBwdSlots4;
    long chunks = (long)(a.block_size == 8 ? 2 : 16) * device_cus() / nblk;
    const long most = (a.B + nslot - 1) / nslot;
    if (chunks > most) chunks = most;
    if (chunks < 2) return 0;
    return (size_t)chunks * kStepSlabPlanes * a.M * a.N * a.K * sizeof(float);
}

int step_forward_fast(const StepArgs &a, hipStream_t st) {
    if (fwd_rows_supports(a)) return fwd_rows_launch(a, st);  // one inner iteration: a plain stencil, by whole rows
    return dispatch<false>(a, st);
}
int step_backward_fast(const StepArgs &a, hipStream_t st) {
    if (bwd_rows_supports(a)) return bwd_rows_launch(a, st);  // one inner iteration: by whole rows
    return dispatch<true>(a, st);
}

}  // namespace gridnet
