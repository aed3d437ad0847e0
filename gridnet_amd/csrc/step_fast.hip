// Tuned fp32 kernels for the block-local update with normalize=false (every configuration the
// reference's training scripts use: gridnet/scripts/train_mnist.py:51, train_imagenet.py:50).
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
//     (the x window is not re-read in the reverse sweep).  Weights whose tap reads a halo entry
//     see a frozen x there: their gradient is x_halo * sum_i delta_i, one pass per batch element;
//   * cells of neighbouring blocks (the window's halo) receive sum_t W[t,c'] * delta_i[c'] summed
//     over i; W does not depend on i, so one pass per batch element over D = sum_i delta_i
//     suffices.  It runs in gather form from a small LDS table (<= 9 (source, weight) pairs per
//     halo entry, built once per workgroup) and is written, compacted, to a scratch buffer;
//   * a second kernel adds each cell's <= 7 halo contributions from its neighbouring blocks to dx
//     in a fixed order.
// Parameter gradients leave the kernel once per workgroup: reduced across slots through LDS and,
// when one workgroup owns the whole batch of its block, written with plain stores.  Results are
// bitwise reproducible in that case.

#include "common.h"
#include "launch.h"

namespace gridnet {

namespace {

template <int BS, int CPT> struct Tile {
    static constexpr int S = BS + 2;              // window side
    static constexpr int KT = BS / CPT;           // threads along a K-row
    static constexpr int TPS = BS * BS * KT;      // threads per slot
    static constexpr int RS = (S + 3) / 4 * 4;    // LDS row stride (floats)
    static constexpr int PS = S * RS;             // LDS plane stride
    static constexpr int WIN = S * PS;            // floats per window copy
    static constexpr int NWIN = S * S * S;        // window entries
    static_assert(BS % CPT == 0, "cells per thread must divide the block side");
};

// Workgroup barrier that orders LDS traffic only.  __syncthreads() also waits for every global
// load in flight, which would stall each inner iteration on the prefetch of the next batch
// element; global memory needs no ordering inside these kernels.
__device__ __forceinline__ void lds_barrier() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

// Wait for every global load issued so far (s_waitcnt vmcnt(0) only).  Placed once after the
// per-workgroup parameter loads: with those known complete, the waits the compiler inserts
// inside the batch loop no longer cover the prefetch of the next batch element as well.
__device__ __forceinline__ void wait_global_loads() {
    __builtin_amdgcn_sched_barrier(0);   // keep the loads above and the loop below where they are
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt = 0, expcnt = 7, lgkmcnt = 15 (gfx9 encoding)
    __builtin_amdgcn_sched_barrier(0);
}

// Read CPT+2 consecutive floats starting at an address that is CPT-float aligned.
template <int CPT> __device__ __forceinline__ void load_row(const float *p, float (&v)[CPT + 2]);
template <> __device__ __forceinline__ void load_row<1>(const float *p, float (&v)[3]) {
    v[0] = p[0]; v[1] = p[1]; v[2] = p[2];
}
template <> __device__ __forceinline__ void load_row<2>(const float *p, float (&v)[4]) {
    const float2 a = *reinterpret_cast<const float2 *>(p);
    const float2 b = *reinterpret_cast<const float2 *>(p + 2);
    v[0] = a.x; v[1] = a.y; v[2] = b.x; v[3] = b.y;
}
template <> __device__ __forceinline__ void load_row<4>(const float *p, float (&v)[6]) {
    const float4 a = *reinterpret_cast<const float4 *>(p);
    const float2 b = *reinterpret_cast<const float2 *>(p + 4);
    v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y;
}
template <> __device__ __forceinline__ void load_row<8>(const float *p, float (&v)[10]) {
    const float4 a = *reinterpret_cast<const float4 *>(p);
    const float4 b = *reinterpret_cast<const float4 *>(p + 4);
    const float2 c = *reinterpret_cast<const float2 *>(p + 8);
    v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
    v[8] = c.x; v[9] = c.y;
}

template <int CPT> __device__ __forceinline__ void load_cells(const float *p, float (&v)[CPT]) {
    if constexpr (CPT == 1) {
        v[0] = p[0];
    } else if constexpr (CPT == 2) {
        const float2 a = *reinterpret_cast<const float2 *>(p);
        v[0] = a.x; v[1] = a.y;
    } else {
#pragma unroll
        for (int q = 0; q < CPT / 4; ++q) {
            const float4 a = *reinterpret_cast<const float4 *>(p + 4 * q);
            v[4 * q] = a.x; v[4 * q + 1] = a.y; v[4 * q + 2] = a.z; v[4 * q + 3] = a.w;
        }
    }
}

template <int CPT> __device__ __forceinline__ void store_cells(float *p, const float (&v)[CPT]) {
    if constexpr (CPT == 1) {
        p[0] = v[0];
    } else if constexpr (CPT == 2) {
        *reinterpret_cast<float2 *>(p) = make_float2(v[0], v[1]);
    } else {
#pragma unroll
        for (int q = 0; q < CPT / 4; ++q)
            *reinterpret_cast<float4 *>(p + 4 * q) =
                make_float4(v[4 * q], v[4 * q + 1], v[4 * q + 2], v[4 * q + 3]);
    }
}

template <int CPT> __device__ __forceinline__ void add_cells(float *p, const float (&v)[CPT]) {
    float old[CPT];
    load_cells<CPT>(p, old);
#pragma unroll
    for (int c = 0; c < CPT; ++c) old[c] += v[c];
    store_cells<CPT>(p, old);
}

// Where a thread sits: its slot, its cells, and the LDS offsets it uses every iteration.
template <typename TL, int CPT, int NSLOT> struct Place {
    int slot, lane;
    int i, j, kt;         // cell row (i, j) and K-segment within the block
    int p0, q0, r0;       // block origin in the grid
    int gc;               // grid index (within a sample) of the first owned cell
    int row00;            // LDS offset of window row (i, j) at column kt*CPT (tap a = b = 0)
    int own;              // LDS offset of the first owned cell
    __device__ __forceinline__ Place(int tid, int blk, int N, int K) {
        constexpr int bs = TL::S - 2;
        slot = NSLOT == 1 ? 0 : tid / TL::TPS;
        lane = tid - slot * TL::TPS;
        // kt fastest, then i, then j: the lanes an LDS access serves together then differ in
        // the plane index, and the plane stride (S*RS = 120 or 48 floats) spreads them over banks
        kt = lane % TL::KT;
        i = (lane / TL::KT) % bs;
        j = lane / (TL::KT * bs);
        const int kb = K / bs, nb = N / bs;
        p0 = (blk / (kb * nb)) * bs;
        q0 = ((blk / kb) % nb) * bs;
        r0 = (blk % kb) * bs;
        gc = ((p0 + i) * N + (q0 + j)) * K + (r0 + kt * CPT);
        row00 = i * TL::PS + j * TL::RS + kt * CPT;
        own = row00 + TL::PS + TL::RS + 1;
    }
};

// Fetching a window: one thread per HALF window row (2*S*S half rows of S/2 entries; the first
// threads of a slot take one each, or several when the slot is small).  A half row is one end
// entry plus bs/2 cells of the block; the cells are contiguous and 16-byte (bs=8) or 8-byte
// (bs=4) aligned in the grid and come in as one vector.  End entries belong to the
// neighbouring blocks, or lie outside the grid and read as zero (gridnet/backend_torch.py:63).
template <typename TL> struct Fetch {
    static constexpr int S = TL::S, BS = TL::S - 2, HL = S / 2, HC = BS / 2;
    static constexpr int NHALF = 2 * S * S;
    static constexpr int RPT = (NHALF + TL::TPS - 1) / TL::TPS;  // half rows per thread
    int goff[RPT];   // grid offset (within a sample) of the half row's first block cell; rows
                     // outside the grid point at a valid address and are zeroed when committed
    int loff[RPT];   // LDS offset of the half row's first entry, -1: none for this thread
    int edge[RPT];   // address delta of the end entry relative to goff (0 when it is off-grid)
    bool ok[RPT];    // the row lies inside the grid
    bool edge_ok[RPT];
    bool hi[RPT];    // second half: [cells..., end entry] instead of [end entry, cells...]
    __device__ __forceinline__ Fetch(int lane, int p0, int q0, int r0, int M, int N, int K) {
#pragma unroll
        for (int e = 0; e < RPT; ++e) {
            const int id = lane + e * TL::TPS;
            const int half = id & 1, row = id >> 1;
            const int wj = row % S, wi = row / S;
            const int gi = p0 + wi - 1, gj = q0 + wj - 1;
            const bool have = id < NHALF;
            hi[e] = half != 0;
            ok[e] = have && gi >= 0 && gi < M && gj >= 0 && gj < N;
            edge_ok[e] = half ? (r0 + BS < K) : (r0 > 0);
            edge[e] = edge_ok[e] ? (half ? HC : -1) : 0;
            loff[e] = have ? wi * TL::PS + wj * TL::RS + half * HL : -1;
            // rows outside the grid (and threads without a row) read row (0, 0) of the sample at
            // the block's own columns: in bounds, also for the end entry, whose delta is
            // non-zero only when that column exists
            goff[e] = (ok[e] ? (gi * N + gj) * K : 0) + r0 + half * HC;
        }
    }
    // Unconditional loads (no branches, no register initialisation in front of them).
    __device__ __forceinline__ void fetch(const float *xs, float (&v)[RPT][HL]) const {
#pragma unroll
        for (int e = 0; e < RPT; ++e) {
            const float *p = xs + goff[e];
            float c[HC];
            load_cells<HC>(p, c);
            const float end = p[edge[e]];
            // lay the values out in window order for either half
#pragma unroll
            for (int q = 0; q < HC; ++q) v[e][q] = c[q];
            v[e][HC] = end;
        }
    }
    // Both window copies receive every entry (the halo must be in both; the block itself is
    // overwritten by the iterations anyway).
    template <int COPIES = 2>
    __device__ __forceinline__ void commit(float *win, const float (&v)[RPT][HL]) const {
#pragma unroll
        for (int e = 0; e < RPT; ++e)
            if (loff[e] >= 0) {
                const float end = (ok[e] && edge_ok[e]) ? v[e][HC] : 0.f;
#pragma unroll
                for (int copy = 0; copy < COPIES; ++copy) {
                    float *row = win + copy * TL::WIN + loff[e];
                    // first half: [end, cells...]; second half: [cells..., end]
                    row[hi[e] ? HC : 0] = end;
#pragma unroll
                    for (int q = 0; q < HC; ++q) row[q + (hi[e] ? 0 : 1)] = ok[e] ? v[e][q] : 0.f;
                }
            }
    }
};

// Visit the 9 neighbour rows of a thread in tap order with the LDS reads running DEPTH rows
// ahead of the arithmetic: row r + DEPTH is requested before row r is consumed, and scheduling
// barriers keep the compiler from collapsing that order when registers are tight (it otherwise
// falls back to load, wait, 12 FMAs, load, ... and every row pays the full LDS latency).
template <typename TL, int CPT, int DEPTH, typename F>
__device__ __forceinline__ void for_each_row(const float *rows, F &&consume) {
    float buf[DEPTH][CPT + 2];
#pragma unroll
    for (int r = 0; r < DEPTH && r < 9; ++r)
        load_row<CPT>(rows + (r / 3) * TL::PS + (r % 3) * TL::RS, buf[r]);
#pragma unroll
    for (int r = 0; r < 9; ++r) {
        __builtin_amdgcn_sched_barrier(0);
        consume(r, buf[r % DEPTH]);
        if (r + DEPTH < 9) {
            __builtin_amdgcn_sched_barrier(0);
            load_row<CPT>(rows + ((r + DEPTH) / 3) * TL::PS + ((r + DEPTH) % 3) * TL::RS, buf[r % DEPTH]);
        }
    }
    __builtin_amdgcn_sched_barrier(0);
}

// u[c] = init[c] + sum over the 27 taps of w[t][c] * window value, taps in raster order.
template <typename TL, int CPT, int DEPTH = 9>
__device__ __forceinline__ void stencil(const float *win, int row00, const float (&w)[27][CPT],
                                        const float (&init)[CPT], float (&u)[CPT]) {
#pragma unroll
    for (int c = 0; c < CPT; ++c) u[c] = init[c];
    if constexpr (DEPTH >= 9) {  // all rows requested up front; the compiler orders the rest
#pragma unroll
        for (int a = 0; a < 3; ++a)
#pragma unroll
            for (int b = 0; b < 3; ++b) {
                float v[CPT + 2];
                load_row<CPT>(win + row00 + a * TL::PS + b * TL::RS, v);
#pragma unroll
                for (int cc = 0; cc < 3; ++cc)
#pragma unroll
                    for (int c = 0; c < CPT; ++c)
                        u[c] = fmaf(w[a * 9 + b * 3 + cc][c], v[c + cc], u[c]);
            }
    } else {
        for_each_row<TL, CPT, DEPTH>(win + row00, [&](int r, const float (&v)[CPT + 2]) {
#pragma unroll
            for (int cc = 0; cc < 3; ++cc)
#pragma unroll
                for (int c = 0; c < CPT; ++c) u[c] = fmaf(w[r * 3 + cc][c], v[c + cc], u[c]);
        });
    }
}

constexpr int kFwdDepth = 9;  // neighbour rows requested ahead of the arithmetic

template <int BS, int CPT, int NSLOT, int ACT>
__global__ __launch_bounds__((Tile<BS, CPT>::TPS * NSLOT)) void step_fwd_fast(
    const float *__restrict__ weight, const float *__restrict__ bias,
    const float *__restrict__ scale, const float *__restrict__ x, float *__restrict__ y, int B, int M,
    int N, int K, int inner, int nblk, int nchunk, int chunk_len) {
    using TL = Tile<BS, CPT>;
    __shared__ __attribute__((aligned(16))) float lds[NSLOT * 2 * TL::WIN];

    int blk, chunk;
    if (!split_block_id(blockIdx.x, nblk, nchunk, blk, chunk)) return;  // grid padding
    const Place<TL, CPT, NSLOT> pl(threadIdx.x, blk, N, K);
    const Fetch<TL> fx(pl.lane, pl.p0, pl.q0, pl.r0, M, N, K);
    float *win = lds + pl.slot * (2 * TL::WIN);
    const long cells = (long)M * N * K;

    float w[27][CPT], bv[CPT], rv[CPT];
#pragma unroll
    for (int t = 0; t < 27; ++t) load_cells<CPT>(weight + t * cells + pl.gc, w[t]);
    load_cells<CPT>(bias + pl.gc, bv);
    load_cells<CPT>(scale + pl.gc, rv);
    wait_global_loads();

    const int s0 = chunk * chunk_len, s1 = min(B, s0 + chunk_len);
    float pre[Fetch<TL>::RPT][Fetch<TL>::HL];
    if (s0 + pl.slot < s1) fx.fetch(x + (s0 + pl.slot) * cells, pre);
    // The result of an element is stored one element late, after the next window has been
    // committed: the wait for the prefetched window would otherwise also wait for a store that
    // was issued an instant earlier (loads and stores share one in-order counter).
    float done[CPT];
    int done_s = -1;
    for (int sb = s0; sb < s1; sb += NSLOT) {
        const int s = sb + pl.slot;
        const bool active = s < s1;  // a slot past the end idles through the barriers
        if (active) fx.commit(win, pre);
        lds_barrier();
        if (done_s >= 0) store_cells<CPT>(y + done_s * cells + pl.gc, done);
        if (s + NSLOT < s1) fx.fetch(x + (s + NSLOT) * cells, pre);  // next element, in flight
        float cur[CPT];
        if (active) {
#pragma unroll
            for (int c = 0; c < CPT; ++c) cur[c] = win[pl.own + c];
        }
        for (int it = 0; it < inner; ++it) {
            if (active) {
                float u[CPT];
                stencil<TL, CPT, kFwdDepth>(win + (it & 1) * TL::WIN, pl.row00, w, bv, u);
#pragma unroll
                for (int c = 0; c < CPT; ++c) {
                    cur[c] = fmaf(rv[c], Act<ACT, float>::f(u[c]), cur[c]);
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

// ---- backward ------------------------------------------------------------------------------
constexpr int kBwdDepth = 4;  // neighbour rows requested ahead of the arithmetic

// LDS layout of the backward kernel (floats): per slot [x window x2 | delta window x2 |
// history: inner slabs of TPS*2*CPT].
template <int BS, int CPT> __host__ __device__ constexpr int bwd_slot_floats(int inner) {
    return 4 * Tile<BS, CPT>::WIN + inner * Tile<BS, CPT>::TPS * 2 * CPT;
}
template <int BS, int CPT, int NSLOT> size_t bwd_lds_bytes(int inner) {
    return (size_t)NSLOT * bwd_slot_floats<BS, CPT>(inner) * sizeof(float);
}

// Commit R x C gradient values to base[index(r, c)] for the entries with ok(r, c).  One code path
// per mode (the mode is uniform).  In the add-in-place mode the accumulators were STARTED from
// the old contents (see the kernels' set-up), so that mode stores like the overwrite mode: an
// old value fetched at the end instead would put a serial trip to memory at the tail of every
// workgroup, where nothing is left to hide it.
template <int R, int C, typename Index, typename Ok>
__device__ __forceinline__ void commit_grads(float *base, const float (&val)[R][C], int mode,
                                             Index &&index, Ok &&ok) {
    if (mode != kParamAtomic) {
#pragma unroll
        for (int r = 0; r < R; ++r)
#pragma unroll
            for (int c = 0; c < C; ++c)
                if (ok(r, c)) base[index(r, c)] = val[r][c];
    } else {
#pragma unroll
        for (int r = 0; r < R; ++r)
#pragma unroll
            for (int c = 0; c < C; ++c)
                if (ok(r, c)) unsafeAtomicAdd(base + index(r, c), val[r][c]);
    }
}

template <int BS, int CPT, int NSLOT, int ACT>
__global__ __launch_bounds__((Tile<BS, CPT>::TPS * NSLOT)) __attribute__((amdgpu_waves_per_eu(2)))
void step_bwd_fast(
    const float *__restrict__ weight, const float *__restrict__ bias,
    const float *__restrict__ scale, const float *__restrict__ x, const float *__restrict__ dy,
    float *__restrict__ dweight, float *__restrict__ dbias, float *__restrict__ dscale,
    float *__restrict__ dx, float *__restrict__ dsum_out, int B, int M, int N, int K, int inner,
    int nblk, int nchunk, int chunk_len, int param_mode, int dx_accumulate) {
    using TL = Tile<BS, CPT>;
    extern __shared__ __attribute__((aligned(16))) float lds[];
    const int slot_floats = bwd_slot_floats<BS, CPT>(inner);

    int blk, chunk;
    if (!split_block_id(blockIdx.x, nblk, nchunk, blk, chunk)) return;  // grid padding
    const Place<TL, CPT, NSLOT> pl(threadIdx.x, blk, N, K);
    const Fetch<TL> fx(pl.lane, pl.p0, pl.q0, pl.r0, M, N, K);
    float *win = lds + pl.slot * slot_floats;
    float *dwin = win + 2 * TL::WIN;
    float *hist = dwin + 2 * TL::WIN + pl.lane * CPT;  // + it*TPS*2*CPT (x_i), + TPS*CPT more (u_i)
    const long cells = (long)M * N * K;

    // nw[t][c] belongs to the weight of the neighbour at c + off_t, where that lies in this block
    auto in_block = [&](int t, int c) {
        const int ni = pl.i + t / 9 - 1, nj = pl.j + (t / 3) % 3 - 1, nk = pl.kt * CPT + c + t % 3 - 1;
        return ni >= 0 && ni < BS && nj >= 0 && nj < BS && nk >= 0 && nk < BS;
    };
    auto neighbour_weight = [&](int t, int c) {
        return (26 - t) * cells + pl.gc + c + ((t / 9 - 1) * N + ((t / 3) % 3 - 1)) * K + (t % 3 - 1);
    };

    // ---- once per workgroup: parameters and mirrored neighbour weights ----
    // w : this cell's weights (forward recompute)
    // v : V[t][c] = W[26-t, c + off_t], what the neighbour at c + off_t multiplies cell c by
    // nw: gradient of that same neighbour weight; it is the product of this cell's x and the
    //     neighbour's delta summed over iterations and batch, so this thread owns it completely
    float w[27][CPT], v[27][CPT], nw[27][CPT], bv[CPT], rv[CPT], db[CPT], dr[CPT];
#pragma unroll
    for (int t = 0; t < 27; ++t) {
        load_cells<CPT>(weight + t * cells + pl.gc, w[t]);
#pragma unroll
        for (int c = 0; c < CPT; ++c) {
            v[t][c] = in_block(t, c) ? weight[neighbour_weight(t, c)] : 0.f;
            nw[t][c] = 0.f;
        }
    }
    load_cells<CPT>(bias + pl.gc, bv);
    load_cells<CPT>(scale + pl.gc, rv);
#pragma unroll
    for (int c = 0; c < CPT; ++c) db[c] = dr[c] = 0.f;

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
            for (int c = 0; c < CPT; ++c)
                if (in_block(t, c)) nw[t][c] = dweight[neighbour_weight(t, c)];
#pragma unroll
        for (int c = 0; c < CPT; ++c) {
            db[c] = dbias[pl.gc + c];
            dr[c] = dscale[pl.gc + c];
        }
    }

    const int s0 = chunk * chunk_len, s1 = min(B, s0 + chunk_len);
    float pre[Fetch<TL>::RPT][Fetch<TL>::HL], g[CPT];
    if (s0 + pl.slot < s1) {
        fx.fetch(x + (s0 + pl.slot) * cells, pre);
        load_cells<CPT>(dy + (s0 + pl.slot) * cells + pl.gc, g);
    }
    // Per element: commit its window, barrier, [stores of the PREVIOUS element], recompute,
    // reverse sweep, commit the next window.  The stores are issued one element late, away from
    // the wait on the prefetched window (loads and stores share one in-order counter).  Besides
    // the gradient of its own cells a thread leaves D = sum_i delta_i of them: what the cells
    // of neighbouring blocks and the weights of taps that read the frozen halo receive depends
    // on the iterations only through D, and a second kernel (step_bwd_cross) works it out.
    float g_done[CPT], d_done[CPT];
    int done_s = -1;
    auto finish_done = [&]() {
        if (done_s < 0) return;
        const long o = (long)done_s * cells + pl.gc;
        store_cells<CPT>(dsum_out + o, d_done);
        if (dx_accumulate) add_cells<CPT>(dx + o, g_done);
        else store_cells<CPT>(dx + o, g_done);
        done_s = -1;
    };
    if (s0 + pl.slot < s1) fx.commit(win, pre);
    for (int sb = s0; sb < s1; sb += NSLOT) {
        const int s = sb + pl.slot;
        const bool active = s < s1;  // a slot past the end idles through the barriers
        lds_barrier();               // this element's window
        finish_done();
        float gnext[CPT];
        if (s + NSLOT < s1) {
            fx.fetch(x + (s + NSLOT) * cells, pre);
            load_cells<CPT>(dy + (s + NSLOT) * cells + pl.gc, gnext);
        }
        float cur[CPT];
        if (active) {
#pragma unroll
            for (int c = 0; c < CPT; ++c) cur[c] = win[pl.own + c];
        }

        // ---- forward recompute, remembering x_i and u_i of the owned cells ----
        for (int it = 0; it < inner; ++it) {
            if (active) {
                float u[CPT];
                stencil<TL, CPT, kBwdDepth>(win + (it & 1) * TL::WIN, pl.row00, w, bv, u);
                float *h = hist + it * (TL::TPS * 2 * CPT);
                store_cells<CPT>(h, cur);
                store_cells<CPT>(h + TL::TPS * CPT, u);
                if (it + 1 < inner) {  // x_inner itself is never needed
#pragma unroll
                    for (int c = 0; c < CPT; ++c) {
                        cur[c] = fmaf(rv[c], Act<ACT, float>::f(u[c]), cur[c]);
                        win[((it + 1) & 1) * TL::WIN + pl.own + c] = cur[c];
                    }
                }
            }
            if (it + 1 < inner) lds_barrier();
        }

        // ---- reverse sweep: delta window copy (it & 1) holds delta_it ----
        float dsum[CPT], xi[CPT];
#pragma unroll
        for (int c = 0; c < CPT; ++c) dsum[c] = 0.f;
        for (int it = inner - 1; it >= 0; --it) {
            if (active) {
                const float *h = hist + it * (TL::TPS * 2 * CPT);
                float u[CPT];
                load_cells<CPT>(h, xi);
                load_cells<CPT>(h + TL::TPS * CPT, u);
#pragma unroll
                for (int c = 0; c < CPT; ++c) {
                    float f, d;
                    Act<ACT, float>::fd(u[c], f, d);
                    const float delta = d * g[c] * rv[c];
                    dr[c] = fmaf(f, g[c], dr[c]);
                    db[c] += delta;
                    dsum[c] += delta;
                    dwin[(it & 1) * TL::WIN + pl.own + c] = delta;
                }
            }
            lds_barrier();
            if (active) {
                const float *dwn = dwin + (it & 1) * TL::WIN + pl.row00;
                for_each_row<TL, CPT, kBwdDepth>(dwn, [&](int r, const float (&dv)[CPT + 2]) {
#pragma unroll
                    for (int cc = 0; cc < 3; ++cc)
#pragma unroll
                        for (int c = 0; c < CPT; ++c) {
                            nw[r * 3 + cc][c] = fmaf(xi[c], dv[c + cc], nw[r * 3 + cc][c]);
                            g[c] = fmaf(v[r * 3 + cc][c], dv[c + cc], g[c]);
                        }
                });
            }
        }

        if (inner == 0) lds_barrier();  // no barrier since the top: others may still read LDS
        done_s = active ? s : -1;
#pragma unroll
        for (int c = 0; c < CPT; ++c) {
            g_done[c] = g[c];
            d_done[c] = dsum[c];
            g[c] = gnext[c];
        }
        // the x windows are free (the reverse sweep does not read them): commit the next one
        if (s + NSLOT < s1) fx.commit(win, pre);
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
        }
        if (pl.slot != 0) return;
    }
    commit_grads<27, CPT>(dweight, nw, param_mode, neighbour_weight, in_block);
    float one[1][CPT];
    auto own_cell = [&](int, int c) { return pl.gc + c; };
    auto always = [](int, int) { return true; };
#pragma unroll
    for (int c = 0; c < CPT; ++c) one[0][c] = db[c];
    commit_grads<1, CPT>(dbias, one, param_mode, own_cell, always);
#pragma unroll
    for (int c = 0; c < CPT; ++c) one[0][c] = dr[c];
    commit_grads<1, CPT>(dscale, one, param_mode, own_cell, always);
}

// ---- backward, second kernel: everything that crosses a block boundary ----------------------
// The window halo is frozen during the inner iterations, so both the gradient that the cells of
// NEIGHBOURING blocks receive and the gradient of a weight whose tap reads a halo entry depend
// on the iterations only through D = sum_i delta_i, which step_bwd_fast leaves in `dsum`:
//   dx[c]    += sum over taps t with c + off_t in another block of W[26-t, c + off_t] * D[c + off_t]
//   dW[t, c] += D[c] * x[c + off_t]          for the taps t whose c + off_t lies outside c's block
// Same mapping as the main kernel (a slot per (block, batch element), CPT cells per thread,
// weights and gradient accumulators in registers) with the x window and the D window of the
// element in LDS, both with their REAL halo this time: the neighbouring blocks' values, zero
// outside the grid.  One stencil-shaped pass per element; no atomics, fixed order.  Two stages
// of windows alternate, which leaves one barrier per element.
constexpr int kCrossDepth = 4;  // neighbour rows requested ahead of the arithmetic

template <int BS, int CPT, int NSLOT>
__global__ __launch_bounds__((Tile<BS, CPT>::TPS * NSLOT)) void step_bwd_cross(
    const float *__restrict__ weight, const float *__restrict__ x, const float *__restrict__ dsum,
    float *__restrict__ dweight, float *__restrict__ dx, int B, int M, int N, int K, int nblk,
    int nchunk, int chunk_len, int param_mode) {
    using TL = Tile<BS, CPT>;
    constexpr int STAGE = 2 * TL::WIN;  // [x window | D window]
    __shared__ __attribute__((aligned(16))) float lds[NSLOT * 2 * STAGE];

    int blk, chunk;
    if (!split_block_id(blockIdx.x, nblk, nchunk, blk, chunk)) return;  // grid padding
    const Place<TL, CPT, NSLOT> pl(threadIdx.x, blk, N, K);
    const Fetch<TL> fx(pl.lane, pl.p0, pl.q0, pl.r0, M, N, K);
    float *stages = lds + pl.slot * (2 * STAGE);
    const long cells = (long)M * N * K;

    auto leaves_block = [&](int t, int c) {
        const int ni = pl.i + t / 9 - 1, nj = pl.j + (t / 3) % 3 - 1, nk = pl.kt * CPT + c + t % 3 - 1;
        return !(ni >= 0 && ni < BS && nj >= 0 && nj < BS && nk >= 0 && nk < BS);
    };
    // vx: V[t][c] = W[26-t, c + off_t] where the neighbour lies in ANOTHER block of the grid
    //     (the complement of the main kernel's v); cw: gradient of this cell's own tap t.
    float vx[27][CPT], cw[27][CPT];
    bool any_cross = false;
#pragma unroll
    for (int t = 0; t < 27; ++t) {
        const int a = t / 9, b = (t / 3) % 3, cc = t % 3;
        const int ni = pl.i + a - 1, nj = pl.j + b - 1;
        const bool row_in = ni >= 0 && ni < BS && nj >= 0 && nj < BS;
        const int gi = pl.p0 + ni, gj = pl.q0 + nj;
        const bool row_grid = gi >= 0 && gi < M && gj >= 0 && gj < N;
#pragma unroll
        for (int c = 0; c < CPT; ++c) {
            const int nk = pl.kt * CPT + c + cc - 1, gk = pl.r0 + nk;
            const bool leaves = !(row_in && nk >= 0 && nk < BS);
            const bool cross = leaves && row_grid && gk >= 0 && gk < K;
            vx[t][c] = cross ? weight[(26 - t) * cells + pl.gc + c + ((a - 1) * N + (b - 1)) * K + (cc - 1)]
                             : 0.f;
            cw[t][c] = 0.f;
            any_cross = any_cross || cross;
        }
    }
    wait_global_loads();
    // add-in-place mode: slot 0's accumulators start from what the gradient buffer holds
    if (param_mode == kParamAddExclusive && pl.slot == 0) {
#pragma unroll
        for (int t = 0; t < 27; ++t)
#pragma unroll
            for (int c = 0; c < CPT; ++c)
                if (leaves_block(t, c)) cw[t][c] = dweight[t * cells + pl.gc + c];
    }

    // Windows are fetched TWO elements ahead (two register buffers, used alternately): with one
    // stencil pass per element there is too little arithmetic to cover a trip to memory.
    const int s0 = chunk * chunk_len, s1 = min(B, s0 + chunk_len);
    using Buf = float[Fetch<TL>::RPT][Fetch<TL>::HL];
    Buf ax, ad, bx, bd;
    auto fetch_into = [&](int s, Buf &px, Buf &pd) {
        if (s < s1) {
            fx.fetch(x + (long)s * cells, px);
            fx.fetch(dsum + (long)s * cells, pd);
        }
    };
    auto commit_from = [&](int s, int st, const Buf &px, const Buf &pd) {
        if (s < s1) {
            fx.template commit<1>(stages + st * STAGE, px);
            fx.template commit<1>(stages + st * STAGE + TL::WIN, pd);
        }
    };
    // One element: stage `st` holds it, `px/pd` hold the next one (in flight or arrived), the
    // other buffer pair `qx/qd` is free and receives the element after that.
    auto element = [&](int s, int st, const Buf &px, const Buf &pd, Buf &qx, Buf &qd) {
        const bool active = s < s1;
        lds_barrier();  // stage `st` is complete; every reader of the other stage is done
        float gx[CPT];  // dx of the owned cells so far (their own block's part)
        float *out = dx + (long)s * cells + pl.gc;
        if (active && any_cross) load_cells<CPT>(out, gx);  // before the prefetch: it is awaited first
        fetch_into(s + 2 * NSLOT, qx, qd);
        if (active) {
            const float *xw = stages + st * STAGE, *dw = xw + TL::WIN;
            float dc[CPT], g[CPT];
#pragma unroll
            for (int c = 0; c < CPT; ++c) {
                dc[c] = dw[pl.own + c];
                g[c] = 0.f;
            }
            for_each_row<TL, CPT, kCrossDepth>(dw + pl.row00, [&](int r, const float (&dv)[CPT + 2]) {
#pragma unroll
                for (int cc = 0; cc < 3; ++cc)
#pragma unroll
                    for (int c = 0; c < CPT; ++c) g[c] = fmaf(vx[r * 3 + cc][c], dv[c + cc], g[c]);
            });
            for_each_row<TL, CPT, kCrossDepth>(xw + pl.row00, [&](int r, const float (&xv)[CPT + 2]) {
#pragma unroll
                for (int cc = 0; cc < 3; ++cc)
#pragma unroll
                    for (int c = 0; c < CPT; ++c)
                        cw[r * 3 + cc][c] = fmaf(dc[c], xv[c + cc], cw[r * 3 + cc][c]);
            });
            if (any_cross) {
#pragma unroll
                for (int c = 0; c < CPT; ++c) gx[c] += g[c];
                store_cells<CPT>(out, gx);
            }
        }
        commit_from(s + NSLOT, st ^ 1, px, pd);
    };
    fetch_into(s0 + pl.slot, ax, ad);
    fetch_into(s0 + pl.slot + NSLOT, bx, bd);
    commit_from(s0 + pl.slot, 0, ax, ad);
    for (int sb = s0; sb < s1; sb += 2 * NSLOT) {
        element(sb + pl.slot, 0, bx, bd, ax, ad);
        element(sb + pl.slot + NSLOT, 1, ax, ad, bx, bd);  // may lie past the end: idles
    }

    if (NSLOT > 1) {
        float *red = lds;  // NSLOT * TPS floats, reused value by value
#pragma unroll
        for (int t = 0; t < 27; ++t)
#pragma unroll
            for (int c = 0; c < CPT; ++c) {
                lds_barrier();
                red[pl.slot * TL::TPS + pl.lane] = cw[t][c];
                lds_barrier();
                if (pl.slot == 0) {
#pragma unroll
                    for (int q = 1; q < NSLOT; ++q) cw[t][c] += red[q * TL::TPS + pl.lane];
                }
            }
        if (pl.slot != 0) return;
    }
    // every tap that leaves the block is committed, also where it reads the zero padding outside
    // the grid (its gradient is exactly zero and a store-mode caller expects every entry written)
    commit_grads<27, CPT>(
        dweight, cw, param_mode, [&](int t, int c) { return t * cells + pl.gc + c; },
        leaves_block);
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

template <int BS, int CPT, int NSLOT, int ACT> int launch_fwd(const StepArgs &a, hipStream_t st) {
    using TL = Tile<BS, CPT>;
    auto kern = step_fwd_fast<BS, CPT, NSLOT, ACT>;
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
                       p.chunk_len);
    return check_launch("step_fwd_fast");
}

constexpr size_t kMaxLds = 160 * 1024;

// the cross-block kernel's own shapes (it shares the main kernel's blocks and batch chunks)
constexpr int kCrossCpt8 = 2, kCrossSlots8 = 1;  // bs=8: 256 threads
constexpr int kCrossCpt4 = 1, kCrossSlots4 = 4;  // bs=4: four one-wave slots

template <int BS, int CPT, int NSLOT, int ACT> int launch_bwd(const StepArgs &a, hipStream_t st) {
    using TL = Tile<BS, CPT>;
    const long cells = (long)a.M * a.N * a.K;
    const size_t lds = bwd_lds_bytes<BS, CPT, NSLOT>(a.inner);
    auto kern = step_bwd_fast<BS, CPT, NSLOT, ACT>;
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
    const Plan p = make_plan(a, NSLOT, per_cu * device_cus(), whole);
    const bool new_params = (a.flags & GRIDNET_OVERWRITE_PARAMS) != 0;
    int param_mode = kParamAtomic;
    if (p.nchunk == 1) {
        param_mode = new_params ? kParamStore : kParamAddExclusive;
    } else if (new_params) {
        if (int rc = fill_zero((float *)a.dweight, 27 * cells, st)) return rc;
        if (int rc = fill_zero((float *)a.dbias, cells, st)) return rc;
        if (int rc = fill_zero((float *)a.dscale, cells, st)) return rc;
    }
    const int dx_accumulate = (a.flags & GRIDNET_OVERWRITE_DX) ? 0 : 1;
    hipLaunchKernelGGL(kern, dim3(padded_grid(p.nblk, p.nchunk)), dim3(TL::TPS * NSLOT), lds, st,
                       (const float *)a.weight, (const float *)a.bias, (const float *)a.scale,
                       (const float *)a.x, (const float *)a.dy, (float *)a.dweight, (float *)a.dbias,
                       (float *)a.dscale, (float *)a.dx, (float *)a.workspace, a.B, a.M, a.N, a.K,
                       a.inner, p.nblk, p.nchunk, p.chunk_len, param_mode, dx_accumulate);
    if (int rc = check_launch("step_bwd_fast")) return rc;
    // same blocks, same batch chunks, same way of committing parameter gradients (the two
    // kernels write disjoint entries of dweight)
    constexpr int XCPT = BS == 8 ? kCrossCpt8 : kCrossCpt4, XSLOT = BS == 8 ? kCrossSlots8 : kCrossSlots4;
    hipLaunchKernelGGL((step_bwd_cross<BS, XCPT, XSLOT>), dim3(padded_grid(p.nblk, p.nchunk)),
                       dim3(Tile<BS, XCPT>::TPS * XSLOT), 0, st, (const float *)a.weight,
                       (const float *)a.x, (const float *)a.workspace, (float *)a.dweight,
                       (float *)a.dx, a.B, a.M, a.N, a.K, p.nblk, p.nchunk, p.chunk_len, param_mode);
    if (int rc = check_launch("step_bwd_cross")) return rc;
    return GRIDNET_OK;
}

// ---- the tuned shapes ---------------------------------------------------------------------
constexpr int kFwdCpt8 = 4, kFwdSlots8 = 1;   // bs=8 forward: 128 threads, 4 cells each
constexpr int kBwdCpt8 = 2, kBwdSlots8 = 1;   // bs=8 backward: 256 threads, 2 cells each
constexpr int kFwdCpt4 = 2, kFwdSlots4 = 4;   // bs=4: 32-thread slots, 4 per workgroup
constexpr int kBwdCpt4 = 1, kBwdSlots4 = 2;   // bs=4 backward: one wave per slot, one cell per thread

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

bool step_fast_supports(const StepArgs &a, bool backward) {
    if (a.dtype != GRIDNET_F32 || a.normalize) return false;
    if (a.block_size != 4 && a.block_size != 8) return false;
    if (backward) {
        const size_t lds = a.block_size == 8 ? bwd_lds_bytes<8, kBwdCpt8, kBwdSlots8>(a.inner)
                                             : bwd_lds_bytes<4, kBwdCpt4, kBwdSlots4>(a.inner);
        if (lds > kMaxLds) return false;
    }
    return true;
}

size_t step_fast_backward_workspace(const StepArgs &a) {
    // D = sum_i delta_i of every cell, handed from step_bwd_fast to step_bwd_cross
    return (size_t)a.B * a.M * a.N * a.K * sizeof(float);
}

int step_forward_fast(const StepArgs &a, hipStream_t st) { return dispatch<false>(a, st); }
int step_backward_fast(const StepArgs &a, hipStream_t st) { return dispatch<true>(a, st); }

}  // namespace gridnet
