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
    static constexpr int NLOAD = (NWIN + TPS - 1) / TPS;  // window entries fetched per thread
    static constexpr int MID = 4 * S - 4;         // halo entries of a middle plane
    static constexpr int NH = 2 * S * S + BS * MID;  // halo entries of a window
    static constexpr int NPAIR = 9;               // (source, weight) pairs per halo entry
    static_assert(BS % CPT == 0, "cells per thread must divide the block side");
};

// Compact numbering of the halo: the two full planes i=0 and i=S-1, then for each middle plane
// the rows j=0 and j=S-1 and the two end cells of every other row.
template <typename TL>
__host__ __device__ __forceinline__ void halo_coords(int h, int &wi, int &wj, int &wk) {
    constexpr int S = TL::S, P = S * S;
    if (h < 2 * P) {
        wi = h < P ? 0 : S - 1;
        const int r = h < P ? h : h - P;
        wj = r / S;
        wk = r % S;
    } else {
        h -= 2 * P;
        wi = 1 + h / TL::MID;
        int r = h % TL::MID;
        if (r < 2 * S) {
            wj = r < S ? 0 : S - 1;
            wk = r < S ? r : r - S;
        } else {
            r -= 2 * S;
            wj = 1 + r / 2;
            wk = (r & 1) * (S - 1);
        }
    }
}

template <typename TL> __host__ __device__ __forceinline__ int halo_index(int wi, int wj, int wk) {
    constexpr int S = TL::S, P = S * S;
    if (wi == 0) return wj * S + wk;
    if (wi == S - 1) return P + wj * S + wk;
    const int base = 2 * P + (wi - 1) * TL::MID;
    if (wj == 0) return base + wk;
    if (wj == S - 1) return base + S + wk;
    return base + 2 * S + (wj - 1) * 2 + (wk == S - 1 ? 1 : 0);
}

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

// Fetching a window: one thread per window row (S*S rows of S entries; the first S*S threads
// of a slot take one row each, or several when the slot is small).  The bs cells of the block
// that lie in a row are contiguous and 16-byte aligned in the grid, so they come in as float4;
// the two end entries belong to the neighbouring blocks (or lie outside the grid and read as
// zero, gridnet/backend_torch.py:63).
template <typename TL> struct Fetch {
    static constexpr int S = TL::S, BS = TL::S - 2;
    static constexpr int NROW = S * S;
    static constexpr int RPT = (NROW + TL::TPS - 1) / TL::TPS;  // rows per thread
    int goff[RPT];   // grid offset (within a sample) of the row's first block cell; off-grid rows
                     // point at a valid address and are zeroed when committed
    int loff[RPT];   // LDS offset of the row's first entry, -1: no row for this thread
    bool ok[RPT];    // the row lies inside the grid
    int lo_d, hi_d;  // address deltas of the two end entries (0 when they are off-grid)
    bool lo_ok, hi_ok;
    __device__ __forceinline__ Fetch(int lane, int p0, int q0, int r0, int M, int N, int K) {
        lo_ok = r0 > 0;
        hi_ok = r0 + BS < K;
        lo_d = lo_ok ? -1 : 0;
        hi_d = hi_ok ? BS : 0;
#pragma unroll
        for (int e = 0; e < RPT; ++e) {
            const int row = lane + e * TL::TPS;
            const int wj = row % S, wi = row / S;
            const int gi = p0 + wi - 1, gj = q0 + wj - 1;
            const bool have = row < NROW;
            ok[e] = have && gi >= 0 && gi < M && gj >= 0 && gj < N;
            loff[e] = have ? wi * TL::PS + wj * TL::RS : -1;
            // rows outside the grid (and threads without a row) read row (0, 0) of the sample at
            // the block's own columns: always in bounds, also for the two end entries, because
            // lo_d / hi_d are non-zero only when columns r0-1 / r0+bs exist
            goff[e] = ok[e] ? (gi * N + gj) * K + r0 : r0;
        }
    }
    // Unconditional loads (no branches, no register initialisation in front of them).
    __device__ __forceinline__ void fetch(const float *xs, float (&v)[RPT][S]) const {
#pragma unroll
        for (int e = 0; e < RPT; ++e) {
            const float *p = xs + goff[e];
#pragma unroll
            for (int q = 0; q < BS / 4; ++q) {
                const float4 t = *reinterpret_cast<const float4 *>(p + 4 * q);
                v[e][1 + 4 * q] = t.x; v[e][2 + 4 * q] = t.y; v[e][3 + 4 * q] = t.z; v[e][4 + 4 * q] = t.w;
            }
            v[e][0] = p[lo_d];
            v[e][S - 1] = p[hi_d];
        }
    }
    // Both window copies receive every entry (the halo must be in both; the block itself is
    // overwritten by the iterations anyway).  Row starts are 8-byte aligned.
    __device__ __forceinline__ void commit(float *win, const float (&v)[RPT][S]) const {
#pragma unroll
        for (int e = 0; e < RPT; ++e)
            if (loff[e] >= 0) {
                float r[S];
#pragma unroll
                for (int q = 0; q < S; ++q) r[q] = ok[e] ? v[e][q] : 0.f;
                if (!lo_ok) r[0] = 0.f;
                if (!hi_ok) r[S - 1] = 0.f;
#pragma unroll
                for (int copy = 0; copy < 2; ++copy) {
                    float *row = win + copy * TL::WIN + loff[e];
#pragma unroll
                    for (int q = 0; q < S / 2; ++q)
                        *reinterpret_cast<float2 *>(row + 2 * q) = make_float2(r[2 * q], r[2 * q + 1]);
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
    float pre[Fetch<TL>::RPT][TL::S];
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
// history: inner slabs of TPS*2*CPT], then one table per workgroup [NH*9 weights | NH*9 offsets].
template <int BS, int CPT> __host__ __device__ constexpr int bwd_slot_floats(int inner) {
    return 4 * Tile<BS, CPT>::WIN + inner * Tile<BS, CPT>::TPS * 2 * CPT;
}
template <int BS, int CPT, int NSLOT> size_t bwd_lds_bytes(int inner) {
    using TL = Tile<BS, CPT>;
    return ((size_t)NSLOT * bwd_slot_floats<BS, CPT>(inner) + 2 * (size_t)TL::NH * TL::NPAIR) *
           sizeof(float);
}

// Pair q (0..8) of halo entry h: the block cell `src` (window coordinates) whose tap `t` reads
// that halo entry.  Every window axis either pins the source (entry on a window face: the
// adjacent layer of the block) or is free (source at -1, 0, +1 along it); the free axes consume
// the two base-3 digits of q in order, unused digits must be 1 so each pair appears once.
template <typename TL, int BS>
__device__ __forceinline__ bool halo_pair(int h, int q, int &t, int (&src)[3]) {
    int wc[3];
    halo_coords<TL>(h, wc[0], wc[1], wc[2]);
    const int d0 = q / 3, d1 = q % 3;
    int used = 0;
    bool valid = true;
#pragma unroll
    for (int ax = 0; ax < 3; ++ax) {
        if (wc[ax] == 0) {
            src[ax] = 1;
        } else if (wc[ax] == TL::S - 1) {
            src[ax] = BS;
        } else {  // a halo entry has at most two free axes
            src[ax] = wc[ax] + (used == 0 ? d0 : d1) - 1;
            ++used;
            valid = valid && src[ax] >= 1 && src[ax] <= BS;
        }
    }
    if (used < 2) valid = valid && d1 == 1;
    if (used < 1) valid = valid && d0 == 1;
    // halo entry = source + off_t  =>  tap digits = entry - source + 1
    t = (wc[0] - src[0] + 1) * 9 + (wc[1] - src[1] + 1) * 3 + (wc[2] - src[2] + 1);
    return valid;
}

// The decode of every (halo entry, pair) is the same for all workgroups and all calls: it is
// evaluated once per process into a device table, one word per pair:
// bit 31 = valid, bits 16..20 = tap, bits 0..15 = LDS offset of the source cell in a window.
__device__ int g_pair_words8[Tile<8, 1>::NH * Tile<8, 1>::NPAIR];
__device__ int g_pair_words4[Tile<4, 1>::NH * Tile<4, 1>::NPAIR];
template <int BS> __device__ __forceinline__ int *pair_words() {
    if constexpr (BS == 8) return g_pair_words8;
    else return g_pair_words4;
}
template <int BS> __global__ void build_pair_words() {
    using TL = Tile<BS, 1>;
    const int e = blockIdx.x * blockDim.x + threadIdx.x;
    if (e >= TL::NH * TL::NPAIR) return;
    int t, src[3];
    const bool valid = halo_pair<TL, BS>(e / TL::NPAIR, e % TL::NPAIR, t, src);
    pair_words<BS>()[e] = valid ? (int)(0x80000000u | (unsigned)(t << 16) |
                                        (unsigned)(src[0] * TL::PS + src[1] * TL::RS + src[2]))
                                : 0;
}
// Grid index (within a sample) of the source cell of a pair word, for a block at (p0, q0, r0).
template <typename TL>
__device__ __forceinline__ int pair_source_cell(int word, int p0, int q0, int r0, int N, int K) {
    const int off = word & 0xffff;
    const int s0 = off / TL::PS, s1 = (off % TL::PS) / TL::RS, s2 = off % TL::RS;
    return ((p0 + s0 - 1) * N + (q0 + s1 - 1)) * K + (r0 + s2 - 1);
}

__device__ __forceinline__ void commit_grad(float *p, float v, int mode) {
    if (mode == kParamStore) *p = v;
    else if (mode == kParamAddExclusive) *p += v;
    else unsafeAtomicAdd(p, v);
}

template <int BS, int CPT, int NSLOT, int ACT>
__global__ __launch_bounds__((Tile<BS, CPT>::TPS * NSLOT)) void step_bwd_fast(
    const float *__restrict__ weight, const float *__restrict__ bias,
    const float *__restrict__ scale, const float *__restrict__ x, const float *__restrict__ dy,
    float *__restrict__ dweight, float *__restrict__ dbias, float *__restrict__ dscale,
    float *__restrict__ dx, float *__restrict__ halo_out, int B, int M, int N, int K, int inner,
    int nblk, int nchunk, int chunk_len, int param_mode, int dx_accumulate) {
    using TL = Tile<BS, CPT>;
    extern __shared__ __attribute__((aligned(16))) float lds[];
    constexpr int NT = TL::TPS * NSLOT;
    constexpr int NHPT = (TL::NH + TL::TPS - 1) / TL::TPS;  // halo entries per thread
    const int slot_floats = bwd_slot_floats<BS, CPT>(inner);

    int blk, chunk;
    if (!split_block_id(blockIdx.x, nblk, nchunk, blk, chunk)) return;  // grid padding
    const Place<TL, CPT, NSLOT> pl(threadIdx.x, blk, N, K);
    const Fetch<TL> fx(pl.lane, pl.p0, pl.q0, pl.r0, M, N, K);
    float *win = lds + pl.slot * slot_floats;
    float *dwin = win + 2 * TL::WIN;
    float *hist = dwin + 2 * TL::WIN + pl.lane * CPT;  // + it*TPS*2*CPT (x_i), + TPS*CPT more (u_i)
    // per workgroup: (weight, source offset) of every pair, 8 bytes each
    float2 *tab = reinterpret_cast<float2 *>(lds + NSLOT * slot_floats);
    const long cells = (long)M * N * K;

    // ---- once per workgroup: parameters, mirrored neighbour weights, halo table ----
    // w : this cell's weights (forward recompute)
    // v : V[t][c] = W[26-t, c + off_t], what the neighbour at c + off_t multiplies cell c by
    // nw: gradient of that same neighbour weight; it is the product of this cell's x and the
    //     neighbour's delta summed over iterations and batch, so this thread owns it completely
    float w[27][CPT], v[27][CPT], nw[27][CPT], bv[CPT], rv[CPT], db[CPT], dr[CPT];
#pragma unroll
    for (int t = 0; t < 27; ++t) {
        load_cells<CPT>(weight + t * cells + pl.gc, w[t]);
        const int a = t / 9, b = (t / 3) % 3, cc = t % 3;
        const int ni = pl.i + a - 1, nj = pl.j + b - 1;
        const bool row_in = ni >= 0 && ni < BS && nj >= 0 && nj < BS;
#pragma unroll
        for (int c = 0; c < CPT; ++c) {
            const int nk = pl.kt * CPT + c + cc - 1;
            const bool in = row_in && nk >= 0 && nk < BS;
            v[t][c] = in ? weight[(26 - t) * cells + pl.gc + c + ((a - 1) * N + (b - 1)) * K + (cc - 1)]
                         : 0.f;
            nw[t][c] = 0.f;
        }
    }
    load_cells<CPT>(bias + pl.gc, bv);
    load_cells<CPT>(scale + pl.gc, rv);
#pragma unroll
    for (int c = 0; c < CPT; ++c) db[c] = dr[c] = 0.f;

    {
        constexpr int NP = TL::NH * TL::NPAIR, NE = (NP + NT - 1) / NT;
        const int *words = pair_words<BS>();
        int word[NE];
        float wt[NE];
#pragma unroll
        for (int n = 0; n < NE; ++n) {
            const int e = threadIdx.x + n * NT;
            word[n] = e < NP ? words[e] : 0;
        }
#pragma unroll
        for (int n = 0; n < NE; ++n)  // all gathers in flight together
            wt[n] = word[n] < 0 ? weight[((word[n] >> 16) & 31) * cells +
                                         pair_source_cell<TL>(word[n], pl.p0, pl.q0, pl.r0, N, K)]
                                : 0.f;
#pragma unroll
        for (int n = 0; n < NE; ++n) {
            const int e = threadIdx.x + n * NT;
            // invalid pairs read window entry 0, a halo corner of the delta window: zero
            if (e < NP) tab[e] = make_float2(wt[n], __int_as_float(word[n] & 0xffff));
        }
    }
    // the halo entries this thread serves for every batch element, and the gradients of the
    // weights whose tap reads them: x on the halo is frozen, so these need only D = sum_i delta_i
    int hoff[NHPT];
    float hw[NHPT][TL::NPAIR];
#pragma unroll
    for (int k = 0; k < NHPT; ++k) {
        const int hh = pl.lane + k * TL::TPS;
        int wi = 0, wj = 0, wk = 0;
        if (hh < TL::NH) halo_coords<TL>(hh, wi, wj, wk);
        hoff[k] = wi * TL::PS + wj * TL::RS + wk;
#pragma unroll
        for (int q = 0; q < TL::NPAIR; ++q) hw[k][q] = 0.f;
    }
    // delta windows: the halo stays zero for the whole kernel
    for (int idx = pl.lane; idx < 2 * TL::WIN; idx += TL::TPS) dwin[idx] = 0.f;
    wait_global_loads();

    const int s0 = chunk * chunk_len, s1 = min(B, s0 + chunk_len);
    float pre[Fetch<TL>::RPT][TL::S], g[CPT];
    if (s0 + pl.slot < s1) {
        fx.fetch(x + (s0 + pl.slot) * cells, pre);
        load_cells<CPT>(dy + (s0 + pl.slot) * cells + pl.gc, g);
    }
    // Per element: commit its window, barrier, [halo pass and stores of the PREVIOUS element],
    // recompute, reverse sweep, write D = sum_i delta_i into delta copy 1, commit the next
    // window.  Deferring the halo pass past the next barrier saves a barrier per element, lets
    // its dependent LDS look-ups overlap the first stencil loads of the next element, and keeps
    // the stores away from the wait on the prefetched window (loads and stores share one
    // in-order counter).
    float g_done[CPT], xh[NHPT], xh_done[NHPT];
    int done_s = -1;
    auto finish_done = [&]() {  // call only after a barrier that follows the D write
        if (done_s < 0) return;
        float *hs = halo_out + ((long)done_s * nblk + blk) * TL::NH;
#pragma unroll
        for (int k = 0; k < NHPT; ++k) {
            const int hh = pl.lane + k * TL::TPS;
            if (hh < TL::NH) {
                float2 ent[TL::NPAIR];
#pragma unroll
                for (int q = 0; q < TL::NPAIR; ++q) ent[q] = tab[hh * TL::NPAIR + q];
                float acc = 0.f;
#pragma unroll
                for (int q = 0; q < TL::NPAIR; ++q) {
                    const float d = dwin[TL::WIN + __float_as_int(ent[q].y)];
                    acc = fmaf(ent[q].x, d, acc);
                    hw[k][q] = fmaf(xh_done[k], d, hw[k][q]);
                }
                hs[hh] = acc;
            }
        }
        if (dx_accumulate) add_cells<CPT>(dx + done_s * cells + pl.gc, g_done);
        else store_cells<CPT>(dx + done_s * cells + pl.gc, g_done);
        done_s = -1;
    };
    if (s0 + pl.slot < s1) fx.commit(win, pre);
#ifdef EXP_TIMING
    long t_acc[5] = {0, 0, 0, 0, 0};
    long t_prev = clock64();
#define TICK(i) { long t_now = clock64(); t_acc[i] += t_now - t_prev; t_prev = t_now; }
#else
#define TICK(i)
#endif
    for (int sb = s0; sb < s1; sb += NSLOT) {
        const int s = sb + pl.slot;
        const bool active = s < s1;  // a slot past the end idles through the barriers
        lds_barrier();               // this element's window and the previous element's D
        TICK(0)
        finish_done();
        TICK(1)
        float gnext[CPT];
        if (s + NSLOT < s1) {
            fx.fetch(x + (s + NSLOT) * cells, pre);
            load_cells<CPT>(dy + (s + NSLOT) * cells + pl.gc, gnext);
        }
        float cur[CPT];
        if (active) {
#pragma unroll
            for (int c = 0; c < CPT; ++c) cur[c] = win[pl.own + c];
            // x on the halo (identical in both window copies, frozen for the whole element)
#pragma unroll
            for (int k = 0; k < NHPT; ++k) xh[k] = win[hoff[k]];
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

        TICK(2)
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

        TICK(3)
        // ---- cells of the neighbouring blocks need only D = sum_i delta_i (the halo is frozen);
        // D goes to delta copy 1: the last iteration (it = 0) used copy 0 and the readers of
        // copy 1 (it = 1) are past the barrier of it = 0.  The pass itself runs after the next
        // barrier (finish_done).
        if (inner == 0) lds_barrier();  // no barrier since the top: others may still read LDS
        if (active) {
#pragma unroll
            for (int c = 0; c < CPT; ++c) dwin[TL::WIN + pl.own + c] = dsum[c];
        }
        done_s = active ? s : -1;
#pragma unroll
        for (int c = 0; c < CPT; ++c) {
            g_done[c] = g[c];
            g[c] = gnext[c];
        }
#pragma unroll
        for (int k = 0; k < NHPT; ++k) xh_done[k] = xh[k];
        // the x windows are free (the reverse sweep does not read them): commit the next one
        if (s + NSLOT < s1) fx.commit(win, pre);
        TICK(4)
    }
    lds_barrier();
    finish_done();
#ifdef EXP_TIMING
    if (threadIdx.x == 0)
        for (int i = 0; i < 5; ++i) halo_out[blk * 8 + i] = (float)t_acc[i];
#endif

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
#pragma unroll
        for (int k = 0; k < NHPT; ++k)
#pragma unroll
            for (int q = 0; q < TL::NPAIR; ++q) reduce(hw[k][q]);
        if (pl.slot != 0) return;
    }
#pragma unroll
    for (int t = 0; t < 27; ++t) {
        const int a = t / 9, b = (t / 3) % 3, cc = t % 3;
        const int ni = pl.i + a - 1, nj = pl.j + b - 1;
        const bool row_in = ni >= 0 && ni < BS && nj >= 0 && nj < BS;
#pragma unroll
        for (int c = 0; c < CPT; ++c) {
            const int nk = pl.kt * CPT + c + cc - 1;
            if (row_in && nk >= 0 && nk < BS)
                commit_grad(dweight + (26 - t) * cells + pl.gc + c + ((a - 1) * N + (b - 1)) * K + (cc - 1),
                            nw[t][c], param_mode);
        }
    }
#pragma unroll
    for (int k = 0; k < NHPT; ++k) {
        const int hh = pl.lane + k * TL::TPS;
        if (hh < TL::NH) {
#pragma unroll
            for (int q = 0; q < TL::NPAIR; ++q) {
                const int word = pair_words<BS>()[hh * TL::NPAIR + q];
                if (word < 0)
                    commit_grad(dweight + ((word >> 16) & 31) * cells +
                                    pair_source_cell<TL>(word, pl.p0, pl.q0, pl.r0, N, K),
                                hw[k][q], param_mode);
            }
        }
    }
#pragma unroll
    for (int c = 0; c < CPT; ++c) {
        commit_grad(dbias + pl.gc + c, db[c], param_mode);
        commit_grad(dscale + pl.gc + c, dr[c], param_mode);
    }
}

// dx[cell] += the halo contributions of the (up to 7) neighbouring blocks whose window contains
// the cell, added in a fixed order.  One thread owns one K-row of one block (bs cells): whether
// a neighbour in i or j reaches the row is decided once per row, and those contributions are
// bs consecutive floats of the neighbour's compacted halo; only the two end cells of the row
// also see neighbours in k.  blockIdx.y = sample.
template <int BS>
__global__ __launch_bounds__(256) void halo_gather(const float *__restrict__ halo,
                                                   float *__restrict__ dx, int M, int N, int K,
                                                   int nblk, int rows_per_sample) {
    using TL = Tile<BS, 1>;
    const int row = blockIdx.x * blockDim.x + threadIdx.x;  // (gi, gj, bk), bk fastest
    if (row >= rows_per_sample) return;
    const int kb = K / BS, nb = N / BS, mb = M / BS;
    const int bk = row % kb;
    const int gj = (row / kb) % N;
    const int gi = row / (kb * N);
    const int li = gi % BS, lj = gj % BS, bi = gi / BS, bj = gj / BS;
    const int di_lo = (li == 0 && bi > 0) ? -1 : 0, di_hi = (li == BS - 1 && bi < mb - 1) ? 1 : 0;
    const int dj_lo = (lj == 0 && bj > 0) ? -1 : 0, dj_hi = (lj == BS - 1 && bj < nb - 1) ? 1 : 0;
    const float *hs = halo + (size_t)blockIdx.y * nblk * TL::NH;
    float acc[BS];
#pragma unroll
    for (int c = 0; c < BS; ++c) acc[c] = 0.f;
    for (int di = di_lo; di <= di_hi; ++di)
        for (int dj = dj_lo; dj <= dj_hi; ++dj) {
            const int wi = li + 1 - di * BS, wj = lj + 1 - dj * BS;  // row in the neighbour's window
            const int other = ((bi + di) * nb + (bj + dj)) * kb + bk;
            if (di != 0 || dj != 0) {  // the neighbour's halo holds the whole row, contiguously
                const float *src = hs + (size_t)other * TL::NH + halo_index<TL>(wi, wj, 1);
#pragma unroll
                for (int c = 0; c < BS; ++c) acc[c] += src[c];
            }
            // neighbours one block further along k reach only the row's end cells
            if (bk > 0) acc[0] += hs[(size_t)(other - 1) * TL::NH + halo_index<TL>(wi, wj, BS + 1)];
            if (bk < kb - 1) acc[BS - 1] += hs[(size_t)(other + 1) * TL::NH + halo_index<TL>(wi, wj, 0)];
        }
    float *out = dx + ((size_t)blockIdx.y * M * N + (size_t)gi * N + gj) * K + bk * BS;
#pragma unroll
    for (int q = 0; q < BS / 4; ++q) {
        float4 o = *reinterpret_cast<float4 *>(out + 4 * q);
        o.x += acc[4 * q]; o.y += acc[4 * q + 1]; o.z += acc[4 * q + 2]; o.w += acc[4 * q + 3];
        *reinterpret_cast<float4 *>(out + 4 * q) = o;
    }
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
    {   // the pair table of this block size, once per device (idempotent, stream-ordered)
        static bool built[64] = {false};
        int dev = 0;
        if (hipGetDevice(&dev) != hipSuccess) dev = -1;
        if (dev >= 0 && dev < 64 && !built[dev]) {
            constexpr int NP = Tile<BS, 1>::NH * Tile<BS, 1>::NPAIR;
            hipLaunchKernelGGL((build_pair_words<BS>), dim3((NP + 255) / 256), dim3(256), 0, st);
            if (int rc = check_launch("build_pair_words")) return rc;
            built[dev] = true;
        }
    }
    hipLaunchKernelGGL(kern, dim3(padded_grid(p.nblk, p.nchunk)), dim3(TL::TPS * NSLOT), lds, st,
                       (const float *)a.weight, (const float *)a.bias, (const float *)a.scale,
                       (const float *)a.x, (const float *)a.dy, (float *)a.dweight, (float *)a.dbias,
                       (float *)a.dscale, (float *)a.dx, (float *)a.workspace, a.B, a.M, a.N, a.K,
                       a.inner, p.nblk, p.nchunk, p.chunk_len, param_mode, dx_accumulate);
    if (int rc = check_launch("step_bwd_fast")) return rc;
    if (nblk > 1) {
        const int rows = a.M * a.N * (a.K / BS);
        hipLaunchKernelGGL((halo_gather<BS>), dim3((rows + 255) / 256, a.B), dim3(256), 0, st,
                           (const float *)a.workspace, (float *)a.dx, a.M, a.N, a.K, nblk, rows);
        if (int rc = check_launch("halo_gather")) return rc;
    }
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
    const int bs = a.block_size;
    const size_t nblk = (size_t)(a.M / bs) * (a.N / bs) * (a.K / bs);
    const size_t nh = bs == 8 ? Tile<8, 1>::NH : Tile<4, 1>::NH;
    return (size_t)a.B * nblk * nh * sizeof(float);
}

int step_forward_fast(const StepArgs &a, hipStream_t st) { return dispatch<false>(a, st); }
int step_backward_fast(const StepArgs &a, hipStream_t st) { return dispatch<true>(a, st); }

}  // namespace gridnet
