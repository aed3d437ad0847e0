// Building blocks shared by the tuned kernels (step_fast.hip, gated_fast.hip): the geometry of a
// slot and its LDS window, LDS-only barriers, wave priorities, lane reductions, vector loads and
// stores, the window fetch, and the row walk of the 27-tap stencil.  Device code only; every
// translation unit that includes this gets its own copy (internal linkage).
#ifndef GRIDNET_FAST_TILES_H
#define GRIDNET_FAST_TILES_H

#include "common.h"
#include "launch.h"

namespace gridnet {
namespace {

template <int BS, int CPT> struct Tile {
    static constexpr int S = BS + 2;              // window side
    static constexpr int KT = BS / CPT;           // threads along a K-row
    static constexpr int TPS = BS * BS * KT;      // threads per slot
    // 4^3 blocks, two cells per thread: rows are NOT padded and planes get 4 floats of padding,
    // and the lanes of a slot run over i first (see Place).  Measured on this LDS with the
    // instruction the stencil uses (two adjacent 64-bit reads in one, ds_read2_b64): 8.0 cycles
    // per wave instruction with this layout against 16.0 with rows padded to 8 floats and k
    // fastest among the lanes, and the 32-bit writes of the owned cells 2.8 against 5.5.  With
    // the padded layout the kernels for 4^3 blocks kept the LDS busy for 92 % of their time, half
    // of it in bank conflicts.
    static constexpr bool kDense = BS == 4 && CPT == 2;
    static constexpr int RS = kDense ? S : (S + 3) / 4 * 4;   // LDS row stride (floats)
    static constexpr int PS = kDense ? S * S + 4 : S * RS;    // LDS plane stride
    static constexpr int WIN = S * PS;            // floats per window copy
    static constexpr int NWIN = S * S * S;        // window entries
    static_assert(BS % CPT == 0, "cells per thread must divide the block side");
    static_assert(RS % 2 == 0 && PS % 2 == 0, "rows are read as 64-bit pairs");
};

// Workgroup barrier that orders LDS traffic only.  __syncthreads() also waits for every global
// load in flight, which would stall each inner iteration on the prefetch of the next batch
// element; global memory needs no ordering inside these kernels.
__device__ __forceinline__ void lds_barrier() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

// The barrier between the phases of ONE slot.  A slot that lives inside a single wave (32 or 64
// threads: 4^3 blocks) needs no s_barrier: the LDS serves the instructions of a wave in the order
// they were issued, so a read sees what any lane of the same wave wrote before it; only the
// compiler has to be kept from reordering.  The other slots of the workgroup are not waited for.
template <int TPS> __device__ __forceinline__ void slot_barrier() {
    if constexpr (TPS <= kWave) {
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    } else {
        lds_barrier();
    }
}

// Wave priority as a function of the element a workgroup is working on: high for two elements, low
// for the next two.  Left alone the arbiter keeps preferring the waves of the older workgroup of a
// CU, which then finishes early and leaves the CU half empty for the rest of the kernel (workgroups
// of the forward kernel ended anywhere between 46 and 68 us after the start).  With this schedule
// two workgroups that work on the same element have equal priority, and when one falls behind it
// is the one with the higher priority for part of the time: their progress stays within two
// elements.  What matters is that workgroups sharing a CU follow the SAME schedule: measured on the
// chain's backward kernel (one round of 512 workgroups, 64^3 grid, batch 32), any of the block id's
// low bits as phase gives 203 us, no priorities 215 us, and a phase taken from bit 8 of the block id
// -- opposite schedules for the two workgroups of a CU, which the dispatcher places 256 ids apart --
// 214 us; periods of 1, 4 and 8 elements give 206, 209 and 211 us.  2-3 % on the forward kernel with
// 8^3 blocks (nothing, or a loss, in the forward kernel for 4^3 blocks, which does without).
__device__ __forceinline__ void take_turns(int element) {
    if (((element >> 1) ^ blockIdx.x ^ (blockIdx.x >> 2)) & 1) __builtin_amdgcn_s_setprio(1);
    else __builtin_amdgcn_s_setprio(0);
}

// Sum over the 16 lanes of a DPP row (lanes 16q .. 16q+15), delivered to every one of them:
// four rotate-and-add steps on the vector ALU, no LDS traffic.
__device__ __forceinline__ float row16_sum(float v) {
#define GRIDNET_ROR(n) \
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x120 + (n), 0xf, 0xf, false))
    GRIDNET_ROR(8);
    GRIDNET_ROR(4);
    GRIDNET_ROR(2);
    GRIDNET_ROR(1);
#undef GRIDNET_ROR
    return v;
}

// The value of `v` in the lane before / after the caller's in the wave (DPP wave shifts: no LDS
// access).  For kernels whose lanes run along a grid row: the caller masks the ends of its row.
__device__ __forceinline__ float lane_before(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x138, 0xf, 0xf, false));
}
__device__ __forceinline__ float lane_after(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x130, 0xf, 0xf, false));
}

// Sum of `v` over those lanes of the calling wave that belong to the caller's slot: the whole
// wave for slots of 64 threads and more, the caller's half of it for 32-thread slots.  Row
// rotations, then the four row totals are read across as scalars: no LDS, and every lane of the
// slot gets the same bits.
template <int TPS> __device__ __forceinline__ float slot_wave_sum(float v) {
    static_assert(TPS == 32 || TPS % 64 == 0, "slots are half waves or whole waves");
    const int r = __float_as_int(row16_sum(v));
    const float r0 = __int_as_float(__builtin_amdgcn_readlane(r, 0));
    const float r1 = __int_as_float(__builtin_amdgcn_readlane(r, 16));
    const float r2 = __int_as_float(__builtin_amdgcn_readlane(r, 32));
    const float r3 = __int_as_float(__builtin_amdgcn_readlane(r, 48));
    if (TPS == 32) return (threadIdx.x & 32) ? r2 + r3 : r0 + r1;
    return (r0 + r1) + (r2 + r3);
}

// (mean, M2 about that mean) of the cells that the lanes of a slot in this wave hold, from the
// same pair per 16-lane row (each over `row_cells` cells): the rows' means are averaged and the
// M2 combined with the exact pairwise formula, M2 = sum M2_r + row_cells sum (mean_r - mean)^2.
// Every lane of the slot gets the same pair.  TPS as for slot_wave_sum.
template <int TPS>
__device__ __forceinline__ void slot_wave_moments(float row_mean, float row_m2, int row_cells, float &mean,
                                                  float &m2) {
    static_assert(TPS == 32 || TPS % 64 == 0, "slots are half waves or whole waves");
    float m[4], q[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        m[r] = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(row_mean), 16 * r));
        q[r] = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(row_m2), 16 * r));
    }
    if (TPS == 32) {
        const bool upper = (threadIdx.x & 32) != 0;
        const float a = upper ? m[2] : m[0], b = upper ? m[3] : m[1];
        mean = 0.5f * (a + b);
        m2 = (upper ? q[2] + q[3] : q[0] + q[1]) + row_cells * ((a - mean) * (a - mean) + (b - mean) * (b - mean));
    } else {
        mean = 0.25f * ((m[0] + m[1]) + (m[2] + m[3]));
        float dev = 0.f;
#pragma unroll
        for (int r = 0; r < 4; ++r) dev = fmaf(m[r] - mean, m[r] - mean, dev);
        m2 = ((q[0] + q[1]) + (q[2] + q[3])) + row_cells * dev;
    }
}

// Load p[i], i the same for the whole wave, as a VECTOR memory load.  Left alone the compiler
// makes it a scalar load; those return out of order and share their counter with LDS, so one
// that is still on its way stalls the next LDS access for a whole trip to memory -- and the
// per-sample numbers loaded this way are requested an element ahead, in the middle of LDS work.
__device__ __forceinline__ float load_ahead(const float *p, int i) {
    int zero;
    asm volatile("v_mov_b32 %0, 0" : "=v"(zero));
    return p[i + zero];
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
        if constexpr (TL::kDense) {
            // i fastest, then j, then kt: with the unpadded rows of this layout the lanes that an
            // LDS access serves together fall on different banks
            i = lane % bs;
            j = (lane / bs) % bs;
            kt = lane / (bs * bs);
        } else {
            // kt fastest, then i, then j: the lanes an LDS access serves together then differ in
            // the plane index, and the plane stride (S*RS = 120 or 48 floats) spreads them over banks
            kt = lane % TL::KT;
            i = (lane / TL::KT) % bs;
            j = lane / (TL::KT * bs);
        }
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
template <typename TL, int NT = TL::TPS> struct Fetch {  // NT: threads of a slot
    static constexpr int S = TL::S, BS = TL::S - 2, HL = S / 2, HC = BS / 2;
    static constexpr int NHALF = 2 * S * S;
    static constexpr int RPT = (NHALF + NT - 1) / NT;  // half rows per thread
    using Buf = float[RPT][HL];
    int goff[RPT];   // grid offset (within a sample) of the half row's first block cell; rows
                     // outside the grid point at a valid address and are zeroed when committed
    int loff[RPT];   // LDS offset of the half row's first entry, -1: none for this thread
    int edge[RPT];   // address delta of the end entry relative to goff (0 when it is off-grid)
    bool ok[RPT];    // the row lies inside the grid
    bool edge_ok[RPT];
    bool hi[RPT];    // second half: [cells..., end entry] instead of [end entry, cells...]
    int lane0;       // the thread's index in its slot
    __device__ __forceinline__ Fetch(int lane, int p0, int q0, int r0, int M, int N, int K) {
        lane0 = lane;
#pragma unroll
        for (int e = 0; e < RPT; ++e) {
            const int id = lane + e * NT;
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
    // Unconditional loads (no branches, no register initialisation in front of them).  The lane
    // offsets are handed over as unsigned BYTE offsets beside the uniform base: that is an
    // addressing mode (scalar base + 32-bit lane offset); a signed element index is widened and
    // scaled into a register pair per load.
    __device__ __forceinline__ void fetch(const float *xs, Buf &v) const {
#pragma unroll
        for (int e = 0; e < RPT; ++e) {
            const char *base = reinterpret_cast<const char *>(xs);
            const unsigned at = 4u * (unsigned)goff[e];
            const float *p = reinterpret_cast<const float *>(base + at);
            float c[HC];
            load_cells<HC>(p, c);
            const float end = *reinterpret_cast<const float *>(base + (at + 4u * (unsigned)edge[e]));
            // lay the values out in window order for either half
#pragma unroll
            for (int q = 0; q < HC; ++q) v[e][q] = c[q];
            v[e][HC] = end;
        }
    }
    // Both window copies receive every entry (the halo must be in both; the block itself is
    // overwritten by the iterations anyway).
    template <int COPIES = 2>
    __device__ __forceinline__ void commit(float *win, const Buf &v) const {
#pragma unroll
        for (int e = 0; e < RPT; ++e)
            if (loff[e] >= 0) {
                const float end = (ok[e] && edge_ok[e]) ? v[e][HC] : 0.f;
                int lo = loff[e];  // opaque: see commit_ln
                asm volatile("" : "+v"(lo));
#pragma unroll
                for (int copy = 0; copy < COPIES; ++copy) {
                    float *row = win + copy * TL::WIN + lo;
                    // first half: [end, cells...]; second half: [cells..., end]
                    row[hi[e] ? HC : 0] = end;
#pragma unroll
                    for (int q = 0; q < HC; ++q) row[q + (hi[e] ? 0 : 1)] = ok[e] ? v[e][q] : 0.f;
                }
            }
    }
    // The commit for the per-window normalisation: every entry is written MINUS `shift` (entries
    // outside the grid, zeros, become -shift) and what is written is added up: (sum, sum of
    // squares) of the halo entries in part[0..1], of the block's own cells in part[2..3].
    // Normalising a window does not care about a common shift of its entries; with `shift` a value
    // from the window itself the sums stay small, and variance = E[x^2] - mean^2 keeps its digits
    // however far the data sits from zero.
    template <int COPIES = 2>
    __device__ __forceinline__ void commit_sums(float *win, const Buf &v, float shift,
                                                float (&part)[4]) const {
#pragma unroll
        for (int q = 0; q < 4; ++q) part[q] = 0.f;
#pragma unroll
        for (int e = 0; e < RPT; ++e)
            if (loff[e] >= 0) {
                const int row = (lane0 + e * NT) >> 1;
                const int wj = row % S, wi = row / S;
                const bool halo_row = wi == 0 || wi == S - 1 || wj == 0 || wj == S - 1;
                const float end = ((ok[e] && edge_ok[e]) ? v[e][HC] : 0.f) - shift;
                float c[HC], s1 = 0.f, s2 = 0.f;
#pragma unroll
                for (int q = 0; q < HC; ++q) {
                    c[q] = (ok[e] ? v[e][q] : 0.f) - shift;
                    s1 += c[q];
                    s2 = fmaf(c[q], c[q], s2);
                }
                part[0] += end + (halo_row ? s1 : 0.f);
                part[1] += fmaf(end, end, halo_row ? s2 : 0.f);
                part[2] += halo_row ? 0.f : s1;
                part[3] += halo_row ? 0.f : s2;
#pragma unroll
                for (int copy = 0; copy < COPIES; ++copy) {
                    float *row_at = win + copy * TL::WIN + loff[e];
                    row_at[hi[e] ? HC : 0] = end;
#pragma unroll
                    for (int q = 0; q < HC; ++q) row_at[q + (hi[e] ? 0 : 1)] = c[q];
                }
            }
    }
    // The same, with the LayerNorm of the producer applied on the way in: an entry becomes
    // (v - mean) * rstd * gamma + beta; entries outside the grid stay zero.  gamma and beta of a
    // thread's half rows sit in LDS packed per half row, [gamma cells | beta cells | gamma end,
    // beta end] at stride GB, so that they come back as three aligned vector reads (read from
    // windows laid out like `win` they were ten scattered 32-bit reads per half row).
    static constexpr int GB = (2 * HC + 2 + 3) / 4 * 4;
    static constexpr int AFFINE = ((NHALF + NT - 1) / NT) * NT * GB;  // floats of the packed table
    __device__ __forceinline__ void pack_affine(float *gb, const Buf &gam, const Buf &bet) const {
#pragma unroll
        for (int e = 0; e < RPT; ++e)
            if (loff[e] >= 0) {
                float *to = gb + (lane0 + e * NT) * GB;
                float g[HC], b[HC];
#pragma unroll
                for (int q = 0; q < HC; ++q) {
                    g[q] = gam[e][q];
                    b[q] = bet[e][q];
                }
                store_cells<HC>(to, g);
                store_cells<HC>(to + HC, b);
                *reinterpret_cast<float2 *>(to + 2 * HC) = make_float2(gam[e][HC], bet[e][HC]);
            }
    }
    template <int COPIES = 2>
    __device__ __forceinline__ void commit_ln(float *win, const Buf &v, const float *gb, float mean,
                                              float rstd) const {
#pragma unroll
        for (int e = 0; e < RPT; ++e)
            if (loff[e] >= 0) {
                const float *from = gb + (lane0 + e * NT) * GB;
                float g[HC], b[HC];
                load_cells<HC>(from, g);
                load_cells<HC>(from + HC, b);
                const float2 ends = *reinterpret_cast<const float2 *>(from + 2 * HC);
                // The row's place is taken through an opaque copy: the two addresses derived from
                // it are worked out here, per element (two instructions), instead of living in
                // registers of their own across the batch loop -- where the backward kernels have
                // none to spare, so that they came back from scratch memory one wait at a time.
                int lo = loff[e];
                asm volatile("" : "+v"(lo));
                const int at_end = lo + (hi[e] ? HC : 0), at_cells = lo + (hi[e] ? 0 : 1);
                const float end = (ok[e] && edge_ok[e]) ? fmaf((v[e][HC] - mean) * rstd, ends.x, ends.y)
                                                        : 0.f;
                float val[HC];
#pragma unroll
                for (int q = 0; q < HC; ++q)
                    val[q] = ok[e] ? fmaf((v[e][q] - mean) * rstd, g[q], b[q]) : 0.f;
#pragma unroll
                for (int copy = 0; copy < COPIES; ++copy) {
                    win[copy * TL::WIN + at_end] = end;
#pragma unroll
                    for (int q = 0; q < HC; ++q) win[copy * TL::WIN + at_cells + q] = val[q];
                }
            }
    }
};

// The same job for a kernel whose time goes into the memory pipeline rather than arithmetic
// (step_bwd_cross): every window row is read as bs/4 + 2 aligned 16-byte vectors by ADJACENT
// lanes -- the vector before the block (only its last float is an entry of the window), the
// block's own vectors, the vector after it (only its first float).  A row then costs the
// vector cache one or two line accesses instead of one per half row plus one per end entry.
// More registers per thread than Fetch, which is why the compute-bound kernels keep that one.
template <typename TL, int NT> struct FetchLines {
    static constexpr int S = TL::S, BS = TL::S - 2, NQ = BS / 4 + 2;
    static constexpr int NVEC = S * S * NQ;
    static constexpr int RPT = (NVEC + NT - 1) / NT;  // vectors per thread
    using Buf = float[RPT][4];
    int goff[RPT];   // grid offset (within a sample) of the vector
    int meta[RPT];   // bits 0..11: LDS offset of the first window entry the vector fills;
                     // bits 12..13: 0 all four floats are entries, 1 only the last, 2 only the
                     // first, 3 nothing (no vector for this thread); bit 14: inside the grid
    __device__ __forceinline__ FetchLines(int lane, int p0, int q0, int r0, int M, int N, int K) {
        static_assert(TL::WIN < 4096, "window offsets must fit 12 bits");
#pragma unroll
        for (int e = 0; e < RPT; ++e) {
            const int id = lane + e * NT;
            const int qd = id % NQ, row = id / NQ;
            const int wj = row % S, wi = row / S;
            const int gi = p0 + wi - 1, gj = q0 + wj - 1, col = r0 + 4 * (qd - 1);
            const bool have = id < NVEC;
            const bool ok = have && gi >= 0 && gi < M && gj >= 0 && gj < N && col >= 0 && col < K;
            const int kind = !have ? 3 : qd == 0 ? 1 : qd == NQ - 1 ? 2 : 0;
            const int wk = qd == 0 ? 0 : qd == NQ - 1 ? S - 1 : 1 + 4 * (qd - 1);
            meta[e] = (have ? wi * TL::PS + wj * TL::RS + wk : 0) | (kind << 12) | (ok ? 1 << 14 : 0);
            // anything outside the grid (and threads without a vector) reads the start of row
            // (0, 0) of the block's own columns: always in bounds
            goff[e] = ok ? (gi * N + gj) * K + col : r0;
        }
    }
    __device__ __forceinline__ void fetch(const float *xs, Buf &v) const {
#pragma unroll
        for (int e = 0; e < RPT; ++e) load_cells<4>(xs + goff[e], v[e]);
    }
    // entries are committed as (v - mean) * rstd (mean 0, rstd 1: as they are); zero outside the grid
    template <int COPIES = 2>
    __device__ __forceinline__ void commit(float *win, const Buf &v, float mean = 0.f,
                                           float rstd = 1.f) const {
#pragma unroll
        for (int e = 0; e < RPT; ++e) {
            const int kind = (meta[e] >> 12) & 3;
            const bool ok = (meta[e] >> 14) & 1;
            float *to = win + (meta[e] & 0xfff);
            if (kind == 0) {
#pragma unroll
                for (int copy = 0; copy < COPIES; ++copy)
#pragma unroll
                    for (int q = 0; q < 4; ++q)
                        to[copy * TL::WIN + q] = ok ? (v[e][q] - mean) * rstd : 0.f;
            } else if (kind != 3) {
                const float end = ok ? ((kind == 1 ? v[e][3] : v[e][0]) - mean) * rstd : 0.f;
#pragma unroll
                for (int copy = 0; copy < COPIES; ++copy) to[copy * TL::WIN] = end;
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

// Commit R x C gradient values to base[index(r, c)] for the entries with ok(r, c): plain stores in
// every mode.  The workgroup is the only one that writes these entries of its arrays (the
// caller's, or its batch chunk's copy of them); in the add-in-place mode the accumulators were
// STARTED from the old contents (see the kernels' set-up): an old value fetched at the end
// instead would put a serial trip to memory at the tail of every workgroup, where nothing is left
// to hide it.
// The test of the (uniform) mode is always true here, the tuned kernels are never launched with
// kParamAtomic; it keeps the stores and their address arithmetic in a basic block of their own,
// which the register allocator rewards: without it the chain's backward kernel reloads three
// more spilled values inside its batch loop (+3 us at the 64^3 / batch 32 shape).
template <int R, int C, typename Index, typename Ok>
__device__ __forceinline__ void commit_grads(float *base, const float (&val)[R][C], int mode,
                                             Index &&index, Ok &&ok) {
    if (mode != kParamAtomic) {
#pragma unroll
        for (int r = 0; r < R; ++r)
#pragma unroll
            for (int c = 0; c < C; ++c)
                if (ok(r, c)) base[index(r, c)] = val[r][c];
    }
}

}  // namespace
}  // namespace gridnet

#endif  // GRIDNET_FAST_TILES_H
