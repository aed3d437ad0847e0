// Backward of one step of the network body "update step, then per-sample LayerNorm" inside a
// CHAIN of such steps: 8^3 blocks, fp32, normalize off, up to 4 inner iterations.
//
// The reference's backward scatters what crosses a block boundary into the grid with global
// atomics (src/gridnet_cuda_kernels.cu:424-435); the tuned kernels of step_fast.hip finish dx in
// a second kernel (step_bwd_cross).  A chain of steps needs neither:
//
//   * what a block's cells send to the cells AROUND the block (one cell deep: the 488 entries
//     of the (8+2)^3 window that are not the block's own) depends on the inner iterations only
//     through D = sum_i delta_i (the halo is frozen).  After the sweep the workgroup writes D
//     into an LDS window and works those 488 values out itself -- entry h receives
//     sum W[t, c] D[c] over the <= 9 pairs (cell c of the block, tap t) with c + off_t = h --
//     and files each with the block that owns cell h.  Nobody adds them to dx: the backward of
//     the step BEFORE this one, whose incoming gradient dx is, picks up the <= 7 values a cell
//     receives while it loads that gradient.  No second kernel, no D tensor written and read back
//     with its halo, no read-modify-write of dx;
//   * the two per-sample sums that the LayerNorm in front of this step needs for its backward,
//     sum(gamma dx) and sum(gamma dx xhat), are linear in dx, so every workgroup adds up its own
//     share -- its cells' part plus what its 488 outgoing values contribute at the cells that
//     receive them (gamma, beta and the normalised input at those cells are at hand: they are the
//     halo of the block's own window) -- and leaves one pair per (element, block).
//
// The first step of a chain must deliver a finished dx: its variant (DEFER = false) leaves D
// instead and is followed by the cross-block kernel of step_fast.hip.
//
// Everything inside the block is step_bwd_fast's way: the inner forward is recomputed from the
// step's input (the pre-activations stay in LDS; x_i is rebuilt on the way back from
// x_i = x_{i+1} - r act(u_i)), the reverse sweep gathers over zero-haloed delta windows with the
// neighbours' mirrored weights in registers.  Keeping the pre-activations in memory instead of
// recomputing them was tried and lost: 4 more activation tensors written and read per step cost
// as much as the 27 FMAs per cell and iteration they save (forward 65 -> 93 us at 64^3 / batch
// 32, with the LayerNorm kernels around it slowed by the cache traffic as well).
//
// Threads: 256 per (block, element), two cells of a K-row each; thread q and q + 256 also own
// entry q of the 488 (computing what it receives).

#include "common.h"
#include "fast_tiles.h"
#include "launch.h"
#include "plan.h"

namespace gridnet {

namespace {

constexpr int kShell = 488;  // (8 + 2)^3 - 8^3 window entries around a block
constexpr int kChainMaxInner = 4;  // the pre-activations of more iterations do not fit: two workgroups
                                    // share the 160 KB of a CU
constexpr int kChainDepth = 4;  // neighbour rows requested ahead of the arithmetic

// The 488 values a block RECEIVES for one element, by where they come from: the neighbouring
// block at offset (si, sj, sk); a non-zero si selects the block's cells with i = 0 (si = -1,
// side 0) or i = 7 (si = +1, side 1), likewise sj, sk.
//   faces   I [side][j][k]   J [side][i][k]   K [side][i][j]       64 values each
//   edges   IJ [si][sj][k]   IK [si][sk][j]   JK [sj][sk][i]        8 values each
//   corners [si][sj][sk]
// The K-contiguous pieces come first: the thread that owns cells (i, j, 2kt), (i, j, 2kt + 1)
// reads its part of them as two-float vectors.
constexpr int kSegI = 0, kSegJ = 128, kSegIJ = 256, kSegK = 288, kSegIK = 416, kSegJK = 448, kSegC = 480;

// Window coordinates (0..9 per axis) of shell entry q.  The entries are numbered by WHERE THEY GO:
// q is the offset of the value in the receiving block's record (layout above), so consecutive
// threads store to consecutive addresses.  A side flag f of the receiving block means the
// entry lies on the far side of this block's window: f = 0 (the receiver's cells with
// coordinate 0) is this window's plane 9, f = 1 its plane 0.
__device__ __forceinline__ void shell_coords(int q, int &wi, int &wj, int &wk) {
    auto far = [](int f) { return f ? 0 : 9; };
    if (q < kSegJ) {
        wi = far(q / 64); wj = 1 + (q / 8) % 8; wk = 1 + q % 8;
    } else if (q < kSegIJ) {
        const int r = q - kSegJ;
        wj = far(r / 64); wi = 1 + (r / 8) % 8; wk = 1 + r % 8;
    } else if (q < kSegK) {
        const int r = q - kSegIJ;
        wi = far(r / 16); wj = far((r / 8) % 2); wk = 1 + r % 8;
    } else if (q < kSegIK) {
        const int r = q - kSegK;
        wk = far(r / 64); wi = 1 + (r / 8) % 8; wj = 1 + r % 8;
    } else if (q < kSegJK) {
        const int r = q - kSegIK;
        wi = far(r / 16); wk = far((r / 8) % 2); wj = 1 + r % 8;
    } else if (q < kSegC) {
        const int r = q - kSegJK;
        wj = far(r / 16); wk = far((r / 8) % 2); wi = 1 + r % 8;
    } else {
        const int r = q - kSegC;
        wi = far(r / 4); wj = far((r / 2) % 2); wk = far(r % 2);
    }
}

// base + a 32-bit BYTE offset per lane: with a uniform base this is one addressing mode (scalar
// base, 32-bit lane offset); an element index would be widened and scaled into a register pair
// per lane, which the compiler then keeps -- or spills -- across the batch loop
template <typename T> __device__ __forceinline__ const T &at_bytes(const float *base, unsigned bytes) {
    return *reinterpret_cast<const T *>(reinterpret_cast<const char *>(base) + bytes);
}
template <typename T> __device__ __forceinline__ T &at_bytes(float *base, unsigned bytes) {
    return *reinterpret_cast<T *>(reinterpret_cast<char *>(base) + bytes);
}

struct ChainBwdArgs {
    const float *weight, *bias, *scale, *gamma, *beta;
    const float *x, *x_stats;  // the step's input as stored (raw output of the step before, or the
                               // chain's input with x_stats == null) and its LayerNorm statistics
    const float *dy;           // gradient with respect to LayerNorm(y_raw); complete, or lacking
                               // what halo_in holds
    const float *y_raw, *y_stats, *y_sums;
    const float *halo_in;      // [B, nblk, 488] or null
    float *dweight, *dbias, *dscale, *dgamma, *dbeta;
    float *dx;                 // the block-local part of the input gradient
    float *out2;               // DEFER: halo_out [B, nblk, 488]; otherwise D [B, cells]
    float *x_part;             // DEFER: [B, nblk, 2] sums for the LayerNorm in front of this step
    int B, M, N, K, inner, nblk, nchunk, chunk_len, param_mode;
    long slab_stride;          // split batch: floats between the chunks' copies of the gradient arrays, else 0
};

// LDS (floats): [x window x2 | delta window x2 | u_i of the owned cells, inner slabs of 512 |
// gamma, beta of the window, packed | sums of the four waves | weights of the shell entries
// [9][512] | per-thread constants [kTab][256]]; at set-up the block's 27 weight planes pass
// through the front of it.
using ChainTile = Tile<8, 2>;
// Table entries.  Small integers are packed (the table is the difference between two workgroups
// per CU and one): In = the seven record offsets of what the thread's cells receive, three 10-bit
// float indices per word; ShellAt = both shell entries' places in the x window, 16 bits each;
// Halo = per shell entry the window offset of its centre source (bits 0-11) and the codes of its
// two strides (bits 12-13, 14-15: 0 -> 1, 1 -> row, 2 -> plane).
enum { kTabDst = 0, kTabIn = 2, kTabShellAt = 5, kTabHalo = 6, kTabShellGamma = 8, kTabShellBeta = 10,
       kTabBeta = 12, kTabGamma = 14, kTabAcc = 16 /* 8 gradient sums */, kTab = 24 };
constexpr int kChainAffine = 200 * Fetch<ChainTile>::GB;  // packed gamma/beta: 200 half rows
__host__ __device__ constexpr int chain_lds_floats(int inner) {
    const int run = 4 * ChainTile::WIN + inner * 512 + kChainAffine + 16 + 9 * 512 + kTab * 256;
    return run > 27 * 512 ? run : 27 * 512;
}
__device__ __forceinline__ int stride_of(unsigned code) {
    return code == 0 ? 1 : code == 1 ? ChainTile::RS : ChainTile::PS;
}

template <int ACT, bool DEFER>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2)))
void chain_bwd(const ChainBwdArgs a) {
    using TL = ChainTile;
    constexpr int BS = 8, CPT = 2, NC = BS * BS * BS;
    extern __shared__ __attribute__((aligned(16))) float lds[];
    const int inner = a.inner;
    float *win = lds;                          // two copies of the x window
    float *dwin = win + 2 * TL::WIN;           // two delta windows, halo zero
    float *hist = dwin + 2 * TL::WIN;          // u_i of this thread's cells at hist + it * 512 + lane * 2
    float *affine = hist + inner * 512;        // gamma and beta of the window, packed per half row
    float *red = affine + kChainAffine;   // [2][4][2], per wave: the two LayerNorm sums of an element, elements alternating
    float *hwl = red + 16;                     // [256][18]: the weights that feed the shell entries
    // ... and what a thread uses once per element: [kTab][256], entry k of thread t at
    // ctab[k * 256 + t].  The register file has no room for these, and a spilled register is
    // worse than an LDS read: spill traffic queues behind the prefetch in the memory pipeline.
    unsigned *ctab = reinterpret_cast<unsigned *>(hwl + 9 * 512);

    int blk, chunk;
    if (!split_block_id(blockIdx.x, a.nblk, a.nchunk, blk, chunk)) return;  // grid padding
    // A split batch: every chunk commits into a copy of the gradient arrays of its own.  Worked out
    // where it is used (before and after the batch loop), not kept: the loop has no register to spare.
    auto slab_offset = [&]() -> long {
        int b2, c2;
        (void)split_block_id(blockIdx.x, a.nblk, a.nchunk, b2, c2);
        return a.slab_stride ? c2 * a.slab_stride : 0;
    };
    const int tid = threadIdx.x;
    const Place<TL, CPT, 1> pl(tid, blk, a.N, a.K);
    const Fetch<TL> fx(tid, pl.p0, pl.q0, pl.r0, a.M, a.N, a.K);
    const long cells = (long)a.M * a.N * a.K;
    const int N = a.N, K = a.K;
    const bool ln_in = a.x_stats != nullptr;
    // the x window copy that would receive x_inner (never needed) gets zeros in the block's cells
    // instead: the window's halo alone, for the weights of the taps that read it
    const float *xhalo = win + (inner & 1) * TL::WIN;
    auto tab = [&](int k) -> unsigned & { return ctab[k * 256 + tid]; };

    auto in_block = [&](int t, int c) {
        const int ni = pl.i + t / 9 - 1, nj = pl.j + (t / 3) % 3 - 1, nk = pl.kt * CPT + c + t % 3 - 1;
        return ni >= 0 && ni < BS && nj >= 0 && nj < BS && nk >= 0 && nk < BS;
    };
    // the weight whose gradient nw[t][c] accumulates: the neighbour's mirrored weight where the
    // neighbour at c + off_t lies in this block, this cell's own weight of tap t where it does
    // not (that tap reads a frozen halo entry; see step_bwd_fast)
    auto owner_of = [&](int t, int c) {
        return in_block(t, c)
                   ? (26 - t) * cells + pl.gc + c + ((t / 9 - 1) * N + ((t / 3) % 3 - 1)) * K + (t % 3 - 1)
                   : t * cells + pl.gc + c;
    };
    auto always = [](int, int) { return true; };

    // ---- once per workgroup ----
    const int kb = K / BS, nb = N / BS, mb = a.M / BS;
    const int bi = blk / (kb * nb), bj = (blk / kb) % nb, bk = blk % kb;
    bool s_in[2];
    float w[27][CPT], v[27][CPT], nw[27][CPT], bv[CPT], rv[CPT];
    // sums over the batch that are touched once per element live in the table, not in registers:
    // dbias, dscale, dgamma, dbeta of the owned cells
    float dgam[CPT], dbet[CPT], db[CPT], dr[CPT], gam[CPT];
#pragma unroll
    for (int t = 0; t < 27; ++t) load_cells<CPT>(a.weight + t * cells + pl.gc, w[t]);
    load_cells<CPT>(a.bias + pl.gc, bv);
    load_cells<CPT>(a.scale + pl.gc, rv);
    load_cells<CPT>(a.gamma + pl.gc, gam);
#pragma unroll
    for (int c = 0; c < CPT; ++c) dgam[c] = dbet[c] = db[c] = dr[c] = 0.f;
    {
        // this block's weights pass through LDS once: every thread picks up the mirrored
        // weights of its cells' in-block neighbours and the weights that feed its shell entries
        float hw[2][9], hgam[2], hbet[2];
        unsigned s_dst[2], s_at[2];
        int h_base[2], h_sb[2], h_sc[2];
        float *wl = lds;  // [27][NC], by block-local cell (i, j, k)
        const int lin = (pl.i * BS + pl.j) * BS + pl.kt * CPT;
#pragma unroll
        for (int t = 0; t < 27; ++t) store_cells<CPT>(wl + t * NC + lin, w[t]);
        lds_barrier();
#pragma unroll
        for (int t = 0; t < 27; ++t)
#pragma unroll
            for (int c = 0; c < CPT; ++c) {
                v[t][c] = in_block(t, c)
                              ? wl[(26 - t) * NC + lin + c + ((t / 9 - 1) * BS + ((t / 3) % 3 - 1)) * BS + (t % 3 - 1)]
                              : 0.f;
                nw[t][c] = 0.f;
            }
#pragma unroll
        for (int e = 0; e < 2; ++e) {
            const int id = tid + e * 256;
            const bool have = id < kShell;
            int wi, wj, wk;
            shell_coords(have ? id : 0, wi, wj, wk);
            const int gi = pl.p0 + wi - 1, gj = pl.q0 + wj - 1, gk = pl.r0 + wk - 1;
            const bool ing = have && gi >= 0 && gi < a.M && gj >= 0 && gj < N && gk >= 0 && gk < K;
            s_in[e] = ing;
            s_at[e] = wi * TL::PS + wj * TL::RS + wk;  // the entry in the x window
            // the block that owns the cell; the entry's number is its place in that block's record
            const int di = wi == 0 ? -1 : wi == 9 ? 1 : 0, dj = wj == 0 ? -1 : wj == 9 ? 1 : 0,
                      dk = wk == 0 ? -1 : wk == 9 ? 1 : 0;
            const int tblk = ((bi + di) * nb + (bj + dj)) * kb + (bk + dk);
            s_dst[e] = 4u * (ing ? tblk * kShell + id : 0);
            // its <= 9 sources: fixed along the first axis on which the entry lies outside the
            // block (A), three candidates around the clamped coordinate along the other two
            const int A = di ? 0 : dj ? 1 : 2;
            const int wB = A == 0 ? wj : wi, wC = A == 2 ? wj : wk;
            const int sB = A == 0 ? TL::RS : TL::PS, sC = A == 2 ? TL::RS : 1;
            const int cA = (A == 0 ? wi : A == 1 ? wj : wk) == 0 ? 1 : 8;
            const int cB0 = min(max(wB, 1), 8), cC0 = min(max(wC, 1), 8);
            h_sb[e] = sB;
            h_sc[e] = sC;
            h_base[e] = cA * (A == 0 ? TL::PS : A == 1 ? TL::RS : 1) + cB0 * sB + cC0 * sC;
#pragma unroll
            for (int slot = 0; slot < 9; ++slot) {
                const int cB = cB0 + slot / 3 - 1, cC = cC0 + slot % 3 - 1;
                const int oA = (A == 0 ? wi : A == 1 ? wj : wk) - cA, oB = wB - cB, oC = wC - cC;
                const bool ok = ing && cB >= 1 && cB <= 8 && cC >= 1 && cC <= 8 && oB >= -1 && oB <= 1 &&
                                oC >= -1 && oC <= 1;
                // (A, B, C) back to (i, j, k)
                const int ci = A == 0 ? cA : cB, cj = A == 0 ? cB : A == 1 ? cA : cC, ck = A == 2 ? cA : cC;
                const int oi = A == 0 ? oA : oB, oj = A == 0 ? oB : A == 1 ? oA : oC, ok_ = A == 2 ? oA : oC;
                const int t = (oi + 1) * 9 + (oj + 1) * 3 + (ok_ + 1);
                const int cell = ((ci - 1) * BS + (cj - 1)) * BS + (ck - 1);
                hw[e][slot] = ok ? wl[t * NC + cell] : 0.f;
            }
            const int goff = ing ? (gi * N + gj) * K + gk : pl.gc;
            hgam[e] = (ln_in && ing) ? a.gamma[goff] : 0.f;
            hbet[e] = (ln_in && ing) ? a.beta[goff] : 0.f;
        }
        lds_barrier();  // everything behind the windows reuses this memory
        auto code_of = [](int stride) { return stride == 1 ? 0u : stride == TL::RS ? 1u : 2u; };
#pragma unroll
        for (int e = 0; e < 2; ++e)
            tab(kTabHalo + e) = (unsigned)h_base[e] | code_of(h_sb[e]) << 12 | code_of(h_sc[e]) << 14;
        tab(kTabGamma) = __float_as_uint(gam[0]);
        tab(kTabGamma + 1) = __float_as_uint(gam[1]);
        if (DEFER) {
#pragma unroll
            for (int e = 0; e < 2; ++e) {
#pragma unroll
                for (int slot = 0; slot < 9; ++slot) hwl[tid * 18 + e * 9 + slot] = hw[e][slot];
                tab(kTabDst + e) = s_dst[e];
                tab(kTabShellGamma + e) = __float_as_uint(hgam[e]);
                tab(kTabShellBeta + e) = __float_as_uint(hbet[e]);
            }
            tab(kTabShellAt) = s_at[0] | s_at[1] << 16;
            float bet[CPT];
            load_cells<CPT>(a.beta + pl.gc, bet);
            tab(kTabBeta) = __float_as_uint(bet[0]);
            tab(kTabBeta + 1) = __float_as_uint(bet[1]);
        }
    }

    // ---- what this thread's cells receive from the blocks around: where, and whether ----
    const int fi = pl.i == 0 ? 0 : pl.i == BS - 1 ? 1 : -1, fj = pl.j == 0 ? 0 : pl.j == BS - 1 ? 1 : -1,
              fk = pl.kt == 0 ? 0 : pl.kt == TL::KT - 1 ? 1 : -1;
    const bool have_in = a.halo_in != nullptr;
    const bool ei = have_in && (fi == 0 ? bi > 0 : fi == 1 ? bi < mb - 1 : false);
    const bool ej = have_in && (fj == 0 ? bj > 0 : fj == 1 ? bj < nb - 1 : false);
    const bool ek = have_in && (fk == 0 ? bk > 0 : fk == 1 ? bk < kb - 1 : false);
    {
        const int zi = max(fi, 0), zj = max(fj, 0), zk = max(fk, 0), k2 = pl.kt * CPT;
        const unsigned o[7] = {unsigned(kSegI + zi * 64 + pl.j * 8 + k2), unsigned(kSegJ + zj * 64 + pl.i * 8 + k2),
                               unsigned(kSegIJ + (zi * 2 + zj) * 8 + k2), unsigned(kSegK + zk * 64 + pl.i * 8 + pl.j),
                               unsigned(kSegIK + (zi * 2 + zk) * 8 + pl.j), unsigned(kSegJK + (zj * 2 + zk) * 8 + pl.i),
                               unsigned(kSegC + zi * 4 + zj * 2 + zk)};
        tab(kTabIn) = o[0] | o[1] << 10 | o[2] << 20;
        tab(kTabIn + 1) = o[3] | o[4] << 10 | o[5] << 20;
        tab(kTabIn + 2) = o[6];
    }
    // without halo_in every flag is off and the (unconditional) loads read dy instead: in bounds
    const float *hin = have_in ? a.halo_in : a.dy;
    const float *xst = ln_in ? a.x_stats : a.y_stats;
    const unsigned ugc = 4u * pl.gc;  // byte offset of the owned cells within a sample

    typename Fetch<TL>::Buf pre;
    if (ln_in) {  // gamma and beta of the window, once per workgroup
        typename Fetch<TL>::Buf bet;
        fx.fetch(a.gamma, pre);
        fx.fetch(a.beta, bet);
        fx.pack_affine(affine, pre, bet);
    }
    // delta windows: the halo stays zero for the whole kernel
    for (int idx = tid; idx < 2 * TL::WIN; idx += 256) dwin[idx] = 0.f;
    wait_global_loads();
    if (a.param_mode == kParamAddExclusive) {
        const long slab_off = slab_offset();
        // the accumulators start from what the gradient buffers hold and are stored at the end;
        // requested here, behind the set-up wait, the old values arrive during the first element
#pragma unroll
        for (int t = 0; t < 27; ++t)
#pragma unroll
            for (int c = 0; c < CPT; ++c) nw[t][c] = (a.dweight + slab_off)[owner_of(t, c)];
        load_cells<CPT>((a.dbias + slab_off) + pl.gc, db);
        load_cells<CPT>((a.dscale + slab_off) + pl.gc, dr);
        load_cells<CPT>((a.dgamma + slab_off) + pl.gc, dgam);
        load_cells<CPT>((a.dbeta + slab_off) + pl.gc, dbet);
    }
    auto acc_ref = [&](int k) -> float & { return reinterpret_cast<float *>(ctab)[(kTabAcc + k) * 256 + tid]; };
#pragma unroll
    for (int c = 0; c < CPT; ++c) {
        acc_ref(c) = db[c];
        acc_ref(2 + c) = dr[c];
        acc_ref(4 + c) = dgam[c];
        acc_ref(6 + c) = dbet[c];
    }

    const int s0 = chunk * a.chunk_len, s1 = min(a.B, s0 + a.chunk_len);
    float nxm = 0.f, nxr = 1.f;  // LayerNorm statistics of the element in `pre`
    auto fetch_window = [&](int s) {
        fx.fetch(a.x + (long)s * cells, pre);
        nxm = load_ahead(xst, 2 * s);
        nxr = load_ahead(xst, 2 * s + 1);
    };
    auto commit_window = [&]() {
        if (ln_in) fx.commit_ln(win, pre, affine, nxm, nxr);
        else fx.commit(win, pre);
    };
    // An element is finished one element late.  Its dx is stored behind the requests of the element
    // after.  With deferred halos, what its delta sums D send to the cells around the block -- the
    // shell values -- is worked out behind the next element's first barrier, next to the start of
    // that element's recompute: D waits in a delta window that nothing writes before the sweep, and
    // the chain of LDS reads, 18 multiply-adds and two wave sums that makes the shell values then
    // runs beside arithmetic that does not depend on it, instead of holding up every wave of the
    // workgroup at the end of its own element.
    float g_done[CPT], o_done[2];     // o_done: the element's D (without deferred halos)
    float t1_done = 0.f, t2_done = 0.f, nh_done[2] = {0.f, 0.f};  // its LayerNorm sums so far; x-hat at the shell entries
    int done_s = -1, sums_s = -1;
    auto store_done = [&]() {
        if (done_s < 0) return;
        const long o = (long)done_s * cells;
        at_bytes<float2>(a.dx + o, ugc) = make_float2(g_done[0], g_done[1]);
        if (!DEFER) at_bytes<float2>(a.out2 + o, ugc) = make_float2(o_done[0], o_done[1]);
    };
    // Where the sources of the thread's two shell entries sit in the D window: read in FRONT of the
    // barrier, so that the reads behind it start from known addresses (one LDS round trip less).
    auto shell_sources = [&](unsigned (&hal)[2]) {
        hal[0] = hal[1] = 0u;
        if (!DEFER || done_s < 0) return;
        hal[0] = tab(kTabHalo);
        hal[1] = tab(kTabHalo + 1);
    };
    // behind a barrier that follows the element's last write of D
    auto shell_of_done = [&](const unsigned (&hals)[2]) {
        const int hs = done_s;
        if (DEFER && hs >= 0) {
            // the thread's 18 shell weights sit side by side (stride 18 floats: nine conflict-free
            // 64-bit reads)
            float hwv[18];
#pragma unroll
            for (int q = 0; q < 9; ++q) {
                const float2 p2 = *reinterpret_cast<const float2 *>(hwl + tid * 18 + 2 * q);
                hwv[2 * q] = p2.x;
                hwv[2 * q + 1] = p2.y;
            }
            float t1 = t1_done, t2 = t2_done;
            float *rec = a.out2 + (long)hs * a.nblk * kShell;
#pragma unroll
            for (int e = 0; e < 2; ++e) {
                const unsigned hal = hals[e];
                const float *src = dwin + TL::WIN + (int)(hal & 0xfffu);
                // entries 0..255 are the I and J faces: their second stride is 1 (along K), known here,
                // so that the three reads of a row get constant offsets from one address
                const int sb = stride_of((hal >> 12) & 3u), sc = e == 0 ? 1 : stride_of((hal >> 14) & 3u);
                float acc = 0.f;
#pragma unroll
                for (int slot = 0; slot < 9; ++slot)
                    acc = fmaf(hwv[e * 9 + slot], src[(slot / 3 - 1) * sb + (slot % 3 - 1) * sc], acc);
                t1 = fmaf(__uint_as_float(tab(kTabShellGamma + e)), acc, t1);
                t2 = fmaf(acc, nh_done[e] - __uint_as_float(tab(kTabShellBeta + e)), t2);
                if (s_in[e]) {
                    // opaque here, so that the offset is widened inside this block, where the
                    // store can still take it as a 32-bit lane offset beside the scalar base
                    unsigned off = tab(kTabDst + e);
                    asm volatile("" : "+v"(off));
                    at_bytes<float>(rec, off) = acc;
                }
            }
            t1 = slot_wave_sum<256>(t1);
            t2 = slot_wave_sum<256>(t2);
            if ((tid & 63) == 0)
                *reinterpret_cast<float2 *>(red + (hs & 1) * 8 + 2 * (tid >> 6)) = make_float2(t1, t2);
        }
        // the sums of the element before that one: its four waves' shares, in a fixed order (they
        // were written a barrier ago, into the other half of `red`)
        if (DEFER && sums_s >= 0 && tid == 0) {
            const float *r = red + (sums_s & 1) * 8;
            float *to = a.x_part + ((long)sums_s * a.nblk + blk) * 2;
            to[0] = (r[0] + r[2]) + (r[4] + r[6]);
            to[1] = (r[1] + r[3]) + (r[5] + r[7]);
        }
        sums_s = hs;
        done_s = -1;
    };

    if (ln_in) lds_barrier();  // the packed gamma and beta
    if (s0 < s1) {
        fetch_window(s0);
        commit_window();
    }
    for (int s = s0; s < s1; ++s) {
        take_turns(s);
        // Requests first, stores behind them: loads and stores retire through one in-order
        // counter, and no wait for a load may include the stores.  This element's gradient (used
        // after the recompute, which hides the trip), then the next element's window.  All of it
        // in front of the barrier: none of it touches the windows, and the wait for the other
        // waves covers the issue.
        const long at = (long)s * cells;
        const float2 dy2 = at_bytes<float2>(a.dy + at, ugc), yr2 = at_bytes<float2>(a.y_raw + at, ugc);
        const float *rec = hin + ((long)s * a.nblk + blk) * kShell;
        const unsigned oa = tab(kTabIn), ob = tab(kTabIn + 1), oc = tab(kTabIn + 2);
        auto off10 = [](unsigned word, int k) { return 4u * ((word >> (10 * k)) & 1023u); };
        const float2 in_i = at_bytes<float2>(rec, off10(oa, 0)), in_j = at_bytes<float2>(rec, off10(oa, 1)),
                     in_ij = at_bytes<float2>(rec, off10(oa, 2));
        const float in_k = at_bytes<float>(rec, off10(ob, 0)), in_ik = at_bytes<float>(rec, off10(ob, 1)),
                    in_jk = at_bytes<float>(rec, off10(ob, 2)), in_c = at_bytes<float>(rec, off10(oc, 0));
        const float ny0 = load_ahead(a.y_stats, 2 * s), ny1 = load_ahead(a.y_stats, 2 * s + 1),
                    ny2 = load_ahead(a.y_sums, 2 * s), ny3 = load_ahead(a.y_sums, 2 * s + 1);
        fetch_window(min(s + 1, s1 - 1));
        store_done();
        unsigned shc[2];
        shell_sources(shc);
        lds_barrier();  // this element's window is in place; the last round's LDS readers are done
        shell_of_done(shc);

        // ---- forward recompute; u_i of the owned cells is remembered ----
        float xcur[CPT];
#pragma unroll
        for (int c = 0; c < CPT; ++c) xcur[c] = win[pl.own + c];
        for (int it = 0; it < inner; ++it) {
            float u[CPT];
            stencil<TL, CPT, kChainDepth>(win + (it & 1) * TL::WIN, pl.row00, w, bv, u);
            store_cells<CPT>(hist + it * 512 + tid * CPT, u);
#pragma unroll
            for (int c = 0; c < CPT; ++c) {
                xcur[c] = fmaf(rv[c], Act<ACT, float>::f(u[c]), xcur[c]);
                // x_inner itself goes nowhere: that window copy becomes the halo-only window
                win[((it + 1) & 1) * TL::WIN + pl.own + c] = it + 1 < inner ? xcur[c] : 0.f;
            }
            if (it + 1 < inner) lds_barrier();
        }

        // ---- the incoming gradient: what the blocks around left for these cells (fixed
        // order), then through the backward of the LayerNorm behind this step ----
        float g[CPT], dsum[CPT];
        {
            float tot[CPT] = {dy2.x, dy2.y};
            if (ei) { tot[0] += in_i.x; tot[1] += in_i.y; }
            if (ej) { tot[0] += in_j.x; tot[1] += in_j.y; }
            if (ei && ej) { tot[0] += in_ij.x; tot[1] += in_ij.y; }
            float ends = 0.f;
            if (ek) ends += in_k;
            if (ei && ek) ends += in_ik;
            if (ej && ek) ends += in_jk;
            if (ei && ej && ek) ends += in_c;
            tot[0] += fk == 0 ? ends : 0.f;
            tot[1] += fk == 1 ? ends : 0.f;
            const float yr[CPT] = {yr2.x, yr2.y};
#pragma unroll
            for (int c = 0; c < CPT; ++c) {
                const float yh = (yr[c] - ny0) * ny1;
                acc_ref(4 + c) = fmaf(tot[c], yh, acc_ref(4 + c));
                acc_ref(6 + c) += tot[c];
                g[c] = ny1 * (__uint_as_float(tab(kTabGamma + c)) * tot[c] - ny2 - yh * ny3);
                dsum[c] = 0.f;
            }
        }

        // ---- reverse sweep: delta window copy (it & 1) holds delta_it; xcur walks back from
        // x_inner to x_0 ----
        float nh[2] = {0.f, 0.f}, dre[CPT] = {0.f, 0.f};
        for (int it = inner - 1; it >= 0; --it) {
            float u[CPT];
            load_cells<CPT>(hist + it * 512 + tid * CPT, u);
#pragma unroll
            for (int c = 0; c < CPT; ++c) {
                float f, d;
                Act<ACT, float>::fd(u[c], f, d);
                const float delta = d * g[c] * rv[c];
                dre[c] = fmaf(f, g[c], dre[c]);
                dsum[c] += delta;
                xcur[c] = fmaf(-rv[c], f, xcur[c]);  // x_it
                dwin[(it & 1) * TL::WIN + pl.own + c] = delta;
            }
            if (it == 0) {
                // D is complete: the weights of the taps that read the (frozen) halo.  Before this
                // iteration's barrier, so that nobody commits the next window while the halo is
                // read; behind a barrier of its own when the zeros of the halo window were
                // written in the iteration just before (inner == 1).
                if (inner == 1) lds_barrier();
                for_each_row<TL, CPT, kChainDepth>(xhalo + pl.row00, [&](int r, const float (&xv)[CPT + 2]) {
#pragma unroll
                    for (int cc = 0; cc < 3; ++cc)
#pragma unroll
                        for (int c = 0; c < CPT; ++c)
                            nw[r * 3 + cc][c] = fmaf(xv[c + cc], dsum[c], nw[r * 3 + cc][c]);
                });
                if (DEFER) {  // the normalised input at this thread's shell entries
                    const unsigned at2 = tab(kTabShellAt);
                    nh[0] = xhalo[at2 & 0xffffu];
                    nh[1] = xhalo[at2 >> 16];
                }
            }
            lds_barrier();
            for_each_row<TL, CPT, kChainDepth>(dwin + (it & 1) * TL::WIN + pl.row00,
                                               [&](int r, const float (&dv)[CPT + 2]) {
#pragma unroll
                for (int cc = 0; cc < 3; ++cc)
#pragma unroll
                    for (int c = 0; c < CPT; ++c) {
                        nw[r * 3 + cc][c] = fmaf(xcur[c], dv[c + cc], nw[r * 3 + cc][c]);
                        g[c] = fmaf(v[r * 3 + cc][c], dv[c + cc], g[c]);
                    }
            });
        }
        // g: the block's own part of the input gradient; dsum: D (also this element's share of
        // dbias); xcur: x_0 as the forward saw it
#pragma unroll
        for (int c = 0; c < CPT; ++c) {
            acc_ref(c) += dsum[c];
            acc_ref(2 + c) += dre[c];
        }

        if (DEFER) {
            // D into the delta window that the last gather did not read (its halo is zero); the own
            // cells' share of the two LayerNorm sums
#pragma unroll
            for (int c = 0; c < CPT; ++c) dwin[TL::WIN + pl.own + c] = dsum[c];
            const float bet0 = __uint_as_float(tab(kTabBeta)), bet1 = __uint_as_float(tab(kTabBeta + 1));
            t1_done = fmaf(__uint_as_float(tab(kTabGamma)), g[0], __uint_as_float(tab(kTabGamma + 1)) * g[1]);
            t2_done = fmaf(g[0], xcur[0] - bet0, g[1] * (xcur[1] - bet1));
            nh_done[0] = nh[0];
            nh_done[1] = nh[1];
        } else {
            if (inner == 0) lds_barrier();
#pragma unroll
            for (int c = 0; c < CPT; ++c) o_done[c] = dsum[c];
        }
        done_s = s;
#pragma unroll
        for (int c = 0; c < CPT; ++c) g_done[c] = g[c];
        // the x windows are free (nothing reads them after the last barrier of the sweep)
        if (s + 1 < s1) commit_window();
    }
    store_done();
    unsigned shc[2];
    shell_sources(shc);
    lds_barrier();  // the last element's D
    shell_of_done(shc);
    lds_barrier();  // its sums
    shell_of_done(shc);

    // ---- parameter gradients ----
    const long slab_off = slab_offset();
#pragma unroll
    for (int c = 0; c < CPT; ++c) {
        db[c] = acc_ref(c);
        dr[c] = acc_ref(2 + c);
        dgam[c] = acc_ref(4 + c);
        dbet[c] = acc_ref(6 + c);
    }
    commit_grads<27, CPT>((a.dweight + slab_off), nw, a.param_mode, owner_of, always);
    float one[1][CPT];
    auto own_cell = [&](int, int c) { return pl.gc + c; };
#pragma unroll
    for (int c = 0; c < CPT; ++c) one[0][c] = db[c];
    commit_grads<1, CPT>((a.dbias + slab_off), one, a.param_mode, own_cell, always);
#pragma unroll
    for (int c = 0; c < CPT; ++c) one[0][c] = dr[c];
    commit_grads<1, CPT>((a.dscale + slab_off), one, a.param_mode, own_cell, always);
#pragma unroll
    for (int c = 0; c < CPT; ++c) one[0][c] = dgam[c];
    commit_grads<1, CPT>((a.dgamma + slab_off), one, a.param_mode, own_cell, always);
#pragma unroll
    for (int c = 0; c < CPT; ++c) one[0][c] = dbet[c];
    commit_grads<1, CPT>((a.dbeta + slab_off), one, a.param_mode, own_cell, always);
}

template <int ACT, bool DEFER> int launch_chain(const StepArgs &a, hipStream_t st) {
    auto kern = chain_bwd<ACT, DEFER>;
    const size_t lds = (size_t)chain_lds_floats(a.inner) * sizeof(float);
    static bool big_lds_enabled = false;           // per instantiation
    static int per_cu_cache[kChainMaxInner + 1];   // per instantiation, by inner iterations
    if (lds > 64 * 1024 && !big_lds_enabled) {
        hipError_t e = hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize,
                                           (int)((size_t)chain_lds_floats(kChainMaxInner) * sizeof(float)));
        if (e != hipSuccess)
            return fail(GRIDNET_ERR_LAUNCH, "cannot enable %zu bytes of LDS: %s", lds, hipGetErrorString(e));
        big_lds_enabled = true;
    }
    int &per_cu = per_cu_cache[a.inner];
    if (per_cu == 0) {
        int n = 0;
        if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, kern, 256, lds) != hipSuccess || n < 1) n = 1;
        per_cu = n;
    }
    const long cells = (long)a.M * a.N * a.K;
    ChainBwdArgs k{};
    k.nblk = (a.M / 8) * (a.N / 8) * (a.K / 8);
    // one workgroup owns the whole batch of its block as soon as the blocks alone give every CU
    // a workgroup: plain stores for the parameter gradients, bitwise reproducible
    const bool whole = k.nblk >= plan_device_cus();
    plan_batch_chunks(a.B, k.nblk, 1, per_cu * plan_device_cus(), whole, k.nchunk, k.chunk_len);
    const bool new_params = (a.flags & GRIDNET_OVERWRITE_PARAMS) != 0;
    // A split batch: every chunk gets a copy of the gradient arrays in the scratch; with less
    // room than chunks the batch is split less (down to not at all).
    const long slab_floats = kStepSlabPlanes * cells;
    if (k.nchunk > 1) {
        const int room = plan_split_room(plan_slab_capacity(a.slabs, a.slab_bytes, slab_floats), a.B, k.chunk_len);
        if (room < k.nchunk)
            plan_batch_chunks(a.B, k.nblk, 1, (room < 2 ? 1 : room) * k.nblk, room < 2, k.nchunk, k.chunk_len);
    }
    const bool split = k.nchunk > 1;
    k.param_mode = split || new_params ? kParamStore : kParamAddExclusive;
    k.slab_stride = split ? slab_floats : 0;
    float *slab = (float *)a.slabs;
    k.weight = (const float *)a.weight; k.bias = (const float *)a.bias; k.scale = (const float *)a.scale;
    k.gamma = a.ln.gamma; k.beta = a.ln.beta;
    k.x = (const float *)a.x; k.x_stats = a.ln.x_stats;
    k.dy = (const float *)a.dy; k.y_raw = a.ln.y_raw; k.y_stats = a.ln.y_stats; k.y_sums = a.ln.y_sums;
    k.halo_in = a.ln.halo_in;
    k.dweight = split ? slab : (float *)a.dweight;
    k.dbias = split ? slab + 27 * cells : (float *)a.dbias;
    k.dscale = split ? slab + 28 * cells : (float *)a.dscale;
    k.dgamma = split ? slab + 29 * cells : a.ln.dgamma;
    k.dbeta = split ? slab + 30 * cells : a.ln.dbeta;
    k.dx = (float *)a.dx;
    k.out2 = DEFER ? a.ln.halo_out : (float *)a.workspace;
    k.x_part = a.ln.x_part;
    k.B = a.B; k.M = a.M; k.N = a.N; k.K = a.K; k.inner = a.inner;
    hipLaunchKernelGGL(kern, dim3(padded_grid(k.nblk, k.nchunk)), dim3(256), lds, st, k);
    if (int rc = check_launch("chain_bwd")) return rc;
    if (split) {
        SlabTargets t{};
        t.dst[0] = (float *)a.dweight; t.end[0] = 27 * cells;
        t.dst[1] = (float *)a.dbias;   t.end[1] = 28 * cells;
        t.dst[2] = (float *)a.dscale;  t.end[2] = 29 * cells;
        t.dst[3] = a.ln.dgamma;        t.end[3] = 30 * cells;
        t.dst[4] = a.ln.dbeta;         t.end[4] = 31 * cells;
        t.count = 5;
        if (int rc = plan_reduce_slabs(slab, k.nchunk, slab_floats, t, new_params ? 0 : 1, st)) return rc;
    }
    if (DEFER) return GRIDNET_OK;
    // dx is wanted finished: the cross-block kernel completes it from D (same blocks, same chunks)
    return step_cross_launch(a, k.nchunk, k.chunk_len, st);
}

template <int ACT> int dispatch_defer(const StepArgs &a, hipStream_t st) {
    return a.ln.halo_out ? launch_chain<ACT, true>(a, st) : launch_chain<ACT, false>(a, st);
}

}  // namespace

bool chain_supports(const StepArgs &a) {
    return a.dtype == GRIDNET_F32 && a.block_size == 8 && !a.normalize && a.inner >= 1 &&
           a.inner <= kChainMaxInner;
}

size_t chain_halo_floats(const StepArgs &a) {
    return (size_t)a.B * (a.M / 8) * (a.N / 8) * (a.K / 8) * kShell;
}

int chain_backward(const StepArgs &a, hipStream_t st) {
    if (!chain_supports(a))
        return fail(GRIDNET_ERR_ARGUMENT, "the chain backward covers 1 to %d inner iterations, got %d",
                    kChainMaxInner, a.inner);
    switch (a.activation) {
        case GRIDNET_ACT_RELU: return dispatch_defer<GRIDNET_ACT_RELU>(a, st);
        case GRIDNET_ACT_LEAKY_RELU: return dispatch_defer<GRIDNET_ACT_LEAKY_RELU>(a, st);
        case GRIDNET_ACT_SILU: return dispatch_defer<GRIDNET_ACT_SILU>(a, st);
        case GRIDNET_ACT_TANH: return dispatch_defer<GRIDNET_ACT_TANH>(a, st);
    }
    return fail(GRIDNET_ERR_ACTIVATION, "unknown activation function: id %d", a.activation);
}

}  // namespace gridnet
