// Backward of one step of the network body "update step, then per-sample LayerNorm" inside a
// CHAIN of such steps: 8^3 blocks, fp32, normalize off, up to 8 inner iterations.
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
constexpr int kChainMaxInner = 8;  // the pre-activations of more iterations do not fit: two workgroups
                                    // share the 160 KB of a CU
constexpr int kChainNarrowInner = 4;  // up to here the table below has its full 24 rows
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
    // ---- ALL: every step of the chain in one launch (see chain_bwd) ----
    // y_raw and y_stats then point at step 0's and the steps lie step_floats / 2 B floats apart;
    // dy is the gradient handed to the last step; x, x_stats, y_sums, halo_in, dx, out2 are unused.
    const float *x0;           // input of step 0 (no LayerNorm in front of it)
    float *sums;               // [steps * B][2] by item: the LayerNorm sums an item asks for; those of
                               // the last step's items are given, the others are formed here
    float *dx_even, *dx_odd;      // step j leaves the block-local part of its input gradient in the one of its parity
    float *halo_even, *halo_odd;  // ... and what crosses block boundaries
    unsigned *status;          // one word, zero on entry: set when a bounded wait ran out
    unsigned *arrive, *ready;  // by item, (steps - 1) * B each, zero on entry
    int steps, spin_limit;     // spin_limit < 0: never publish (the give-up path under test), limit = -spin_limit
    long step_floats;          // floats between y_raw of consecutive steps
};

// Coherent accesses for data that workgroups on other XCDs write or read WHILE THE KERNEL RUNS:
// relaxed atomics at agent scope compile to loads and stores that bypass the XCD-private L2
// (write-through stores, loads that do not hit a stale line); plain accesses only see other
// XCDs' writes across a kernel boundary.
template <typename T> __device__ __forceinline__ T ld_agent(const T *p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
template <typename T> __device__ __forceinline__ void st_agent(T *p, T v) {
    __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ float2 ld_agent2(const float *p) {
    const unsigned long long u = ld_agent(reinterpret_cast<const unsigned long long *>(p));
    return make_float2(__uint_as_float((unsigned)u), __uint_as_float((unsigned)(u >> 32)));
}
// the same word for every lane, loaded as a vector load (see load_ahead)
template <typename T> __device__ __forceinline__ T ld_agent_uniform(const T *p) {
    int zero;
    asm volatile("v_mov_b32 %0, 0" : "=v"(zero));
    return ld_agent(p + zero);
}

// LDS (floats): [x window x2 | delta window x2 | u_i of the owned cells, inner slabs of 512 |
// gamma, beta of the window, packed | sums of the four waves | weights of the shell entries
// [9][512] | per-thread constants [rows][256]]; at set-up the block's 27 weight planes pass
// through the front of it.
using ChainTile = Tile<8, 2>;
// Table entries.  Small integers are packed (the table is the difference between two workgroups
// per CU and one): In = the seven record offsets of what the thread's cells receive, three 10-bit
// float indices per word; ShellAt = both shell entries' places in the x window, 16 bits each;
// Halo = per shell entry the window offset of its centre source (bits 0-11) and the codes of its
// two strides (bits 12-13, 14-15: 0 -> 1, 1 -> row, 2 -> plane).
// WIDE (5 to 8 inner iterations): the history of pre-activations needs the room of eight table
// rows.  gamma and beta of the owned cells and of the shell entries then come out of the packed
// gamma/beta window (which holds them anyway: the shell entries are the window's halo) through
// two rows of offsets, OwnAff and ShellAff (per shell entry 15 bits of offset and a flag: the
// entry is a row's end entry, whose beta sits 1 float behind its gamma instead of 4), and the
// pre-activations of the last iteration, which the sweep uses first, stay in registers.
template <bool WIDE> struct ChainTab {
    static constexpr int Dst = 0, In = 2, ShellAt = 5, Halo = 6;
    static constexpr int ShellGamma = 8, ShellBeta = 10, Beta = 12, Gamma = 14;  // narrow only
    static constexpr int OwnAff = 8, ShellAff = 9;                               // WIDE only
    static constexpr int Acc = WIDE ? 10 : 16;  // 8 gradient sums
    static constexpr int Rows = WIDE ? 18 : 24;
};
constexpr int kChainAffine = 200 * Fetch<ChainTile>::GB;  // packed gamma/beta: 200 half rows
__host__ __device__ constexpr int chain_lds_floats(int inner) {
    const bool wide = inner > kChainNarrowInner;
    const int run = 4 * ChainTile::WIN + (wide ? inner - 1 : inner) * 512 + kChainAffine + 16 + 9 * 512 +
                    (wide ? ChainTab<true>::Rows : ChainTab<false>::Rows) * 256;
    return run > 27 * 512 ? run : 27 * 512;
}
static_assert(chain_lds_floats(kChainMaxInner) * 4 * 2 <= 160 * 1024, "two workgroups share a CU's LDS");
__device__ __forceinline__ int stride_of(unsigned code) {
    return code == 0 ? 1 : code == 1 ? ChainTile::RS : ChainTile::PS;
}

// ALL: one launch walks every step of the chain, last to first.  A workgroup keeps its block for the
// whole chain: the weights, the mirrored weights, the tables and -- with one parameter set shared
// by the steps -- the gradient accumulators stay where they are from step to step (no set-up,
// no drain, no read-modify-write of the gradient arrays per step), and nobody waits for the
// slowest workgroup of a step.  The workgroups must all be resident (cooperative launch).
// What step j-1 needs of step j for batch element s -- the values its neighbours' blocks send
// across the block boundaries and the two per-sample sums of the LayerNorm between the steps,
// which every block contributes to -- travels through memory behind a counter per (step,
// element): a workgroup adds 1 once its stores for the pair have been acknowledged.  Pair number m
// has a workgroup in charge, m modulo the number of workgroups -- NOT the last one to arrive: that
// is the slowest workgroup of the moment every time, and the extra work would keep it the
// slowest (measured: one workgroup fell 25 % behind and the whole grid followed at its pace).
// The one in charge looks at the counter once per iteration; when it reads the number of blocks
// it sums the blocks' shares in block order (always the same bits), stores the two means and
// then sets the pair's ready word.
// A workgroup looks at that word before it requests the pair's data for step j-1.  By then the
// pair is a whole batch old, so the look normally costs nothing: the word is requested an
// element ahead, together with the window.  Waits are bounded: a wave that runs out of tries
// sets the status word and stops waiting for good (results are then invalid, the host falls
// back to one launch per step), so every workgroup reaches the end whatever happens.
template <int ACT, bool DEFER, bool ALL = false, bool WIDE = false>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2)))
void chain_bwd(const ChainBwdArgs a) {
    static_assert(DEFER || !ALL, "inside one launch every step hands its halo values on");
    using TL = ChainTile;
    using TB = ChainTab<WIDE>;
    constexpr int kTabDst = TB::Dst, kTabIn = TB::In, kTabShellAt = TB::ShellAt, kTabHalo = TB::Halo,
                  kTabShellGamma = TB::ShellGamma, kTabShellBeta = TB::ShellBeta, kTabBeta = TB::Beta,
                  kTabGamma = TB::Gamma, kTabAcc = TB::Acc;
    constexpr int BS = 8, CPT = 2, NC = BS * BS * BS;
    extern __shared__ __attribute__((aligned(16))) float lds[];
    const int inner = a.inner;
    float *win = lds;                          // two copies of the x window
    float *dwin = win + 2 * TL::WIN;           // two delta windows, halo zero
    float *hist = dwin + 2 * TL::WIN;          // u_i of this thread's cells at hist + it * 512 + lane * 2
    float *affine = hist + (WIDE ? inner - 1 : inner) * 512;  // gamma and beta of the window, packed per half row
    float *red = affine + kChainAffine;   // [2][4][2], per wave: the two LayerNorm sums of an element, elements alternating
    float *hwl = red + 16;                     // [256][18]: the weights that feed the shell entries
    // ... and what a thread uses once per element: [rows][256], entry k of thread t at
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
    const bool ln_in = ALL || a.x_stats != nullptr;  // ALL: every step but the first
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
        unsigned s_dst[2], s_at[2], s_aff[2];
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
            {   // ... and in the packed gamma/beta window: an end entry of its row, or one of its cells
                const bool is_end = wk == 0 || wk == TL::S - 1;
                const int half_row = (wi * TL::S + wj) * 2 + (wk >= TL::S / 2 ? 1 : 0);
                s_aff[e] = (unsigned)(half_row * Fetch<TL>::GB + (is_end ? 2 * Fetch<TL>::HC : (wk - 1) % Fetch<TL>::HC)) |
                           (is_end ? 1u << 15 : 0u);
            }
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
        if (!WIDE) {
            tab(kTabGamma) = __float_as_uint(gam[0]);
            tab(kTabGamma + 1) = __float_as_uint(gam[1]);
        } else {
            // where the packed window keeps gamma of the thread's two cells (beta: 4 floats on)
            const int half_row = ((pl.i + 1) * TL::S + pl.j + 1) * 2 + (pl.kt >> 1);
            tab(TB::OwnAff) = (unsigned)(half_row * Fetch<TL>::GB + (pl.kt & 1) * 2);
        }
        if (DEFER) {
#pragma unroll
            for (int e = 0; e < 2; ++e) {
#pragma unroll
                for (int slot = 0; slot < 9; ++slot) hwl[tid * 18 + e * 9 + slot] = hw[e][slot];
                tab(kTabDst + e) = s_dst[e];
                if (!WIDE) {
                    tab(kTabShellGamma + e) = __float_as_uint(hgam[e]);
                    tab(kTabShellBeta + e) = __float_as_uint(hbet[e]);
                }
            }
            tab(kTabShellAt) = s_at[0] | s_at[1] << 16;
            if (!WIDE) {
                float bet[CPT];
                load_cells<CPT>(a.beta + pl.gc, bet);
                tab(kTabBeta) = __float_as_uint(bet[0]);
                tab(kTabBeta + 1) = __float_as_uint(bet[1]);
            } else {
                tab(TB::ShellAff) = s_aff[0] | s_aff[1] << 16;
            }
        }
    }

    // ---- what this thread's cells receive from the blocks around: where, and whether ----
    const int fi = pl.i == 0 ? 0 : pl.i == BS - 1 ? 1 : -1, fj = pl.j == 0 ? 0 : pl.j == BS - 1 ? 1 : -1,
              fk = pl.kt == 0 ? 0 : pl.kt == TL::KT - 1 ? 1 : -1;
    const bool have_in = ALL || a.halo_in != nullptr;  // ALL: every step but the last, see the loop
    const bool ei0 = have_in && (fi == 0 ? bi > 0 : fi == 1 ? bi < mb - 1 : false);
    const bool ej0 = have_in && (fj == 0 ? bj > 0 : fj == 1 ? bj < nb - 1 : false);
    const bool ek0 = have_in && (fk == 0 ? bk > 0 : fk == 1 ? bk < kb - 1 : false);
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
    const float *hin = ALL ? nullptr : have_in ? a.halo_in : a.dy;
    const float *xst = ALL ? nullptr : ln_in ? a.x_stats : a.y_stats;
    const unsigned ugc = 4u * pl.gc;  // byte offset of the owned cells within a sample

    typename Fetch<TL>::Buf pre;
    if (ln_in || WIDE) {  // gamma and beta of the window, once per workgroup
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

    const int s0 = ALL ? 0 : chunk * a.chunk_len, s1 = ALL ? a.B : min(a.B, s0 + a.chunk_len);
    // ALL: the walk is last step first, the elements of a step in order: item n is element n % B of
    // step steps - 1 - n / B.  Counters, ready words and LayerNorm sums are numbered by item.  What
    // depends on the step alone is kept in (scalar) variables that change once per step.
    const int items = ALL ? a.steps * a.B : s1 - s0;
    const int counted = ALL ? (a.steps - 1) * a.B : 0;  // the items of every step but the first hand something on
    const float *c_dy = a.dy, *c_rec = hin, *c_yr = a.y_raw, *c_ystat = a.y_stats;  // the element's gradient,
                                                       // what the blocks around left for it, its raw output
    const float *c_x = a.x, *c_xst = xst;              // the step's input and its statistics
    float *c_dxo = a.dx, *c_halo = a.out2;             // where the step leaves dx and its halo values
    bool c_later = true, c_ln = ln_in;                 // a later step exists; the input passes a LayerNorm
    auto enter_step = [&](int jj) {
        const bool odd = (jj & 1) != 0;
        c_later = jj < a.steps - 1;
        c_dy = c_later ? (odd ? a.dx_even : a.dx_odd) : a.dy;
        c_rec = c_later ? (odd ? a.halo_even : a.halo_odd) : a.dy;  // no later step: every flag is off
        c_yr = a.y_raw + jj * a.step_floats;
        c_ystat = a.y_stats + (long)jj * 2 * a.B;
        c_ln = jj > 0;
        c_x = c_ln ? a.y_raw + (jj - 1) * a.step_floats : a.x0;
        c_xst = a.y_stats + (long)(c_ln ? jj - 1 : 0) * 2 * a.B;
        c_dxo = odd ? a.dx_odd : a.dx_even;
        c_halo = odd ? a.halo_odd : a.halo_even;
    };
    float nxm = 0.f, nxr = 1.f;  // LayerNorm statistics of the element in `pre`
    bool nx_ln = ln_in;          // ... and whether it passes a LayerNorm on the way in
    auto fetch_window = [&](const float *xs, const float *st, bool ln, int s) {
        nx_ln = ln;
        fx.fetch(xs + (long)s * cells, pre);
        nxm = load_ahead(st, 2 * s);
        nxr = load_ahead(st, 2 * s + 1);
    };
    auto commit_window = [&]() {
        if (nx_ln) fx.commit_ln(win, pre, affine, nxm, nxr);
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
    // ALL: where the step of the finished element leaves its results
    float *d_dxo = a.dx, *d_halo = a.out2;
    auto store_done = [&]() {
        if (done_s < 0) return;
        const long o = (long)done_s * cells;
        at_bytes<float2>(d_dxo + o, ugc) = make_float2(g_done[0], g_done[1]);
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
    // behind a barrier that follows the element's last write of D; `n`: the iteration (ALL: the
    // finished element is item n - 1, the one whose sums are complete item n - 2)
    auto shell_of_done = [&](const unsigned (&hals)[2], int n) {
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
            float *rec = d_halo + (long)hs * a.nblk * kShell;
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
                float gam_at, bet_at;  // gamma and beta at the cell that receives the value
                if (WIDE) {
                    const unsigned code = (tab(TB::ShellAff) >> (16 * e)) & 0xffffu;
                    const float *at = affine + (code & 0x7fffu);
                    gam_at = at[0];
                    bet_at = (code >> 15) ? at[1] : at[Fetch<TL>::HC];
                } else {
                    gam_at = __uint_as_float(tab(kTabShellGamma + e));
                    bet_at = __uint_as_float(tab(kTabShellBeta + e));
                }
                t1 = fmaf(gam_at, acc, t1);
                t2 = fmaf(acc, nh_done[e] - bet_at, t2);
                if (s_in[e]) {
                    // opaque here, so that the offset is widened inside this block, where the
                    // store can still take it as a 32-bit lane offset beside the scalar base
                    unsigned off = tab(kTabDst + e);
                    asm volatile("" : "+v"(off));
                    if (ALL) st_agent(&at_bytes<float>(rec, off), acc);
                    else at_bytes<float>(rec, off) = acc;
                }
            }
            t1 = slot_wave_sum<256>(t1);
            t2 = slot_wave_sum<256>(t2);
            // the two halves of `red` alternate by element; ALL: by iteration (a step may have an odd
            // number of elements)
            if ((tid & 63) == 0)
                *reinterpret_cast<float2 *>(red + ((ALL ? n + 1 : hs) & 1) * 8 + 2 * (tid >> 6)) = make_float2(t1, t2);
        }
        // the sums of the element before that one: its four waves' shares, in a fixed order (they
        // were written a barrier ago, into the other half of `red`)
        if (DEFER && sums_s >= 0 && tid == 0 && (!ALL || n - 2 < counted)) {
            const float *r = red + ((ALL ? n : sums_s) & 1) * 8;
            float *to = a.x_part + ((long)sums_s * a.nblk + blk) * 2;
            const float p0 = (r[0] + r[2]) + (r[4] + r[6]), p1 = (r[1] + r[3]) + (r[5] + r[7]);
            if (ALL) {
                st_agent(to, p0);
                st_agent(to + 1, p1);
            } else {
                to[0] = p0;
                to[1] = p1;
            }
        }
        sums_s = hs;
        done_s = -1;
    };

    if (ln_in || WIDE) lds_barrier();  // the packed gamma and beta
    // ALL: `ready_word` is the ready word of the item at hand's counterpart in the step after
    // (item n - B), requested while the element before was worked on.  `duty` is the next item this
    // workgroup is in charge of (blk, blk + nblk, ...), `duty_count` what its counter read an
    // iteration ago (0: not asked yet).
    int j = ALL ? a.steps - 1 : 0, s = s0;
    unsigned ready_word = 1u, duty_count = 0u;
    int duty = blk;
    bool gave_up = false;
    // The workgroup in charge of item m (element fs of its step), once every block has counted
    // itself in: the blocks' shares become the two means of the LayerNorm backward in front of that
    // step (wave 0, block order, in double: always the same bits) -- the sums that item m + B will
    // ask for -- and, once those are in memory, the item's ready word is set.
    auto finalize = [&](int m) {
        const int fs = m % a.B;
        const float *part = a.x_part + (long)fs * a.nblk * 2;
        double t1 = 0.0, t2 = 0.0;
        for (int i0 = 0; i0 < a.nblk; i0 += 512) {
            float2 v[8];
#pragma unroll
            for (int q = 0; q < 8; ++q) v[q] = ld_agent2(part + 2 * min(i0 + q * 64 + tid, a.nblk - 1));
#pragma unroll
            for (int q = 0; q < 8; ++q)
                if (i0 + q * 64 + tid < a.nblk) {
                    t1 += (double)v[q].x;
                    t2 += (double)v[q].y;
                }
        }
        t1 = wave_sum(t1);
        t2 = wave_sum(t2);
        if (tid == 0) {
            float *to = a.sums + 2 * (long)(m + a.B);
            st_agent(to, (float)(t1 / (double)cells));
            st_agent(to + 1, (float)(t2 / (double)cells));
        }
        wait_global_loads();  // ... and stores: the two means have been acknowledged
        if (tid == 0 && a.spin_limit >= 0) st_agent(a.ready + m, 1u);
    };
    // Wave 0: the item in charge of is complete when its counter reads the number of blocks.
    auto do_duty = [&](unsigned count) {
        if (duty < counted && __builtin_amdgcn_readfirstlane(count) == (unsigned)a.nblk) {
            finalize(duty);
            duty += a.nblk;
        }
    };
    // A bounded wait for a ready word (one wave; the loop runs on the scalar unit).  Wave 0 keeps
    // looking after the item it is in charge of meanwhile: the word it waits for may be that very one.
    auto wait_ready = [&](const unsigned *word, unsigned seen) {
        unsigned v = __builtin_amdgcn_readfirstlane(seen);
        const int limit = a.spin_limit < 0 ? -a.spin_limit : a.spin_limit;
        int spins = 0;
        while (v == 0u && !gave_up) {
            __builtin_amdgcn_s_sleep(16);
            if (tid < 64 && duty < counted) do_duty(ld_agent_uniform(a.arrive + duty));
            v = __builtin_amdgcn_readfirstlane(ld_agent_uniform(word));
            if (v == 0u && (++spins > limit || __builtin_amdgcn_readfirstlane(ld_agent_uniform(a.status)) != 0u)) {
                gave_up = true;
                if ((tid & 63) == 0) st_agent(a.status, 1u);
            }
        }
    };
    if (ALL) enter_step(j);
    if (items > 0) {
        fetch_window(c_x, c_xst, c_ln, s0);
        commit_window();
    }
    for (int n = 0; n < items; ++n) {
        take_turns(ALL ? n : s);
        if (ALL) {
            // the walk's counters are the same for every lane; said here, where the loop's joins
            // (one wave finalizes, one thread counts in) would otherwise make the compiler keep
            // them, and every address built on them, in vector registers
            j = __builtin_amdgcn_readfirstlane(j);
            s = __builtin_amdgcn_readfirstlane(s);
            // Everything this wave has stored so far was issued an iteration ago or earlier; once it
            // is acknowledged, the barrier below lets thread 0 count the workgroup in for the item
            // those stores complete.
            wait_global_loads();
            if (tid < 64) do_duty(duty_count);
            if (n >= a.B) wait_ready(a.ready + (n - a.B), ready_word);
        }
        // Requests first, stores behind them: loads and stores retire through one in-order
        // counter, and no wait for a load may include the stores.  This element's gradient (used
        // after the recompute, which hides the trip), then the next element's window.  All of it
        // in front of the barrier: none of it touches the windows, and the wait for the other
        // waves covers the issue.
        const long at = (long)s * cells;
        // ALL: with a later step, its workgroups left this element's gradient (this workgroup its
        // own cells' part, the neighbours the rest)
        const bool ei = ALL ? c_later && ei0 : ei0, ej = ALL ? c_later && ej0 : ej0, ek = ALL ? c_later && ek0 : ek0;
        const float2 dy2 = at_bytes<float2>(c_dy + at, ugc), yr2 = at_bytes<float2>(c_yr + at, ugc);
        const float *rec = c_rec + ((long)s * a.nblk + blk) * kShell;
        const unsigned oa = tab(kTabIn), ob = tab(kTabIn + 1), oc = tab(kTabIn + 2);
        auto off10 = [](unsigned word, int k) { return 4u * ((word >> (10 * k)) & 1023u); };
        constexpr bool COH = ALL;
        auto in2 = [&](unsigned off) { return COH ? ld_agent2(&at_bytes<float>(rec, off)) : at_bytes<float2>(rec, off); };
        auto in1 = [&](unsigned off) { return COH ? ld_agent(&at_bytes<float>(rec, off)) : at_bytes<float>(rec, off); };
        const float2 in_i = in2(off10(oa, 0)), in_j = in2(off10(oa, 1)), in_ij = in2(off10(oa, 2));
        const float in_k = in1(off10(ob, 0)), in_ik = in1(off10(ob, 1)), in_jk = in1(off10(ob, 2)),
                    in_c = in1(off10(oc, 0));
        const float ny0 = load_ahead(c_ystat, 2 * s), ny1 = load_ahead(c_ystat, 2 * s + 1),
                    ny2 = ALL ? ld_agent_uniform(a.sums + 2 * n) : load_ahead(a.y_sums, 2 * s),
                    ny3 = ALL ? ld_agent_uniform(a.sums + 2 * n + 1) : load_ahead(a.y_sums, 2 * s + 1);
        // the element after this one: the next of the step, or the first of the step before
        int s2 = ALL ? s + 1 : min(s + 1, s1 - 1);
        bool wrap = false;
        if (ALL) {
            if (n + 1 == items) s2 = s;
            else if (s2 == a.B) {
                s2 = 0;
                wrap = true;
            }
        }
        if (ALL && wrap) {  // once per step
            const bool ln2 = j > 1;
            fetch_window(ln2 ? a.y_raw + (j - 2) * a.step_floats : a.x0, a.y_stats + (long)(ln2 ? j - 2 : 0) * 2 * a.B,
                         ln2, 0);
        } else {
            fetch_window(c_x, c_xst, c_ln, s2);
        }
        if (ALL) {
            ready_word = (n + 1 >= a.B && n + 1 < items) ? ld_agent_uniform(a.ready + (n + 1 - a.B)) : 1u;
            // the item in charge of: this workgroup itself counts in for item m in iteration m + 3
            duty_count = (tid < 64 && duty < counted && duty + 3 <= n) ? ld_agent_uniform(a.arrive + duty) : 0u;
        }
        store_done();
        unsigned shc[2];
        shell_sources(shc);
        lds_barrier();  // this element's window is in place; the last round's LDS readers are done
        if (ALL && n >= 3 && n - 3 < counted) {
            // Item n - 3 is counted in: every wave has seen its stores for it acknowledged (halo
            // values two iterations ago, the LayerNorm shares one), and the barrier has gathered the
            // waves.  (This file is compiled with the compiler's rewrite of uniform atomics switched
            // off: it turns the add into a wave-wide reduction with a returned count that it waits
            // for at once, and with it for every request issued above.)
            if (tid == 0)
                (void)__hip_atomic_fetch_add(a.arrive + (n - 3), 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        shell_of_done(shc, n);

        // ---- forward recompute; u_i of the owned cells is remembered ----
        float xcur[CPT], u_last[CPT] = {0.f, 0.f};  // WIDE: the last iteration's pre-activations
#pragma unroll
        for (int c = 0; c < CPT; ++c) xcur[c] = win[pl.own + c];
        for (int it = 0; it < inner; ++it) {
            float u[CPT];
            stencil<TL, CPT, kChainDepth>(win + (it & 1) * TL::WIN, pl.row00, w, bv, u);
            if (!WIDE || it + 1 < inner) store_cells<CPT>(hist + it * 512 + tid * CPT, u);
            if (WIDE) {
#pragma unroll
                for (int c = 0; c < CPT; ++c) u_last[c] = u[c];
            }
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
            float gm[CPT];
            if (WIDE) {
                const float2 g2 = *reinterpret_cast<const float2 *>(affine + tab(TB::OwnAff));
                gm[0] = g2.x;
                gm[1] = g2.y;
            } else {
                gm[0] = __uint_as_float(tab(kTabGamma));
                gm[1] = __uint_as_float(tab(kTabGamma + 1));
            }
#pragma unroll
            for (int c = 0; c < CPT; ++c) {
                const float yh = (yr[c] - ny0) * ny1;
                acc_ref(4 + c) = fmaf(tot[c], yh, acc_ref(4 + c));
                acc_ref(6 + c) += tot[c];
                g[c] = ny1 * (gm[c] * tot[c] - ny2 - yh * ny3);
                dsum[c] = 0.f;
            }
        }

        // ---- reverse sweep: delta window copy (it & 1) holds delta_it; xcur walks back from
        // x_inner to x_0 ----
        float nh[2] = {0.f, 0.f}, dre[CPT] = {0.f, 0.f};
        for (int it = inner - 1; it >= 0; --it) {
            float u[CPT];
            if (WIDE && it == inner - 1) {
#pragma unroll
                for (int c = 0; c < CPT; ++c) u[c] = u_last[c];
            } else {
                load_cells<CPT>(hist + it * 512 + tid * CPT, u);
            }
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
            float bet0, bet1, gam0, gam1;
            if (WIDE) {
                const float *at = affine + tab(TB::OwnAff);
                const float2 g2 = *reinterpret_cast<const float2 *>(at);
                const float2 b2 = *reinterpret_cast<const float2 *>(at + Fetch<TL>::HC);
                gam0 = g2.x; gam1 = g2.y; bet0 = b2.x; bet1 = b2.y;
            } else {
                bet0 = __uint_as_float(tab(kTabBeta));
                bet1 = __uint_as_float(tab(kTabBeta + 1));
                gam0 = __uint_as_float(tab(kTabGamma));
                gam1 = __uint_as_float(tab(kTabGamma + 1));
            }
            t1_done = fmaf(gam0, g[0], gam1 * g[1]);
            t2_done = fmaf(g[0], xcur[0] - bet0, g[1] * (xcur[1] - bet1));
            nh_done[0] = nh[0];
            nh_done[1] = nh[1];
        } else {
            if (inner == 0) lds_barrier();
#pragma unroll
            for (int c = 0; c < CPT; ++c) o_done[c] = dsum[c];
        }
        done_s = s;
        if (ALL) {
            d_dxo = c_dxo;
            d_halo = c_halo;
        }
#pragma unroll
        for (int c = 0; c < CPT; ++c) g_done[c] = g[c];
        // the x windows are free (nothing reads them after the last barrier of the sweep)
        if (n + 1 < items) commit_window();
        if (ALL && wrap) enter_step(--j);
        s = ALL ? s2 : s + 1;
    }
    store_done();
    unsigned shc[2];
    shell_sources(shc);
    lds_barrier();  // the last element's D
    shell_of_done(shc, items);
    lds_barrier();  // its sums
    shell_of_done(shc, items + 1);

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

template <int ACT, bool DEFER, bool WIDE> int launch_chain(const StepArgs &a, hipStream_t st) {
    auto kern = chain_bwd<ACT, DEFER, false, WIDE>;
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

// What the first step of a one-launch chain leaves in its records is added to dx here: the
// chain's input gradient is wanted finished.  Same adds in the same order as chain_bwd makes
// them for the steps inside the chain.  A workgroup takes one element and a ROW of blocks along
// K (up to kGatherRow of them at a time): their records lie side by side in memory and the dx
// rows they cover are whole, so every access is a run of 256 bytes and more (one workgroup per
// block reads and writes 32-byte pieces 16 KB apart: 43 us instead of these for 64^3 / batch 32).
constexpr int kGatherRow = 8;
__global__ __launch_bounds__(256) void chain_halo_gather(float *__restrict__ dx, const float *__restrict__ halo,
                                                         int M, int N, int K, int nblk) {
    constexpr int BS = 8;
    __shared__ __attribute__((aligned(16))) float rec[kGatherRow * kShell];
    const int kb = K / BS, nb = N / BS, mb = M / BS;
    const int bi = blockIdx.x / nb, bj = blockIdx.x % nb, s = blockIdx.y, tid = threadIdx.x;
    float *dxs = dx + (long)s * M * N * K;
    for (int bk0 = 0; bk0 < kb; bk0 += kGatherRow) {
        const int nrow = min(kGatherRow, kb - bk0), blk0 = (bi * nb + bj) * kb + bk0;
        const float2 *from = reinterpret_cast<const float2 *>(halo + ((long)s * nblk + blk0) * kShell);
        __syncthreads();  // the last round's readers are done
        for (int q = tid; q < nrow * kShell / 2; q += 256) *reinterpret_cast<float2 *>(rec + 2 * q) = from[q];
        __syncthreads();
        const int pairs_per_row = nrow * BS / 2;
        for (int p = tid; p < BS * BS * pairs_per_row; p += 256) {
            const int kk = (p % pairs_per_row) * 2, row = p / pairs_per_row, i = row / BS, j = row % BS;
            const int bk = bk0 + kk / BS, k2 = kk % BS;
            const int fi = i == 0 ? 0 : i == BS - 1 ? 1 : -1, fj = j == 0 ? 0 : j == BS - 1 ? 1 : -1,
                      fk = k2 == 0 ? 0 : k2 == BS - 2 ? 1 : -1;
            const bool ei = fi == 0 ? bi > 0 : fi == 1 ? bi < mb - 1 : false;
            const bool ej = fj == 0 ? bj > 0 : fj == 1 ? bj < nb - 1 : false;
            const bool ek = fk == 0 ? bk > 0 : fk == 1 ? bk < kb - 1 : false;
            if (!(ei || ej || ek)) continue;
            const int zi = max(fi, 0), zj = max(fj, 0), zk = max(fk, 0);
            const float *r = rec + (kk / BS) * kShell;
            float2 *at = reinterpret_cast<float2 *>(dxs + ((long)(bi * BS + i) * N + bj * BS + j) * K + bk0 * BS + kk);
            float2 t = *at;
            auto pair_at = [&](int off) { return *reinterpret_cast<const float2 *>(r + off); };
            if (ei) { const float2 v = pair_at(kSegI + zi * 64 + j * 8 + k2); t.x += v.x; t.y += v.y; }
            if (ej) { const float2 v = pair_at(kSegJ + zj * 64 + i * 8 + k2); t.x += v.x; t.y += v.y; }
            if (ei && ej) { const float2 v = pair_at(kSegIJ + (zi * 2 + zj) * 8 + k2); t.x += v.x; t.y += v.y; }
            float ends = 0.f;
            if (ek) ends += r[kSegK + zk * 64 + i * 8 + j];
            if (ei && ek) ends += r[kSegIK + (zi * 2 + zk) * 8 + j];
            if (ej && ek) ends += r[kSegJK + (zj * 2 + zk) * 8 + i];
            if (ei && ej && ek) ends += r[kSegC + zi * 4 + zj * 2 + zk];
            t.x += fk == 0 ? ends : 0.f;
            t.y += fk == 1 ? ends : 0.f;
            *at = t;
        }
    }
}

// ---- the whole chain in one launch -----------------------------------------------------------
// workspace: [status word, counters, ready words | LayerNorm sums by item | LayerNorm shares of the
// blocks | two halo buffers | the second dx buffer | scratch of the last LayerNorm's sums]
struct ChainAllLayout {
    size_t sync_words, sums_at, part_at, halo_at, halo_floats, dx_at, ln_at, total;
};
ChainAllLayout chain_all_layout(const ChainAll &c) {
    auto up = [](size_t v) { return (v + 255) / 256 * 256; };
    const size_t cells = (size_t)c.M * c.N * c.K, nblk = cells / 512;
    ChainAllLayout l{};
    l.sync_words = 64 + 2 * (size_t)c.outer * c.B;
    l.sums_at = up(l.sync_words * 4);
    l.part_at = up(l.sums_at + (size_t)c.outer * c.B * 2 * 4);
    l.halo_at = up(l.part_at + (size_t)c.B * nblk * 2 * 4);
    l.halo_floats = (size_t)c.B * nblk * kShell;
    l.dx_at = up(l.halo_at + 2 * l.halo_floats * 4);
    l.ln_at = up(l.dx_at + (size_t)c.B * cells * 4);
    l.total = l.ln_at + layernorm_workspace(GRIDNET_F32, c.B, (long)cells);
    return l;
}

template <int ACT, bool WIDE> int launch_chain_all(const ChainAll &c, hipStream_t st) {
    auto kern = chain_bwd<ACT, true, true, WIDE>;
    const size_t lds = (size_t)chain_lds_floats(c.inner) * sizeof(float);
    static bool big_lds_enabled = false;
    if (lds > 64 * 1024 && !big_lds_enabled) {
        hipError_t e = hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize,
                                           (int)((size_t)chain_lds_floats(kChainMaxInner) * sizeof(float)));
        if (e != hipSuccess)
            return fail(GRIDNET_ERR_LAUNCH, "cannot enable %zu bytes of LDS: %s", lds, hipGetErrorString(e));
        big_lds_enabled = true;
    }
    const long cells = (long)c.M * c.N * c.K;
    const ChainAllLayout l = chain_all_layout(c);
    char *ws = (char *)c.workspace;
    ChainBwdArgs k{};
    k.nblk = (int)(cells / 512);
    k.nchunk = 1;
    k.chunk_len = c.B;
    k.param_mode = (c.flags & GRIDNET_OVERWRITE_PARAMS) ? kParamStore : kParamAddExclusive;
    k.weight = c.weight; k.bias = c.bias; k.scale = c.scale; k.gamma = c.gamma; k.beta = c.beta;
    k.x0 = c.x0; k.y_raw = c.y_raw; k.y_stats = c.stats; k.sums = (float *)(ws + l.sums_at); k.dy = c.dy;
    k.dweight = c.dweight; k.dbias = c.dbias; k.dscale = c.dscale; k.dgamma = c.dgamma; k.dbeta = c.dbeta;
    k.x_part = (float *)(ws + l.part_at);
    k.halo_even = (float *)(ws + l.halo_at);
    k.halo_odd = k.halo_even + l.halo_floats;
    k.dx_even = c.dx;
    k.dx_odd = (float *)(ws + l.dx_at);
    k.status = (unsigned *)ws;
    k.arrive = k.status + 64;
    k.ready = k.arrive + (size_t)c.outer * c.B;  // (the last step's share of either array stays unused)
    k.steps = c.outer;
    k.spin_limit = c.spin_limit;
    k.step_floats = (long)c.B * cells;
    k.B = c.B; k.M = c.M; k.N = c.N; k.K = c.K; k.inner = c.inner;
    // the sums of the last LayerNorm come from the gradient handed in
    const long last = c.outer - 1;
    if (int rc = layernorm_backward_sums(c.dy, c.y_raw + last * k.step_floats, c.stats + last * 2 * c.B, c.gamma,
                                         k.sums, c.B, cells, (float *)(ws + l.ln_at), st))
        return rc;
    if (int rc = plan_fill_zero((float *)ws, (long)l.sync_words, st)) return rc;
    void *args[] = {&k};
    hipError_t e = hipLaunchCooperativeKernel((const void *)kern, dim3(padded_grid(k.nblk, 1)), dim3(256), args,
                                              (unsigned)lds, st);
    if (e != hipSuccess) {
        (void)hipGetLastError();
        return fail(GRIDNET_ERR_LAUNCH, "chain_bwd (whole chain): cooperative launch failed: %s", hipGetErrorString(e));
    }
    hipLaunchKernelGGL(chain_halo_gather, dim3((c.M / 8) * (c.N / 8), c.B), dim3(256), 0, st, c.dx, k.halo_even, c.M,
                       c.N, c.K, k.nblk);
    return check_launch("chain_halo_gather");
}

template <int ACT> int dispatch_defer(const StepArgs &a, hipStream_t st) {
    if (a.inner > kChainNarrowInner)
        return a.ln.halo_out ? launch_chain<ACT, true, true>(a, st) : launch_chain<ACT, false, true>(a, st);
    return a.ln.halo_out ? launch_chain<ACT, true, false>(a, st) : launch_chain<ACT, false, false>(a, st);
}

}  // namespace

bool chain_supports(const StepArgs &a) {
    return a.dtype == GRIDNET_F32 && a.block_size == 8 && !a.normalize && a.inner >= 1 &&
           a.inner <= kChainMaxInner;
}

size_t chain_halo_floats(const StepArgs &a) {
    return (size_t)a.B * (a.M / 8) * (a.N / 8) * (a.K / 8) * kShell;
}

// The whole chain fits one launch when every block gets a workgroup of its own and all of them
// are resident at once; a pair (step, element) must have been counted in and finalized (four
// iterations after it was worked on) before the same workgroup can need it (B iterations after).
constexpr int kChainAllMinBatch = 6;
bool chain_all_supports(int B, int M, int N, int K, int inner, int outer) {
    if (M <= 0 || N <= 0 || K <= 0 || M % 8 || N % 8 || K % 8) return false;
    if (inner < 1 || inner > kChainMaxInner || outer < 2 || B < kChainAllMinBatch) return false;
    if ((long)M * N * K * 27 >= (1L << 31)) return false;
    static int per_cu_cache[kChainMaxInner + 1];
    int &per_cu = per_cu_cache[inner];
    if (per_cu == 0) {
        const void *kern = inner > kChainNarrowInner ? (const void *)chain_bwd<GRIDNET_ACT_LEAKY_RELU, true, true, true>
                                                     : (const void *)chain_bwd<GRIDNET_ACT_LEAKY_RELU, true, true, false>;
        const size_t lds = (size_t)chain_lds_floats(inner) * sizeof(float);
        if (lds > 64 * 1024 &&
            hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize,
                                (int)((size_t)chain_lds_floats(kChainMaxInner) * sizeof(float))) != hipSuccess)
            return false;
        int n = 0;
        if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, kern, 256, lds) != hipSuccess || n < 1) n = -1;
        per_cu = n;
    }
    if (per_cu < 1) return false;
    const long nblk = (long)(M / 8) * (N / 8) * (K / 8);
    return padded_grid((int)nblk, 1) <= (long)per_cu * plan_device_cus();
}

size_t chain_all_workspace(const ChainAll &c) { return chain_all_layout(c).total; }

template <int ACT> int dispatch_all(const ChainAll &c, hipStream_t st) {
    return c.inner > kChainNarrowInner ? launch_chain_all<ACT, true>(c, st) : launch_chain_all<ACT, false>(c, st);
}

int chain_backward_all(const ChainAll &c, hipStream_t st) {
    switch (c.activation) {
        case GRIDNET_ACT_RELU: return dispatch_all<GRIDNET_ACT_RELU>(c, st);
        case GRIDNET_ACT_LEAKY_RELU: return dispatch_all<GRIDNET_ACT_LEAKY_RELU>(c, st);
        case GRIDNET_ACT_SILU: return dispatch_all<GRIDNET_ACT_SILU>(c, st);
        case GRIDNET_ACT_TANH: return dispatch_all<GRIDNET_ACT_TANH>(c, st);
    }
    return fail(GRIDNET_ERR_ACTIVATION, "unknown activation function: id %d", c.activation);
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
