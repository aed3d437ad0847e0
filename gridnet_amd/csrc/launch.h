// Host-side argument bundles and the launch functions each .hip file provides.
#pragma once

#include <hip/hip_runtime.h>

#include <cstddef>

namespace gridnet {

// LayerNorm folded into the step kernels: one outer step of the body "update step, then
// per-sample LayerNorm over the grid" without a pass of its own for the LayerNorm.  A step reads
// the RAW output of the step before it (before that step's LayerNorm) and normalises it while
// loading; it writes its own raw output and what the next step needs to do the same.  All
// members may be null; statistics are (mean, rstd) pairs, sums are the two per-sample means of
// the LayerNorm backward, one pair per batch element, fp32.
struct LnFold {
    const float *gamma, *beta;  // [M,N,K]
    const float *x_stats;       // [B,2]: LayerNorm applied to x on load; null: x is used as is
    float *y_part;              // forward: partial (mean, M2) of the output, one pair per wave
                                // (per slot, for half-wave slots): [B, nblk, parts, 2]
    // backward: the incoming gradient is with respect to LayerNorm(y_raw)
    const float *y_raw;         // [B,M,N,K] this step's forward output before its LayerNorm
    const float *y_stats;       // [B,2]
    const float *y_sums;        // [B,2]: mean(g), mean(g * yhat) with g = gamma * incoming gradient
    float *dgamma, *dbeta;      // [M,N,K], summed over the batch, committed like dbias
    float *x_part;              // partial sums for the LayerNorm backward of x: [B, nblk, parts, 2]
    float *x_sums;              // [B,2] or null: where a backward that finishes the sums itself leaves them
                                // (bwd_rows_leaves_sums); otherwise the caller finalizes x_part
    // The reference's outer_residual form of the loop (gridnet/scripts/train_imagenet.py:81-83):
    // h' = h + (step(n) - n), n = LayerNorm(h).  Forward: the output is x + (result - n); needs
    // x_stats.  Backward of the step that produced h' from h = x, with G' the gradient with
    // respect to h': the step's incoming gradient is G' itself, which is either given (`dy`,
    // when y_raw is null: the last step of a chain) or formed on load as
    // g_prev + LayerNorm'(dy; y_raw, y_stats, y_sums), the gradient with respect to h'' of the
    // step after plus that step's dn taken through its LayerNorm, and then also stored to g_out;
    // dx receives dn = (gradient with respect to n) - G' (the first kernel takes G' off the part
    // of dx that it writes), and x_part its LayerNorm sums.
    int residual;
    const float *g_prev;  // [B,M,N,K] or null
    float *g_out;         // [B,M,N,K] or null
    // The backward of a chain (chain_bwd.hip) hands what crosses a block boundary to the backward
    // of the step BEFORE it instead of completing dx itself: per (element, block) the 488
    // values that the cells around the block receive from it, filed per RECEIVING block
    // ([B, nblk, 488], see chain_bwd.hip).  halo_in: what the step after left for this one (null:
    // dy is complete); halo_out: where this step leaves its own (null: dx is completed here).
    const float *halo_in;
    float *halo_out;
    // forward: workgroups take the blocks in reverse order.  Results do not depend on it; a chain
    // whose steps alternate finds what the step before touched last (its output, the parameter
    // planes it fetched last) still in the last-level cache when its working set exceeds that cache.
    int walk_reverse;
};

struct StepArgs {
    int dtype;
    const void *weight, *bias, *scale, *x;
    void *y;                           // forward only
    const void *dy;                    // backward only
    void *dweight, *dbias, *dscale, *dx;
    int B, M, N, K, inner, block_size;
    double eps;
    int normalize, activation, flags;
    void *workspace;
    size_t workspace_bytes;
    LnFold ln;  // all null: the plain step
    // backward on grids where the batch of a block is split over workgroups: room for every
    // chunk's own copy of the gradient arrays (see plan.h); may be null (the batch is then not split)
    void *slabs;
    size_t slab_bytes;
};

// floats per cell in one copy of the plain step's gradient arrays (see plan.h): 27 weight planes,
// bias, scale and, with the folded LayerNorm, gamma and beta
constexpr int kStepSlabPlanes = 31;
// ... and of the gated step's: 54 weight planes, 2 bias planes
constexpr int kGatedSlabPlanes = 56;

// How a workgroup commits its parameter gradients.
enum ParamMode {
    kParamStore = 0,         // sole owner of the cells, output uninitialised: plain store
    kParamAddExclusive = 1,  // sole owner, output holds a prior sum: read-add-write
    kParamAtomic = 2         // several workgroups (batch chunks) share the cells (generic kernels only)
};

struct LayerNormArgs {
    int dtype;
    const void *x, *gamma, *beta, *dy, *mean_in, *rstd_in;
    void *y, *mean, *rstd, *dx, *dgamma, *dbeta;
    int B;
    long n;
    double eps;
    int flags;
    void *workspace;
    size_t workspace_bytes;
};

// step_generic.hip
int step_forward_generic(const StepArgs &a, hipStream_t st);
int step_backward_generic(const StepArgs &a, hipStream_t st);

// step_fast.hip: fp32, block sizes 4 and 8, normalize on or off (off only with the folded LayerNorm)
bool step_fast_supports(const StepArgs &a, bool backward);
size_t step_fast_backward_workspace(const StepArgs &a);   // what the backward cannot do without
size_t step_fast_slab_bytes(const StepArgs &a);           // room for the gradient copies of a split batch
int step_forward_fast(const StepArgs &a, hipStream_t st);
int step_backward_fast(const StepArgs &a, hipStream_t st);
// partial statistics per (block, batch element) that the kernels above write when asked to
int step_fast_forward_parts(int block_size);   // (mean, M2) pairs per block at most, each over forward_part_count cells
int step_fast_forward_part_count(int block_size);
int step_fast_forward_pairs(const StepArgs &a);       // pairs per sample that the forward of `a` leaves ...
int step_fast_forward_pair_count(const StepArgs &a);  // ... and the cells behind each
int step_fast_backward_parts(int block_size);  // (sum g, sum g*xhat) pairs per (block, element), at most
int step_fast_backward_pairs(const StepArgs &a);  // pairs per sample that the backward of `a` leaves
int step_fast_cross_pairs(const StepArgs &a);     // the same for step_cross_launch alone (behind chain_bwd)

// fwd_rows.hip: the forward of a step with ONE inner iteration, dealt by whole K-rows (fp32, normalize
// off, K of 16, 32, 64 or 128; the folded LayerNorm and the residual form as a.ln says)
bool fwd_rows_supports(const StepArgs &a);
int fwd_rows_pairs(const StepArgs &a);  // (mean, M2) pairs per sample in a.ln.y_part, 256 cells each
int fwd_rows_launch(const StepArgs &a, hipStream_t st);

// bwd_rows.hip: the backward of a step with ONE inner iteration by whole K-rows (with
// cross_rows_full_launch behind it); fp32, normalize off, K of 16, 32 or 64; a.slabs as for
// step_backward_fast
bool bwd_rows_supports(const StepArgs &a);
size_t bwd_rows_slab_bytes(const StepArgs &a);
int bwd_rows_launch(const StepArgs &a, hipStream_t st);
// LayerNorm sum pairs per sample in a.ln.x_part after bwd_rows_launch (the plain loop: the first
// kernel forms them, one pair per wave; the residual loop: cross_rows_pairs)
int bwd_rows_pairs(const StepArgs &a);
// bwd_rows_launch leaves a.ln.x_sums finished (no finalize call behind it)
bool bwd_rows_leaves_sums(const StepArgs &a);

// cross_rows.hip: the cross-block part of the backward for 4^3 blocks, dealt by whole K-rows
// (a.workspace holds D, a.dx the block-local part; LayerNorm fold as a.ln says); K of 16, 32, 64
// or 128, normalize off
bool cross_rows_supports(const StepArgs &a);
int cross_rows_pairs(const StepArgs &a);  // LayerNorm sum pairs per sample that it leaves in a.ln.x_part
int cross_rows_launch(const StepArgs &a, hipStream_t st);
// all 27 taps, for bwd_rows.hip; ln_sums: with the LayerNorm sums of the finished rows (a.ln.x_part)
int cross_rows_full_launch(const StepArgs &a, hipStream_t st, bool ln_sums);
bool cross_rows_gated_supports(const StepArgs &a);  // the gated update: two weight sets, D0 and D1 in `dsum`
int cross_rows_gated_launch(const StepArgs &a, const float *dsum, hipStream_t st);

// step_fast.hip: the cross-block kernel alone (8^3 blocks, folded LayerNorm arguments in a.ln, the
// D tensor in a.workspace), for chain_bwd.hip
int step_cross_launch(const StepArgs &a, int nchunk, int chunk_len, hipStream_t st);

// chain_bwd.hip: backward of one step of a chain with the cross-block part deferred to the step
// before (a.ln.halo_in / halo_out); fp32, 8^3 blocks, 1..8 inner iterations, normalize off
bool chain_supports(const StepArgs &a);
size_t chain_halo_floats(const StepArgs &a);
int chain_backward(const StepArgs &a, hipStream_t st);

// chain_bwd.hip: the backward of a whole chain of `outer` steps (one parameter set) in ONE launch
// of resident workgroups that hand the cross-block values and the LayerNorm sums from step to
// step through memory behind per-(step, element) counters.  y_raw [outer,B,M,N,K], stats
// [outer,B,2]; dx receives the gradient of the chain's input x0.  The first word of the
// workspace is a status: non-zero after the launch means a bounded wait ran out and the results
// are invalid.
struct ChainAll {
    const float *weight, *bias, *scale, *gamma, *beta;
    const float *x0, *y_raw, *stats, *dy;
    float *dweight, *dbias, *dscale, *dgamma, *dbeta, *dx;
    int B, M, N, K, inner, outer, activation, flags;
    void *workspace;
    size_t workspace_bytes;
    int spin_limit;  // polls before a wait gives up; negative: ready words are never set (tests of the give-up path)
};
bool chain_all_supports(int B, int M, int N, int K, int inner, int outer);
size_t chain_all_workspace(const ChainAll &c);
int chain_backward_all(const ChainAll &c, hipStream_t st);

// step_fast.hip: the cross-block kernel on two weight sets, for gated_fast.hip
int gated_cross_launch(const StepArgs &a, const float *dsum, int nchunk, int chunk_len, hipStream_t st);

// gated_fast.hip: fp32, block sizes 4 and 8, as many inner iterations as the LDS holds
bool gated_fast_supports(const StepArgs &a, bool backward);
size_t gated_fast_backward_workspace(const StepArgs &a);
size_t gated_fast_slab_bytes(const StepArgs &a);
int gated_forward_fast(const StepArgs &a, hipStream_t st);
int gated_backward_fast(const StepArgs &a, hipStream_t st);

// gated_generic.hip (weight [27,2,M,N,K], bias [2,M,N,K]; scale, eps, normalize unused)
int gated_forward(const StepArgs &a, hipStream_t st);
int gated_backward(const StepArgs &a, hipStream_t st);

// layernorm.hip
// (mean, M2) pairs over `count` cells each -> (mean, rstd) per sample
int layernorm_finalize_stats(const float *part, int parts_per_sample, int count, float *stats, int B,
                             double eps, hipStream_t st);
// (sum, sum) pairs -> their means over n cells per sample
int layernorm_finalize_sums(const float *part, int parts_per_sample, long n, float *sums, int B,
                            hipStream_t st);
// y = (x - mean) * rstd * gamma + beta with given statistics
int layernorm_apply_stats(const float *x, const float *stats, const float *gamma, const float *beta,
                          float *y, int B, long n, hipStream_t st);
// the two per-sample means of the LayerNorm backward from interleaved (mean, rstd) statistics;
// `partial` holds layernorm_workspace() bytes
int layernorm_backward_sums(const float *dy, const float *x, const float *stats, const float *gamma,
                            float *sums, int B, long n, float *partial, hipStream_t st);
size_t layernorm_workspace(int dtype, int B, long n);
int layernorm_forward(const LayerNormArgs &a, hipStream_t st);
int layernorm_backward(const LayerNormArgs &a, hipStream_t st);

}  // namespace gridnet
