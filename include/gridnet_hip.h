/*
 * gridnet_hip.h -- C ABI of libgridnet_hip.so: the block-local grid update of gridnet
 * (3x3x3 per-cell-weight stencil with stale halos, its backward, and the per-sample
 * LayerNorm the callers interleave with it) as hand-written HIP kernels for gfx950.
 *
 * Conventions shared by every entry point
 *   - All pointers are DEVICE pointers into memory the caller owns.  The library never
 *     allocates, frees, retains or synchronises; every call only enqueues kernels on
 *     `stream` (a hipStream_t passed as void*, NULL = the default stream).
 *   - Tensors are dense, row-major, K fastest: weight [27, M, N, K] with tap index
 *     t = 9a + 3b + c addressing neighbour (i+a-1, j+b-1, k+c-1); bias, scale [M, N, K];
 *     activations [B, M, N, K].  (gridnet/__init__.py:42-49, gridnet/backend_torch.py:283-298)
 *   - `dtype` is GRIDNET_F32 or GRIDNET_F64 and applies to every tensor of the call.
 *   - A tensor may start at any address that is a multiple of its element size (for example
 *     a view one element into a larger buffer), as with the reference's element-wise
 *     accessors (src/gridnet_cuda_kernels.cu:103-107); the workspace likewise.
 *   - Sizes: the cells of one sample are indexed with 32 bits, so 27*M*N*K (54*M*N*K for
 *     the gated op) must stay below 2^31; samples are indexed with 64 bits, so B*M*N*K may
 *     exceed 2^31 (the reference's 32-bit accessors, src/gridnet_cuda_kernels.cu:103-107,
 *     stop there).
 *   - Return value 0 = enqueued.  Non-zero = nothing was enqueued; the message is
 *     available from gridnet_hip_last_error() on the calling thread.
 */
#ifndef GRIDNET_HIP_H
#define GRIDNET_HIP_H

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

enum gridnet_dtype { GRIDNET_F32 = 0, GRIDNET_F64 = 1 };

/* Activation ids; the names are the strings the reference dispatches on
 * (src/activations.h:6-17, gridnet/backend_torch.py:270-280). */
enum gridnet_activation {
    GRIDNET_ACT_RELU = 0,
    GRIDNET_ACT_LEAKY_RELU = 1, /* slope 0.01 */
    GRIDNET_ACT_SILU = 2,
    GRIDNET_ACT_TANH = 3
};

/* Status codes. */
enum gridnet_status {
    GRIDNET_OK = 0,
    GRIDNET_ERR_ARGUMENT = 1,   /* bad shape / block size / pointer / dtype */
    GRIDNET_ERR_ACTIVATION = 2, /* "unknown activation function: X" (src/activations.h:16) */
    GRIDNET_ERR_ITERATIONS = 3, /* "cannot backprop through more than 32 inner iterations"
                                   (src/gridnet_cuda_kernels.cu:836) */
    GRIDNET_ERR_WORKSPACE = 4,  /* workspace missing or too small */
    GRIDNET_ERR_LAUNCH = 5      /* hipGetLastError() after the launch */
};

/* Flags for the backward entry points. */
enum gridnet_flags {
    /* Default (0): every gradient output is ACCUMULATED into, as the reference's kernels do
     * with atomicAdd into buffers its wrapper zero-filled (gridnet/backend_cuda.py:78-81,
     * src/gridnet_cuda_kernels.cu:424-449).  With a flag set, that output need not be
     * initialised: it is fully written. */
    GRIDNET_OVERWRITE_PARAMS = 1, /* dweight, dbias, dscale (LayerNorm: dgamma, dbeta) */
    GRIDNET_OVERWRITE_DX = 2,     /* dx (LayerNorm: dx is always fully written) */
    GRIDNET_OVERWRITE = 3
};

/* Library build id (monotonic integer) -- lets a binding check it loaded what it expects. */
int gridnet_hip_version(void);

/* Thread-local message of the last non-zero status returned on this thread ("" if none). */
const char *gridnet_hip_last_error(void);

/* Map an activation name to its id, or -1 (and set the reference's message
 * "unknown activation function: <name>").  Replaces APPLY_ACTIVATION, src/activations.h:6-17. */
int gridnet_hip_activation_id(const char *name);

/*
 * One outer step, forward.  Replaces gridnet_cuda_forward, src/gridnet_cuda_kernels.cu:736-784
 * (bound as `forward`, src/gridnet_cuda.cpp:61-89,190).
 *   y is fully overwritten.  inner >= 0.  block_size in {4, 8} and must divide M, N and K.
 *   eps/normalize: per-window normalisation (x-mean)/(std+eps) over the (bs+2)^3 window.
 */
int gridnet_hip_forward(int dtype, const void *weight, const void *bias, const void *scale,
                        const void *x, void *y, int B, int M, int N, int K, int inner,
                        int block_size, double eps, int normalize, int activation,
                        void *stream);

/*
 * Scratch that gridnet_hip_backward wants for this problem (bytes, may be 0).  On grids with
 * fewer blocks than the GPU has compute units it includes room for one copy of the gradient
 * arrays per batch chunk: the batch of a block is then split over workgroups, each leaves its
 * share in its own copy with plain stores and the copies are added in chunk order (no atomics,
 * the same bits on every run).  A caller may hand over less, down to B*M*N*K elements (plus two
 * floats per block and batch element with normalize): the batch is then split less, or not at
 * all; the results agree to rounding.
 */
size_t gridnet_hip_backward_workspace_bytes(int dtype, int B, int M, int N, int K, int inner,
                                            int block_size, int normalize);

/*
 * One outer step, backward.  Replaces gridnet_cuda_backward, src/gridnet_cuda_kernels.cu:786-851
 * (bound as `backward`, src/gridnet_cuda.cpp:91-131,191).  Recomputes the inner forward
 * from x; inner <= 32.  dweight [27,M,N,K], dbias, dscale [M,N,K] are summed over the batch;
 * dx [B,M,N,K].  `workspace` must hold gridnet_hip_backward_workspace_bytes() bytes (contents
 * need no initialisation).
 */
int gridnet_hip_backward(int dtype, const void *weight, const void *bias, const void *scale,
                         const void *x, const void *dy, void *dweight, void *dbias,
                         void *dscale, void *dx, int B, int M, int N, int K, int inner,
                         int block_size, double eps, int normalize, int activation, int flags,
                         void *workspace, size_t workspace_bytes, void *stream);

/*
 * gridnet_hip_backward without a workspace argument and without any allocation.  It has no
 * counterpart in the reference; it exists for callers that cannot allocate device memory:
 * code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.
 * The scratch that gridnet_hip_backward takes as `workspace` lives in a static device array of
 * GRIDNET_STATIC_SCRATCH_BYTES inside the library instead (one copy per GPU, held until the
 * process ends).  What must fit is the part gridnet_hip_backward cannot do without: B*M*N*K
 * elements, plus two per (batch element, block) with normalize; a problem that needs more is
 * rejected with GRIDNET_ERR_WORKSPACE and nothing is enqueued.  (The figure that
 * gridnet_hip_backward_workspace_bytes() returns also counts, on grids with fewer blocks than
 * compute units, room for one copy of the gradient arrays per batch chunk; with less of that
 * room than gridnet_hip_backward was given the batch is split over fewer workgroups and the
 * parameter gradients are summed in another order: equal to rounding, and still the same bits
 * on every run.)  Same arguments and flags as gridnet_hip_backward, same kernels.
 * Every call on a GPU shares that GPU's array: calls that may overlap on one GPU (different
 * streams, different threads) race and must be serialised by the caller.  The array's
 * contents need not be, and are not, preserved between calls.
 * gridnet_hip_static_init() looks the array up for the CURRENT device (hipGetSymbolAddress; no
 * allocation either); gridnet_hip_backward_static does the same on its first call on a
 * device, so a caller that is going to capture a graph calls the init once beforehand.
 */
#define GRIDNET_STATIC_SCRATCH_BYTES (40u << 20)

int gridnet_hip_static_init(void);

int gridnet_hip_backward_static(int dtype, const void *weight, const void *bias, const void *scale,
                                const void *x, const void *dy, void *dweight, void *dbias,
                                void *dscale, void *dx, int B, int M, int N, int K, int inner,
                                int block_size, double eps, int normalize, int activation,
                                int flags, void *stream);

/*
 * Gated variant: x' = gate*x + (1-gate)*act(pre), weight [27,2,M,N,K] (channel 0: pre,
 * channel 1: gate), bias [2,M,N,K]; no scale, eps or normalisation.  Replace
 * gated_gridnet_cuda_forward / gated_gridnet_cuda_backward, src/gridnet_cuda_kernels.cu:853-930
 * (bound as `forward_gated` / `backward_gated`, src/gridnet_cuda.cpp:133-186,192-193).
 * Backward: inner <= 32; dweight [27,2,M,N,K], dbias [2,M,N,K] summed over the batch; flags as
 * for gridnet_hip_backward; `workspace` must hold gridnet_hip_backward_gated_workspace_bytes()
 * bytes (may be 0; contents need no initialisation).
 */
int gridnet_hip_forward_gated(int dtype, const void *weight, const void *bias, const void *x,
                              void *y, int B, int M, int N, int K, int inner, int block_size,
                              int activation, void *stream);

size_t gridnet_hip_backward_gated_workspace_bytes(int dtype, int B, int M, int N, int K, int inner,
                                                  int block_size);

int gridnet_hip_backward_gated(int dtype, const void *weight, const void *bias, const void *x,
                               const void *dy, void *dweight, void *dbias, void *dx, int B, int M,
                               int N, int K, int inner, int block_size, int activation, int flags,
                               void *workspace, size_t workspace_bytes, void *stream);

/*
 * Per-sample LayerNorm over all n = M*N*K cells with elementwise affine, the op the callers
 * place after every outer step (torch.nn.LayerNorm((M,N,K)): gridnet/scripts/train_mnist.py:54,64,
 * gridnet/scripts/train_imagenet.py:67,86).  y = (x-mean)*rstd*gamma + beta, biased variance,
 * rstd = 1/sqrt(var+eps).  mean, rstd: [B] outputs kept for the backward.
 */
size_t gridnet_hip_layernorm_workspace_bytes(int dtype, int B, long n);

int gridnet_hip_layernorm_forward(int dtype, const void *x, const void *gamma, const void *beta,
                                  void *y, void *mean, void *rstd, int B, long n, double eps,
                                  void *workspace, size_t workspace_bytes, void *stream);

/* dx [B,n] (always fully written); dgamma, dbeta [n] summed over the batch (accumulated
 * unless GRIDNET_OVERWRITE_PARAMS). */
int gridnet_hip_layernorm_backward(int dtype, const void *dy, const void *x, const void *gamma,
                                   const void *mean, const void *rstd, void *dx, void *dgamma,
                                   void *dbeta, int B, long n, int flags, void *workspace,
                                   size_t workspace_bytes, void *stream);

/*
 * ---- The network body with the LayerNorm folded into the step kernels ----------------------
 * The reference's callers run `h = norm(net(h))` op by op, `outer` times
 * (gridnet/scripts/train_mnist.py:62-64, gridnet/scripts/train_imagenet.py:76-86); these entry
 * points compute the same chain without a pass over the activations for each LayerNorm: a step
 * reads the RAW output of the step before it and normalises it while loading, and leaves its own
 * raw output together with that output's LayerNorm statistics.  They have no counterpart in the
 * reference's extension; results agree with the op-by-op chain to rounding.
 *
 * float32, normalize = false, inner >= 1, block_size in {4, 8}; other problems are rejected with
 * GRIDNET_ERR_ARGUMENT (use the step and LayerNorm entry points above).
 *   stats  [B, 2]: (mean, rstd) of a LayerNorm over one sample's M*N*K cells
 *   sums   [B, 2]: the two per-sample means its backward needs, mean(gamma*g) and
 *                  mean(gamma*g*xhat), g the gradient with respect to the LayerNorm's output
 */
size_t gridnet_hip_fused_workspace_bytes(int B, int M, int N, int K, int inner, int block_size,
                                         int backward);

/* y_raw = step(LayerNorm(x; x_stats, gamma, beta)), y_stats = statistics of y_raw.
 * x_stats == NULL: x is used as it is (the first step of a chain). */
int gridnet_hip_fused_forward(int dtype, const void *weight, const void *bias, const void *scale,
                              const void *gamma, const void *beta, const void *x,
                              const void *x_stats, void *y_raw, void *y_stats, int B, int M, int N,
                              int K, int inner, int block_size, double ln_eps, int activation,
                              void *workspace, size_t workspace_bytes, void *stream);

/* Either of the two forward calls around this one (gridnet_hip_fused_forward,
 * gridnet_hip_fused_forward_residual with GRIDNET_FUSED_RESIDUAL) with one more choice:
 * GRIDNET_FUSED_WALK_REVERSE makes the workgroups take the blocks in reverse order.  The results
 * are the same bits either way.  A chain of steps (gridnet/scripts/train_imagenet.py:76-86) that
 * sets it for every other step finds what the step before touched last -- the end of its output,
 * the parameter planes it fetched last -- still in the GPU's last-level cache when one step's
 * working set exceeds that cache (a 128^3 grid: 243 MB of parameters per step against 256 MB of
 * cache; 162 -> 156 us per step there, nothing to gain at 64^3). */
enum { GRIDNET_FUSED_RESIDUAL = 1, GRIDNET_FUSED_WALK_REVERSE = 2 };
int gridnet_hip_fused_forward_flags(int dtype, const void *weight, const void *bias, const void *scale,
                                    const void *gamma, const void *beta, const void *x,
                                    const void *x_stats, void *y, void *y_stats, int B, int M, int N,
                                    int K, int inner, int block_size, double ln_eps, int activation,
                                    int flags, void *workspace, size_t workspace_bytes, void *stream);

/* The reference's outer_residual form of one outer step, forward
 * (gridnet/scripts/train_imagenet.py:81-83: n = norm(h); h = h + (net(n) - n)):
 * y = x + (step(n) - n) with n = LayerNorm(x; x_stats, gamma, beta), y_stats = statistics of y,
 * which the next step of such a chain takes as its x_stats.  x_stats is required (the
 * statistics of the chain's first input come from gridnet_hip_layernorm_forward).  The result of
 * a chain is the y of its last step as it is.  Workspace as for gridnet_hip_fused_forward. */
int gridnet_hip_fused_forward_residual(int dtype, const void *weight, const void *bias,
                                       const void *scale, const void *gamma, const void *beta,
                                       const void *x, const void *x_stats, void *y, void *y_stats,
                                       int B, int M, int N, int K, int inner, int block_size,
                                       double ln_eps, int activation, void *workspace,
                                       size_t workspace_bytes, void *stream);

/* y = (x - mean) * rstd * gamma + beta with statistics that are already known: the LayerNorm
 * after the LAST step of a chain, whose output is needed as a tensor. */
int gridnet_hip_layernorm_apply(int dtype, const void *x, const void *stats, const void *gamma,
                                const void *beta, void *y, int B, long n, void *stream);

/* `sums` of a LayerNorm from the gradient dy with respect to its output: what the backward of a
 * chain starts from.  workspace: gridnet_hip_layernorm_workspace_bytes(). */
int gridnet_hip_layernorm_backward_sums(int dtype, const void *dy, const void *x, const void *stats,
                                        const void *gamma, void *sums, int B, long n,
                                        void *workspace, size_t workspace_bytes, void *stream);

/* Backward of gridnet_hip_fused_forward.  dy is the gradient with respect to
 * LayerNorm(y_raw; y_stats); y_sums are that LayerNorm's sums.  dweight, dbias, dscale, dgamma,
 * dbeta (dgamma, dbeta: of the LayerNorm after this step) are accumulated, or written with
 * GRIDNET_OVERWRITE_PARAMS.  dx is always fully written: the gradient with respect to
 * LayerNorm(x; x_stats) -- the dy of the step before -- and x_sums receives its sums; with
 * x_stats == NULL (first step) dx is the gradient with respect to x and x_sums must be NULL. */
int gridnet_hip_fused_backward(int dtype, const void *weight, const void *bias, const void *scale,
                               const void *gamma, const void *beta, const void *x,
                               const void *x_stats, const void *dy, const void *y_raw,
                               const void *y_stats, const void *y_sums, void *dweight, void *dbias,
                               void *dscale, void *dgamma, void *dbeta, void *dx, void *x_sums, int B,
                               int M, int N, int K, int inner, int block_size, int activation,
                               int flags, void *workspace, size_t workspace_bytes, void *stream);

/* Backward of gridnet_hip_fused_forward_residual for the step that made h' = y from h = x.
 * With G' the gradient with respect to h':
 *   - the last step of a chain is given it: dy = G', and y_raw, y_stats, y_sums, g_prev, g_out
 *     are all NULL;
 *   - any other step forms it while loading: G' = g_prev + LayerNorm'(dy), where dy is the dx
 *     that the call for the step AFTER this one wrote, y_raw = h' (that step's input),
 *     y_stats / y_sums its statistics and the x_sums of that call, and g_prev the G'' of that
 *     call (its g_out, or its dy if it was the last step); G' is also stored to g_out.
 * dx receives dn = (gradient with respect to LayerNorm(x)) - G' and x_sums its LayerNorm sums;
 * dgamma, dbeta receive the gradients of the LayerNorm that dy was taken through.  What remains
 * for the caller after the first step of the chain (x = the chain's input): the gradient of that
 * input is G' + LayerNorm'(dx), with the LayerNorm's dgamma, dbeta on top: one
 * gridnet_hip_layernorm_backward call and an addition.  Flags, workspace and everything else as
 * gridnet_hip_fused_backward. */
int gridnet_hip_fused_backward_residual(int dtype, const void *weight, const void *bias,
                                        const void *scale, const void *gamma, const void *beta,
                                        const void *x, const void *x_stats, const void *dy,
                                        const void *y_raw, const void *y_stats, const void *y_sums,
                                        const void *g_prev, void *g_out, void *dweight, void *dbias,
                                        void *dscale, void *dgamma, void *dbeta, void *dx,
                                        void *x_sums, int B, int M, int N, int K, int inner,
                                        int block_size, int activation, int flags, void *workspace,
                                        size_t workspace_bytes, void *stream);

/*
 * ---- The backward of a chain that hands gradients across block boundaries from step to step --
 * gridnet_hip_fused_backward with one change that a caller who runs the whole chain can afford
 * (no counterpart in the reference, which scatters across block boundaries with global atomics,
 * src/gridnet_cuda_kernels.cu:424-435): a call may leave dx UNFINISHED.  What the cells of other
 * blocks receive (one cell deep around every block) is not added to dx but filed, 488 floats per
 * (element, block), in halo_out [B, nblk, 488]; the call for the step BEFORE takes that buffer as
 * its halo_in and adds the values while it loads its incoming gradient.  One kernel per step
 * instead of two, and no scratch tensor written and read back.
 * float32, normalize = false, block_size 8, 1 <= inner <= 8; gridnet_hip_chain_supported() tells,
 * other problems use gridnet_hip_fused_backward.  Results agree with it to rounding.
 */
int gridnet_hip_chain_supported(int dtype, int inner, int block_size, int normalize);

/* floats of one halo buffer: B * nblk * 488 */
size_t gridnet_hip_chain_halo_floats(int B, int M, int N, int K, int block_size);

/*   halo_in  == NULL: dy is complete (the last step of a chain);
 *            != NULL: dy lacks what the call for the step after left there;
 *   halo_out != NULL: dx receives the block-local part only and halo_out the rest; x_stats and
 *                     x_sums are required (x_sums is complete: the sums do not wait for dx);
 *            == NULL: dx is finished here (the first step of a chain), as by
 *                     gridnet_hip_fused_backward.
 * Workspace: gridnet_hip_fused_workspace_bytes(.., 1).  Everything else as gridnet_hip_fused_backward. */
int gridnet_hip_chain_backward(int dtype, const void *weight, const void *bias, const void *scale,
                               const void *gamma, const void *beta, const void *x,
                               const void *x_stats, const void *dy, const void *y_raw,
                               const void *y_stats, const void *y_sums, const void *halo_in,
                               void *halo_out, void *dweight, void *dbias, void *dscale, void *dgamma,
                               void *dbeta, void *dx, void *x_sums, int B, int M, int N, int K,
                               int inner, int block_size, int activation, int flags, void *workspace,
                               size_t workspace_bytes, void *stream);

/*
 * ---- The backward of a whole chain in one launch ------------------------------------------------
 * The loop the reference's training scripts run around the step,
 *     for i in range(outer): h = norm(net(h))          gridnet/scripts/train_imagenet.py:76-86
 * (one Gridnet, one LayerNorm, shared by the steps), taken backward by ONE kernel whose workgroups
 * stay resident for all `outer` steps: each keeps its block, its weights and its gradient
 * accumulators from step to step and hands what crosses block boundaries, and the sums of the
 * LayerNorm between two steps, to the workgroups that need them through memory, behind one
 * counter per (step, batch element).  No set-up, drain or gradient read-modify-write per step.
 *   x0      [B,M,N,K]        input of the chain
 *   y_raw   [outer,B,M,N,K]  raw output of every step (gridnet_hip_fused_forward's y_raw)
 *   stats   [outer,B,2]      their LayerNorm statistics (its y_stats)
 *   dy      [B,M,N,K]        gradient with respect to LayerNorm(y_raw[outer-1])
 *   dweight, dbias, dscale, dgamma, dbeta   accumulated, or written with GRIDNET_OVERWRITE_PARAMS
 *   dx      [B,M,N,K]        gradient with respect to x0, fully written
 * float32, normalize = false, block_size 8, 1 <= inner <= 8, outer >= 2, B >= 6, and a grid whose
 * blocks all fit the GPU at once (M/8 * N/8 * K/8 workgroups resident: 512 on an MI355X, a 64^3
 * grid); gridnet_hip_chain_all_supported() tells.  Results agree with the chain of
 * gridnet_hip_chain_backward calls to rounding and are the same bits on every run.
 * The kernel is launched cooperatively.  Every wait inside it is bounded: should one run out (the
 * workgroups were not all resident after all), the kernel still ends, and the FIRST 4 BYTES OF THE
 * WORKSPACE, zero otherwise, are non-zero once the stream has passed the call: the results are
 * then invalid and the caller repeats the backward with gridnet_hip_chain_backward, whose inputs
 * this call leaves untouched.
 */
int gridnet_hip_chain_all_supported(int dtype, int B, int M, int N, int K, int inner, int outer,
                                    int block_size, int normalize);
size_t gridnet_hip_chain_all_workspace_bytes(int B, int M, int N, int K, int inner, int outer,
                                             int block_size);
int gridnet_hip_chain_backward_all(int dtype, const void *weight, const void *bias, const void *scale,
                                   const void *gamma, const void *beta, const void *x0,
                                   const void *y_raw, const void *stats, const void *dy,
                                   void *dweight, void *dbias, void *dscale, void *dgamma,
                                   void *dbeta, void *dx, int B, int M, int N, int K, int inner,
                                   int outer, int block_size, int activation, int flags,
                                   void *workspace, size_t workspace_bytes, void *stream);
/* How often a wait inside the one-launch chain kernels polls before it gives up (default 200000,
 * about a second).  A negative value makes the kernels never signal completion to each other, so
 * that every wait runs out after -limit polls: the give-up path, for tests.  Returns the old value. */
int gridnet_hip_chain_set_spin_limit(int limit);

#ifdef __cplusplus
}
#endif
#endif /* GRIDNET_HIP_H */
