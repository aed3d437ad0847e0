// extern "C" surface of libgridnet_hip.so: argument validation, error messages, dispatch.
// Nothing here allocates, frees or synchronises; every entry point only enqueues kernels.

#include <cstring>
#include <mutex>

#include "common.h"
#include "launch.h"

namespace gridnet {

char *error_buffer() {
    static thread_local char buf[512] = {0};
    return buf;
}

int fail(int status, const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(error_buffer(), 512, fmt, ap);
    va_end(ap);
    return status;
}

int check_launch(const char *what) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess)
        return fail(GRIDNET_ERR_LAUNCH, "%s: launch failed: %s", what, hipGetErrorString(e));
    return GRIDNET_OK;
}

namespace {

int check_step(const StepArgs &a, bool backward, bool gated = false) {
    if (a.dtype != GRIDNET_F32 && a.dtype != GRIDNET_F64)
        return fail(GRIDNET_ERR_ARGUMENT, "unsupported dtype id %d", a.dtype);
    if (a.B < 0 || a.M <= 0 || a.N <= 0 || a.K <= 0)
        return fail(GRIDNET_ERR_ARGUMENT, "bad shape B=%d M=%d N=%d K=%d", a.B, a.M, a.N, a.K);
    if (a.block_size != 4 && a.block_size != 8)
        return fail(GRIDNET_ERR_ARGUMENT, "block_size %d not supported (4 or 8)", a.block_size);
    if (a.M % a.block_size || a.N % a.block_size || a.K % a.block_size)
        return fail(GRIDNET_ERR_ARGUMENT, "block_size=%d incompatible with grid (%d, %d, %d)",
                    a.block_size, a.M, a.N, a.K);
    if (a.inner < 0) return fail(GRIDNET_ERR_ARGUMENT, "negative inner iteration count %d", a.inner);
    if (backward && a.inner > kMaxBackwardIters)
        return fail(GRIDNET_ERR_ITERATIONS, "cannot backprop through more than 32 inner iterations");
    if (a.activation < GRIDNET_ACT_RELU || a.activation > GRIDNET_ACT_TANH)
        return fail(GRIDNET_ERR_ACTIVATION, "unknown activation function: id %d", a.activation);
    // 32-bit cell indexing inside a sample; 64-bit across the batch
    if ((long)a.M * a.N * a.K * 27 >= (1L << 31))
        return fail(GRIDNET_ERR_ARGUMENT, "grid too large: 27*M*N*K must be below 2^31");
    if (a.B == 0) return GRIDNET_OK;
    if (!a.weight || !a.bias || (!a.scale && !gated) || !a.x)
        return fail(GRIDNET_ERR_ARGUMENT, "null input pointer");
    if (!backward && !a.y) return fail(GRIDNET_ERR_ARGUMENT, "null output pointer");
    if (backward && (!a.dy || !a.dweight || !a.dbias || (!a.dscale && !gated) || !a.dx))
        return fail(GRIDNET_ERR_ARGUMENT, "null gradient pointer");
    return GRIDNET_OK;
}

}  // namespace
}  // namespace gridnet

// ---- scratch for the entry point that takes no workspace ----------------------------------
// One array per GPU (every device that loads this code object gets its own copy at its own
// address), held until the process ends.  In host code the array's name is only a handle for
// hipGetSymbolAddress, not a device address: kernels are given the looked-up pointer.
static __device__ __align__(256) unsigned char scratch[GRIDNET_STATIC_SCRATCH_BYTES];

namespace gridnet {
namespace {

constexpr int kMaxDevices = 64;
std::mutex scratch_lock;
void *scratch_ptr[kMaxDevices];  // by device ordinal, looked up on first use with that device current

int static_scratch_pointer(void **out) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess || dev < 0 || dev >= kMaxDevices)
        return fail(GRIDNET_ERR_LAUNCH, "static scratch: no usable current device (%s, ordinal %d)",
                    hipGetErrorString(e), dev);
    std::lock_guard<std::mutex> hold(scratch_lock);
    if (!scratch_ptr[dev]) {
        void *p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !p)
            return fail(GRIDNET_ERR_LAUNCH, "static scratch: hipGetSymbolAddress failed on device %d: %s",
                        dev, hipGetErrorString(e));
        scratch_ptr[dev] = p;
    }
    *out = scratch_ptr[dev];
    return GRIDNET_OK;
}

}  // namespace
}  // namespace gridnet

using namespace gridnet;

extern "C" {

int gridnet_hip_version(void) { return 8; }  // 2: fused body; 3: residual forward and backward; 4: gated backward takes a workspace; 5: backward on static scratch; 6: chain backward, gradient copies for split batches; 7: whole chain in one launch; 8: fused forward with flags

const char *gridnet_hip_last_error(void) { return error_buffer(); }

int gridnet_hip_activation_id(const char *name) {
    if (name) {
        if (!strcmp(name, "relu")) return GRIDNET_ACT_RELU;
        if (!strcmp(name, "leaky_relu")) return GRIDNET_ACT_LEAKY_RELU;
        if (!strcmp(name, "silu")) return GRIDNET_ACT_SILU;
        if (!strcmp(name, "tanh")) return GRIDNET_ACT_TANH;
    }
    fail(GRIDNET_ERR_ACTIVATION, "unknown activation function: %s", name ? name : "(null)");
    return -1;
}

int gridnet_hip_forward(int dtype, const void *weight, const void *bias, const void *scale,
                        const void *x, void *y, int B, int M, int N, int K, int inner,
                        int block_size, double eps, int normalize, int activation, void *stream) {
    StepArgs a{};
    a.dtype = dtype; a.weight = weight; a.bias = bias; a.scale = scale; a.x = x; a.y = y;
    a.B = B; a.M = M; a.N = N; a.K = K; a.inner = inner; a.block_size = block_size;
    a.eps = eps; a.normalize = normalize != 0; a.activation = activation;
    if (int rc = check_step(a, false)) return rc;
    if (B == 0) return GRIDNET_OK;
    hipStream_t st = (hipStream_t)stream;
    if (step_fast_supports(a, false)) return step_forward_fast(a, st);
    return step_forward_generic(a, st);
}

// What lies behind the first `used` bytes of a workspace (rounded up to 256) is room for the
// gradient copies of a split batch (launch.h: StepArgs::slabs); callers that hand over only the
// required part get a batch that is split less, the result is the same.
static void give_slabs(StepArgs &a, void *workspace, size_t workspace_bytes, size_t used) {
    const size_t at = (used + 255) / 256 * 256;
    a.slabs = nullptr;
    a.slab_bytes = 0;
    if (workspace && workspace_bytes > at) {
        a.slabs = (char *)workspace + at;
        a.slab_bytes = workspace_bytes - at;
    }
}

size_t gridnet_hip_backward_workspace_bytes(int dtype, int B, int M, int N, int K, int inner,
                                            int block_size, int normalize) {
    StepArgs a{};
    a.dtype = dtype; a.B = B; a.M = M; a.N = N; a.K = K; a.inner = inner;
    a.block_size = block_size; a.normalize = normalize != 0; a.activation = GRIDNET_ACT_RELU;
    if (B <= 0 || M <= 0 || N <= 0 || K <= 0) return 0;
    if (!step_fast_supports(a, true)) return 0;
    const size_t slabs = step_fast_slab_bytes(a);
    return slabs ? (step_fast_backward_workspace(a) + 255) / 256 * 256 + slabs : step_fast_backward_workspace(a);
}

static int backward_step(int dtype, const void *weight, const void *bias, const void *scale,
                         const void *x, const void *dy, void *dweight, void *dbias, void *dscale,
                         void *dx, int B, int M, int N, int K, int inner, int block_size,
                         double eps, int normalize, int activation, int flags, void *workspace,
                         size_t workspace_bytes, void *stream, bool static_scratch) {
    StepArgs a{};
    a.dtype = dtype; a.weight = weight; a.bias = bias; a.scale = scale; a.x = x; a.dy = dy;
    a.dweight = dweight; a.dbias = dbias; a.dscale = dscale; a.dx = dx;
    a.B = B; a.M = M; a.N = N; a.K = K; a.inner = inner; a.block_size = block_size;
    a.eps = eps; a.normalize = normalize != 0; a.activation = activation; a.flags = flags;
    if (int rc = check_step(a, true)) return rc;
    if (B == 0) return GRIDNET_OK;
    hipStream_t st = (hipStream_t)stream;
    if (!step_fast_supports(a, true)) return step_backward_generic(a, st);  // needs no scratch
    const size_t need = step_fast_backward_workspace(a);
    if (static_scratch) {
        // sizes first: a problem that does not fit is refused before anything touches the device
        if (need > (size_t)GRIDNET_STATIC_SCRATCH_BYTES)
            return fail(GRIDNET_ERR_WORKSPACE,
                        "backward needs %zu bytes of scratch, the static array holds %zu: use "
                        "gridnet_hip_backward with a workspace",
                        need, (size_t)GRIDNET_STATIC_SCRATCH_BYTES);
        if (int rc = static_scratch_pointer(&workspace)) return rc;
        workspace_bytes = GRIDNET_STATIC_SCRATCH_BYTES;
    }
    if (need && (!workspace || workspace_bytes < need))
        return fail(GRIDNET_ERR_WORKSPACE, "backward needs %zu bytes of workspace, got %zu", need,
                    workspace ? workspace_bytes : (size_t)0);
    a.workspace = workspace; a.workspace_bytes = workspace_bytes;
    give_slabs(a, workspace, workspace_bytes, need);
    return step_backward_fast(a, st);
}

int gridnet_hip_backward(int dtype, const void *weight, const void *bias, const void *scale,
                         const void *x, const void *dy, void *dweight, void *dbias, void *dscale,
                         void *dx, int B, int M, int N, int K, int inner, int block_size,
                         double eps, int normalize, int activation, int flags, void *workspace,
                         size_t workspace_bytes, void *stream) {
    return backward_step(dtype, weight, bias, scale, x, dy, dweight, dbias, dscale, dx, B, M, N, K,
                         inner, block_size, eps, normalize, activation, flags, workspace,
                         workspace_bytes, stream, false);
}

int gridnet_hip_static_init(void) {
    void *unused = nullptr;
    return static_scratch_pointer(&unused);
}

int gridnet_hip_backward_static(int dtype, const void *weight, const void *bias, const void *scale,
                                const void *x, const void *dy, void *dweight, void *dbias,
                                void *dscale, void *dx, int B, int M, int N, int K, int inner,
                                int block_size, double eps, int normalize, int activation,
                                int flags, void *stream) {
    return backward_step(dtype, weight, bias, scale, x, dy, dweight, dbias, dscale, dx, B, M, N, K,
                         inner, block_size, eps, normalize, activation, flags, nullptr, 0, stream,
                         true);
}

int gridnet_hip_forward_gated(int dtype, const void *weight, const void *bias, const void *x, void *y,
                              int B, int M, int N, int K, int inner, int block_size, int activation,
                              void *stream) {
    StepArgs a{};
    a.dtype = dtype; a.weight = weight; a.bias = bias; a.x = x; a.y = y;
    a.B = B; a.M = M; a.N = N; a.K = K; a.inner = inner; a.block_size = block_size;
    a.activation = activation;
    if (int rc = check_step(a, false, true)) return rc;
    if ((long)M * N * K * 54 >= (1L << 31))
        return fail(GRIDNET_ERR_ARGUMENT, "grid too large: 54*M*N*K must be below 2^31");
    if (B == 0) return GRIDNET_OK;
    if (gated_fast_supports(a, false)) return gated_forward_fast(a, (hipStream_t)stream);
    return gated_forward(a, (hipStream_t)stream);
}

size_t gridnet_hip_backward_gated_workspace_bytes(int dtype, int B, int M, int N, int K, int inner,
                                                  int block_size) {
    StepArgs a{};
    a.dtype = dtype; a.B = B; a.M = M; a.N = N; a.K = K; a.inner = inner;
    a.block_size = block_size; a.activation = GRIDNET_ACT_RELU;
    if (B <= 0 || M <= 0 || N <= 0 || K <= 0) return 0;
    if (!gated_fast_supports(a, true)) return 0;
    const size_t slabs = gated_fast_slab_bytes(a);
    return slabs ? (gated_fast_backward_workspace(a) + 255) / 256 * 256 + slabs : gated_fast_backward_workspace(a);
}

int gridnet_hip_backward_gated(int dtype, const void *weight, const void *bias, const void *x,
                               const void *dy, void *dweight, void *dbias, void *dx, int B, int M,
                               int N, int K, int inner, int block_size, int activation, int flags,
                               void *workspace, size_t workspace_bytes, void *stream) {
    StepArgs a{};
    a.dtype = dtype; a.weight = weight; a.bias = bias; a.x = x; a.dy = dy;
    a.dweight = dweight; a.dbias = dbias; a.dx = dx;
    a.B = B; a.M = M; a.N = N; a.K = K; a.inner = inner; a.block_size = block_size;
    a.activation = activation; a.flags = flags;
    a.workspace = workspace; a.workspace_bytes = workspace_bytes;
    if (int rc = check_step(a, true, true)) return rc;
    if ((long)M * N * K * 54 >= (1L << 31))
        return fail(GRIDNET_ERR_ARGUMENT, "grid too large: 54*M*N*K must be below 2^31");
    if (B == 0) return GRIDNET_OK;
    if (gated_fast_supports(a, true)) {
        const size_t need = gated_fast_backward_workspace(a);
        if (!workspace || workspace_bytes < need)
            return fail(GRIDNET_ERR_WORKSPACE, "backward needs %zu bytes of workspace, got %zu", need,
                        workspace ? workspace_bytes : (size_t)0);
        give_slabs(a, workspace, workspace_bytes, need);
        return gated_backward_fast(a, (hipStream_t)stream);
    }
    return gated_backward(a, (hipStream_t)stream);
}

size_t gridnet_hip_layernorm_workspace_bytes(int dtype, int B, long n) {
    if (B <= 0 || n <= 0) return 0;
    return layernorm_workspace(dtype, B, n);
}

static int check_ln(const LayerNormArgs &a) {
    if (a.dtype != GRIDNET_F32 && a.dtype != GRIDNET_F64)
        return fail(GRIDNET_ERR_ARGUMENT, "unsupported dtype id %d", a.dtype);
    if (a.B < 0 || a.n <= 0) return fail(GRIDNET_ERR_ARGUMENT, "bad shape B=%d n=%ld", a.B, a.n);
    if (a.B == 0) return GRIDNET_OK;
    const size_t need = layernorm_workspace(a.dtype, a.B, a.n);
    if (!a.workspace || a.workspace_bytes < need)
        return fail(GRIDNET_ERR_WORKSPACE, "layernorm needs %zu bytes of workspace, got %zu", need,
                    a.workspace ? a.workspace_bytes : (size_t)0);
    return GRIDNET_OK;
}

int gridnet_hip_layernorm_forward(int dtype, const void *x, const void *gamma, const void *beta,
                                  void *y, void *mean, void *rstd, int B, long n, double eps,
                                  void *workspace, size_t workspace_bytes, void *stream) {
    LayerNormArgs a{};
    a.dtype = dtype; a.x = x; a.gamma = gamma; a.beta = beta; a.y = y; a.mean = mean; a.rstd = rstd;
    a.B = B; a.n = n; a.eps = eps; a.workspace = workspace; a.workspace_bytes = workspace_bytes;
    if (int rc = check_ln(a)) return rc;
    if (B == 0) return GRIDNET_OK;
    if (!x || !gamma || !beta || !y || !mean || !rstd)
        return fail(GRIDNET_ERR_ARGUMENT, "null pointer");
    return layernorm_forward(a, (hipStream_t)stream);
}

int gridnet_hip_layernorm_backward(int dtype, const void *dy, const void *x, const void *gamma,
                                   const void *mean, const void *rstd, void *dx, void *dgamma,
                                   void *dbeta, int B, long n, int flags, void *workspace,
                                   size_t workspace_bytes, void *stream) {
    LayerNormArgs a{};
    a.dtype = dtype; a.dy = dy; a.x = x; a.gamma = gamma; a.mean_in = mean; a.rstd_in = rstd;
    a.dx = dx; a.dgamma = dgamma; a.dbeta = dbeta; a.B = B; a.n = n; a.flags = flags;
    a.workspace = workspace; a.workspace_bytes = workspace_bytes;
    if (int rc = check_ln(a)) return rc;
    if (B == 0) return GRIDNET_OK;
    if (!dy || !x || !gamma || !mean || !rstd || !dx || !dgamma || !dbeta)
        return fail(GRIDNET_ERR_ARGUMENT, "null pointer");
    return layernorm_backward(a, (hipStream_t)stream);
}

// ---- network body with the LayerNorm folded into the step kernels -------------------------
static int check_fused(const StepArgs &a, bool backward) {
    if (a.dtype != GRIDNET_F32)
        return fail(GRIDNET_ERR_ARGUMENT, "the fused body is float32 only (dtype id %d)", a.dtype);
    if (int rc = check_step(a, backward)) return rc;
    if (a.inner < 1)
        return fail(GRIDNET_ERR_ARGUMENT, "the fused body needs at least one inner iteration");
    if (!step_fast_supports(a, backward))
        return fail(GRIDNET_ERR_ARGUMENT,
                    "the fused body does not cover this problem (inner=%d block_size=%d): use the "
                    "step and LayerNorm entry points",
                    a.inner, a.block_size);
    return GRIDNET_OK;
}

static size_t fused_forward_workspace(const StepArgs &a) {
    const size_t nblk = (size_t)(a.M / a.block_size) * (a.N / a.block_size) * (a.K / a.block_size);
    return (size_t)a.B * nblk * step_fast_forward_parts(a.block_size) * 2 * sizeof(float);
}

// backward workspace: [D of every cell | partial sums of the cross-block kernel]
static size_t fused_backward_dsum(const StepArgs &a) {
    return (step_fast_backward_workspace(a) + 255) / 256 * 256;
}
static size_t fused_backward_parts(const StepArgs &a) {
    const size_t nblk = (size_t)(a.M / a.block_size) * (a.N / a.block_size) * (a.K / a.block_size);
    size_t pairs = nblk * step_fast_backward_parts(a.block_size);
    if (bwd_rows_supports(a)) {  // one inner iteration, by rows: a pair per wave of its first kernel
        StepArgs plain = a;
        plain.ln.residual = 0;
        const size_t rows = (size_t)bwd_rows_pairs(plain);
        if (rows > pairs) pairs = rows;
    }
    return (size_t)a.B * pairs * 2 * sizeof(float);
}

size_t gridnet_hip_fused_workspace_bytes(int B, int M, int N, int K, int inner, int block_size,
                                         int backward) {
    StepArgs a{};
    a.dtype = GRIDNET_F32; a.B = B; a.M = M; a.N = N; a.K = K; a.inner = inner;
    a.block_size = block_size; a.activation = GRIDNET_ACT_RELU;
    if (B <= 0 || M <= 0 || N <= 0 || K <= 0 || (block_size != 4 && block_size != 8)) return 0;
    if (!backward) return fused_forward_workspace(a);
    const size_t need = fused_backward_dsum(a) + fused_backward_parts(a), slabs = step_fast_slab_bytes(a);
    return slabs ? (need + 255) / 256 * 256 + slabs : need;
}

static int fused_forward(int dtype, const void *weight, const void *bias, const void *scale,
                         const void *gamma, const void *beta, const void *x, const void *x_stats,
                         void *y_raw, void *y_stats, int B, int M, int N, int K, int inner,
                         int block_size, double ln_eps, int activation, void *workspace,
                         size_t workspace_bytes, void *stream, int residual, int walk_reverse = 0) {
    StepArgs a{};
    a.dtype = dtype; a.weight = weight; a.bias = bias; a.scale = scale; a.x = x; a.y = y_raw;
    a.B = B; a.M = M; a.N = N; a.K = K; a.inner = inner; a.block_size = block_size;
    a.activation = activation;
    if (int rc = check_fused(a, false)) return rc;
    if (B == 0) return GRIDNET_OK;
    if (!gamma || !beta || !y_stats) return fail(GRIDNET_ERR_ARGUMENT, "null pointer");
    if (residual && !x_stats)
        return fail(GRIDNET_ERR_ARGUMENT, "the residual form normalises its input: x_stats is required");
    const size_t need = fused_forward_workspace(a);
    if (!workspace || workspace_bytes < need)
        return fail(GRIDNET_ERR_WORKSPACE, "fused forward needs %zu bytes of workspace, got %zu", need,
                    workspace ? workspace_bytes : (size_t)0);
    hipStream_t st = (hipStream_t)stream;
    a.ln.gamma = (const float *)gamma;
    a.ln.beta = (const float *)beta;
    a.ln.x_stats = (const float *)x_stats;
    a.ln.y_part = (float *)workspace;
    a.ln.residual = residual;
    a.ln.walk_reverse = walk_reverse;
    if (int rc = step_forward_fast(a, st)) return rc;
    return layernorm_finalize_stats((const float *)workspace, step_fast_forward_pairs(a),
                                    step_fast_forward_pair_count(a), (float *)y_stats, B, ln_eps, st);
}

int gridnet_hip_fused_forward(int dtype, const void *weight, const void *bias, const void *scale,
                              const void *gamma, const void *beta, const void *x,
                              const void *x_stats, void *y_raw, void *y_stats, int B, int M, int N,
                              int K, int inner, int block_size, double ln_eps, int activation,
                              void *workspace, size_t workspace_bytes, void *stream) {
    return fused_forward(dtype, weight, bias, scale, gamma, beta, x, x_stats, y_raw, y_stats, B, M, N,
                         K, inner, block_size, ln_eps, activation, workspace, workspace_bytes, stream, 0);
}

int gridnet_hip_fused_forward_flags(int dtype, const void *weight, const void *bias, const void *scale,
                                    const void *gamma, const void *beta, const void *x,
                                    const void *x_stats, void *y, void *y_stats, int B, int M, int N,
                                    int K, int inner, int block_size, double ln_eps, int activation,
                                    int flags, void *workspace, size_t workspace_bytes, void *stream) {
    if (flags & ~(GRIDNET_FUSED_RESIDUAL | GRIDNET_FUSED_WALK_REVERSE))
        return fail(GRIDNET_ERR_ARGUMENT, "unknown flag bits: %d", flags);
    return fused_forward(dtype, weight, bias, scale, gamma, beta, x, x_stats, y, y_stats, B, M, N, K, inner,
                         block_size, ln_eps, activation, workspace, workspace_bytes, stream,
                         (flags & GRIDNET_FUSED_RESIDUAL) ? 1 : 0, (flags & GRIDNET_FUSED_WALK_REVERSE) ? 1 : 0);
}

int gridnet_hip_fused_forward_residual(int dtype, const void *weight, const void *bias,
                                       const void *scale, const void *gamma, const void *beta,
                                       const void *x, const void *x_stats, void *y, void *y_stats,
                                       int B, int M, int N, int K, int inner, int block_size,
                                       double ln_eps, int activation, void *workspace,
                                       size_t workspace_bytes, void *stream) {
    return fused_forward(dtype, weight, bias, scale, gamma, beta, x, x_stats, y, y_stats, B, M, N, K,
                         inner, block_size, ln_eps, activation, workspace, workspace_bytes, stream, 1);
}

int gridnet_hip_layernorm_apply(int dtype, const void *x, const void *stats, const void *gamma,
                                const void *beta, void *y, int B, long n, void *stream) {
    if (dtype != GRIDNET_F32)
        return fail(GRIDNET_ERR_ARGUMENT, "layernorm_apply is float32 only (dtype id %d)", dtype);
    if (B < 0 || n <= 0) return fail(GRIDNET_ERR_ARGUMENT, "bad shape B=%d n=%ld", B, n);
    if (B == 0) return GRIDNET_OK;
    if (!x || !stats || !gamma || !beta || !y) return fail(GRIDNET_ERR_ARGUMENT, "null pointer");
    return layernorm_apply_stats((const float *)x, (const float *)stats, (const float *)gamma,
                                 (const float *)beta, (float *)y, B, n, (hipStream_t)stream);
}

int gridnet_hip_layernorm_backward_sums(int dtype, const void *dy, const void *x, const void *stats,
                                        const void *gamma, void *sums, int B, long n,
                                        void *workspace, size_t workspace_bytes, void *stream) {
    if (dtype != GRIDNET_F32)
        return fail(GRIDNET_ERR_ARGUMENT, "layernorm_backward_sums is float32 only (dtype id %d)", dtype);
    if (B < 0 || n <= 0) return fail(GRIDNET_ERR_ARGUMENT, "bad shape B=%d n=%ld", B, n);
    if (B == 0) return GRIDNET_OK;
    if (!dy || !x || !stats || !gamma || !sums) return fail(GRIDNET_ERR_ARGUMENT, "null pointer");
    const size_t need = layernorm_workspace(GRIDNET_F32, B, n);
    if (!workspace || workspace_bytes < need)
        return fail(GRIDNET_ERR_WORKSPACE, "layernorm needs %zu bytes of workspace, got %zu", need,
                    workspace ? workspace_bytes : (size_t)0);
    return layernorm_backward_sums((const float *)dy, (const float *)x, (const float *)stats,
                                   (const float *)gamma, (float *)sums, B, n, (float *)workspace,
                                   (hipStream_t)stream);
}

static int fused_backward(int dtype, const void *weight, const void *bias, const void *scale,
                          const void *gamma, const void *beta, const void *x, const void *x_stats,
                          const void *dy, const void *y_raw, const void *y_stats, const void *y_sums,
                          void *dweight, void *dbias, void *dscale, void *dgamma, void *dbeta,
                          void *dx, void *x_sums, int B, int M, int N, int K, int inner,
                          int block_size, int activation, int flags, void *workspace,
                          size_t workspace_bytes, void *stream, int residual, const void *g_prev,
                          void *g_out) {
    StepArgs a{};
    a.dtype = dtype; a.weight = weight; a.bias = bias; a.scale = scale; a.x = x; a.dy = dy;
    a.dweight = dweight; a.dbias = dbias; a.dscale = dscale; a.dx = dx;
    a.B = B; a.M = M; a.N = N; a.K = K; a.inner = inner; a.block_size = block_size;
    a.activation = activation;
    a.flags = (flags & GRIDNET_OVERWRITE_PARAMS) | GRIDNET_OVERWRITE_DX;  // dx is always written
    a.ln.gamma = (const float *)gamma;  // before the checks: the LDS budget depends on it
    if (int rc = check_fused(a, true)) return rc;
    if (B == 0) return GRIDNET_OK;
    if (!gamma || !beta || !dgamma || !dbeta) return fail(GRIDNET_ERR_ARGUMENT, "null pointer");
    if (!residual) {
        if (!y_raw || !y_stats || !y_sums) return fail(GRIDNET_ERR_ARGUMENT, "null pointer");
    } else {
        // the last step of a chain is handed G' itself; every other one forms it
        const bool given = !y_raw;
        if (given ? (y_stats || y_sums || g_prev || g_out) : (!y_stats || !y_sums || !g_prev || !g_out))
            return fail(GRIDNET_ERR_ARGUMENT,
                        "y_raw, y_stats, y_sums, g_prev and g_out go together: all or none");
        if (!x_stats)
            return fail(GRIDNET_ERR_ARGUMENT, "the residual form normalises its input: x_stats is required");
    }
    if ((x_stats == nullptr) != (x_sums == nullptr))
        return fail(GRIDNET_ERR_ARGUMENT, "x_stats and x_sums go together: both or neither");
    const size_t dsum_bytes = fused_backward_dsum(a), need = dsum_bytes + fused_backward_parts(a);
    if (!workspace || workspace_bytes < need)
        return fail(GRIDNET_ERR_WORKSPACE, "fused backward needs %zu bytes of workspace, got %zu", need,
                    workspace ? workspace_bytes : (size_t)0);
    hipStream_t st = (hipStream_t)stream;
    a.workspace = workspace; a.workspace_bytes = dsum_bytes;
    give_slabs(a, workspace, workspace_bytes, need);
    a.ln.beta = (const float *)beta;
    a.ln.x_stats = (const float *)x_stats;
    a.ln.y_raw = (const float *)y_raw;
    a.ln.y_stats = (const float *)y_stats;
    a.ln.y_sums = (const float *)y_sums;
    a.ln.dgamma = (float *)dgamma;
    a.ln.dbeta = (float *)dbeta;
    a.ln.x_part = x_stats ? (float *)((char *)workspace + dsum_bytes) : nullptr;
    a.ln.residual = residual;
    a.ln.g_prev = (const float *)g_prev;
    a.ln.g_out = (float *)g_out;
    a.ln.x_sums = (float *)x_sums;
    if (int rc = step_backward_fast(a, st)) return rc;
    if (!x_stats || bwd_rows_leaves_sums(a)) return GRIDNET_OK;
    return layernorm_finalize_sums(a.ln.x_part, step_fast_backward_pairs(a),
                                   (long)M * N * K, (float *)x_sums, B, st);
}

int gridnet_hip_fused_backward(int dtype, const void *weight, const void *bias, const void *scale,
                               const void *gamma, const void *beta, const void *x,
                               const void *x_stats, const void *dy, const void *y_raw,
                               const void *y_stats, const void *y_sums, void *dweight, void *dbias,
                               void *dscale, void *dgamma, void *dbeta, void *dx, void *x_sums, int B,
                               int M, int N, int K, int inner, int block_size, int activation,
                               int flags, void *workspace, size_t workspace_bytes, void *stream) {
    return fused_backward(dtype, weight, bias, scale, gamma, beta, x, x_stats, dy, y_raw, y_stats,
                          y_sums, dweight, dbias, dscale, dgamma, dbeta, dx, x_sums, B, M, N, K, inner,
                          block_size, activation, flags, workspace, workspace_bytes, stream, 0, nullptr,
                          nullptr);
}

int gridnet_hip_fused_backward_residual(int dtype, const void *weight, const void *bias,
                                        const void *scale, const void *gamma, const void *beta,
                                        const void *x, const void *x_stats, const void *dy,
                                        const void *y_raw, const void *y_stats, const void *y_sums,
                                        const void *g_prev, void *g_out, void *dweight, void *dbias,
                                        void *dscale, void *dgamma, void *dbeta, void *dx,
                                        void *x_sums, int B, int M, int N, int K, int inner,
                                        int block_size, int activation, int flags, void *workspace,
                                        size_t workspace_bytes, void *stream) {
    return fused_backward(dtype, weight, bias, scale, gamma, beta, x, x_stats, dy, y_raw, y_stats,
                          y_sums, dweight, dbias, dscale, dgamma, dbeta, dx, x_sums, B, M, N, K, inner,
                          block_size, activation, flags, workspace, workspace_bytes, stream, 1, g_prev,
                          g_out);
}

int gridnet_hip_chain_supported(int dtype, int inner, int block_size, int normalize) {
    StepArgs a{};
    a.dtype = dtype; a.inner = inner; a.block_size = block_size; a.normalize = normalize != 0;
    return chain_supports(a) ? 1 : 0;
}

size_t gridnet_hip_chain_halo_floats(int B, int M, int N, int K, int block_size) {
    if (B <= 0 || M <= 0 || N <= 0 || K <= 0 || block_size != 8) return 0;
    StepArgs a{};
    a.B = B; a.M = M; a.N = N; a.K = K; a.block_size = block_size;
    return chain_halo_floats(a);
}

int gridnet_hip_chain_backward(int dtype, const void *weight, const void *bias, const void *scale,
                               const void *gamma, const void *beta, const void *x,
                               const void *x_stats, const void *dy, const void *y_raw,
                               const void *y_stats, const void *y_sums, const void *halo_in,
                               void *halo_out, void *dweight, void *dbias, void *dscale, void *dgamma,
                               void *dbeta, void *dx, void *x_sums, int B, int M, int N, int K,
                               int inner, int block_size, int activation, int flags, void *workspace,
                               size_t workspace_bytes, void *stream) {
    StepArgs a{};
    a.dtype = dtype; a.weight = weight; a.bias = bias; a.scale = scale;
    a.x = x; a.dy = dy; a.dweight = dweight; a.dbias = dbias; a.dscale = dscale; a.dx = dx;
    a.B = B; a.M = M; a.N = N; a.K = K; a.inner = inner; a.block_size = block_size;
    a.activation = activation;
    a.flags = (flags & GRIDNET_OVERWRITE_PARAMS) | GRIDNET_OVERWRITE_DX;  // dx is always written
    a.ln.gamma = (const float *)gamma;
    if (!chain_supports(a))
        return fail(GRIDNET_ERR_ARGUMENT,
                    "the chain entry points cover float32, block_size 8 and 1 to 8 inner iterations "
                    "(dtype id %d, block_size %d, inner %d): use gridnet_hip_fused_backward",
                    dtype, block_size, inner);
    if (int rc = check_fused(a, true)) return rc;
    if (B == 0) return GRIDNET_OK;
    if (!gamma || !beta || !dgamma || !dbeta || !y_raw || !y_stats || !y_sums)
        return fail(GRIDNET_ERR_ARGUMENT, "null pointer");
    if ((x_stats == nullptr) != (x_sums == nullptr))
        return fail(GRIDNET_ERR_ARGUMENT, "x_stats and x_sums go together: both or neither");
    if (halo_out && !x_stats)
        return fail(GRIDNET_ERR_ARGUMENT,
                    "an unfinished dx (halo_out) is for a step whose input passes a LayerNorm: "
                    "x_stats and x_sums are required");
    const size_t dsum_bytes = fused_backward_dsum(a), need = dsum_bytes + fused_backward_parts(a);
    if (!workspace || workspace_bytes < need)
        return fail(GRIDNET_ERR_WORKSPACE, "chain backward needs %zu bytes of workspace, got %zu", need,
                    workspace ? workspace_bytes : (size_t)0);
    hipStream_t st = (hipStream_t)stream;
    a.workspace = workspace; a.workspace_bytes = dsum_bytes;
    give_slabs(a, workspace, workspace_bytes, need);
    a.ln.beta = (const float *)beta;
    a.ln.x_stats = (const float *)x_stats;
    a.ln.y_raw = (const float *)y_raw;
    a.ln.y_stats = (const float *)y_stats;
    a.ln.y_sums = (const float *)y_sums;
    a.ln.dgamma = (float *)dgamma;
    a.ln.dbeta = (float *)dbeta;
    a.ln.x_part = x_stats ? (float *)((char *)workspace + dsum_bytes) : nullptr;
    a.ln.halo_in = (const float *)halo_in;
    a.ln.halo_out = (float *)halo_out;
    if (int rc = chain_backward(a, st)) return rc;
    if (!x_stats) return GRIDNET_OK;
    // the sums come from chain_bwd itself (a pair per block) when dx is left unfinished, from the
    // cross-block kernel otherwise
    const int nblk = (M / block_size) * (N / block_size) * (K / block_size);
    return layernorm_finalize_sums(a.ln.x_part, halo_out ? nblk : step_fast_cross_pairs(a),
                                   (long)M * N * K, (float *)x_sums, B, st);
}

static int chain_spin_limit = 200000;

int gridnet_hip_chain_set_spin_limit(int limit) {
    const int old = chain_spin_limit;
    chain_spin_limit = limit;
    return old;
}

int gridnet_hip_chain_all_supported(int dtype, int B, int M, int N, int K, int inner, int outer,
                                    int block_size, int normalize) {
    if (dtype != GRIDNET_F32 || block_size != 8 || normalize) return 0;
    return chain_all_supports(B, M, N, K, inner, outer) ? 1 : 0;
}

size_t gridnet_hip_chain_all_workspace_bytes(int B, int M, int N, int K, int inner, int outer,
                                             int block_size) {
    if (B <= 0 || M <= 0 || N <= 0 || K <= 0 || outer <= 0 || block_size != 8 || M % 8 || N % 8 || K % 8)
        return 0;
    ChainAll c{};
    c.B = B; c.M = M; c.N = N; c.K = K; c.inner = inner; c.outer = outer;
    return chain_all_workspace(c);
}

int gridnet_hip_chain_backward_all(int dtype, const void *weight, const void *bias, const void *scale,
                                   const void *gamma, const void *beta, const void *x0,
                                   const void *y_raw, const void *stats, const void *dy,
                                   void *dweight, void *dbias, void *dscale, void *dgamma,
                                   void *dbeta, void *dx, int B, int M, int N, int K, int inner,
                                   int outer, int block_size, int activation, int flags,
                                   void *workspace, size_t workspace_bytes, void *stream) {
    StepArgs a{};
    a.dtype = dtype; a.weight = weight; a.bias = bias; a.scale = scale; a.x = x0; a.dy = dy;
    a.dweight = dweight; a.dbias = dbias; a.dscale = dscale; a.dx = dx;
    a.B = B; a.M = M; a.N = N; a.K = K; a.inner = inner; a.block_size = block_size;
    a.activation = activation;
    if (dtype != GRIDNET_F32 || block_size != 8)
        return fail(GRIDNET_ERR_ARGUMENT, "the one-launch chain is float32 with block_size 8 (dtype id %d, block_size %d)",
                    dtype, block_size);
    if (int rc = check_step(a, true)) return rc;
    if (!chain_all_supports(B, M, N, K, inner, outer))
        return fail(GRIDNET_ERR_ARGUMENT,
                    "the one-launch chain does not cover this problem (B=%d grid %dx%dx%d inner=%d outer=%d): "
                    "see gridnet_hip_chain_all_supported; use gridnet_hip_chain_backward",
                    B, M, N, K, inner, outer);
    if (!gamma || !beta || !y_raw || !stats || !dgamma || !dbeta)
        return fail(GRIDNET_ERR_ARGUMENT, "null pointer");
    ChainAll c{};
    c.weight = (const float *)weight; c.bias = (const float *)bias; c.scale = (const float *)scale;
    c.gamma = (const float *)gamma; c.beta = (const float *)beta;
    c.x0 = (const float *)x0; c.y_raw = (const float *)y_raw; c.stats = (const float *)stats;
    c.dy = (const float *)dy;
    c.dweight = (float *)dweight; c.dbias = (float *)dbias; c.dscale = (float *)dscale;
    c.dgamma = (float *)dgamma; c.dbeta = (float *)dbeta; c.dx = (float *)dx;
    c.B = B; c.M = M; c.N = N; c.K = K; c.inner = inner; c.outer = outer;
    c.activation = activation; c.flags = flags;
    c.workspace = workspace; c.workspace_bytes = workspace_bytes;
    c.spin_limit = chain_spin_limit;
    const size_t need = chain_all_workspace(c);
    if (!workspace || workspace_bytes < need)
        return fail(GRIDNET_ERR_WORKSPACE, "the one-launch chain needs %zu bytes of workspace, got %zu", need,
                    workspace ? workspace_bytes : (size_t)0);
    return chain_backward_all(c, (hipStream_t)stream);
}

}  // extern "C"
