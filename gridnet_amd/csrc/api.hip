// extern "C" surface of libgridnet_hip.so: argument validation, error messages, dispatch.
// Nothing here allocates, frees or synchronises; every entry point only enqueues kernels.

#include <cstring>

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

using namespace gridnet;

extern "C" {

int gridnet_hip_version(void) { return 1; }

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

size_t gridnet_hip_backward_workspace_bytes(int dtype, int B, int M, int N, int K, int inner,
                                            int block_size, int normalize) {
    StepArgs a{};
    a.dtype = dtype; a.B = B; a.M = M; a.N = N; a.K = K; a.inner = inner;
    a.block_size = block_size; a.normalize = normalize != 0; a.activation = GRIDNET_ACT_RELU;
    if (B <= 0 || M <= 0 || N <= 0 || K <= 0) return 0;
    if (step_fast_supports(a, true)) return step_fast_backward_workspace(a);
    return 0;
}

int gridnet_hip_backward(int dtype, const void *weight, const void *bias, const void *scale,
                         const void *x, const void *dy, void *dweight, void *dbias, void *dscale,
                         void *dx, int B, int M, int N, int K, int inner, int block_size,
                         double eps, int normalize, int activation, int flags, void *workspace,
                         size_t workspace_bytes, void *stream) {
    StepArgs a{};
    a.dtype = dtype; a.weight = weight; a.bias = bias; a.scale = scale; a.x = x; a.dy = dy;
    a.dweight = dweight; a.dbias = dbias; a.dscale = dscale; a.dx = dx;
    a.B = B; a.M = M; a.N = N; a.K = K; a.inner = inner; a.block_size = block_size;
    a.eps = eps; a.normalize = normalize != 0; a.activation = activation; a.flags = flags;
    a.workspace = workspace; a.workspace_bytes = workspace_bytes;
    if (int rc = check_step(a, true)) return rc;
    if (B == 0) return GRIDNET_OK;
    hipStream_t st = (hipStream_t)stream;
    if (step_fast_supports(a, true)) {
        const size_t need = step_fast_backward_workspace(a);
        if (need && (!workspace || workspace_bytes < need))
            return fail(GRIDNET_ERR_WORKSPACE, "backward needs %zu bytes of workspace, got %zu", need,
                        workspace ? workspace_bytes : (size_t)0);
        return step_backward_fast(a, st);
    }
    return step_backward_generic(a, st);
}

int gridnet_hip_forward_gated(int dtype, const void *weight, const void *bias, const void *x, void *y,
                              int B, int M, int N, int K, int inner, int block_size, int activation,
                              void *stream) {
    StepArgs a{};
    a.dtype = dtype; a.weight = weight; a.bias = bias; a.x = x; a.y = y;
    a.B = B; a.M = M; a.N = N; a.K = K; a.inner = inner; a.block_size = block_size;
    a.activation = activation;
    if (int rc = check_step(a, false, true)) return rc;
    if (B == 0) return GRIDNET_OK;
    return gated_forward(a, (hipStream_t)stream);
}

int gridnet_hip_backward_gated(int dtype, const void *weight, const void *bias, const void *x,
                               const void *dy, void *dweight, void *dbias, void *dx, int B, int M,
                               int N, int K, int inner, int block_size, int activation, int flags,
                               void *stream) {
    StepArgs a{};
    a.dtype = dtype; a.weight = weight; a.bias = bias; a.x = x; a.dy = dy;
    a.dweight = dweight; a.dbias = dbias; a.dx = dx;
    a.B = B; a.M = M; a.N = N; a.K = K; a.inner = inner; a.block_size = block_size;
    a.activation = activation; a.flags = flags;
    if (int rc = check_step(a, true, true)) return rc;
    if ((long)M * N * K * 54 >= (1L << 31))
        return fail(GRIDNET_ERR_ARGUMENT, "grid too large: 54*M*N*K must be below 2^31");
    if (B == 0) return GRIDNET_OK;
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

}  // extern "C"
