// Host-side argument bundles and the launch functions each .hip file provides.
#pragma once

#include <hip/hip_runtime.h>

#include <cstddef>

namespace gridnet {

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
};

// How a workgroup commits its parameter gradients.
enum ParamMode {
    kParamStore = 0,         // sole owner of the cells, output uninitialised: plain store
    kParamAddExclusive = 1,  // sole owner, output holds a prior sum: read-add-write
    kParamAtomic = 2         // several workgroups (batch chunks) share the cells
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

// step_fast.hip: fp32, normalize=false; return -1 when the problem is outside what they cover
bool step_fast_supports(const StepArgs &a, bool backward);
size_t step_fast_backward_workspace(const StepArgs &a);
int step_forward_fast(const StepArgs &a, hipStream_t st);
int step_backward_fast(const StepArgs &a, hipStream_t st);

// gated_generic.hip (weight [27,2,M,N,K], bias [2,M,N,K]; scale, eps, normalize unused)
int gated_forward(const StepArgs &a, hipStream_t st);
int gated_backward(const StepArgs &a, hipStream_t st);

// layernorm.hip
size_t layernorm_workspace(int dtype, int B, long n);
int layernorm_forward(const LayerNormArgs &a, hipStream_t st);
int layernorm_backward(const LayerNormArgs &a, hipStream_t st);

}  // namespace gridnet
