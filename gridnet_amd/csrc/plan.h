// Host-side launch planning shared by the tuned kernels' launchers: how many CUs the current
// device has, how the batch is dealt to workgroups, and a zero-fill that is a kernel (a
// hipMemsetAsync node in a captured graph has given wrong results on replay on this platform).
// Every translation unit that includes this gets its own copy (internal linkage).
#ifndef GRIDNET_PLAN_H
#define GRIDNET_PLAN_H

#include "common.h"

namespace gridnet {
namespace {

int plan_device_cus() {
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

// The batch is dealt to workgroups in chunks, a chunk is walked `nslot` elements at a time.
// `resident` = workgroups the chip holds at once: when the blocks alone do not fill it the batch
// is split so that the grid is one full round of workgroups; `whole`: never split.
void plan_batch_chunks(int B, int nblk, int nslot, int resident, bool whole, int &nchunk, int &chunk_len) {
    nchunk = whole ? 1 : resident / nblk;
    const int max_chunks = (B + nslot - 1) / nslot;
    if (nchunk > max_chunks) nchunk = max_chunks;
    if (nchunk < 1) nchunk = 1;
    chunk_len = (B + nchunk - 1) / nchunk;
    chunk_len = (chunk_len + nslot - 1) / nslot * nslot;
    nchunk = (B + chunk_len - 1) / chunk_len;
}

__global__ void plan_fill_zero_f32(float *p, long n) {
    long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    const long stride = (long)gridDim.x * blockDim.x;
    for (; i < n; i += stride) p[i] = 0.f;
}

int plan_fill_zero(float *p, long n, hipStream_t st) {
    if (n <= 0) return GRIDNET_OK;
    long blocks = (n + 1023) / 1024;
    if (blocks > 8192) blocks = 8192;
    hipLaunchKernelGGL(plan_fill_zero_f32, dim3((unsigned)blocks), dim3(256), 0, st, p, n);
    return check_launch("fill_zero");
}

}  // namespace
}  // namespace gridnet

#endif  // GRIDNET_PLAN_H
