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

// ---- parameter gradients of a batch that is split over workgroups -----------------------------
// On grids with fewer blocks than the chip has CUs the batch of a block is dealt to several
// workgroups.  Each of them leaves its share of the gradient arrays in a copy of its own (a
// "slab": the arrays one behind the other, `planes` x cells floats) with plain stores, and one
// small kernel adds the copies in chunk order into the caller's arrays: no atomics, the same bits
// on every run.
struct SlabTargets {
    float *dst[5];   // the caller's gradient arrays, in slab order
    long end[5];     // end of each array within a slab, in floats (multiples of 4)
    int count;
};

// The slabs are 256-byte aligned and read as 16-byte vectors.  The caller's arrays are accessed as
// 16-byte vectors too although the C ABI asks them to be aligned to their element size only:
// gfx950 serves global accesses at any 4-byte alignment (a misaligned vector costs a second
// request, nothing else); tests/test_gpu_alignment.py runs this with arrays 4 bytes off.
// Work for spare workgroups of the kernel below: the last step of the LayerNorm backward's sums
// (common.h), one workgroup per sample, where those sums are ready when the gradient copies are.
// It saves a launch of its own (4.4 us, a thirtieth of a training step with one inner iteration).
struct SumsJob {
    const float *part;  // [B, parts, 2]
    int parts, B;       // B = 0: no job
    long n;
    float *sums;        // [B, 2]
};

__global__ __launch_bounds__(256) void plan_reduce_slabs_f32(const float *slabs, int ncopies, long stride,
                                                             SlabTargets t, long total4, int accumulate,
                                                             int reduce_blocks, SumsJob job) {
    if ((int)blockIdx.x >= reduce_blocks) {
        __shared__ double red[256 / kWave][2];
        finalize_sums_of_sample<256>(job.part, job.parts, job.n, job.sums, blockIdx.x - reduce_blocks, red);
        return;
    }
    long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    const long step = (long)reduce_blocks * blockDim.x;
    for (; i < total4; i += step) {
        const long at = 4 * i;
        float4 sum = *reinterpret_cast<const float4 *>(slabs + at);
        for (int q = 1; q < ncopies; ++q) {
            const float4 v = *reinterpret_cast<const float4 *>(slabs + q * stride + at);
            sum.x += v.x; sum.y += v.y; sum.z += v.z; sum.w += v.w;
        }
        int k = 0;
        long begin = 0;
        while (k + 1 < t.count && at >= t.end[k]) begin = t.end[k++];
        float4 *to = reinterpret_cast<float4 *>(t.dst[k] + (at - begin));
        if (accumulate) {
            const float4 old = *to;
            sum.x += old.x; sum.y += old.y; sum.z += old.z; sum.w += old.w;
        }
        *to = sum;
    }
}

// how many chunks the slabs region can take (0: none)
int plan_slab_capacity(const void *slabs, size_t slab_bytes, long slab_floats) {
    if (!slabs || slab_floats <= 0) return 0;
    const size_t n = slab_bytes / ((size_t)slab_floats * sizeof(float));
    return n > 65535 ? 65535 : (int)n;
}

// Splitting the batch of a block costs one more kernel and a pass over a copy of the gradient
// arrays per chunk.  Back to back on a stream the split is never slower (32^3 grid, 8^3 blocks,
// 4 inner iterations: 28.6 against 29.9 us at batch 2, 30.8 against 34.7 us at batch 3, 48 against
// 91 us at batch 16); a caller that waits for every call sees the extra launch instead, and at
// batch 2 -- the shape of the reference's own benchmark -- the unsplit call returns 9 % sooner.
// So the batch is split when that shortens the walk of a workgroup by two elements or more.
constexpr int kSplitMinSaved = 2;
int plan_split_room(int room, int B, int chunk_len) { return B - chunk_len < kSplitMinSaved ? 1 : room; }

int plan_reduce_slabs(const float *slabs, int ncopies, long stride, const SlabTargets &t, int accumulate,
                      hipStream_t st, const SumsJob &job = SumsJob{nullptr, 0, 0, 0, nullptr}) {
    const long total4 = t.end[t.count - 1] / 4;
    long blocks = (total4 + 255) / 256;
    if (blocks > 4096) blocks = 4096;
    hipLaunchKernelGGL(plan_reduce_slabs_f32, dim3((unsigned)(blocks + job.B)), dim3(256), 0, st, slabs, ncopies,
                       stride, t, total4, accumulate, (int)blocks, job);
    return check_launch("reduce_slabs");
}

}  // namespace
}  // namespace gridnet

#endif  // GRIDNET_PLAN_H
