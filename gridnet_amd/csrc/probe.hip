// Machine ceilings measured with the library's own compiler flags, for the benchmark to quote
// beside the vendor peaks: sustained unpacked fp32 FMA rate, LDS read rate, core clock under load
// and an HBM copy.  A library of its own (libgridnet_probe.so) that only bench.py and its test
// load: unlike libgridnet_hip.so it allocates, runs on the null stream and synchronises.
//   gridnet_probe(what, &result): 0 on success
//     0 FMA    sustained fp32 FMA rate without packed instructions, TFMA/s (x2 = TFLOP/s)
//     1 LDS    conflict-free 16-byte LDS reads over all CUs, GB/s
//     2 CLOCK  core clock while every CU runs the FMA loop, GHz
//     3 COPY   device-to-device copy of 1 GiB, 16 bytes per lane, four requests in flight per
//              lane, read + write GB/s
//     4..7     cycles of one CU's LDS pipe per wave-level read instruction: 32-, 64-, 128-bit,
//              and one two-address 64-bit read; lanes at consecutive addresses, 8 waves
//   gridnet_probe_last_error(): message of the last failure on the calling thread
#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdio>

namespace gridnet {
namespace {

enum { GRIDNET_PROBE_FMA = 0, GRIDNET_PROBE_LDS = 1, GRIDNET_PROBE_CLOCK = 2, GRIDNET_PROBE_COPY = 3,
       GRIDNET_PROBE_LDS_B32 = 4, GRIDNET_PROBE_LDS_B64 = 5, GRIDNET_PROBE_LDS_B128 = 6,
       GRIDNET_PROBE_LDS_2XB64 = 7, GRIDNET_PROBE_READ = 8 };
enum { GRIDNET_OK = 0, GRIDNET_ERR_ARGUMENT = 1, GRIDNET_ERR_LAUNCH = 5 };

char *probe_error() {
    static thread_local char buf[256] = {0};
    return buf;
}
int fail(int status, const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(probe_error(), 256, fmt, ap);
    va_end(ap);
    return status;
}

constexpr int kProbeThreads = 256;

// 16 independent FMA chains per lane, 128 FMAs per trip: enough to hide the ALU latency.
__global__ __launch_bounds__(kProbeThreads) void probe_fma(float *out, int trips, float a, float b) {
    float v[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) v[i] = threadIdx.x * 1e-3f + i;
    for (int t = 0; t < trips; ++t) {
#pragma unroll
        for (int r = 0; r < 8; ++r)
#pragma unroll
            for (int i = 0; i < 16; ++i) v[i] = fmaf(v[i], a, b);
    }
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < 16; ++i) s += v[i];
    out[(size_t)blockIdx.x * kProbeThreads + threadIdx.x] = s;
}

// Every lane reads 16 B from consecutive addresses (no bank conflicts), 8 reads per trip.
__global__ __launch_bounds__(kProbeThreads) void probe_lds(float *out, int trips) {
    __shared__ __attribute__((aligned(16))) float lds[8192];
    for (int i = threadIdx.x; i < 8192; i += kProbeThreads) lds[i] = i * 1e-4f;
    __syncthreads();
    const float4 *p = reinterpret_cast<const float4 *>(lds);
    float acc = 0.f;
    for (int t = 0; t < trips; ++t) {
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const float4 q = p[(threadIdx.x + 256 * ((u + t) & 7)) & 2047];
            acc += q.x + q.y + q.z + q.w;
        }
    }
    out[(size_t)blockIdx.x * kProbeThreads + threadIdx.x] = acc;
}

// Core clock against the fixed 100 MHz counter while every CU runs the FMA loop.
__global__ __launch_bounds__(kProbeThreads) void probe_clock(float *out, long long *ticks, int trips, float a, float b) {
    float v[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) v[i] = threadIdx.x * 1e-3f + i;
    const long long c0 = clock64(), w0 = wall_clock64();
    for (int t = 0; t < trips; ++t) {
#pragma unroll
        for (int r = 0; r < 8; ++r)
#pragma unroll
            for (int i = 0; i < 16; ++i) v[i] = fmaf(v[i], a, b);
    }
    const long long c1 = clock64(), w1 = wall_clock64();
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < 16; ++i) s += v[i];
    out[(size_t)blockIdx.x * kProbeThreads + threadIdx.x] = s;
    if (blockIdx.x == 0 && threadIdx.x == 0) {
        ticks[0] = c1 - c0;
        ticks[1] = w1 - w0;
    }
}

// One workgroup of 8 waves on one CU: cycles of the CU's LDS pipe per wave-level read instruction of
// a given width, lanes at consecutive addresses (no bank conflicts).  W: 1, 2, 4 = 32-, 64-, 128-bit
// reads; 22 = two 64-bit reads that the compiler fuses into one two-address instruction.
template <int W>
__global__ __launch_bounds__(512) void probe_lds_width(float *out, long long *ticks, int trips) {
    __shared__ __attribute__((aligned(16))) float lds[16384];
    for (int i = threadIdx.x; i < 16384; i += 512) lds[i] = i * 1e-4f;
    __syncthreads();
    const int lane = threadIdx.x & 63;
    // the pair of 64-bit reads as the backward kernels issue it: four floats from an 8-byte-aligned
    // address, neighbouring lanes two floats apart (their rows overlap)
    const int at = W == 22 ? lane * 2 : lane * W;
    float acc = 0.f;
    __syncthreads();
    const long long c0 = clock64();
    for (int t = 0; t < trips; ++t) {
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const float *p = lds + at + ((u + t) & 7) * 1024;
            if (W == 4) {
                const float4 q = *reinterpret_cast<const float4 *>(p);
                acc += q.x + q.y + q.z + q.w;
            } else if (W == 2) {
                const float2 q = *reinterpret_cast<const float2 *>(p);
                acc += q.x + q.y;
            } else if (W == 22) {
                const float2 q = *reinterpret_cast<const float2 *>(p);
                const float2 r = *reinterpret_cast<const float2 *>(p + 2);
                acc += q.x + q.y + r.x + r.y;
            } else {
                acc += p[0];
            }
        }
    }
    const long long c1 = clock64();
    out[threadIdx.x] = acc;
    if (lane == 0) ticks[threadIdx.x / 64] = c1 - c0;
}

// 16 bytes per lane and request, four requests in flight per lane before the first store (n is a
// multiple of 4 * the grid's threads)
__global__ __launch_bounds__(kProbeThreads) void probe_copy(const float4 *src, float4 *dst, size_t n) {
    const size_t stride = (size_t)gridDim.x * kProbeThreads;
    for (size_t i = (size_t)blockIdx.x * kProbeThreads + threadIdx.x; i + 3 * stride < n; i += 4 * stride) {
        const float4 a = src[i], b = src[i + stride], c = src[i + 2 * stride], d = src[i + 3 * stride];
        dst[i] = a;
        dst[i + stride] = b;
        dst[i + 2 * stride] = c;
        dst[i + 3 * stride] = d;
    }
}

// the same requests, nothing written but one value per thread: what reads alone get from HBM
// (a kernel that reads more than it writes sits between this figure and the copy's)
__global__ __launch_bounds__(kProbeThreads) void probe_read(const float4 *src, float *out, size_t n) {
    const size_t stride = (size_t)gridDim.x * kProbeThreads;
    float acc = 0.f;
    for (size_t i = (size_t)blockIdx.x * kProbeThreads + threadIdx.x; i + 3 * stride < n; i += 4 * stride) {
        const float4 a = src[i], b = src[i + stride], c = src[i + 2 * stride], d = src[i + 3 * stride];
        acc += (a.x + a.y + a.z + a.w) + (b.x + b.y + b.z + b.w) + (c.x + c.y + c.z + c.w) + (d.x + d.y + d.z + d.w);
    }
    out[(size_t)blockIdx.x * kProbeThreads + threadIdx.x] = acc;
}

struct Timer {
    hipEvent_t e0 = nullptr, e1 = nullptr;
    bool ok;
    Timer() { ok = hipEventCreate(&e0) == hipSuccess && hipEventCreate(&e1) == hipSuccess; }
    ~Timer() {
        if (e0) (void)hipEventDestroy(e0);
        if (e1) (void)hipEventDestroy(e1);
    }
    // best of `reps` launches, in seconds; negative on failure
    template <class F> double best(int reps, F launch) {
        double best_s = -1.0;
        for (int r = 0; ok && r < reps; ++r) {
            if (hipEventRecord(e0, 0) != hipSuccess) return -1.0;
            launch();
            if (hipEventRecord(e1, 0) != hipSuccess || hipEventSynchronize(e1) != hipSuccess) return -1.0;
            float ms = 0.f;
            if (hipEventElapsedTime(&ms, e0, e1) != hipSuccess) return -1.0;
            if (best_s < 0 || ms * 1e-3 < best_s) best_s = ms * 1e-3;
        }
        return hipGetLastError() == hipSuccess ? best_s : -1.0;
    }
};

}  // namespace
}  // namespace gridnet

using namespace gridnet;

extern "C" const char *gridnet_probe_last_error(void) { return probe_error(); }

extern "C" int gridnet_probe(int what, double *result) {
    if (!result) return fail(GRIDNET_ERR_ARGUMENT, "probe: result is null");
    int dev = 0, cus = 0;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
        return fail(GRIDNET_ERR_LAUNCH, "probe: no device");
    const int blocks = cus * 8;
    Timer timer;
    if (!timer.ok) return fail(GRIDNET_ERR_LAUNCH, "probe: hipEventCreate failed");
    float *out = nullptr;
    long long *ticks = nullptr;
    float4 *src = nullptr, *dst = nullptr;
    int rc = GRIDNET_OK;
    double s = -1.0;
    if (hipMalloc(&out, (size_t)blocks * kProbeThreads * sizeof(float)) != hipSuccess)
        return fail(GRIDNET_ERR_LAUNCH, "probe: hipMalloc failed");
    switch (what) {
    case GRIDNET_PROBE_FMA: {  // TFMA/s (one FMA = 2 flop)
        const int trips = 4000;
        s = timer.best(4, [&] { hipLaunchKernelGGL(probe_fma, dim3(blocks), dim3(kProbeThreads), 0, 0, out, trips, 0.999f, 0.001f); });
        if (s > 0) *result = (double)blocks * kProbeThreads * trips * 128.0 / s / 1e12;
        break;
    }
    case GRIDNET_PROBE_LDS: {  // GB/s over the whole chip
        const int trips = 4000;
        s = timer.best(4, [&] { hipLaunchKernelGGL(probe_lds, dim3(blocks), dim3(kProbeThreads), 0, 0, out, trips); });
        if (s > 0) *result = (double)blocks * kProbeThreads * trips * 8.0 * 16.0 / s / 1e9;
        break;
    }
    case GRIDNET_PROBE_CLOCK: {  // GHz
        if (hipMalloc(&ticks, 2 * sizeof(long long)) != hipSuccess) { rc = fail(GRIDNET_ERR_LAUNCH, "probe: hipMalloc failed"); break; }
        const int trips = 4000;
        s = timer.best(2, [&] { hipLaunchKernelGGL(probe_clock, dim3(blocks), dim3(kProbeThreads), 0, 0, out, ticks, trips, 0.999f, 0.001f); });
        long long h[2] = {0, 0};
        if (s > 0 && hipMemcpy(h, ticks, sizeof(h), hipMemcpyDeviceToHost) == hipSuccess && h[1] > 0)
            *result = (double)h[0] / (double)h[1] * 0.1;
        else
            s = -1.0;
        break;
    }
    case GRIDNET_PROBE_COPY: {  // GB/s, read + write
        const size_t n = (size_t)1 << 26;  // 1 GiB each way
        if (hipMalloc(&src, n * sizeof(float4)) != hipSuccess || hipMalloc(&dst, n * sizeof(float4)) != hipSuccess) {
            rc = fail(GRIDNET_ERR_LAUNCH, "probe: hipMalloc failed");
            break;
        }
        hipLaunchKernelGGL(probe_copy, dim3(cus * 32), dim3(kProbeThreads), 0, 0, dst, src, n);  // first touch
        s = timer.best(4, [&] { hipLaunchKernelGGL(probe_copy, dim3(cus * 32), dim3(kProbeThreads), 0, 0, src, dst, n); });
        if (s > 0) *result = 2.0 * (double)n * sizeof(float4) / s / 1e9;
        break;
    }
    case GRIDNET_PROBE_READ: {  // GB/s, reads only
        const size_t n = (size_t)1 << 26;  // 1 GiB
        if (hipMalloc(&src, n * sizeof(float4)) != hipSuccess ||
            hipMalloc(&dst, (size_t)cus * 32 * kProbeThreads * sizeof(float)) != hipSuccess) {
            rc = fail(GRIDNET_ERR_LAUNCH, "probe: hipMalloc failed");
            break;
        }
        if (hipMemset(src, 0, n * sizeof(float4)) != hipSuccess) { rc = fail(GRIDNET_ERR_LAUNCH, "probe: hipMemset failed"); break; }
        s = timer.best(4, [&] { hipLaunchKernelGGL(probe_read, dim3(cus * 32), dim3(kProbeThreads), 0, 0, src, (float *)dst, n); });
        if (s > 0) *result = (double)n * sizeof(float4) / s / 1e9;
        break;
    }
    case GRIDNET_PROBE_LDS_B32:
    case GRIDNET_PROBE_LDS_B64:
    case GRIDNET_PROBE_LDS_B128:
    case GRIDNET_PROBE_LDS_2XB64: {  // LDS-pipe cycles per wave-level read instruction
        if (hipMalloc(&ticks, 8 * sizeof(long long)) != hipSuccess) { rc = fail(GRIDNET_ERR_LAUNCH, "probe: hipMalloc failed"); break; }
        const int trips = 2000;
        double best = -1.0;
        for (int rep = 0; rep < 3; ++rep) {
            if (what == GRIDNET_PROBE_LDS_B32) hipLaunchKernelGGL(probe_lds_width<1>, dim3(1), dim3(512), 0, 0, out, ticks, trips);
            else if (what == GRIDNET_PROBE_LDS_B64) hipLaunchKernelGGL(probe_lds_width<2>, dim3(1), dim3(512), 0, 0, out, ticks, trips);
            else if (what == GRIDNET_PROBE_LDS_B128) hipLaunchKernelGGL(probe_lds_width<4>, dim3(1), dim3(512), 0, 0, out, ticks, trips);
            else hipLaunchKernelGGL(probe_lds_width<22>, dim3(1), dim3(512), 0, 0, out, ticks, trips);
            long long h[8] = {0};
            if (hipDeviceSynchronize() != hipSuccess ||
                hipMemcpy(h, ticks, sizeof(h), hipMemcpyDeviceToHost) != hipSuccess) { best = -1.0; break; }
            long long mx = 0;
            for (int w = 0; w < 8; ++w) mx = h[w] > mx ? h[w] : mx;
            const double per = (double)mx / (trips * 8.0 * 8.0);  // 8 reads per trip, 8 waves share the pipe
            if (best < 0 || per < best) best = per;
        }
        if (best > 0) { *result = best; s = 1.0; }
        break;
    }
    default:
        rc = fail(GRIDNET_ERR_ARGUMENT, "probe: unknown quantity");
    }
    (void)hipDeviceSynchronize();
    (void)hipFree(out);
    if (ticks) (void)hipFree(ticks);
    if (src) (void)hipFree(src);
    if (dst) (void)hipFree(dst);
    if (rc == GRIDNET_OK && s <= 0) rc = fail(GRIDNET_ERR_LAUNCH, "probe: launch or timing failed");
    return rc;
}
