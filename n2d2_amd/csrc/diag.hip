// Diagnostics of the library: the engine clock the chip holds while its int8 matrix cores are busy, which is what a
// fraction of the matrix-core peak has to be read against (the published peak assumes the maximum clock).
#include <vector>

#include "common.h"
#include "mfma_util.hpp"

namespace n2d2hip {

// Every wave runs `iters` rounds of four independent 32 x 32 x 32 int8 matrix instructions; lane 0 of each block
// records how many shader clocks (s_memtime) and how many ticks of the constant 100 MHz counter (s_memrealtime) that took.
__global__ __launch_bounds__(256) void clock_probe_kernel(int iters, long long* out, int* sink)
{
    v16i acc[4] = {};
    v4i a = {(int)threadIdx.x, 1, 2, 3}, b = {4, 5, (int)blockIdx.x, 7};
    const long long c0 = clock64(), w0 = wall_clock64();
    for (int i = 0; i < iters; ++i) {
#pragma unroll
        for (int k = 0; k < 4; ++k)
            acc[k] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, acc[k], 0, 0, 0);
    }
    int s = 0;
#pragma unroll
    for (int k = 0; k < 4; ++k) s += acc[k][0] + acc[k][15];
    const long long c1 = clock64(), w1 = wall_clock64();
    if (threadIdx.x == 0) {
        out[2 * blockIdx.x] = c1 - c0;
        out[2 * blockIdx.x + 1] = w1 - w0;
    }
    if (s == 0x7fffffff) *sink = s;      // keeps the arithmetic alive
}

} // namespace n2d2hip

#ifdef N2D2HIP_PROFILE
#include "n2d2hip_probe.h"

namespace n2d2hip {

// The probe buffer of the process: device memory the caller owns, checked on the host when it is handed over.
static long long* g_probe = nullptr;
static long long g_probe_records = 0, g_probe_used = 0;

long long* probe_take(unsigned blocks, long long* first)
{
    if (!g_probe || g_probe_used + (long long)blocks > g_probe_records)
        return nullptr;
    *first = g_probe_used;
    long long* at = g_probe + g_probe_used * N2D2HIP_PROBE_RECORD;
    g_probe_used += blocks;
    return at;
}

} // namespace n2d2hip
#endif

using namespace n2d2hip;

#ifdef N2D2HIP_PROFILE
extern "C" int n2d2hip_probe_begin(void* device_buffer, size_t bytes)
{
    N2D2HIP_REQUIRE(device_buffer != nullptr && bytes >= N2D2HIP_PROBE_RECORD * sizeof(long long) && (uintptr_t)device_buffer % 8 == 0,
                    N2D2HIP_ERR_INVALID, "probe_begin: an 8-byte aligned device buffer of at least one record");
    // The buffer must be device memory of the current device and the whole range must lie inside one allocation:
    // the kernels write through this pointer.
    hipPointerAttribute_t attr;
    N2D2HIP_HIP_CHECK(hipPointerGetAttributes(&attr, device_buffer));
    int dev = 0;
    N2D2HIP_HIP_CHECK(hipGetDevice(&dev));
    N2D2HIP_REQUIRE(attr.type == hipMemoryTypeDevice && attr.device == dev, N2D2HIP_ERR_INVALID,
                    "probe_begin: the buffer is not memory of the current device");
    hipDeviceptr_t base = nullptr;
    size_t size = 0;
    N2D2HIP_HIP_CHECK(hipMemGetAddressRange(&base, &size, (hipDeviceptr_t)device_buffer));
    N2D2HIP_REQUIRE((const char*)device_buffer + bytes <= (const char*)base + size, N2D2HIP_ERR_INVALID,
                    "probe_begin: %zu bytes reach past the end of the allocation", bytes);
    g_probe = (long long*)device_buffer;
    g_probe_records = (long long)(bytes / (N2D2HIP_PROBE_RECORD * sizeof(long long)));
    g_probe_used = 0;
    return N2D2HIP_OK;
}

extern "C" int n2d2hip_probe_end(long long* records_used)
{
    if (records_used) *records_used = g_probe_used;
    g_probe = nullptr;
    g_probe_records = g_probe_used = 0;
    return N2D2HIP_OK;
}
#endif

extern "C" int n2d2hip_measure_clock(double busy_microseconds, double* mhz, n2d2hip_stream_t stream_)
{
    N2D2HIP_REQUIRE(mhz != nullptr && busy_microseconds > 0 && busy_microseconds <= 1e5, N2D2HIP_ERR_INVALID,
                    "measure_clock: a duration between 0 and 100 ms and a result pointer");
    hipStream_t st = (hipStream_t)stream_;
    hipDeviceProp_t prop;
    int dev = 0;
    N2D2HIP_HIP_CHECK(hipGetDevice(&dev));
    N2D2HIP_HIP_CHECK(hipGetDeviceProperties(&prop, dev));
    const int blocks = 2 * std::max(1, prop.multiProcessorCount);
    // two waves per SIMD, 32 cycles per instruction and wave pair at full rate: about 256 cycles per round
    const int iters = std::max(1, (int)(busy_microseconds * 2000.0 / 256.0));
    long long* d_out = nullptr;
    int* d_sink = nullptr;
    N2D2HIP_HIP_CHECK(hipMalloc((void**)&d_out, (size_t)blocks * 2 * sizeof(long long) + sizeof(int)));
    d_sink = (int*)(d_out + (size_t)blocks * 2);
    hipLaunchKernelGGL(clock_probe_kernel, dim3(blocks), dim3(256), 0, st, iters, d_out, d_sink);
    std::vector<long long> h((size_t)blocks * 2);
    hipError_t e = hipGetLastError();
    if (e == hipSuccess) e = hipStreamSynchronize(st);
    if (e == hipSuccess) e = hipMemcpy(h.data(), d_out, h.size() * sizeof(long long), hipMemcpyDeviceToHost);
    (void)hipFree(d_out);
    if (e != hipSuccess)
        return fail(N2D2HIP_ERR_HIP, "measure_clock: %s", hipGetErrorString(e));
    double clocks = 0, ticks = 0;
    for (int i = 0; i < blocks; ++i) { clocks += (double)h[2 * i]; ticks += (double)h[2 * i + 1]; }
    N2D2HIP_REQUIRE(ticks > 0, N2D2HIP_ERR_HIP, "measure_clock: the constant-rate counter did not advance");
    *mhz = clocks / ticks * 100.0;
    return N2D2HIP_OK;
}
