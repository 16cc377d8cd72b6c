// SAT and LSQ fake-quantization kernels (float32), forward and backward.
// Element-wise work is one coalesced grid-stride pass; the global reductions
// (max |tanh w|, mean, variance, step-size / alpha gradients) are
// wavefront-reduced with cross-lane shuffles, block-reduced through LDS, and
// finished by a one-block kernel over at most PARTIALS block results, so the
// result does not depend on scheduling.  Sums are carried in double.
#include <algorithm>
#include <mutex>

#include "common.h"
#include "epilogue.hpp"

namespace n2d2hip {

constexpr int PARTIALS = 1024;   // max blocks of a reducing pass
constexpr int QBLOCK = 256;

__device__ __forceinline__ double wave_sum(double v)
{
#pragma unroll
    for (int off = 32; off > 0; off >>= 1)
        v += __shfl_xor(v, off, 64);
    return v;
}
__device__ __forceinline__ float wave_max(float v)
{
#pragma unroll
    for (int off = 32; off > 0; off >>= 1)
        v = fmaxf(v, __shfl_xor(v, off, 64));
    return v;
}
__device__ __forceinline__ double block_sum(double v)
{
    __shared__ double red[QBLOCK / 64];
    v = wave_sum(v);
    __syncthreads();
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
    __syncthreads();
    double t = 0.0;
#pragma unroll
    for (int i = 0; i < QBLOCK / 64; ++i) t += red[i];
    return t;
}
__device__ __forceinline__ float block_max(float v)
{
    __shared__ float redm[QBLOCK / 64];
    v = wave_max(v);
    __syncthreads();
    if ((threadIdx.x & 63) == 0) redm[threadIdx.x >> 6] = v;
    __syncthreads();
    float t = redm[0];
#pragma unroll
    for (int i = 1; i < QBLOCK / 64; ++i) t = fmaxf(t, redm[i]);
    return t;
}

// ------------------------------------------------------------ SAT weights

__global__ __launch_bounds__(QBLOCK) void sat_absmax_partial(const float* __restrict__ w, size_t n, float* __restrict__ partial)
{
    float m = 0.0f;
    for (size_t i = (size_t)blockIdx.x * QBLOCK + threadIdx.x; i < n; i += (size_t)gridDim.x * QBLOCK)
        m = fmaxf(m, fabsf(tanhf(w[i])));
    m = block_max(m);
    if (threadIdx.x == 0) partial[blockIdx.x] = m;
}
__global__ __launch_bounds__(QBLOCK) void sat_absmax_final(const float* __restrict__ partial, int count, float* __restrict__ stats)
{
    float m = 0.0f;
    for (int i = threadIdx.x; i < count; i += QBLOCK) m = fmaxf(m, partial[i]);
    m = block_max(m);
    if (threadIdx.x == 0) { stats[0] = m; stats[1] = 1.0f; }
}

// ref: src/Quantizer/QAT/Kernel/SATQuantizer_Frame_Kernels.cpp:66-238
__global__ __launch_bounds__(QBLOCK) void sat_weight_quantize(const float* __restrict__ w, float* __restrict__ wq, size_t n,
                                                              float range, int mode, const float* __restrict__ stats)
{
    const float tmax = stats[0];
    if (mode == N2D2HIP_SAT_SYMRANGE || mode == N2D2HIP_SAT_ASYMRANGE || mode == N2D2HIP_SAT_NONE_ASYM)
        range = floorf(range / 2.0f);
    const float inv_range = 1.0f / range;
    const float full_a = 1.0f + 0.9998f / range, full_b = 0.4999f / range;
    const float asym_a = 1.0f + 1.0f / (2.0f * range), asym_b = 1.0f / (2.0f * range);
    for (size_t i = (size_t)blockIdx.x * QBLOCK + threadIdx.x; i < n; i += (size_t)gridDim.x * QBLOCK) {
        const float t = tanhf(w[i]);
        float q;
        switch (mode) {
        case N2D2HIP_SAT_NONE:
            q = t / tmax;
            break;
        case N2D2HIP_SAT_DEFAULT:
            q = __fmul_rn(0.5f, __fadd_rn(t / tmax, 1.0f));
            q = __fmul_rn(inv_range, rintf(__fmul_rn(q, range)));
            q = __fsub_rn(__fmul_rn(q, 2.0f), 1.0f);
            break;
        case N2D2HIP_SAT_FULLRANGE:
            q = __fmul_rn(0.5f, __fadd_rn(t / tmax, 1.0f));
            q = __fsub_rn(__fmul_rn(full_a, q), full_b);
            q = __fmul_rn(inv_range, rintf(__fmul_rn(q, range)));
            q = __fsub_rn(__fmul_rn(q, 2.0f), 1.0f);
            break;
        case N2D2HIP_SAT_SYMRANGE:
            q = t / tmax;
            q = __fmul_rn(inv_range, rintf(__fmul_rn(q, range)));
            break;
        case N2D2HIP_SAT_ASYMRANGE:
            q = t / tmax;
            q = __fsub_rn(__fmul_rn(asym_a, q), asym_b);
            q = __fmul_rn(inv_range, rintf(__fmul_rn(q, range)));
            break;
        default:
            q = t / tmax;
            q = __fsub_rn(__fmul_rn(asym_a, q), asym_b);
            break;
        }
        wq[i] = q;
    }
}

// SAT scaling, ref: SATQuantizer_Frame_Kernels.cpp:244-262: mean, unbiased variance about that
// mean, scaling = sqrt(var * outputs_size).
__global__ __launch_bounds__(QBLOCK) void sum_partial(const float* __restrict__ x, size_t n, double* __restrict__ partial)
{
    double s = 0.0;
    for (size_t i = (size_t)blockIdx.x * QBLOCK + threadIdx.x; i < n; i += (size_t)gridDim.x * QBLOCK)
        s += (double)x[i];
    s = block_sum(s);
    if (threadIdx.x == 0) partial[blockIdx.x] = s;
}
__global__ __launch_bounds__(QBLOCK) void mean_final(const double* __restrict__ partial, int count, size_t n, float* __restrict__ mean)
{
    double s = 0.0;
    for (int i = threadIdx.x; i < count; i += QBLOCK) s += partial[i];
    s = block_sum(s);
    if (threadIdx.x == 0) mean[0] = (float)((float)s / (float)n);
}
__global__ __launch_bounds__(QBLOCK) void sqdev_partial(const float* __restrict__ x, size_t n, const float* __restrict__ mean,
                                                        double* __restrict__ partial)
{
    const float m = mean[0];
    double s = 0.0;
    for (size_t i = (size_t)blockIdx.x * QBLOCK + threadIdx.x; i < n; i += (size_t)gridDim.x * QBLOCK) {
        const float d = __fsub_rn(x[i], m);
        s += (double)__fmul_rn(d, d);
    }
    s = block_sum(s);
    if (threadIdx.x == 0) partial[blockIdx.x] = s;
}
__global__ __launch_bounds__(QBLOCK) void sat_scaling_final(const double* __restrict__ partial, int count, size_t n, unsigned factor,
                                                            float* __restrict__ stats)
{
    double s = 0.0;
    for (int i = threadIdx.x; i < count; i += QBLOCK) s += partial[i];
    s = block_sum(s);
    if (threadIdx.x == 0) {
        const float var = (float)s / ((float)n - 1.0f);
        stats[1] = sqrtf(var * (float)factor);
    }
}
__global__ __launch_bounds__(QBLOCK) void divide_by_stat(float* __restrict__ x, size_t n, const float* __restrict__ stat)
{
    const float s = stat[0];
    for (size_t i = (size_t)blockIdx.x * QBLOCK + threadIdx.x; i < n; i += (size_t)gridDim.x * QBLOCK)
        x[i] = x[i] / s;
}

// ref: SATQuantizer_Frame_Kernels.cpp:349-404
__global__ __launch_bounds__(QBLOCK) void sat_weight_backward_kernel(const float* __restrict__ dq, const float* __restrict__ w,
                                                                     float* __restrict__ dw, size_t n, float mode_factor, int use_mode_factor,
                                                                     int apply_scaling, const float* __restrict__ stats)
{
    const float factor = apply_scaling ? __fmul_rn(stats[0], stats[1]) : stats[0];
    const float inv_factor = 1.0f / factor;
    for (size_t i = (size_t)blockIdx.x * QBLOCK + threadIdx.x; i < n; i += (size_t)gridDim.x * QBLOCK) {
        const float inv_cosh = 1.0f / coshf(w[i]);
        float grad = __fmul_rn(__fmul_rn(inv_cosh, inv_cosh), inv_factor);
        if (use_mode_factor)
            grad = __fmul_rn(grad, mode_factor);
        dw[i] = __fmul_rn(dq[i], grad);
    }
}

// -------------------------------------------------------- SAT activations

// ref: SATQuantizer_Frame_Kernels.cpp:268-322 (std::round: half away from zero)
__global__ __launch_bounds__(QBLOCK) void sat_act_forward_kernel(float* __restrict__ x, float* __restrict__ fp, size_t n, float range,
                                                                 const float* __restrict__ alpha)
{
    const float a = fabsf(alpha[0]);
    for (size_t i = (size_t)blockIdx.x * QBLOCK + threadIdx.x; i < n; i += (size_t)gridDim.x * QBLOCK) {
        const float v = x[i];
        if (fp) fp[i] = v;
        const float xc = (v < 0.0f) ? 0.0f : (v < a) ? v : a;
        float q = xc / a;
        q = round_half_away(__fmul_rn(range, q)) / range;
        x[i] = __fmul_rn(q, a);
    }
}

// ref: SATQuantizer_Frame_Kernels.cpp:410-448; the alpha-gradient terms are summed instead of stored
__global__ __launch_bounds__(QBLOCK) void sat_act_backward_kernel(const float* dy, const float* __restrict__ fp,
                                                                  float* dx, size_t n, float range,
                                                                  const float* __restrict__ alpha, double* __restrict__ partial)
{
    const float a = fabsf(alpha[0]);
    double s = 0.0;
    for (size_t i = (size_t)blockIdx.x * QBLOCK + threadIdx.x; i < n; i += (size_t)gridDim.x * QBLOCK) {
        const float x = fp[i];
        const float g = dy[i];
        const float xc = (x < 0.0f) ? 0.0f : (x < a) ? x : a;
        const float q = xc / a;
        const float qd = round_half_away(__fmul_rn(range, q)) / range;
        const float dqa = (x >= a) ? 1.0f : __fsub_rn(qd, q);
        s += (double)__fmul_rn(dqa, g);
        const float dact = (x <= 0.0f) ? 0.0f : (x > a) ? 0.0f : 1.0f;
        dx[i] = __fmul_rn(dact, g);
    }
    s = block_sum(s);
    if (threadIdx.x == 0) partial[blockIdx.x] = s;
}
// result[0] = (sum + beta * result[0]) * scale
__global__ __launch_bounds__(QBLOCK) void accumulate_final(const double* __restrict__ partial, int count, float beta, float scale,
                                                           float* __restrict__ result)
{
    double s = 0.0;
    for (int i = threadIdx.x; i < count; i += QBLOCK) s += partial[i];
    s = block_sum(s);
    if (threadIdx.x == 0) {
        float acc = (float)s;
        if (beta != 0.0f)
            acc = __fadd_rn(acc, __fmul_rn(beta, result[0]));
        result[0] = __fmul_rn(acc, scale);
    }
}

// -------------------------------------------------------------------- LSQ

// ref: LSQQuantizerCell_Frame.cpp:194-208, LSQQuantizerActivation_Frame.cpp:131-141
__global__ __launch_bounds__(QBLOCK) void lsq_forward_kernel(const float* __restrict__ x, float* __restrict__ xq, size_t n,
                                                             const float* __restrict__ step, int lo, int hi)
{
    const float s = step[0];
    const float lob = __fmul_rn((float)lo, s), hib = __fmul_rn((float)hi, s);
    for (size_t i = (size_t)blockIdx.x * QBLOCK + threadIdx.x; i < n; i += (size_t)gridDim.x * QBLOCK) {
        const float q = x[i] / s;
        xq[i] = (q <= (float)lo) ? lob : (q >= (float)hi) ? hib : __fmul_rn(round_half_away(q), s);
    }
}
// ref: LSQQuantizerCell_Frame.cpp:234-303, LSQQuantizerActivation_Frame.cpp:193-262
__global__ __launch_bounds__(QBLOCK) void lsq_backward_kernel(const float* dq, const float* __restrict__ fp,
                                                              float* dfp, size_t n, const float* __restrict__ step,
                                                              int lo, int hi, double* __restrict__ partial)
{
    const float s = step[0];
    double acc = 0.0;
    for (size_t i = (size_t)blockIdx.x * QBLOCK + threadIdx.x; i < n; i += (size_t)gridDim.x * QBLOCK) {
        const float q = fp[i] / s;
        const float g = dq[i];
        const bool below = q <= (float)lo, above = q >= (float)hi;
        dfp[i] = __fmul_rn(g, (below || above) ? 0.0f : 1.0f);
        const float term = below ? (float)lo : above ? (float)hi : __fsub_rn(round_half_away(q), q);
        acc += (double)__fmul_rn(term, g);
    }
    acc = block_sum(acc);
    if (threadIdx.x == 0) partial[blockIdx.x] = acc;
}

} // namespace n2d2hip

using namespace n2d2hip;

namespace {
int blocks_for(size_t n)
{
    size_t b = (n + QBLOCK - 1) / QBLOCK;
    return (int)std::max<size_t>(1, std::min<size_t>(b, PARTIALS));
}
unsigned ew_grid(size_t n)
{
    size_t b = (n + QBLOCK - 1) / QBLOCK;
    return (unsigned)std::max<size_t>(1, std::min<size_t>(b, 256 * 32));
}
} // namespace

// Scratch of the entry point that allocates nothing: the block partials and the mean of the SAT weight quantizer's
// reductions.  Every GPU the library runs on holds its own copy of this array until the process ends.  In host code the
// array's name is only a handle for hipGetSymbolAddress, never a device address.
constexpr size_t STATIC_SCRATCH_BYTES = (size_t)PARTIALS * sizeof(double) + 256;
static __device__ __align__(256) unsigned char scratch[STATIC_SCRATCH_BYTES];

namespace {
constexpr int MAX_DEVICES = 64;
std::mutex scratch_mutex;
void* scratch_ptr[MAX_DEVICES] = {};     // device address of `scratch` on each device, looked up once per device

// Device address of the current device's copy of `scratch`; no allocation.
int static_scratch(void** ptr)
{
    int dev = 0;
    N2D2HIP_HIP_CHECK(hipGetDevice(&dev));
    N2D2HIP_REQUIRE(dev >= 0 && dev < MAX_DEVICES, N2D2HIP_ERR_UNSUPPORTED, "static scratch: device ordinal %d (at most %d devices)", dev, MAX_DEVICES);
    std::lock_guard<std::mutex> lock(scratch_mutex);
    if (!scratch_ptr[dev]) {
        void* p = nullptr;
        N2D2HIP_HIP_CHECK(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
        N2D2HIP_REQUIRE(p != nullptr, N2D2HIP_ERR_HIP, "static scratch: hipGetSymbolAddress returned a null address");
        scratch_ptr[dev] = p;
    }
    *ptr = scratch_ptr[dev];
    return N2D2HIP_OK;
}
} // namespace

extern "C" {

size_t n2d2hip_quantizer_workspace_bytes(size_t) { return (size_t)PARTIALS * sizeof(double) + 256; }

// The kernel sequence of the SAT weight quantizer over a workspace of n2d2hip_quantizer_workspace_bytes() bytes.
static int sat_weight_forward_impl(const char* who, const float* w, float* wq, size_t n, float range, int mode, int apply_scaling,
                                   unsigned outputs_size, float* stats, void* workspace, hipStream_t st)
{
    N2D2HIP_REQUIRE(n > 0, N2D2HIP_ERR_INVALID, "%s: empty tensor", who);
    N2D2HIP_REQUIRE(mode >= N2D2HIP_SAT_NONE && mode <= N2D2HIP_SAT_NONE_ASYM, N2D2HIP_ERR_INVALID, "%s: bad mode %d", who, mode);
    N2D2HIP_REQUIRE(range >= 1.0f, N2D2HIP_ERR_INVALID, "%s: range %g", who, (double)range);
    N2D2HIP_REQUIRE(!apply_scaling || n > 1, N2D2HIP_ERR_INVALID, "%s: SAT scaling needs more than one weight", who);
    const int nb = blocks_for(n);
    double* partial = (double*)workspace;
    float* mean = (float*)((char*)workspace + (size_t)PARTIALS * sizeof(double));
    hipLaunchKernelGGL(sat_absmax_partial, dim3(nb), dim3(QBLOCK), 0, st, w, n, (float*)partial);
    hipLaunchKernelGGL(sat_absmax_final, dim3(1), dim3(QBLOCK), 0, st, (const float*)partial, nb, stats);
    hipLaunchKernelGGL(sat_weight_quantize, dim3(ew_grid(n)), dim3(QBLOCK), 0, st, w, wq, n, range, mode, (const float*)stats);
    if (apply_scaling) {
        hipLaunchKernelGGL(sum_partial, dim3(nb), dim3(QBLOCK), 0, st, (const float*)wq, n, partial);
        hipLaunchKernelGGL(mean_final, dim3(1), dim3(QBLOCK), 0, st, (const double*)partial, nb, n, mean);
        hipLaunchKernelGGL(sqdev_partial, dim3(nb), dim3(QBLOCK), 0, st, (const float*)wq, n, (const float*)mean, partial);
        hipLaunchKernelGGL(sat_scaling_final, dim3(1), dim3(QBLOCK), 0, st, (const double*)partial, nb, n, outputs_size, stats);
        hipLaunchKernelGGL(divide_by_stat, dim3(ew_grid(n)), dim3(QBLOCK), 0, st, wq, n, (const float*)(stats + 1));
    }
    N2D2HIP_HIP_CHECK(hipGetLastError());
    return N2D2HIP_OK;
}

int n2d2hip_sat_weight_forward(const float* w, float* wq, size_t n, float range, int mode, int apply_scaling,
                               unsigned outputs_size, float* stats, void* workspace, size_t workspace_bytes, n2d2hip_stream_t stream_)
{
    N2D2HIP_REQUIRE(w && wq && stats && workspace, N2D2HIP_ERR_INVALID, "sat_weight_forward: null argument");
    N2D2HIP_REQUIRE(workspace_bytes >= n2d2hip_quantizer_workspace_bytes(n), N2D2HIP_ERR_WORKSPACE, "sat_weight_forward: workspace of %zu bytes needed",
                    n2d2hip_quantizer_workspace_bytes(n));
    return sat_weight_forward_impl("sat_weight_forward", w, wq, n, range, mode, apply_scaling, outputs_size, stats, workspace, (hipStream_t)stream_);
}

int n2d2hip_sat_weight_forward_static(const float* w, float* wq, size_t n, float range, int mode, int apply_scaling,
                                      unsigned outputs_size, float* stats, n2d2hip_stream_t stream_)
{
    N2D2HIP_REQUIRE(w && wq && stats, N2D2HIP_ERR_INVALID, "sat_weight_forward_static: null argument");
    N2D2HIP_REQUIRE(n <= (size_t)N2D2HIP_SAT_STATIC_MAX_WEIGHTS, N2D2HIP_ERR_UNSUPPORTED,
                    "sat_weight_forward_static: %zu weights, at most %zu are served from the static scratch; use n2d2hip_sat_weight_forward",
                    n, (size_t)N2D2HIP_SAT_STATIC_MAX_WEIGHTS);
    static_assert(STATIC_SCRATCH_BYTES >= (size_t)PARTIALS * sizeof(double) + sizeof(float), "scratch holds the partials and the mean");
    void* ws = nullptr;
    int rc = static_scratch(&ws);
    if (rc != N2D2HIP_OK)
        return rc;
    // Nothing in the scratch has to start from zero: every pass writes the partials it then reads (the same block count
    // both times), and the mean is written before it is read.
    return sat_weight_forward_impl("sat_weight_forward_static", w, wq, n, range, mode, apply_scaling, outputs_size, stats, ws, (hipStream_t)stream_);
}

int n2d2hip_sat_weight_backward(const float* diff_wq, const float* w, float* diff_w, size_t n, float range, int mode,
                                int apply_scaling, const float* stats, n2d2hip_stream_t stream_)
{
    N2D2HIP_REQUIRE(diff_wq && w && diff_w && stats, N2D2HIP_ERR_INVALID, "sat_weight_backward: null argument");
    N2D2HIP_REQUIRE(n > 0, N2D2HIP_ERR_INVALID, "sat_weight_backward: empty tensor");
    N2D2HIP_REQUIRE(mode >= N2D2HIP_SAT_NONE && mode <= N2D2HIP_SAT_NONE_ASYM, N2D2HIP_ERR_INVALID, "sat_weight_backward: bad mode %d", mode);
    // ref: SATQuantizerCell_Frame.cpp:249-283: Asymmetric and FullRange have their own slope factor
    float mf = 1.0f;
    int use = 0;
    if (mode == N2D2HIP_SAT_FULLRANGE) { mf = 1.0f + 0.9998f / range; use = 1; }
    else if (mode == N2D2HIP_SAT_ASYMRANGE || mode == N2D2HIP_SAT_NONE_ASYM) { const float r2 = floorf(range / 2.0f); mf = 1.0f + 1.0f / (2.0f * r2); use = 1; }
    hipLaunchKernelGGL(sat_weight_backward_kernel, dim3(ew_grid(n)), dim3(QBLOCK), 0, (hipStream_t)stream_, diff_wq, w, diff_w, n, mf, use,
                       apply_scaling, stats);
    N2D2HIP_HIP_CHECK(hipGetLastError());
    return N2D2HIP_OK;
}

int n2d2hip_sat_act_forward(float* x, float* fp_copy, size_t n, float range, const float* alpha, n2d2hip_stream_t stream_)
{
    N2D2HIP_REQUIRE(x && alpha, N2D2HIP_ERR_INVALID, "sat_act_forward: null argument");
    N2D2HIP_REQUIRE(n > 0, N2D2HIP_ERR_INVALID, "sat_act_forward: empty tensor");
    hipLaunchKernelGGL(sat_act_forward_kernel, dim3(ew_grid(n)), dim3(QBLOCK), 0, (hipStream_t)stream_, x, fp_copy, n, range, alpha);
    N2D2HIP_HIP_CHECK(hipGetLastError());
    return N2D2HIP_OK;
}

int n2d2hip_sat_act_backward(const float* diff_in, const float* fp_x, float* diff_out, size_t n, float range, const float* alpha,
                             float beta, float* diff_alpha, void* workspace, size_t workspace_bytes, n2d2hip_stream_t stream_)
{
    hipStream_t st = (hipStream_t)stream_;
    N2D2HIP_REQUIRE(diff_in && fp_x && diff_out && alpha && diff_alpha && workspace, N2D2HIP_ERR_INVALID, "sat_act_backward: null argument");
    N2D2HIP_REQUIRE(n > 0, N2D2HIP_ERR_INVALID, "sat_act_backward: empty tensor");
    N2D2HIP_REQUIRE(workspace_bytes >= n2d2hip_quantizer_workspace_bytes(n), N2D2HIP_ERR_WORKSPACE, "sat_act_backward: workspace of %zu bytes needed",
                    n2d2hip_quantizer_workspace_bytes(n));
    const int nb = blocks_for(n);
    double* partial = (double*)workspace;
    hipLaunchKernelGGL(sat_act_backward_kernel, dim3(nb), dim3(QBLOCK), 0, st, diff_in, fp_x, diff_out, n, range, alpha, partial);
    hipLaunchKernelGGL(accumulate_final, dim3(1), dim3(QBLOCK), 0, st, (const double*)partial, nb, beta, 1.0f, diff_alpha);
    N2D2HIP_HIP_CHECK(hipGetLastError());
    return N2D2HIP_OK;
}

int n2d2hip_lsq_forward(const float* x, float* xq, size_t n, const float* step, int lo, int hi, n2d2hip_stream_t stream_)
{
    N2D2HIP_REQUIRE(x && xq && step, N2D2HIP_ERR_INVALID, "lsq_forward: null argument");
    N2D2HIP_REQUIRE(n > 0 && lo < hi, N2D2HIP_ERR_INVALID, "lsq_forward: empty tensor or empty range [%d,%d]", lo, hi);
    hipLaunchKernelGGL(lsq_forward_kernel, dim3(ew_grid(n)), dim3(QBLOCK), 0, (hipStream_t)stream_, x, xq, n, step, lo, hi);
    N2D2HIP_HIP_CHECK(hipGetLastError());
    return N2D2HIP_OK;
}

int n2d2hip_lsq_backward(const float* diff_q, const float* fp_x, float* diff_fp, size_t n, const float* step, int lo, int hi,
                         float grad_scale, float beta, float* diff_step, void* workspace, size_t workspace_bytes, n2d2hip_stream_t stream_)
{
    hipStream_t st = (hipStream_t)stream_;
    N2D2HIP_REQUIRE(diff_q && fp_x && diff_fp && step && diff_step && workspace, N2D2HIP_ERR_INVALID, "lsq_backward: null argument");
    N2D2HIP_REQUIRE(n > 0 && lo < hi, N2D2HIP_ERR_INVALID, "lsq_backward: empty tensor or empty range [%d,%d]", lo, hi);
    N2D2HIP_REQUIRE(workspace_bytes >= n2d2hip_quantizer_workspace_bytes(n), N2D2HIP_ERR_WORKSPACE, "lsq_backward: workspace of %zu bytes needed",
                    n2d2hip_quantizer_workspace_bytes(n));
    const int nb = blocks_for(n);
    double* partial = (double*)workspace;
    hipLaunchKernelGGL(lsq_backward_kernel, dim3(nb), dim3(QBLOCK), 0, st, diff_q, fp_x, diff_fp, n, step, lo, hi, partial);
    hipLaunchKernelGGL(accumulate_final, dim3(1), dim3(QBLOCK), 0, st, (const double*)partial, nb, beta, grad_scale, diff_step);
    N2D2HIP_HIP_CHECK(hipGetLastError());
    return N2D2HIP_OK;
}

} // extern "C"
