// Float32 cells of a quantization-aware training step: convolution forward, its three backward kernels, softmax,
// the loss at the output and the SGD update.  Tensors are N2D2's own NCHW / OCHW float tensors (X fastest), so a
// training graph exchanges them without conversion.
//
// These are direct kernels: one thread per produced element, walking channels and taps in the reference's order
// (so forward and backward-data give the reference's float sums term for term), and one block per weight for
// backward-filter, whose long sum over batch and pixels is wavefront-reduced in double.
#include <cstdlib>

#include "common.h"
#include "conv_f32_gemm.hpp"

namespace n2d2hip {

constexpr int TBLOCK = 256;

struct ConvF32 {
    int B, C, H, W, O, oH, oW, kW, kH, Cw;      // Cw = C / groups
    int sx, sy, pl, pt, pr, pb, dx, dy;
    int depthwise;                                // groups == C == O
    int choice;                                   // the descriptor's kernel_choice bits
};

__device__ __forceinline__ double wave_sum_d(double v)
{
#pragma unroll
    for (int off = 32; off > 0; off >>= 1)
        v += __shfl_xor(v, off, 64);
    return v;
}
__device__ __forceinline__ double block_sum_d(double v)
{
    __shared__ double red[TBLOCK / 64];
    v = wave_sum_d(v);
    __syncthreads();
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
    __syncthreads();
    double t = 0.0;
#pragma unroll
    for (int i = 0; i < TBLOCK / 64; ++i) t += red[i];
    return t;
}

// out[b,o,oy,ox] = alpha-less weighted sum (+ bias) + beta * out.  The window is clipped at the borders (no padded
// zeros are read); a full 3x3 window is summed row by row, then the rows, as the reference's unrolled branch does.
__global__ __launch_bounds__(TBLOCK) void conv_f32_forward_kernel(ConvF32 q, const float* __restrict__ x, const float* __restrict__ w,
                                                                  const float* __restrict__ bias, float beta, float* __restrict__ y)
{
    const size_t total = (size_t)q.B * q.O * q.oH * q.oW;
    for (size_t idx = (size_t)blockIdx.x * TBLOCK + threadIdx.x; idx < total; idx += (size_t)gridDim.x * TBLOCK) {
        const int ox = idx % q.oW, oy = (idx / q.oW) % q.oH;
        const int o = (idx / ((size_t)q.oW * q.oH)) % q.O, b = idx / ((size_t)q.oW * q.oH * q.O);
        const int dilKx = q.kW + (q.dx - 1) * (q.kW - 1), dilKy = q.kH + (q.dy - 1) * (q.kH - 1);
        const int sxMin = max(q.pl - ox * q.sx, 0), syMin = max(q.pt - oy * q.sy, 0);
        const int sxMax = min(max(q.W + q.pl - ox * q.sx, 0), dilKx), syMax = min(max(q.H + q.pt - oy * q.sy, 0), dilKy);
        const int ix = ox * q.sx - q.pl, iy = oy * q.sy - q.pt;
        const int c0 = q.depthwise ? o : 0, c1 = q.depthwise ? o + 1 : q.C;
        const bool full3 = sxMin == 0 && syMin == 0 && sxMax == 3 && syMax == 3 && q.kW == 3 && q.kH == 3;
        float sum = 0.0f;
        for (int c = c0; c < c1; ++c) {
            const float* xc = x + ((size_t)b * q.C + c) * q.H * q.W;
            const float* wc = w + ((size_t)o * q.Cw + (q.depthwise ? 0 : c)) * q.kH * q.kW;
            if (full3) {
                const float* r0 = xc + (size_t)iy * q.W + ix;
                const float* r1 = r0 + q.W;
                const float* r2 = r1 + q.W;
                sum = sum + (wc[0] * r0[0] + wc[1] * r0[1] + wc[2] * r0[2])
                          + (wc[3] * r1[0] + wc[4] * r1[1] + wc[5] * r1[2])
                          + (wc[6] * r2[0] + wc[7] * r2[1] + wc[8] * r2[2]);
            } else {
                for (int ty = syMin; ty * q.dy < syMax; ++ty)
                    for (int tx = sxMin; tx * q.dx < sxMax; ++tx)
                        sum += wc[ty * q.kW + tx] * xc[(size_t)(iy + ty * q.dy) * q.W + ix + tx * q.dx];
            }
        }
        float r = sum + (beta != 0.0f ? beta * y[idx] : 0.0f);
        if (bias) r = bias[o] + r;
        y[idx] = r;
    }
}

// dx[b,c,iy,ix] = sum over connected outputs (ascending) and over the taps reaching this element + beta * dx.
__global__ __launch_bounds__(TBLOCK) void conv_f32_backward_data_kernel(ConvF32 q, const float* __restrict__ w, const float* __restrict__ dy,
                                                                        float beta, float* __restrict__ dx)
{
    const size_t total = (size_t)q.B * q.C * q.H * q.W;
    const int oxStride = q.sx * q.oW, oyStride = q.sy * q.oH;
    for (size_t idx = (size_t)blockIdx.x * TBLOCK + threadIdx.x; idx < total; idx += (size_t)gridDim.x * TBLOCK) {
        const int ix = idx % q.W, iy = (idx / q.W) % q.H;
        const int c = (idx / ((size_t)q.W * q.H)) % q.C, b = idx / ((size_t)q.W * q.H * q.C);
        const int ixPad = ix + q.pl, iyPad = iy + q.pt;
        const int sxMin = ixPad % q.sx + max(ixPad - ixPad % q.sx - oxStride + q.sx, 0);
        const int syMin = iyPad % q.sy + max(iyPad - iyPad % q.sy - oyStride + q.sy, 0);
        const int sxMax = min(q.kW, ixPad + 1), syMax = min(q.kH, iyPad + 1);
        const bool full3 = syMax - syMin == 3 && q.sy == 1 && sxMax - sxMin == 3 && q.sx == 1;
        const int o0 = q.depthwise ? c : 0, o1 = q.depthwise ? c + 1 : q.O;
        float g = 0.0f;
        for (int o = o0; o < o1; ++o) {
            const float* wo = w + ((size_t)o * q.Cw + (q.depthwise ? 0 : c)) * q.kH * q.kW;
            const float* dyo = dy + ((size_t)b * q.O + o) * q.oH * q.oW;
            if (full3) {
                const int ox = ixPad - sxMin, oy = iyPad - syMin;
#pragma unroll
                for (int t = 0; t < 9; ++t)
                    g = g + wo[(syMin + t / 3) * q.kW + sxMin + t % 3] * dyo[(size_t)(oy - t / 3) * q.oW + ox - t % 3];
            } else {
                for (int ty = syMin; ty < syMax; ty += q.sy)
                    for (int tx = sxMin; tx < sxMax; tx += q.sx)
                        g += wo[ty * q.kW + tx] * dyo[(size_t)((iyPad - ty) / q.sy) * q.oW + (ixPad - tx) / q.sx];
            }
        }
        dx[idx] = g + (beta != 0.0f ? beta * dx[idx] : 0.0f);
    }
}

// dw[o,c',ty,tx] = sum over batch and the output pixels whose tap (ty,tx) falls inside the input + beta * dw.
// One block per weight.
__global__ __launch_bounds__(TBLOCK) void conv_f32_backward_filter_kernel(ConvF32 q, const float* __restrict__ x, const float* __restrict__ dy,
                                                                          float beta, float* __restrict__ dw)
{
    const int widx = blockIdx.x;
    const int tx = widx % q.kW, ty = (widx / q.kW) % q.kH;
    const int cw = (widx / (q.kW * q.kH)) % q.Cw, o = widx / (q.kW * q.kH * q.Cw);
    const int c = q.depthwise ? o : cw;
    // ox range with 0 <= ox*sx + tx - pl < W
    const int oxMin = max((q.pl - tx + q.sx - 1) / q.sx, 0), oyMin = max((q.pt - ty + q.sy - 1) / q.sy, 0);
    const int oxMax = min((q.W + q.pl - tx + q.sx - 1) / q.sx, q.oW), oyMax = min((q.H + q.pt - ty + q.sy - 1) / q.sy, q.oH);
    const int nx = max(oxMax - oxMin, 0), ny = max(oyMax - oyMin, 0);
    const size_t total = (size_t)q.B * ny * nx;
    double acc = 0.0;
    for (size_t i = threadIdx.x; i < total; i += TBLOCK) {
        const int ox = oxMin + i % nx, oy = oyMin + (i / nx) % ny, b = i / ((size_t)nx * ny);
        const float xv = x[(((size_t)b * q.C + c) * q.H + (oy * q.sy + ty - q.pt)) * q.W + ox * q.sx + tx - q.pl];
        const float dv = dy[(((size_t)b * q.O + o) * q.oH + oy) * q.oW + ox];
        acc += (double)(xv * dv);
    }
    acc = block_sum_d(acc);
    if (threadIdx.x == 0)
        dw[widx] = (float)acc + (beta != 0.0f ? beta * dw[widx] : 0.0f);
}

// db[o] = sum over batch and pixels + beta * db.  One block per output channel.
__global__ __launch_bounds__(TBLOCK) void conv_f32_backward_bias_kernel(int B, int O, int plane, const float* __restrict__ dy, float beta,
                                                                        float* __restrict__ db)
{
    const int o = blockIdx.x;
    double acc = 0.0;
    for (size_t i = threadIdx.x; i < (size_t)B * plane; i += TBLOCK)
        acc += (double)dy[((size_t)(i / plane) * O + o) * plane + i % plane];
    acc = block_sum_d(acc);
    if (threadIdx.x == 0)
        db[o] = (float)acc + (beta != 0.0f ? beta * db[o] : 0.0f);
}

// Softmax over the channels of each pixel: exp(x - max) / sum, zeros if the sum is not positive.
__global__ __launch_bounds__(TBLOCK) void softmax_f32_kernel(const float* __restrict__ x, float* __restrict__ y, int B, int C, int plane)
{
    const size_t total = (size_t)B * plane;
    for (size_t idx = (size_t)blockIdx.x * TBLOCK + threadIdx.x; idx < total; idx += (size_t)gridDim.x * TBLOCK) {
        const size_t base = (idx / plane) * (size_t)C * plane + idx % plane;
        float m = x[base];
        for (int c = 1; c < C; ++c) m = fmaxf(m, x[base + (size_t)c * plane]);
        float s = 0.0f;
        for (int c = 0; c < C; ++c) s += expf(x[base + (size_t)c * plane] - m);
        for (int c = 0; c < C; ++c) y[base + (size_t)c * plane] = s > 0.0f ? expf(x[base + (size_t)c * plane] - m) / s : 0.0f;
    }
}

// diff = target - output, formed in double; partial[block] = sum of squares (double).
__global__ __launch_bounds__(TBLOCK) void loss_f32_kernel(const float* target, const float* __restrict__ out, float* diff,
                                                          size_t n, double* __restrict__ partial)
{
    double acc = 0.0;
    for (size_t i = (size_t)blockIdx.x * TBLOCK + threadIdx.x; i < n; i += (size_t)gridDim.x * TBLOCK) {
        const double e = (double)target[i] - (double)out[i];
        diff[i] = (float)e;
        acc += e * e;
    }
    acc = block_sum_d(acc);
    if (threadIdx.x == 0) partial[blockIdx.x] = acc;
}
__global__ __launch_bounds__(TBLOCK) void loss_finish_kernel(const double* __restrict__ partial, int nb, double inv_batch, double* __restrict__ loss)
{
    double acc = 0.0;
    for (int i = threadIdx.x; i < nb; i += TBLOCK) acc += partial[i];
    acc = block_sum_d(acc);
    if (threadIdx.x == 0) loss[0] = acc * inv_batch;
}

// SGDSolver_Frame::update for one tensor.
__global__ __launch_bounds__(TBLOCK) void sgd_f32_kernel(float* __restrict__ data, const float* __restrict__ diff, size_t n, float rate_diff,
                                                         float momentum, float decay_rate, float* __restrict__ mom, float lo, float hi, int clamp)
{
    for (size_t i = (size_t)blockIdx.x * TBLOCK + threadIdx.x; i < n; i += (size_t)gridDim.x * TBLOCK) {
        float v;
        if (mom) {
            float m = mom[i] * momentum;
            m += rate_diff * diff[i];
            if (decay_rate != 0.0f) m += -decay_rate * data[i];
            mom[i] = m;
            v = data[i] + m;
        } else {
            v = data[i] + rate_diff * diff[i];
        }
        data[i] = clamp ? fminf(fmaxf(v, lo), hi) : v;
    }
}

// Rectifier on a float tensor, in place: x > 0 ? min(x, clipping) : leak * x (clipping == 0: none).
__global__ __launch_bounds__(TBLOCK) void rectifier_f32_forward_kernel(float* __restrict__ x, size_t n, float leak, float clipping)
{
    for (size_t i = (size_t)blockIdx.x * TBLOCK + threadIdx.x; i < n; i += (size_t)gridDim.x * TBLOCK) {
        const float v = x[i];
        x[i] = v > 0.0f ? (clipping > 0.0f ? fminf(v, clipping) : v) : leak * v;
    }
}
// diff_out = diff_in * (out == clipping ? 0 : out > 0 ? 1 : leak); `out` is what the cell holds after its activation.
__global__ __launch_bounds__(TBLOCK) void rectifier_f32_backward_kernel(const float* __restrict__ out, const float* diff_in,
                                                                        float* diff_out, size_t n, float leak, float clipping)
{
    for (size_t i = (size_t)blockIdx.x * TBLOCK + threadIdx.x; i < n; i += (size_t)gridDim.x * TBLOCK) {
        const float o = out[i];
        const float f = (clipping > 0.0f && o == clipping) ? 0.0f : (o > 0.0f ? 1.0f : leak);
        diff_out[i] = diff_in[i] * f;
    }
}

// Batch statistics of one channel per block: mean, then the mean of the squared deviations (two passes, as the
// reference), and the running statistics' step towards them (the variance with the factor size / (size - 1)).
__global__ __launch_bounds__(TBLOCK) void batchnorm_f32_stats_kernel(int B, int C, int plane, const float* __restrict__ x, float* __restrict__ mean,
                                                                     float* __restrict__ variance, float* __restrict__ saved_mean,
                                                                     float* __restrict__ saved_variance, double momentum)
{
    const int c = blockIdx.x;
    const size_t n = (size_t)B * plane;
    double acc = 0.0;
    for (size_t i = threadIdx.x; i < n; i += TBLOCK)
        acc += (double)x[((size_t)(i / plane) * C + c) * plane + i % plane];
    const float m = (float)(block_sum_d(acc) / (double)n);
    acc = 0.0;
    for (size_t i = threadIdx.x; i < n; i += TBLOCK) {
        const float zeroed = x[((size_t)(i / plane) * C + c) * plane + i % plane] - m;
        acc += (double)(zeroed * zeroed);
    }
    const float v = (float)(block_sum_d(acc) / (double)n);
    if (threadIdx.x == 0) {
        saved_mean[c] = m;
        saved_variance[c] = v;
        const float unbiased = v * ((float)n / ((float)n - 1.0f));
        mean[c] = (float)((double)m * momentum + (double)mean[c] * (1.0 - momentum));
        variance[c] = (float)((double)unbiased * momentum + (double)variance[c] * (1.0 - momentum));
    }
}

// y = scale * (x - mean) / sqrt(variance + epsilon) + bias.  eps_in_float: the inference branch of the reference adds
// the epsilon in float and takes a float square root; the learning branch adds the double and rounds the root.
__global__ __launch_bounds__(TBLOCK) void batchnorm_f32_apply_kernel(int planes, int C, int plane, const float* __restrict__ x,
                                                                     const float* __restrict__ scale, const float* __restrict__ bias,
                                                                     const float* __restrict__ mean, const float* __restrict__ variance, double epsilon,
                                                                     int eps_in_float, int vec, float* __restrict__ y)
{
    // blockIdx.y walks the (batch, channel) planes, so that the channel's constants are worked out once per plane;
    // planes whose size is a multiple of 4 move 16 bytes per lane
    for (int bc = blockIdx.y; bc < planes; bc += gridDim.y) {
        const int c = bc % C;
        const float var = eps_in_float ? sqrtf(variance[c] + (float)epsilon) : (float)sqrt((double)variance[c] + epsilon);
        const float m = mean[c], g = scale[c], b = bias[c];
        const float* xp = x + (size_t)bc * plane;
        float* yp = y + (size_t)bc * plane;
        if (vec) {
            for (int i = blockIdx.x * TBLOCK + threadIdx.x; i < plane / 4; i += gridDim.x * TBLOCK) {
                const float4 v = ((const float4*)xp)[i];
                float4 o;
                o.x = g * ((v.x - m) / var) + b;
                o.y = g * ((v.y - m) / var) + b;
                o.z = g * ((v.z - m) / var) + b;
                o.w = g * ((v.w - m) / var) + b;
                ((float4*)yp)[i] = o;
            }
        } else {
            for (int i = blockIdx.x * TBLOCK + threadIdx.x; i < plane; i += gridDim.x * TBLOCK)
                yp[i] = g * ((xp[i] - m) / var) + b;
        }
    }
}

// The same for small planes: one lane per value, the channel found by division.
__global__ __launch_bounds__(TBLOCK) void batchnorm_f32_apply_flat_kernel(size_t total, int C, int plane, const float* __restrict__ x,
                                                                     const float* __restrict__ scale, const float* __restrict__ bias,
                                                                     const float* __restrict__ mean, const float* __restrict__ variance, double epsilon,
                                                                     int eps_in_float, float* __restrict__ y)
{
    for (size_t i = (size_t)blockIdx.x * TBLOCK + threadIdx.x; i < total; i += (size_t)gridDim.x * TBLOCK) {
        const int c = (int)((i / plane) % C);
        const float var = eps_in_float ? sqrtf(variance[c] + (float)epsilon) : (float)sqrt((double)variance[c] + epsilon);
        const float normalized = (x[i] - mean[c]) / var;
        y[i] = scale[c] * normalized + bias[c];
    }
}

// The five sums of BatchNormCell_Frame<T>::backPropagate over one channel, and what follows from them.
__global__ __launch_bounds__(TBLOCK) void batchnorm_f32_backward_sums_kernel(int B, int C, int plane, const float* __restrict__ x,
                                                                             const float* __restrict__ scale, const float* __restrict__ saved_mean,
                                                                             const float* __restrict__ saved_variance, double epsilon,
                                                                             const float* __restrict__ dy, float beta_scale, float* __restrict__ diff_scale,
                                                                             float beta_bias, float* __restrict__ diff_bias,
                                                                             float* __restrict__ diff_saved_mean, float* __restrict__ diff_saved_variance)
{
    const int c = blockIdx.x;
    const size_t n = (size_t)B * plane;
    const float m = saved_mean[c], g = scale[c];
    const float var = (float)sqrt((double)saved_variance[c] + epsilon);
    double s_scale = 0.0, s_bias = 0.0, s_mean1 = 0.0, s_mean2 = 0.0, s_var = 0.0;
    for (size_t i = threadIdx.x; i < n; i += TBLOCK) {
        const size_t idx = ((size_t)(i / plane) * C + c) * plane + i % plane;
        const float centred = x[idx] - m;
        const float normalized = centred / var;
        const float d = dy[idx];
        const float diff_normalized = d * g;
        s_scale += (double)(d * normalized);
        s_bias += (double)d;
        s_mean1 += (double)diff_normalized;
        s_mean2 += (double)(float)(-2.0 * (double)centred);
        s_var += (double)(diff_normalized * centred);
    }
    const float sum_scale = (float)block_sum_d(s_scale);
    const float sum_bias = (float)block_sum_d(s_bias);
    const float sum_mean1 = (float)block_sum_d(s_mean1);
    const float sum_mean2 = (float)block_sum_d(s_mean2);
    const float sum_var = (float)block_sum_d(s_var);
    if (threadIdx.x == 0) {
        const float dv = (float)((double)sum_var * (-1.0 / 2.0) * pow((double)saved_variance[c] + epsilon, -3.0 / 2.0));
        diff_saved_variance[c] = dv;
        diff_saved_mean[c] = (float)((double)sum_mean1 * (-1.0 / (double)var) + (double)(dv * sum_mean2 / (float)n));
        diff_scale[c] = sum_scale + (beta_scale != 0.0f ? beta_scale * diff_scale[c] : 0.0f);
        diff_bias[c] = sum_bias + (beta_bias != 0.0f ? beta_bias * diff_bias[c] : 0.0f);
    }
}

// dx = dy * scale / sigma + dVar * 2 (x - mean) / size + dMean / size, plane by plane as the apply kernel
__device__ __forceinline__ float bn_dx(float x, float d, float g, float var, float m, double dv2, double size, double dmean_over_size)
{
    const float diff_normalized = d * g;
    return (float)((double)(diff_normalized / var) + dv2 * (double)(x - m) / size + dmean_over_size);
}
__global__ __launch_bounds__(TBLOCK) void batchnorm_f32_backward_data_kernel(int planes, int C, int plane, float size, const float* __restrict__ x,
                                                                            const float* __restrict__ scale, const float* __restrict__ saved_mean,
                                                                            const float* __restrict__ saved_variance, double epsilon, const float* dy,
                                                                            const float* __restrict__ diff_saved_mean,
                                                                            const float* __restrict__ diff_saved_variance, int vec, float* dx)
{
    for (int bc = blockIdx.y; bc < planes; bc += gridDim.y) {
        const int c = bc % C;
        const float var = (float)sqrt((double)saved_variance[c] + epsilon);
        const float m = saved_mean[c], g = scale[c];
        const double dv2 = (double)diff_saved_variance[c] * 2.0, sz = (double)size, dm = (double)(diff_saved_mean[c] / size);
        const float* xp = x + (size_t)bc * plane;
        const float* dp = dy + (size_t)bc * plane;
        float* op = dx + (size_t)bc * plane;
        if (vec) {
            for (int i = blockIdx.x * TBLOCK + threadIdx.x; i < plane / 4; i += gridDim.x * TBLOCK) {
                const float4 v = ((const float4*)xp)[i];
                const float4 d = ((const float4*)dp)[i];
                float4 o;
                o.x = bn_dx(v.x, d.x, g, var, m, dv2, sz, dm);
                o.y = bn_dx(v.y, d.y, g, var, m, dv2, sz, dm);
                o.z = bn_dx(v.z, d.z, g, var, m, dv2, sz, dm);
                o.w = bn_dx(v.w, d.w, g, var, m, dv2, sz, dm);
                ((float4*)op)[i] = o;
            }
        } else {
            for (int i = blockIdx.x * TBLOCK + threadIdx.x; i < plane; i += gridDim.x * TBLOCK)
                op[i] = bn_dx(xp[i], dp[i], g, var, m, dv2, sz, dm);
        }
    }
}

// The same for small planes: one lane per value.
__global__ __launch_bounds__(TBLOCK) void batchnorm_f32_backward_data_flat_kernel(size_t total, int C, int plane, float size, const float* __restrict__ x,
                                                                            const float* __restrict__ scale, const float* __restrict__ saved_mean,
                                                                            const float* __restrict__ saved_variance, double epsilon, const float* dy,
                                                                            const float* __restrict__ diff_saved_mean,
                                                                            const float* __restrict__ diff_saved_variance, float* dx)
{
    for (size_t i = (size_t)blockIdx.x * TBLOCK + threadIdx.x; i < total; i += (size_t)gridDim.x * TBLOCK) {
        const int c = (int)((i / plane) % C);
        const float var = (float)sqrt((double)saved_variance[c] + epsilon);
        const float diff_normalized = dy[i] * scale[c];
        const double gradient = (double)(diff_normalized / var) + (double)diff_saved_variance[c] * 2.0 * (double)(x[i] - saved_mean[c]) / (double)size
                                + (double)(diff_saved_mean[c] / size);
        dx[i] = (float)gradient;
    }
}

// The same sums spread over `splits` blocks per channel (blockIdx.y), each adding its slice in double into a partial of
// its own; the partials are then added in slice order, so the result does not depend on timing.
__device__ __forceinline__ void bn_slice(size_t n, int splits, size_t* begin, size_t* end)
{
    const size_t chunk = (n + splits - 1) / splits;
    *begin = (size_t)blockIdx.y * chunk;
    *end = *begin + chunk < n ? *begin + chunk : n;
}
__device__ __forceinline__ double bn_total(const double* partial, int splits, int stride)
{
    double t = 0.0;
    for (int s = 0; s < splits; ++s)
        t += partial[(size_t)s * stride];
    return t;
}

__global__ __launch_bounds__(TBLOCK) void batchnorm_f32_sum_partial_kernel(int B, int C, int plane, int splits, const float* __restrict__ x,
                                                                           double* __restrict__ ws)
{
    const int c = blockIdx.x;
    size_t i0, i1;
    bn_slice((size_t)B * plane, splits, &i0, &i1);
    double acc = 0.0;
    for (size_t i = i0 + threadIdx.x; i < i1; i += TBLOCK)
        acc += (double)x[((size_t)(i / plane) * C + c) * plane + i % plane];
    acc = block_sum_d(acc);
    if (threadIdx.x == 0)
        ws[(size_t)c * splits + blockIdx.y] = acc;
}

__global__ __launch_bounds__(TBLOCK) void batchnorm_f32_sq_partial_kernel(int B, int C, int plane, int splits, const float* __restrict__ x,
                                                                          const double* __restrict__ ws_sum, double* __restrict__ ws_sq)
{
    const int c = blockIdx.x;
    const size_t n = (size_t)B * plane;
    const float m = (float)(bn_total(ws_sum + (size_t)c * splits, splits, 1) / (double)n);
    size_t i0, i1;
    bn_slice(n, splits, &i0, &i1);
    double acc = 0.0;
    for (size_t i = i0 + threadIdx.x; i < i1; i += TBLOCK) {
        const float zeroed = x[((size_t)(i / plane) * C + c) * plane + i % plane] - m;
        acc += (double)(zeroed * zeroed);
    }
    acc = block_sum_d(acc);
    if (threadIdx.x == 0)
        ws_sq[(size_t)c * splits + blockIdx.y] = acc;
}

__global__ __launch_bounds__(TBLOCK) void batchnorm_f32_stats_finish_kernel(int C, size_t n, int splits, const double* __restrict__ ws_sum,
                                                                            const double* __restrict__ ws_sq, float* __restrict__ mean,
                                                                            float* __restrict__ variance, float* __restrict__ saved_mean,
                                                                            float* __restrict__ saved_variance, double momentum)
{
    const int c = blockIdx.x * TBLOCK + threadIdx.x;
    if (c >= C)
        return;
    const float m = (float)(bn_total(ws_sum + (size_t)c * splits, splits, 1) / (double)n);
    const float v = (float)(bn_total(ws_sq + (size_t)c * splits, splits, 1) / (double)n);
    saved_mean[c] = m;
    saved_variance[c] = v;
    const float unbiased = v * ((float)n / ((float)n - 1.0f));
    mean[c] = (float)((double)m * momentum + (double)mean[c] * (1.0 - momentum));
    variance[c] = (float)((double)unbiased * momentum + (double)variance[c] * (1.0 - momentum));
}

__global__ __launch_bounds__(TBLOCK) void batchnorm_f32_backward_partial_kernel(int B, int C, int plane, int splits, const float* __restrict__ x,
                                                                                const float* __restrict__ scale, const float* __restrict__ saved_mean,
                                                                                const float* __restrict__ saved_variance, double epsilon,
                                                                                const float* __restrict__ dy, double* __restrict__ ws)
{
    const int c = blockIdx.x;
    const float m = saved_mean[c], g = scale[c];
    const float var = (float)sqrt((double)saved_variance[c] + epsilon);
    size_t i0, i1;
    bn_slice((size_t)B * plane, splits, &i0, &i1);
    double s_scale = 0.0, s_bias = 0.0, s_mean1 = 0.0, s_mean2 = 0.0, s_var = 0.0;
    for (size_t i = i0 + threadIdx.x; i < i1; i += TBLOCK) {
        const size_t idx = ((size_t)(i / plane) * C + c) * plane + i % plane;
        const float centred = x[idx] - m;
        const float normalized = centred / var;
        const float d = dy[idx];
        const float diff_normalized = d * g;
        s_scale += (double)(d * normalized);
        s_bias += (double)d;
        s_mean1 += (double)diff_normalized;
        s_mean2 += (double)(float)(-2.0 * (double)centred);
        s_var += (double)(diff_normalized * centred);
    }
    s_scale = block_sum_d(s_scale);
    s_bias = block_sum_d(s_bias);
    s_mean1 = block_sum_d(s_mean1);
    s_mean2 = block_sum_d(s_mean2);
    s_var = block_sum_d(s_var);
    if (threadIdx.x == 0) {
        double* o = ws + ((size_t)c * splits + blockIdx.y) * 5;
        o[0] = s_scale; o[1] = s_bias; o[2] = s_mean1; o[3] = s_mean2; o[4] = s_var;
    }
}

__global__ __launch_bounds__(TBLOCK) void batchnorm_f32_backward_finish_kernel(int C, size_t n, int splits, const double* __restrict__ ws,
                                                                               const float* __restrict__ saved_variance, double epsilon,
                                                                               float beta_scale, float* __restrict__ diff_scale, float beta_bias,
                                                                               float* __restrict__ diff_bias, float* __restrict__ diff_saved_mean,
                                                                               float* __restrict__ diff_saved_variance)
{
    const int c = blockIdx.x * TBLOCK + threadIdx.x;
    if (c >= C)
        return;
    const double* p = ws + (size_t)c * splits * 5;
    const float sum_scale = (float)bn_total(p + 0, splits, 5), sum_bias = (float)bn_total(p + 1, splits, 5);
    const float sum_mean1 = (float)bn_total(p + 2, splits, 5), sum_mean2 = (float)bn_total(p + 3, splits, 5);
    const float sum_var = (float)bn_total(p + 4, splits, 5);
    const float var = (float)sqrt((double)saved_variance[c] + epsilon);
    const float dv = (float)((double)sum_var * (-1.0 / 2.0) * pow((double)saved_variance[c] + epsilon, -3.0 / 2.0));
    diff_saved_variance[c] = dv;
    diff_saved_mean[c] = (float)((double)sum_mean1 * (-1.0 / (double)var) + (double)(dv * sum_mean2 / (float)n));
    diff_scale[c] = sum_scale + (beta_scale != 0.0f ? beta_scale * diff_scale[c] : 0.0f);
    diff_bias[c] = sum_bias + (beta_bias != 0.0f ? beta_bias * diff_bias[c] : 0.0f);
}

struct PoolF32 {
    int B, C, H, W, oH, oW, pw, ph, sx, sy, px, py;
};

// Max pooling of float NCHW with the unit mapping; argmax keeps iy * W + ix of the first largest element of the
// window in row-major order (-1: empty window, output 0).
__global__ __launch_bounds__(TBLOCK) void pool_max_f32_forward_kernel(PoolF32 q, const float* __restrict__ x, float* __restrict__ y, int* __restrict__ argmax)
{
    const size_t total = (size_t)q.B * q.C * q.oH * q.oW;
    for (size_t i = (size_t)blockIdx.x * TBLOCK + threadIdx.x; i < total; i += (size_t)gridDim.x * TBLOCK) {
        const int ox = (int)(i % q.oW), oy = (int)((i / q.oW) % q.oH);
        const size_t bc = i / ((size_t)q.oW * q.oH);
        const float* in = x + bc * (size_t)q.H * q.W;
        const int x0 = ox * q.sx - q.px, y0 = oy * q.sy - q.py;
        const int sx_min = max(-x0, 0), sy_min = max(-y0, 0);
        const int sx_max = min(max(q.W - x0, 0), q.pw), sy_max = min(max(q.H - y0, 0), q.ph);
        float best = 0.0f;
        int where = -1;
        for (int sy = sy_min; sy < sy_max; ++sy)
            for (int sx = sx_min; sx < sx_max; ++sx) {
                const float v = in[(size_t)(y0 + sy) * q.W + x0 + sx];
                if (where < 0 || v > best) {
                    best = v;
                    where = (y0 + sy) * q.W + x0 + sx;
                }
            }
        y[i] = best;
        argmax[i] = where;
    }
}

// Every input collects the gradients of the outputs that chose it, in the reference's order (window rows, then columns,
// from the input's own residue modulo the stride upwards).
__global__ __launch_bounds__(TBLOCK) void pool_max_f32_backward_kernel(PoolF32 q, const float* __restrict__ dy, const int* __restrict__ argmax, float beta,
                                                                       float* __restrict__ dx)
{
    const size_t total = (size_t)q.B * q.C * q.H * q.W;
    for (size_t i = (size_t)blockIdx.x * TBLOCK + threadIdx.x; i < total; i += (size_t)gridDim.x * TBLOCK) {
        const int ix = (int)(i % q.W), iy = (int)((i / q.W) % q.H);
        const size_t bc = i / ((size_t)q.W * q.H);
        const int ix_pad = ix + q.px, iy_pad = iy + q.py;
        const int sx_max = min(q.pw, ix_pad + 1), sy_max = min(q.ph, iy_pad + 1);
        float acc = 0.0f;
        for (int sy = iy_pad % q.sy; sy < sy_max; sy += q.sy) {
            if (iy_pad >= q.sy * q.oH + sy)
                continue;
            const int oy = (iy_pad - sy) / q.sy;
            for (int sx = ix_pad % q.sx; sx < sx_max; sx += q.sx) {
                if (ix_pad >= q.sx * q.oW + sx)
                    continue;
                const int ox = (ix_pad - sx) / q.sx;
                const size_t o = (bc * q.oH + oy) * q.oW + ox;
                if (argmax[o] == iy * q.W + ix)
                    acc += dy[o];
            }
        }
        dx[i] = acc + (beta != 0.0f ? beta * dx[i] : 0.0f);
    }
}

static int grid_for(size_t total)
{
    const size_t blocks = (total + TBLOCK - 1) / TBLOCK;
    return (int)std::min<size_t>(std::max<size_t>(blocks, 1), 256 * 32);
}

static int make_conv(const n2d2hip_conv_desc* d, int B, int H, int W, bool backward, ConvF32* q, const char* who)
{
    N2D2HIP_REQUIRE(d != nullptr, N2D2HIP_ERR_INVALID, "%s: null descriptor", who);
    N2D2HIP_REQUIRE(B > 0 && H > 0 && W > 0 && d->C > 0 && d->O > 0 && d->kW > 0 && d->kH > 0 && d->strideX > 0 && d->strideY > 0
                        && d->dilX > 0 && d->dilY > 0 && d->padL >= 0 && d->padT >= 0 && d->padR >= 0 && d->padB >= 0,
                    N2D2HIP_ERR_INVALID, "%s: bad shape", who);
    N2D2HIP_REQUIRE(d->groups == 1 || (d->groups == d->C && d->C == d->O), N2D2HIP_ERR_UNSUPPORTED,
                    "%s: groups=%d (C=%d, O=%d): only ungrouped and depthwise convolutions", who, d->groups, d->C, d->O);
    N2D2HIP_REQUIRE(!backward || (d->dilX == 1 && d->dilY == 1), N2D2HIP_ERR_UNSUPPORTED,
                    "%s: the reference's backward kernels do not read the dilation", who);
    int oH = 0, oW = 0;
    const int st = n2d2hip_conv_out_dims(d, H, W, &oH, &oW);
    if (st != N2D2HIP_OK) return st;
    N2D2HIP_REQUIRE(oH > 0 && oW > 0, N2D2HIP_ERR_INVALID, "%s: empty output", who);
    N2D2HIP_REQUIRE((size_t)B * std::max(d->C, d->O) * std::max((size_t)H * W, (size_t)oH * oW) < ((size_t)1 << 40), N2D2HIP_ERR_INVALID,
                    "%s: tensor too large", who);
    *q = ConvF32{B, d->C, H, W, d->O, oH, oW, d->kW, d->kH, d->C / d->groups, d->strideX, d->strideY,
                 d->padL, d->padT, d->padR, d->padB, d->dilX, d->dilY, d->groups > 1 ? 1 : 0, d->kernel_choice};
    return N2D2HIP_OK;
}

// The matrix-core kernel serves ungrouped convolutions without dilation that are worth a 128 x 128 tile; the direct
// kernels keep the rest (depthwise, dilated, tiny).  The descriptor's kernel_choice (N2D2HIP_KERNEL_F32_DIRECT / _GEMM) overrides the size rule.
static bool use_gemm(const ConvF32& q)
{
    if (q.depthwise || q.dx != 1 || q.dy != 1)
        return false;
    if (q.choice & N2D2HIP_KERNEL_F32_DIRECT) return false;
    if (q.choice & N2D2HIP_KERNEL_F32_GEMM) return true;
    return 2.0 * q.B * q.O * q.oH * q.oW * q.C * q.kH * q.kW >= 2.0e7;
}

static GemmF32 make_gemm(const ConvF32& q, int mode)
{
    GemmF32 g = {q.B, q.C, q.H, q.W, q.O, q.oH, q.oW, q.kW, q.kH, q.sx, q.sy, q.pl, q.pt, 0, 0, 0, 0, 0, 0};
    const unsigned xb = (unsigned)((size_t)q.B * q.C * q.H * q.W * 4), yb = (unsigned)((size_t)q.B * q.O * q.oH * q.oW * 4);
    const unsigned wb = (unsigned)((size_t)q.O * q.C * q.kH * q.kW * 4);
    if (mode == GEMM_FWD) { g.P = q.B * q.oH * q.oW; g.Q = q.O; g.K = q.C * q.kH * q.kW; g.bytesP = xb; g.bytesQ = wb; }
    else if (mode == GEMM_BWD_DATA) { g.P = q.B * q.H * q.W; g.Q = q.C; g.K = q.O * q.kH * q.kW; g.bytesP = yb; g.bytesQ = wb; }
    else { g.P = q.C * q.kH * q.kW; g.Q = q.O; g.K = q.B * q.oH * q.oW; g.bytesP = xb; g.bytesQ = yb; }
    g.kchunk = round_up(g.K, GK);
    return g;
}

// K ranges of backward-filter: enough blocks to fill the chip, each range at least 32 steps long
static int filter_splits(GemmF32* g)
{
    const long tiles = (long)((g->P + GT - 1) / GT) * (g->Q <= 64 ? 1 : (g->Q + GT - 1) / GT);
    long splits = std::max(1L, 1024 / tiles);
    splits = std::min<long>(splits, std::max(1, g->K / (32 * GK)));
    g->kchunk = round_up((int)((g->K + splits - 1) / splits), GK);
    return (g->K + g->kchunk - 1) / g->kchunk;
}

// K ranges of forward / backward-data when the tiles alone leave most of the chip idle (three blocks fit a CU): each
// range at least 16 steps long
static int pass_splits(GemmF32* g)
{
    const long tiles = (long)((g->P + GT - 1) / GT) * (g->Q <= 64 ? 1 : (g->Q + GT - 1) / GT);
    long splits = tiles >= 384 ? 1 : std::max(1L, 768 / tiles);
    splits = std::min<long>(splits, std::max(1, g->K / (16 * GK)));
    g->kchunk = round_up((int)((g->K + splits - 1) / splits), GK);
    return (g->K + g->kchunk - 1) / g->kchunk;
}

static bool fits_int(const ConvF32& q)
{
    // the GEMM kernel reads tensors of at most 2 GiB through buffer descriptors and keeps one validity bit per tap
    const size_t lim = (size_t)1 << 29;
    return (size_t)q.B * q.C * q.H * q.W < lim && (size_t)q.B * q.O * q.oH * q.oW < lim && (size_t)q.O * q.C * q.kH * q.kW < lim
           && q.kH * q.kW <= 64;
}

} // namespace n2d2hip

using namespace n2d2hip;

extern "C" {

int n2d2hip_conv2d_f32_forward(const n2d2hip_conv_desc* desc, int B, int H, int W, const float* x, const float* w, const float* bias,
                               float beta, float* y, void* workspace, size_t workspace_bytes, n2d2hip_stream_t stream)
{
    ConvF32 q;
    const int st = make_conv(desc, B, H, W, false, &q, "n2d2hip_conv2d_f32_forward");
    if (st != N2D2HIP_OK) return st;
    N2D2HIP_REQUIRE(x && w && y, N2D2HIP_ERR_INVALID, "n2d2hip_conv2d_f32_forward: null pointer");
    if (use_gemm(q) && fits_int(q)) {
        GemmF32 g = make_gemm(q, GEMM_FWD);
        const size_t n = (size_t)g.P * g.Q;
        int splits = pass_splits(&g);
        if (splits > 1 && (!workspace || workspace_bytes < (size_t)splits * n * sizeof(float))) {
            splits = 1;                                     // no room for partial results: one range
            g.kchunk = round_up(g.K, GK);
        }
        float* dst = splits > 1 ? (float*)workspace : y;
        if (g.Q <= 64)
            hipLaunchKernelGGL((conv_f32_gemm_kernel<GEMM_FWD, 64>), dim3((g.P + GT - 1) / GT, 1, splits), dim3(256), 0, (hipStream_t)stream,
                               g, x, w, bias, beta, dst);
        else
            hipLaunchKernelGGL((conv_f32_gemm_kernel<GEMM_FWD, 128>), dim3((g.P + GT - 1) / GT, (g.Q + GT - 1) / GT, splits), dim3(256), 0,
                               (hipStream_t)stream, g, x, w, bias, beta, dst);
        if (splits > 1)
            hipLaunchKernelGGL(conv_f32_reduce_partials_kernel, dim3(grid_for(n)), dim3(256), 0, (hipStream_t)stream, (const float*)workspace, splits, n,
                               beta, y, bias, q.oH * q.oW, q.O);
        N2D2HIP_HIP_CHECK(hipGetLastError());
        return N2D2HIP_OK;
    }
    hipLaunchKernelGGL(conv_f32_forward_kernel, dim3(grid_for((size_t)q.B * q.O * q.oH * q.oW)), dim3(TBLOCK), 0, (hipStream_t)stream,
                       q, x, w, bias, beta, y);
    N2D2HIP_HIP_CHECK(hipGetLastError());
    return N2D2HIP_OK;
}

int n2d2hip_conv2d_f32_backward_data(const n2d2hip_conv_desc* desc, int B, int H, int W, const float* w, const float* diff_y, float beta,
                                     float* diff_x, void* workspace, size_t workspace_bytes, n2d2hip_stream_t stream)
{
    ConvF32 q;
    const int st = make_conv(desc, B, H, W, true, &q, "n2d2hip_conv2d_f32_backward_data");
    if (st != N2D2HIP_OK) return st;
    N2D2HIP_REQUIRE(w && diff_y && diff_x, N2D2HIP_ERR_INVALID, "n2d2hip_conv2d_f32_backward_data: null pointer");
    if (use_gemm(q) && fits_int(q)) {
        GemmF32 g = make_gemm(q, GEMM_BWD_DATA);
        const size_t n = (size_t)g.P * g.Q;
        int splits = pass_splits(&g);
        if (splits > 1 && (!workspace || workspace_bytes < (size_t)splits * n * sizeof(float))) {
            splits = 1;
            g.kchunk = round_up(g.K, GK);
        }
        float* dst = splits > 1 ? (float*)workspace : diff_x;
        if (g.Q <= 64)
            hipLaunchKernelGGL((conv_f32_gemm_kernel<GEMM_BWD_DATA, 64>), dim3((g.P + GT - 1) / GT, 1, splits), dim3(256), 0, (hipStream_t)stream,
                               g, diff_y, w, (const float*)nullptr, beta, dst);
        else
            hipLaunchKernelGGL((conv_f32_gemm_kernel<GEMM_BWD_DATA, 128>), dim3((g.P + GT - 1) / GT, (g.Q + GT - 1) / GT, splits), dim3(256), 0,
                               (hipStream_t)stream, g, diff_y, w, (const float*)nullptr, beta, dst);
        if (splits > 1)
            hipLaunchKernelGGL(conv_f32_reduce_partials_kernel, dim3(grid_for(n)), dim3(256), 0, (hipStream_t)stream, (const float*)workspace, splits, n,
                               beta, diff_x, (const float*)nullptr, 1, 1);
        N2D2HIP_HIP_CHECK(hipGetLastError());
        return N2D2HIP_OK;
    }
    hipLaunchKernelGGL(conv_f32_backward_data_kernel, dim3(grid_for((size_t)q.B * q.C * q.H * q.W)), dim3(TBLOCK), 0, (hipStream_t)stream,
                       q, w, diff_y, beta, diff_x);
    N2D2HIP_HIP_CHECK(hipGetLastError());
    return N2D2HIP_OK;
}

size_t n2d2hip_conv2d_f32_workspace_bytes(const n2d2hip_conv_desc* desc, int B, int H, int W)
{
    ConvF32 q;
    if (make_conv(desc, B, H, W, true, &q, "n2d2hip_conv2d_f32_workspace_bytes") != N2D2HIP_OK || !use_gemm(q) || !fits_int(q))
        return 0;
    GemmF32 g = make_gemm(q, GEMM_BWD_FILTER);
    size_t need = (size_t)filter_splits(&g) * g.Q * g.P;
    for (int mode : {GEMM_FWD, GEMM_BWD_DATA}) {
        g = make_gemm(q, mode);
        const int splits = pass_splits(&g);
        if (splits > 1)
            need = std::max(need, (size_t)splits * g.Q * g.P);
    }
    return need * sizeof(float);
}

int n2d2hip_conv2d_f32_backward_filter(const n2d2hip_conv_desc* desc, int B, int H, int W, const float* x, const float* diff_y, float beta,
                                       float* diff_w, void* workspace, size_t workspace_bytes, n2d2hip_stream_t stream)
{
    ConvF32 q;
    const int st = make_conv(desc, B, H, W, true, &q, "n2d2hip_conv2d_f32_backward_filter");
    if (st != N2D2HIP_OK) return st;
    N2D2HIP_REQUIRE(x && diff_y && diff_w, N2D2HIP_ERR_INVALID, "n2d2hip_conv2d_f32_backward_filter: null pointer");
    const size_t nw = (size_t)q.O * q.Cw * q.kH * q.kW;
    N2D2HIP_REQUIRE(nw < ((size_t)1 << 31), N2D2HIP_ERR_INVALID, "n2d2hip_conv2d_f32_backward_filter: too many weights");
    if (use_gemm(q) && fits_int(q)) {
        GemmF32 g = make_gemm(q, GEMM_BWD_FILTER);
        const int splits = filter_splits(&g);
        const size_t need = (size_t)splits * nw * sizeof(float);
        N2D2HIP_REQUIRE(workspace && workspace_bytes >= need, N2D2HIP_ERR_WORKSPACE,
                        "n2d2hip_conv2d_f32_backward_filter: workspace of %zu bytes, %zu needed (n2d2hip_conv2d_f32_workspace_bytes)",
                        workspace_bytes, need);
        if (g.Q <= 64)
            hipLaunchKernelGGL((conv_f32_gemm_kernel<GEMM_BWD_FILTER, 64>), dim3((g.P + GT - 1) / GT, 1, splits), dim3(256), 0,
                               (hipStream_t)stream, g, x, diff_y, (const float*)nullptr, 0.0f, (float*)workspace);
        else
            hipLaunchKernelGGL((conv_f32_gemm_kernel<GEMM_BWD_FILTER, 128>), dim3((g.P + GT - 1) / GT, (g.Q + GT - 1) / GT, splits), dim3(256), 0,
                               (hipStream_t)stream, g, x, diff_y, (const float*)nullptr, 0.0f, (float*)workspace);
        hipLaunchKernelGGL(conv_f32_reduce_partials_kernel, dim3(grid_for(nw)), dim3(256), 0, (hipStream_t)stream, (const float*)workspace, splits, nw,
                           beta, diff_w, (const float*)nullptr, 1, 1);
        N2D2HIP_HIP_CHECK(hipGetLastError());
        return N2D2HIP_OK;
    }
    hipLaunchKernelGGL(conv_f32_backward_filter_kernel, dim3((unsigned)nw), dim3(TBLOCK), 0, (hipStream_t)stream, q, x, diff_y, beta, diff_w);
    N2D2HIP_HIP_CHECK(hipGetLastError());
    return N2D2HIP_OK;
}

int n2d2hip_conv2d_f32_backward_bias(int B, int O, int oH, int oW, const float* diff_y, float beta, float* diff_bias, n2d2hip_stream_t stream)
{
    N2D2HIP_REQUIRE(B > 0 && O > 0 && oH > 0 && oW > 0 && diff_y && diff_bias, N2D2HIP_ERR_INVALID, "n2d2hip_conv2d_f32_backward_bias: bad argument");
    hipLaunchKernelGGL(conv_f32_backward_bias_kernel, dim3(O), dim3(TBLOCK), 0, (hipStream_t)stream, B, O, oH * oW, diff_y, beta, diff_bias);
    N2D2HIP_HIP_CHECK(hipGetLastError());
    return N2D2HIP_OK;
}

int n2d2hip_softmax_f32_forward(const float* x, float* y, int B, int C, int H, int W, n2d2hip_stream_t stream)
{
    N2D2HIP_REQUIRE(B > 0 && C > 0 && H > 0 && W > 0 && x && y, N2D2HIP_ERR_INVALID, "n2d2hip_softmax_f32_forward: bad argument");
    hipLaunchKernelGGL(softmax_f32_kernel, dim3(grid_for((size_t)B * H * W)), dim3(TBLOCK), 0, (hipStream_t)stream, x, y, B, C, H * W);
    N2D2HIP_HIP_CHECK(hipGetLastError());
    return N2D2HIP_OK;
}

int n2d2hip_rectifier_f32_forward(float* x, size_t n, float leak_slope, float clipping, n2d2hip_stream_t stream)
{
    N2D2HIP_REQUIRE(x && n > 0 && clipping >= 0.0f, N2D2HIP_ERR_INVALID, "n2d2hip_rectifier_f32_forward: bad argument");
    hipLaunchKernelGGL(rectifier_f32_forward_kernel, dim3(grid_for(n)), dim3(TBLOCK), 0, (hipStream_t)stream, x, n, leak_slope, clipping);
    N2D2HIP_HIP_CHECK(hipGetLastError());
    return N2D2HIP_OK;
}

int n2d2hip_rectifier_f32_backward(const float* output, const float* diff_in, float* diff_out, size_t n, float leak_slope, float clipping,
                                   n2d2hip_stream_t stream)
{
    N2D2HIP_REQUIRE(output && diff_in && diff_out && n > 0 && clipping >= 0.0f, N2D2HIP_ERR_INVALID, "n2d2hip_rectifier_f32_backward: bad argument");
    hipLaunchKernelGGL(rectifier_f32_backward_kernel, dim3(grid_for(n)), dim3(TBLOCK), 0, (hipStream_t)stream, output, diff_in, diff_out, n,
                       leak_slope, clipping);
    N2D2HIP_HIP_CHECK(hipGetLastError());
    return N2D2HIP_OK;
}

// Blocks per channel for the sums over batch and pixels: about 1024 blocks in all, at least 4096 values each, at most 64.
static int bn_splits(int B, int C, int H, int W)
{
    const size_t n = (size_t)B * H * W;
    const size_t by_size = n / 4096;
    const size_t by_grid = (size_t)std::max(1024 / C, 1);
    return (int)std::max<size_t>(1, std::min<size_t>(std::min(by_size, by_grid), 64));
}

size_t n2d2hip_batchnorm_f32_workspace_bytes(int B, int C, int H, int W)
{
    if (B <= 0 || C <= 0 || H <= 0 || W <= 0)
        return 0;
    return (size_t)C * bn_splits(B, C, H, W) * 5 * sizeof(double);
}

int n2d2hip_batchnorm_f32_forward(int B, int C, int H, int W, const float* x, const float* scale, const float* bias, float* mean,
                                  float* variance, float* saved_mean, float* saved_variance, double epsilon, double moving_average_momentum,
                                  int use_running, float* y, void* workspace, size_t workspace_bytes, n2d2hip_stream_t stream)
{
    N2D2HIP_REQUIRE(B > 0 && C > 0 && H > 0 && W > 0 && x && scale && bias && mean && variance && y && epsilon > 0.0, N2D2HIP_ERR_INVALID,
                    "n2d2hip_batchnorm_f32_forward: bad argument");
    N2D2HIP_REQUIRE((size_t)B * C < ((size_t)1 << 31) && (size_t)H * W < ((size_t)1 << 31), N2D2HIP_ERR_INVALID,
                    "n2d2hip_batchnorm_f32_forward: tensor too large");
    const bool running = use_running || moving_average_momentum == 0.0;
    if (!running) {
        N2D2HIP_REQUIRE(saved_mean && saved_variance, N2D2HIP_ERR_INVALID, "n2d2hip_batchnorm_f32_forward: the learning pass needs saved_mean and saved_variance");
        N2D2HIP_REQUIRE((size_t)B * H * W > 1, N2D2HIP_ERR_INVALID, "n2d2hip_batchnorm_f32_forward: batch statistics need more than one value per channel");
        const int splits = bn_splits(B, C, H, W);
        if (splits > 1 && workspace && workspace_bytes >= n2d2hip_batchnorm_f32_workspace_bytes(B, C, H, W)) {
            double* ws_sum = (double*)workspace;
            double* ws_sq = ws_sum + (size_t)C * splits;
            hipLaunchKernelGGL(batchnorm_f32_sum_partial_kernel, dim3(C, splits), dim3(TBLOCK), 0, (hipStream_t)stream, B, C, H * W, splits, x, ws_sum);
            hipLaunchKernelGGL(batchnorm_f32_sq_partial_kernel, dim3(C, splits), dim3(TBLOCK), 0, (hipStream_t)stream, B, C, H * W, splits, x,
                               (const double*)ws_sum, ws_sq);
            hipLaunchKernelGGL(batchnorm_f32_stats_finish_kernel, dim3((C + TBLOCK - 1) / TBLOCK), dim3(TBLOCK), 0, (hipStream_t)stream, C,
                               (size_t)B * H * W, splits, (const double*)ws_sum, (const double*)ws_sq, mean, variance, saved_mean, saved_variance,
                               moving_average_momentum);
        } else {
            hipLaunchKernelGGL(batchnorm_f32_stats_kernel, dim3(C), dim3(TBLOCK), 0, (hipStream_t)stream, B, C, H * W, x, mean, variance, saved_mean,
                               saved_variance, moving_average_momentum);
        }
    }
    const int plane = H * W;
    // 16 bytes per lane when every plane starts on a 16-byte boundary
    const int vec = plane % 4 == 0 && ((uintptr_t)x | (uintptr_t)y) % 16 == 0;
    const dim3 plane_grid((unsigned)std::max(1, std::min(((vec ? plane / 4 : plane) + TBLOCK - 1) / TBLOCK, 64)),
                          (unsigned)std::min<size_t>((size_t)B * C, 32768));
    if (plane >= 512)
        hipLaunchKernelGGL(batchnorm_f32_apply_kernel, plane_grid, dim3(TBLOCK), 0, (hipStream_t)stream, B * C, C, plane, x, scale, bias,
                           running ? (const float*)mean : (const float*)saved_mean, running ? (const float*)variance : (const float*)saved_variance,
                           epsilon, running ? 1 : 0, vec, y);
    else
        hipLaunchKernelGGL(batchnorm_f32_apply_flat_kernel, dim3(grid_for((size_t)B * C * plane)), dim3(TBLOCK), 0, (hipStream_t)stream,
                           (size_t)B * C * plane, C, plane, x, scale, bias, running ? (const float*)mean : (const float*)saved_mean,
                           running ? (const float*)variance : (const float*)saved_variance, epsilon, running ? 1 : 0, y);
    N2D2HIP_HIP_CHECK(hipGetLastError());
    return N2D2HIP_OK;
}

int n2d2hip_batchnorm_f32_backward(int B, int C, int H, int W, const float* x, const float* scale, const float* saved_mean,
                                   const float* saved_variance, double epsilon, const float* diff_y, float beta_scale, float* diff_scale,
                                   float beta_bias, float* diff_bias, float* diff_saved_mean, float* diff_saved_variance, float* diff_x,
                                   void* workspace, size_t workspace_bytes, n2d2hip_stream_t stream)
{
    N2D2HIP_REQUIRE(B > 0 && C > 0 && H > 0 && W > 0 && x && scale && saved_mean && saved_variance && diff_y && diff_scale && diff_bias
                        && diff_saved_mean && diff_saved_variance && epsilon > 0.0,
                    N2D2HIP_ERR_INVALID, "n2d2hip_batchnorm_f32_backward: bad argument");
    N2D2HIP_REQUIRE((size_t)B * C < ((size_t)1 << 31) && (size_t)H * W < ((size_t)1 << 31), N2D2HIP_ERR_INVALID,
                    "n2d2hip_batchnorm_f32_backward: tensor too large");
    const int splits = bn_splits(B, C, H, W);
    if (splits > 1 && workspace && workspace_bytes >= n2d2hip_batchnorm_f32_workspace_bytes(B, C, H, W)) {
        hipLaunchKernelGGL(batchnorm_f32_backward_partial_kernel, dim3(C, splits), dim3(TBLOCK), 0, (hipStream_t)stream, B, C, H * W, splits, x, scale,
                           saved_mean, saved_variance, epsilon, diff_y, (double*)workspace);
        hipLaunchKernelGGL(batchnorm_f32_backward_finish_kernel, dim3((C + TBLOCK - 1) / TBLOCK), dim3(TBLOCK), 0, (hipStream_t)stream, C,
                           (size_t)B * H * W, splits, (const double*)workspace, saved_variance, epsilon, beta_scale, diff_scale, beta_bias, diff_bias,
                           diff_saved_mean, diff_saved_variance);
    } else {
        hipLaunchKernelGGL(batchnorm_f32_backward_sums_kernel, dim3(C), dim3(TBLOCK), 0, (hipStream_t)stream, B, C, H * W, x, scale, saved_mean,
                           saved_variance, epsilon, diff_y, beta_scale, diff_scale, beta_bias, diff_bias, diff_saved_mean, diff_saved_variance);
    }
    const int plane = H * W;
    const int vec = plane % 4 == 0 && ((uintptr_t)x | (uintptr_t)diff_y | (uintptr_t)diff_x) % 16 == 0;
    const dim3 plane_grid((unsigned)std::max(1, std::min(((vec ? plane / 4 : plane) + TBLOCK - 1) / TBLOCK, 64)),
                          (unsigned)std::min<size_t>((size_t)B * C, 32768));
    if (diff_x && plane >= 512)
        hipLaunchKernelGGL(batchnorm_f32_backward_data_kernel, plane_grid, dim3(TBLOCK), 0, (hipStream_t)stream, B * C, C, plane,
                           (float)((size_t)B * H * W), x, scale, saved_mean, saved_variance, epsilon, diff_y, (const float*)diff_saved_mean,
                           (const float*)diff_saved_variance, vec, diff_x);
    else if (diff_x)
        hipLaunchKernelGGL(batchnorm_f32_backward_data_flat_kernel, dim3(grid_for((size_t)B * C * plane)), dim3(TBLOCK), 0, (hipStream_t)stream,
                           (size_t)B * C * plane, C, plane, (float)((size_t)B * H * W), x, scale, saved_mean, saved_variance, epsilon, diff_y,
                           (const float*)diff_saved_mean, (const float*)diff_saved_variance, diff_x);
    N2D2HIP_HIP_CHECK(hipGetLastError());
    return N2D2HIP_OK;
}

static int make_pool(int B, int C, int H, int W, int pool_w, int pool_h, int stride_x, int stride_y, int pad_x, int pad_y, PoolF32* q, const char* who)
{
    N2D2HIP_REQUIRE(B > 0 && C > 0 && H > 0 && W > 0 && pool_w > 0 && pool_h > 0 && stride_x > 0 && stride_y > 0 && pad_x >= 0 && pad_y >= 0,
                    N2D2HIP_ERR_INVALID, "%s: bad argument", who);
    N2D2HIP_REQUIRE(pad_x < pool_w && pad_y < pool_h, N2D2HIP_ERR_INVALID, "%s: padding must be smaller than the window", who);
    q->B = B; q->C = C; q->H = H; q->W = W;
    q->pw = pool_w; q->ph = pool_h; q->sx = stride_x; q->sy = stride_y; q->px = pad_x; q->py = pad_y;
    // PoolCell::setOutputsDims (src/Cell/PoolCell.cpp:219-240)
    q->oW = (int)((W + 2 * pad_x - pool_w + stride_x) / (double)stride_x);
    q->oH = (int)((H + 2 * pad_y - pool_h + stride_y) / (double)stride_y);
    N2D2HIP_REQUIRE(q->oW > 0 && q->oH > 0, N2D2HIP_ERR_INVALID, "%s: the window does not fit the input", who);
    N2D2HIP_REQUIRE((size_t)H * W < ((size_t)1 << 31) && (size_t)B * C * H * W < ((size_t)1 << 40), N2D2HIP_ERR_INVALID, "%s: tensor too large", who);
    return N2D2HIP_OK;
}

int n2d2hip_pool_max_f32_forward(int B, int C, int H, int W, int pool_w, int pool_h, int stride_x, int stride_y, int pad_x, int pad_y,
                                 const float* x, float* y, int* argmax, n2d2hip_stream_t stream)
{
    PoolF32 q;
    const int rc = make_pool(B, C, H, W, pool_w, pool_h, stride_x, stride_y, pad_x, pad_y, &q, "n2d2hip_pool_max_f32_forward");
    if (rc != N2D2HIP_OK) return rc;
    N2D2HIP_REQUIRE(x && y && argmax, N2D2HIP_ERR_INVALID, "n2d2hip_pool_max_f32_forward: null pointer");
    hipLaunchKernelGGL(pool_max_f32_forward_kernel, dim3(grid_for((size_t)B * C * q.oH * q.oW)), dim3(TBLOCK), 0, (hipStream_t)stream, q, x, y, argmax);
    N2D2HIP_HIP_CHECK(hipGetLastError());
    return N2D2HIP_OK;
}

int n2d2hip_pool_max_f32_backward(int B, int C, int H, int W, int pool_w, int pool_h, int stride_x, int stride_y, int pad_x, int pad_y,
                                  const float* diff_y, const int* argmax, float beta, float* diff_x, n2d2hip_stream_t stream)
{
    PoolF32 q;
    const int rc = make_pool(B, C, H, W, pool_w, pool_h, stride_x, stride_y, pad_x, pad_y, &q, "n2d2hip_pool_max_f32_backward");
    if (rc != N2D2HIP_OK) return rc;
    N2D2HIP_REQUIRE(diff_y && argmax && diff_x, N2D2HIP_ERR_INVALID, "n2d2hip_pool_max_f32_backward: null pointer");
    hipLaunchKernelGGL(pool_max_f32_backward_kernel, dim3(grid_for((size_t)B * C * H * W)), dim3(TBLOCK), 0, (hipStream_t)stream, q, diff_y, argmax, beta,
                       diff_x);
    N2D2HIP_HIP_CHECK(hipGetLastError());
    return N2D2HIP_OK;
}

}  // extern "C"

// Average pooling of float NCHW with the unit mapping: the window's values are added in row-major order and divided
// by the window's size (count_include_padding) or by the number of values inside the input.
__global__ __launch_bounds__(TBLOCK) void pool_average_f32_forward_kernel(PoolF32 q, int count_include_padding, const float* __restrict__ x,
                                                                          float* __restrict__ y)
{
    const size_t total = (size_t)q.B * q.C * q.oH * q.oW;
    for (size_t i = (size_t)blockIdx.x * TBLOCK + threadIdx.x; i < total; i += (size_t)gridDim.x * TBLOCK) {
        const int ox = (int)(i % q.oW), oy = (int)((i / q.oW) % q.oH);
        const size_t bc = i / ((size_t)q.oW * q.oH);
        const float* in = x + bc * (size_t)q.H * q.W;
        const int x0 = ox * q.sx - q.px, y0 = oy * q.sy - q.py;
        const int sx_min = max(-x0, 0), sy_min = max(-y0, 0);
        const int sx_max = min(max(q.W - x0, 0), q.pw), sy_max = min(max(q.H - y0, 0), q.ph);
        float acc = 0.0f;
        for (int sy = sy_min; sy < sy_max; ++sy)
            for (int sx = sx_min; sx < sx_max; ++sx)
                acc += in[(size_t)(y0 + sy) * q.W + x0 + sx];
        const int inside = max(sx_max - sx_min, 0) * max(sy_max - sy_min, 0);
        const unsigned count = count_include_padding ? (unsigned)(q.pw * q.ph) : (unsigned)inside;
        y[i] = count > 0 ? acc / (float)count : 0.0f;
    }
}

// Every input collects the gradients of the windows it lies in, in the reference's order (window rows, then columns,
// from the input's own residue modulo the stride upwards); the sum is divided by the window's size.
__global__ __launch_bounds__(TBLOCK) void pool_average_f32_backward_kernel(PoolF32 q, const float* __restrict__ dy, float beta, float* __restrict__ dx)
{
    const size_t total = (size_t)q.B * q.C * q.H * q.W;
    const float count = (float)(unsigned)(q.pw * q.ph);
    for (size_t i = (size_t)blockIdx.x * TBLOCK + threadIdx.x; i < total; i += (size_t)gridDim.x * TBLOCK) {
        const int ix = (int)(i % q.W), iy = (int)((i / q.W) % q.H);
        const size_t bc = i / ((size_t)q.W * q.H);
        const int ix_pad = ix + q.px, iy_pad = iy + q.py;
        const int sx_max = min(q.pw, ix_pad + 1), sy_max = min(q.ph, iy_pad + 1);
        float acc = 0.0f;
        for (int sy = iy_pad % q.sy; sy < sy_max; sy += q.sy) {
            if (iy_pad >= q.sy * q.oH + sy)
                continue;
            const int oy = (iy_pad - sy) / q.sy;
            for (int sx = ix_pad % q.sx; sx < sx_max; sx += q.sx) {
                if (ix_pad >= q.sx * q.oW + sx)
                    continue;
                const int ox = (ix_pad - sx) / q.sx;
                acc += dy[(bc * q.oH + oy) * q.oW + ox];
            }
        }
        const float g = acc / count;
        dx[i] = beta != 0.0f ? __fadd_rn(g, __fmul_rn(beta, dx[i])) : g;
    }
}

extern "C" {

int n2d2hip_pool_average_f32_forward(int B, int C, int H, int W, int pool_w, int pool_h, int stride_x, int stride_y, int pad_x, int pad_y,
                                     int count_include_padding, const float* x, float* y, n2d2hip_stream_t stream)
{
    PoolF32 q;
    const int rc = make_pool(B, C, H, W, pool_w, pool_h, stride_x, stride_y, pad_x, pad_y, &q, "n2d2hip_pool_average_f32_forward");
    if (rc != N2D2HIP_OK) return rc;
    N2D2HIP_REQUIRE(x && y, N2D2HIP_ERR_INVALID, "n2d2hip_pool_average_f32_forward: null pointer");
    hipLaunchKernelGGL(pool_average_f32_forward_kernel, dim3(grid_for((size_t)B * C * q.oH * q.oW)), dim3(TBLOCK), 0, (hipStream_t)stream, q,
                       count_include_padding ? 1 : 0, x, y);
    N2D2HIP_HIP_CHECK(hipGetLastError());
    return N2D2HIP_OK;
}

int n2d2hip_pool_average_f32_backward(int B, int C, int H, int W, int pool_w, int pool_h, int stride_x, int stride_y, int pad_x, int pad_y,
                                      int count_include_padding, const float* diff_y, float beta, float* diff_x, n2d2hip_stream_t stream)
{
    PoolF32 q;
    const int rc = make_pool(B, C, H, W, pool_w, pool_h, stride_x, stride_y, pad_x, pad_y, &q, "n2d2hip_pool_average_f32_backward");
    if (rc != N2D2HIP_OK) return rc;
    // the reference throws for the other case (src/Cell/PoolCell_Frame_Kernels.cpp:210-213)
    N2D2HIP_REQUIRE(count_include_padding, N2D2HIP_ERR_UNSUPPORTED, "n2d2hip_pool_average_f32_backward: exclude padding not implemented");
    N2D2HIP_REQUIRE(diff_y && diff_x, N2D2HIP_ERR_INVALID, "n2d2hip_pool_average_f32_backward: null pointer");
    hipLaunchKernelGGL(pool_average_f32_backward_kernel, dim3(grid_for((size_t)B * C * H * W)), dim3(TBLOCK), 0, (hipStream_t)stream, q, diff_y, beta,
                       diff_x);
    N2D2HIP_HIP_CHECK(hipGetLastError());
    return N2D2HIP_OK;
}

}  // extern "C"

// Weighted sum of up to N2D2HIP_ELEMWISE_F32_MAX_INPUTS float tensors of one shape: products and sums are rounded one
// by one, in the order of the inputs, as the reference's scalar loop does.
struct ElemWiseF32 {
    const float* x[N2D2HIP_ELEMWISE_F32_MAX_INPUTS];
    float w[N2D2HIP_ELEMWISE_F32_MAX_INPUTS], s[N2D2HIP_ELEMWISE_F32_MAX_INPUTS];
    int n;
};

__device__ __forceinline__ float elemwise_sum_one(const ElemWiseF32& e, const float* v)
{
    float acc = __fadd_rn(__fmul_rn(e.w[0], v[0]), e.s[0]);
#pragma unroll
    for (int k = 1; k < N2D2HIP_ELEMWISE_F32_MAX_INPUTS; ++k)
        if (k < e.n)
            acc = __fadd_rn(acc, __fadd_rn(__fmul_rn(e.w[k], v[k]), e.s[k]));
    return acc;
}

template <int VEC>
__global__ __launch_bounds__(TBLOCK) void elemwise_sum_f32_forward_kernel(ElemWiseF32 e, size_t total, float* __restrict__ y)
{
    for (size_t i = (size_t)blockIdx.x * TBLOCK + threadIdx.x; i < total / VEC; i += (size_t)gridDim.x * TBLOCK) {
        if (VEC == 4) {
            float4 v[N2D2HIP_ELEMWISE_F32_MAX_INPUTS];
#pragma unroll
            for (int k = 0; k < N2D2HIP_ELEMWISE_F32_MAX_INPUTS; ++k)
                if (k < e.n)
                    v[k] = ((const float4*)e.x[k])[i];
            float a[N2D2HIP_ELEMWISE_F32_MAX_INPUTS], b[N2D2HIP_ELEMWISE_F32_MAX_INPUTS], c[N2D2HIP_ELEMWISE_F32_MAX_INPUTS],
                d[N2D2HIP_ELEMWISE_F32_MAX_INPUTS];
#pragma unroll
            for (int k = 0; k < N2D2HIP_ELEMWISE_F32_MAX_INPUTS; ++k)
                if (k < e.n) {
                    a[k] = v[k].x; b[k] = v[k].y; c[k] = v[k].z; d[k] = v[k].w;
                }
            float4 o;
            o.x = elemwise_sum_one(e, a);
            o.y = elemwise_sum_one(e, b);
            o.z = elemwise_sum_one(e, c);
            o.w = elemwise_sum_one(e, d);
            ((float4*)y)[i] = o;
        } else {
            float a[N2D2HIP_ELEMWISE_F32_MAX_INPUTS];
#pragma unroll
            for (int k = 0; k < N2D2HIP_ELEMWISE_F32_MAX_INPUTS; ++k)
                if (k < e.n)
                    a[k] = e.x[k][i];
            y[i] = elemwise_sum_one(e, a);
        }
    }
}

// diff_x = weight * diff_y + beta * diff_x
template <int VEC>
__global__ __launch_bounds__(TBLOCK) void elemwise_sum_f32_backward_kernel(size_t total, float weight, const float* __restrict__ dy, float beta, float* dx)
{
    for (size_t i = (size_t)blockIdx.x * TBLOCK + threadIdx.x; i < total / VEC; i += (size_t)gridDim.x * TBLOCK) {
        if (VEC == 4) {
            const float4 d = ((const float4*)dy)[i];
            float4 o = make_float4(__fmul_rn(weight, d.x), __fmul_rn(weight, d.y), __fmul_rn(weight, d.z), __fmul_rn(weight, d.w));
            if (beta != 0.0f) {
                const float4 p = ((const float4*)dx)[i];
                o.x = __fadd_rn(o.x, __fmul_rn(beta, p.x));
                o.y = __fadd_rn(o.y, __fmul_rn(beta, p.y));
                o.z = __fadd_rn(o.z, __fmul_rn(beta, p.z));
                o.w = __fadd_rn(o.w, __fmul_rn(beta, p.w));
            }
            ((float4*)dx)[i] = o;
        } else {
            const float g = __fmul_rn(weight, dy[i]);
            dx[i] = beta != 0.0f ? __fadd_rn(g, __fmul_rn(beta, dx[i])) : g;
        }
    }
}

extern "C" {

int n2d2hip_elemwise_sum_f32_forward(int nb_inputs, const float* const* inputs, size_t n, const float* weights, const float* shifts, float* y,
                                     n2d2hip_stream_t stream)
{
    N2D2HIP_REQUIRE(nb_inputs > 0 && inputs && weights && shifts && y && n > 0, N2D2HIP_ERR_INVALID, "n2d2hip_elemwise_sum_f32_forward: bad argument");
    N2D2HIP_REQUIRE(nb_inputs <= N2D2HIP_ELEMWISE_F32_MAX_INPUTS, N2D2HIP_ERR_UNSUPPORTED, "n2d2hip_elemwise_sum_f32_forward: at most %d inputs",
                    N2D2HIP_ELEMWISE_F32_MAX_INPUTS);
    ElemWiseF32 e = {};
    e.n = nb_inputs;
    uintptr_t align = (uintptr_t)y;
    for (int k = 0; k < nb_inputs; ++k) {
        N2D2HIP_REQUIRE(inputs[k], N2D2HIP_ERR_INVALID, "n2d2hip_elemwise_sum_f32_forward: input %d is null", k);
        e.x[k] = inputs[k];
        e.w[k] = weights[k];
        e.s[k] = shifts[k];
        align |= (uintptr_t)inputs[k];
    }
    if (n % 4 == 0 && align % 16 == 0)
        hipLaunchKernelGGL(elemwise_sum_f32_forward_kernel<4>, dim3(grid_for(n / 4)), dim3(TBLOCK), 0, (hipStream_t)stream, e, n, y);
    else
        hipLaunchKernelGGL(elemwise_sum_f32_forward_kernel<1>, dim3(grid_for(n)), dim3(TBLOCK), 0, (hipStream_t)stream, e, n, y);
    N2D2HIP_HIP_CHECK(hipGetLastError());
    return N2D2HIP_OK;
}

int n2d2hip_elemwise_sum_f32_backward(size_t n, float weight, const float* diff_y, float beta, float* diff_x, n2d2hip_stream_t stream)
{
    N2D2HIP_REQUIRE(n > 0 && diff_y && diff_x, N2D2HIP_ERR_INVALID, "n2d2hip_elemwise_sum_f32_backward: bad argument");
    if (n % 4 == 0 && ((uintptr_t)diff_y | (uintptr_t)diff_x) % 16 == 0)
        hipLaunchKernelGGL(elemwise_sum_f32_backward_kernel<4>, dim3(grid_for(n / 4)), dim3(TBLOCK), 0, (hipStream_t)stream, n, weight, diff_y, beta, diff_x);
    else
        hipLaunchKernelGGL(elemwise_sum_f32_backward_kernel<1>, dim3(grid_for(n)), dim3(TBLOCK), 0, (hipStream_t)stream, n, weight, diff_y, beta, diff_x);
    N2D2HIP_HIP_CHECK(hipGetLastError());
    return N2D2HIP_OK;
}

size_t n2d2hip_loss_workspace_bytes(size_t n)
{
    return (size_t)grid_for(n) * sizeof(double);
}

int n2d2hip_loss_f32(const float* target, const float* output, float* diff, size_t n, int batch, double* loss,
                     void* workspace, size_t workspace_bytes, n2d2hip_stream_t stream)
{
    N2D2HIP_REQUIRE(target && output && diff && loss && n > 0 && batch > 0, N2D2HIP_ERR_INVALID, "n2d2hip_loss_f32: bad argument");
    const int nb = grid_for(n);
    N2D2HIP_REQUIRE(workspace && workspace_bytes >= (size_t)nb * sizeof(double), N2D2HIP_ERR_WORKSPACE,
                    "n2d2hip_loss_f32: workspace of %zu bytes, %zu needed", workspace_bytes, (size_t)nb * sizeof(double));
    hipLaunchKernelGGL(loss_f32_kernel, dim3(nb), dim3(TBLOCK), 0, (hipStream_t)stream, target, output, diff, n, (double*)workspace);
    hipLaunchKernelGGL(loss_finish_kernel, dim3(1), dim3(TBLOCK), 0, (hipStream_t)stream, (const double*)workspace, nb, 1.0 / batch, loss);
    N2D2HIP_HIP_CHECK(hipGetLastError());
    return N2D2HIP_OK;
}

int n2d2hip_sgd_update_f32(float* data, const float* diff, size_t n, float rate_diff, float momentum, float decay_times_rate,
                           float* momentum_data, int clamp, float clamp_min, float clamp_max, n2d2hip_stream_t stream)
{
    N2D2HIP_REQUIRE(data && diff && n > 0, N2D2HIP_ERR_INVALID, "n2d2hip_sgd_update_f32: bad argument");
    N2D2HIP_REQUIRE(momentum_data || (momentum == 0.0f && decay_times_rate == 0.0f), N2D2HIP_ERR_INVALID,
                    "n2d2hip_sgd_update_f32: momentum or decay without a momentum buffer");
    hipLaunchKernelGGL(sgd_f32_kernel, dim3(grid_for(n)), dim3(TBLOCK), 0, (hipStream_t)stream, data, diff, n, rate_diff, momentum,
                       decay_times_rate, momentum_data, clamp_min, clamp_max, clamp);
    N2D2HIP_HIP_CHECK(hipGetLastError());
    return N2D2HIP_OK;
}

} // extern "C"
