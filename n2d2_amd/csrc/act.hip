// Error plumbing, tensor checks, the per-cell rescale/activation tables, the
// stand-alone Scaling kernel and the graph-edge conversion kernel.
#include <cmath>
#include <limits>

#include "common.h"
#include "epilogue.hpp"

namespace n2d2hip {

static thread_local std::string g_last_error;

int fail(int code, const char* fmt, ...)
{
    char buf[1024];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof(buf), fmt, ap);
    va_end(ap);
    g_last_error = buf;
    return code;
}

// ---- launch log of the calling thread
struct LaunchRecord {
    std::string name;
    unsigned grid, block;
    long long slot;
};
static thread_local bool g_log_open = false;
static thread_local std::vector<LaunchRecord> g_log;

void launch_log_add(const char* pretty, unsigned grid, unsigned block, long long slot)
{
    if (!g_log_open)
        return;
    // "... [K = &n2d2hip::kernel<args>]" -> "kernel<args>"
    std::string name(pretty);
    const size_t eq = name.find("K = ");
    if (eq != std::string::npos) {
        name = name.substr(eq + 4);
        if (!name.empty() && name.back() == ']') name.pop_back();
        if (!name.empty() && name[0] == '&') name.erase(0, 1);
        if (!name.empty() && name[0] == '(') { name.erase(0, 1); if (!name.empty() && name.back() == ')') name.pop_back(); }
        for (size_t at; (at = name.find("n2d2hip::")) != std::string::npos;) name.erase(at, 9);
    }
    g_log.push_back(LaunchRecord{name, grid, block, slot});
}

int check_tensor(const n2d2hip_tensor* t, const char* what, bool halo_ok, bool s2d_ok)
{
    N2D2HIP_REQUIRE(t != nullptr, N2D2HIP_ERR_INVALID, "%s: null tensor descriptor", what);
    N2D2HIP_REQUIRE(t->data != nullptr, N2D2HIP_ERR_INVALID, "%s: null data pointer", what);
    N2D2HIP_REQUIRE(t->dtype >= N2D2HIP_U8 && t->dtype <= N2D2HIP_U8B, N2D2HIP_ERR_INVALID, "%s: bad dtype %d", what, t->dtype);
    N2D2HIP_REQUIRE(t->layout == N2D2HIP_NCHW || t->layout == N2D2HIP_NHWC || t->layout == N2D2HIP_S2D, N2D2HIP_ERR_INVALID,
                    "%s: bad layout %d", what, t->layout);
    N2D2HIP_REQUIRE(t->B > 0 && t->C > 0 && t->H > 0 && t->W > 0, N2D2HIP_ERR_INVALID,
                    "%s: empty tensor %dx%dx%dx%d", what, t->B, t->C, t->H, t->W);
    if (t->layout == N2D2HIP_NHWC)
        N2D2HIP_REQUIRE(t->cs >= t->C && (t->cs % 16 == 0 || t->cs == 4), N2D2HIP_ERR_INVALID,
                        "%s: NHWC channel stride %d invalid for %d channels (multiple of 16, or 4)", what, t->cs, t->C);
    N2D2HIP_REQUIRE(t->halo >= 0 && t->halo <= 16, N2D2HIP_ERR_INVALID, "%s: halo %d", what, t->halo);
    if (t->layout == N2D2HIP_S2D) {
        N2D2HIP_REQUIRE(s2d_ok, N2D2HIP_ERR_UNSUPPORTED, "%s: space-to-depth tensors are not accepted here", what);
        N2D2HIP_REQUIRE(t->C <= 4 && t->cs == 16 && elem_size(t->dtype) == 1, N2D2HIP_ERR_INVALID,
                        "%s: a space-to-depth tensor has at most 4 channels of bytes and 16-byte pixels (cs 16)", what);
        return N2D2HIP_OK;
    }
    if (t->halo > 0) {
        N2D2HIP_REQUIRE(halo_ok, N2D2HIP_ERR_UNSUPPORTED, "%s: tensors with a halo are not accepted here", what);
        N2D2HIP_REQUIRE(t->layout == N2D2HIP_NHWC && elem_size(t->dtype) == 1, N2D2HIP_ERR_INVALID,
                        "%s: only NHWC byte tensors have a halo", what);
    }
    return N2D2HIP_OK;
}

// floor(a / b) and ceil(a / b) for b > 0 on 128-bit integers
static __int128 floor_div(__int128 a, __int128 b) { __int128 q = a / b; return (a % b != 0 && ((a < 0) != (b < 0))) ? q - 1 : q; }
static __int128 ceil_div(__int128 a, __int128 b) { return -floor_div(-a, b); }
static long long clamp_ll(__int128 v, long long lo, long long hi) { return v < lo ? lo : (v > hi ? hi : (long long)v); }

// -------------------------------------------------------------- kernels

// One thread per element of the OUTPUT tensor.  Handles every dtype / layout
// pair; used at graph edges and by the stand-alone ScalingCell.
template <bool WITH_EPI>
__global__ void elementwise_kernel(const void* __restrict__ in, int in_dtype, int in_layout, int in_cs, int in_halo,
                                   void* __restrict__ out, int out_dtype, int out_layout, int out_cs,
                                   int B, int C, int H, int W, EpiArgs epi)
{
    const size_t outC = (out_layout == N2D2HIP_NHWC) ? (size_t)out_cs : (size_t)C;
    const size_t total = (size_t)B * H * W * outC;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x) {
        int b, c, y, x;
        if (out_layout == N2D2HIP_NHWC) {
            c = (int)(i % outC);
            size_t r = i / outC;
            x = (int)(r % W); r /= W;
            y = (int)(r % H);
            b = (int)(r / H);
        } else {
            x = (int)(i % W);
            size_t r = i / W;
            y = (int)(r % H); r /= H;
            c = (int)(r % C);
            b = (int)(r / C);
        }
        int v = 0;
        if (c < C) {
            const size_t j = (in_layout == N2D2HIP_NHWC)
                ? (((size_t)b * (H + 2 * in_halo) + y + in_halo) * (W + 2 * in_halo) + x + in_halo) * (size_t)in_cs + c
                : (((size_t)b * C + c) * H + y) * (size_t)W + x;
            v = load_value(in, j, in_dtype);
            if (WITH_EPI)
                v = epi_apply_dyn(epi, v, c);
        }
        store_value(out, i, out_dtype, v);
    }
}

} // namespace n2d2hip

using namespace n2d2hip;

extern "C" {

const char* n2d2hip_strerror(int status)
{
    switch (status) {
    case N2D2HIP_OK: return "success";
    case N2D2HIP_ERR_INVALID: return "invalid argument";
    case N2D2HIP_ERR_UNSUPPORTED: return "unsupported on the Frame_HIP path";
    case N2D2HIP_ERR_HIP: return "HIP runtime error";
    case N2D2HIP_ERR_NOT_QUANTIZED: return "integer scaling can only be used on a quantized network";
    case N2D2HIP_ERR_WORKSPACE: return "workspace too small";
    default: return "unknown status";
    }
}

const char* n2d2hip_last_error(void) { return g_last_error.c_str(); }

const char* n2d2hip_version(void) { return "n2d2hip 0.1 (gfx950)"; }

int n2d2hip_launch_log_begin(void)
{
    g_log.clear();
    g_log_open = true;
    return N2D2HIP_OK;
}

int n2d2hip_launch_log_end(int* count)
{
    N2D2HIP_REQUIRE(g_log_open, N2D2HIP_ERR_INVALID, "launch_log_end: no log is open on this thread");
    g_log_open = false;
    if (count) *count = (int)g_log.size();
    return N2D2HIP_OK;
}

int n2d2hip_launch_log_entry(int index, char* name, size_t capacity, int* grid, int* block, long long* probe_slot)
{
    N2D2HIP_REQUIRE(!g_log_open, N2D2HIP_ERR_INVALID, "launch_log_entry: the log is still open");
    N2D2HIP_REQUIRE(index >= 0 && (size_t)index < g_log.size(), N2D2HIP_ERR_INVALID, "launch_log_entry: index %d of %zu entries", index,
                    g_log.size());
    const LaunchRecord& r = g_log[(size_t)index];
    if (name && capacity > 0) {
        const size_t n = std::min(capacity - 1, r.name.size());
        memcpy(name, r.name.data(), n);
        name[n] = 0;
    }
    if (grid) *grid = (int)r.grid;
    if (block) *block = (int)r.block;
    if (probe_slot) *probe_slot = r.slot;
    return N2D2HIP_OK;
}

int n2d2hip_nhwc_cs(int C) { return C <= 4 ? 4 : round_up(C, 16); }

size_t n2d2hip_tensor_bytes(const n2d2hip_tensor* t)
{
    if (!t) return 0;
    if (t->layout == N2D2HIP_S2D)
        return (size_t)t->B * ((t->H + 1) / 2 + 2 * t->halo) * ((t->W + 1) / 2 + 2 * t->halo) * 16;
    const size_t c = (t->layout == N2D2HIP_NHWC) ? (size_t)t->cs : (size_t)t->C;
    return (size_t)t->B * (t->H + 2 * t->halo) * (t->W + 2 * t->halo) * c * (size_t)elem_size(t->dtype);
}

namespace n2d2hip {
__global__ void fill_bytes_kernel(uint4* __restrict__ p, size_t n16, unsigned v)
{
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n16; i += (size_t)gridDim.x * blockDim.x)
        p[i] = uint4{v, v, v, v};
}
} // namespace n2d2hip

int n2d2hip_tensor_clear(const n2d2hip_tensor* t, n2d2hip_stream_t stream)
{
    int rc;
    if ((rc = check_tensor(t, "tensor_clear", true)))
        return rc;
    N2D2HIP_REQUIRE(t->layout == N2D2HIP_NHWC && elem_size(t->dtype) == 1 && t->cs % 16 == 0, N2D2HIP_ERR_UNSUPPORTED,
                    "tensor_clear: NHWC byte tensors with a channel stride that is a multiple of 16");
    const size_t n16 = n2d2hip_tensor_bytes(t) / 16;
    const size_t blocks = std::min<size_t>((n16 + 255) / 256, 256 * 32);
    N2D2HIP_LAUNCH(fill_bytes_kernel, dim3((unsigned)std::max<size_t>(blocks, 1)), dim3(256), 0, (hipStream_t)stream, (uint4*)t->data, n16,
                       t->dtype == N2D2HIP_U8B ? 0x80808080u : 0u);
    N2D2HIP_HIP_CHECK(hipGetLastError());
    return N2D2HIP_OK;
}

namespace n2d2hip {
// Graph-edge conversion into the space-to-depth form: a thread writes two neighbouring 16-byte pixels of the stored image
// (32 bytes), border and empty channel slots included; it reads, per channel and input row, the four input pixels they
// hold, which for an NCHW source are contiguous bytes that neighbouring threads continue.
__global__ __launch_bounds__(256) void to_s2d_kernel(const void* __restrict__ in, int in_dtype, int in_layout, int in_cs, int in_halo,
                                                     signed char* __restrict__ out, int out_dtype, int B, int C, int H, int W, int halo)
{
    const int Hp = (H + 1) / 2 + 2 * halo, Wp = (W + 1) / 2 + 2 * halo, Wpairs = (Wp + 1) / 2;
    const int zero = out_dtype == N2D2HIP_U8B ? -128 : 0;
    // a wave per row of the stored image (4 rows per block), lanes along the row: no division by the row length
    const int rows = B * Hp;
    for (int row = (int)blockIdx.x * 4 + (int)(threadIdx.x >> 6); row < rows; row += (int)gridDim.x * 4)
    for (int xp = (int)(threadIdx.x & 63); xp < Wpairs; xp += 64) {
        const int b = row / Hp, Y = row - b * Hp;
        // the two pixels as eight dwords: dword (k >> 1) * 4 + dy * 2 + (k & 1) holds input column x0 + k of row dy, channel c in
        // byte c
        const unsigned zero4 = (unsigned)(zero & 255) * 0x01010101u;
        unsigned px[8];
#pragma unroll
        for (int k = 0; k < 8; ++k) px[k] = zero4;
        auto stored = [&](int v) -> unsigned {             // logical value -> the destination's stored byte
            if (out_dtype == N2D2HIP_U8B) return (unsigned)(clamp_i32(v, 0, 255) - 128) & 255u;
            if (out_dtype == N2D2HIP_U8) return (unsigned)clamp_i32(v, 0, 255);
            return (unsigned)clamp_i32(v, -128, 127) & 255u;
        };
        const int x0 = 2 * (2 * xp - halo);                  // first of the four input columns the two pixels hold
        // Byte planes whose four columns are one aligned dword inside the row: one load per channel and input row, all eight
        // requested before the first is used (a lane whose dword does not exist reads the tensor's first one and drops it)
        const bool planes = in_layout == N2D2HIP_NCHW && in_dtype != N2D2HIP_I32 && in_dtype != N2D2HIP_F32 && (W & 3) == 0 && (halo & 1) == 0;
        if (planes) {
            const bool cols = x0 >= 0 && x0 + 3 < W;          // (x0 is a multiple of 4 and so is W: all four columns or none)
            unsigned w[2][4];
            bool have[2];
#pragma unroll
            for (int dy = 0; dy < 2; ++dy) {
                const int y = 2 * (Y - halo) + dy;
                have[dy] = cols && y >= 0 && y < H;
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    const size_t at = (have[dy] && c < C) ? (((size_t)b * C + c) * H + y) * (size_t)W + x0 : 0;
                    w[dy][c] = *(const unsigned*)((const unsigned char*)in + at);
                }
            }
            // stored forms that differ by the sign bit at most (uint8 planes into the value - 128 form, or the same form on both
            // sides): the bytes are flipped four at a time and a 4 x 4 byte transpose puts the channels of a column side by side
            const bool same = in_dtype == out_dtype || (in_dtype == N2D2HIP_U8 && out_dtype == N2D2HIP_U8B) || (in_dtype == N2D2HIP_U8B && out_dtype == N2D2HIP_U8);
            if (same) {
                const unsigned flip = in_dtype == out_dtype ? 0u : 0x80808080u;
#pragma unroll
                for (int dy = 0; dy < 2; ++dy) {
                    if (!have[dy])
                        continue;
                    unsigned ch[4];
#pragma unroll
                    for (int c = 0; c < 4; ++c)
                        ch[c] = c < C ? (w[dy][c] ^ flip) : zero4;
                    const unsigned ab_lo = __builtin_amdgcn_perm(ch[1], ch[0], 0x05010400u), ab_hi = __builtin_amdgcn_perm(ch[1], ch[0], 0x07030602u);
                    const unsigned cd_lo = __builtin_amdgcn_perm(ch[3], ch[2], 0x05010400u), cd_hi = __builtin_amdgcn_perm(ch[3], ch[2], 0x07030602u);
                    px[0 * 4 + dy * 2 + 0] = __builtin_amdgcn_perm(cd_lo, ab_lo, 0x05040100u);      // column x0
                    px[0 * 4 + dy * 2 + 1] = __builtin_amdgcn_perm(cd_lo, ab_lo, 0x07060302u);      // column x0 + 1
                    px[1 * 4 + dy * 2 + 0] = __builtin_amdgcn_perm(cd_hi, ab_hi, 0x05040100u);      // column x0 + 2
                    px[1 * 4 + dy * 2 + 1] = __builtin_amdgcn_perm(cd_hi, ab_hi, 0x07060302u);      // column x0 + 3
                }
            } else {
#pragma unroll
                for (int dy = 0; dy < 2; ++dy)
#pragma unroll
                    for (int c = 0; c < 4; ++c) {
                        if (!have[dy] || c >= C)
                            continue;
                        const unsigned keep = ~(255u << (8 * c));
#pragma unroll
                        for (int k = 0; k < 4; ++k) {
                            const int byte = (int)((w[dy][c] >> (8 * k)) & 255u);
                            const int v = in_dtype == N2D2HIP_U8 ? byte : (in_dtype == N2D2HIP_I8 ? (int)(signed char)byte : (int)(signed char)byte + 128);
                            unsigned& d = px[(k >> 1) * 4 + dy * 2 + (k & 1)];
                            d = (d & keep) | (stored(v) << (8 * c));
                        }
                    }
            }
        } else {
#pragma unroll
            for (int dy = 0; dy < 2; ++dy) {
                const int y = 2 * (Y - halo) + dy;
                if (y < 0 || y >= H)
                    continue;
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    if (c >= C)
                        continue;
                    const unsigned keep = ~(255u << (8 * c));
#pragma unroll
                    for (int k = 0; k < 4; ++k) {
                        const int x = x0 + k, X = 2 * xp + (k >> 1);
                        if (X >= Wp || x < 0 || x >= W)
                            continue;
                        const size_t src = (in_layout == N2D2HIP_NHWC)
                            ? (((size_t)b * (H + 2 * in_halo) + y + in_halo) * (W + 2 * in_halo) + x + in_halo) * (size_t)in_cs + c
                            : (((size_t)b * C + c) * H + y) * (size_t)W + x;
                        unsigned& d = px[(k >> 1) * 4 + dy * 2 + (k & 1)];
                        d = (d & keep) | (stored(load_value(in, src, in_dtype)) << (8 * c));
                    }
                }
            }
        }
        signed char* dst = out + (((size_t)b * Hp + Y) * Wp + 2 * xp) * 16;
        *(uint4*)dst = uint4{px[0], px[1], px[2], px[3]};
        if (2 * xp + 1 < Wp)
            *(uint4*)(dst + 16) = uint4{px[4], px[5], px[6], px[7]};
    }
}
} // namespace n2d2hip

static int same_shape(const n2d2hip_tensor* a, const n2d2hip_tensor* b, const char* what)
{
    N2D2HIP_REQUIRE(a->B == b->B && a->C == b->C && a->H == b->H && a->W == b->W, N2D2HIP_ERR_INVALID,
                    "%s: shape mismatch %dx%dx%dx%d vs %dx%dx%dx%d", what, a->B, a->C, a->H, a->W, b->B, b->C, b->H, b->W);
    return N2D2HIP_OK;
}

static unsigned grid_for(size_t total, int block)
{
    size_t g = (total + block - 1) / block;
    const size_t cap = 256 * 32;
    return (unsigned)(g < 1 ? 1 : (g > cap ? cap : g));
}

int n2d2hip_convert(const n2d2hip_tensor* in, const n2d2hip_tensor* out, n2d2hip_stream_t stream)
{
    int rc;
    if ((rc = check_tensor(in, "convert input", true)) || (rc = check_tensor(out, "convert output", false, true)) || (rc = same_shape(in, out, "convert")))
        return rc;
    if (out->layout == N2D2HIP_S2D) {
        const int Hp = (out->H + 1) / 2 + 2 * out->halo, Wp = (out->W + 1) / 2 + 2 * out->halo;
        N2D2HIP_REQUIRE((long long)out->B * Hp * Wp * 16 < (1ll << 31), N2D2HIP_ERR_UNSUPPORTED, "convert: space-to-depth tensor too large");
        N2D2HIP_LAUNCH(to_s2d_kernel, dim3(grid_for((size_t)out->B * Hp, 4)), dim3(256), 0, (hipStream_t)stream, in->data, in->dtype, in->layout, in->cs,
                       in->halo, (signed char*)out->data, out->dtype, out->B, out->C, out->H, out->W, out->halo);
        N2D2HIP_HIP_CHECK(hipGetLastError());
        return N2D2HIP_OK;
    }
    const size_t total = (size_t)out->B * out->H * out->W * (out->layout == N2D2HIP_NHWC ? out->cs : out->C);
    EpiArgs none = {};
    N2D2HIP_LAUNCH_T(elementwise_kernel, (false), dim3(grid_for(total, 256)), dim3(256), 0, (hipStream_t)stream,
                       in->data, in->dtype, in->layout, in->cs, in->halo, out->data, out->dtype, out->layout, out->cs,
                       out->B, out->C, out->H, out->W, none);
    N2D2HIP_HIP_CHECK(hipGetLastError());
    return N2D2HIP_OK;
}

int n2d2hip_act_create(const n2d2hip_activation* desc, int nb_channels, n2d2hip_act_t* act)
{
    N2D2HIP_REQUIRE(desc && act, N2D2HIP_ERR_INVALID, "act_create: null argument");
    N2D2HIP_REQUIRE(nb_channels > 0, N2D2HIP_ERR_INVALID, "act_create: nb_channels = %d", nb_channels);
    N2D2HIP_REQUIRE(desc->kind == N2D2HIP_ACT_LINEAR || desc->kind == N2D2HIP_ACT_RECTIFIER, N2D2HIP_ERR_INVALID,
                    "act_create: bad activation kind %d", desc->kind);
    N2D2HIP_REQUIRE(desc->scaling_mode >= N2D2HIP_SCALING_NONE && desc->scaling_mode <= N2D2HIP_SCALING_DOUBLE_SHIFT,
                    N2D2HIP_ERR_INVALID, "act_create: Unsupported scaling propagation (mode %d)", desc->scaling_mode);
    // The reference rescales and saturates first and multiplies what is left below zero by the slope, in float
    // (ref: include/Activation/RectifierActivation_Frame.hpp:66-82).  Behind a rescale that saturates to an unsigned range
    // nothing is left below zero and the slope does nothing; anywhere else the products are not integers.
    N2D2HIP_REQUIRE(!(desc->kind == N2D2HIP_ACT_RECTIFIER && desc->leak_slope != 0.0f)
                        || (desc->unsigned_out && desc->scaling_mode != N2D2HIP_SCALING_NONE),
                    N2D2HIP_ERR_UNSUPPORTED,
                    "act_create: Rectifier LeakSlope %g gives non-integer outputs on a cell with signed or un-rescaled outputs; the integer "
                    "path takes it only where the rescale saturates to an unsigned range (where it changes nothing)",
                    (double)desc->leak_slope);
    const int mode = desc->scaling_mode;
    const bool relu = desc->kind == N2D2HIP_ACT_RECTIFIER;
    if (mode != N2D2HIP_SCALING_NONE) {
        N2D2HIP_REQUIRE(desc->scaling != nullptr, N2D2HIP_ERR_INVALID, "act_create: null scaling vector");
        if (mode != N2D2HIP_SCALING_FLOAT_MULT)
            N2D2HIP_REQUIRE(desc->nb_bits > 0, N2D2HIP_ERR_NOT_QUANTIZED,
                            "%s::propagate can only be used on quantized network.",
                            mode == N2D2HIP_SCALING_SINGLE_SHIFT ? "SingleShiftScaling"
                            : mode == N2D2HIP_SCALING_DOUBLE_SHIFT ? "DoubleShiftScaling" : "FixedPointScaling");
        N2D2HIP_REQUIRE(desc->nb_bits > 0, N2D2HIP_ERR_UNSUPPORTED,
                        "act_create: FloatingPointScaling on a non-quantized cell produces non-integer outputs");
        N2D2HIP_REQUIRE(desc->nb_bits <= 30, N2D2HIP_ERR_UNSUPPORTED, "act_create: nb_bits %d > 30", desc->nb_bits);
    }
    const bool clipped = desc->is_clipped && (mode == N2D2HIP_SCALING_FLOAT_MULT || mode == N2D2HIP_SCALING_FIXED_MULT16
                                              || mode == N2D2HIP_SCALING_FIXED_MULT32);   // the shift modes ignore the clip on CPU
    if (clipped)
        N2D2HIP_REQUIRE(desc->clipping != nullptr, N2D2HIP_ERR_INVALID, "act_create: is_clipped without clipping vector");

    n2d2hip_act_s* a = new n2d2hip_act_s();
    a->desc = *desc;
    a->desc.scaling = nullptr;
    a->desc.clipping = nullptr;
    a->nb_channels = nb_channels;
    a->cpad = round_up(nb_channels, 256);
    a->tables = nullptr;
    a->clipped = clipped;
    EpiArgs& e = a->args;
    e = EpiArgs();

    if (mode == N2D2HIP_SCALING_NONE) {
        e.kind = EPI_RAW;
        e.relu = relu;
        e.lo = std::numeric_limits<int>::min();
        e.hi = std::numeric_limits<int>::max();
        a->min_out = relu ? 0 : e.lo;
        a->max_out = e.hi;
        *act = a;
        return N2D2HIP_OK;
    }

    const long long L0 = desc->unsigned_out ? 0 : -(1ll << (desc->nb_bits - 1));
    const long long H = desc->unsigned_out ? (1ll << desc->nb_bits) - 1 : (1ll << (desc->nb_bits - 1)) - 1;
    const long long L = relu ? (L0 > 0 ? L0 : 0) : L0;
    e.lo = (int)L;
    e.hi = (int)H;
    a->min_out = e.lo;
    a->max_out = e.hi;

    const int cp = a->cpad;
    std::vector<int> t(5 * (size_t)cp, 0);
    int* ta = t.data();
    int* tb = ta + cp;
    int* tc = tb + cp;
    int* td = tc + cp;
    int* te = td + cp;
    const long long IMIN = std::numeric_limits<int>::min(), IMAX = std::numeric_limits<int>::max();

    if (mode == N2D2HIP_SCALING_FLOAT_MULT) {
        e.kind = EPI_F32;
        const float* sc = (const float*)desc->scaling;
        const float inf = std::numeric_limits<float>::infinity();
        for (int c = 0; c < cp; ++c) {
            const int cc = c < nb_channels ? c : nb_channels - 1;
            float lo = -inf, hi = inf;
            if (clipped) {
                const float cl = desc->clipping[cc];
                if (cl > 0.0f) { lo = 0.0f; hi = cl; } else { lo = cl; hi = 0.0f; }
            }
            memcpy(&ta[c], &lo, 4);
            memcpy(&tb[c], &hi, 4);
            memcpy(&tc[c], &sc[cc], 4);
        }
    } else {
        bool fast = true;
        for (int c = 0; c < cp; ++c) {
            const int cc = c < nb_channels ? c : nb_channels - 1;
            long long M;
            int sh;
            if (mode == N2D2HIP_SCALING_SINGLE_SHIFT) {
                M = 1;
                sh = ((const uint8_t*)desc->scaling)[cc];
            } else if (mode == N2D2HIP_SCALING_DOUBLE_SHIFT) {
                const int first = ((const uint8_t*)desc->scaling)[2 * cc];
                sh = ((const uint8_t*)desc->scaling)[2 * cc + 1];
                if (first > 30) { delete a; return fail(N2D2HIP_ERR_UNSUPPORTED, "act_create: double-shift first = %d > 30", first); }
                M = 1 + (1ll << first);
            } else {
                M = ((const int32_t*)desc->scaling)[cc];
                sh = desc->frac_bits;
            }
            if (sh < 0 || sh > 62) { delete a; return fail(N2D2HIP_ERR_UNSUPPORTED, "act_create: shift %d outside [0,62]", sh); }
            long long cmin = IMIN, cmax = IMAX;
            if (clipped) {
                // Clip(value, clip) then round(): monotone, so it acts on integers as a clamp
                // to [0, round(clip)] (clip > 0) or [round(clip), 0] (clip <= 0).
                const double cl = (double)desc->clipping[cc];
                const long long r = (long long)std::llround(cl);
                if (cl > 0.0) { cmin = 0; cmax = r; } else { cmin = r; cmax = 0; }
            }
            const __int128 half = sh > 0 ? ((__int128)1 << (sh - 1)) : 0;
            long long lo = cmin, hi = cmax;
            if (M > 0) {
                // smallest v with f(v) >= H, largest v with f(v) <= L  (f monotone non-decreasing)
                const long long vhi = clamp_ll(ceil_div(((__int128)H << sh) - half, M), IMIN, IMAX);
                const long long vlo = clamp_ll(floor_div((((__int128)L + 1) << sh) - half - 1, M), IMIN, IMAX);
                lo = clamp_ll(cmin, vlo, vhi);
                hi = clamp_ll(cmax, vlo, vhi);
            }
            ta[c] = (int)lo;
            tb[c] = (int)hi;
            tc[c] = (int)M;
            td[c] = (int)(sh > 0 && sh <= 31 ? (1ll << (sh - 1)) : 0);
            te[c] = sh;
            const long long lim24 = 1ll << 23;
            const __int128 p0 = (__int128)lo * M + half, p1 = (__int128)hi * M + half;
            const __int128 lim31 = ((__int128)1 << 31) - 1;
            if (!(M > 0 && M < lim24 && lo > -lim24 && hi < lim24 && sh <= 31 && p0 >= -lim31 && p0 <= lim31 && p1 >= -lim31 && p1 <= lim31))
                fast = false;
        }
        e.kind = fast ? EPI_I24 : EPI_I64;
    }

    a->htab = t;
    hipError_t herr = hipMalloc((void**)&a->tables, t.size() * sizeof(int));
    if (herr == hipSuccess)
        herr = hipMemcpy(a->tables, t.data(), t.size() * sizeof(int), hipMemcpyHostToDevice);
    if (herr != hipSuccess) {
        if (a->tables) (void)hipFree(a->tables);
        delete a;
        return fail(N2D2HIP_ERR_HIP, "act_create: device table upload failed: %s", hipGetErrorString(herr));
    }
    e.a = a->tables;
    e.b = a->tables + cp;
    e.c = a->tables + 2 * cp;
    e.d = a->tables + 3 * cp;
    e.e = a->tables + 4 * cp;
    *act = a;
    return N2D2HIP_OK;
}

int n2d2hip_act_destroy(n2d2hip_act_t act)
{
    if (!act) return N2D2HIP_OK;
    if (act->tables) (void)hipFree(act->tables);
    delete act;
    return N2D2HIP_OK;
}

int n2d2hip_scaling_forward(n2d2hip_act_t act, const n2d2hip_tensor* in, const n2d2hip_tensor* out, n2d2hip_stream_t stream)
{
    int rc;
    N2D2HIP_REQUIRE(act != nullptr, N2D2HIP_ERR_INVALID, "scaling_forward: null activation");
    if ((rc = check_tensor(in, "scaling input")) || (rc = check_tensor(out, "scaling output")) || (rc = same_shape(in, out, "scaling")))
        return rc;
    N2D2HIP_REQUIRE(in->C == act->nb_channels, N2D2HIP_ERR_INVALID, "scaling_forward: %d channels, activation built for %d", in->C, act->nb_channels);
    N2D2HIP_REQUIRE(in->layout == out->layout, N2D2HIP_ERR_INVALID, "scaling_forward: input and output layouts differ");
    if (is_byte_type(out->dtype)) {
        const int lo = out->dtype == N2D2HIP_I8 ? -128 : 0, hi = out->dtype == N2D2HIP_I8 ? 127 : 255;
        N2D2HIP_REQUIRE(act->min_out >= lo && act->max_out <= hi, N2D2HIP_ERR_INVALID,
                        "scaling_forward: output range [%d,%d] does not fit the output dtype", act->min_out, act->max_out);
    }
    if (in->layout == N2D2HIP_NHWC && is_byte_type(in->dtype) && in->cs == out->cs && out->dtype != N2D2HIP_F32)
        return run_scaling_nhwc(act, in, out, (hipStream_t)stream);
    const size_t total = (size_t)out->B * out->H * out->W * (out->layout == N2D2HIP_NHWC ? out->cs : out->C);
    N2D2HIP_LAUNCH_T(elementwise_kernel, (true), dim3(grid_for(total, 256)), dim3(256), 0, (hipStream_t)stream,
                       in->data, in->dtype, in->layout, in->cs, 0, out->data, out->dtype, out->layout, out->cs,
                       out->B, out->C, out->H, out->W, act->args);
    N2D2HIP_HIP_CHECK(hipGetLastError());
    return N2D2HIP_OK;
}

} // extern "C"
