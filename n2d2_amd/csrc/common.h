// Internal definitions shared by the HIP translation units of libn2d2hip.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <string>
#include <type_traits>
#include <vector>

#include "n2d2hip.h"

namespace n2d2hip {

// Records the message returned by n2d2hip_last_error() and returns `code`.
int fail(int code, const char* fmt, ...) __attribute__((format(printf, 2, 3)));

#define N2D2HIP_HIP_CHECK(expr)                                                            \
    do {                                                                                   \
        hipError_t e__ = (expr);                                                           \
        if (e__ != hipSuccess)                                                             \
            return ::n2d2hip::fail(N2D2HIP_ERR_HIP, "%s failed: %s (%s:%d)", #expr,      \
                                   hipGetErrorString(e__), __FILE__, __LINE__);            \
    } while (0)

#define N2D2HIP_REQUIRE(cond, code, ...)                                                   \
    do {                                                                                   \
        if (!(cond))                                                                       \
            return ::n2d2hip::fail(code, __VA_ARGS__);                                    \
    } while (0)

inline int elem_size(int dtype)
{
    return (dtype == N2D2HIP_I32 || dtype == N2D2HIP_F32) ? 4 : 1;
}
inline bool is_byte_type(int dtype)
{
    return dtype == N2D2HIP_U8 || dtype == N2D2HIP_I8 || dtype == N2D2HIP_U8B;
}
// Value added to a stored byte to obtain the logical value.
inline int zero_point(int dtype)
{
    return dtype == N2D2HIP_U8B ? 128 : 0;
}
inline int round_up(int x, int m)
{
    return (x + m - 1) / m * m;
}
int check_tensor(const n2d2hip_tensor* t, const char* what, bool halo_ok = false, bool s2d_ok = false);

// ---------------------------------------------------------------- launches
// The kernels of the integer path are launched through launch_kernel<&kernel>(), so that the launch log
// (n2d2hip_launch_log_*) can name what a call launched, template arguments included, and its grid.
// __PRETTY_FUNCTION__ of this function carries the kernel's full name ("... [K = &n2d2hip::kernel<1, 2>]").
template <auto K>
const char* kernel_pretty()
{
    return __PRETTY_FUNCTION__;
}
// Adds a launch to the calling thread's log when one is open; `slot` is the launch's first probe record or -1.
void launch_log_add(const char* pretty, unsigned grid, unsigned block, long long slot);
#ifdef N2D2HIP_PROFILE
// Probe builds: records (8 counters each) for the blocks of the next launch inside the buffer given to
// n2d2hip_probe_begin(); null when there is none or it is full.  *first is the index of the first record.
long long* probe_take(unsigned blocks, long long* first);
template <class T>
auto set_probe(T& a, long long* p, int) -> decltype(a.prof = p, void())
{
    a.prof = p;
}
template <class T>
void set_probe(T&, long long*, long)
{
}
#endif

template <auto K, class A0, class... A>
void launch_kernel(const char* name, dim3 grid, dim3 block, unsigned lds, hipStream_t stream, A0 a0, A... a)
{
    long long slot = -1;
#ifdef N2D2HIP_PROFILE
    set_probe(a0, probe_take(grid.x * grid.y * grid.z, &slot), 0);
#endif
    launch_log_add(name ? name : kernel_pretty<K>(), grid.x * grid.y * grid.z, block.x * block.y * block.z, slot);
    hipLaunchKernelGGL(K, grid, block, lds, stream, a0, a...);
}
// "<4, 128, true>": the values of a kernel's template arguments, for its name in the launch log
inline void targ_text(std::string& s, bool v) { s += v ? "true" : "false"; }
inline void targ_text(std::string& s, long long v) { s += std::to_string(v); }
template <auto K, auto... V>
const char* targs_of(const char* kernel)
{
    static const std::string text = [kernel] {
        std::string s = std::string(kernel) + "<";
        bool first = true;
        ((s += first ? "" : ", ", first = false,
          targ_text(s, static_cast<std::conditional_t<std::is_same<decltype(V), bool>::value, bool, long long>>(V))), ...);
        return s + ">";
    }();
    return text.c_str();
}
#define N2D2HIP_UNPAREN(...) __VA_ARGS__
// N2D2HIP_LAUNCH(kernel, ...): a kernel without template arguments (or whose arguments need not show in the log);
// N2D2HIP_LAUNCH_T(kernel, (template arguments), ...): the log names the kernel with the arguments' values.
#define N2D2HIP_LAUNCH(K, grid, block, lds, stream, ...) ::n2d2hip::launch_kernel<&K>(nullptr, grid, block, lds, stream, __VA_ARGS__)
#define N2D2HIP_LAUNCH_T(K, TARGS, grid, block, lds, stream, ...)                                              \
    ::n2d2hip::launch_kernel<&K<N2D2HIP_UNPAREN TARGS>>(::n2d2hip::targs_of<&K<N2D2HIP_UNPAREN TARGS>, N2D2HIP_UNPAREN TARGS>(#K), grid, block, lds, stream, __VA_ARGS__)

// ---------------------------------------------------------------- epilogue
// Device-side form of "Scaling::propagate, saturate, Rectifier/Linear" for one
// cell.  Per-channel tables live in one device allocation of 5 int arrays of
// `cpad` entries each (channels >= C replicate neutral values).
enum EpiKind {
    EPI_RAW = 0, // ScalingMode NONE: value passes through (ReLU if rectifier)
    EPI_I24 = 1, // integer rescale, every intermediate fits 32 bits (24-bit multiply)
    EPI_I64 = 2, // integer rescale with a 64-bit product
    EPI_F32 = 3  // FloatingPointScaling: float32 multiply, round half away
};

struct EpiArgs {
    int kind;
    int lo, hi;        // saturation range with the ReLU folded in
    int relu;          // EPI_RAW only
    const int* a;      // I24/I64: pre-clamp low  | F32: clip low  (float bits)
    const int* b;      // I24/I64: pre-clamp high | F32: clip high (float bits)
    const int* c;      // I24/I64: multiplier     | F32: scale     (float bits)
    const int* d;      // I24: rounding half (int32)
    const int* e;      // I24/I64: right shift
};

} // namespace n2d2hip

struct n2d2hip_act_s;
namespace n2d2hip {
// Fast path of the stand-alone Scaling for NHWC byte inputs (bandwidth.hip).
int run_scaling_nhwc(const n2d2hip_act_s* act, const n2d2hip_tensor* in, const n2d2hip_tensor* out, hipStream_t stream);
}

struct n2d2hip_act_s {
    n2d2hip_activation desc;   // pointers inside are NOT kept valid; do not dereference
    int nb_channels;
    int cpad;
    int* tables;               // device, 5 * cpad ints
    n2d2hip::EpiArgs args;
    int min_out, max_out;      // range of produced values (for dtype checks); RAW: INT range
    std::vector<int> htab;     // host copy of the tables (empty for RAW)
    bool clipped;              // the Scaling applies a Clip
};

struct n2d2hip_elemwise_s {
    int nb_inputs, nb_channels, cpad;
    n2d2hip_act_t act;
    float* d_coeff;     // w then s, each [nb_inputs][cpad]
    bool unit_coeff;    // every weight 1 and every shift 0
    int pre_input;      // input carrying a folded ScalingCell (-1: none)
    n2d2hip_act_t pre_act;
};
