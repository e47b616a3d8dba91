// Runs the constant-pad kernel (daceml_amd/csrc/pad.hip, compiled for the host against emu.h) through its own host
// function. TEST INFRASTRUCTURE ONLY; built and driven by tests/test_kernel_emulation.py.
#include <stdarg.h>
#include <stdio.h>

#include "emu.h"

// the host function launches through this: record the launch and run it after the host function returns
namespace {
struct Launch {
    const float* x;
    float* y;
    int64_t n;
    unsigned grid;
    float value;
    char dims[512];
    bool set;
} g_launch;
alignas(16) char lds[160 * 1024];
}  // namespace

#undef hipLaunchKernelGGL
#define hipLaunchKernelGGL(kern, grid_, block_, lds_, stream_, x_, y_, n_, d_, value_)                      \
    do {                                                                                                  \
        static_assert(sizeof(d_) <= sizeof(g_launch.dims), "dims");                                       \
        g_launch.x = (const float*)(x_); g_launch.y = (float*)(y_); g_launch.n = (n_); g_launch.grid = (grid_); \
        g_launch.value = (value_); memcpy(g_launch.dims, &(d_), sizeof(d_)); g_launch.set = true;         \
    } while (0)

#include "pad_emu.h"

namespace dml {
void set_error(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vfprintf(stderr, fmt, ap);
    va_end(ap);
    fputc('\n', stderr);
}
int launch_status(const char*) { return 0; }
namespace {
void run(void*) {
    PadDims d;
    memcpy(&d, g_launch.dims, sizeof(d));
    pad_constant_kernel<float>(g_launch.x, g_launch.y, g_launch.n, d, g_launch.value);
}
}  // namespace
}  // namespace dml

// fp32 only (the kernel is the same template for fp16). Returns the host function's status, or 100 + the scheduler's.
extern "C" int emu_pad(const float* x, float* y, int ndim, const int64_t* shape, const int64_t* begin, const int64_t* end,
                       float value, unsigned seed) {
    g_launch.set = false;
    const int status = dmlhip_pad_constant_f32(x, y, ndim, shape, begin, end, value, nullptr);
    if (status != 0 || !g_launch.set) return status;
    const int r = emu::run_grid(dml::run, nullptr, g_launch.grid, 256, seed, 0, lds);
    return r ? 100 + r : 0;
}
