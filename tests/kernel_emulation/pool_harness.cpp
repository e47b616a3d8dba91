// Runs the MaxPool kernels (daceml_amd/csrc/pool.hip, compiled for the host against emu.h) through their own host
// functions. TEST INFRASTRUCTURE ONLY; built and driven by tests/test_kernel_emulation.py.
#include <stdarg.h>
#include <stdio.h>

#include "emu.h"

namespace {
struct Launch {
    const float *x, *dy;
    float* out;
    int64_t n;
    unsigned grid;
    char args[128];
    bool backward, set;
} g_launch;
alignas(16) char lds[160 * 1024];

// the two launches differ in their argument count: record either (element type as the template instantiates it;
// only the fp32 instantiations are run)
template <typename K, typename P, typename A>
void record(K, unsigned grid, const P* x, P* y, int64_t n, const A& a) {
    static_assert(sizeof(A) <= sizeof(g_launch.args), "args");
    g_launch = Launch();
    g_launch.x = (const float*)x; g_launch.out = (float*)y; g_launch.n = n; g_launch.grid = grid;
    g_launch.backward = false; g_launch.set = true;
    memcpy(g_launch.args, &a, sizeof(A));
}
template <typename K, typename P, typename A>
void record(K, unsigned grid, const P* x, const P* dy, P* dx, int64_t n, const A& a) {
    static_assert(sizeof(A) <= sizeof(g_launch.args), "args");
    g_launch = Launch();
    g_launch.x = (const float*)x; g_launch.dy = (const float*)dy; g_launch.out = (float*)dx; g_launch.n = n;
    g_launch.grid = grid; g_launch.backward = true; g_launch.set = true;
    memcpy(g_launch.args, &a, sizeof(A));
}
}  // namespace

#undef hipLaunchKernelGGL
#define hipLaunchKernelGGL(kern, grid_, block_, lds_, stream_, ...) record(0, grid_, __VA_ARGS__)

#include "pool_emu.h"

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
    PoolArgs a;
    memcpy(&a, g_launch.args, sizeof(a));
    if (g_launch.backward) maxpool2d_bwd_kernel<float>(g_launch.x, g_launch.dy, g_launch.out, g_launch.n, a);
    else maxpool2d_kernel<float>(g_launch.x, g_launch.out, g_launch.n, a);
}
}  // namespace
}  // namespace dml

// fp32 (the kernels are the same templates for fp16). dy == NULL: forward into `out`; else backward into `out`.
// Returns the host function's status, or 100 + the scheduler's.
extern "C" int emu_maxpool(const float* x, const float* dy, float* out, int64_t planes, int64_t h, int64_t w, int64_t kh,
                           int64_t kw, int64_t sh, int64_t sw, unsigned seed) {
    g_launch.set = false;
    const int status = dy ? dmlhip_maxpool2d_backward_f32(x, dy, out, planes, h, w, kh, kw, sh, sw, nullptr)
                          : dmlhip_maxpool2d_f32(x, out, planes, h, w, kh, kw, sh, sw, nullptr);
    if (status != 0 || !g_launch.set) return status;
    const int r = emu::run_grid(dml::run, nullptr, g_launch.grid, 256, seed, 0, lds);
    return r ? 100 + r : 0;
}
