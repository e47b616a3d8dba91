// Runs the fused pointwise + depthwise convolution kernels (daceml_amd/csrc/conv_fused.hip, compiled for the host
// against emu.h) on one problem. TEST INFRASTRUCTURE ONLY; built and driven by tests/test_kernel_emulation.py.
#include <stdarg.h>
#include <stdio.h>

namespace dml {
namespace {
alignas(16) float lds_f[160 * 1024 / 4];
}
}  // namespace dml

#include "conv_fused_emu.h"

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

struct Call {
    const float *x, *we, *be, *wd, *bd;
    float* y;
    FusedArgs strip;
    RollArgs roll;
};

template <int A1, int A2> void strips(void* p) {
    const Call* c = static_cast<const Call*>(p);
    expand_depthwise_kernel<A1, A2>(c->x, c->we, c->be, c->wd, c->bd, c->y, c->strip);
}
template <int A1, int A2, int STRIDE, int WAVES> void rolling(void* p) {
    const Call* c = static_cast<const Call*>(p);
    expand_depthwise_rolling_kernel<A1, A2, STRIDE, WAVES>(c->x, c->we, c->be, c->wd, c->bd, c->y, c->roll);
}

template <int A1, int A2> emu::kernel_fn pick_rolling(int stride, int waves) {
    if (stride == 1) return waves == 16 ? rolling<A1, A2, 1, 16> : rolling<A1, A2, 1, 8>;
    return waves == 16 ? rolling<A1, A2, 2, 16> : rolling<A1, A2, 2, 8>;
}

}  // namespace
}  // namespace dml

using namespace dml;

// mode 0: the strip kernel with `rows` output rows per strip; mode 1: the rolling-window kernel with at most `rows`
// output rows per batch (0: the most that fit) and `waves` wavefronts per workgroup, its workgroups spread as for `cus`
// compute units. acts: 0 = none / none, 1 = swish / swish, 2 = relu / none. geometry (optional) receives
// {rows per batch, ring rows, rows per segment, segments}. Returns 0, 1 on a deadlock, negative when the geometry
// does not fit.
extern "C" int emu_expand_depthwise(int mode, int rows, int waves, int cus, int acts, int n, int cin, int cmid, int h,
                                    int w, int stride, const float* x, const float* we, const float* be,
                                    const float* wd, const float* bd, float* y, unsigned seed, int* geometry) {
    Call c = {};
    c.x = x; c.we = we; c.be = be; c.wd = wd; c.bd = bd; c.y = y;
    if (cin % 16 || cmid % kCB || (stride != 1 && stride != 2)) return -1;
    emu::kernel_fn fn;
    unsigned blocks, threads;
    if (mode == 0) {
        FusedArgs& a = c.strip;
        a.n = n; a.cin = cin; a.cmid = cmid; a.h = h; a.w = w; a.stride = stride;
        a.oh = (h + 2 - 3) / stride + 1;
        a.ow = (w + 2 - 3) / stride + 1;
        a.toh = rows < a.oh ? rows : a.oh;
        a.ih = (a.toh - 1) * stride + 3;
        a.wp = w + 2;
        a.strips = (a.oh + a.toh - 1) / a.toh;
        a.cblocks = cmid / kCB;
        if (fused_lds_bytes(a.toh, stride, w, cin) > 156 * 1024) return -2;
        blocks = (unsigned)(n * a.strips * a.cblocks);
        threads = kFusedThreads;
        fn = acts == 1 ? strips<DMLHIP_ACT_SWISH, DMLHIP_ACT_SWISH>
           : acts == 2 ? strips<DMLHIP_ACT_RELU, DMLHIP_ACT_NONE> : strips<DMLHIP_ACT_NONE, DMLHIP_ACT_NONE>;
    } else {
        if (!fill_rolling(n, cin, cmid, h, w, stride, rows, cus, c.roll)) return -2;
        if (geometry) {
            geometry[0] = c.roll.r; geometry[1] = c.roll.ring; geometry[2] = c.roll.seg_rows; geometry[3] = c.roll.segs;
        }
        blocks = c.roll.total;
        threads = (unsigned)(waves == 16 ? 16 : 8) * 64;
        fn = acts == 1 ? pick_rolling<DMLHIP_ACT_SWISH, DMLHIP_ACT_SWISH>(stride, waves)
           : acts == 2 ? pick_rolling<DMLHIP_ACT_RELU, DMLHIP_ACT_NONE>(stride, waves)
                       : pick_rolling<DMLHIP_ACT_NONE, DMLHIP_ACT_NONE>(stride, waves);
    }
    return emu::run_grid(fn, &c, blocks, threads, seed, 0, (char*)lds_f);
}
