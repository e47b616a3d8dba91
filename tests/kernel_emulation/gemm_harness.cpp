// Runs the pipelined fp16 GEMM kernel (daceml_amd/csrc/gemm_f16_pipe.h, compiled for the host against emu.h) on one
// problem. TEST INFRASTRUCTURE ONLY; built and driven by tests/test_kernel_emulation.py.
#include "gemm_f16_pipe.h"

#include <stdarg.h>
#include <stdio.h>

namespace dml {
void set_error(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vfprintf(stderr, fmt, ap);
    va_end(ap);
    fputc('\n', stderr);
}
int launch_status(const char*) { return 0; }

namespace gemm16 {
namespace {

alignas(16) char lds[160 * 1024];   // the array the kernel declares `extern __shared__`

struct Call {
    const _Float16 *a, *b;
    void* c;
    const void *bias, *res;
    void* pre;
    GemmArgs g;
};

template <int BM, int BN, int WM, int WN, int AK, int BKD, int NSTAGE, bool KSUM, bool ASUM, bool ILV>
void entry(void* p) {
    const Call* c = static_cast<const Call*>(p);
    gemm_f16_pipe_kernel<BM, BN, WM, WN, AK, BKD, NSTAGE, EPI_PLAIN, KSUM, ASUM, ILV>(c->a, c->b, c->c, c->bias, c->res, c->pre,
                                                                                     c->g);
}

template <int BM, int BN, int WM, int WN, int NSTAGE, bool KSUM, bool ASUM, bool ILV>
emu::kernel_fn pick(int ak, int bk) {
    if (ak == 0 && bk == 0) return entry<BM, BN, WM, WN, 0, 0, NSTAGE, KSUM, ASUM, ILV>;
#ifdef EMU_MINIMAL   // the builds that show a planted defect being found need one layout of the interleaved loop only
    return nullptr;
#else
    if (ak == 0 && bk == 1) return entry<BM, BN, WM, WN, 0, 1, NSTAGE, KSUM, ASUM, ILV>;
    if (ak == 1 && bk == 0) return entry<BM, BN, WM, WN, 1, 0, NSTAGE, KSUM, ASUM, ILV>;
    return entry<BM, BN, WM, WN, 1, 1, NSTAGE, KSUM, ASUM, ILV>;
#endif
}

template <bool KSUM, bool ASUM>
emu::kernel_fn pick_cfg(int cfg, int ak, int bk, int* bm, int* bn) {
    *bm = *bn = 128;
#ifdef EMU_MINIMAL
    if constexpr (KSUM || ASUM) return nullptr;
    else
#endif
    {
    if constexpr (!KSUM && !ASUM) {
        if (cfg == 1 || cfg == 6) { *bm = 256; }
        if (cfg == 2 || cfg == 4) { *bm = 256; *bn = 256; }
        if (cfg == 8 || cfg == 9) { *bn = 64; }
        switch (cfg) {
#ifndef EMU_MINIMAL
            case 1: return pick<256, 128, 128, 64, 3, false, false, false>(ak, bk);
            case 2: return pick<256, 256, 128, 128, 2, false, false, false>(ak, bk);
#endif
            case 4: return pick<256, 256, 128, 128, 2, false, false, true>(ak, bk);
            case 6: return pick<256, 128, 128, 64, 3, false, false, true>(ak, bk);
#ifndef EMU_MINIMAL
            case 8: return pick<128, 64, 64, 32, 3, false, false, false>(ak, bk);
            case 9: return pick<128, 64, 64, 32, 3, false, false, true>(ak, bk);
#endif
            default: break;
        }
    }
    switch (cfg) {
#ifndef EMU_MINIMAL
        case 0: return pick<128, 128, 64, 64, 4, KSUM, ASUM, false>(ak, bk);
        case 3: return pick<128, 128, 64, 64, 2, KSUM, ASUM, false>(ak, bk);
#endif
        case 5: return pick<128, 128, 64, 64, 4, KSUM, ASUM, true>(ak, bk);
        case 7: return pick<128, 128, 64, 64, 2, KSUM, ASUM, true>(ak, bk);
        default: return nullptr;
    }
    }
}

}  // namespace
}  // namespace gemm16
}  // namespace dml

using namespace dml::gemm16;

// C[m, n] (fp32, dense) = sum over `pairs` operand pairs of A_i B_i. akind / bkind: 0 = the operand is stored with K
// contiguous ([rows][k]), 1 = with its rows contiguous ([k][rows]). variant: 0 plain (pairs = 1), 1 K-concatenated
// pairs, 2 plain with row sums of A into asum[m] (fp32). Returns 0, 1 on a deadlock, 2 for a combination the kernel
// does not have.
extern "C" int emu_gemm(int cfg, int variant, int akind, int bkind, int m, int n, int k, int pairs, const void* const* a,
                        const void* const* b, float* c, float* asum, unsigned seed, int late_dma) {
    Call call = {};
    GemmArgs& g = call.g;
    g.m = m; g.n = n; g.k = k;
    g.sam = akind ? 1 : k; g.sak = akind ? m : 1;
    g.sbn = bkind ? 1 : k; g.sbk = bkind ? n : 1;
    g.scm = n;
    g.batch1 = g.batch2 = 1;
    g.alpha = 1.f; g.beta = 0.f;
    g.out_f32 = 1; g.c_vec = n % 8 == 0;
    int bm, bn;
    emu::kernel_fn fn = variant == 1 ? pick_cfg<true, false>(cfg, akind, bkind, &bm, &bn)
                      : variant == 2 ? pick_cfg<false, true>(cfg, akind, bkind, &bm, &bn)
                                     : pick_cfg<false, false>(cfg, akind, bkind, &bm, &bn);
    if (!fn || pairs < 1 || pairs > DMLHIP_GROUP_MAX || (variant != 1 && pairs != 1) || k % BK) return 2;
    g.tiles_m = (m + bm - 1) / bm;
    g.tiles_n = (n + bn - 1) / bn;
    g.total_blocks = (long long)g.tiles_m * g.tiles_n;
    call.a = (const _Float16*)a[0];
    call.b = (const _Float16*)b[0];
    call.c = c;
    if (variant == 1) {
        g.ksum = 1;
        g.groups = pairs;
        for (int i = 0; i < pairs; ++i) { g.ga[i] = (const _Float16*)a[i]; g.gb[i] = (const _Float16*)b[i]; }
    }
    if (variant == 2) { g.asum = asum; g.asum_f32 = 1; }
    return emu::run_grid(fn, &call, (unsigned)g.total_blocks, kThreads, seed, late_dma, lds);
}
