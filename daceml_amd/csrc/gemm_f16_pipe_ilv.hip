// The interleaved-loop configurations of the pipelined fp16 GEMM kernel (gemm_f16_pipe.h), a translation unit of their
// own so that they compile beside the others.
#include "gemm_f16_pipe.h"

namespace dml {
namespace gemm16 {

int launch_pipelined_ilv(GemmArgs& g, const _Float16* a, const _Float16* b, void* c, const void* bias, const void* residual,
                         void* pre, int ak, int bk, int cfg, long long batch, hipStream_t st) {
    // row sums of A alongside, and K-concatenated operand pairs: on the 128 x 128 tile only, as in the plain loop
    if (g.asum || (g.groups && g.gasum[0])) {
        if (g.ksum || (cfg != 5 && cfg != 7)) {
            set_error("gemm_f16: the interleaved loop sums rows in configurations 5 and 7 only, and not over operand pairs");
            return DMLHIP_ERR_UNSUPPORTED;
        }
        if (cfg == 7) return launch_tile<128, 128, 64, 64, 2, false, true, true>(g, a, b, c, bias, residual, pre, ak, bk, batch, st);
        return launch_tile<128, 128, 64, 64, 4, false, true, true>(g, a, b, c, bias, residual, pre, ak, bk, batch, st);
    }
    if (g.ksum) {
        if (cfg != 5 && cfg != 7) {
            set_error("gemm_f16: the interleaved loop takes operand pairs in configurations 5 and 7 only");
            return DMLHIP_ERR_UNSUPPORTED;
        }
        if (cfg == 7) return launch_tile<128, 128, 64, 64, 2, true, false, true>(g, a, b, c, bias, residual, pre, ak, bk, batch, st);
        return launch_tile<128, 128, 64, 64, 4, true, false, true>(g, a, b, c, bias, residual, pre, ak, bk, batch, st);
    }
    switch (cfg) {
        case 7: return launch_tile<128, 128, 64, 64, 2, false, false, true>(g, a, b, c, bias, residual, pre, ak, bk, batch, st);
        case 4: return launch_tile<256, 256, 128, 128, 2, false, false, true>(g, a, b, c, bias, residual, pre, ak, bk, batch, st);
        case 5: return launch_tile<128, 128, 64, 64, 4, false, false, true>(g, a, b, c, bias, residual, pre, ak, bk, batch, st);
        case 6: return launch_tile<256, 128, 128, 64, 3, false, false, true>(g, a, b, c, bias, residual, pre, ak, bk, batch, st);
        case 9: return launch_tile<128, 64, 64, 32, 3, false, false, true>(g, a, b, c, bias, residual, pre, ak, bk, batch, st);
        default:
            set_error("gemm_f16: %d is not an interleaved-loop configuration", cfg);
            return DMLHIP_ERR_UNSUPPORTED;
    }
}

}  // namespace gemm16
}  // namespace dml
