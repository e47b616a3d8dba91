// The pipelined fp16 GEMM kernel (gemm_f16_pipe.h) in the tile configurations the library chooses from, and its
// K-concatenated and row-sum variants. The interleaved-loop configurations are compiled in gemm_f16_pipe_ilv.hip.
#include "gemm_f16_pipe.h"

namespace dml {
namespace gemm16 {

int launch_pipelined(GemmArgs& g, const _Float16* a, const _Float16* b, void* c, const void* bias, const void* residual,
                     void* pre, int amode, int bmode, int cfg, long long batch, hipStream_t st) {
    const int ak = amode == 4 ? 1 : 0, bk = bmode == 4 ? 1 : 0;
    // 4 - 7: the interleaved K loop on the tiles of 2, 0, 1 and 3 (5 and 7 also with row sums or operand pairs); 9: on
    // the 128 x 64 tile of 8. A forced 4, 6, 8 or 9 leaves the row-sum and operand-pair products on the plain loop of the
    // 128 x 128 tile.
    if (cfg == 5 || cfg == 7 || ((cfg == 4 || cfg == 6 || cfg == 9) && !g.ksum && !g.asum && !(g.groups && g.gasum[0])))
        return launch_pipelined_ilv(g, a, b, c, bias, residual, pre, ak, bk, cfg, batch, st);
    if (g.asum || (g.groups && g.gasum[0])) {  // row sums of A alongside: the two 128x128 configurations only
        if (g.ksum) {
            set_error("gemm_f16: row sums are not combined with K-concatenated operand pairs");
            return DMLHIP_ERR_UNSUPPORTED;
        }
        if (cfg == 3) return launch_tile<128, 128, 64, 64, 2, false, true>(g, a, b, c, bias, residual, pre, ak, bk, batch, st);
        return launch_tile<128, 128, 64, 64, 4, false, true>(g, a, b, c, bias, residual, pre, ak, bk, batch, st);
    }
    if (g.ksum) {  // K-concatenated operand pairs: the two 128x128 configurations only
        if (cfg == 3) return launch_tile<128, 128, 64, 64, 2, true>(g, a, b, c, bias, residual, pre, ak, bk, batch, st);
        return launch_tile<128, 128, 64, 64, 4, true>(g, a, b, c, bias, residual, pre, ak, bk, batch, st);
    }
    switch (cfg) {
        case 2: return launch_tile<256, 256, 128, 128, 2>(g, a, b, c, bias, residual, pre, ak, bk, batch, st);
        case 1: return launch_tile<256, 128, 128, 64, 3>(g, a, b, c, bias, residual, pre, ak, bk, batch, st);
        case 3: return launch_tile<128, 128, 64, 64, 2>(g, a, b, c, bias, residual, pre, ak, bk, batch, st);
        // 128 x 64 tile, three stages (72 KB: two workgroups per compute unit): twice the workgroups of the 128 x 128 tile
        // for products that otherwise give each compute unit a single tile.
        case 8: return launch_tile<128, 64, 64, 32, 3>(g, a, b, c, bias, residual, pre, ak, bk, batch, st);
        default: return launch_tile<128, 128, 64, 64, 4>(g, a, b, c, bias, residual, pre, ak, bk, batch, st);
    }
}

}  // namespace gemm16
}  // namespace dml
