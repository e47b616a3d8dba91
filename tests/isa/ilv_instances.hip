// A few instantiations of the pipelined GEMM kernel's interleaved K loop, compiled to assembly by
// tests/test_isa_hazards.py (never linked, never run): one per tile configuration and operand-layout pair, plain
// epilogue. The full set lives in daceml_amd/csrc/gemm_f16_pipe_ilv.hip and takes minutes to compile.
#include "../../daceml_amd/csrc/gemm_f16_pipe.h"

namespace dml {
namespace gemm16 {

#define ILV_KERNELS(BM, BN, WM, WN, NSTAGE)                                                         \
    (const void*)gemm_f16_pipe_kernel<BM, BN, WM, WN, 0, 0, NSTAGE, EPI_PLAIN, false, false, true>, \
    (const void*)gemm_f16_pipe_kernel<BM, BN, WM, WN, 0, 1, NSTAGE, EPI_PLAIN, false, false, true>, \
    (const void*)gemm_f16_pipe_kernel<BM, BN, WM, WN, 1, 0, NSTAGE, EPI_PLAIN, false, false, true>, \
    (const void*)gemm_f16_pipe_kernel<BM, BN, WM, WN, 1, 1, NSTAGE, EPI_PLAIN, false, false, true>

const void* isa_check_kernels[] = {ILV_KERNELS(256, 256, 128, 128, 2), ILV_KERNELS(128, 128, 64, 64, 4),
                                   ILV_KERNELS(256, 128, 128, 64, 3)};

}  // namespace gemm16
}  // namespace dml
