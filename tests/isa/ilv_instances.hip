// A few instantiations of the pipelined GEMM kernel's interleaved K loop, compiled to assembly by
// tests/test_isa_hazards.py (never linked, never run): one per tile configuration and operand-layout pair, plain
// epilogue. The full set lives in daceml_amd/csrc/gemm_f16_pipe_ilv.hip and takes minutes to compile.
#include "../../daceml_amd/csrc/gemm_f16_pipe.h"

namespace dml {
namespace gemm16 {

#define ILV_KERNELS(BM, BN, WM, WN, NSTAGE, KSUM, ASUM)                                           \
    (const void*)gemm_f16_pipe_kernel<BM, BN, WM, WN, 0, 0, NSTAGE, EPI_PLAIN, KSUM, ASUM, true>, \
    (const void*)gemm_f16_pipe_kernel<BM, BN, WM, WN, 0, 1, NSTAGE, EPI_PLAIN, KSUM, ASUM, true>, \
    (const void*)gemm_f16_pipe_kernel<BM, BN, WM, WN, 1, 0, NSTAGE, EPI_PLAIN, KSUM, ASUM, true>, \
    (const void*)gemm_f16_pipe_kernel<BM, BN, WM, WN, 1, 1, NSTAGE, EPI_PLAIN, KSUM, ASUM, true>

const void* isa_check_kernels[] = {
    ILV_KERNELS(256, 256, 128, 128, 2, false, false), ILV_KERNELS(128, 128, 64, 64, 4, false, false),
    ILV_KERNELS(256, 128, 128, 64, 3, false, false),
    ILV_KERNELS(128, 128, 64, 64, 2, false, false), ILV_KERNELS(128, 64, 64, 32, 3, false, false),
    ILV_KERNELS(128, 128, 64, 64, 4, true, false),   // K-concatenated operand pairs
    ILV_KERNELS(128, 128, 64, 64, 4, false, true)};  // row sums of A alongside

}  // namespace gemm16
}  // namespace dml
