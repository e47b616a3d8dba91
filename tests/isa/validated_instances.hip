// The instantiations of the pipelined GEMM kernel that one step of the benchmarked BERT layer launches, and the fused
// expand + depthwise strip kernel of the benchmarked MBConv block, compiled to assembly by
// tests/test_validated_kernels.py (never linked, never run) and compared with the instruction digests recorded when
// these kernels last passed their tests on the GPU.
#include "../../daceml_amd/csrc/gemm_f16_pipe.h"

namespace dml {
namespace gemm16 {

const void* validated_gemm_kernels[] = {
    (const void*)gemm_f16_pipe_kernel<128, 128, 64, 64, 1, 1, 4, EPI_PLAIN, false, true>,    // weight + bias gradients
    (const void*)gemm_f16_pipe_kernel<128, 128, 64, 64, 0, 0, 2, EPI_PLAIN, false, false>,   // the two FFN products
    (const void*)gemm_f16_pipe_kernel<128, 128, 64, 64, 0, 0, 4, EPI_GENERAL, false, false>, // q/k/v and o projections
    (const void*)gemm_f16_pipe_kernel<128, 128, 64, 64, 0, 1, 4, EPI_GENERAL, false, false>, // FFN1 input gradient
    (const void*)gemm_f16_pipe_kernel<128, 128, 64, 64, 0, 1, 2, EPI_PLAIN, false, false>,   // FFN2 input gradient
    (const void*)gemm_f16_pipe_kernel<128, 128, 64, 64, 0, 1, 4, EPI_GENERAL, true, false>,  // q/k/v input gradients summed
    (const void*)gemm_f16_pipe_kernel<128, 128, 64, 64, 0, 1, 4, EPI_PLAIN, false, false>,   // o input gradient
    (const void*)gemm_f16_pipe_kernel<256, 256, 128, 128, 0, 0, 2, EPI_PLAIN, false, false>,
    (const void*)gemm_f16_pipe_kernel<256, 128, 128, 64, 1, 0, 3, EPI_PLAIN, false, false>};

}  // namespace gemm16
}  // namespace dml
