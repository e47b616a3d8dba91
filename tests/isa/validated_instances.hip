// The instantiations of the pipelined GEMM kernel that one step of the benchmarked BERT layer launches (the fused expand +
// depthwise kernels and the attention kernels are taken from their own source files), compiled to assembly by
// tests/test_validated_kernels.py (never linked, never run) and compared with the instruction digests recorded when
// these kernels last passed their tests on the GPU.
#include "../../daceml_amd/csrc/gemm_f16_pipe.h"

namespace dml {
namespace gemm16 {

const void* validated_gemm_kernels[] = {
    // BM, BN, WM, WN, A kind, B kind, stages, epilogue, K-concatenated pairs, row sums, interleaved loop
    (const void*)gemm_f16_pipe_kernel<128, 128, 64, 64, 1, 1, 4, EPI_PLAIN, false, true, true>,      // weight + bias gradients
    (const void*)gemm_f16_pipe_kernel<128, 128, 64, 64, 0, 0, 4, EPI_PLAIN, false, false, true>,     // q/k/v projections (grouped)
    (const void*)gemm_f16_pipe_kernel<128, 128, 64, 64, 0, 0, 4, EPI_GENERAL, false, false, true>,   // o and FFN2 with residual
    (const void*)gemm_f16_pipe_kernel<256, 256, 128, 128, 0, 0, 2, EPI_PLAIN, false, false, true>,   // FFN1
    (const void*)gemm_f16_pipe_kernel<256, 256, 128, 128, 0, 1, 2, EPI_PLAIN, false, false, true>,   // FFN2 input gradient
    (const void*)gemm_f16_pipe_kernel<128, 128, 64, 64, 0, 1, 4, EPI_GENERAL, false, false, true>,   // FFN1 input gradient
    (const void*)gemm_f16_pipe_kernel<128, 128, 64, 64, 0, 1, 4, EPI_GENERAL, true, false, true>,    // q/k/v input gradients summed
    (const void*)gemm_f16_pipe_kernel<128, 128, 64, 64, 0, 1, 4, EPI_PLAIN, false, false, true>,     // o input gradient
    (const void*)gemm_f16_pipe_kernel<128, 64, 64, 32, 0, 0, 3, EPI_PLAIN, false, false, true>};     // few tiles, long K

}  // namespace gemm16
}  // namespace dml
