"""The interleaved-K-loop configurations of the pipelined fp16 GEMM kernel (4: 256 x 256 tile, 5: 128 x 128 with a
four-stage ring, 6: 256 x 128, 7: 128 x 128 with two stages, 9: 128 x 64 - and 8, the plain loop on that tile), each
pinned through ``dmlhip_debug_force_gemm_config`` (the library chooses 4, 5 and 9 by itself for products with at least
eight K steps) on the cases the other configurations are tested with, plus products with enough K steps to run the ring's steady state, its tail and every operand layout."""
import numpy as np
import pytest
import torch

from oracle import ops as O
from tests import test_gpu_kernels as TK
from tests.util import assert_close, dev, host

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("cfg", [4, 5, 6, 7, 8, 9])
@pytest.mark.parametrize("eq,sa,sb", TK.GEMM_CASES)
def test_einsum_f16_interleaved(cfg, eq, sa, sb):
    TK.test_einsum_f16(cfg, eq, sa, sb)


#: K = 64 .. 1536: 1 to 24 K steps (fewer than the ring is deep, exactly as deep, and many more), every pair of operand
#: layouts, ragged M and N, batches
LONG_K_CASES = [
    ("aik,jk->aij", (2, 256, 1024), (384, 1024)),      # both K-contiguous
    ("aik,kj->aij", (1, 512, 1024), (1024, 640)),      # B row-contiguous
    ("aij,aik->jk", (4, 384, 256), (4, 384, 200)),     # both row-contiguous, K = 1536
    ("ki,jk->ij", (512, 300), (260, 512)),             # A row-contiguous, B K-contiguous
    ("aik,jk->aij", (1, 130, 64), (70, 64)),           # a single K step
    ("aik,jk->aij", (1, 130, 192), (70, 192)),         # three K steps: as many as the deepest ring looks ahead
    ("aik,jk->aij", (1, 130, 256), (70, 256)),         # four
    ("baik,bakj->baij", (2, 3, 200, 320), (2, 3, 320, 136)),
]


@pytest.mark.parametrize("cfg", [4, 5, 6, 7, 8, 9])
@pytest.mark.parametrize("eq,sa,sb", LONG_K_CASES)
def test_long_products_interleaved(cfg, eq, sa, sb):
    from daceml_amd import kernels as K
    a, a64 = TK._inputs(600, sa, torch.float16)
    b, b64 = TK._inputs(601, sb, torch.float16, 0.2)
    want = O.einsum(eq, a64, b64)
    TK._set_cfg(-1)
    base = K.einsum(eq, dev(a), dev(b), out_dtype=torch.float32)
    TK._set_cfg(cfg)
    got = K.einsum(eq, dev(a), dev(b), out_dtype=torch.float32)
    got16 = K.einsum(eq, dev(a), dev(b))
    TK._set_cfg(-1)
    kdim = a.size * b.size // max(want.size, 1)
    assert_close(host(got), want, torch.float32, "einsum %s cfg=%d" % (eq, cfg), rtol=1e-4, atol=2e-4 * max(1.0, np.sqrt(kdim / 256)))
    assert_close(host(got16), want, torch.float16, "einsum %s cfg=%d fp16 out" % (eq, cfg))
    # same MFMA sequence per accumulator as the plain loop: the fp32 results agree to the last bit
    assert torch.equal(got, base)


@pytest.mark.parametrize("cfg", [4, 5, 6, 7, 8, 9])
def test_epilogues_interleaved(cfg):
    TK._set_cfg(cfg)
    TK.test_gemm_f16_epilogue()
    TK._set_cfg(cfg)
    TK.test_gemm_f16_config_shapes()


def test_grouped_summed_and_row_sum_products_interleaved():
    """Configurations 5 and 7 also carry the K-concatenated and the row-sum forms."""
    for cfg in (5, 7):
        _grouped_forms(cfg)


def _grouped_forms(cfg):
    for case in [("aik,jk->aij", (2, 256, 128), (192, 128), True, torch.float16),
                 ("aij,jk->aik", (2, 128, 192), (192, 256), False, torch.float16),
                 ("aij,aik->jk", (2, 256, 128), (2, 256, 64), False, torch.float32)]:
        TK._set_cfg(cfg)
        TK._einsum_grouped_case(*case)
    for case in [("aij,jk->aik", (2, 256, 128), (128, 192), 3, True, torch.float16, True),
                 ("aik,jk->aij", (2, 128, 256), (128, 256), 4, True, torch.float16, True),
                 ("aij,aik->jk", (2, 256, 128), (2, 256, 64), 3, False, torch.float32, True)]:
        TK._set_cfg(cfg)
        TK.test_einsum_sum(*case)
    for case in [((2, 256, 128), (2, 256, 64), 1, torch.float32, True), ((2, 256, 256), (2, 256, 128), 3, torch.float32, True),
                 ((4, 128, 384), (4, 128, 192), 4, torch.float16, True), ((2, 256, 200), (2, 256, 72), 2, torch.float32, True)]:
        TK._set_cfg(cfg)
        TK.test_einsum_grouped_asum(*case)
    TK._set_cfg(-1)
