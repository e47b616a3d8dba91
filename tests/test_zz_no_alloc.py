"""The entry point that allocates nothing: dmlhip_layernorm_backward_noalloc_f16 keeps its partial sums in a fixed
device array inside the library instead of a caller-provided workspace. Its results must equal those of
dmlhip_layernorm_backward_f16 bit for bit (same kernels, same summation order), also on a second call with a smaller
input that reuses the array while it still holds the first call's partial sums."""
import ctypes

import numpy as np
import pytest
import torch

from oracle import ops as O
from tests.util import assert_close, host, rng

pytestmark = pytest.mark.gpu


def _case(lib, rows, cols, seed):
    r = rng(seed)
    x = torch.from_numpy(r.standard_normal((rows, cols)).astype(np.float16)).cuda()
    dy = torch.from_numpy(r.standard_normal((rows, cols)).astype(np.float16)).cuda()
    gamma = torch.from_numpy(r.uniform(0.5, 1.5, cols).astype(np.float16)).cuda()
    x32 = x.float()
    mean = x32.mean(-1).contiguous()
    rstd = (1.0 / torch.sqrt(x32.var(-1, unbiased=False) + 1e-5)).contiguous()
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    p = lambda t: ctypes.c_void_p(t.data_ptr())  # noqa: E731

    def outputs():
        return (torch.full((rows, cols), float("nan"), dtype=torch.float16, device="cuda"),
                torch.full((cols, ), float("nan"), dtype=torch.float32, device="cuda"),
                torch.full((cols, ), float("nan"), dtype=torch.float32, device="cuda"))

    need = lib.dmlhip_layernorm_backward_workspace_bytes(rows, cols)
    ws = torch.empty(max(need, 16), dtype=torch.uint8, device="cuda")
    dx0, dg0, db0 = outputs()
    assert lib.dmlhip_layernorm_backward_f16(p(dy), p(x), p(mean), p(rstd), p(gamma), p(dx0), p(dg0), p(db0), rows,
                                             cols, p(ws), need, stream) == 0
    dx1, dg1, db1 = outputs()
    # one call first: the first call on a device looks up the address of the built-in buffer
    assert lib.dmlhip_layernorm_backward_noalloc_f16(p(dy), p(x), p(mean), p(rstd), p(gamma), p(dx1), p(dg1), p(db1),
                                                     rows, cols, stream) == 0
    dx1, dg1, db1 = outputs()
    torch.cuda.synchronize()
    # free bytes of the device as the driver reports them: a hipMalloc inside the library would show here (torch's own
    # counters only see torch's allocator)
    free_before = torch.cuda.mem_get_info()[0]
    assert lib.dmlhip_layernorm_backward_noalloc_f16(p(dy), p(x), p(mean), p(rstd), p(gamma), p(dx1), p(dg1), p(db1),
                                                     rows, cols, stream) == 0
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before
    assert torch.equal(dx0, dx1) and torch.equal(dg0, dg1) and torch.equal(db0, db1), \
        "the no-allocation entry point differs from dmlhip_layernorm_backward_f16 at %d x %d" % (rows, cols)
    # and both agree with the oracle
    want_dx, want_dg, want_db = O.layernorm_backward(host(dy).astype(np.float64), host(x).astype(np.float64),
                                                     host(gamma).astype(np.float64), 1e-5)
    assert_close(host(dx1), want_dx, torch.float16, "dx %d x %d" % (rows, cols))
    # fp32 sums over the rows of products of the given fp16 values: the stated tolerance as it stands
    assert_close(host(dg1), want_dg, torch.float16, "dgamma")
    assert_close(host(db1), want_db, torch.float16, "dbeta")


def test_no_allocation_entry_point_matches_the_workspace_one(lib):
    from daceml_amd import _lib as L
    assert lib.dmlhip_layernorm_backward_noalloc_max_bytes() == 8 << 20
    _case(lib, 4096, 1024, 21)       # the BERT-large shape: 256 partial rows of 8 KiB
    _case(lib, 37, 768, 22)          # smaller, right after: the array still holds the first call's partial sums
    _case(lib, 5, 100, 23)           # a shape of the generic (workgroup-per-row) path
    # beyond the built-in buffer: refused on the host, nothing launched
    p = ctypes.c_void_p(64)
    assert lib.dmlhip_layernorm_backward_workspace_bytes(1 << 20, 4096) > 8 << 20
    assert lib.dmlhip_layernorm_backward_noalloc_f16(p, p, p, p, p, p, p, p, 1 << 20, 4096, None) == L.ERR_WORKSPACE
    assert b"built-in buffer" in lib.dmlhip_last_error_string()
