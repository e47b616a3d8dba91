"""The kernels that place their own LDS reads and waits (fused attention, the interleaved GEMM loop) are compiled to
assembly and checked: no instruction touches a register that an outstanding LDS read still has to write
(tests/isa_hazards.py says why that can happen). Needs hipcc, no GPU."""
import os
import shutil
import subprocess

import pytest

from tests import isa_hazards

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _assembly(src, tmp_path):
    from daceml_amd.csrc import build as B
    if not (shutil.which("hipcc") or os.path.exists("/opt/rocm/bin/hipcc")):
        pytest.skip("no hipcc")
    out = str(tmp_path / (os.path.basename(src) + ".s"))
    cmd = [B.hipcc(), *B.COMMON_FLAGS, "-x", "hip", "--offload-device-only", "-S", src, "-o", out]
    res = subprocess.run(cmd, capture_output=True, text=True)
    assert res.returncode == 0, res.stderr[-4000:]
    return out


def _report(found):
    lines = []
    for name, bad in found.items():
        lines.append("%s: %d" % (name, len(bad)))
        for ln in sorted(bad)[:5]:
            lines.append("   line %d: %s (registers %s, reads issued at lines %s)" % ((ln, ) + tuple(bad[ln])))
    return "\n".join(lines)


def test_the_check_finds_a_register_reused_under_an_outstanding_read(tmp_path):
    """What the check is for, in eight instructions: the result of the first read is never used, so its registers
    carry an address by the time the data arrives."""
    text = """
_Z6kernelv:
	ds_read_b128 v[4:7], v1
	v_lshl_add_u64 v[4:5], v[10:11], 1, s[0:1]
	global_load_lds_dwordx4 v[4:5], off
	s_waitcnt lgkmcnt(0)
	v_mov_b32_e32 v6, 0
	s_endpgm
.Lfunc_end0:
"""
    p = tmp_path / "k.s"
    p.write_text(text)
    count, found = isa_hazards.check_file(str(p))
    assert count == 1 and sorted(found["_Z6kernelv"]) == [4, 5]
    # the same with the wait ahead of the reuse is clean; so is a partial wait that retires the older of two reads
    p.write_text(text.replace("\tds_read_b128 v[4:7], v1\n", "\tds_read_b128 v[4:7], v1\n\ts_waitcnt lgkmcnt(0)\n"))
    assert isa_hazards.check_file(str(p))[1] == {}
    p.write_text(text.replace("\tds_read_b128 v[4:7], v1\n",
                              "\tds_read_b128 v[4:7], v1\n\tds_read_b128 v[12:15], v1\n\ts_waitcnt lgkmcnt(1)\n"))
    assert isa_hazards.check_file(str(p))[1] == {}


def test_fused_attention_kernels(tmp_path):
    count, found = isa_hazards.check_file(_assembly(os.path.join(ROOT, "daceml_amd", "csrc", "attention.hip"), tmp_path))
    assert count == 6, "forward, dQ and dK/dV kernels, each with and without a mask"
    assert not found, _report(found)


def test_interleaved_gemm_loop(tmp_path):
    count, found = isa_hazards.check_file(_assembly(os.path.join(ROOT, "tests", "isa", "ilv_instances.hip"), tmp_path))
    assert count == 28, "five tile configurations, operand pairs and row sums x four operand-layout pairs"
    assert not found, _report(found)


def test_wide_stores_in_inline_assembly_carry_their_wait_states(tmp_path):
    """lds_ops.h stores GEMM results with an inline-assembly ``global_store_dwordx4 ... sc1``; the two wait states the
    compiler would have kept between such a store and the next write to its data registers are part of the statement."""
    p = tmp_path / "k.s"
    p.write_text("_Z1kv:\n\t;;#ASMSTART\n\tglobal_store_dwordx4 v[0:1], v[4:7], off sc1\n\t;;#ASMEND\n"
                 "\tv_mov_b32_e32 v4, 0\n\ts_endpgm\n")
    assert isa_hazards.check_store_data(str(p)) == {"_Z1kv": [3]}
    p.write_text("_Z1kv:\n\t;;#ASMSTART\n\tglobal_store_dwordx4 v[0:1], v[4:7], off sc1\n\ts_nop 1\n\t;;#ASMEND\n"
                 "\tv_mov_b32_e32 v4, 0\n\ts_endpgm\n")
    assert isa_hazards.check_store_data(str(p)) == {}
    asm = _assembly(os.path.join(ROOT, "tests", "isa", "ilv_instances.hip"), tmp_path)
    text = open(asm).read()
    assert " sc1" in text, "the GEMM epilogue stores its fp16 results through the L2"
    assert isa_hazards.check_store_data(asm) == {}


def test_dropping_the_value_of_an_lds_read_does_not_compile(tmp_path):
    """The readers of lds_ops.h are [[nodiscard]] and the library's flags turn the warning into an error: the pattern
    behind the register race (a read issued, its value never used) is rejected by the compiler."""
    from daceml_amd.csrc import build as B
    if not (shutil.which("hipcc") or os.path.exists("/opt/rocm/bin/hipcc")):
        pytest.skip("no hipcc")
    header = os.path.join(ROOT, "daceml_amd", "csrc", "lds_ops.h")
    body = {"dropped": "dml::lds_read_b128<0>(0u); dml::lds_read_tr16_b64<0>(0u); o[0] = 1.f;",
            "used": "const dml::half8 v = dml::lds_read_b128<0>(0u); dml::wait_lgkm<0>(); o[0] = (float)v[0];"}
    results = {}
    for name, text in body.items():
        src = tmp_path / (name + ".hip")
        src.write_text('#include "%s"\n__global__ void k(float* o) { %s }\n' % (header, text))
        cmd = [B.hipcc(), *B.COMMON_FLAGS, "-x", "hip", "--offload-device-only", "-c", str(src), "-o",
               str(tmp_path / (name + ".o"))]
        results[name] = subprocess.run(cmd, capture_output=True, text=True)
    assert results["used"].returncode == 0, results["used"].stderr[-2000:]
    assert results["dropped"].returncode != 0 and "nodiscard" in results["dropped"].stderr
