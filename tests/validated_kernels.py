"""Instruction digests of kernels that have passed their tests on the GPU (TEST INFRASTRUCTURE ONLY).

Work on the kernel templates that happens without a GPU - a new template parameter, a new tile shape, a shared helper
rewritten - must leave the instantiations the library runs by default exactly as they were when they last ran on
hardware. The compiler's assembly output is the evidence: a kernel's instructions, with comments and the numbering of
block labels removed, are hashed, and the hashes recorded at validation time live in
tests/golden/validated_kernel_digests.json."""
import hashlib
import os
import re
import shutil
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SOURCES = [os.path.join(ROOT, "tests", "isa", "validated_instances.hip"),
           os.path.join(ROOT, "daceml_amd", "csrc", "conv_fused.hip"),
           os.path.join(ROOT, "daceml_amd", "csrc", "attention.hip")]
#: kernels of SOURCES that are recorded
RECORDED = re.compile(r"gemm_f16_pipe_kernel|expand_depthwise_kernel|expand_depthwise_rolling_kernel|attention_fwd_kernel|"
                      r"attention_bwd_dq_kernel|attention_bwd_dkv_kernel")


def have_hipcc():
    return bool(shutil.which("hipcc") or os.path.exists("/opt/rocm/bin/hipcc"))


def compiler_version():
    from daceml_amd.csrc import build as B
    out = subprocess.run([B.hipcc(), "--version"], capture_output=True, text=True).stdout
    m = re.search(r"clang version \S+", out)
    return m.group(0) if m else out.strip().splitlines()[0]


def kernel_bodies(path):
    """{mangled name: [instruction lines]} of an assembly file."""
    out, name, body = {}, None, []
    for line in open(path):
        m = re.match(r"^(_Z\w+):", line)
        if m:
            name, body = m.group(1), []
            continue
        if name is None:
            continue
        text = line.split(";")[0].strip()
        if text:
            body.append(re.sub(r"\.LBB\d+_", ".LBB_", text))
        if "s_endpgm" in line:
            out[name] = body
            name = None
    return out


def digest(body):
    return hashlib.sha256("\n".join(body).encode()).hexdigest()


def current_digests(tmp):
    from daceml_amd.csrc import build as B
    digests = {}
    for src in SOURCES:
        out = os.path.join(tmp, os.path.basename(src) + ".s")
        cmd = [B.hipcc(), *B.COMMON_FLAGS, "-x", "hip", "--offload-device-only", "-S", src, "-o", out]
        res = subprocess.run(cmd, capture_output=True, text=True)
        assert res.returncode == 0, res.stderr[-4000:]
        for name, body in kernel_bodies(out).items():
            if RECORDED.search(name):
                digests[name.replace("12_GLOBAL__N_1", "")] = digest(body)
    return digests
