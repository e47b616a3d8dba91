"""Writes tests/golden/validated_kernel_digests.json: one SHA-256 per kernel of tests/isa/validated_instances.hip, of
the fused expand + depthwise kernels of daceml_amd/csrc/conv_fused.hip and of the attention kernels of
daceml_amd/csrc/attention.hip, over the kernel's instructions as the compiler emits them
(comments and block-label numbers removed).

Run it on a tree whose kernels have just passed the GPU tests - the digests are a record of what was validated on
hardware, and tests/test_validated_kernels.py compares later builds with them:

    python tests/golden/make_validated_kernel_digests.py
"""
import json
import os
import sys
import tempfile

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from tests import validated_kernels as V  # noqa: E402


def main():
    with tempfile.TemporaryDirectory() as tmp:
        digests = V.current_digests(tmp)
    out = os.path.join(ROOT, "tests", "golden", "validated_kernel_digests.json")
    json.dump({"compiler": V.compiler_version(), "kernels": digests}, open(out, "w"), indent=1, sort_keys=True)
    print("wrote %d digests to %s" % (len(digests), out))


if __name__ == "__main__":
    main()
