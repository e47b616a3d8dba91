"""The kernels the library runs by default compile to the instructions that were validated on hardware.

tests/golden/validated_kernel_digests.json records, per kernel, a digest of its instructions at the time it last
passed the GPU tests (tests/validated_kernels.py says how; tests/golden/make_validated_kernel_digests.py writes it).
Work done on the templates without a GPU must not move them: a mismatch here means that a kernel of the default path
is no longer the one that was tested, and either the change is undone or the kernel goes back to the GPU and the
digests are recorded again. Needs hipcc (and the compiler the digests were made with), no GPU."""
import json
import os

import pytest

from tests import validated_kernels as V


def test_default_kernels_are_the_ones_that_ran_on_hardware(tmp_path):
    if not V.have_hipcc():
        pytest.skip("no hipcc")
    recorded = json.load(open(os.path.join(V.ROOT, "tests", "golden", "validated_kernel_digests.json")))
    if recorded["compiler"] != V.compiler_version():
        pytest.skip("digests were recorded with %s, this is %s" % (recorded["compiler"], V.compiler_version()))
    current = V.current_digests(str(tmp_path))
    assert sorted(current) == sorted(recorded["kernels"]), "the set of recorded kernels changed"
    changed = [name for name, d in recorded["kernels"].items() if current[name] != d]
    assert not changed, "instructions differ from the validated build:\n" + "\n".join(changed)


def test_the_digest_sees_a_changed_instruction(tmp_path):
    text = "_Z1kv:\n\tv_add_f32_e32 v0, v1, v2 ; comment\n.LBB3_1:\n\ts_cbranch_scc1 .LBB3_1\n\ts_endpgm\n"
    a, b, c = tmp_path / "a.s", tmp_path / "b.s", tmp_path / "c.s"
    a.write_text(text)
    b.write_text(text.replace("LBB3_", "LBB7_").replace("; comment", "; another comment"))
    c.write_text(text.replace("v1, v2", "v2, v1"))
    da, db, dc = (V.digest(V.kernel_bodies(str(p))["_Z1kv"]) for p in (a, b, c))
    assert da == db and da != dc
