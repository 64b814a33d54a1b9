"""CPU: the flags of neuzip_amd/_build.py act on the gfx950 pass of the
library's own sources (the warning about an unknown feature comes from the
x86 host pass of the same hipcc command)."""
import os
import re
import subprocess

import pytest

from neuzip_amd import _build

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")


@pytest.mark.skipif(not os.path.exists(HIPCC), reason="hipcc not installed")
def test_device_code_has_no_packed_fp32_forms(tmp_path):
    out = tmp_path / "nz_api.s"
    flags = [f for f in _build.HIPCC_FLAGS if f not in ("-shared", "-fPIC")]
    cmd = [HIPCC, *flags, "--cuda-device-only", "-S", os.path.join(_build.CSRC, "nz_api.hip"), "-o", str(out)]
    res = subprocess.run(cmd, cwd=_build.CSRC, capture_output=True, text=True)
    assert res.returncode == 0, res.stderr
    # the device pass knows the feature: no complaint when the host pass is left out
    assert "not a recognized feature" not in res.stderr
    text = out.read_text()
    assert "nz_decode_kernel" in text and "amdgcn" in text
    assert not re.search(r"\bv_pk_(add|mul|fma)_f32\b", text)
