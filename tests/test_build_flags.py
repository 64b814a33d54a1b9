"""CPU: the flags of neuzip_amd/_build.py act on the gfx950 pass of the
library's own sources (the note about an unknown feature comes from the x86
host pass of the same hipcc command)."""
import os
import re
import subprocess

import pytest

from neuzip_amd import _build

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")


@pytest.mark.skipif(not os.path.exists(HIPCC), reason="hipcc not installed")
@pytest.mark.parametrize("source,extra,kernel", [("nz_api.hip", [], "nz_absmax_kernel"),
                                                 ("nz_launch.hip", ["-DNZ_S=3"], "nz_decode_kernel")])
def test_device_code_has_no_packed_fp32_forms(tmp_path, source, extra, kernel):
    out = tmp_path / (source + ".s")
    flags = [f for f in _build.HIPCC_FLAGS if f != "-fPIC"]
    cmd = [HIPCC, *flags, *extra, "--cuda-device-only", "-S", os.path.join(_build.CSRC, source), "-o", str(out)]
    res = subprocess.run(cmd, cwd=_build.CSRC, capture_output=True, text=True)
    assert res.returncode == 0, res.stderr
    # the device pass knows the feature: no complaint when the host pass is left out
    assert "not a recognized feature" not in res.stderr
    text = out.read_text()
    assert kernel in text and "amdgcn" in text
    assert not re.search(r"\bv_pk_(add|mul|fma)_f32\b", text)


def test_every_precision_has_a_translation_unit(tmp_path):
    units = _build.units(str(tmp_path))
    # every precision in two parts (encode; decode family and fused products), compiled side by side
    assert [u[1] for u in units[1:]] == [[f"-DNZ_S={s}", f"-DNZ_PART={p}"] for s in (7, 3, 1, 0) for p in (0, 12)]
    assert all(os.path.exists(u[0]) for u in units)
