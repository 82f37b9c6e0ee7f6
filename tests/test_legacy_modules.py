"""The code objects built for an unmodified host of the reference (adrastea_amd/lib/legacy/):
they must exist after a build and export the device symbols that host looks up
(adrastea_models/src/kernels.rs:472-473, 485-486)."""
import os

import pytest

from adrastea_amd import build

EXPECTED = {
    "matmul.co": [b"matmul_f16", b"matmul_f16_fast", b"matmul_f16_raw"],
    "error_stats.co": [b"error_stats_f16", b"error_stats_f32"],
}


@pytest.mark.parametrize("module", sorted(EXPECTED))
def test_legacy_module_exports_the_reference_symbols(module):
    build.build_legacy_modules()
    path = os.path.join(build.LEGACY_DIR, module)
    assert os.path.exists(path)
    blob = open(path, "rb").read()
    for sym in EXPECTED[module]:
        # a kernel `name` has the symbol itself and its descriptor `name.kd`
        assert sym + b"\x00" in blob and sym + b".kd\x00" in blob, sym
