"""Host-side checks of the C-ABI library that need no GPU: it loads, exports every
symbol the header declares, and its shape/validation logic matches the oracle."""
import ctypes
import os
import re

import pytest

import dlprimitives_amd as dlp
from conv_cases import REFERENCE_MATRIX, case_id

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "dlprim_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(dlp_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    L = ctypes.CDLL(dlp.library_path())
    names = declared_symbols()
    assert len(names) >= 20
    for n in names:
        assert hasattr(L, n), "missing export " + n


def test_version_and_error_string():
    L = dlp.lib()
    assert L.dlp_version() >= 100
    assert isinstance(L.dlp_last_error(), bytes)


@pytest.mark.parametrize("c", REFERENCE_MATRIX, ids=case_id)
def test_output_shape_matches_oracle(oracle_mod, c):
    for (b, h, w) in [(1, 32, 32), (2, 19, 21), (64, 224, 224)]:
        lkh, lkw = c["dilate"][0] * (c["kernel"][0] - 1) + 1, c["dilate"][1] * (c["kernel"][1] - 1) + 1
        if h + 2 * c["pad"][0] < lkh or w + 2 * c["pad"][1] < lkw:
            continue
        st = dlp.Conv2DSettings(c["cin"], c["cout"], c["kernel"], c["stride"], c["dilate"], c["pad"], c["groups"], (b, c["cin"], h, w))
        cfg = oracle_mod.make_cfg(c["cin"], c["cout"], c["kernel"], c["stride"], c["dilate"], c["pad"], c["groups"])
        assert dlp.conv2d_output_shape(st, (b, c["cin"], h, w)) == oracle_mod.conv2d_output_shape(cfg, (b, c["cin"], h, w))


def test_output_shape_validation_errors():
    st = dlp.Conv2DSettings(3, 8, 5, 1, 1, 0, 1, (1, 3, 8, 8))
    with pytest.raises(dlp.ValidationError):
        dlp.conv2d_output_shape(st, (1, 4, 8, 8))  # channels mismatch (src/core/conv.cpp:21)
    with pytest.raises(dlp.ValidationError):
        dlp.conv2d_output_shape(st, (1, 3, 2, 2))  # empty output (src/core/conv.cpp:26-27)


def test_create_rejects_bad_settings_before_touching_the_gpu():
    with pytest.raises(dlp.ValidationError):
        dlp.Conv2DForward.create(dlp.Conv2DSettings(6, 8, 3, 1, 1, 1, 4, (1, 6, 8, 8)), False)  # 6 % 4 != 0
    with pytest.raises(dlp.ValidationError):
        dlp.Conv2DForward.create(dlp.Conv2DSettings(4, 8, 3, 1, 1, 1, 1, (1, 4, 8, 8)), False, algo="fft")
    with pytest.raises(dlp.NotImplementedErrorDlprim):  # reference: DLPRIM_CHECK(dtype == float_data)
        dlp.Conv2DForward.create(dlp.Conv2DSettings(4, 8, 3, 1, 1, 1, 1, (1, 4, 8, 8), dtype=4), False)
    with pytest.raises(dlp.ValidationError):
        dlp.IPForward.create(dlp.IPSettings(0, 5), True)
