"""The C-ABI library without a GPU: it loads, exports every function the header
declares, and its host-only entry points and argument checks behave."""
import ctypes
import os
import re

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    import glob
    headers = sorted(glob.glob(os.path.join(ROOT, "include", "*.h")))
    assert [os.path.basename(h) for h in headers] == ["tagi_hip.h", "tagi_hip_test_hooks.h"]
    text = "".join(open(h).read() for h in headers)
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(tagi_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    from cutagi_amd import capi
    names = _declared()
    assert len(names) >= 20
    for n in names:
        assert hasattr(capi.lib, n), "missing export: " + n
        assert n in capi.SIGNATURES, "binding missing for: " + n
    assert sorted(capi.SIGNATURES) == names
    assert capi.version() == 106


def test_error_strings_and_device_count():
    from cutagi_amd import capi
    assert capi.lib.tagi_hip_error_string(0) == b"ok"
    assert b"invalid" in capi.lib.tagi_hip_error_string(capi.ERR_INVALID_ARG)
    assert capi.device_count() >= 0


def test_null_and_bad_sizes_are_rejected_before_any_launch():
    from cutagi_amd import capi
    L = capi.lib
    one = ctypes.c_void_p(16)  # never dereferenced: the size check fires first
    assert L.tagi_linear_fwd(None, one, one, one, one, one, 4, 4, 4, 1, one, one, None) == capi.ERR_INVALID_ARG
    assert L.tagi_linear_fwd(one, one, one, one, one, one, 0, 4, 4, 1, one, one, None) == capi.ERR_INVALID_ARG
    assert L.tagi_linear_fwd(one, one, None, None, one, one, 4, 4, 4, 1, one, one, None) == capi.ERR_INVALID_ARG
    assert L.tagi_linear_bwd_dz(one, one, one, one, 4, -1, 4, one, one, None) == capi.ERR_INVALID_ARG
    assert L.tagi_linear_bwd_dw(one, one, one, None, 4, 4, 4, one, one, None) == capi.ERR_INVALID_ARG
    assert L.tagi_param_update(one, one, 0.0, 4, one, one, None, None) == capi.ERR_INVALID_ARG
    assert L.tagi_layer_update(one, one, 4, one, one, None, None, 0, None, None, 2.0, None, 2,
                               None) == capi.ERR_INVALID_ARG      # slot is 0 or 1
    assert L.tagi_layer_update(one, one, 4, one, one, None, None, 3, None, None, 2.0, None, 0,
                               None) == capi.ERR_INVALID_ARG      # biases announced, none given
    assert L.tagi_hip_tune(b"no.such.key", 1) == capi.ERR_INVALID_ARG
    with pytest.raises(capi.TagiHipError):
        capi.check(capi.ERR_INVALID_ARG)


def test_newer_entry_points_reject_bad_arguments_before_any_launch():
    import ctypes
    from cutagi_amd import capi
    L = capi.lib
    one = ctypes.c_void_p(16)  # never dereferenced: the checks fire first
    # fused activation: only ReLU (1) and MixtureReLU (2); the Jacobian output is required
    assert L.tagi_linear_fwd_act(one, one, one, one, one, one, 4, 4, 4, 1, 0, one, one, one,
                                 None) == capi.ERR_INVALID_ARG
    assert L.tagi_linear_fwd_act(one, one, one, one, one, one, 4, 4, 4, 1, 3, one, one, one,
                                 None) == capi.ERR_INVALID_ARG
    assert L.tagi_linear_fwd_act(one, one, one, one, one, one, 4, 4, 4, 1, 1, one, one, None,
                                 None) == capi.ERR_INVALID_ARG
    assert L.tagi_conv2d_fwd_act(one, one, one, one, one, one, one, 4, 4, 4, 4, 3, 2, 1, 7, one,
                                 one, one, None) == capi.ERR_INVALID_ARG
    # heteroscedastic update: negative count, null arrays, arrays that are not 8-byte aligned
    assert L.tagi_out_update_heteros(one, one, one, one, -1, one, one, None) == capi.ERR_INVALID_ARG
    assert L.tagi_out_update_heteros(None, one, one, one, 4, one, one, None) == capi.ERR_INVALID_ARG
    odd = ctypes.c_void_p(20)
    assert L.tagi_out_update_heteros(odd, one, one, one, 4, one, one, None) == capi.ERR_INVALID_ARG
    assert L.tagi_param_raw_update(None, one, 4, one, one, None) == capi.ERR_INVALID_ARG
    # model update: a null table, a layer with weights announced and none given, a bad slot
    assert L.tagi_model_update(None, 2, None) == capi.ERR_INVALID_ARG
    assert L.tagi_model_update(None, 0, None) == capi.OK
    items = (capi.UpdateItem * 1)()
    items[0].num_weights, items[0].cap_factor, items[0].slot = 8, 2.0, 0
    assert L.tagi_model_update(ctypes.cast(items, ctypes.c_void_p), 1, None) == capi.ERR_INVALID_ARG
    for name in ("delta_mu_w", "delta_var_w", "mu_w", "var_w"):
        setattr(items[0], name, 16)
    items[0].slot = 2
    assert L.tagi_model_update(ctypes.cast(items, ctypes.c_void_p), 1, None) == capi.ERR_INVALID_ARG
    items[0].slot, items[0].cap_factor = 0, 0.0
    assert L.tagi_model_update(ctypes.cast(items, ctypes.c_void_p), 1, None) == capi.ERR_INVALID_ARG


def test_host_only_entry_points(oracle_lib):
    from cutagi_amd import capi
    for b in (-1, 0, 1, 2, 255, 256, 5000):
        assert capi.cap_factor(b, 1.25) == pytest.approx(oracle_lib.cap_factor(b, 1.25))
    assert capi.conv2d_out_size(3, 1, 32, 32, 1, 1) == (32, 32)
    assert capi.conv2d_out_size(3, 2, 32, 32, 1, 2) == (16, 16)
    assert capi.conv2d_out_size(2, 2, 32, 32, 0, 1) == (16, 16)
    with pytest.raises(capi.TagiHipError):   # stride does not divide: the reference throws
        capi.conv2d_out_size(3, 2, 8, 8, 0, 1)
    a = capi.conv2d_build_idx(3, 1, 32, 32, 1, 1, 64 * 64 * 9 + 1)
    b = oracle_lib.conv2d_build_idx(3, 1, 32, 32, 1, 1, 64 * 64 * 9 + 1)
    for key in ("Fmwa_2", "FCzwa_1", "Szz_ud", "w", "h"):
        assert np.array_equal(a[key], b[key])
    assert (a["w"], a["h"]) == (1024, 9)


def test_bench_refuses_more_than_one_gpu():
    """bench.py measures one GPU; asking for more ends with a message and a non-zero
    status before anything touches a device."""
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    res = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"],
                         capture_output=True, text=True, timeout=120)
    assert res.returncode != 0
    assert "one GPU" in res.stderr
    assert res.stdout.strip() == ""


def test_tuning_switches_are_not_part_of_the_boundary_header():
    """The drop-in boundary (tagi_hip.h) offers no kernel-selection switch; the test
    hook lives in a header of its own that a binding of the reference never includes."""
    text = open(os.path.join(ROOT, "include", "tagi_hip.h")).read()
    assert "tagi_hip_tune" not in text
    assert "tagi_hip_tune" in open(os.path.join(ROOT, "include", "tagi_hip_test_hooks.h")).read()
