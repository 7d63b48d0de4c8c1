"""Parity of the HIP Conv2d path (through the C ABI) against the CPU oracle."""
import numpy as np
import pytest

from util import assert_close, conv_inputs

pytestmark = pytest.mark.gpu

# (kernel, stride, pad, pad_type, wi, fi, fo, B): the geometries of the ResNet-18
# configuration (3x3 s1 p1, 3x3 s2 p1 type 2, 2x2 s2 shortcut), odd channel
# counts (27 = 3*9 reduction, the first ResNet conv), 1x1, 5x5 and 7x7 kernels.
GEOMS = [
    (3, 1, 1, 1, 8, 4, 8, 3),
    (3, 1, 1, 1, 16, 3, 16, 2),
    (3, 2, 1, 2, 8, 8, 16, 4),
    (2, 2, 0, 1, 8, 8, 16, 2),
    (1, 1, 0, 1, 6, 5, 7, 3),
    (5, 1, 2, 1, 9, 2, 3, 2),
    (3, 1, 0, 1, 10, 6, 5, 2),
    (3, 1, 1, 1, 32, 16, 32, 2),
    (3, 1, 1, 1, 12, 70, 66, 1),
    (4, 2, 1, 1, 10, 3, 5, 2),
    (7, 2, 3, 1, 17, 3, 40, 2),  # per-tap table + staged tiles exceed 64 KB of LDS
    (3, 1, 1, 1, 4, 128, 96, 3),  # late-stage shape: few pixels, long reduction (sliced)
    (2, 2, 0, 1, 8, 64, 130, 2),  # projection shortcut, more than 128 output channels
]


def _setup(oracle_lib, geom, bias, seed):
    import torch
    from cutagi_amd import capi
    k, s, p, pt, wi, fi, fo, B = geom
    idx = capi.conv2d_build_idx(k, s, wi, wi, p, pt, k * k * fi * fo + 1)
    ref_idx = oracle_lib.conv2d_build_idx(k, s, wi, wi, p, pt, k * k * fi * fo + 1)
    for key in ("Fmwa_2", "FCzwa_1", "Szz_ud"):
        assert np.array_equal(idx[key], ref_idx[key]), key
    assert idx["w"] == wi * wi, "every input pixel must be covered"
    wihi, woho = wi * wi, idx["wo"] * idx["ho"]
    d = conv_inputs(fi, fo, k, wihi, woho, B, seed=seed, bias=bias, jcb_random=True)
    t = {n: (None if v is None else torch.from_numpy(v).cuda()) for n, v in d.items()}
    ti = {n: torch.from_numpy(idx[n]).cuda() for n in ("Fmwa_2", "FCzwa_1", "Szz_ud")}
    return idx, d, t, ti, wihi, woho


@pytest.mark.parametrize("geom", GEOMS)
@pytest.mark.parametrize("bias", [False, True])
def test_conv2d_forward(oracle_lib, geom, bias):
    import cutagi_amd.functional as F
    k, s, p, pt, wi, fi, fo, B = geom
    idx, d, t, ti, wihi, woho = _setup(oracle_lib, geom, bias, seed=sum(geom))
    mu_z, var_z = F.conv2d_fwd(t["mu_w"], t["var_w"], t["mu_b"], t["var_b"], t["mu_a"], t["var_a"],
                               ti["Fmwa_2"], woho, fo, wihi, fi, k, B)
    ref = oracle_lib.conv2d_fwd(d["mu_w"], d["var_w"], d["mu_b"], d["var_b"], d["mu_a"],
                                d["var_a"], idx["Fmwa_2"], woho, fo, wihi, fi, k, B, threads=4)
    assert_close(mu_z.cpu().numpy(), ref[0], "mu_z")
    assert_close(var_z.cpu().numpy(), ref[1], "var_z")
    assert float(var_z.min()) >= 0.0


@pytest.mark.parametrize("geom", GEOMS)
def test_conv2d_backward(oracle_lib, geom):
    import cutagi_amd.functional as F
    k, s, p, pt, wi, fi, fo, B = geom
    idx, d, t, ti, wihi, woho = _setup(oracle_lib, geom, True, seed=3 + sum(geom))
    dz = F.conv2d_bwd_dz(t["mu_w"], t["jcb"], t["delta_mu"], t["delta_var"], ti["FCzwa_1"],
                         ti["Szz_ud"], woho, fo, wihi, fi, k, idx["h"], B)
    ref_dz = oracle_lib.conv2d_bwd_dz(d["mu_w"], d["jcb"], d["delta_mu"], d["delta_var"],
                                      idx["FCzwa_1"], idx["Szz_ud"], woho, fo, wihi, fi, k,
                                      idx["h"], B, threads=4)
    assert_close(dz[0].cpu().numpy(), ref_dz[0], "delta_mu_z")
    assert_close(dz[1].cpu().numpy(), ref_dz[1], "delta_var_z")
    dw = F.conv2d_bwd_dw(t["var_w"], t["var_b"], t["mu_a"], t["delta_mu"], t["delta_var"],
                         ti["Fmwa_2"], B, fo, woho, wihi, fi, k)
    ref_dw = oracle_lib.conv2d_bwd_dw(d["var_w"], d["var_b"], d["mu_a"], d["delta_mu"],
                                      d["delta_var"], idx["Fmwa_2"], B, fo, woho, wihi, fi, k,
                                      threads=4)
    for name, got, ref in zip(["delta_mu_w", "delta_var_w", "delta_mu_b", "delta_var_b"], dw,
                              ref_dw):
        assert_close(got.cpu().numpy(), ref, name)
    assert float(dz[1].max()) <= 0.0 and float(dw[1].max()) <= 0.0
