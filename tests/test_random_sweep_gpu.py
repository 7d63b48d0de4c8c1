"""Seeded random sweeps of the Linear and Conv2d paths against the CPU oracle: shapes
nobody picked by hand (odd sizes, every batch class, kernels 1..5, strides 1..3, both
padding types), all three passes of each, every output held to the parity gate."""
import numpy as np
import pytest

from util import SAME_SIGN, assert_close, conv_inputs, linear_inputs

pytestmark = pytest.mark.gpu


def _dev(d):
    import torch
    return {k: (None if v is None else torch.from_numpy(v).cuda()) for k, v in d.items()}


def _linear_shapes(n, seed):
    rng = np.random.default_rng(seed)
    out = []
    for _ in range(n):
        kind = rng.integers(0, 4)
        B = int([rng.integers(1, 9), rng.integers(9, 17), rng.integers(17, 65),
                 rng.integers(65, 300)][kind])
        K = int(rng.integers(1, 1200)) if rng.random() < 0.7 else int(4 * rng.integers(1, 400))
        N = int(rng.integers(1, 700)) if rng.random() < 0.7 else int(4 * rng.integers(1, 200))
        out.append((K, N, B))
    return out


@pytest.mark.parametrize("K,N,B", _linear_shapes(48, seed=2024))
def test_linear_random_shape(oracle_lib, K, N, B):
    import cutagi_amd.functional as F
    bias = (K + N + B) % 3 != 0
    d = linear_inputs(K, N, B, seed=K * 31 + N * 7 + B, bias=bias, jcb_random=True)
    t = _dev(d)
    z = F.linear_fwd(t["mu_w"], t["var_w"], t["mu_b"], t["var_b"], t["mu_a"], t["var_a"])
    ref = oracle_lib.linear_fwd(d["mu_w"], d["var_w"], d["mu_b"], d["var_b"], d["mu_a"],
                                d["var_a"], threads=4)
    assert_close(z[0].cpu().numpy(), ref[0], "mu_z")
    assert_close(z[1].cpu().numpy(), ref[1], "var_z", same_sign=True)
    vb = t["var_b"] if bias else None
    out = F.linear_bwd(t["mu_w"], t["var_w"], vb, t["mu_a"], t["jcb"], t["delta_mu"],
                       t["delta_var"])
    want = (oracle_lib.linear_bwd_dz(d["mu_w"], d["jcb"], d["delta_mu"], d["delta_var"], threads=4)
            + oracle_lib.linear_bwd_dw(d["var_w"], d["mu_a"], d["delta_mu"], d["delta_var"], threads=4))
    names = ["delta_mu_z", "delta_var_z", "delta_mu_w", "delta_var_w"]
    if bias:
        want = want + oracle_lib.linear_bwd_db(d["var_b"], d["delta_mu"], d["delta_var"])
        names += ["delta_mu_b", "delta_var_b"]
    for name, got, r in zip(names, out, want):
        assert_close(got.cpu().numpy(), r, name, same_sign=name in SAME_SIGN)


def _conv_geoms(n, seed):
    """Random valid geometries: the output size formula must divide (the reference
    throws otherwise) and every input pixel must be covered (its kernels assume it)."""
    from cutagi_amd import capi
    rng = np.random.default_rng(seed)
    out = []
    while len(out) < n:
        k = int(rng.integers(1, 6))
        s = int(rng.integers(1, 4))
        pt = int(rng.integers(1, 3))
        p = int(rng.integers(0, k))
        wi = int(rng.integers(max(k, 3), 21))
        try:
            idx = capi.conv2d_build_idx(k, s, wi, wi, p, pt, 7)
        except capi.TagiHipError:
            continue
        if idx["w"] != wi * wi or idx["wo"] < 1:
            continue
        fi, fo = int(rng.integers(1, 40)), int(rng.integers(1, 80))
        if rng.random() < 0.3:
            fi, fo = int(8 * rng.integers(1, 12)), int(64 * rng.integers(1, 3))
        B = int(rng.integers(1, 7))
        out.append((k, s, p, pt, wi, fi, fo, B))
    return out


@pytest.mark.parametrize("geom", _conv_geoms(40, seed=77))
def test_conv2d_random_geometry(oracle_lib, geom):
    import torch
    import cutagi_amd.functional as F
    from cutagi_amd import capi
    k, s, p, pt, wi, fi, fo, B = geom
    bias = sum(geom) % 2 == 0
    idx = capi.conv2d_build_idx(k, s, wi, wi, p, pt, k * k * fi * fo + 1)
    ref_idx = oracle_lib.conv2d_build_idx(k, s, wi, wi, p, pt, k * k * fi * fo + 1)
    for key in ("Fmwa_2", "FCzwa_1", "Szz_ud"):
        assert np.array_equal(idx[key], ref_idx[key]), key
    wihi, woho = wi * wi, idx["wo"] * idx["ho"]
    d = conv_inputs(fi, fo, k, wihi, woho, B, seed=sum(geom) * 3 + 1, bias=bias, jcb_random=True)
    t = _dev(d)
    ti = {n: torch.from_numpy(idx[n]).cuda() for n in ("Fmwa_2", "FCzwa_1", "Szz_ud")}
    z = F.conv2d_fwd(t["mu_w"], t["var_w"], t["mu_b"], t["var_b"], t["mu_a"], t["var_a"],
                     ti["Fmwa_2"], woho, fo, wihi, fi, k, B)
    ref = oracle_lib.conv2d_fwd(d["mu_w"], d["var_w"], d["mu_b"], d["var_b"], d["mu_a"], d["var_a"],
                                idx["Fmwa_2"], woho, fo, wihi, fi, k, B, 4)
    assert_close(z[0].cpu().numpy(), ref[0], "mu_z")
    assert_close(z[1].cpu().numpy(), ref[1], "var_z", same_sign=True)
    dz = F.conv2d_bwd_dz(t["mu_w"], t["jcb"], t["delta_mu"], t["delta_var"], ti["FCzwa_1"],
                         ti["Szz_ud"], woho, fo, wihi, fi, k, idx["h"], B)
    ref = oracle_lib.conv2d_bwd_dz(d["mu_w"], d["jcb"], d["delta_mu"], d["delta_var"],
                                   idx["FCzwa_1"], idx["Szz_ud"], woho, fo, wihi, fi, k, idx["h"],
                                   B, 4)
    assert_close(dz[0].cpu().numpy(), ref[0], "delta_mu_z")
    assert_close(dz[1].cpu().numpy(), ref[1], "delta_var_z", same_sign=True)
    dw = F.conv2d_bwd_dw(t["var_w"], t["var_b"], t["mu_a"], t["delta_mu"], t["delta_var"],
                         ti["Fmwa_2"], B, fo, woho, wihi, fi, k)
    ref = oracle_lib.conv2d_bwd_dw(d["var_w"], d["var_b"], d["mu_a"], d["delta_mu"],
                                   d["delta_var"], idx["Fmwa_2"], B, fo, woho, wihi, fi, k, 4)
    names = ["delta_mu_w", "delta_var_w"] + (["delta_mu_b", "delta_var_b"] if bias else [])
    for name, got, r in zip(names, dw, ref):
        assert_close(got.cpu().numpy(), r, name, same_sign=name in SAME_SIGN)
