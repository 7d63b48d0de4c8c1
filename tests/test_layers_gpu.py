"""Parity of the layers between the contractions (MixtureReLU, BatchNorm2d,
AvgPool2d, residual adds) against the CPU oracle, through the C ABI."""
import numpy as np
import pytest

from util import assert_close, batchnorm_inputs, pool_inputs

pytestmark = pytest.mark.gpu


def _dev(d):
    import torch
    return {k: (None if v is None else torch.from_numpy(v).cuda()) for k, v in d.items()}


def test_mixture_relu(oracle_lib):
    import torch
    import cutagi_amd.functional as F
    rng = np.random.default_rng(2)
    mu = (rng.standard_normal(100003) * 3).astype(np.float32)
    var = rng.uniform(1e-3, 4.0, 100003).astype(np.float32)
    mu_a, var_a, jcb = F.mixture_relu_fwd(torch.from_numpy(mu).cuda(), torch.from_numpy(var).cuda())
    ref = oracle_lib.mixture_relu_fwd(mu, var, 4)
    assert_close(mu_a.cpu().numpy(), ref[0], "mu_a")
    assert_close(jcb.cpu().numpy(), ref[2], "jcb")
    # (the variance is a difference of terms of size mu^2: its single-precision
    # noise is absolute, which the parity metric's rms normalisation accounts for)
    got = var_a.cpu().numpy()
    assert_close(got, ref[1], "var_a")
    floor = np.float32(1e-6)
    assert got.min() >= floor and mu_a.cpu().numpy().min() >= floor


def test_mixture_relu_distribution_function_in_the_tails():
    """The activation computes the normal density and distribution function from one
    exponential and a fitted Mills ratio. The Jacobian it returns IS the distribution
    function: elementwise relative error against float64 (scipy) from alpha = -9 to 9,
    where Phi spans 1e-19 .. 1 - the rms-normalised parity metric above would not see a
    wrong tail - and the first moment against its float64 closed form where that is not
    a difference of nearly equal terms (alpha >= -2)."""
    import torch
    from scipy.stats import norm
    import cutagi_amd.functional as F
    alpha = np.linspace(-9.0, 9.0, 360001)
    sd = np.float32(0.75)
    mu = (alpha * float(sd)).astype(np.float32)
    var = np.full_like(mu, sd * sd)
    mu_a, var_a, jcb = F.mixture_relu_fwd(torch.from_numpy(mu).cuda(), torch.from_numpy(var).cuda())
    a64 = mu.astype(np.float64) / np.sqrt(var.astype(np.float64))     # what the kernel was given
    want = norm.cdf(a64)
    rel = np.abs(jcb.cpu().numpy().astype(np.float64) / want - 1.0)
    # fp32: alpha carries 6e-8 of rounding, which the tail amplifies by about alpha^2
    assert rel.max() <= 2e-5, rel.max()
    assert rel[np.abs(a64) <= 3].max() <= 2e-6
    keep = a64 >= -2.0
    s64 = np.sqrt(var.astype(np.float64))
    first = mu.astype(np.float64) * want + s64 * norm.pdf(a64)
    rel1 = np.abs(mu_a.cpu().numpy().astype(np.float64)[keep] / first[keep] - 1.0)
    assert rel1.max() <= 5e-6, rel1.max()
    # degenerate inputs: zero variance (alpha = +-inf) and huge |alpha|
    m = np.array([2.0, -2.0, 1e4, -1e4, 0.5], np.float32)
    v = np.array([0.0, 0.0, 1e-6, 1e-6, 1e-30], np.float32)
    o = [x.cpu().numpy() for x in F.mixture_relu_fwd(torch.from_numpy(m).cuda(), torch.from_numpy(v).cuda())]
    np.testing.assert_allclose(o[0], [2.0, 1e-6, 1e4, 1e-6, 0.5], rtol=1e-6)
    np.testing.assert_allclose(o[2], [1.0, 0.0, 1.0, 0.0, 1.0], atol=1e-30)
    assert np.all(o[1] >= 1e-6) and np.all(np.isfinite(o[1]))


# (wihi, fi, B): feature maps of the ResNet-18 configuration scaled down in
# batch, odd sizes, one sample per chunk, and the fully-connected form (wihi = 1)
BN_SHAPES = [(1024, 64, 4), (256, 128, 3), (16, 512, 8), (49, 5, 7), (1, 300, 16), (9, 3, 2),
             (64, 700, 2)]


@pytest.mark.parametrize("wihi,fi,B", BN_SHAPES)
@pytest.mark.parametrize("bias", [True, False])
def test_batchnorm2d(oracle_lib, wihi, fi, B, bias):
    import cutagi_amd.functional as F
    d = batchnorm_inputs(wihi, fi, B, seed=wihi + fi + B)
    t = _dev(d)
    mb, vb = (d["mu_b"], d["var_b"]) if bias else (None, None)
    tmb, tvb = (t["mu_b"], t["var_b"]) if bias else (None, None)

    ref_s = oracle_lib.batchnorm2d_stats(d["mu_a"], d["var_a"], wihi, fi, B, 0.9, d["mu_ra"],
                                         d["var_ra"], 4)
    mu_ra, var_ra = t["mu_ra"].clone(), t["var_ra"].clone()
    mu_s, var_s = F.batchnorm2d_stats(t["mu_a"], t["var_a"], wihi, fi, B, 0.9, mu_ra, var_ra)
    for name, got, ref in zip(("mu_s", "var_s", "mu_ra", "var_ra"), (mu_s, var_s, mu_ra, var_ra),
                              ref_s):
        assert_close(got.cpu().numpy(), ref, name)
    assert float(var_s.min()) > 0

    # forward and backward on the oracle's statistics, so that each stage is
    # compared on identical inputs
    import torch
    ms, vs = torch.from_numpy(ref_s[0]).cuda(), torch.from_numpy(ref_s[1]).cuda()
    mu_z, var_z = F.batchnorm2d_fwd(t["mu_w"], t["var_w"], tmb, tvb, t["mu_a"], t["var_a"], ms, vs,
                                    1e-5, wihi, fi, B)
    ref = oracle_lib.batchnorm2d_fwd(d["mu_w"], d["var_w"], mb, vb, d["mu_a"], d["var_a"],
                                     ref_s[0], ref_s[1], 1e-5, wihi, fi, B, 4)
    assert_close(mu_z.cpu().numpy(), ref[0], "mu_z")
    assert_close(var_z.cpu().numpy(), ref[1], "var_z")
    assert float(var_z.min()) >= 0

    out = F.batchnorm2d_bwd(t["mu_w"], t["var_w"], tvb, t["mu_a"], t["jcb"], ms, vs, t["dmu"],
                            t["dvar"], 1e-5, wihi, fi, B)
    rz = oracle_lib.batchnorm2d_bwd_dz(d["mu_w"], d["jcb"], ref_s[1], d["dmu"], d["dvar"], 1e-5,
                                       wihi, fi, B, 4)
    rw = oracle_lib.batchnorm2d_bwd_dw(d["var_w"], vb, d["mu_a"], ref_s[0], ref_s[1], d["dmu"],
                                       d["dvar"], 1e-5, wihi, fi, B, 4)
    names = ["delta_mu", "delta_var", "delta_mu_w", "delta_var_w", "delta_mu_b", "delta_var_b"]
    for name, got, ref in zip(names, out, rz + rw):
        if ref is None:
            assert got is None
            continue
        assert_close(got.cpu().numpy(), ref, name)
    assert float(out[1].max()) <= 0 and float(out[3].max()) <= 0


@pytest.mark.parametrize("wihi,fi,B", BN_SHAPES + [(16, 70, 9), (64, 256, 8), (20, 6, 3)])
@pytest.mark.parametrize("bias", [True, False])
@pytest.mark.parametrize("residual", [False, True])
def test_batchnorm2d_training_forward_in_one_call(oracle_lib, wihi, fi, B, bias, residual):
    """tagi_batchnorm2d_fwd_train = statistics, running averages, normalisation and the
    optional residual add. Bit for bit what the separate entry points give (the fused
    kernel repeats their arithmetic), with the merge of the statistics inside the
    normalising kernel and as a launch of its own; and the oracle's result."""
    import torch
    from cutagi_amd import capi
    d = batchnorm_inputs(wihi, fi, B, seed=3 * wihi + fi + B)
    t = _dev(d)
    n = B * fi * wihi
    rng = np.random.default_rng(n)
    res = None
    if residual:
        res = [torch.from_numpy(rng.standard_normal(n).astype(np.float32)).cuda(),
               torch.from_numpy(rng.uniform(0.01, 0.5, n).astype(np.float32)).cuda()]
    mb, vb = (t["mu_b"], t["var_b"]) if bias else (None, None)
    stream = torch.cuda.current_stream().cuda_stream

    def fused():
        ra = [t["mu_ra"].clone(), t["var_ra"].clone()]
        st = [torch.empty(fi, device="cuda"), torch.empty(fi, device="cuda")]
        z = [torch.empty(n, device="cuda"), torch.empty(n, device="cuda")]
        capi.check(capi.lib.tagi_batchnorm2d_fwd_train(
            capi.ptr(t["mu_w"]), capi.ptr(t["var_w"]), capi.ptr(mb), capi.ptr(vb), capi.ptr(t["mu_a"]),
            capi.ptr(t["var_a"]), capi.ptr(res[0]) if res else None, capi.ptr(res[1]) if res else None,
            int(bias), 0.9, 1e-5, wihi, fi, B, capi.ptr(st[0]), capi.ptr(st[1]), capi.ptr(ra[0]),
            capi.ptr(ra[1]), capi.ptr(z[0]), capi.ptr(z[1]), stream))
        return st + ra + z

    got = fused()
    capi.tune("batchnorm.fused_train", 0)
    try:
        plain = fused()
    finally:
        capi.tune("batchnorm.fused_train", 1)
    # the separate entry points
    import cutagi_amd.functional as F
    ra = [t["mu_ra"].clone(), t["var_ra"].clone()]
    st = F.batchnorm2d_stats(t["mu_a"], t["var_a"], wihi, fi, B, 0.9, ra[0], ra[1])
    z = [torch.empty(n, device="cuda"), torch.empty(n, device="cuda")]
    if residual:
        capi.check(capi.lib.tagi_batchnorm2d_fwd_res(
            capi.ptr(t["mu_w"]), capi.ptr(t["var_w"]), capi.ptr(mb), capi.ptr(vb), capi.ptr(t["mu_a"]),
            capi.ptr(t["var_a"]), capi.ptr(st[0]), capi.ptr(st[1]), capi.ptr(res[0]), capi.ptr(res[1]),
            int(bias), 1e-5, wihi, fi, B, capi.ptr(z[0]), capi.ptr(z[1]), stream))
    else:
        z = list(F.batchnorm2d_fwd(t["mu_w"], t["var_w"], mb, vb, t["mu_a"], t["var_a"], st[0], st[1],
                                   1e-5, wihi, fi, B))
    names = ("mu_s", "var_s", "mu_ra", "var_ra", "mu_z", "var_z")
    for name, a, b, c in zip(names, got, plain, list(st) + ra + z):
        assert torch.equal(a, c), name + " (fused merge)"
        assert torch.equal(b, c), name + " (merge as a launch of its own)"
    ref_s = oracle_lib.batchnorm2d_stats(d["mu_a"], d["var_a"], wihi, fi, B, 0.9, d["mu_ra"],
                                         d["var_ra"], 4)
    for name, a, r in zip(names[:4], got[:4], ref_s):
        assert_close(a.cpu().numpy(), r, name)


def test_batchnorm2d_backward_switches(oracle_lib):
    import cutagi_amd.functional as F
    import torch
    d = batchnorm_inputs(16, 8, 4, seed=1)
    t = _dev(d)
    a = (t["mu_w"], t["var_w"], t["var_b"], t["mu_a"], t["jcb"], t["mu_ra"], t["var_ra"], t["dmu"],
         t["dvar"], 1e-5, 16, 8, 4)
    out = F.batchnorm2d_bwd(*a, state_update=False)
    assert out[0] is None and out[2] is not None
    out = F.batchnorm2d_bwd(*a, param_update=False)
    assert out[2] is None and out[0] is not None
    torch.cuda.synchronize()


# (kernel, stride, pad, pad_type, wi, channels, B)
POOLS = [(4, -1, 0, 0, 4, 512, 8), (2, 2, 0, 0, 8, 3, 2), (3, 2, 1, 2, 8, 5, 3),
         (3, 1, 1, 1, 6, 2, 2), (2, 1, 0, 0, 5, 3, 1), (8, -1, 0, 0, 8, 7, 2), (3, 2, 1, 1, 9, 4, 2)]


@pytest.mark.parametrize("geom", POOLS)
def test_avgpool2d(oracle_lib, geom):
    import torch
    import cutagi_amd.functional as F
    from cutagi_amd import capi
    k, s, p, pt, wi, fo, B = geom
    idx = capi.avgpool2d_build_idx(k, s, wi, wi, p, pt)
    ref_idx = oracle_lib.avgpool2d_build_idx(k, s, wi, wi, p, pt)
    assert np.array_equal(idx["pool_idx"], ref_idx["pool_idx"])
    assert idx["overlap"] == ref_idx["overlap"] and (idx["w"], idx["h"]) == (ref_idx["w"], ref_idx["h"])
    assert np.array_equal(idx["z_ud_idx"], ref_idx["z_ud_idx"])
    wihi, woho = wi * wi, idx["wo"] * idx["ho"]
    d = pool_inputs(wihi, woho, fo, B, seed=sum(geom))
    t = _dev(d)
    pool = torch.from_numpy(idx["pool_idx"]).cuda()
    zud = torch.from_numpy(idx["z_ud_idx"]).cuda() if idx["overlap"] else None
    mu_z, var_z = F.avgpool2d_fwd(t["mu_a"], t["var_a"], pool, woho, wihi, k, B * fo * woho)
    ref = oracle_lib.avgpool2d_fwd(d["mu_a"], d["var_a"], idx["pool_idx"], woho, wihi, k,
                                   B * fo * woho, idx["overlap"], 4)
    assert_close(mu_z.cpu().numpy(), ref[0], "mu_z")
    assert_close(var_z.cpu().numpy(), ref[1], "var_z")
    om, ov = F.avgpool2d_bwd_dz(t["jcb"], t["dmu"], t["dvar"], zud, woho, wihi, k, idx["h"],
                                idx["wo"], idx["overlap"])
    ref = oracle_lib.avgpool2d_bwd_dz(d["jcb"], d["dmu"], d["dvar"], idx["z_ud_idx"], woho, wihi,
                                      k, idx["h"], idx["wo"], idx["overlap"], 4)
    assert_close(om.cpu().numpy(), ref[0], "delta_mu")
    assert_close(ov.cpu().numpy(), ref[1], "delta_var")


def test_shortcut_adds(oracle_lib):
    import torch
    import cutagi_amd.functional as F
    rng = np.random.default_rng(9)
    v = [rng.standard_normal(70001).astype(np.float32) for _ in range(5)]
    t = [torch.from_numpy(a).cuda() for a in v]
    mu, var = t[2].clone(), t[3].clone()
    F.add_shortcut(t[0], t[1], mu, var)
    ref = oracle_lib.add_shortcut(v[0], v[1], v[2], v[3])
    assert np.array_equal(mu.cpu().numpy(), ref[0]) and np.array_equal(var.cpu().numpy(), ref[1])
    mu, var = t[2].clone(), t[3].clone()
    F.add_shortcut_delta(t[0], t[1], t[4], mu, var)
    ref = oracle_lib.add_shortcut_delta(v[0], v[1], v[4], v[2], v[3])
    assert_close(mu.cpu().numpy(), ref[0], "mu", tol=1e-6)
    assert_close(var.cpu().numpy(), ref[1], "var", tol=1e-6)


def test_batchnorm2d_forward_with_residual(oracle_lib):
    """tagi_batchnorm2d_fwd_res = the layer's forward followed by the residual add."""
    import torch
    from cutagi_amd import capi
    from util import assert_close, batchnorm_inputs
    for (wihi, fi, B, bias) in [(16, 8, 4, True), (64, 3, 5, False), (1, 37, 6, True)]:
        d = batchnorm_inputs(wihi, fi, B, seed=wihi + fi + B)
        rng = np.random.default_rng(wihi * 7 + fi)
        n = B * fi * wihi
        res_mu = rng.standard_normal(n).astype(np.float32)
        res_var = rng.uniform(0.01, 0.5, n).astype(np.float32)
        mu_s = rng.standard_normal(fi).astype(np.float32)
        var_s = rng.uniform(0.5, 2.0, fi).astype(np.float32)
        mb, vb = (d["mu_b"], d["var_b"]) if bias else (None, None)
        z = oracle_lib.batchnorm2d_fwd(d["mu_w"], d["var_w"], mb, vb, d["mu_a"], d["var_a"], mu_s,
                                       var_s, 1e-5, wihi, fi, B, 2)
        want = oracle_lib.add_shortcut(res_mu, res_var, z[0].ravel(), z[1].ravel())
        t = lambda a: None if a is None else torch.from_numpy(a).cuda()
        dev = {k: t(v) for k, v in dict(mu_w=d["mu_w"], var_w=d["var_w"], mu_b=mb, var_b=vb,
                                        mu_a=d["mu_a"], var_a=d["var_a"], mu_s=mu_s, var_s=var_s,
                                        res_mu=res_mu, res_var=res_var).items()}
        mu_z, var_z = torch.empty(n, device="cuda"), torch.empty(n, device="cuda")
        capi.check(capi.lib.tagi_batchnorm2d_fwd_res(
            capi.ptr(dev["mu_w"]), capi.ptr(dev["var_w"]), capi.ptr(dev["mu_b"]),
            capi.ptr(dev["var_b"]), capi.ptr(dev["mu_a"]), capi.ptr(dev["var_a"]),
            capi.ptr(dev["mu_s"]), capi.ptr(dev["var_s"]), capi.ptr(dev["res_mu"]),
            capi.ptr(dev["res_var"]), int(bias), 1e-5, wihi, fi, B, capi.ptr(mu_z),
            capi.ptr(var_z), None))
        torch.cuda.synchronize()
        assert_close(mu_z.cpu().numpy(), want[0], "mu_z + residual")
        assert_close(var_z.cpu().numpy(), want[1], "var_z + residual", same_sign=True)
