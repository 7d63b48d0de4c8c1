"""What the mathematics fixes, independent of any implementation: the oracle
against fp64 closed forms (numpy matmul; torch conv2d / conv_transpose2d / unfold
in float64), invariants, and a brute-force im2col check of the index tables. A
dropped term, a transposed operand or a wrong index fails one of these."""
import numpy as np
import pytest

from util import assert_close, conv_inputs, linear_inputs, rel_err


@pytest.mark.parametrize("K,N,B", [(37, 19, 5), (128, 64, 16), (300, 11, 32)])
def test_linear_closed_forms(oracle_lib, K, N, B):
    d = linear_inputs(K, N, B, seed=K, jcb_random=True)
    D = {k: (None if v is None else v.astype(np.float64)) for k, v in d.items()}
    mu_z, var_z = oracle_lib.linear_fwd(d["mu_w"], d["var_w"], d["mu_b"], d["var_b"], d["mu_a"],
                                        d["var_a"])
    assert_close(mu_z, D["mu_a"] @ D["mu_w"].T + D["mu_b"], "mu_z", 1e-5)
    assert_close(var_z, (D["var_a"] + D["mu_a"] ** 2) @ D["var_w"].T
                 + D["var_a"] @ (D["mu_w"] ** 2).T + D["var_b"], "var_z", 1e-5)
    dz = oracle_lib.linear_bwd_dz(d["mu_w"], d["jcb"], d["delta_mu"], d["delta_var"])
    assert_close(dz[0], (D["delta_mu"] @ D["mu_w"]) * D["jcb"], "dz mu", 1e-5)
    assert_close(dz[1], (D["delta_var"] @ D["mu_w"] ** 2) * D["jcb"] ** 2, "dz var", 1e-5)
    dw = oracle_lib.linear_bwd_dw(d["var_w"], d["mu_a"], d["delta_mu"], d["delta_var"])
    assert_close(dw[0], (D["delta_mu"].T @ D["mu_a"]) * D["var_w"], "dw mu", 1e-5)
    assert_close(dw[1], (D["delta_var"].T @ D["mu_a"] ** 2) * D["var_w"] ** 2, "dw var", 1e-5)
    db = oracle_lib.linear_bwd_db(d["var_b"], d["delta_mu"], d["delta_var"])
    assert_close(db[0], D["delta_mu"].sum(0) * D["var_b"], "db mu", 1e-5)
    assert_close(db[1], D["delta_var"].sum(0) * D["var_b"] ** 2, "db var", 1e-5)


def test_linear_invariants(oracle_lib):
    d = linear_inputs(64, 32, 8, seed=1, jcb_random=True)
    z = np.zeros_like
    # deterministic weights and inputs: var_z == var_b, mu_z a plain product
    mu_z, var_z = oracle_lib.linear_fwd(d["mu_w"], z(d["var_w"]), d["mu_b"], d["var_b"], d["mu_a"],
                                        z(d["var_a"]))
    assert np.array_equal(var_z, np.broadcast_to(d["var_b"], var_z.shape))
    assert (oracle_lib.linear_fwd(d["mu_w"], d["var_w"], None, None, d["mu_a"], d["var_a"])[1] >= 0).all()
    # zero Jacobian kills the state innovation; linearity in delta_mu
    dz = oracle_lib.linear_bwd_dz(d["mu_w"], z(d["jcb"]), d["delta_mu"], d["delta_var"])
    assert not dz[0].any() and not dz[1].any()
    a = oracle_lib.linear_bwd_dz(d["mu_w"], d["jcb"], d["delta_mu"], d["delta_var"])[0]
    b = oracle_lib.linear_bwd_dz(d["mu_w"], d["jcb"], 2 * d["delta_mu"], d["delta_var"])[0]
    np.testing.assert_allclose(b, 2 * a, rtol=1e-6)
    # delta_var <= 0 keeps every variance innovation <= 0
    for r in (oracle_lib.linear_bwd_dz(d["mu_w"], d["jcb"], d["delta_mu"], d["delta_var"])[1],
              oracle_lib.linear_bwd_dw(d["var_w"], d["mu_a"], d["delta_mu"], d["delta_var"])[1],
              oracle_lib.linear_bwd_db(d["var_b"], d["delta_mu"], d["delta_var"])[1]):
        assert (r <= 0).all()


GEOMS = [(3, 1, 1, 1, 8), (3, 2, 1, 2, 8), (2, 2, 0, 1, 8), (1, 1, 0, 1, 5), (5, 1, 2, 1, 9),
         (3, 1, 0, 1, 6), (4, 2, 1, 1, 10), (3, 1, 2, 2, 6), (2, 1, 1, 2, 5)]


def _torch_pad(p, pt):
    # F.pad order: (left, right, top, bottom); type 2 pads right and bottom only
    return (p, p, p, p) if pt == 1 else (0, p, 0, p)


@pytest.mark.parametrize("geom", GEOMS)
def test_index_tables_are_im2col(oracle_lib, geom):
    """Fmwa_2 equals the unfold (im2col) of an image of pixel ids; FCzwa_1 / Szz_ud
    list, per input pixel, exactly the (tap, output pixel) pairs that read it."""
    import torch
    import torch.nn.functional as F
    k, s, p, pt, wi = geom
    idx = oracle_lib.conv2d_build_idx(k, s, wi, wi, p, pt, 999)
    img = torch.arange(1, wi * wi + 1, dtype=torch.float64).reshape(1, 1, wi, wi)
    padded = F.pad(img, _torch_pad(p, pt), value=-1.0) if p > 0 else img
    cols = F.unfold(padded, k, stride=s)[0]                  # [k*k, wo*ho]
    assert np.array_equal(idx["Fmwa_2"].reshape(-1, k * k), cols.T.numpy().astype(np.int32))
    w, h = idx["w"], idx["h"]
    zw = idx["FCzwa_1"].reshape(w, h)
    zud = idx["Szz_ud"].reshape(h, w)
    fm = idx["Fmwa_2"].reshape(-1, k * k)
    pixels = sorted(set(fm[fm > 0].tolist()))
    assert len(pixels) == w
    for c, px in enumerate(pixels):
        pairs = [(t + 1, o + 1) for o in range(fm.shape[0]) for t in range(k * k) if fm[o, t] == px]
        got = [(int(zw[c, j]), int(zud[j, c])) for j in range(h) if zud[j, c] > -1]
        assert got == pairs
        assert all(zw[c, j] == 999 for j in range(len(pairs), h))


@pytest.mark.parametrize("geom", [(3, 1, 1, 1, 8), (3, 2, 1, 2, 8), (2, 2, 0, 1, 8),
                                  (5, 1, 2, 1, 9), (3, 1, 0, 1, 6)])
def test_conv_closed_forms(oracle_lib, geom):
    import torch
    import torch.nn.functional as F
    k, s, p, pt, wi = geom
    fi, fo, B = 3, 4, 2
    idx = oracle_lib.conv2d_build_idx(k, s, wi, wi, p, pt, k * k * fi * fo + 1)
    wo = idx["wo"]
    wihi, woho = wi * wi, wo * wo
    d = conv_inputs(fi, fo, k, wihi, woho, B, seed=sum(geom), bias=True, jcb_random=True)
    T = lambda a, *shape: torch.from_numpy(a.astype(np.float64)).reshape(*shape)
    mw, vw = T(d["mu_w"], fo, fi, k, k), T(d["var_w"], fo, fi, k, k)
    ma, va = T(d["mu_a"], B, fi, wi, wi), T(d["var_a"], B, fi, wi, wi)
    pad = lambda x: F.pad(x, _torch_pad(p, pt)) if p > 0 else x
    conv = lambda x, w: F.conv2d(pad(x), w, stride=s)
    mu_z, var_z = oracle_lib.conv2d_fwd(d["mu_w"], d["var_w"], d["mu_b"], d["var_b"], d["mu_a"],
                                        d["var_a"], idx["Fmwa_2"], woho, fo, wihi, fi, k, B)
    bias = lambda b: T(b, 1, fo, 1, 1)
    assert_close(mu_z, (conv(ma, mw) + bias(d["mu_b"])).numpy(), "mu_z", 1e-5)
    assert_close(var_z, (conv(va + ma ** 2, vw) + conv(va, mw ** 2) + bias(d["var_b"])).numpy(),
                 "var_z", 1e-5)
    # backward through autograd of the linear maps: d/dx <delta, conv(x, w)>
    dm, dv = T(d["delta_mu"], B, fo, wo, wo), T(d["delta_var"], B, fo, wo, wo)
    jc = T(d["jcb"], B, fi, wi, wi)

    def vjp_x(w, delta):
        x = torch.zeros(B, fi, wi, wi, dtype=torch.float64, requires_grad=True)
        (conv(x, w) * delta).sum().backward()
        return x.grad

    def vjp_w(x, delta):
        w = torch.zeros(fo, fi, k, k, dtype=torch.float64, requires_grad=True)
        (conv(x, w) * delta).sum().backward()
        return w.grad

    dz = oracle_lib.conv2d_bwd_dz(d["mu_w"], d["jcb"], d["delta_mu"], d["delta_var"],
                                  idx["FCzwa_1"], idx["Szz_ud"], woho, fo, wihi, fi, k, idx["h"], B)
    assert_close(dz[0], (vjp_x(mw, dm) * jc).numpy(), "dz mu", 1e-5)
    assert_close(dz[1], (vjp_x(mw ** 2, dv) * jc ** 2).numpy(), "dz var", 1e-5)
    dw = oracle_lib.conv2d_bwd_dw(d["var_w"], d["var_b"], d["mu_a"], d["delta_mu"], d["delta_var"],
                                  idx["Fmwa_2"], B, fo, woho, wihi, fi, k)
    assert_close(dw[0], (vjp_w(ma, dm) * vw).numpy(), "dw mu", 1e-5)
    assert_close(dw[1], (vjp_w(ma ** 2, dv) * vw ** 2).numpy(), "dw var", 1e-5)
    vb = T(d["var_b"], fo)
    assert_close(dw[2], (dm.sum((0, 2, 3)) * vb).numpy(), "db mu", 1e-5)
    assert_close(dw[3], (dv.sum((0, 2, 3)) * vb ** 2).numpy(), "db var", 1e-5)


def test_param_update_special_cases(oracle_lib):
    f = np.float32
    mu = np.array([1, 1, 1, 1, 1], f)
    var = np.array([0.04, 0.04, 0.04, 0.04, 1e-4], f)
    dmu = np.array([0, 100, -100, 0.01, 0], f)
    dvar = np.array([0, 100, -100, -0.01, -1], f)
    m, v, c = oracle_lib.param_update(mu, var, dmu, dvar, 2.0)
    bar = np.sqrt(f(0.04)) / f(2.0)                       # 0.1
    np.testing.assert_allclose(m, [1, 1 + bar, 1 - bar, 1.01, 1], rtol=1e-6)
    # zero delta: unchanged; huge delta: moves exactly sqrt(var)/cap; a variance
    # pushed to <= 0 becomes 1e-5 and is counted
    np.testing.assert_allclose(v, [0.04, 0.04 + bar, 1e-5, 0.03, 1e-5], rtol=1e-5)
    assert c == 2
    assert oracle_lib.param_update(mu, var, dmu, dvar, 2.0, weights=False)[2] == 0
    assert [oracle_lib.cap_factor(b, 7.0) for b in (0, 1, 2, 255, 256)] == \
        [7.0, pytest.approx(0.1), 2.0, 2.0, 3.0]


def test_output_updater_closed_form(oracle_lib):
    rng = np.random.default_rng(2)
    n = 64
    mu_a, var_a = rng.normal(0, 1, n).astype(np.float32), rng.uniform(0.1, 1, n).astype(np.float32)
    jcb = rng.uniform(0.5, 1, n).astype(np.float32)
    y, vy = rng.normal(0, 1, n).astype(np.float32), np.full(n, 0.5, np.float32)
    z = np.zeros(n, np.float32)
    dm, dv = oracle_lib.out_update_dense(mu_a, var_a, jcb, y, vy, z, z)
    g = jcb.astype(np.float64) / (var_a.astype(np.float64) + 0.5)
    np.testing.assert_allclose(dm, g * (y.astype(np.float64) - mu_a), rtol=1e-5)
    np.testing.assert_allclose(dv, -g * jcb, rtol=1e-5)
    # indexed: only the selected (1-based) positions of each sample are written
    B, n_obs, n_enc = 4, 16, 3
    sel = np.array([1, 5, 16, 2, 3, 4, 16, 15, 14, 7, 8, 9], np.int32)
    yy, vv = y[:B * n_enc].copy(), vy[:B * n_enc].copy()
    dm, dv = oracle_lib.out_update_indexed(mu_a, var_a, jcb, yy, vv, sel, n_obs, n_enc, z, z)
    pos = [sel[c] - 1 + (c // n_enc) * n_obs for c in range(B * n_enc)]
    assert sorted(np.nonzero(dm)[0].tolist()) == sorted(pos)
    for c, i in enumerate(pos):
        gi = float(jcb[i]) / (float(var_a[i]) + 0.5)
        assert dm[i] == pytest.approx(gi * (float(yy[c]) - float(mu_a[i])), rel=1e-5)
        assert dv[i] == pytest.approx(-gi * float(jcb[i]), rel=1e-5)


# ---- layers around the hot path ----------------------------------------------------

def test_mixture_relu_is_rectified_gaussian(oracle_lib):
    """Moments of max(z, 0) for z ~ N(mu, var): E = mu*Phi + sd*phi,
    E[a^2] = (mu^2 + var)*Phi + mu*sd*phi; the Jacobian is Phi."""
    from scipy.special import ndtr
    rng = np.random.default_rng(3)
    mu = (rng.standard_normal(5000) * 2).astype(np.float32)
    var = rng.uniform(0.05, 3.0, 5000).astype(np.float32)
    mu_a, var_a, jcb = oracle_lib.mixture_relu_fwd(mu, var, 2)
    m, v = mu.astype(np.float64), var.astype(np.float64)
    sd = np.sqrt(v)
    al = m / sd
    Phi, phi = ndtr(al), np.exp(-0.5 * al * al) / np.sqrt(2 * np.pi)
    e1 = m * Phi + sd * phi
    e2 = (m * m + v) * Phi + m * sd * phi
    assert rel_err(jcb, Phi) < 1e-5
    assert rel_err(mu_a, np.maximum(e1, 1e-6)) < 1e-5
    assert rel_err(var_a, np.maximum(e2 - e1 * e1, 1e-6)) < 2e-4  # cancellation in fp32
    assert mu_a.min() >= 1e-6 and var_a.min() >= 1e-6


@pytest.mark.parametrize("wihi,fi,B", [(16, 6, 5), (1, 19, 7), (49, 3, 2)])
def test_batchnorm2d_closed_forms(oracle_lib, wihi, fi, B):
    from util import batchnorm_inputs
    d = batchnorm_inputs(wihi, fi, B, seed=wihi + fi)
    x = d["mu_a"].astype(np.float64).reshape(B, fi, wihi)
    vx = d["var_a"].astype(np.float64).reshape(B, fi, wihi)
    n = B * wihi
    mean = x.mean(axis=(0, 2))
    var = (((x - mean[None, :, None]) ** 2).sum(axis=(0, 2)) + vx.sum(axis=(0, 2))) / (n - 1)
    mu_s, var_s, mu_ra, var_ra = oracle_lib.batchnorm2d_stats(
        d["mu_a"], d["var_a"], wihi, fi, B, 0.9, d["mu_ra"], d["var_ra"], 2)
    assert rel_err(mu_s, mean) < 1e-5 and rel_err(var_s, var) < 1e-5
    assert rel_err(mu_ra, 0.9 * d["mu_ra"] + 0.1 * mean) < 1e-5
    assert rel_err(var_ra, 0.9 * d["var_ra"] + 0.1 * var) < 1e-5
    # momentum 0 replaces the running averages by the batch statistics
    r0 = oracle_lib.batchnorm2d_stats(d["mu_a"], d["var_a"], wihi, fi, B, 0.0, d["mu_ra"],
                                      d["var_ra"], 1)
    assert np.array_equal(r0[2], r0[0]) and np.array_equal(r0[3], r0[1])

    c = lambda a: a.astype(np.float64)[None, :, None]
    inv = 1.0 / np.sqrt(c(var_s) + 1e-5)
    xt = x - c(mu_s)
    mu_z = inv * xt * c(d["mu_w"]) + c(d["mu_b"])
    var_z = inv ** 2 * (vx * (c(d["mu_w"]) ** 2 + c(d["var_w"])) + c(d["var_w"]) * xt ** 2) + c(d["var_b"])
    got = oracle_lib.batchnorm2d_fwd(d["mu_w"], d["var_w"], d["mu_b"], d["var_b"], d["mu_a"],
                                     d["var_a"], mu_s, var_s, 1e-5, wihi, fi, B, 3)
    assert rel_err(got[0], mu_z) < 1e-5 and rel_err(got[1], var_z) < 1e-5
    assert got[1].min() >= 0

    dm = d["dmu"].astype(np.float64).reshape(B, fi, wihi)
    dv = d["dvar"].astype(np.float64).reshape(B, fi, wihi)
    j = d["jcb"].astype(np.float64).reshape(B, fi, wihi)
    t = inv * c(d["mu_w"]) * j
    got = oracle_lib.batchnorm2d_bwd_dz(d["mu_w"], d["jcb"], var_s, d["dmu"], d["dvar"], 1e-5,
                                        wihi, fi, B, 2)
    assert rel_err(got[0], t * dm) < 1e-5 and rel_err(got[1], t * t * dv) < 1e-5
    tw = inv * xt * c(d["var_w"])
    got = oracle_lib.batchnorm2d_bwd_dw(d["var_w"], d["var_b"], d["mu_a"], mu_s, var_s, d["dmu"],
                                        d["dvar"], 1e-5, wihi, fi, B, 2)
    assert rel_err(got[0], (tw * dm).sum(axis=(0, 2))) < 1e-4
    assert rel_err(got[1], (tw * tw * dv).sum(axis=(0, 2))) < 1e-4
    vb = d["var_b"].astype(np.float64)
    assert rel_err(got[2], vb * dm.sum(axis=(0, 2))) < 1e-4
    assert rel_err(got[3], vb * vb * dv.sum(axis=(0, 2))) < 1e-4
    # the mean path is what torch's batch norm computes with these statistics
    import torch
    ref = torch.nn.functional.batch_norm(
        torch.from_numpy(x.reshape(B, fi, wihi, 1)), torch.from_numpy(c(mu_s).ravel()),
        torch.from_numpy(c(var_s).ravel()), torch.from_numpy(c(d["mu_w"]).ravel()),
        torch.from_numpy(c(d["mu_b"]).ravel()), training=False, eps=1e-5)
    assert rel_err(mu_z, ref.numpy()) < 1e-9


@pytest.mark.parametrize("geom", [(4, -1, 0, 0, 4), (2, 2, 0, 0, 8), (3, 2, 1, 1, 9),
                                  (3, 1, 1, 1, 6), (2, 1, 0, 0, 5)])
def test_avgpool2d_is_torch_avg_pool(oracle_lib, geom):
    """Mean: torch's avg_pool2d with the padding counted in the divisor;
    variance: the same window sum divided by k^4; backward: its adjoint times
    the Jacobian (squared for the variance)."""
    import torch
    from util import pool_inputs
    k, s, p, pt, wi = geom
    idx = oracle_lib.avgpool2d_build_idx(k, s, wi, wi, p, pt)
    fo, B = 3, 2
    wihi, woho = wi * wi, idx["wo"] * idx["ho"]
    d = pool_inputs(wihi, woho, fo, B, seed=sum(geom))
    stride = k if s < 0 else s
    x = torch.from_numpy(d["mu_a"].astype(np.float64)).reshape(B, fo, wi, wi).requires_grad_(True)
    v = torch.from_numpy(d["var_a"].astype(np.float64)).reshape(B, fo, wi, wi).requires_grad_(True)
    pool = lambda a: torch.nn.functional.avg_pool2d(a, k, stride, p, count_include_pad=True)
    ym, yv = pool(x), pool(v) / (k * k)
    got = oracle_lib.avgpool2d_fwd(d["mu_a"], d["var_a"], idx["pool_idx"], woho, wihi, k,
                                   B * fo * woho, idx["overlap"], 2)
    assert rel_err(got[0], ym.detach().numpy()) < 1e-5
    assert rel_err(got[1], yv.detach().numpy()) < 1e-5
    dm = torch.from_numpy(d["dmu"].astype(np.float64)).reshape(ym.shape)
    dv = torch.from_numpy(d["dvar"].astype(np.float64)).reshape(ym.shape)
    gm, = torch.autograd.grad(ym, x, dm)
    gv, = torch.autograd.grad(yv, v, dv)   # adjoint of (window sum)/k^4, times k^2 below
    j = d["jcb"].astype(np.float64).reshape(B, fo, wi, wi)
    got = oracle_lib.avgpool2d_bwd_dz(d["jcb"], d["dmu"], d["dvar"], idx["z_ud_idx"], woho, wihi,
                                      k, idx["h"], idx["wo"], idx["overlap"], 2)
    assert rel_err(got[0], gm.numpy() * j) < 1e-5
    assert rel_err(got[1], gv.numpy() * j * j) < 1e-5
