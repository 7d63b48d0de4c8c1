"""The CPU oracle against the reference's own sources compiled in place
(oracle/_ref, built by `make -C oracle ref` where the reference tree is mounted):
bit-for-bit on seeded inputs, serial and threaded. Skipped where that library
does not exist."""
import numpy as np
import pytest

from util import batchnorm_inputs, conv_inputs, linear_inputs, pool_inputs


@pytest.fixture(scope="module")
def ref(ref_lib):
    if ref_lib is None:
        pytest.skip("oracle/_ref/libtagi_ref.so not built (no reference tree here)")
    return ref_lib


def _eq(a, b):
    return all(np.array_equal(x, y, equal_nan=True) for x, y in zip(a, b))


@pytest.mark.parametrize("K,N,B", [(5, 3, 2), (784, 128, 32), (129, 67, 9), (512, 256, 64),
                                   (1000, 11, 7), (64, 64, 1)])
@pytest.mark.parametrize("threads", [1, 4, 7])
def test_linear(oracle_lib, ref, K, N, B, threads):
    d = linear_inputs(K, N, B, seed=K + N + B + threads, jcb_random=True)
    for bias in (True, False):
        mb, vb = (d["mu_b"], d["var_b"]) if bias else (None, None)
        assert _eq(oracle_lib.linear_fwd(d["mu_w"], d["var_w"], mb, vb, d["mu_a"], d["var_a"], threads),
                   ref.linear_fwd(d["mu_w"], d["var_w"], mb, vb, d["mu_a"], d["var_a"], threads))
    a = (d["mu_w"], d["jcb"], d["delta_mu"], d["delta_var"], threads)
    assert _eq(oracle_lib.linear_bwd_dz(*a), ref.linear_bwd_dz(*a))
    a = (d["var_w"], d["mu_a"], d["delta_mu"], d["delta_var"], threads)
    assert _eq(oracle_lib.linear_bwd_dw(*a), ref.linear_bwd_dw(*a))
    a = (d["var_b"], d["delta_mu"], d["delta_var"], threads)
    assert _eq(oracle_lib.linear_bwd_db(*a), ref.linear_bwd_db(*a))


GEOMS = [(k, s, p, pt, wi) for k in (1, 2, 3, 4, 5) for s in (1, 2) for p in (0, 1, 2)
         for pt in (1, 2) for wi in (4, 7, 8, 12)]


def test_index_tables_sweep(oracle_lib, ref):
    """Every geometry both sides accept gives identical tables; both reject the
    same geometries (the reference throws where the stride does not divide)."""
    from cutagi_amd import capi
    checked = 0
    for g in GEOMS:
        k, s, p, pt, wi = g
        if k > wi:
            continue
        try:
            b = ref.conv2d_build_idx(k, s, wi, wi, p, pt, 1234)
        except ValueError:
            with pytest.raises(ValueError):
                oracle_lib.conv2d_build_idx(k, s, wi, wi, p, pt, 1234)
            continue
        a = oracle_lib.conv2d_build_idx(k, s, wi, wi, p, pt, 1234)
        c = capi.conv2d_build_idx(k, s, wi, wi, p, pt, 1234)
        for key in ("Fmwa_2", "FCzwa_1", "Szz_ud", "w", "h", "wo", "ho"):
            assert np.array_equal(a[key], b[key]), (g, key)
            assert np.array_equal(c[key], b[key]), (g, key, "product builder")
        checked += 1
    assert checked > 100


@pytest.mark.parametrize("geom", [(3, 1, 1, 1, 8, 3, 4, 2), (3, 2, 1, 2, 8, 4, 6, 2),
                                  (2, 2, 0, 1, 8, 4, 4, 3), (5, 1, 2, 1, 9, 2, 3, 1),
                                  (3, 1, 1, 1, 16, 8, 8, 2), (4, 2, 1, 1, 10, 3, 5, 2)])
@pytest.mark.parametrize("threads", [1, 3])
def test_conv(oracle_lib, ref, geom, threads):
    k, s, p, pt, wi, fi, fo, B = geom
    idx = ref.conv2d_build_idx(k, s, wi, wi, p, pt, k * k * fi * fo + 1)
    wihi, woho = wi * wi, idx["wo"] * idx["ho"]
    d = conv_inputs(fi, fo, k, wihi, woho, B, seed=sum(geom) + threads, bias=True, jcb_random=True)
    a = (d["mu_w"], d["var_w"], d["mu_b"], d["var_b"], d["mu_a"], d["var_a"], idx["Fmwa_2"], woho,
         fo, wihi, fi, k, B, threads)
    assert _eq(oracle_lib.conv2d_fwd(*a), ref.conv2d_fwd(*a))
    a = (d["mu_w"], d["jcb"], d["delta_mu"], d["delta_var"], idx["FCzwa_1"], idx["Szz_ud"], woho,
         fo, wihi, fi, k, idx["h"], B, threads)
    assert _eq(oracle_lib.conv2d_bwd_dz(*a), ref.conv2d_bwd_dz(*a))
    a = (d["var_w"], d["var_b"], d["mu_a"], d["delta_mu"], d["delta_var"], idx["Fmwa_2"], B, fo,
         woho, wihi, fi, k, threads)
    assert _eq(oracle_lib.conv2d_bwd_dw(*a), ref.conv2d_bwd_dw(*a))


def test_update_output_relu(oracle_lib, ref):
    rng = np.random.default_rng(3)
    n = 20000
    mu = rng.normal(0, 1, n).astype(np.float32)
    var = rng.uniform(1e-5, 1, n).astype(np.float32)
    dmu = rng.normal(0, 1, n).astype(np.float32)
    dvar = rng.normal(0, 0.5, n).astype(np.float32)
    for cap in (0.1, 2.0, 3.0):
        for w in (True, False):
            a = oracle_lib.param_update(mu, var, dmu, dvar, cap, w)
            b = ref.param_update(mu, var, dmu, dvar, cap, w)
            assert np.array_equal(a[0], b[0]) and np.array_equal(a[1], b[1]) and a[2] == b[2]
    for bs in (-3, 0, 1, 2, 100, 255, 256, 100000):
        assert oracle_lib.cap_factor(bs, 1.5) == ref.cap_factor(bs, 1.5)
    m = rng.normal(0, 1, 999).astype(np.float32)
    v = rng.uniform(0, 1, 999).astype(np.float32)
    assert _eq(oracle_lib.relu_fwd(m, v), ref.relu_fwd(m, v))


def test_out_update_heteros(oracle_lib, ref):
    from util import heteros_inputs
    for n, seed in ((64, 1), (1001, 2)):
        d = heteros_inputs(n, seed)
        z = np.full(2 * n, 7.0, np.float32)   # every entry is written
        a = oracle_lib.out_update_heteros(d["mu_a"], d["var_a"], d["jcb"], d["obs"], z, z)
        b = ref.out_update_heteros(d["mu_a"], d["var_a"], d["jcb"], d["obs"], z, z)
        assert np.array_equal(a[0], b[0], equal_nan=True) and np.array_equal(a[1], b[1], equal_nan=True)
        assert a[0][6] == 0 and a[0][7] == 0 and a[0][16] == 0 and a[0][10] == 0


# ---- layers around the hot path: MixtureReLU, BatchNorm2d, AvgPool2d, residual adds ----

@pytest.mark.parametrize("threads", [1, 4])
def test_mixture_relu(oracle_lib, ref, threads):
    rng = np.random.default_rng(11 + threads)
    mu_z = (rng.standard_normal(4099) * 3).astype(np.float32)
    var_z = rng.uniform(1e-4, 4.0, 4099).astype(np.float32)
    assert _eq(oracle_lib.mixture_relu_fwd(mu_z, var_z, threads),
               ref.mixture_relu_fwd(mu_z, var_z, threads))


@pytest.mark.parametrize("wihi,fi,B", [(16, 8, 4), (64, 3, 5), (1, 37, 6), (9, 5, 2)])
@pytest.mark.parametrize("threads", [1, 3])
def test_batchnorm2d(oracle_lib, ref, wihi, fi, B, threads):
    d = batchnorm_inputs(wihi, fi, B, seed=wihi + fi + B + threads)
    for momentum in (0.0, 0.9):
        a = (d["mu_a"], d["var_a"], wihi, fi, B, momentum, d["mu_ra"], d["var_ra"], threads)
        so, sr = oracle_lib.batchnorm2d_stats(*a), ref.batchnorm2d_stats(*a)
        assert _eq(so, sr)
    mu_s, var_s = so[0], so[1]
    for bias in (True, False):
        mb, vb = (d["mu_b"], d["var_b"]) if bias else (None, None)
        a = (d["mu_w"], d["var_w"], mb, vb, d["mu_a"], d["var_a"], mu_s, var_s, 1e-5, wihi, fi, B,
             threads)
        assert _eq(oracle_lib.batchnorm2d_fwd(*a), ref.batchnorm2d_fwd(*a))
        a = (d["var_w"], vb, d["mu_a"], mu_s, var_s, d["dmu"], d["dvar"], 1e-5, wihi, fi, B, threads)
        x, y = oracle_lib.batchnorm2d_bwd_dw(*a), ref.batchnorm2d_bwd_dw(*a)
        assert _eq(x[:2], y[:2]) and (not bias or _eq(x[2:], y[2:]))
    a = (d["mu_w"], d["jcb"], var_s, d["dmu"], d["dvar"], 1e-5, wihi, fi, B, threads)
    assert _eq(oracle_lib.batchnorm2d_bwd_dz(*a), ref.batchnorm2d_bwd_dz(*a))


# (kernel, stride, pad, pad_type, wi): global pooling with the default stride -1,
# non-overlapping windows, overlapping windows with and without padding
POOLS = [(4, -1, 0, 0, 4), (2, 2, 0, 0, 8), (3, 2, 1, 2, 8), (3, 1, 1, 1, 6), (2, 1, 0, 0, 5),
         (8, -1, 0, 0, 8), (3, 2, 1, 1, 9)]


@pytest.mark.parametrize("geom", POOLS)
@pytest.mark.parametrize("threads", [1, 4])
def test_avgpool2d(oracle_lib, ref, geom, threads):
    k, s, p, pt, wi = geom
    a, b = oracle_lib.avgpool2d_build_idx(k, s, wi, wi, p, pt), ref.avgpool2d_build_idx(k, s, wi, wi, p, pt)
    assert np.array_equal(a["pool_idx"], b["pool_idx"])
    assert a["overlap"] == b["overlap"] and (a["wo"], a["ho"]) == (b["wo"], b["ho"])
    if a["overlap"]:
        assert np.array_equal(a["z_ud_idx"], b["z_ud_idx"]) and (a["w"], a["h"]) == (b["w"], b["h"])
    fo, B = 3, 2
    wihi, woho = wi * wi, a["wo"] * a["ho"]
    d = pool_inputs(wihi, woho, fo, B, seed=sum(geom) + threads)
    mu_a, var_a, jcb, dmu, dvar = d["mu_a"], d["var_a"], d["jcb"], d["dmu"], d["dvar"]
    args = (mu_a, var_a, a["pool_idx"], woho, wihi, k, B * fo * woho, a["overlap"], threads)
    assert _eq(oracle_lib.avgpool2d_fwd(*args), ref.avgpool2d_fwd(*args))
    args = (jcb, dmu, dvar, a["z_ud_idx"], woho, wihi, k, a["h"], a["wo"], a["overlap"], threads)
    assert _eq(oracle_lib.avgpool2d_bwd_dz(*args), ref.avgpool2d_bwd_dz(*args))


def test_shortcut_adds(oracle_lib, ref):
    rng = np.random.default_rng(5)
    v = [rng.standard_normal(1001).astype(np.float32) for _ in range(5)]
    assert _eq(oracle_lib.add_shortcut(v[0], v[1], v[2], v[3]), ref.add_shortcut(v[0], v[1], v[2], v[3]))
    assert _eq(oracle_lib.add_shortcut_delta(v[0], v[1], v[4], v[2], v[3]),
               ref.add_shortcut_delta(v[0], v[1], v[4], v[2], v[3]))


@pytest.mark.parametrize("n_classes", [2, 3, 5, 8, 10, 17, 33, 100, 1000])
def test_hierarchical_softmax_encoding(ref, n_classes):
    """cutagi_amd.resnet.hrc_softmax (what a training script feeds the output
    updater) against the reference's class_to_obs."""
    from cutagi_amd.resnet import hrc_softmax
    obs, idx, n_obs, length = hrc_softmax(n_classes)
    r_obs, r_idx, r_n, r_len = ref.class_to_obs(n_classes)
    assert (n_obs, length) == (r_n, r_len)
    assert np.array_equal(obs, r_obs) and np.array_equal(idx, r_idx)
