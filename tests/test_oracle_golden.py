"""The CPU oracle against the golden vectors the compiled reference produced
(tests/golden/*.npz, written by tests/golden/make_golden.py): bit-exact."""
import os

import numpy as np
import pytest

from golden.make_golden import CONV_GEOMS, IDX_GEOMS, LINEAR_SHAPES, layer_vectors
from util import conv_inputs, linear_inputs

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def _load(name):
    return np.load(os.path.join(GOLD, name), allow_pickle=False)


def _same(a, b, what):
    assert a.shape == b.shape and np.array_equal(a, b, equal_nan=True), what


@pytest.mark.parametrize("geom", IDX_GEOMS)
def test_index_tables(oracle_lib, geom):
    g = _load("conv_idx.npz")
    k, s, p, pt, wi = geom
    idx = oracle_lib.conv2d_build_idx(k, s, wi, wi, p, pt, k * k * 12 + 1)
    tag = "idx_k%d_s%d_p%d_t%d_w%d" % geom
    for key in ("Fmwa_2", "FCzwa_1", "Szz_ud"):
        _same(idx[key], g[tag + "_" + key], key)
    assert [idx["w"], idx["h"], idx["wo"], idx["ho"]] == list(g[tag + "_wh"])


@pytest.mark.parametrize("geom", IDX_GEOMS)
def test_index_tables_product_builder(geom):
    """The library's own host-side builder (closed form) against the same vectors."""
    from cutagi_amd import capi
    g = _load("conv_idx.npz")
    k, s, p, pt, wi = geom
    idx = capi.conv2d_build_idx(k, s, wi, wi, p, pt, k * k * 12 + 1)
    tag = "idx_k%d_s%d_p%d_t%d_w%d" % geom
    for key in ("Fmwa_2", "FCzwa_1", "Szz_ud"):
        _same(idx[key], g[tag + "_" + key], key)
    assert [idx["w"], idx["h"], idx["wo"], idx["ho"]] == list(g[tag + "_wh"])


@pytest.mark.parametrize("shape", LINEAR_SHAPES)
def test_linear(oracle_lib, shape):
    g = _load("linear.npz")
    K, N, B = shape
    d = linear_inputs(K, N, B, seed=K * 7 + N * 3 + B, bias=True, jcb_random=True)
    tag = "lin_%d_%d_%d" % shape
    for th in (1, 3):
        t = tag + "_t%d" % th
        r = oracle_lib.linear_fwd(d["mu_w"], d["var_w"], d["mu_b"], d["var_b"], d["mu_a"],
                                  d["var_a"], th)
        _same(r[0], g[t + "_mu_z"], "mu_z"); _same(r[1], g[t + "_var_z"], "var_z")
        r = oracle_lib.linear_bwd_dz(d["mu_w"], d["jcb"], d["delta_mu"], d["delta_var"], th)
        _same(r[0], g[t + "_dz_mu"], "dz_mu"); _same(r[1], g[t + "_dz_var"], "dz_var")
        r = oracle_lib.linear_bwd_dw(d["var_w"], d["mu_a"], d["delta_mu"], d["delta_var"], th)
        _same(r[0], g[t + "_dw_mu"], "dw_mu"); _same(r[1], g[t + "_dw_var"], "dw_var")
        r = oracle_lib.linear_bwd_db(d["var_b"], d["delta_mu"], d["delta_var"], th)
        _same(r[0], g[t + "_db_mu"], "db_mu"); _same(r[1], g[t + "_db_var"], "db_var")
    r = oracle_lib.linear_fwd(d["mu_w"], d["var_w"], None, None, d["mu_a"], d["var_a"], 1)
    _same(r[0], g[tag + "_nobias_mu_z"], "mu_z nobias")
    _same(r[1], g[tag + "_nobias_var_z"], "var_z nobias")


@pytest.mark.parametrize("geom", CONV_GEOMS)
def test_conv(oracle_lib, geom):
    g = _load("conv.npz")
    k, s, p, pt, wi, fi, fo, B = geom
    idx = oracle_lib.conv2d_build_idx(k, s, wi, wi, p, pt, k * k * fi * fo + 1)
    wihi, woho = wi * wi, idx["wo"] * idx["ho"]
    d = conv_inputs(fi, fo, k, wihi, woho, B, seed=sum(geom), bias=True, jcb_random=True)
    tag = "conv_" + "_".join(map(str, geom))
    r = oracle_lib.conv2d_fwd(d["mu_w"], d["var_w"], d["mu_b"], d["var_b"], d["mu_a"], d["var_a"],
                              idx["Fmwa_2"], woho, fo, wihi, fi, k, B, 2)
    _same(r[0], g[tag + "_mu_z"], "mu_z"); _same(r[1], g[tag + "_var_z"], "var_z")
    r = oracle_lib.conv2d_bwd_dz(d["mu_w"], d["jcb"], d["delta_mu"], d["delta_var"],
                                 idx["FCzwa_1"], idx["Szz_ud"], woho, fo, wihi, fi, k, idx["h"],
                                 B, 2)
    _same(r[0], g[tag + "_dz_mu"], "dz_mu"); _same(r[1], g[tag + "_dz_var"], "dz_var")
    r = oracle_lib.conv2d_bwd_dw(d["var_w"], d["var_b"], d["mu_a"], d["delta_mu"], d["delta_var"],
                                 idx["Fmwa_2"], B, fo, woho, wihi, fi, k, 2)
    for got, key in zip(r, ("dw_mu", "dw_var", "db_mu", "db_var")):
        _same(got, g[tag + "_" + key], key)


def test_update_output_relu(oracle_lib):
    g = _load("misc.npz")
    for cap in (0.1, 2.0, 3.0):
        for w in (1, 0):
            m, v, c = oracle_lib.param_update(g["upd_mu"], g["upd_var"], g["upd_dmu"],
                                              g["upd_dvar"], cap, bool(w))
            t = "upd_cap%g_w%d" % (cap, w)
            _same(m, g[t + "_mu"], t); _same(v, g[t + "_var"], t)
            assert c == int(g[t + "_cnt"][0])
    assert int(g["upd_cap0.1_w1_cnt"][0]) > 0  # the fixture does exercise the clamp
    caps = [oracle_lib.cap_factor(b, 1.0) for b in (0, 1, 2, 255, 256, 4096)]
    assert np.array_equal(np.array(caps, np.float32), g["cap_factors"])
    z = np.zeros_like(g["out_mu_a"])
    r = oracle_lib.out_update_dense(g["out_mu_a"], g["out_var_a"], g["out_jcb"], g["out_obs"],
                                    g["out_var_obs"], z, z)
    _same(r[0], g["out_dense_dmu"], "dense dmu"); _same(r[1], g["out_dense_dvar"], "dense dvar")
    r = oracle_lib.out_update_indexed(g["out_mu_a"], g["out_var_a"], g["out_jcb"], g["out_y"],
                                      g["out_vy"], g["out_sel"], 11, 4, z, z)
    _same(r[0], g["out_idx_dmu"], "idx dmu"); _same(r[1], g["out_idx_dvar"], "idx dvar")
    from util import heteros_inputs
    d = heteros_inputs(257, seed=13)
    zz = np.zeros(2 * 257, np.float32)
    r = oracle_lib.out_update_heteros(d["mu_a"], d["var_a"], d["jcb"], d["obs"], zz, zz)
    _same(r[0], g["out_het_dmu"], "heteros dmu"); _same(r[1], g["out_het_dvar"], "heteros dvar")
    r = oracle_lib.relu_fwd(g["relu_mu_z"], g["relu_var_z"])
    _same(r[0], g["relu_mu_a"], "relu mu"); _same(r[1], g["relu_var_a"], "relu var")
    _same(r[2], g["relu_jcb"], "relu jcb")


def test_layer_vectors(oracle_lib):
    """MixtureReLU, BatchNorm2d, AvgPool2d (tables and arithmetic) and the
    residual adds: the oracle reproduces every stored reference output."""
    g = _load("layers.npz")
    mine = layer_vectors(oracle_lib)
    assert set(mine) == set(g.files)
    for key in g.files:
        _same(mine[key], g[key], key)
