"""Writes the golden vectors under tests/golden/ from the reference's own CPU
sources, compiled in place by oracle/Makefile (`make -C oracle ref`, which needs
the reference tree). The fixtures are data only: seeded inputs and the outputs
the compiled reference produced for them.

    python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
sys.path.insert(0, os.path.dirname(HERE))

import oracle  # noqa: E402
import full_size_cases as fs  # noqa: E402
from model_cases import CASES, REF_THREADS, case_inputs, sample_index  # noqa: E402
from util import (batchnorm_inputs, conv_inputs, heteros_inputs, linear_inputs,  # noqa: E402
                  pool_inputs)

# (kernel, stride, pad, pad_type, wi): every geometry of the Conv2d and ResNet-18
# configurations plus a few odd ones
IDX_GEOMS = [(3, 1, 1, 1, 32), (3, 1, 1, 1, 16), (3, 1, 1, 1, 8), (3, 1, 1, 1, 4),
             (3, 2, 1, 2, 32), (3, 2, 1, 2, 16), (3, 2, 1, 2, 8),
             (2, 2, 0, 1, 32), (2, 2, 0, 1, 16), (2, 2, 0, 1, 8),
             (1, 1, 0, 1, 4), (5, 1, 2, 1, 9), (4, 2, 1, 1, 10), (3, 1, 0, 1, 6),
             (5, 2, 2, 1, 7), (3, 1, 2, 2, 6), (2, 1, 1, 2, 5), (3, 2, 1, 1, 7), (1, 2, 0, 1, 7)]
LINEAR_SHAPES = [(5, 3, 2), (7, 4, 1), (33, 17, 9), (784, 32, 8), (128, 11, 32), (96, 64, 16)]
CONV_GEOMS = [(3, 1, 1, 1, 8, 3, 4, 2), (3, 2, 1, 2, 8, 4, 6, 2), (2, 2, 0, 1, 8, 4, 4, 3),
              (5, 1, 2, 1, 9, 2, 3, 1)]
# (wihi, fi, B) of the batch-norm vectors; (kernel, stride, pad, pad_type, wi, fo, B)
# of the pooling vectors (global pooling with the default stride -1 is the
# ResNet-18 head)
BN_SHAPES = [(16, 8, 4), (64, 3, 5), (1, 37, 6), (9, 5, 2)]
POOL_GEOMS = [(4, -1, 0, 0, 4, 8, 3), (2, 2, 0, 0, 8, 3, 2), (3, 2, 1, 2, 8, 3, 2),
              (3, 1, 1, 1, 6, 2, 2), (2, 1, 0, 0, 5, 3, 1)]


def layer_vectors(lib):
    """Outputs of MixtureReLU, BatchNorm2d, AvgPool2d and the residual adds."""
    out = {}
    rng = np.random.default_rng(23)
    mz = (rng.standard_normal(2048) * 3).astype(np.float32)
    vz = rng.uniform(1e-4, 4.0, 2048).astype(np.float32)
    out["mrelu_mu_z"], out["mrelu_var_z"] = mz, vz
    out["mrelu_mu_a"], out["mrelu_var_a"], out["mrelu_jcb"] = lib.mixture_relu_fwd(mz, vz, 1)
    for (wihi, fi, B) in BN_SHAPES:
        d = batchnorm_inputs(wihi, fi, B, seed=wihi * 5 + fi * 3 + B)
        t = "bn_%d_%d_%d" % (wihi, fi, B)
        for mom in (0.0, 0.9):
            r = lib.batchnorm2d_stats(d["mu_a"], d["var_a"], wihi, fi, B, mom, d["mu_ra"],
                                      d["var_ra"], 2)
            for key, a in zip(("mu_s", "var_s", "mu_ra", "var_ra"), r):
                out["%s_m%g_%s" % (t, mom, key)] = a
        mu_s, var_s = r[0], r[1]
        out[t + "_mu_z"], out[t + "_var_z"] = lib.batchnorm2d_fwd(
            d["mu_w"], d["var_w"], d["mu_b"], d["var_b"], d["mu_a"], d["var_a"], mu_s, var_s,
            1e-5, wihi, fi, B, 2)
        out[t + "_nobias_mu_z"], out[t + "_nobias_var_z"] = lib.batchnorm2d_fwd(
            d["mu_w"], d["var_w"], None, None, d["mu_a"], d["var_a"], mu_s, var_s, 1e-5, wihi,
            fi, B, 1)
        out[t + "_dz_mu"], out[t + "_dz_var"] = lib.batchnorm2d_bwd_dz(
            d["mu_w"], d["jcb"], var_s, d["dmu"], d["dvar"], 1e-5, wihi, fi, B, 2)
        r = lib.batchnorm2d_bwd_dw(d["var_w"], d["var_b"], d["mu_a"], mu_s, var_s, d["dmu"],
                                   d["dvar"], 1e-5, wihi, fi, B, 2)
        out[t + "_dw_mu"], out[t + "_dw_var"], out[t + "_db_mu"], out[t + "_db_var"] = r
    for g in POOL_GEOMS:
        k, s, p, pt, wi, fo, B = g
        idx = lib.avgpool2d_build_idx(k, s, wi, wi, p, pt)
        wihi, woho = wi * wi, idx["wo"] * idx["ho"]
        d = pool_inputs(wihi, woho, fo, B, seed=sum(g))
        t = "pool_" + "_".join(map(str, g))
        out[t + "_pool_idx"] = idx["pool_idx"]
        out[t + "_z_ud_idx"] = idx["z_ud_idx"] if idx["overlap"] else np.zeros(0, np.int32)
        out[t + "_meta"] = np.array([idx["w"] if idx["overlap"] else 0,
                                     idx["h"] if idx["overlap"] else 0, idx["wo"], idx["ho"],
                                     int(idx["overlap"])], np.int32)
        out[t + "_mu_z"], out[t + "_var_z"] = lib.avgpool2d_fwd(
            d["mu_a"], d["var_a"], idx["pool_idx"], woho, wihi, k, B * fo * woho, idx["overlap"], 2)
        out[t + "_dz_mu"], out[t + "_dz_var"] = lib.avgpool2d_bwd_dz(
            d["jcb"], d["dmu"], d["dvar"], idx["z_ud_idx"], woho, wihi, k, idx["h"], idx["wo"],
            idx["overlap"], 2)
    v = [rng.standard_normal(777).astype(np.float32) for _ in range(5)]
    for i, a in enumerate(v):
        out["sc_in%d" % i] = a
    out["sc_mu"], out["sc_var"] = lib.add_shortcut(v[0], v[1], v[2], v[3])
    out["scd_mu"], out["scd_var"] = lib.add_shortcut_delta(v[0], v[1], v[4], v[2], v[3])
    return out


def model_vectors(ref):
    """Training steps of whole networks through the reference's own Sequential,
    LayerBlock, ResNetBlock and OutputUpdater (oracle/ref_model.cpp): outputs of every
    forward, input innovations where asked for, every parameter after every step (a
    strided sample plus float64 sums for the large MLP) and the clamped-variance
    counters. Inputs are regenerated from the seeds in tests/model_cases.py."""
    out = {}
    for name, c in CASES.items():
        inp = case_inputs(name)
        r = ref.model_run(c["spec"], inp["params"], inp["mu_x"], inp["var_x"], inp["y"],
                          inp["var_y"], inp["sel"], c["B"], c["update"], c.get("n_enc", 0),
                          c.get("input_state_update", False), c.get("eval_forward", False),
                          8 if c.get("big") else REF_THREADS)
        assert r["n_out"] == inp["n_out"]
        assert np.all(np.isfinite(r["params"])) and np.all(np.isfinite(r["out_mu"])), name
        out[name + "_out_mu"], out[name + "_out_var"] = r["out_mu"], r["out_var"]
        if c.get("input_state_update", False):
            out[name + "_in_dmu"], out[name + "_in_dvar"] = r["in_dmu"], r["in_dvar"]
        idx = sample_index(r["params"].shape[1])
        out[name + "_params"] = r["params"][:, idx]
        out[name + "_params_sum"] = r["params"].astype(np.float64).sum(axis=1)
        out[name + "_neg"] = r["neg"]
    return out


def full_size_vectors(ref, threads=8):
    """The benchmark configurations at their full sizes through the reference's CPU
    kernels (seconds each with 8 threads): sampled entries and sums of every output."""
    out = {}
    for name in fs.LINEAR:
        d = fs.linear_inputs(name)
        r = ref.linear_fwd(d["mu_w"], d["var_w"], d["mu_b"], d["var_b"], d["mu_a"], d["var_a"],
                           threads)
        r += ref.linear_bwd_dz(d["mu_w"], d["jcb"], d["delta_mu"], d["delta_var"], threads)
        r += ref.linear_bwd_dw(d["var_w"], d["mu_a"], d["delta_mu"], d["delta_var"], threads)
        r += ref.linear_bwd_db(d["var_b"], d["delta_mu"], d["delta_var"], threads)
        out.update(fs.summarize(name, dict(zip(fs.LINEAR_OUTPUTS, r))))
        print(name, "done", flush=True)
    for name, g in fs.CONV.items():
        fi, fo, k, wi, B = g["fi"], g["fo"], g["k"], g["wi"], g["B"]
        pix = wi * wi
        idx = ref.conv2d_build_idx(k, 1, wi, wi, 1, 1, k * k * fi * fo + 1)
        d = fs.conv_inputs(name)
        r = ref.conv2d_fwd(d["mu_w"], d["var_w"], None, None, d["mu_a"], d["var_a"],
                           idx["Fmwa_2"], pix, fo, pix, fi, k, B, threads)
        r += ref.conv2d_bwd_dz(d["mu_w"], d["jcb"], d["delta_mu"], d["delta_var"], idx["FCzwa_1"],
                               idx["Szz_ud"], pix, fo, pix, fi, k, idx["h"], B, threads)
        r += ref.conv2d_bwd_dw(d["var_w"], None, d["mu_a"], d["delta_mu"], d["delta_var"],
                               idx["Fmwa_2"], B, fo, pix, pix, fi, k, threads)[:2]
        out.update(fs.summarize(name, dict(zip(fs.CONV_OUTPUTS, r))))
        print(name, "done", flush=True)
    return out


def main():
    ref = oracle.load_ref()
    if ref is None:
        raise SystemExit("oracle/_ref/libtagi_ref.so is missing: run `make -C oracle ref`")
    out = {}
    for g in IDX_GEOMS:
        k, s, p, pt, wi = g
        idx = ref.conv2d_build_idx(k, s, wi, wi, p, pt, k * k * 12 + 1)
        tag = "idx_k%d_s%d_p%d_t%d_w%d" % g
        for key in ("Fmwa_2", "FCzwa_1", "Szz_ud"):
            out[tag + "_" + key] = idx[key]
        out[tag + "_wh"] = np.array([idx["w"], idx["h"], idx["wo"], idx["ho"]], np.int32)
    np.savez_compressed(os.path.join(HERE, "conv_idx.npz"), **out)

    out = {}
    for (K, N, B) in LINEAR_SHAPES:
        d = linear_inputs(K, N, B, seed=K * 7 + N * 3 + B, bias=True, jcb_random=True)
        tag = "lin_%d_%d_%d" % (K, N, B)
        for th in (1, 3):
            t = tag + "_t%d" % th
            out[t + "_mu_z"], out[t + "_var_z"] = ref.linear_fwd(
                d["mu_w"], d["var_w"], d["mu_b"], d["var_b"], d["mu_a"], d["var_a"], th)
            out[t + "_dz_mu"], out[t + "_dz_var"] = ref.linear_bwd_dz(
                d["mu_w"], d["jcb"], d["delta_mu"], d["delta_var"], th)
            out[t + "_dw_mu"], out[t + "_dw_var"] = ref.linear_bwd_dw(
                d["var_w"], d["mu_a"], d["delta_mu"], d["delta_var"], th)
            out[t + "_db_mu"], out[t + "_db_var"] = ref.linear_bwd_db(
                d["var_b"], d["delta_mu"], d["delta_var"], th)
        out[tag + "_nobias_mu_z"], out[tag + "_nobias_var_z"] = ref.linear_fwd(
            d["mu_w"], d["var_w"], None, None, d["mu_a"], d["var_a"], 1)
    np.savez_compressed(os.path.join(HERE, "linear.npz"), **out)

    out = {}
    for g in CONV_GEOMS:
        k, s, p, pt, wi, fi, fo, B = g
        idx = ref.conv2d_build_idx(k, s, wi, wi, p, pt, k * k * fi * fo + 1)
        wihi, woho = wi * wi, idx["wo"] * idx["ho"]
        d = conv_inputs(fi, fo, k, wihi, woho, B, seed=sum(g), bias=True, jcb_random=True)
        tag = "conv_" + "_".join(map(str, g))
        out[tag + "_mu_z"], out[tag + "_var_z"] = ref.conv2d_fwd(
            d["mu_w"], d["var_w"], d["mu_b"], d["var_b"], d["mu_a"], d["var_a"], idx["Fmwa_2"],
            woho, fo, wihi, fi, k, B, 2)
        out[tag + "_dz_mu"], out[tag + "_dz_var"] = ref.conv2d_bwd_dz(
            d["mu_w"], d["jcb"], d["delta_mu"], d["delta_var"], idx["FCzwa_1"], idx["Szz_ud"],
            woho, fo, wihi, fi, k, idx["h"], B, 2)
        r = ref.conv2d_bwd_dw(d["var_w"], d["var_b"], d["mu_a"], d["delta_mu"], d["delta_var"],
                              idx["Fmwa_2"], B, fo, woho, wihi, fi, k, 2)
        out[tag + "_dw_mu"], out[tag + "_dw_var"], out[tag + "_db_mu"], out[tag + "_db_var"] = r
    np.savez_compressed(os.path.join(HERE, "conv.npz"), **out)

    out = {}
    rng = np.random.default_rng(11)
    n = 4096
    mu = rng.normal(0, 1, n).astype(np.float32)
    var = rng.uniform(1e-4, 1, n).astype(np.float32)
    dmu = rng.normal(0, 1, n).astype(np.float32)
    dvar = rng.normal(0, 0.5, n).astype(np.float32)
    dmu[::7] = 0
    out["upd_mu"], out["upd_var"], out["upd_dmu"], out["upd_dvar"] = mu, var, dmu, dvar
    for cap in (0.1, 2.0, 3.0):
        for w in (1, 0):
            m, v, c = ref.param_update(mu, var, dmu, dvar, cap, bool(w))
            t = "upd_cap%g_w%d" % (cap, w)
            out[t + "_mu"], out[t + "_var"], out[t + "_cnt"] = m, v, np.array([c], np.int32)
    out["cap_factors"] = np.array([ref.cap_factor(b, 1.0) for b in (0, 1, 2, 255, 256, 4096)],
                                  np.float32)
    B, n_obs, n_enc = 8, 11, 4
    mu_a = rng.normal(0, 1, B * n_obs).astype(np.float32)
    var_a = rng.uniform(0.1, 1, B * n_obs).astype(np.float32)
    jcb = rng.uniform(0.5, 1, B * n_obs).astype(np.float32)
    obs = rng.normal(0, 1, B * n_obs).astype(np.float32)
    obs[3] = np.nan
    var_obs = np.ones(B * n_obs, np.float32)
    var_obs[6] = -var_a[6]
    z = np.zeros(B * n_obs, np.float32)
    sel = np.concatenate([rng.choice(n_obs, n_enc, replace=False) + 1
                          for _ in range(B)]).astype(np.int32)
    y = rng.normal(0, 1, B * n_enc).astype(np.float32)
    vy = np.ones(B * n_enc, np.float32)
    for name, a in dict(mu_a=mu_a, var_a=var_a, jcb=jcb, obs=obs, var_obs=var_obs, sel=sel, y=y,
                        vy=vy).items():
        out["out_" + name] = a
    out["out_dense_dmu"], out["out_dense_dvar"] = ref.out_update_dense(mu_a, var_a, jcb, obs,
                                                                      var_obs, z, z)
    out["out_idx_dmu"], out["out_idx_dvar"] = ref.out_update_indexed(mu_a, var_a, jcb, y, vy, sel,
                                                                    n_obs, n_enc, z, z)
    d = heteros_inputs(257, seed=13)
    zz = np.zeros(2 * 257, np.float32)
    out["out_het_dmu"], out["out_het_dvar"] = ref.out_update_heteros(d["mu_a"], d["var_a"],
                                                                    d["jcb"], d["obs"], zz, zz)
    mz = rng.normal(0, 1, 512).astype(np.float32)
    mz[::9] = 0
    vz = rng.uniform(0.1, 1, 512).astype(np.float32)
    out["relu_mu_z"], out["relu_var_z"] = mz, vz
    out["relu_mu_a"], out["relu_var_a"], out["relu_jcb"] = ref.relu_fwd(mz, vz)
    np.savez_compressed(os.path.join(HERE, "misc.npz"), **out)
    np.savez_compressed(os.path.join(HERE, "layers.npz"), **layer_vectors(ref))
    np.savez_compressed(os.path.join(HERE, "models.npz"), **model_vectors(ref))
    np.savez_compressed(os.path.join(HERE, "full_size.npz"), **full_size_vectors(ref))
    for f in ("conv_idx.npz", "linear.npz", "conv.npz", "misc.npz", "layers.npz", "models.npz",
              "full_size.npz"):
        print(f, os.path.getsize(os.path.join(HERE, f)))


if __name__ == "__main__":
    main()
