"""The benchmark configurations at their full sizes (Linear 4096^2 batch 256, Linear
8192^2 batch 8, Conv2d 3x3 64->64 on 32x32 maps batch 128): the CPU oracle would
take too long there, so the HIP path is held against what the mathematics fixes --
the closed forms of the layer evaluated in float64 with library routines (torch
matmul / unfold on the same GPU) -- and against size-independent properties:
variances >= 0, variance innovations <= 0, linearity in the incoming innovations,
and the deterministic layer (zero variances) reducing to a plain product.
Tolerance: the parity gate of the small-shape tests (util.TOL = 1e-4)."""
import numpy as np
import pytest

from util import TOL

pytestmark = pytest.mark.gpu


def _err(x, ref):
    """max |x - ref| / max(|ref|, rms(ref)), on the device, in float64."""
    import torch
    x = x.double().reshape(-1)
    ref = ref.double().reshape(-1)
    rms = torch.sqrt(torch.mean(ref * ref)).clamp_min(1e-30)
    return float(torch.max((x - ref).abs() / torch.maximum(ref.abs(), rms)))


def _check(x, ref, what):
    import torch
    assert bool(torch.isfinite(x).all()), what + ": non-finite values"
    e = _err(x, ref)
    assert e <= TOL, "%s: rel err %.3e > %.1e" % (what, e, TOL)


def _linear_inputs(K, N, B, seed):
    import torch
    g = torch.Generator(device="cuda")
    g.manual_seed(seed)
    r = lambda *s: torch.randn(*s, device="cuda", generator=g)
    u = lambda *s: torch.rand(*s, device="cuda", generator=g)
    return dict(mu_w=r(N, K) * K ** -0.5, var_w=(0.5 + u(N, K)) / K, mu_b=r(N) * 0.5,
                var_b=(0.5 + u(N)) / K, mu_a=r(B, K), var_a=0.01 + 0.09 * u(B, K),
                jcb=u(B, K), delta_mu=0.1 * r(B, N), delta_var=-1e-3 * u(B, N))


# (the third shape: the 16-wide streaming kernels at the full weight size)
@pytest.mark.parametrize("K,N,B", [(4096, 4096, 256), (8192, 8192, 8), (8192, 8192, 16)])
def test_linear_full_size_against_float64_closed_forms(K, N, B):
    import torch
    import cutagi_amd.functional as F
    t = _linear_inputs(K, N, B, seed=K + B)
    d = {k: v.double() for k, v in t.items()}
    mu_z, var_z = F.linear_fwd(t["mu_w"], t["var_w"], t["mu_b"], t["var_b"], t["mu_a"], t["var_a"])
    _check(mu_z, d["mu_a"] @ d["mu_w"].T + d["mu_b"], "mu_z")
    _check(var_z, (d["mu_a"] ** 2 + d["var_a"]) @ d["var_w"].T + d["var_a"] @ (d["mu_w"] ** 2).T
           + d["var_b"], "var_z")
    assert float(var_z.min()) >= 0.0

    out = F.linear_bwd(t["mu_w"], t["var_w"], t["var_b"], t["mu_a"], t["jcb"], t["delta_mu"],
                       t["delta_var"])
    _check(out[0], (d["delta_mu"] @ d["mu_w"]) * d["jcb"], "delta_mu_z")
    _check(out[1], (d["delta_var"] @ d["mu_w"] ** 2) * d["jcb"] ** 2, "delta_var_z")
    _check(out[2], (d["delta_mu"].T @ d["mu_a"]) * d["var_w"], "delta_mu_w")
    _check(out[3], (d["delta_var"].T @ d["mu_a"] ** 2) * d["var_w"] ** 2, "delta_var_w")
    _check(out[4], d["delta_mu"].sum(0) * d["var_b"], "delta_mu_b")
    _check(out[5], d["delta_var"].sum(0) * d["var_b"] ** 2, "delta_var_b")
    for i in (1, 3, 5):
        assert float(out[i].max()) <= 0.0

    # a deterministic layer: zero variances in, the bias variance out, plain product
    zero_w, zero_a = torch.zeros_like(t["var_w"]), torch.zeros_like(t["var_a"])
    mu0, var0 = F.linear_fwd(t["mu_w"], zero_w, t["mu_b"], t["var_b"], t["mu_a"], zero_a)
    assert torch.equal(mu0, mu_z)
    _check(var0, d["var_b"].expand(B, N), "var_z of the deterministic layer")
    # linearity in the incoming innovations: doubling them doubles every output
    out2 = F.linear_bwd(t["mu_w"], t["var_w"], t["var_b"], t["mu_a"], t["jcb"], 2 * t["delta_mu"],
                        2 * t["delta_var"])
    for a, b in zip(out, out2):
        assert torch.equal(2 * a, b)


# Large batches (the tiled kernels far above the 256 rows of the benchmark shape; the
# second shape also has a ragged reduction): float64 closed forms for every entry, and
# the CPU oracle on a sample -- whole batch rows for the forward and the state backward
# (rows of a batch do not interact), whole output units for the weight / bias backward
# (a unit's innovations depend on its own column of the incoming innovations only).
@pytest.mark.parametrize("K,N,B", [(2048, 1024, 1024), (1000, 512, 4096)])
def test_linear_large_batch_against_float64_and_sampled_oracle(oracle_lib, K, N, B):
    import torch
    import cutagi_amd.functional as F
    from util import SAME_SIGN, assert_close
    t = _linear_inputs(K, N, B, seed=K + B)
    d = {k: v.double() for k, v in t.items()}
    mu_z, var_z = F.linear_fwd(t["mu_w"], t["var_w"], t["mu_b"], t["var_b"], t["mu_a"], t["var_a"])
    _check(mu_z, d["mu_a"] @ d["mu_w"].T + d["mu_b"], "mu_z")
    _check(var_z, (d["mu_a"] ** 2 + d["var_a"]) @ d["var_w"].T + d["var_a"] @ (d["mu_w"] ** 2).T
           + d["var_b"], "var_z")
    assert float(var_z.min()) >= 0.0
    out = F.linear_bwd(t["mu_w"], t["var_w"], t["var_b"], t["mu_a"], t["jcb"], t["delta_mu"],
                       t["delta_var"])
    _check(out[0], (d["delta_mu"] @ d["mu_w"]) * d["jcb"], "delta_mu_z")
    _check(out[1], (d["delta_var"] @ d["mu_w"] ** 2) * d["jcb"] ** 2, "delta_var_z")
    _check(out[2], (d["delta_mu"].T @ d["mu_a"]) * d["var_w"], "delta_mu_w")
    _check(out[3], (d["delta_var"].T @ d["mu_a"] ** 2) * d["var_w"] ** 2, "delta_var_w")
    _check(out[4], d["delta_mu"].sum(0) * d["var_b"], "delta_mu_b")
    _check(out[5], d["delta_var"].sum(0) * d["var_b"] ** 2, "delta_var_b")

    h = {k: v.cpu().numpy() for k, v in t.items()}
    rng = np.random.default_rng(B)
    rows = np.sort(rng.choice(B, 6, replace=False))       # batch rows
    units = np.sort(rng.choice(N, 6, replace=False))      # output units
    ref = oracle_lib.linear_fwd(h["mu_w"], h["var_w"], h["mu_b"], h["var_b"],
                                np.ascontiguousarray(h["mu_a"][rows]),
                                np.ascontiguousarray(h["var_a"][rows]), threads=4)
    assert_close(mu_z.cpu().numpy()[rows], ref[0], "mu_z rows vs oracle")
    assert_close(var_z.cpu().numpy()[rows], ref[1], "var_z rows vs oracle", same_sign=True)
    ref = oracle_lib.linear_bwd_dz(h["mu_w"], np.ascontiguousarray(h["jcb"][rows]),
                                   np.ascontiguousarray(h["delta_mu"][rows]),
                                   np.ascontiguousarray(h["delta_var"][rows]), threads=4)
    assert_close(out[0].cpu().numpy()[rows], ref[0], "delta_mu_z rows vs oracle")
    assert_close(out[1].cpu().numpy()[rows], ref[1], "delta_var_z rows vs oracle", same_sign=True)
    dmu_u = np.ascontiguousarray(h["delta_mu"][:, units])
    dvar_u = np.ascontiguousarray(h["delta_var"][:, units])
    ref = oracle_lib.linear_bwd_dw(np.ascontiguousarray(h["var_w"][units]), h["mu_a"], dmu_u,
                                   dvar_u, threads=4)
    assert_close(out[2].cpu().numpy()[units], ref[0], "delta_mu_w units vs oracle")
    assert_close(out[3].cpu().numpy()[units], ref[1], "delta_var_w units vs oracle", same_sign=True)
    ref = oracle_lib.linear_bwd_db(np.ascontiguousarray(h["var_b"][units]), dmu_u, dvar_u)
    assert_close(out[4].cpu().numpy()[units], ref[0], "delta_mu_b units vs oracle")
    assert_close(out[5].cpu().numpy()[units], ref[1], "delta_var_b units vs oracle", same_sign=True)


def test_conv2d_full_size_against_float64_closed_forms():
    """Config 4 through the regular-stencil kernels (the library's own tables)."""
    import torch
    import torch.nn.functional as TF
    import cutagi_amd.functional as F
    from cutagi_amd import capi
    fi = fo = 64
    k, wi, B = 3, 32, 128
    pix = wi * wi
    idx = capi.conv2d_build_idx(k, 1, wi, wi, 1, 1, k * k * fi * fo + 1)
    ti = {n: torch.from_numpy(idx[n]).cuda() for n in ("Fmwa_2", "FCzwa_1", "Szz_ud")}
    g = torch.Generator(device="cuda")
    g.manual_seed(4)
    r = lambda *s: torch.randn(*s, device="cuda", generator=g)
    u = lambda *s: torch.rand(*s, device="cuda", generator=g)
    R = k * k * fi
    mu_w, var_w = r(fo, R) * R ** -0.5, (0.5 + u(fo, R)) / R
    mu_a, var_a, jcb = r(B, fi, pix), 0.01 + 0.09 * u(B, fi, pix), u(B, fi, pix)
    dmu, dvar = 0.1 * r(B, fo, pix), -1e-3 * u(B, fo, pix)

    def cols(x):  # [B][c][pix] -> im2col [B][c*9][pix] in float64
        return TF.unfold(x.double().reshape(B, -1, wi, wi), k, padding=1)

    def chunks(fn, n=8):  # keep the float64 im2col matrices small
        return torch.cat([fn(slice(i * B // n, (i + 1) * B // n)) for i in range(n)])

    W, V = mu_w.double(), var_w.double()
    mu_z, var_z = F.conv2d_fwd(mu_w.reshape(-1), var_w.reshape(-1), None, None, mu_a.reshape(-1),
                               var_a.reshape(-1), ti["Fmwa_2"], pix, fo, pix, fi, k, B)
    _check(mu_z, chunks(lambda s: W @ cols(mu_a)[s]), "mu_z")
    _check(var_z, chunks(lambda s: V @ cols(mu_a ** 2 + var_a)[s] + W ** 2 @ cols(var_a)[s]),
           "var_z")
    assert float(var_z.min()) >= 0.0

    # state backward = the adjoint of im2col applied to W^T delta
    def fold(c):
        return TF.fold(c, (wi, wi), k, padding=1).reshape(-1, fi, pix)

    dz = F.conv2d_bwd_dz(mu_w.reshape(-1), jcb.reshape(-1), dmu.reshape(-1), dvar.reshape(-1),
                         ti["FCzwa_1"], ti["Szz_ud"], pix, fo, pix, fi, k, idx["h"], B)
    J = jcb.double()
    _check(dz[0], chunks(lambda s: fold(W.T @ dmu.double()[s]) * J[s]), "delta_mu_z")
    _check(dz[1], chunks(lambda s: fold((W ** 2).T @ dvar.double()[s]) * J[s] ** 2), "delta_var_z")
    assert float(dz[1].max()) <= 0.0

    dw = F.conv2d_bwd_dw(var_w.reshape(-1), None, mu_a.reshape(-1), dmu.reshape(-1),
                         dvar.reshape(-1), ti["Fmwa_2"], B, fo, pix, pix, fi, k)
    sum_mu = sum((dmu.double()[s] @ cols(mu_a)[s].transpose(1, 2)).sum(0)
                 for s in (slice(i * 16, (i + 1) * 16) for i in range(B // 16)))
    sum_var = sum((dvar.double()[s] @ cols(mu_a ** 2)[s].transpose(1, 2)).sum(0)
                  for s in (slice(i * 16, (i + 1) * 16) for i in range(B // 16)))
    _check(dw[0], sum_mu * V, "delta_mu_w")
    _check(dw[1], sum_var * V ** 2, "delta_var_w")
    assert float(dw[1].max()) <= 0.0


# ---- against the reference's own fp32 CPU results at the full sizes ---------------------
# tests/golden/full_size.npz holds, for every output tensor of the three Linear shapes
# and the Conv2d configuration, the values the compiled reference produced at a seeded
# sample of entries plus float64 sums over the whole tensor (tests/golden/make_golden.py;
# the inputs regenerate from tests/full_size_cases.py on any machine). Three checks per
# tensor: the 1e-4 gate against the reference's values (elementwise as well for the
# same-signed tensors), the whole-tensor sum, and the distance to the float64 closed
# form, which may not exceed twice the reference's own distance to it.

def _against_reference(name, outputs, truth, gold):
    import full_size_cases as fs
    from util import SAME_SIGN, assert_close, rel_err
    report = []
    for tensor, got in outputs.items():
        flat = got.reshape(-1)
        idx = fs.sample_of(name, tensor, flat.numel())
        import torch
        sample = flat[torch.from_numpy(idx).cuda()].cpu().numpy()
        ref = gold["%s_%s" % (name, tensor)]
        assert_close(sample, ref, "%s %s vs reference CPU" % (name, tensor),
                     same_sign=tensor in SAME_SIGN)
        ref_sum, ref_abs = gold["%s_%s_sums" % (name, tensor)]
        got_sum = float(flat.double().sum())
        assert abs(got_sum - ref_sum) <= 1e-4 * ref_abs, (name, tensor, got_sum, ref_sum)
        e_gpu, e_ref = rel_err(sample, truth[tensor]), rel_err(ref, truth[tensor])
        report.append("%-12s gpu-vs-f64 %.2e  reference-vs-f64 %.2e" % (tensor, e_gpu, e_ref))
        assert e_gpu <= max(2 * e_ref, 2e-6), "%s %s: %.3e from float64, the reference %.3e" % (
            name, tensor, e_gpu, e_ref)
    print("\n" + name + "\n  " + "\n  ".join(report))


@pytest.mark.parametrize("name", ["linear_4096_b256", "linear_8192_b8", "linear_8192_b16"])
def test_linear_full_size_against_reference_cpu(name):
    import os
    import torch
    import cutagi_amd.functional as F
    import full_size_cases as fs
    gold = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden",
                                "full_size.npz"), allow_pickle=False)
    d = fs.linear_inputs(name)
    t = {k: torch.from_numpy(v).cuda() for k, v in d.items()}
    out = list(F.linear_fwd(t["mu_w"], t["var_w"], t["mu_b"], t["var_b"], t["mu_a"], t["var_a"]))
    out += list(F.linear_bwd(t["mu_w"], t["var_w"], t["var_b"], t["mu_a"], t["jcb"],
                             t["delta_mu"], t["delta_var"]))
    torch.cuda.synchronize()
    _against_reference(name, dict(zip(fs.LINEAR_OUTPUTS, out)), fs.linear_float64(name, d), gold)


def test_conv2d_full_size_against_reference_cpu():
    import os
    import torch
    import cutagi_amd.functional as F
    import full_size_cases as fs
    from cutagi_amd import capi
    name = "conv_3x3_64_32_b128"
    gold = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden",
                                "full_size.npz"), allow_pickle=False)
    g = fs.CONV[name]
    fi, fo, k, wi, B = g["fi"], g["fo"], g["k"], g["wi"], g["B"]
    pix = wi * wi
    idx = capi.conv2d_build_idx(k, 1, wi, wi, 1, 1, k * k * fi * fo + 1)
    ti = {n: torch.from_numpy(idx[n]).cuda() for n in ("Fmwa_2", "FCzwa_1", "Szz_ud")}
    d = fs.conv_inputs(name)
    t = {key: torch.from_numpy(v).cuda() for key, v in d.items()}
    out = list(F.conv2d_fwd(t["mu_w"], t["var_w"], None, None, t["mu_a"], t["var_a"],
                            ti["Fmwa_2"], pix, fo, pix, fi, k, B))
    out += list(F.conv2d_bwd_dz(t["mu_w"], t["jcb"], t["delta_mu"], t["delta_var"], ti["FCzwa_1"],
                                ti["Szz_ud"], pix, fo, pix, fi, k, idx["h"], B))
    out += list(F.conv2d_bwd_dw(t["var_w"], None, t["mu_a"], t["delta_mu"], t["delta_var"],
                                ti["Fmwa_2"], B, fo, pix, pix, fi, k))[:2]
    torch.cuda.synchronize()
    _against_reference(name, dict(zip(fs.CONV_OUTPUTS, out)), fs.conv_float64(name, d), gold)
