"""Parity of the small kernels (update, output updater, ReLU, state bookkeeping)."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _t(a):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


@pytest.mark.parametrize("cap", [0.1, 2.0, 3.0])
def test_param_update(oracle_lib, cap):
    import torch
    import cutagi_amd.functional as F
    rng = np.random.default_rng(int(cap * 10))
    n = 100003
    mu = rng.normal(0, 1, n).astype(np.float32)
    var = rng.uniform(1e-4, 1, n).astype(np.float32)
    dmu = rng.normal(0, 1, n).astype(np.float32)
    dvar = rng.normal(0, 0.5, n).astype(np.float32)
    dmu[::7] = 0.0
    dvar[::11] = 0.0
    ref_mu, ref_var, ref_cnt = oracle_lib.param_update(mu, var, dmu, dvar, cap)
    t_mu, t_var = _t(mu), _t(var)
    cnt = torch.zeros(1, dtype=torch.int32, device="cuda")
    F.param_update(_t(dmu), _t(dvar), cap, t_mu, t_var, cnt)
    # identical up to the last bit of sqrt/divide; the clamp decisions must agree
    np.testing.assert_allclose(t_mu.cpu().numpy(), ref_mu, rtol=1e-6, atol=1e-7)
    np.testing.assert_allclose(t_var.cpu().numpy(), ref_var, rtol=1e-6, atol=1e-7)
    assert int(cnt.item()) == ref_cnt
    assert ref_cnt > 0 or cap > 1.0
    assert float(t_var.min()) > 0.0


@pytest.mark.parametrize("nw,nb", [(100003, 257), (4096, 0), (5, 3)])
def test_layer_update_one_launch(oracle_lib, nw, nb):
    """Weights and biases in one launch: the same numbers as the two separate
    updates of the oracle; the counter of the call's slot holds the clamped weight
    variances, the other slot is reset."""
    import torch
    import cutagi_amd.functional as F
    rng = np.random.default_rng(nw + nb)
    cap = 2.0
    def params(n):
        return (rng.normal(0, 1, n).astype(np.float32), rng.uniform(1e-4, 1, n).astype(np.float32),
                rng.normal(0, 1, n).astype(np.float32), rng.normal(0, 0.5, n).astype(np.float32))
    mu_w, var_w, dmu_w, dvar_w = params(nw)
    mu_b, var_b, dmu_b, dvar_b = params(nb)
    ref_mw, ref_vw, ref_cnt = oracle_lib.param_update(mu_w, var_w, dmu_w, dvar_w, cap)
    t_mw, t_vw = _t(mu_w), _t(var_w)
    cnt = torch.tensor([7, 9], dtype=torch.int32, device="cuda")   # stale values in both slots
    if nb:
        ref_mb, ref_vb, _ = oracle_lib.param_update(mu_b, var_b, dmu_b, dvar_b, cap)
        t_mb, t_vb = _t(mu_b), _t(var_b)
        cnt[1] = 0                                                  # what the previous call left
        F.layer_update(_t(dmu_w), _t(dvar_w), t_mw, t_vw, _t(dmu_b), _t(dvar_b), t_mb, t_vb, cap,
                       cnt, slot=1)
        np.testing.assert_allclose(t_mb.cpu().numpy(), ref_mb, rtol=1e-6, atol=1e-7)
        np.testing.assert_allclose(t_vb.cpu().numpy(), ref_vb, rtol=1e-6, atol=1e-7)
        assert cnt.tolist() == [0, ref_cnt]
    else:
        cnt[0] = 0
        F.layer_update(_t(dmu_w), _t(dvar_w), t_mw, t_vw, None, None, None, None, cap, cnt, slot=0)
        assert cnt.tolist() == [ref_cnt, 0]
    np.testing.assert_allclose(t_mw.cpu().numpy(), ref_mw, rtol=1e-6, atol=1e-7)
    np.testing.assert_allclose(t_vw.cpu().numpy(), ref_vw, rtol=1e-6, atol=1e-7)
    assert float(t_vw.min()) > 0.0


def test_out_update_dense_and_indexed(oracle_lib):
    import torch
    import cutagi_amd.functional as F
    rng = np.random.default_rng(5)
    B, n_obs, n_enc = 32, 11, 4
    mu_a = rng.normal(0, 1, B * n_obs).astype(np.float32)
    var_a = rng.uniform(0.1, 1, B * n_obs).astype(np.float32)
    jcb = np.ones(B * n_obs, np.float32)
    # dense
    obs = rng.normal(0, 1, B * n_obs).astype(np.float32)
    obs[5] = np.nan
    var_obs = np.ones(B * n_obs, np.float32)
    var_obs[9] = -var_a[9]  # division by zero -> inf -> zeroed
    z = np.zeros(B * n_obs, np.float32)
    ref = oracle_lib.out_update_dense(mu_a, var_a, jcb, obs, var_obs, z, z)
    dm, dv = _t(z), _t(z)
    F.out_update_dense(_t(mu_a), _t(var_a), _t(jcb), _t(obs), _t(var_obs), dm, dv)
    np.testing.assert_allclose(dm.cpu().numpy(), ref[0], rtol=1e-6, atol=1e-7)
    np.testing.assert_allclose(dv.cpu().numpy(), ref[1], rtol=1e-6, atol=1e-7)
    assert ref[0][5] == 0 and ref[0][9] == 0
    # indexed: 4 distinct 1-based positions per sample
    sel = np.concatenate([rng.choice(n_obs, n_enc, replace=False) + 1 for _ in range(B)]).astype(np.int32)
    y = rng.normal(0, 1, B * n_enc).astype(np.float32)
    vy = np.ones(B * n_enc, np.float32)
    ref = oracle_lib.out_update_indexed(mu_a, var_a, jcb, y, vy, sel, n_obs, n_enc, z, z)
    dm, dv = _t(z), _t(z)
    F.out_update_indexed(_t(mu_a), _t(var_a), _t(jcb), _t(y), _t(vy), _t(sel), n_obs, n_enc, dm, dv)
    np.testing.assert_allclose(dm.cpu().numpy(), ref[0], rtol=1e-6, atol=1e-7)
    np.testing.assert_allclose(dv.cpu().numpy(), ref[1], rtol=1e-6, atol=1e-7)
    assert np.count_nonzero(ref[0]) == B * n_enc


def test_out_update_heteros(oracle_lib):
    """Learned error variance: pairs (mean, expected squared error), with nan / inf
    observations and zero denominators among the inputs."""
    import cutagi_amd.functional as F
    from util import heteros_inputs
    for n in (40, 3001):
        d = heteros_inputs(n, seed=n)
        z = np.full(2 * n, 7.0, np.float32)
        ref = oracle_lib.out_update_heteros(d["mu_a"], d["var_a"], d["jcb"], d["obs"], z, z)
        dm, dv = _t(z), _t(z)
        F.out_update_heteros(_t(d["mu_a"]), _t(d["var_a"]), _t(d["jcb"]), _t(d["obs"]), dm, dv)
        np.testing.assert_allclose(dm.cpu().numpy(), ref[0], rtol=1e-5, atol=1e-7)
        np.testing.assert_allclose(dv.cpu().numpy(), ref[1], rtol=1e-5, atol=1e-7)
        assert ref[0][6] == 0 and ref[0][16] == 0 and ref[0][10] == 0 and ref[1][23] == 0


def test_param_raw_update():
    import torch
    from cutagi_amd import capi
    rng = np.random.default_rng(8)
    n = 70001
    mu, var, dmu, dvar = (rng.normal(0, 1, n).astype(np.float32) for _ in range(4))
    t_mu, t_var, t_dmu, t_dvar = _t(mu), _t(var), _t(dmu), _t(dvar)
    capi.check(capi.lib.tagi_param_raw_update(capi.ptr(t_dmu), capi.ptr(t_dvar), n,
                                              capi.ptr(t_mu), capi.ptr(t_var), None))
    torch.cuda.synchronize()
    assert np.array_equal(t_mu.cpu().numpy(), mu + dmu)      # one fp32 addition: exact
    assert np.array_equal(t_var.cpu().numpy(), var + dvar)   # no floor: may be negative


def test_relu_and_store_states(oracle_lib):
    import torch
    import cutagi_amd.functional as F
    rng = np.random.default_rng(6)
    n = 5000
    mu_z = rng.normal(0, 1, n).astype(np.float32)
    mu_z[::13] = 0.0
    var_z = rng.uniform(0.1, 1, n).astype(np.float32)
    ref = oracle_lib.relu_fwd(mu_z, var_z)
    got = F.relu_fwd(_t(mu_z), _t(var_z))
    for g, r in zip(got, ref):
        assert np.array_equal(g.cpu().numpy(), r)
    # in place
    a, v = _t(mu_z), _t(var_z)
    j = torch.empty_like(a)
    F.relu_fwd(a, v, a, j, v)
    assert np.array_equal(a.cpu().numpy(), ref[0]) and np.array_equal(v.cpu().numpy(), ref[1])
    # store_states: copies the first n_in entries and resets the output Jacobian
    mu_a, jcb = _t(mu_z), _t(var_z)
    bm, bj = torch.zeros(n, device="cuda"), torch.zeros(n, device="cuda")
    oj = torch.zeros(2 * n, device="cuda")
    F.store_states(mu_a, jcb, 3000, bm, bj, oj, 7000)
    assert torch.equal(bm[:3000], mu_a[:3000]) and float(bm[3000:].abs().max()) == 0.0
    assert torch.equal(bj[:3000], jcb[:3000])
    assert float(oj[:7000].min()) == 1.0 and float(oj[7000:].max()) == 0.0


def test_model_update_matches_layer_updates(oracle_lib):
    """tagi_model_update (all layers of a model in one launch per 24) against the
    oracle's capped step, layer by layer, counters included; 30 layers make two
    launches, one layer has no biases and one is empty."""
    import ctypes
    import torch
    from cutagi_amd import capi
    rng = np.random.default_rng(21)
    sizes = [(int(rng.integers(1, 5000)), int(rng.integers(0, 200))) for _ in range(30)]
    sizes[3] = (70000, 0)
    sizes[7] = (0, 0)
    items = (capi.UpdateItem * len(sizes))()
    keep, want = [], []
    for i, (nw, nb) in enumerate(sizes):
        cap = [0.1, 2.0, 3.0][i % 3]
        host = [rng.normal(0, 1, nw).astype(np.float32), rng.uniform(1e-4, 1, nw).astype(np.float32),
                rng.normal(0, 1, nw).astype(np.float32), rng.normal(0, 0.5, nw).astype(np.float32),
                rng.normal(0, 1, nb).astype(np.float32), rng.uniform(1e-4, 1, nb).astype(np.float32),
                rng.normal(0, 1, nb).astype(np.float32), rng.normal(0, 0.5, nb).astype(np.float32)]
        dev = [_t(a) for a in host]
        cnt = torch.tensor([5, 7], dtype=torch.int32, device="cuda")   # what earlier steps left
        slot = i % 2
        keep.append((dev, cnt, slot))
        mw, vw, c = oracle_lib.param_update(host[0], host[1], host[2], host[3], cap, True)
        mb, vb, _ = oracle_lib.param_update(host[4], host[5], host[6], host[7], cap, False)
        want.append((mw, vw, mb, vb, c))
        it = items[i]
        it.mu_w, it.var_w, it.delta_mu_w, it.delta_var_w = (capi.ptr(dev[k]) if nw else None for k in range(4))
        it.mu_b, it.var_b, it.delta_mu_b, it.delta_var_b = (capi.ptr(dev[k]) if nb else None for k in range(4, 8))
        it.num_weights, it.num_biases, it.cap_factor = nw, nb, cap
        it.neg_var_count, it.slot = capi.ptr(cnt), slot
    capi.check(capi.lib.tagi_model_update(ctypes.cast(items, ctypes.c_void_p), len(sizes), None))
    torch.cuda.synchronize()
    for i, ((dev, cnt, slot), (mw, vw, mb, vb, c)) in enumerate(zip(keep, want)):
        np.testing.assert_allclose(dev[0].cpu().numpy(), mw, rtol=1e-6, atol=1e-7)
        np.testing.assert_allclose(dev[1].cpu().numpy(), vw, rtol=1e-6, atol=1e-7)
        np.testing.assert_allclose(dev[4].cpu().numpy(), mb, rtol=1e-6, atol=1e-7)
        np.testing.assert_allclose(dev[5].cpu().numpy(), vb, rtol=1e-6, atol=1e-7)
        got = cnt.tolist()
        if sizes[i] == (0, 0):
            assert got == [5, 7]                       # an empty layer launches nothing
        else:
            assert got[slot] == [5, 7][slot] + c and got[1 - slot] == 0, (i, got, c)
