"""tagi_upload_input / tagi_download_outputs through the C ABI: the kernels that move
a batch of network inputs from pinned host memory into a state buffer, and the first
entries of a state buffer back into pinned host memory. They replace copy-engine
transfers, so the check is byte equality with what was sent."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

SIZES = [1, 3, 64, 785, 25088, 100003, 262144]


@pytest.mark.parametrize("n", SIZES)
@pytest.mark.parametrize("with_var", [True, False])
def test_upload_input_copies_means_and_variances(n, with_var):
    import torch
    from cutagi_amd import capi
    rng = np.random.default_rng(n)
    host_mu = torch.from_numpy(rng.standard_normal(n).astype(np.float32)).pin_memory()
    host_var = torch.from_numpy(rng.uniform(0, 1, n).astype(np.float32)).pin_memory()
    # the state buffer is larger than the batch: entries past n stay as they were
    mu_a = torch.full((n + 5,), 7.0, device="cuda")
    var_a = torch.full((n + 5,), 7.0, device="cuda")
    stream = torch.cuda.current_stream().cuda_stream
    capi.check(capi.lib.tagi_upload_input(host_mu.data_ptr(),
                                          host_var.data_ptr() if with_var else None, n,
                                          capi.ptr(mu_a), capi.ptr(var_a), stream))
    torch.cuda.synchronize()
    assert torch.equal(mu_a[:n].cpu(), host_mu)
    if with_var:
        assert torch.equal(var_a[:n].cpu(), host_var)
    else:
        assert float(var_a[:n].abs().max()) == 0.0     # no variances given: zeros
    assert float(mu_a[n:].min()) == 7.0 and float(var_a[n:].max()) == 7.0


@pytest.mark.parametrize("n", SIZES)
@pytest.mark.parametrize("with_flag", [False, True])
def test_download_outputs_writes_pinned_memory(n, with_flag):
    import torch
    from cutagi_amd import capi
    rng = np.random.default_rng(n + 1)
    mu = torch.from_numpy(rng.standard_normal(n + 3).astype(np.float32)).cuda()
    var = torch.from_numpy(rng.uniform(0, 1, n + 3).astype(np.float32)).cuda()
    host = torch.full((2 * n + 2,), -3.0).pin_memory()
    flag = torch.zeros(16, dtype=torch.int32).pin_memory()
    stream = torch.cuda.current_stream().cuda_stream
    capi.check(capi.lib.tagi_download_outputs(capi.ptr(mu), capi.ptr(var), n, host.data_ptr(),
                                              host.data_ptr() + 4 * n,
                                              flag.data_ptr() if with_flag else None, 77, stream))
    if with_flag:
        # the flag is the completion signal: poll it (bounded), then read without a
        # stream synchronisation
        import time
        t0 = time.time()
        while int(flag[0]) != 77 and time.time() - t0 < 10.0:
            pass
        assert int(flag[0]) == 77
    else:
        torch.cuda.synchronize()
        assert int(flag[0]) == 0
    assert torch.equal(host[:n], mu[:n].cpu())
    assert torch.equal(host[n:2 * n], var[:n].cpu())
    assert float(host[2 * n:].max()) == -3.0


def test_transfers_reject_null_pointers_and_accept_empty_batches():
    import torch
    from cutagi_amd import capi
    x = torch.zeros(8, device="cuda")
    h = torch.zeros(8).pin_memory()
    assert capi.lib.tagi_upload_input(None, None, 8, capi.ptr(x), capi.ptr(x), None) == capi.ERR_INVALID_ARG
    assert capi.lib.tagi_upload_input(h.data_ptr(), None, 8, None, capi.ptr(x), None) == capi.ERR_INVALID_ARG
    assert capi.lib.tagi_download_outputs(capi.ptr(x), capi.ptr(x), 8, None, h.data_ptr(), None, 0, None) == capi.ERR_INVALID_ARG
    assert capi.lib.tagi_download_outputs(capi.ptr(x), capi.ptr(x), (1 << 20) + 1, h.data_ptr(), h.data_ptr(), h.data_ptr(), 1, None) == capi.ERR_UNSUPPORTED
    assert capi.lib.tagi_upload_input(None, None, 0, None, None, None) == capi.OK
    assert capi.lib.tagi_download_outputs(None, None, 0, None, None, None, 0, None) == capi.OK
    torch.cuda.synchronize()


def test_network_outputs_survive_the_pinned_path():
    """Sequential.get_outputs after a forward equals the state buffer read with an
    ordinary copy (output_to_host keeps using the same buffers)."""
    import torch  # noqa: F401  (initialises the device before the module's first call)
    from cutagi_amd import cutagi as c
    c.manual_seed(3)
    net = c.Sequential([c.Linear(20, 16), c.ReLU(), c.Linear(16, 5)])
    net.to_device("cuda")
    x = np.random.default_rng(0).standard_normal(4 * 20).astype(np.float32)
    net.forward(x)
    m1, v1 = net.get_outputs()
    m2, v2 = net.get_outputs()
    assert np.array_equal(m1, m2) and np.array_equal(v1, v2)
    assert m1.shape[0] == 4 * 5 and np.all(np.isfinite(m1)) and np.all(v1 > 0)


@pytest.mark.parametrize("B,n_obs,n_enc,extra", [(32, 11, 4, 25000), (7, 300, 300, 0), (1, 5, 1, 3),
                                                   (64, 1030, 10, 12345), (3, 600, 520, 77)])
@pytest.mark.parametrize("pinned", [False, True])
def test_indexed_update_with_reset_equals_clear_then_update(oracle_lib, B, n_obs, n_enc, extra,
                                                            pinned):
    """tagi_out_update_indexed_reset against the oracle (1e-6: one division and two
    products per entry) and, bit for bit, against a cleared buffer followed by
    tagi_out_update_indexed; the buffers start full of a guard value and are longer than
    the outputs, with the observations in device or in pinned host memory. Includes a
    non-finite gain (zero denominator) and more observations per sample than a workgroup
    has threads."""
    import torch
    from cutagi_amd import capi
    rng = np.random.default_rng(B + n_obs)
    f = np.float32
    mu_a = rng.standard_normal(B * n_obs).astype(f)
    var_a = rng.uniform(0.1, 1, B * n_obs).astype(f)
    jcb = rng.uniform(0, 1, B * n_obs).astype(f)
    sel = np.concatenate([rng.choice(n_obs, n_enc, replace=False) + 1 for _ in range(B)]).astype(np.int32)
    y = rng.standard_normal(B * n_enc).astype(f)
    vy = rng.uniform(0.5, 1, B * n_enc).astype(f)
    vy[0] = -var_a[sel[0] - 1]                      # zero denominator -> that entry stays 0
    z = np.zeros(B * n_obs, f)
    ref = oracle_lib.out_update_indexed(mu_a, var_a, jcb, y, vy, sel, n_obs, n_enc, z, z)
    dev = lambda a: torch.from_numpy(a).cuda()
    place = (lambda a: torch.from_numpy(a).pin_memory()) if pinned else dev
    t_mu, t_var, t_jcb = dev(mu_a), dev(var_a), dev(jcb)
    t_y, t_vy, t_sel = place(y), place(vy), place(sel)
    n_len = B * n_obs + extra
    got_mu = torch.full((n_len,), 9.0, device="cuda")
    got_var = torch.full((n_len,), 9.0, device="cuda")
    stream = torch.cuda.current_stream().cuda_stream
    capi.check(capi.lib.tagi_out_update_indexed_reset(
        capi.ptr(t_mu), capi.ptr(t_var), capi.ptr(t_jcb), t_y.data_ptr(), t_vy.data_ptr(),
        t_sel.data_ptr(), n_obs, n_enc, B * n_enc, capi.ptr(got_mu), capi.ptr(got_var), n_len,
        stream))
    want_mu, want_var = torch.zeros(n_len, device="cuda"), torch.zeros(n_len, device="cuda")
    d_y, d_vy, d_sel = dev(y), dev(vy), dev(sel)
    capi.check(capi.lib.tagi_out_update_indexed(
        capi.ptr(t_mu), capi.ptr(t_var), capi.ptr(t_jcb), capi.ptr(d_y), capi.ptr(d_vy),
        capi.ptr(d_sel), n_obs, n_enc, B * n_enc, capi.ptr(want_mu), capi.ptr(want_var), stream))
    torch.cuda.synchronize()
    assert torch.equal(got_mu, want_mu) and torch.equal(got_var, want_var)
    np.testing.assert_allclose(got_mu[:B * n_obs].cpu().numpy(), ref[0], rtol=1e-6, atol=1e-7)
    np.testing.assert_allclose(got_var[:B * n_obs].cpu().numpy(), ref[1], rtol=1e-6, atol=1e-7)
    assert float(got_mu[B * n_obs:].abs().max() if extra else 0.0) == 0.0
    assert np.count_nonzero(ref[0]) == B * n_enc - 1


def test_indexed_update_with_reset_rejects_short_buffers():
    import torch
    from cutagi_amd import capi
    x = torch.zeros(64, device="cuda")
    i = torch.ones(8, dtype=torch.int32, device="cuda")
    call = lambda n, n_enc, n_len: capi.lib.tagi_out_update_indexed_reset(
        capi.ptr(x), capi.ptr(x), capi.ptr(x), capi.ptr(x), capi.ptr(x), capi.ptr(i), 8, n_enc, n,
        capi.ptr(x), capi.ptr(x), n_len, None)
    assert call(8, 4, 15) == capi.ERR_INVALID_ARG     # 2 samples x 8 outputs need 16 entries
    assert call(7, 4, 64) == capi.ERR_INVALID_ARG     # not whole samples
    assert call(8, 4, 16) == capi.OK
    torch.cuda.synchronize()
