"""Parity of the HIP Linear path (through the C ABI) against the CPU oracle."""
import numpy as np
import pytest

from util import SAME_SIGN, assert_close, linear_inputs

pytestmark = pytest.mark.gpu

# (K, N, B): tiled path (aligned / ragged / odd), skinny path, layer shapes of
# the MLP configuration, and the reference's odd-size smoke shape (785 -> 6000)
# scaled down (its real size: test_pack_size_network_at_its_real_size below).
SHAPES = [
    (256, 256, 128), (512, 384, 256), (100, 36, 40), (785, 600, 16), (784, 128, 32),
    (128, 128, 32), (128, 11, 32), (64, 32, 1), (256, 512, 8), (1024, 256, 5),
    (516, 260, 16), (130, 70, 17), (5, 3, 2), (4, 4, 4), (333, 129, 77),
    # skinny path: several grid rows of fold workgroups, ragged row blocks, one row block
    (2048, 48, 7), (768, 1000, 3), (4096, 16, 16), (260, 20, 9),
    # 9..16 samples: the 16-wide streaming kernels (several slices, ragged rows and columns)
    (1024, 512, 16), (1536, 260, 12), (72, 1028, 10), (2052, 300, 13), (512, 2048, 9),
    # 17..32 samples: the same kernels with two groups of sixteen samples
    (1024, 512, 32), (1536, 260, 24), (72, 1028, 17), (516, 300, 31), (4096, 256, 20),
]


def _dev(d):
    import torch
    return {k: (None if v is None else torch.from_numpy(v).cuda()) for k, v in d.items()}


@pytest.mark.parametrize("K,N,B", SHAPES)
@pytest.mark.parametrize("bias", [True, False])
def test_linear_forward(oracle_lib, linear_kernel_choice, K, N, B, bias):
    import cutagi_amd.functional as F
    d = linear_inputs(K, N, B, seed=K + N + B, bias=bias)
    t = _dev(d)
    mu_z, var_z = F.linear_fwd(t["mu_w"], t["var_w"], t["mu_b"], t["var_b"], t["mu_a"], t["var_a"])
    ref_mu, ref_var = oracle_lib.linear_fwd(d["mu_w"], d["var_w"], d["mu_b"], d["var_b"],
                                            d["mu_a"], d["var_a"], threads=4)
    assert_close(mu_z.cpu().numpy(), ref_mu, "mu_z")
    assert_close(var_z.cpu().numpy(), ref_var, "var_z", same_sign=True)
    assert float(var_z.min()) >= 0.0


@pytest.mark.parametrize("K,N,B", SHAPES)
def test_linear_backward(oracle_lib, linear_kernel_choice, K, N, B):
    import cutagi_amd.functional as F
    d = linear_inputs(K, N, B, seed=7 * K + N + B, bias=True, jcb_random=True)
    t = _dev(d)
    out = F.linear_bwd(t["mu_w"], t["var_w"], t["var_b"], t["mu_a"], t["jcb"], t["delta_mu"],
                       t["delta_var"])
    dz = oracle_lib.linear_bwd_dz(d["mu_w"], d["jcb"], d["delta_mu"], d["delta_var"], threads=4)
    dw = oracle_lib.linear_bwd_dw(d["var_w"], d["mu_a"], d["delta_mu"], d["delta_var"], threads=4)
    db = oracle_lib.linear_bwd_db(d["var_b"], d["delta_mu"], d["delta_var"])
    names = ["delta_mu_z", "delta_var_z", "delta_mu_w", "delta_var_w", "delta_mu_b", "delta_var_b"]
    for name, got, ref in zip(names, out, dz + dw + db):
        assert_close(got.cpu().numpy(), ref, name, same_sign=name in SAME_SIGN)
    # innovations of the variance keep the sign of delta_var (<= 0)
    assert float(out[1].max()) <= 0.0 and float(out[3].max()) <= 0.0 and float(out[5].max()) <= 0.0


@pytest.mark.parametrize("K,N,B", [(512, 384, 256), (100, 36, 40), (784, 128, 32)])
def test_linear_backward_separate_launches(oracle_lib, K, N, B):
    """The tiled backward with the bias innovations and the state-backward fold as
    launches of their own (tuning switch) instead of riding along with the weight
    backward: same results."""
    import cutagi_amd.functional as F
    from cutagi_amd import capi
    d = linear_inputs(K, N, B, seed=K + 3 * N + B, bias=True, jcb_random=True)
    t = _dev(d)
    capi.tune("linear.dw_side", 0)
    try:
        out = F.linear_bwd(t["mu_w"], t["var_w"], t["var_b"], t["mu_a"], t["jcb"], t["delta_mu"],
                           t["delta_var"])
    finally:
        capi.tune("linear.dw_side", -1)
    ref = (oracle_lib.linear_bwd_dz(d["mu_w"], d["jcb"], d["delta_mu"], d["delta_var"], threads=4)
           + oracle_lib.linear_bwd_dw(d["var_w"], d["mu_a"], d["delta_mu"], d["delta_var"], threads=4)
           + oracle_lib.linear_bwd_db(d["var_b"], d["delta_mu"], d["delta_var"]))
    for i, (got, want) in enumerate(zip(out, ref)):
        assert_close(got.cpu().numpy(), want, "output %d" % i)
    riding = F.linear_bwd(t["mu_w"], t["var_w"], t["var_b"], t["mu_a"], t["jcb"], t["delta_mu"],
                          t["delta_var"])
    for a, b in zip(out[:4], riding[:4]):   # same arithmetic, same order: same bits
        assert bool((a == b).all())


def test_linear_backward_skips(oracle_lib):
    """state_update / param_update switches of LinearCuda::backward."""
    import torch
    import cutagi_amd.functional as F
    d = linear_inputs(64, 32, 8, seed=3)
    t = _dev(d)
    out = F.linear_bwd(t["mu_w"], t["var_w"], t["var_b"], t["mu_a"], t["jcb"], t["delta_mu"],
                       t["delta_var"], state_update=False)
    assert out[0] is None and out[2] is not None
    out = F.linear_bwd(t["mu_w"], t["var_w"], t["var_b"], t["mu_a"], t["jcb"], t["delta_mu"],
                       t["delta_var"], param_update=False)
    assert out[2] is None and out[4] is None and out[0] is not None
    torch.cuda.synchronize()


def test_size_mismatch_raises():
    """The reference throws on an input-size mismatch (Linear::forward)."""
    import cutagi_amd.functional as F
    d = linear_inputs(64, 32, 8, seed=3)
    t = _dev(d)
    with pytest.raises(ValueError):
        F.linear_fwd(t["mu_w"], t["var_w"], t["mu_b"], t["var_b"], t["mu_a"][:, :32].contiguous(),
                     t["var_a"][:, :32].contiguous())


# The reference's odd-size survival test at its real size: Linear(785, 6000) - ReLU -
# Linear(6000, 784), batch 16, one forward / dense output update / backward / step
# (test/cpp_unit/test_pack_size.cpp:26-62; it only asserts that the run survives).
# Here each layer at that size is also held against the oracle.
@pytest.mark.parametrize("K,N", [(785, 6000), (6000, 784)])
def test_pack_size_layers_at_their_real_size(oracle_lib, K, N):
    import cutagi_amd.functional as F
    B = 16
    d = linear_inputs(K, N, B, seed=K + N, bias=True, jcb_random=True)
    t = _dev(d)
    z = F.linear_fwd(t["mu_w"], t["var_w"], t["mu_b"], t["var_b"], t["mu_a"], t["var_a"])
    ref = oracle_lib.linear_fwd(d["mu_w"], d["var_w"], d["mu_b"], d["var_b"], d["mu_a"],
                                d["var_a"], threads=8)
    assert_close(z[0].cpu().numpy(), ref[0], "mu_z")
    assert_close(z[1].cpu().numpy(), ref[1], "var_z", same_sign=True)
    out = F.linear_bwd(t["mu_w"], t["var_w"], t["var_b"], t["mu_a"], t["jcb"], t["delta_mu"],
                       t["delta_var"])
    want = (oracle_lib.linear_bwd_dz(d["mu_w"], d["jcb"], d["delta_mu"], d["delta_var"], threads=8)
            + oracle_lib.linear_bwd_dw(d["var_w"], d["mu_a"], d["delta_mu"], d["delta_var"], threads=8)
            + oracle_lib.linear_bwd_db(d["var_b"], d["delta_mu"], d["delta_var"]))
    names = ["delta_mu_z", "delta_var_z", "delta_mu_w", "delta_var_w", "delta_mu_b", "delta_var_b"]
    for name, got, r in zip(names, out, want):
        assert_close(got.cpu().numpy(), r, name, same_sign=name in SAME_SIGN)


def test_pack_size_network_at_its_real_size():
    from cutagi_amd import cutagi
    cutagi.manual_seed(0)
    net = cutagi.Sequential([cutagi.Linear(785, 6000), cutagi.ReLU(), cutagi.Linear(6000, 784)])
    net.to_device("cuda")
    updater = cutagi.OutputUpdater(net.device)
    rng = np.random.default_rng(0)
    B = 16
    x = rng.uniform(0, 1, (B, 785)).astype(np.float32)
    y = rng.uniform(0, 1, B * 784).astype(np.float32)
    var_y = np.ones(B * 784, np.float32)
    before = {k: [np.array(a) for a in v] for k, v in net.state_dict().items()}
    net.forward(x)
    mu, var = net.get_outputs()
    updater.update(net.output_z_buffer, y, var_y, net.input_delta_z_buffer)
    net.backward()
    net.step()
    assert mu.size == B * 784 and np.all(np.isfinite(mu)) and var.min() >= 0
    after = net.state_dict()
    for key, arrays in after.items():
        for a, b in zip(arrays, before[key]):
            a = np.asarray(a)
            assert np.all(np.isfinite(a))
        # the step moved the weight means and shrank no variance below zero
        assert not np.array_equal(np.asarray(arrays[0]), before[key][0])
        assert np.asarray(arrays[1]).min() >= 0


@pytest.mark.parametrize("K,N,B", [(1024, 512, 16), (1536, 260, 12), (72, 1028, 10),
                                   (2052, 300, 13), (4096, 256, 9), (516, 1000, 20),
                                   (2048, 1027 * 4, 32), (36, 52, 12)])
def test_forward_load_patterns_for_9_to_16_samples(oracle_lib, K, N, B):
    """The 16-wide streaming forward loads its weights as whole 128-byte lines (lanes
    then exchange a float4) with streaming loads, plain loads or one of each per matrix,
    or as sixteen rows x 64 bytes per instruction. The library picks by size; all must
    agree bit for bit (the same registers reach the same MFMAs)."""
    import cutagi_amd.functional as F
    from cutagi_amd import capi
    d = linear_inputs(K, N, B, seed=K + N + B, bias=True)
    t = _dev(d)
    ref = oracle_lib.linear_fwd(d["mu_w"], d["var_w"], d["mu_b"], d["var_b"], d["mu_a"],
                                d["var_a"], threads=4)
    got = {}
    capi.tune("linear.stream_min_weights", 0)     # these shapes are small: force the kernels
    try:
        for waves in (8, 16):                     # workgroups of 128 or 256 rows
            capi.tune("linear.gemv16.fwd_waves", waves)
            for pattern in (0, 1, 2, 3, 4):
                capi.tune("linear.gemv16.whole_lines", pattern)
                z = F.linear_fwd(t["mu_w"], t["var_w"], t["mu_b"], t["var_b"], t["mu_a"], t["var_a"])
                got[pattern] = (z[0].cpu().numpy(), z[1].cpu().numpy())
                what = "(pattern %d, %d waves)" % (pattern, waves)
                assert_close(got[pattern][0], ref[0], "mu_z " + what)
                assert_close(got[pattern][1], ref[1], "var_z " + what, same_sign=True)
            for pattern in (1, 2, 3, 4):
                assert np.array_equal(got[pattern][0], got[0][0])
                assert np.array_equal(got[pattern][1], got[0][1])
    finally:
        capi.tune("linear.gemv16.whole_lines", -1)
        capi.tune("linear.gemv16.fwd_waves", -1)
        capi.tune("linear.stream_min_weights", -1)


@pytest.mark.parametrize("K,N,B", [(1024, 512, 32), (1536, 260, 24), (516, 300, 31)])
def test_state_backward_streaming_kernel_for_17_to_32_samples(oracle_lib, K, N, B):
    """The two-group form of the 16-wide state backward (not the default above 16
    samples: the tiled kernel measures faster there) still gives the oracle's result."""
    import cutagi_amd.functional as F
    from cutagi_amd import capi
    d = linear_inputs(K, N, B, seed=K + N + B, bias=True, jcb_random=True)
    t = _dev(d)
    ref = oracle_lib.linear_bwd_dz(d["mu_w"], d["jcb"], d["delta_mu"], d["delta_var"], threads=4)
    capi.tune("linear.gemv32", 2)
    capi.tune("linear.stream_min_weights", 0)
    try:
        dz = F.linear_bwd_dz(t["mu_w"], t["jcb"], t["delta_mu"], t["delta_var"])
        out = F.linear_bwd(t["mu_w"], t["var_w"], t["var_b"], t["mu_a"], t["jcb"], t["delta_mu"],
                           t["delta_var"])
    finally:
        capi.tune("linear.gemv32", -1)
        capi.tune("linear.stream_min_weights", -1)
    for got in (dz, out[:2]):
        assert_close(got[0].cpu().numpy(), ref[0], "delta_mu_z")
        assert_close(got[1].cpu().numpy(), ref[1], "delta_var_z", same_sign=True)
