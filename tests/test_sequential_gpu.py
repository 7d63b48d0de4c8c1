"""The C++ host classes (Sequential, Linear, Conv2d, ReLU, OutputUpdater behind the
pybind11 module `cutagi`) end to end on the GPU, against an emulation of the same
training step made of CPU-oracle calls."""
import os

import numpy as np
import pytest

from model_emulation import Conv, Emulator, Lin, Relu
from util import assert_close

pytestmark = pytest.mark.gpu


def _mlp(cutagi, sizes, seed=0):
    """MLP with the parameters of the benchmark's MLP configuration:
    mu_w ~ N(0, 1/K), var_w = 1/K, mu_b = 0, var_b = 1/K."""
    rng = np.random.default_rng(seed)
    layers, emu, sd = [], [], {}
    for i, (K, N) in enumerate(zip(sizes[:-1], sizes[1:])):
        layers.append(cutagi.Linear(K, N))
        mu_w = rng.normal(0, K ** -0.5, N * K).astype(np.float32)
        var_w = np.full(N * K, 1.0 / K, np.float32)
        mu_b = np.zeros(N, np.float32)
        var_b = np.full(N, 1.0 / K, np.float32)
        sd["LinearCuda.%d" % (2 * i)] = (mu_w.tolist(), var_w.tolist(), mu_b.tolist(), var_b.tolist())
        emu.append(Lin(mu_w, var_w, mu_b, var_b, K, N))
        if i < len(sizes) - 2:
            layers.append(cutagi.ReLU())
            emu.append(Relu())
    return layers, emu, sd


def test_mlp_training_step(oracle_lib):
    """784 -> 128 -> 128 -> 11 with ReLU, batch 32: forward, update_using_indices,
    backward, step; outputs and every parameter after the step are compared."""
    from cutagi_amd import cutagi
    rng = np.random.default_rng(0)
    B, sizes = 32, [784, 128, 128, 11]
    layers, emu_layers, sd = _mlp(cutagi, sizes)
    net = cutagi.Sequential(layers)
    net.to_device("cuda")
    net.load_state_dict(sd)
    assert sorted(net.state_dict().keys()) == sorted(sd.keys())
    updater = cutagi.OutputUpdater(net.device)

    emu = Emulator(oracle_lib, emu_layers)
    for it in range(2):  # two steps: the second runs on updated parameters
        mu_x = rng.normal(0, 1, (B, sizes[0])).astype(np.float32)
        var_x = np.zeros_like(mu_x)
        sel = np.concatenate([rng.choice(11, 4, replace=False) + 1 for _ in range(B)]).astype(np.int32)
        y = rng.normal(0, 1, B * 4).astype(np.float32)
        var_y = np.ones(B * 4, np.float32)

        net.forward(mu_x, var_x)
        mu, var = net.get_outputs()
        ref_mu, ref_var = emu.forward(mu_x, var_x, B)
        assert_close(mu, ref_mu, "mu_pred step %d" % it)
        assert_close(var, ref_var, "var_pred step %d" % it)
        assert var.min() >= 0

        updater.update_using_indices(net.output_z_buffer, y.tolist(), var_y.tolist(), sel.tolist(),
                                     net.input_delta_z_buffer)
        emu.update_indexed(y, var_y, sel, 11, 4)
        net.backward()
        emu.backward()
        net.step()
        emu.step()
        got = net.state_dict()
        for i, L in enumerate(emu_layers):
            if isinstance(L, Relu):
                continue
            p = got["LinearCuda.%d" % i]
            for name, g, r in zip(("mu_w", "var_w", "mu_b", "var_b"), p,
                                  (L.mu_w, L.var_w, L.mu_b, L.var_b)):
                assert_close(np.array(g, np.float32), r.ravel(), "layer %d %s step %d" % (i, name, it))
            assert min(p[1]) > 0 and min(p[3]) > 0
        counters = net.get_neg_var_w_counter()
        assert {int(k.split(".")[1]): v for k, v in counters.items()} == emu.neg


def test_input_state_update_and_batch_change(oracle_lib):
    from cutagi_amd import cutagi
    rng = np.random.default_rng(1)
    layers, emu_layers, sd = _mlp(cutagi, [20, 12, 6], seed=1)
    net = cutagi.Sequential(layers)
    net.to_device("cuda:0")
    net.load_state_dict(sd)
    net.input_state_update = True
    updater = cutagi.OutputUpdater("cuda:0")
    emu = Emulator(oracle_lib, emu_layers)
    for B in (4, 9, 2):  # growing and shrinking batches reuse / regrow the buffers
        mu_x = rng.normal(0, 1, (B, 20)).astype(np.float32)
        var_x = rng.uniform(0.01, 0.1, (B, 20)).astype(np.float32)
        y = rng.normal(0, 1, B * 6).astype(np.float32)
        var_y = np.full(B * 6, 0.5, np.float32)
        net.forward(mu_x, var_x)
        ref = emu.forward(mu_x, var_x, B)
        mu, var = net.get_outputs()
        assert mu.shape == (B * 6,)
        assert_close(mu, ref[0], "mu B=%d" % B)
        updater.update(net.output_z_buffer, y.tolist(), var_y.tolist(), net.input_delta_z_buffer)
        emu.update_dense(y, var_y)
        net.backward()
        emu.backward(input_state_update=True)
        dm, dv = net.get_input_states()
        assert_close(dm, emu.input_delta[0], "input delta mu B=%d" % B)
        assert_close(dv, emu.input_delta[1], "input delta var B=%d" % B)


def test_conv_net_training_step(oracle_lib):
    from cutagi_amd import cutagi
    cutagi.manual_seed(3)
    rng = np.random.default_rng(3)
    B, wi = 4, 8
    net = cutagi.Sequential([cutagi.Conv2d(3, 8, 3, True, 1, 1, 1, wi, wi), cutagi.ReLU(),
                             cutagi.Conv2d(8, 8, 3, False, 2, 1, 2), cutagi.ReLU(),
                             cutagi.Linear(8 * 4 * 4, 5)])
    net.to_device("cuda")
    net.preinit_layer()
    sd = net.state_dict()
    assert sorted(sd) == ["Conv2dCuda.0", "Conv2dCuda.2", "LinearCuda.4"]
    f = lambda t: [np.array(a, np.float32) for a in t]
    emu_layers = [Conv(*f(sd["Conv2dCuda.0"]), 3, 8, 3, 1, 1, 1, 8), Relu(),
                  Conv(*f(sd["Conv2dCuda.2"]), 8, 8, 3, 2, 1, 2, 8), Relu(),
                  Lin(*f(sd["LinearCuda.4"]), 128, 5)]
    emu = Emulator(oracle_lib, emu_layers)
    updater = cutagi.OutputUpdater(net.device)
    mu_x = rng.normal(0, 1, (B, 3 * wi * wi)).astype(np.float32)
    y = rng.normal(0, 1, B * 5).astype(np.float32)
    var_y = np.ones(B * 5, np.float32)
    net.forward(mu_x)
    ref = emu.forward(mu_x, np.zeros_like(mu_x), B)
    mu, var = net.get_outputs()
    assert_close(mu, ref[0], "mu_pred")
    assert_close(var, ref[1], "var_pred")
    updater.update(net.output_z_buffer, y.tolist(), var_y.tolist(), net.input_delta_z_buffer)
    emu.update_dense(y, var_y)
    net.backward()
    emu.backward()
    net.step()
    emu.step()
    got = net.state_dict()
    for key, L in zip(sorted(got), [emu_layers[0], emu_layers[2], emu_layers[4]]):
        for name, g, r in zip(("mu_w", "var_w", "mu_b", "var_b"), got[key],
                              (L.mu_w, L.var_w, L.mu_b, L.var_b)):
            if r is None:
                assert len(g) == 0
                continue
            assert_close(np.array(g, np.float32), r.ravel(), key + " " + name)


def test_errors_and_checkpoint_round_trip(tmp_path):
    from cutagi_amd import cutagi
    layers, _, sd = _mlp(cutagi, [16, 8, 4], seed=2)
    net = cutagi.Sequential(layers)
    with pytest.raises(RuntimeError):
        net.to_device("cuda:99")      # invalid device index
    with pytest.raises(RuntimeError):
        net.forward(np.zeros((2, 16), np.float32))   # not on the device yet
    net.to_device("cuda")
    net.load_state_dict(sd)
    with pytest.raises(RuntimeError):
        net.forward(np.zeros((2, 15), np.float32))   # input size mismatch
    path = os.path.join(tmp_path, "model.bin")
    net.save(path)
    layers2, _, _ = _mlp(cutagi, [16, 8, 4], seed=9)
    net2 = cutagi.Sequential(layers2)
    net2.to_device("cuda")
    net2.load(path)
    a, b = net.state_dict(), net2.state_dict()
    assert a.keys() == b.keys() and all(a[k] == b[k] for k in a)   # bit-equal
    x = np.random.default_rng(0).normal(0, 1, (3, 16)).astype(np.float32)
    net.forward(x)
    net2.forward(x)
    assert np.array_equal(net.get_outputs()[0], net2.get_outputs()[0])
    with pytest.raises(RuntimeError):
        cutagi.OutputUpdater("cpu").update(net.output_z_buffer, [0.0] * 12, [1.0] * 12,
                                           net.input_delta_z_buffer)


def test_output_updater_reads_numpy_arrays_in_place():
    """float32 / int32 numpy arrays take the binding's direct path; lists (the
    reference's binding) and arrays of another type take the std::vector path.
    Both give the same innovations, and wrong sizes or indices raise."""
    from cutagi_amd import cutagi
    cutagi.manual_seed(2)
    rng = np.random.default_rng(2)
    B, N = 16, 11
    net = cutagi.Sequential([cutagi.Linear(20, N)])
    net.to_device("cuda")
    net.forward(rng.normal(0, 1, (B, 20)).astype(np.float32))
    upd = cutagi.OutputUpdater(net.device)
    d = net.input_delta_z_buffer

    def deltas():
        d.to_host()
        return np.array(d.delta_mu[:B * N], np.float32), np.array(d.delta_var[:B * N], np.float32)

    y = rng.normal(0, 1, B * N).astype(np.float32)
    v = rng.uniform(0.5, 1.5, B * N).astype(np.float32)
    upd.update(net.output_z_buffer, y.tolist(), v.tolist(), d)
    want = deltas()
    upd.update(net.output_z_buffer, y, v, d)
    got = deltas()
    assert np.array_equal(got[0], want[0]) and np.array_equal(got[1], want[1])
    upd.update(net.output_z_buffer, y.astype(np.float64), v.astype(np.float64), d)  # converted
    got = deltas()
    assert np.array_equal(got[0], want[0]) and np.array_equal(got[1], want[1])

    n_enc = 4
    ys = rng.normal(0, 1, B * n_enc).astype(np.float32)
    vs = np.ones(B * n_enc, np.float32)
    sel = rng.integers(1, N + 1, B * n_enc).astype(np.int32)
    upd.update_using_indices(net.output_z_buffer, ys.tolist(), vs.tolist(), sel.tolist(), d)
    want = deltas()
    assert np.any(want[0] != 0)
    upd.update_using_indices(net.output_z_buffer, ys, vs, sel, d)
    got = deltas()
    assert np.array_equal(got[0], want[0]) and np.array_equal(got[1], want[1])
    upd.update_using_indices(net.output_z_buffer, ys, vs, sel.astype(np.int64), d)  # converted
    got = deltas()
    assert np.array_equal(got[0], want[0]) and np.array_equal(got[1], want[1])

    with pytest.raises(RuntimeError):
        upd.update(net.output_z_buffer, y, v[:-1], d)
    with pytest.raises(RuntimeError):
        upd.update_using_indices(net.output_z_buffer, ys, vs, sel[:-1], d)
    bad = sel.copy()
    bad[5] = N + 1
    with pytest.raises(RuntimeError):
        upd.update_using_indices(net.output_z_buffer, ys, vs, bad, d)
    bad[5] = 0
    with pytest.raises(RuntimeError):
        upd.update_using_indices(net.output_z_buffer, ys, vs, bad, d)


def test_device_queries():
    from cutagi_amd import cutagi
    assert cutagi.is_cuda_available() and cutagi.get_cuda_device_count() >= 1
    assert cutagi.get_cuda_current_device() == 0 and cutagi.set_cuda_device(0) is True
    assert cutagi.is_cuda_device_available(0) and not cutagi.is_cuda_device_available(99)
    assert "gfx950" in cutagi.get_cuda_device_properties(0)
    free, total = cutagi.get_cuda_device_memory(0)
    assert 0 < free <= total and total > 100 * 2 ** 30
    with pytest.raises(RuntimeError):
        cutagi.set_cuda_device(99)
