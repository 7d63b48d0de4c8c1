"""MixtureReLU, BatchNorm2d, AvgPool2d, LayerBlock and ResNetBlock of the C++ host
classes end to end on the GPU: a scaled-down ResNet (same layer pattern as the
CIFAR ResNet-18 configuration: stem, identity block, strided block with a
projection shortcut, global pooling, Linear head, hierarchical-softmax update)
against an emulation of the same training step made of CPU-oracle calls."""
import numpy as np
import pytest

from model_emulation import BNorm, Block, Conv, Emulator, Lin, MRelu, Pool, Res, param_layers
from util import assert_close

pytestmark = pytest.mark.gpu


def _main_block(c, i, o, stride=1, pt=1):
    return c.LayerBlock([c.Conv2d(i, o, 3, bias=False, stride=stride, padding=1, padding_type=pt),
                         c.MixtureReLU(), c.BatchNorm2d(o),
                         c.Conv2d(o, o, 3, bias=False, padding=1), c.MixtureReLU(), c.BatchNorm2d(o)])


def _small_resnet(c, wi=8):
    return c.Sequential([
        c.Conv2d(3, 8, 3, bias=False, padding=1, in_width=wi, in_height=wi), c.MixtureReLU(),
        c.BatchNorm2d(8),
        c.ResNetBlock(_main_block(c, 8, 8)),
        c.ResNetBlock(_main_block(c, 8, 16, 2, 2),
                      c.LayerBlock([c.Conv2d(8, 16, 2, bias=False, stride=2), c.MixtureReLU(),
                                    c.BatchNorm2d(16)])),
        c.AvgPool2d(wi // 2), c.Linear(16, 11)])


def _emulation(sd, wi=8):
    """The same network for the emulator, with the parameters of a state dict."""
    f = lambda key: [np.array(a, np.float32) for a in sd[key]]
    conv = lambda key, fi, fo, k, s, p, pt, w: Conv(*f("Conv2dCuda." + key), fi, fo, k, s, p, pt, w)
    bn = lambda key, nf: BNorm(*f("BatchNorm2dCuda." + key), nf)

    def main(i, fi, fo, s, pt, w):
        p = "main.%d." % i
        return Block([conv(p + "0", fi, fo, 3, s, 1, pt, w), MRelu(), bn(p + "2", fo),
                      conv(p + "3", fo, fo, 3, 1, 1, 1, w // s), MRelu(), bn(p + "5", fo)])

    h = wi // 2
    return [conv("0", 3, 8, 3, 1, 1, 1, wi), MRelu(), bn("2", 8),
            Res(main(3, 8, 8, 1, 1, wi)),
            Res(main(4, 8, 16, 2, 2, wi),
                Block([conv("shortcut.4.0", 8, 16, 2, 2, 0, 1, wi), MRelu(), bn("shortcut.4.2", 16)])),
            Pool(h, -1, 0, 0, h, 16), Lin(*f("LinearCuda.6"), 16, 11)]


# hierarchical softmax of 10 classes: 4 observations per label among 11 outputs
HRC_IDX = {0: (1, 2, 4, 7), 1: (1, 2, 4, 7), 2: (1, 2, 4, 8), 3: (1, 2, 4, 8), 4: (1, 2, 5, 9),
           5: (1, 2, 5, 9), 6: (1, 2, 5, 10), 7: (1, 2, 5, 10), 8: (1, 3, 6, 11), 9: (1, 3, 6, 11)}


def _hrc_obs(label):
    bits = [(label >> s) & 1 for s in (3, 2, 1, 0)]
    return [(-1.0) ** b for b in bits]


def test_resnet_training_steps(oracle_lib):
    from cutagi_amd import cutagi
    cutagi.manual_seed(7)
    rng = np.random.default_rng(7)
    B, wi = 6, 8
    net = _small_resnet(cutagi, wi)
    net.to_device("cuda")
    net.preinit_layer()
    sd = net.state_dict()
    emu_layers = _emulation(sd, wi)
    expected_keys = sorted(("Linear" if isinstance(L, Lin) else "Conv2d" if isinstance(L, Conv)
                            else "BatchNorm2d") + "Cuda." + sfx
                           for sfx, L in param_layers(emu_layers))
    assert sorted(sd) == expected_keys
    emu = Emulator(oracle_lib, emu_layers)
    updater = cutagi.OutputUpdater(net.device)

    for it in range(2):  # the second step runs on updated parameters and running averages
        mu_x = rng.normal(0, 1, (B, 3 * wi * wi)).astype(np.float32)
        labels = rng.integers(0, 10, B)
        y = np.array([v for l in labels for v in _hrc_obs(int(l))], np.float32)
        sel = np.array([v for l in labels for v in HRC_IDX[int(l)]], np.int32)
        var_y = np.ones(B * 4, np.float32)

        net.forward(mu_x)
        ref = emu.forward(mu_x, np.zeros_like(mu_x), B)
        mu, var = net.get_outputs()
        assert mu.shape == (B * 11,)
        assert_close(mu, ref[0], "mu_pred step %d" % it)
        assert_close(var, ref[1], "var_pred step %d" % it)
        assert var.min() >= 0

        updater.update_using_indices(net.output_z_buffer, y.tolist(), var_y.tolist(), sel.tolist(),
                                     net.input_delta_z_buffer)
        emu.update_indexed(y, var_y, sel, 11, 4)
        net.backward()
        emu.backward()
        net.step()
        emu.step()

        got = net.state_dict()
        for sfx, L in param_layers(emu_layers):
            name = ("Linear" if isinstance(L, Lin) else "Conv2d" if isinstance(L, Conv)
                    else "BatchNorm2d") + "Cuda." + sfx
            for pname, g, r in zip(("mu_w", "var_w", "mu_b", "var_b"), got[name],
                                   (L.mu_w, L.var_w, L.mu_b, L.var_b)):
                if r is None:
                    assert len(g) == 0
                    continue
                assert_close(np.array(g, np.float32), r.ravel(), "%s %s step %d" % (name, pname, it))
                if pname.startswith("var"):
                    assert min(g) > 0

    # running averages of the stem's batch norm after two batches
    stats = net.layers[2].get_norm_mean_var()
    bn = emu_layers[2]
    for name, g, r in zip(("mu_ra", "var_ra", "mu_norm_batch", "var_norm_batch"), stats,
                          (bn.mu_ra, bn.var_ra, bn.mu_s, bn.var_s)):
        assert_close(np.array(g, np.float32), r, "stem batch norm " + name)


def test_resnet_checkpoint_and_eval(tmp_path, oracle_lib):
    """save/load keeps parameters and running averages; eval mode normalises with
    the running averages and gives the same outputs after the round trip."""
    import os
    from cutagi_amd import cutagi
    cutagi.manual_seed(11)
    rng = np.random.default_rng(11)
    net = _small_resnet(cutagi)
    net.to_device("cuda")
    x = rng.normal(0, 1, (4, 3 * 64)).astype(np.float32)
    net.forward(x)      # one training batch moves the running averages
    path = os.path.join(tmp_path, "resnet.bin")
    net.save(path)
    net2 = _small_resnet(cutagi)
    net2.to_device("cuda")
    net2.load(path)
    a, b = net.state_dict(), net2.state_dict()
    assert a.keys() == b.keys() and all(a[k] == b[k] for k in a)
    assert net.layers[2].get_norm_mean_var()[:2] == net2.layers[2].get_norm_mean_var()[:2]
    net.eval()
    net2.eval()
    net.forward(x)
    net2.forward(x)
    assert np.array_equal(net.get_outputs()[0], net2.get_outputs()[0])
    assert np.all(np.isfinite(net.get_outputs()[0]))


def test_resnet18_full_size_step():
    """The ResNet-18 configuration at its real size (batch 128): one training step
    through the host classes. Too large for the CPU emulation; checked through what
    holds at any size: finite outputs, non-negative output variances, every
    parameter variance positive after the step, running variances positive."""
    from cutagi_amd import cutagi
    from cutagi_amd.resnet import hrc_softmax, resnet18_cifar10
    B = 128
    cutagi.manual_seed(0)
    net = resnet18_cifar10(cutagi)
    net.to_device("cuda")
    updater = cutagi.OutputUpdater(net.device)
    obs, idx, n_obs, n_out = hrc_softmax(10)
    rng = np.random.default_rng(0)
    x = rng.normal(0, 1, (B, 3 * 32 * 32)).astype(np.float32)
    labels = rng.integers(0, 10, B)
    for _ in range(2):
        net.forward(x)
        mu, var = net.get_outputs()
        assert mu.shape == (B * n_out,) and np.all(np.isfinite(mu)) and np.all(np.isfinite(var))
        assert var.min() >= 0
        updater.update_using_indices(net.output_z_buffer, obs[labels].ravel().tolist(),
                                     [1.0] * (B * n_obs), idx[labels].ravel().tolist(),
                                     net.input_delta_z_buffer)
        net.backward()
        net.step()
    sd = net.state_dict()
    assert len(sd) == 41  # 20 convolutions, 20 batch norms, 1 linear
    for key, (mu_w, var_w, mu_b, var_b) in sd.items():
        assert np.all(np.isfinite(mu_w)) and min(var_w) > 0, key
        if len(var_b):
            assert np.all(np.isfinite(mu_b)) and min(var_b) > 0, key
    assert min(net.layers[2].get_norm_mean_var()[1][0]) > 0  # one entry per norm layer


def test_resnet18_learns_a_synthetic_classification_task():
    """The reference's accuracy gate for this model (test/cpp_unit/test_resnet.cpp:
    267-270: CIFAR error rate below 0.8 after 100 batches of 64), on synthetic images
    since no dataset travels: noisy copies of ten random prototypes; chance is 0.9."""
    from cutagi_amd import cutagi
    from cutagi_amd.nn import HRCSoftmaxMetric, Utils
    from cutagi_amd.resnet import resnet18_cifar10
    cutagi.manual_seed(2)
    rng = np.random.default_rng(2)
    protos = rng.normal(0, 1, (10, 3 * 32 * 32)).astype(np.float32)
    net = resnet18_cifar10(cutagi, gain_w=0.1, gain_b=0.1)
    net.to_device("cuda")
    updater = cutagi.OutputUpdater(net.device)
    metric = HRCSoftmaxMetric(10)
    batch = 64
    var_y = np.full(batch * 4, 1.0, np.float32)
    errors = []
    for _ in range(100):
        label = rng.integers(0, 10, batch)
        x = protos[label] + rng.normal(0, 0.5, (batch, 3072)).astype(np.float32)
        y, idx, _ = Utils().label_to_obs(label, 10)
        net.forward(x)
        m_pred, v_pred = net.get_outputs()
        errors.append(metric.error_rate(m_pred, v_pred, label))
        updater.update_using_indices(net.output_z_buffer, y, var_y, idx, net.input_delta_z_buffer)
        net.backward()
        net.step()
    assert np.all(np.isfinite(m_pred)) and v_pred.min() >= 0
    assert np.mean(errors[-20:]) < 0.8, errors[-20:]
