"""HIP graph replay of a Sequential's forward / backward passes (enable_graphs):
the same training run with replay on and off gives the same bits, step after step,
through batch-size changes, mode switches and parameter reloads; the replays are
separated by the eager parts of a step (input transfer, output update, parameter
update, output read-back with its synchronisation), as they are in use."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _mlp(cutagi):
    cutagi.manual_seed(0)
    net = cutagi.Sequential([cutagi.Linear(784, 128), cutagi.ReLU(), cutagi.Linear(128, 128),
                             cutagi.ReLU(), cutagi.Linear(128, 11)])
    net.to_device("cuda")
    return net


def _cnn(cutagi):
    cutagi.manual_seed(1)
    net = cutagi.Sequential([
        cutagi.Conv2d(3, 8, 3, bias=False, padding=1, in_width=8, in_height=8), cutagi.MixtureReLU(),
        cutagi.BatchNorm2d(8), cutagi.Conv2d(8, 8, 3, bias=True, stride=2, padding=1, padding_type=2),
        cutagi.ReLU(), cutagi.AvgPool2d(2, 2), cutagi.Linear(8 * 2 * 2, 5)])
    net.to_device("cuda")
    net.preinit_layer()
    return net


def _train(net, cutagi, xs, ys, n_out, observe=None):
    updater = cutagi.OutputUpdater(net.device)
    trace = []
    for step, (x, y) in enumerate(zip(xs, ys)):
        if observe is not None:
            observe(step, net)
        net.forward(x)
        mu, var = net.get_outputs()
        updater.update(net.output_z_buffer, y, np.full(y.size, 0.5, np.float32),
                       net.input_delta_z_buffer)
        net.backward()
        net.step()
        trace.append((mu.copy(), var.copy()))
    return trace, net.state_dict()


@pytest.mark.parametrize("make,n_in,n_out", [(_mlp, 784, 11), (_cnn, 3 * 8 * 8, 5)])
def test_replay_gives_the_eager_bits(make, n_in, n_out):
    from cutagi_amd import cutagi
    rng = np.random.default_rng(0)
    # the batch size changes twice; every size is seen often enough to be recorded
    sizes = [32] * 6 + [16] * 5 + [32] * 4
    xs = [rng.normal(0, 1, (b, n_in)).astype(np.float32) for b in sizes]
    ys = [rng.normal(0, 1, b * n_out).astype(np.float32) for b in sizes]
    eager_net = make(cutagi)
    eager, eager_params = _train(eager_net, cutagi, xs, ys, n_out)
    net = make(cutagi)
    net.enable_graphs(True)
    assert net.graphs_enabled()
    captured = []
    replay, replay_params = _train(net, cutagi, xs, ys, n_out,
                                   observe=lambda s, n: captured.append(n.graphs_captured()))
    for s, ((m0, v0), (m1, v1)) in enumerate(zip(eager, replay)):
        assert np.array_equal(m0, m1) and np.array_equal(v0, v1), "outputs differ at step %d" % s
    assert eager_params == replay_params
    # two eager runs per key, then a forward and a backward graph for batch 32, later for 16
    assert captured[2] == 0 and captured[4] == 2 and max(captured) >= 4
    net.enable_graphs(False)
    assert net.graphs_captured() == 0


def test_mode_switches_and_reloads_drop_the_recordings():
    from cutagi_amd import cutagi
    rng = np.random.default_rng(1)
    net = _mlp(cutagi)
    net.enable_graphs(True)
    twin = _mlp(cutagi)
    x = rng.normal(0, 1, (8, 784)).astype(np.float32)
    y = rng.normal(0, 1, 8 * 11).astype(np.float32)
    _train(net, cutagi, [x] * 5, [y] * 5, 11)
    _train(twin, cutagi, [x] * 5, [y] * 5, 11)
    assert net.graphs_captured() == 2
    net.eval()
    assert net.graphs_captured() == 0
    twin.eval()
    for _ in range(4):      # eval-mode forwards: eager twice, then recorded, same outputs
        net.forward(x)
        twin.forward(x)
        assert np.array_equal(net.get_outputs()[0], twin.get_outputs()[0])
    assert net.graphs_captured() == 1
    net.train()
    twin.train()
    # other parameters under a recorded graph: the recording must not survive the reload
    other = _mlp(cutagi)
    _train(other, cutagi, [x] * 2, [y] * 2, 11)
    sd = other.state_dict()
    net.load_state_dict(sd)
    twin.load_state_dict(sd)
    assert net.graphs_captured() == 0
    a, pa = _train(net, cutagi, [x] * 5, [y] * 5, 11)
    b, pb = _train(twin, cutagi, [x] * 5, [y] * 5, 11)
    assert all(np.array_equal(p[0], q[0]) for p, q in zip(a, b)) and pa == pb


def test_networks_with_blocks_stay_eager():
    from cutagi_amd import cutagi
    cutagi.manual_seed(2)
    block = cutagi.LayerBlock([cutagi.Conv2d(2, 2, 3, padding=1, in_width=4, in_height=4),
                               cutagi.ReLU(), cutagi.Conv2d(2, 2, 3, padding=1)])
    res = cutagi.ResNetBlock(block)
    res.in_width, res.in_height, res.in_channels = 4, 4, 2
    net = cutagi.Sequential([res, cutagi.Linear(32, 3)])
    net.to_device("cuda")
    net.enable_graphs(True)
    rng = np.random.default_rng(2)
    x = rng.normal(0, 1, (4, 32)).astype(np.float32)
    y = rng.normal(0, 1, 12).astype(np.float32)
    trace, _ = _train(net, cutagi, [x] * 5, [y] * 5, 3)
    assert net.graphs_captured() == 0 and all(np.all(np.isfinite(m)) for m, _ in trace)
