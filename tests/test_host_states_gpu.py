"""State containers of the host classes in the corners the model cases do not reach:
state buffers built by the caller (odd sizes, reuse over several steps), and a
ResNetBlock whose buffers are not a multiple of four floats."""
import numpy as np
import pytest

from util import assert_close

pytestmark = pytest.mark.gpu


N_IN = 2 * 6 * 6


def _net_with_block(cutagi):
    cutagi.manual_seed(3)
    # two passes through the block's ping-pong buffers (each Conv2d absorbs its ReLU):
    # the block ends by trading arrays with the caller's input state
    block = cutagi.LayerBlock([cutagi.Conv2d(2, 3, 3, padding=1, in_width=6, in_height=6),
                               cutagi.ReLU(), cutagi.Conv2d(3, 2, 3, padding=1), cutagi.ReLU()])
    block.in_width, block.in_height, block.in_channels = 6, 6, 2
    net = cutagi.Sequential([block, cutagi.Linear(N_IN, 5)])
    net.to_device("cuda")
    net.preinit_layer()     # convolutions draw their weights here, not at the first forward
    return net


def test_callers_input_state_can_be_reused_over_steps():
    """A HiddenStates object handed to a network that opens with a LayerBlock stays the
    caller's: set again and fed again, every step gives what the array-input path
    gives on an identically initialised network, and the object is never taken for
    one of the network's own ping-pong buffers."""
    from cutagi_amd import cutagi
    B = 6
    rng = np.random.default_rng(0)
    xs = [rng.normal(0, 1, (B, N_IN)).astype(np.float32) for _ in range(3)]
    ys = [rng.normal(0, 1, B * 5).astype(np.float32) for _ in range(3)]
    var_y = np.full(B * 5, 0.5, np.float32)

    net_a, net_b = _net_with_block(cutagi), _net_with_block(cutagi)
    upd_a, upd_b = cutagi.OutputUpdater(net_a.device), cutagi.OutputUpdater(net_b.device)
    state = cutagi.HiddenStateCuda(B * 3 * 6 * 6 + 3, B)       # caller-owned, odd capacity
    for x, y in zip(xs, ys):
        state.set_input_x(x.ravel().tolist(), [], B)
        net_a.forward(state)
        net_b.forward(x)
        out_a, out_b = net_a.get_outputs(), net_b.get_outputs()
        assert np.array_equal(out_a[0], out_b[0]) and np.array_equal(out_a[1], out_b[1])
        upd_a.update(net_a.output_z_buffer, y, var_y, net_a.input_delta_z_buffer)
        upd_b.update(net_b.output_z_buffer, y, var_y, net_b.input_delta_z_buffer)
        net_a.backward()
        net_b.backward()
        net_a.step()
        net_b.step()
    assert net_a.state_dict() == net_b.state_dict()


def test_heteros_update_into_an_odd_sized_delta_state(oracle_lib):
    """A caller-built DeltaStates of odd size: both of its arrays still satisfy the
    alignment the heteroscedastic update asks for."""
    from cutagi_amd import cutagi
    cutagi.manual_seed(1)
    B, n_out = 3, 6                                     # 3 (mean, error-variance) pairs per sample
    net = cutagi.Sequential([cutagi.Linear(5, n_out)])
    net.to_device("cuda")
    rng = np.random.default_rng(1)
    net.forward(rng.normal(0, 1, (B, 5)).astype(np.float32))
    mu, var = net.get_outputs()
    # the error-variance units must be positive for the update to be defined
    y = rng.normal(0, 1, B * n_out // 2).astype(np.float32)
    delta = cutagi.DeltaStateCuda(B * n_out + 1, B)     # 19 floats
    updater = cutagi.OutputUpdater(net.device)
    updater.update_heteros(net.output_z_buffer, y, delta)
    delta.to_host()
    n = B * n_out
    zeros = np.zeros(n, np.float32)
    want_mu, want_var = oracle_lib.out_update_heteros(
        np.ascontiguousarray(mu.ravel()), np.ascontiguousarray(var.ravel()),
        np.ones(n, np.float32), y, zeros, zeros)
    got_mu, got_var = np.array(delta.delta_mu)[:n], np.array(delta.delta_var)[:n]
    ok = np.isfinite(want_mu) & np.isfinite(want_var)
    assert_close(got_mu[ok], want_mu[ok], "delta_mu")
    assert_close(got_var[ok], want_var[ok], "delta_var")


def test_resnet_block_whose_buffers_are_not_a_multiple_of_four(oracle_lib):
    """states * batch = 3 * 5 * 5 * 3 = 225 floats: the block's own delta buffers then
    start their variance array at an aligned offset, and the block runs (forward and
    backward) exactly as the same layers do outside a block plus the identity add."""
    from cutagi_amd import cutagi
    B, C, W = 3, 3, 5

    def layers():
        return [cutagi.Conv2d(C, C, 3, bias=False, stride=1, padding=1, padding_type=1,
                              in_width=W, in_height=W), cutagi.ReLU(),
                cutagi.Conv2d(C, C, 3, bias=False, stride=1, padding=1, padding_type=1)]

    cutagi.manual_seed(5)
    block = cutagi.ResNetBlock(cutagi.LayerBlock(layers()))
    block.in_width, block.in_height, block.in_channels = W, W, C
    res = cutagi.Sequential([block])
    cutagi.manual_seed(5)
    plain = cutagi.Sequential(layers())
    for net in (res, plain):
        cutagi.manual_seed(5)
        net.to_device("cuda")
        net.preinit_layer()
        net.input_state_update = True
    rng = np.random.default_rng(2)
    x = rng.normal(0, 1, (B, C * W * W)).astype(np.float32)
    n = B * C * W * W
    assert n % 4 != 0
    dmu = rng.normal(0, 0.1, n).astype(np.float32)
    dvar = (-rng.uniform(0, 1e-3, n)).astype(np.float32)
    outs, deltas = [], []
    for net in (res, plain):
        net.forward(x)
        outs.append(net.get_outputs())
        cap = net.input_delta_z_buffer.size      # set_delta_z takes whole-buffer vectors
        pad = lambda v: np.concatenate([v, np.zeros(cap - v.size, np.float32)])
        net.set_delta_z(pad(dmu), pad(dvar))
        net.backward()
        net.delta_z_to_host()
        d = net.output_delta_z_buffer
        deltas.append((np.array(d.delta_mu)[:n], np.array(d.delta_var)[:n]))
    # forward: block = plain + identity (input variance is zero)
    assert_close(outs[0][0].ravel(), outs[1][0].ravel() + x.ravel(), "mu_z of the block")
    assert_close(outs[0][1].ravel(), outs[1][1].ravel(), "var_z of the block")
    # backward: innovations of the main branch plus the identity's (input Jacobian is one)
    assert_close(deltas[0][0], deltas[1][0] + dmu, "delta_mu of the block")
    assert_close(deltas[0][1], deltas[1][1] + dvar, "delta_var of the block")
