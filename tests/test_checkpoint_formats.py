"""Checkpoint files are interchangeable with the reference's: a binary checkpoint the
reference's own layer classes wrote loads into the host classes and is written back
byte for byte, a file the host classes wrote loads with the reference's loader, and
the text (csv) format reads and writes the same numbers.

The reference side is the compiled reference (oracle/_ref); the tests skip where it
is not built. Model 1 covers every layer kind that owns a file section: Conv2d,
BatchNorm2d (with its running averages), activations and AvgPool2d (a name only),
LayerBlock and ResNetBlock (their members in order), Linear."""
import os

import numpy as np
import pytest

import oracle


@pytest.fixture(scope="module")
def ref():
    r = oracle.load_ref()
    if r is None or not hasattr(r.lib, "ref_checkpoint_save"):
        pytest.skip("compiled reference not available")
    return r


def build(model):
    from cutagi_amd import cutagi as ct
    if model == 0:
        return ct.Sequential([ct.Linear(13, 7), ct.ReLU(), ct.Linear(7, 3)])
    main = ct.LayerBlock([ct.Conv2d(4, 8, 3, False, 2, 1, 2), ct.ReLU(), ct.BatchNorm2d(8)])
    shortcut = ct.LayerBlock([ct.Conv2d(4, 8, 2, False, 2)])
    return ct.Sequential([ct.Conv2d(3, 4, 3, False, 1, 1, 1, 8, 8), ct.BatchNorm2d(4),
                          ct.MixtureReLU(), ct.ResNetBlock(main, shortcut), ct.AvgPool2d(4),
                          ct.Linear(8, 5)])


def pattern(sizes):
    """value(leaf, array, i) of ref_checkpoint_save for leaves with the given array sizes."""
    out = []
    for leaf, arrays in enumerate(sizes):
        for a, n in enumerate(arrays):
            out.append(np.float32(leaf + 1) + np.float32(0.1) * np.float32(a + 1)
                       + np.float32(1e-4) * np.arange(n, dtype=np.float32))
    return np.concatenate(out).astype(np.float32)


SIZES = {
    0: [(91, 91, 7, 7), (0, 0, 0, 0), (21, 21, 3, 3)],
    1: [(108, 108, 0, 0), (4, 4, 4, 4, 4, 4), (0, 0, 0, 0), (288, 288, 0, 0), (0, 0, 0, 0),
        (8, 8, 8, 8, 8, 8), (128, 128, 0, 0), (0, 0, 0, 0), (40, 40, 5, 5)],
}


@pytest.mark.parametrize("model", [0, 1])
def test_reference_checkpoint_loads_and_is_rewritten_byte_for_byte(ref, model, tmp_path):
    theirs = str(tmp_path / "ref.bin")
    n = ref.checkpoint_save(model, theirs)
    assert n == sum(sum(a) for a in SIZES[model])
    net = build(model)
    net.load(theirs)
    # the parameters arrived where they belong
    sd = net.state_dict()
    first = "Linear.0" if model == 0 else "Conv2d.0"
    want = pattern(SIZES[model])
    n_w = SIZES[model][0][0]
    assert np.array_equal(np.asarray(sd[first][0], np.float32), want[:n_w])
    assert np.array_equal(np.asarray(sd[first][1], np.float32), want[n_w:2 * n_w])
    # and every byte of the file is reproduced (names, order, running averages)
    ours = str(tmp_path / "sub" / "ours.bin")  # the directory is created, as in the reference
    net.save(ours)
    assert open(ours, "rb").read() == open(theirs, "rb").read()


@pytest.mark.parametrize("model", [0, 1])
def test_host_checkpoint_loads_with_the_reference_loader(ref, model, tmp_path):
    theirs = str(tmp_path / "ref.bin")
    ref.checkpoint_save(model, theirs)
    net = build(model)
    net.load(theirs)
    # change one value so that the file is ours, not a copy
    sd = net.state_dict()
    key = "Linear.2" if model == 0 else "Linear.5"
    mu_w, var_w, mu_b, var_b = [list(v) for v in sd[key]]
    mu_w[3] = -7.25
    sd[key] = (mu_w, var_w, mu_b, var_b)
    net.load_state_dict(sd)
    ours = str(tmp_path / "ours.bin")
    net.save(ours)
    got = ref.checkpoint_load(model, ours)
    want = pattern(SIZES[model])
    at = sum(sum(a) for a in SIZES[model][:-1]) + 3
    want[at] = -7.25
    assert got is not None and np.array_equal(got, want)


def test_reference_loader_rejects_a_different_architecture(ref, tmp_path):
    net = build(0)
    path = str(tmp_path / "mlp.bin")
    net.preinit_layer()
    net.save(path)
    assert ref.checkpoint_load(1, path) is None
    with pytest.raises(RuntimeError):
        build(1).load(path)


def test_csv_checkpoint_matches_the_reference_text_format(ref, tmp_path):
    from cutagi_amd import cutagi as ct
    ct.manual_seed(3)
    net = ct.Sequential([ct.Linear(13, 7), ct.ReLU(), ct.Linear(7, 3)])
    stem = str(tmp_path / "csv" / "net")
    net.save_csv(stem)
    sd = net.state_dict()
    cols = [np.concatenate([np.asarray(sd[k][j], np.float32) for k in ("Linear.0", "Linear.2")])
            for j in range(4)]
    for j, suffix in enumerate(("_1_mw.csv", "_2_Sw.csv", "_3_mb.csv", "_4_Sb.csv")):
        # the same text as the reference's writer produces for these numbers
        ref.write_csv(str(tmp_path / "theirs.csv"), cols[j])
        assert open(stem + suffix).read() == open(str(tmp_path / "theirs.csv")).read()
        # and the reference's reader recovers what ours wrote
        back = ref.read_csv(stem + suffix, cols[j].size)
        assert back is not None and np.allclose(back, cols[j], rtol=1e-5, atol=0)
    # loading: files written by the reference's writer from other numbers
    rng = np.random.default_rng(0)
    new = [rng.standard_normal(c.size).astype(np.float32) * (1 if j % 2 == 0 else 0) +
           (0 if j % 2 == 0 else rng.uniform(0.1, 1, c.size).astype(np.float32))
           for j, c in enumerate(cols)]
    stem2 = str(tmp_path / "theirs")
    for j, suffix in enumerate(("_1_mw.csv", "_2_Sw.csv", "_3_mb.csv", "_4_Sb.csv")):
        ref.write_csv(stem2 + suffix, new[j])
    net.load_csv(stem2)
    sd = net.state_dict()
    for j in range(4):
        got = np.concatenate([np.asarray(sd[k][j], np.float32) for k in ("Linear.0", "Linear.2")])
        want = ref.read_csv(stem2 + ("_1_mw.csv", "_2_Sw.csv", "_3_mb.csv", "_4_Sb.csv")[j],
                            got.size)
        assert np.array_equal(got, want)
    # a file that is too short is an error, as in the reference
    open(stem2 + "_1_mw.csv", "w").write("1.0\n2.0\n")
    with pytest.raises(RuntimeError):
        net.load_csv(stem2)
    assert ref.read_csv(stem2 + "_1_mw.csv", cols[0].size) is None


@pytest.mark.gpu
def test_model_trained_on_the_gpu_loads_with_the_reference_loader(ref, tmp_path):
    """One training step of zoo model 1 on the GPU, saved from the device classes
    (binary and csv); the reference's loader reads back exactly the parameters and
    running averages the device holds."""
    from cutagi_amd import cutagi as ct
    ct.manual_seed(5)
    rng = np.random.default_rng(5)
    net = build(1)
    net.to_device("cuda")
    B = 6
    x = rng.normal(0, 1, (B, 3 * 64)).astype(np.float32)
    net.forward(x)
    upd = ct.OutputUpdater("cuda")
    y = rng.normal(0, 1, B * 5).astype(np.float32)
    upd.update(net.output_z_buffer, y.tolist(), [0.5] * (B * 5), net.input_delta_z_buffer)
    net.backward()
    net.step()
    path = str(tmp_path / "gpu.bin")
    net.save(path)
    got = ref.checkpoint_load(1, path)
    assert got is not None and got.size == sum(sum(a) for a in SIZES[1])
    sd = net.state_dict()
    # leaves in saving order: stem conv, stem norm, (mixture relu), main conv, (relu),
    # main norm, shortcut conv, (pool), linear
    def one(kind, suffix):
        return [np.asarray(v, np.float32) for v in sd[kind + "Cuda." + suffix]]
    stem_bn = net.layers[1].get_norm_mean_var()
    want = []
    want += one("Conv2d", "0")
    want += one("BatchNorm2d", "1") + [np.asarray(stem_bn[0], np.float32).ravel(),
                                         np.asarray(stem_bn[1], np.float32).ravel()]
    want += one("Conv2d", "main.3.0")
    main_bn = one("BatchNorm2d", "main.3.2")
    at = sum(w.size for w in want) + sum(w.size for w in main_bn)
    want += main_bn + [got[at:at + 8], got[at + 8:at + 16]]  # running averages: not in the map
    want += one("Conv2d", "shortcut.3.0")
    want += one("Linear", "5")
    want = np.concatenate([w.ravel() for w in want])
    assert np.array_equal(got, want)
    # the block's norm layer saved averages that one batch has moved (they start at 0 and 1)
    assert np.any(got[at:at + 8] != 0) and np.all(got[at + 8:at + 16] != 1)
    # the parameters moved away from their initial values and variances stay positive
    assert np.all(np.isfinite(got))
    # csv: top-level layers only, read by the reference's reader
    stem = str(tmp_path / "gpu")
    net.save_csv(stem)
    mw = ref.read_csv(stem + "_1_mw.csv", 108 + 4 + 40)
    top = np.concatenate([one("Conv2d", "0")[0], one("BatchNorm2d", "1")[0], one("Linear", "5")[0]])
    assert mw is not None and np.allclose(mw, top, rtol=1e-5, atol=1e-30)
