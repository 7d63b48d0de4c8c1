"""Networks of the model-level parity tests, written once as text and built three
ways from it: by the compiled reference (oracle/ref_model.cpp parses the same
text and runs the reference's own Sequential / LayerBlock / ResNetBlock on the
CPU), by this package's host classes, and by the oracle-call emulation.

Grammar (tokens separated by blanks):
    net   := [ "input" W H C ] layer*
    layer := "Linear" K N bias
           | "Conv2d" fi fo k bias stride pad pad_type in_w in_h
           | "ReLU" | "MixtureReLU"
           | "BatchNorm2d" C eps momentum bias
           | "AvgPool2d" k stride pad pad_type
           | "LayerBlock" "[" layer* "]"
           | "ResNetBlock" "[" layer* "]" "[" layer* "]"   (second list empty: identity)
"input W H C" sets in_width / in_height / in_channels of the first layer, which a
network that starts with a block needs.

Parameters travel as one flat float32 vector in "leaf order": layers in reading
order, blocks expanded in place (main before shortcut), per layer mu_w, var_w,
mu_b, var_b and, for BatchNorm2d, mu_ra, var_ra.
"""
import numpy as np

PARAM_LAYERS = ("Linear", "Conv2d", "BatchNorm2d")
ARITY = {"Linear": 3, "Conv2d": 9, "ReLU": 0, "MixtureReLU": 0, "BatchNorm2d": 4, "AvgPool2d": 4}


def parse(spec):
    """-> (input dims or None, list of layers); a layer is (name, args) with args a
    tuple of numbers, ("LayerBlock", [layers]) or ("ResNetBlock", [main], [shortcut])."""
    tok = spec.split()
    pos = 0

    def block():
        nonlocal pos
        assert tok[pos] == "["
        pos += 1
        out = []
        while tok[pos] != "]":
            out.append(layer())
        pos += 1
        return out

    def layer():
        nonlocal pos
        name = tok[pos]
        pos += 1
        if name == "LayerBlock":
            return (name, block())
        if name == "ResNetBlock":
            main = block()
            return (name, main, block())
        n = ARITY[name]
        args = tuple(float(t) if name == "BatchNorm2d" and i in (1, 2) else int(t)
                     for i, t in enumerate(tok[pos:pos + n]))
        pos += n
        return (name, args)

    dims = None
    if tok and tok[0] == "input":
        dims = tuple(int(t) for t in tok[1:4])
        pos = 4
    layers = []
    while pos < len(tok):
        layers.append(layer())
    return dims, layers


def leaves(layers, prefix="", top=True):
    """(state-dict key suffix, layer) of every layer with parameters, in leaf order.
    Suffixes as the host classes name them: "<i>" at the top level, "<i>.<j>" inside
    a LayerBlock, "main.<i>.<j>" / "shortcut.<i>.<j>" inside a ResNetBlock."""
    out = []
    for i, L in enumerate(layers):
        sfx = str(i) if top else prefix + "." + str(i)
        if L[0] in PARAM_LAYERS:
            out.append((sfx, L))
        elif L[0] == "LayerBlock":
            out += leaves(L[1], sfx, False)
        elif L[0] == "ResNetBlock":
            out += leaves(L[1], "main." + sfx, False)
            out += leaves(L[2], "shortcut." + sfx, False)
    return out


def leaf_sizes(L):
    """Sizes of (mu_w, var_w, mu_b, var_b[, mu_ra, var_ra]) of one layer."""
    name, a = L
    if name == "Linear":
        nw, nb = a[0] * a[1], a[1] * a[2]
        return [nw, nw, nb, nb]
    if name == "Conv2d":
        nw, nb = a[0] * a[1] * a[2] * a[2], a[1] * a[3]
        return [nw, nw, nb, nb]
    c, nb = a[0], a[0] * a[3]
    return [c, c, nb, nb, c, c]


def fan_in(L):
    name, a = L
    return a[0] if name == "Linear" else a[0] * a[2] * a[2] if name == "Conv2d" else 1


def make_params(layers, seed, jitter=True, var_scale=1.0):
    """Seeded parameters in leaf order. Linear / Conv2d: mu_w ~ N(0, 1/K), var_w =
    var_scale/K (jittered by +-50 % so that a wrong index shows, unless jitter is
    off: the MLP configuration fixes var_w = 1/K, mu_b = 0, var_b = 1/K).
    BatchNorm2d: mu_w ~ 1, running averages at their initial 0 / 1."""
    rng = np.random.default_rng(seed)
    f = np.float32
    out = []
    for _, L in leaves(layers):
        sz = leaf_sizes(L)
        K = fan_in(L)
        if L[0] == "BatchNorm2d":
            c = sz[0]
            out += [(1 + 0.1 * rng.standard_normal(c)).astype(f),
                    rng.uniform(0.01, 0.05, c).astype(f),
                    (0.1 * rng.standard_normal(sz[2])).astype(f),
                    rng.uniform(0.01, 0.05, sz[2]).astype(f),
                    np.zeros(c, f), np.ones(c, f)]
            continue
        jw = rng.uniform(0.5, 1.5, sz[0]) if jitter else np.ones(sz[0])
        jb = rng.uniform(0.5, 1.5, sz[2]) if jitter else np.ones(sz[2])
        out += [rng.normal(0, K ** -0.5, sz[0]).astype(f), (var_scale * jw / K).astype(f),
                (rng.normal(0, 0.1, sz[2]) if jitter else np.zeros(sz[2])).astype(f),
                (var_scale * jb / K).astype(f)]
    return out


def layer_name(L):
    return L[0] + "Cuda"


def state_dict_of(layers, arrays):
    """Leaf-order arrays -> the state dict of the host classes (lists of floats)."""
    sd, k = {}, 0
    for sfx, L in leaves(layers):
        n = len(leaf_sizes(L))
        a = arrays[k:k + n]
        k += n
        sd[layer_name(L) + "." + sfx] = tuple(x.tolist() for x in a[:4])
    return sd


def build_host(c, spec):
    """The network from this package's `cutagi` module (not yet on the device)."""
    dims, layers = parse(spec)

    def make(L):
        name = L[0]
        if name == "Linear":
            return c.Linear(L[1][0], L[1][1], bool(L[1][2]))
        if name == "Conv2d":
            fi, fo, k, bias, s, p, pt, w, h = L[1]
            return c.Conv2d(fi, fo, k, bool(bias), s, p, pt, w, h)
        if name == "ReLU":
            return c.ReLU()
        if name == "MixtureReLU":
            return c.MixtureReLU()
        if name == "BatchNorm2d":
            ch, eps, mom, bias = L[1]
            return c.BatchNorm2d(int(ch), eps, mom, bool(bias))
        if name == "AvgPool2d":
            return c.AvgPool2d(*L[1])
        if name == "LayerBlock":
            return c.LayerBlock([make(x) for x in L[1]])
        main = c.LayerBlock([make(x) for x in L[1]])
        shortcut = c.LayerBlock([make(x) for x in L[2]]) if L[2] else None
        return c.ResNetBlock(main, shortcut) if shortcut is not None else c.ResNetBlock(main)

    made = [make(L) for L in layers]
    if dims is not None:
        made[0].in_width, made[0].in_height, made[0].in_channels = dims
    return c.Sequential(made)


def build_emulation(spec, arrays):
    """The network for tests/model_emulation.py with the given leaf-order arrays."""
    from model_emulation import BNorm, Block, Conv, Lin, MRelu, Pool, Relu, Res
    dims, layers = parse(spec)
    it = iter(arrays)
    state = {"w": dims[0] if dims else 0, "c": dims[2] if dims else 0}

    def out_width(k, s, p, pt, w):
        pad = 2 * p if pt == 1 else p if pt == 2 else 0
        return (w - k + pad) // s + 1

    def make(L):
        name = L[0]
        if name == "Linear":
            K, N, _ = L[1]
            return Lin(next(it), next(it), next(it), next(it), K, N)
        if name == "Conv2d":
            fi, fo, k, _, s, p, pt, w, _h = L[1]
            w = w or state["w"]
            layer = Conv(next(it), next(it), next(it), next(it), fi, fo, k, s, p, pt, w)
            state["w"], state["c"] = out_width(k, s, p, pt, w), fo
            return layer
        if name == "ReLU":
            return Relu()
        if name == "MixtureReLU":
            return MRelu()
        if name == "BatchNorm2d":
            ch, eps, mom, _ = L[1]
            layer = BNorm(next(it), next(it), next(it), next(it), int(ch), eps, mom)
            layer.mu_ra, layer.var_ra = next(it).copy(), next(it).copy()
            return layer
        if name == "AvgPool2d":
            k, s, p, pt = L[1]
            layer = Pool(k, s, p, pt, state["w"], state["c"])
            state["w"] = 1 if s == -1 else out_width(k, s, p, pt, state["w"])
            return layer
        if name == "LayerBlock":
            return Block([make(x) for x in L[1]])
        before = dict(state)
        main = Block([make(x) for x in L[1]])
        after = dict(state)
        shortcut = None
        if L[2]:
            state.update(before)
            shortcut = Block([make(x) for x in L[2]])
            state.update(after)
        return Res(main, shortcut)

    return [make(L) for L in layers]


def flat_params_of_emulation(emu_layers):
    """Leaf-order flat parameter vector of an emulated network."""
    from model_emulation import BNorm, param_layers
    out = []
    for _, L in param_layers(emu_layers):
        empty = np.zeros(0, np.float32)
        out += [L.mu_w.ravel(), L.var_w.ravel(), empty if L.mu_b is None else L.mu_b,
                empty if L.var_b is None else L.var_b]
        if isinstance(L, BNorm):
            out += [L.mu_ra, L.var_ra]
    return np.concatenate(out).astype(np.float32)


def flat_params_of_host(net, spec):
    """Leaf-order flat parameter vector of a host-class network (state dict plus the
    running averages of its BatchNorm2d layers)."""
    _, layers = parse(spec)
    sd = net.state_dict()
    ra = []  # running averages in leaf order
    for top in net.layers:
        stats = top.get_norm_mean_var()
        ra += list(zip(stats[0], stats[1]))
    out, k = [], 0
    for sfx, L in leaves(layers):
        p = sd[layer_name(L) + "." + sfx]
        out += [np.asarray(a, np.float32) for a in p]
        if L[0] == "BatchNorm2d":
            out += [np.asarray(ra[k][0], np.float32), np.asarray(ra[k][1], np.float32)]
            k += 1
    return np.concatenate(out)


# ---- the cases --------------------------------------------------------------------------

_RES_MAIN = ("Conv2d {i} {o} 3 0 {s} 1 {pt} 0 0 MixtureReLU BatchNorm2d {o} 1e-5 0.9 1 "
             "Conv2d {o} {o} 3 0 1 1 1 0 0 MixtureReLU BatchNorm2d {o} 1e-5 0.9 1")
_SMALL_RESNET = ("Conv2d 3 8 3 0 1 1 1 8 8 MixtureReLU BatchNorm2d 8 1e-5 0.9 1 "
                 "ResNetBlock [ " + _RES_MAIN.format(i=8, o=8, s=1, pt=1) + " ] [ ] "
                 "ResNetBlock [ " + _RES_MAIN.format(i=8, o=16, s=2, pt=2) + " ] "
                 "[ Conv2d 8 16 2 0 2 0 1 0 0 MixtureReLU BatchNorm2d 16 1e-5 0.9 1 ] "
                 "AvgPool2d 4 -1 0 0 Linear 16 11 1")
_BLOCK_FIRST = ("input 8 8 3 ResNetBlock [ Conv2d 3 8 3 1 1 1 1 8 8 ReLU BatchNorm2d 8 1e-5 0.9 1 "
                "Conv2d 8 8 3 0 1 1 1 0 0 ] [ Conv2d 3 8 1 0 1 0 1 8 8 ReLU BatchNorm2d 8 1e-5 0.9 0 ] "
                "MixtureReLU AvgPool2d 8 -1 0 0 Linear 8 5 1")
_LAYERBLOCK_FIRST = ("input 6 6 2 LayerBlock [ Conv2d 2 4 3 1 1 1 1 6 6 ReLU Conv2d 4 4 3 1 2 1 2 0 0 ] "
                     "ReLU Linear 36 7 1")

# update: 0 dense, 1 selected indices (n_enc observations per sample), 2 heteroscedastic
CASES = {
    # the MLP configuration exactly as the benchmark states it
    "mlp_config1": dict(spec="Linear 784 128 1 ReLU Linear 128 128 1 ReLU Linear 128 11 1",
                        B=32, steps=2, update=1, n_enc=4, jitter=False, var_x=False, seed=0),
    "mlp_input_update": dict(spec="Linear 20 12 1 ReLU Linear 12 6 1", B=5, steps=2, update=0,
                             input_state_update=True, var_x=True, seed=1),
    # variances large against the observation noise: some updated variances go
    # negative, are reset to 1e-5 and counted
    "mlp_negative_variances": dict(spec="Linear 16 24 1 ReLU Linear 24 4 1", B=32, steps=2,
                                   update=0, var_scale=0.16, var_y=1e-4, var_x=True, seed=2),
    "conv_relu_linear": dict(spec="Conv2d 3 8 3 1 1 1 1 8 8 ReLU Conv2d 8 8 3 0 2 1 2 0 0 ReLU "
                                  "Linear 128 5 1", B=4, steps=2, update=0, var_x=False, seed=3),
    "small_resnet": dict(spec=_SMALL_RESNET, B=6, steps=2, update=1, n_enc=4, var_x=False,
                         eval_forward=True, seed=4),
    "resnetblock_first": dict(spec=_BLOCK_FIRST, B=4, steps=2, update=0, var_x=True, seed=5),
    "resnetblock_first_input_update": dict(spec=_BLOCK_FIRST, B=4, steps=2, update=0, var_x=True,
                                           input_state_update=True, seed=6),
    "layerblock_first": dict(spec=_LAYERBLOCK_FIRST, B=3, steps=2, update=0, var_x=True, seed=7),
    "layerblock_first_input_update": dict(spec=_LAYERBLOCK_FIRST, B=3, steps=2, update=0,
                                          var_x=True, input_state_update=True, seed=8),
    "mlp_heteros": dict(spec="Linear 10 16 1 ReLU Linear 16 8 1", B=6, steps=2, update=2,
                        var_x=True, seed=9),
}

# threads of the reference run: above 1, so that BatchNorm2d takes the reference's
# default (multi-threaded) branch, which moves the running averages with the layer's
# momentum from the first batch on
REF_THREADS = 2


def case_inputs(name):
    """Seeded inputs of a case: params (leaf-order list), mu_x, var_x (or None), y,
    var_y, sel (or None), per step."""
    c = CASES[name]
    dims, layers = parse(c["spec"])
    params = make_params(layers, 100 + c["seed"], c.get("jitter", True), c.get("var_scale", 1.0))
    rng = np.random.default_rng(200 + c["seed"])
    first = layers[0]
    while first[0] in ("LayerBlock", "ResNetBlock"):
        first = first[1][0]
    if first[0] == "Linear":
        n_in = first[1][0]
    else:
        w = first[1][7] or dims[0]
        n_in = first[1][0] * w * w
    last = [L for _, L in leaves(layers)][-1]
    n_out = last[1][1]
    B, steps = c["B"], c["steps"]
    f = np.float32
    mu_x = rng.normal(0, 1, (steps, B * n_in)).astype(f)
    var_x = rng.uniform(0.01, 0.1, (steps, B * n_in)).astype(f) if c["var_x"] else None
    sel = None
    if c["update"] == 1:
        n_enc = c["n_enc"]
        sel = np.stack([np.concatenate([rng.choice(n_out, n_enc, replace=False) + 1
                                        for _ in range(B)]) for _ in range(steps)]).astype(np.int32)
        ny = B * n_enc
    elif c["update"] == 2:
        ny = B * n_out // 2
    else:
        ny = B * n_out
    y = rng.normal(0, 1, (steps, ny)).astype(f)
    var_y = np.full((steps, ny), c.get("var_y", 1.0), f)
    return dict(params=params, mu_x=mu_x, var_x=var_x, y=y, var_y=var_y, sel=sel, n_in=n_in,
                n_out=n_out)


def sample_index(n, limit=40000):
    """Entries of a length-n vector kept in a fixture: all of them up to `limit`,
    otherwise an evenly strided subset of about that many."""
    if n <= limit:
        return np.arange(n)
    return np.arange(0, n, -(-n // limit))


def resnet18_spec():
    """The CIFAR ResNet-18 of the reference's examples (examples/tagi_resnet_model.py:
    56-147) as a description: stem, eight residual blocks (three of them strided with a
    2x2 projection shortcut), global average pooling, an 11-unit head."""
    bn = "BatchNorm2d {c} 1e-5 0.9 1"

    def main(i, o, s, pt):
        return ("Conv2d {i} {o} 3 0 {s} 1 {pt} 0 0 MixtureReLU " + bn.format(c=o) +
                " Conv2d {o} {o} 3 0 1 1 1 0 0 MixtureReLU " + bn.format(c=o)).format(
                    i=i, o=o, s=s, pt=pt)

    def same(c):
        return "ResNetBlock [ " + main(c, c, 1, 1) + " ] [ ]"

    def down(i, o):
        return ("ResNetBlock [ " + main(i, o, 2, 2) + " ] [ Conv2d {i} {o} 2 0 2 0 1 0 0 MixtureReLU "
                .format(i=i, o=o) + bn.format(c=o) + " ]")

    return " ".join(["Conv2d 3 64 3 0 1 1 1 32 32 MixtureReLU " + bn.format(c=64),
                     same(64), same(64), down(64, 128), same(128), down(128, 256), same(256),
                     down(256, 512), same(512), "AvgPool2d 4 -1 0 0 Linear 512 11 1"])


# The ResNet-18 configuration at a batch the CPU reference finishes in seconds: one
# training step with the hierarchical-softmax update. `big`: left out of the CPU
# tests that re-run a case through the emulator (tens of seconds there).
CASES["resnet18_cifar_batch8"] = dict(spec=resnet18_spec(), B=8, steps=1, update=1, n_enc=4,
                                      var_x=False, seed=18, big=True)


def random_spec(rng):
    """A random small convolutional network as a description, with the image size
    and channel count tracked so that every layer fits: convolutions (3x3 same, 3x3
    stride 2 with one-sided padding, 2x2 stride 2, 1x1), activations, BatchNorm2d,
    identity and projection ResNetBlocks, LayerBlocks, average pooling, a Linear head.
    Returns (description, number of outputs)."""
    w = int(rng.choice([6, 8, 10, 12]))
    c = int(rng.integers(1, 4))
    first_w, first_c = w, c
    act = lambda: str(rng.choice(["ReLU", "MixtureReLU"]))
    bn = lambda ch: "BatchNorm2d %d 1e-5 0.9 %d" % (ch, int(rng.integers(0, 2)))

    def conv(ci, co, kind, size=0):
        k, s, p, pt = {"same": (3, 1, 1, 1), "down3": (3, 2, 1, 2), "down2": (2, 2, 0, 1),
                       "one": (1, 1, 0, 1)}[kind]
        return "Conv2d %d %d %d %d %d %d %d %d %d" % (ci, co, k, int(rng.integers(0, 2)), s, p, pt,
                                                     size, size)

    parts = []
    n_units = int(rng.integers(2, 5))
    for u in range(n_units):
        size = first_w if u == 0 else 0       # only the first convolution names its input size
        kinds = ["conv", "conv", "identity", "layerblock"]
        if w % 2 == 0 and w >= 4:
            kinds += ["projection", "pool", "convdown"]
        kind = str(rng.choice(kinds))
        if kind == "conv":
            co = int(rng.integers(2, 9))
            parts.append(conv(c, co, str(rng.choice(["same", "one"])), size))
            if rng.random() < 0.8:
                parts.append(act())
            if rng.random() < 0.5:
                parts.append(bn(co))
            c = co
        elif kind == "convdown":
            co = int(rng.integers(2, 9))
            parts.append(conv(c, co, str(rng.choice(["down3", "down2"])), size))
            parts.append(act())
            c, w = co, w // 2
        elif kind == "identity":
            main = [conv(c, c, "same", size), act(), bn(c), conv(c, c, "same")]
            if rng.random() < 0.5:
                main += [act(), bn(c)]
            parts.append("ResNetBlock [ " + " ".join(main) + " ] [ ]")
        elif kind == "projection":
            co = int(rng.integers(2, 9))
            main = [conv(c, co, "down3", size), act(), bn(co), conv(co, co, "same"), act(), bn(co)]
            short = [conv(c, co, "down2", size), act(), bn(co)]
            parts.append("ResNetBlock [ " + " ".join(main) + " ] [ " + " ".join(short) + " ]")
            c, w = co, w // 2
        elif kind == "layerblock":
            co = int(rng.integers(2, 7))
            parts.append("LayerBlock [ " + " ".join([conv(c, co, "same", size), act(),
                                                     conv(co, co, "one")]) + " ]")
            c = co
        else:  # pool
            if u == 0:      # a pooling layer cannot open the network: put a convolution first
                parts.append(conv(c, c, "same", size))
            parts.append("AvgPool2d 2 2 0 0")
            w //= 2
    if rng.random() < 0.5 and w > 1:
        parts.append("AvgPool2d %d -1 0 0" % w)
        w = 1
    if rng.random() < 0.5 and not parts[-1].endswith("ReLU"):   # (never two activations in a row:
        parts.append(act())                                      # MixtureReLU of a zero variance is 0/0)
    n_out = int(rng.integers(2, 8))
    parts.append("Linear %d %d 1" % (c * w * w, n_out))
    spec = " ".join(parts)
    if spec.startswith(("ResNetBlock", "LayerBlock")):
        spec = "input %d %d %d " % (first_w, first_w, first_c) + spec
    return spec, n_out


def _random_cases(n, seed):
    rng = np.random.default_rng(seed)
    out = {}
    for i in range(n):
        spec, n_out = random_spec(rng)
        indexed = n_out >= 3 and rng.random() < 0.4
        out["random_%02d" % i] = dict(spec=spec, B=int(rng.integers(2, 6)), steps=2,
                                      update=1 if indexed else 0, n_enc=min(3, n_out),
                                      var_x=bool(rng.random() < 0.5),
                                      input_state_update=bool(rng.random() < 0.5),
                                      seed=300 + i)
    return out


# ... and at the batch size the benchmark quotes (minutes of CPU for the reference: the
# fixture is written once; the GPU test regenerates the inputs from the seed)
CASES["resnet18_cifar_batch128"] = dict(spec=resnet18_spec(), B=128, steps=1, update=1, n_enc=4,
                                        var_x=False, seed=28, big=True)

# BatchNorm2d behind a fully-connected layer (one "pixel" per feature)
CASES["mlp_batchnorm"] = dict(spec="Linear 10 8 1 BatchNorm2d 8 1e-5 0.9 1 ReLU Linear 8 3 1", B=5,
                              steps=2, update=0, var_x=True, input_state_update=True, seed=19)

# sixteen networks nobody designed by hand
CASES.update(_random_cases(16, seed=4242))
