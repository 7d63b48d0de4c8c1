"""The CIFAR ResNet-18 of the reference's examples
(examples/tagi_resnet_model.py:17-147: `make_layer_block`, `resnet18_cifar10`),
built from this package's `cutagi` module, and the hierarchical-softmax label
encoding a training step needs (reference: class_to_obs, src/cost.cpp:76-143)."""
import numpy as np


def make_layer_block(c, in_c, out_c, stride=1, padding_type=1, gain_weight=1.0, gain_bias=1.0):
    return c.LayerBlock([
        c.Conv2d(in_c, out_c, 3, bias=False, stride=stride, padding=1, padding_type=padding_type,
                 gain_weight=gain_weight, gain_bias=gain_bias),
        c.MixtureReLU(), c.BatchNorm2d(out_c),
        c.Conv2d(out_c, out_c, 3, bias=False, padding=1, gain_weight=gain_weight,
                 gain_bias=gain_bias),
        c.MixtureReLU(), c.BatchNorm2d(out_c)])


def resnet18_cifar10(c=None, gain_w=1.0, gain_b=1.0):
    """3x32x32 input, 11 outputs (10 classes as a hierarchical softmax)."""
    if c is None:
        from . import cutagi as c

    def down(i, o):
        return c.ResNetBlock(
            make_layer_block(c, i, o, 2, 2, gain_weight=gain_w),
            c.LayerBlock([c.Conv2d(i, o, 2, bias=False, stride=2, gain_weight=gain_w),
                          c.MixtureReLU(), c.BatchNorm2d(o)]))

    same = lambda ch: c.ResNetBlock(make_layer_block(c, ch, ch, gain_weight=gain_w))
    return c.Sequential([
        c.Conv2d(3, 64, 3, bias=False, padding=1, in_width=32, in_height=32, gain_weight=gain_w),
        c.MixtureReLU(), c.BatchNorm2d(64),
        same(64), same(64),
        down(64, 128), same(128),
        down(128, 256), same(256),
        down(256, 512), same(512),
        c.AvgPool2d(4), c.Linear(512, 11, gain_weight=gain_w, gain_bias=gain_b)])


def hrc_softmax(num_classes):
    """Binary-tree encoding of `num_classes` labels. Returns (obs, idx, n_obs,
    n_outputs): obs[c] are the +-1 targets of class c along its path (most
    significant bit first), idx[c] the 1-based output units they belong to. Ten
    classes give 4 observations per label among 11 outputs."""
    n_obs = int(np.ceil(np.log2(num_classes)))
    obs = np.zeros((num_classes, n_obs), np.float32)
    idx = np.zeros((num_classes, n_obs), np.int32)
    nodes = {}  # (level, path prefix) -> output unit, numbered level by level
    for level in range(n_obs):
        for cls in range(num_classes):
            nodes.setdefault((level, cls >> (n_obs - level)), None)
    unit = 0
    for key in sorted(nodes):
        unit += 1
        nodes[key] = unit
    for cls in range(num_classes):
        for level in range(n_obs):
            bit = (cls >> (n_obs - 1 - level)) & 1
            obs[cls, level] = -1.0 if bit else 1.0
            idx[cls, level] = nodes[(level, cls >> (n_obs - level))]
    return obs, idx, n_obs, unit


def resnet18_cifar10_macs():
    """(multiply-accumulates per image, propagates innovations to its input) of every
    Conv2d / Linear layer of resnet18_cifar10, in network order: output channels x
    output pixels x kernel taps x input channels. The stem is the network's first
    layer and propagates nothing to the image."""
    out = [(64 * 32 * 32 * 9 * 3, False)]

    def main(i, o, w_out):
        return [(o * w_out * w_out * 9 * i, True), (o * w_out * w_out * 9 * o, True)]

    w, c = 32, 64
    for stage, o in enumerate((64, 128, 256, 512)):
        if stage == 0:
            out += main(c, o, w) + main(o, o, w)
        else:
            w //= 2
            out += main(c, o, w) + [(o * w * w * 4 * c, True)] + main(o, o, w)   # + 2x2 projection
        c = o
    out.append((512 * 11, True))
    return out
