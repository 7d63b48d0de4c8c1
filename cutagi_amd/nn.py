"""The Python layer of the reference's user API (package ``pytagi.nn``) for the
classes on this path, over this package's ``cutagi`` module: code written as

    from pytagi.nn import Linear, OutputUpdater, ReLU, Sequential

runs with ``from cutagi_amd.nn import ...`` instead (reference: pytagi/nn/
sequential.py, linear.py, conv2d.py, activation.py, batch_norm.py, pooling.py,
layer_block.py, resnet_block.py, output_updater.py). The wrappers add no
arithmetic; every call goes to the C++ host classes, which call the HIP library.

``Utils`` and ``HRCSoftmaxMetric`` are the label helpers of the reference's
``pytagi`` package that the README classification example uses (hierarchical
softmax encoding, class probabilities, error rate).

Not here, because they are outside the Linear / Conv2d path: the other layer
families of pytagi.nn (LSTM, attention, normalisations other than BatchNorm2d,
max pooling, further activations), DDP and ``OutputUpdater.update_heteros``.
"""
import math

import numpy as np

from . import cutagi
from .resnet import hrc_softmax

BaseHiddenStates = cutagi.BaseHiddenStates
BaseDeltaStates = cutagi.BaseDeltaStates


def _f32(a):
    return None if a is None else np.ascontiguousarray(a, dtype=np.float32)


class BaseLayer:
    """A layer object of the user API; ``_cpp_backend`` is the C++ layer. Fields of
    the C++ layer (``mu_w``, ``var_w``, ``input_size``, ``device``, ...) read and
    write through."""

    _cpp_backend = None

    def __getattr__(self, name):
        backend = self.__dict__.get("_cpp_backend")
        if backend is None or name.startswith("__"):
            raise AttributeError(name)
        return getattr(backend, name)

    def __setattr__(self, name, value):
        backend = self.__dict__.get("_cpp_backend")
        if name != "_cpp_backend" and backend is not None and hasattr(backend, name) \
                and name not in self.__dict__:
            setattr(backend, name, value)
        else:
            object.__setattr__(self, name, value)

    def get_layer_info(self):
        return self._cpp_backend.get_layer_info()

    def get_layer_name(self):
        return self._cpp_backend.get_layer_name()

    def get_max_num_states(self):
        return self._cpp_backend.get_max_num_states()

    def init_weight_bias(self):
        self._cpp_backend.init_weight_bias()


class Linear(BaseLayer):
    def __init__(self, input_size, output_size, bias=True, gain_weight=1.0, gain_bias=1.0,
                 init_method="He"):
        self._cpp_backend = cutagi.Linear(input_size, output_size, bias, gain_weight, gain_bias,
                                          init_method)


class Conv2d(BaseLayer):
    def __init__(self, in_channels, out_channels, kernel_size, bias=True, stride=1, padding=0,
                 padding_type=1, in_width=0, in_height=0, gain_weight=1.0, gain_bias=1.0,
                 init_method="He"):
        self._cpp_backend = cutagi.Conv2d(in_channels, out_channels, kernel_size, bias, stride,
                                          padding, padding_type, in_width, in_height,
                                          gain_weight, gain_bias, init_method)


class ReLU(BaseLayer):
    def __init__(self):
        self._cpp_backend = cutagi.ReLU()


class MixtureReLU(BaseLayer):
    def __init__(self):
        self._cpp_backend = cutagi.MixtureReLU()


class BatchNorm2d(BaseLayer):
    def __init__(self, num_features, eps=1e-5, momentum=0.9, bias=True, gain_weight=1.0,
                 gain_bias=1.0):
        self._cpp_backend = cutagi.BatchNorm2d(num_features, eps, momentum, bias, gain_weight,
                                               gain_bias)


class AvgPool2d(BaseLayer):
    def __init__(self, kernel_size, stride=-1, padding=0, padding_type=0):
        self._cpp_backend = cutagi.AvgPool2d(kernel_size, stride, padding, padding_type)


class LayerBlock(BaseLayer):
    def __init__(self, *layers):
        self._cpp_backend = cutagi.LayerBlock([layer._cpp_backend for layer in layers])

    def switch_to_cuda(self):
        self._cpp_backend.switch_to_cuda()


class ResNetBlock(BaseLayer):
    def __init__(self, main_block, shortcut=None):
        if shortcut is not None:
            self._cpp_backend = cutagi.ResNetBlock(main_block._cpp_backend, shortcut._cpp_backend)
        else:
            self._cpp_backend = cutagi.ResNetBlock(main_block._cpp_backend)


class Sequential:
    """``net = Sequential(Linear(784, 128), ReLU(), ...); net.to_device("cuda");
    mu, var = net(x)``."""

    _FIELDS = ("output_z_buffer", "input_delta_z_buffer", "output_delta_z_buffer",
               "z_buffer_size", "z_buffer_block_size", "device", "input_state_update",
               "num_samples", "training", "param_update", "input_size")

    def __init__(self, *layers):
        object.__setattr__(self, "_cpp_backend",
                           cutagi.Sequential([layer._cpp_backend for layer in layers]))

    def __getattr__(self, name):
        if name in Sequential._FIELDS or name == "layers":
            return getattr(self._cpp_backend, name)
        raise AttributeError(name)

    def __setattr__(self, name, value):
        if name in Sequential._FIELDS:
            setattr(self._cpp_backend, name, value)
        else:
            object.__setattr__(self, name, value)

    def __call__(self, mu_x, var_x=None):
        return self.forward(mu_x, var_x)

    def to_device(self, device):
        self._cpp_backend.to_device(device)

    def params_to_host(self):
        self._cpp_backend.params_to_host()

    def params_to_device(self):
        self._cpp_backend.params_to_device()

    def set_threads(self, num_threads):
        self._cpp_backend.set_threads(num_threads)

    def train(self):
        self._cpp_backend.train()

    def eval(self):
        self._cpp_backend.eval()

    def forward(self, mu_x, var_x=None):
        if var_x is None:
            self._cpp_backend.forward(_f32(mu_x))
        else:
            self._cpp_backend.forward(_f32(mu_x), _f32(var_x))
        return self.get_outputs()

    def backward(self):
        self._cpp_backend.backward()

    def step(self):
        self._cpp_backend.step()

    def output_to_host(self):
        return self._cpp_backend.output_to_host()

    def delta_z_to_host(self):
        return self._cpp_backend.delta_z_to_host()

    def set_delta_z(self, delta_mu, delta_var):
        self._cpp_backend.set_delta_z(_f32(delta_mu), _f32(delta_var))

    def get_layer_stack_info(self):
        return self._cpp_backend.get_layer_stack_info()

    def preinit_layer(self):
        self._cpp_backend.preinit_layer()

    def get_neg_var_w_counter(self):
        return self._cpp_backend.get_neg_var_w_counter()

    def get_norm_mean_var(self):
        return self._cpp_backend.get_norm_mean_var()

    def save(self, filename):
        self._cpp_backend.save(filename)

    def load(self, filename):
        self._cpp_backend.load(filename)

    def save_csv(self, filename):
        self._cpp_backend.save_csv(filename)

    def load_csv(self, filename):
        self._cpp_backend.load_csv(filename)

    def parameters(self):
        return self._cpp_backend.parameters()

    def state_dict(self):
        return self._cpp_backend.state_dict()

    def load_state_dict(self, state_dict):
        self._cpp_backend.load_state_dict(state_dict)

    def params_from(self, other):
        self._cpp_backend.params_from(other._cpp_backend)

    def get_outputs(self):
        return self._cpp_backend.get_outputs()

    def get_input_states(self):
        return self._cpp_backend.get_input_states()


class OutputUpdater:
    """Innovations of the output layer from observations (dense), from a few
    observed output units per sample (``update_using_indices``, 1-based indices) or
    for an output layer that learns its own error variance (``update_heteros``).
    float32 / int32 numpy arrays are handed to the C++ side in place."""

    def __init__(self, model_device):
        self._cpp_backend = cutagi.OutputUpdater(model_device)

    def update(self, output_states, mu_obs, var_obs, delta_states):
        self._cpp_backend.update(output_states, _f32(mu_obs).ravel(), _f32(var_obs).ravel(),
                                 delta_states)

    def update_using_indices(self, output_states, mu_obs, var_obs, selected_idx, delta_states):
        idx = np.ascontiguousarray(selected_idx, dtype=np.int32).ravel()
        self._cpp_backend.update_using_indices(output_states, _f32(mu_obs).ravel(),
                                               _f32(var_obs).ravel(), idx, delta_states)

    def update_heteros(self, output_states, mu_obs, delta_states):
        """Output layer with a learned error variance: twice as many output units
        (mean, expected squared error) as observations."""
        self._cpp_backend.update_heteros(output_states, _f32(mu_obs).ravel(), delta_states)

    @property
    def device(self):
        return self._cpp_backend.device

    @device.setter
    def device(self, value):
        self._cpp_backend.device = value


class HRCSoftmax:
    """Binary-tree encoding of the class labels: ``obs`` (+-1 per level), ``idx``
    (1-based output unit per level), ``num_obs`` levels, ``len`` output units."""

    def __init__(self, num_classes):
        obs, idx, self.num_obs, self.len = hrc_softmax(num_classes)
        self.obs, self.idx = obs, idx       # [classes][num_obs]


class Utils:
    """Label helpers of the reference's ``pytagi.Utils`` for hierarchical-softmax
    classification (pytagi/tagi_utils.py:24-48,108-215 over src/cost.cpp:76-246)."""

    def get_hierarchical_softmax(self, num_classes):
        return HRCSoftmax(num_classes)

    def label_to_obs(self, labels, num_classes):
        """Observations (+-1) and 1-based output indices of each label's path in the
        binary tree, flattened sample by sample, and the path length."""
        hs = HRCSoftmax(num_classes)
        labels = np.asarray(labels, dtype=np.int64).ravel()
        return (np.ascontiguousarray(hs.obs[labels].ravel(), np.float32),
                np.ascontiguousarray(hs.idx[labels].ravel(), np.int32), hs.num_obs)

    def obs_to_label_prob(self, ma, Sa, hr_softmax, num_classes):
        """Class probabilities [samples][classes] from the output layer's means and
        variances: every tree node is a probit with scale 1/3, a class multiplies
        the branch probabilities along its path (reference: obs_to_class)."""
        ma = np.asarray(ma, np.float64).reshape(-1, hr_softmax.len)
        Sa = np.asarray(Sa, np.float64).reshape(-1, hr_softmax.len)
        z = ma / np.sqrt((1.0 / 3.0) ** 2 + Sa)
        p_node = 0.5 * np.vectorize(math.erfc)(-z / math.sqrt(2.0))
        picked = p_node[:, hr_softmax.idx - 1]                      # [samples][classes][levels]
        branch = np.where(hr_softmax.obs[None] == -1.0, np.abs(picked - 1.0), picked)
        return branch.prod(axis=2)[:, :num_classes].astype(np.float32)

    def get_labels(self, ma, Sa, hr_softmax, num_classes, batch_size):
        """Predicted labels and the class probabilities they come from."""
        prob = self.obs_to_label_prob(ma, Sa, hr_softmax, num_classes)
        assert prob.shape[0] == batch_size
        return prob.argmax(axis=1), prob

    def get_errors(self, ma, Sa, labels, hr_softmax, num_classes, batch_size):
        pred, prob = self.get_labels(ma, Sa, hr_softmax, num_classes, batch_size)
        return (pred != np.asarray(labels).ravel()).astype(np.int32), prob


class HRCSoftmaxMetric:
    """``metric = HRCSoftmaxMetric(10); metric.error_rate(m_pred, v_pred, label)``
    (reference: pytagi/metric.py:7-60)."""

    def __init__(self, num_classes):
        self.num_classes = num_classes
        self.utils = Utils()
        self.hrc_softmax = self.utils.get_hierarchical_softmax(num_classes)

    def get_predicted_labels(self, m_pred, v_pred):
        batch_size = np.asarray(m_pred).size // self.hrc_softmax.len
        return self.utils.get_labels(m_pred, v_pred, self.hrc_softmax, self.num_classes,
                                     batch_size)[0]

    def error_rate(self, m_pred, v_pred, label):
        pred = self.get_predicted_labels(m_pred, v_pred)
        return float(np.mean(pred != np.asarray(label).ravel()))
