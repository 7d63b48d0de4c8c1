// pybind11 module `cutagi`: the Python surface of the reference's extension
// module (src/bindings/*.cpp) for the classes on the hot path, with the same
// class, method and argument names, so that pytagi-style code runs unchanged.
#include <pybind11/numpy.h>
#include <pybind11/pybind11.h>
#include <pybind11/stl.h>

#include <cstring>

#include "../../include/tagi_hip.h"
#include "blocks.h"
#include "sequential.h"

namespace py = pybind11;
using namespace tagi_host;

namespace {
using FloatArray = py::array_t<float, py::array::c_style>;
using IntArray = py::array_t<int, py::array::c_style>;

std::vector<float> to_vec(const py::array_t<float, py::array::c_style | py::array::forcecast> &a) {
    std::vector<float> v(a.size());
    if (a.size()) std::memcpy(v.data(), a.data(), a.size() * sizeof(float));
    return v;
}
py::array_t<float> to_np(const std::vector<float> &v) { return py::array_t<float>(v.size(), v.data()); }
}  // namespace

PYBIND11_MODULE(cutagi, m) {
    m.doc() = "TAGI Linear/Conv2d hot path on MI355X (HIP backend)";

    py::class_<BaseHiddenStates, std::shared_ptr<BaseHiddenStates>>(m, "BaseHiddenStates")
        .def(py::init<size_t, size_t>())
        .def(py::init<>())
        .def_readwrite("mu_a", &BaseHiddenStates::mu_a)
        .def_readwrite("var_a", &BaseHiddenStates::var_a)
        .def_readwrite("jcb", &BaseHiddenStates::jcb)
        .def_readwrite("size", &BaseHiddenStates::size)
        .def_readwrite("block_size", &BaseHiddenStates::block_size)
        .def_readwrite("actual_size", &BaseHiddenStates::actual_size)
        .def_readwrite("width", &BaseHiddenStates::width)
        .def_readwrite("height", &BaseHiddenStates::height)
        .def_readwrite("depth", &BaseHiddenStates::depth)
        .def("set_input_x", &BaseHiddenStates::set_input_x)
        .def("get_name", &BaseHiddenStates::get_name)
        .def("set_size", &BaseHiddenStates::set_size)
        .def("swap", &BaseHiddenStates::swap)
        .def("copy_from", &BaseHiddenStates::copy_from, py::arg("source"), py::arg("num_data") = -1);
    py::class_<HiddenStateHip, BaseHiddenStates, std::shared_ptr<HiddenStateHip>>(m, "HiddenStateCuda")
        .def(py::init<size_t, size_t, int>(), py::arg("size"), py::arg("block_size"),
             py::arg("device_idx") = 0)
        .def("to_host", py::overload_cast<>(&HiddenStateHip::to_host))
        .def("to_device", &HiddenStateHip::to_device);

    py::class_<BaseDeltaStates, std::shared_ptr<BaseDeltaStates>>(m, "BaseDeltaStates")
        .def(py::init<size_t, size_t>())
        .def(py::init<>())
        .def_readwrite("delta_mu", &BaseDeltaStates::delta_mu)
        .def_readwrite("delta_var", &BaseDeltaStates::delta_var)
        .def_readwrite("size", &BaseDeltaStates::size)
        .def_readwrite("block_size", &BaseDeltaStates::block_size)
        .def_readwrite("actual_size", &BaseDeltaStates::actual_size)
        .def("get_name", &BaseDeltaStates::get_name)
        .def("reset_zeros", &BaseDeltaStates::reset_zeros)
        .def("copy_from", &BaseDeltaStates::copy_from, py::arg("source"), py::arg("num_data") = -1)
        .def("set_size", &BaseDeltaStates::set_size)
        .def("swap", &BaseDeltaStates::swap);
    py::class_<DeltaStateHip, BaseDeltaStates, std::shared_ptr<DeltaStateHip>>(m, "DeltaStateCuda")
        .def(py::init<size_t, size_t, int>(), py::arg("size"), py::arg("block_size"),
             py::arg("device_idx") = 0)
        .def("to_host", &DeltaStateHip::to_host)
        .def("to_device", &DeltaStateHip::to_device);

    py::class_<BaseLayer, std::shared_ptr<BaseLayer>>(m, "BaseLayer")
        .def_readwrite("input_size", &BaseLayer::input_size)
        .def_readwrite("output_size", &BaseLayer::output_size)
        .def_readwrite("in_width", &BaseLayer::in_width)
        .def_readwrite("in_height", &BaseLayer::in_height)
        .def_readwrite("in_channels", &BaseLayer::in_channels)
        .def_readwrite("out_width", &BaseLayer::out_width)
        .def_readwrite("out_height", &BaseLayer::out_height)
        .def_readwrite("out_channels", &BaseLayer::out_channels)
        .def_readwrite("bias", &BaseLayer::bias)
        .def_readwrite("num_weights", &BaseLayer::num_weights)
        .def_readwrite("num_biases", &BaseLayer::num_biases)
        .def_readwrite("mu_w", &BaseLayer::mu_w)
        .def_readwrite("var_w", &BaseLayer::var_w)
        .def_readwrite("mu_b", &BaseLayer::mu_b)
        .def_readwrite("var_b", &BaseLayer::var_b)
        .def_readwrite("delta_mu_w", &BaseLayer::delta_mu_w)
        .def_readwrite("delta_var_w", &BaseLayer::delta_var_w)
        .def_readwrite("delta_mu_b", &BaseLayer::delta_mu_b)
        .def_readwrite("delta_var_b", &BaseLayer::delta_var_b)
        .def_readwrite("num_threads", &BaseLayer::num_threads)
        .def_readwrite("training", &BaseLayer::training)
        .def_readwrite("param_update", &BaseLayer::param_update)
        .def_readwrite("cap_factor_update", &BaseLayer::cap_factor_update)
        .def_readwrite("device", &BaseLayer::device)
        .def("forward", &BaseLayer::forward)
        .def("backward", &BaseLayer::backward, py::arg("input_delta_states"),
             py::arg("output_delta_states"), py::arg("temp_states"), py::arg("state_udapte") = true)
        .def("get_layer_info", &BaseLayer::get_layer_info)
        .def("get_layer_name", &BaseLayer::get_layer_name)
        .def("get_max_num_states", &BaseLayer::get_max_num_states)
        .def("preinit_layer", &BaseLayer::preinit_layer)
        .def("params_to_host", &BaseLayer::params_to_host)
        .def("params_to_device", &BaseLayer::params_to_device)
        .def("delta_params_to_host", &BaseLayer::delta_params_to_host)
        .def("delta_params_to_device", &BaseLayer::delta_params_to_device)
        .def("update_weights", &BaseLayer::update_weights)
        .def("update_biases", &BaseLayer::update_biases)
        .def("raw_update_weights", &BaseLayer::raw_update_weights)
        .def("raw_update_biases", &BaseLayer::raw_update_biases)
        .def("set_cuda_threads", [](BaseLayer &self, int num) {
                 // launch shapes are chosen by the kernels here; the value is kept for
                 // code written for the reference's device layers
                 if (auto *d = dynamic_cast<BaseLayerHip *>(&self)) d->set_cuda_threads(num);
             })
        .def("get_norm_mean_var", &BaseLayer::get_norm_mean_var)
        .def("to_cuda", [](BaseLayer &self, int device_idx) {
                 return std::shared_ptr<BaseLayer>(self.to_cuda(device_idx));
             }, py::arg("device_idx") = 0);

    py::class_<Linear, BaseLayer, std::shared_ptr<Linear>>(m, "Linear")
        .def(py::init<size_t, size_t, bool, float, float, std::string, int>(), py::arg("ip_size"),
             py::arg("op_size"), py::arg("bias") = true, py::arg("gain_weight") = 1.0f,
             py::arg("gain_bias") = 1.0f, py::arg("method") = "He", py::arg("device_idx") = 0)
        .def_readwrite("gain_w", &Linear::gain_w)
        .def_readwrite("gain_b", &Linear::gain_b)
        .def_readwrite("init_method", &Linear::init_method)
        .def("init_weight_bias", &Linear::init_weight_bias);
    py::class_<Conv2d, BaseLayer, std::shared_ptr<Conv2d>>(m, "Conv2d")
        .def(py::init<size_t, size_t, size_t, bool, int, int, int, size_t, size_t, float, float,
                      std::string, int>(),
             py::arg("in_channels"), py::arg("out_channels"), py::arg("kernel_size"),
             py::arg("bias") = true, py::arg("stride") = 1, py::arg("padding") = 0,
             py::arg("padding_type") = 1, py::arg("in_width") = 0, py::arg("in_height") = 0,
             py::arg("gain_weight") = 1.0f, py::arg("gain_bias") = 1.0f,
             py::arg("init_method") = "He", py::arg("device_idx") = 0)
        .def_readwrite("gain_w", &Conv2d::gain_w)
        .def_readwrite("gain_b", &Conv2d::gain_b)
        .def_readwrite("init_method", &Conv2d::init_method)
        .def("init_weight_bias", &Conv2d::init_weight_bias);
    py::class_<ReLU, BaseLayer, std::shared_ptr<ReLU>>(m, "ReLU").def(py::init<>());
    py::class_<MixtureReLU, BaseLayer, std::shared_ptr<MixtureReLU>>(m, "MixtureReLU")
        .def(py::init<>());
    // argument names and defaults of the reference's binding
    // (src/bindings/norm_layer_bindings.cpp:31-42)
    py::class_<BatchNorm2d, BaseLayer, std::shared_ptr<BatchNorm2d>>(m, "BatchNorm2d")
        .def(py::init<int, float, float, bool, float, float>(), py::arg("num_features"),
             py::arg("eps") = 1e-4f, py::arg("mometum") = 0.9f, py::arg("bias") = true,
             py::arg("gain_weight") = 1.0f, py::arg("gain_bias") = 1.0f)
        .def_readwrite("mu_ra", &BatchNorm2d::mu_ra)
        .def_readwrite("var_ra", &BatchNorm2d::var_ra)
        .def("init_weight_bias", &BatchNorm2d::init_weight_bias);
    py::class_<BatchNorm2dHip, BaseLayer, std::shared_ptr<BatchNorm2dHip>>(m, "BatchNorm2dCuda")
        .def("get_norm_mean_var", &BatchNorm2dHip::get_norm_mean_var);
    py::class_<AvgPool2d, BaseLayer, std::shared_ptr<AvgPool2d>>(m, "AvgPool2d")
        .def(py::init<size_t, int, int, int, int>(), py::arg("kernel_size"),
             py::arg("stride") = -1, py::arg("padding") = 0, py::arg("padding_type") = 0,
             py::arg("device_idx") = 0);
    py::class_<LayerBlock, BaseLayer, std::shared_ptr<LayerBlock>>(m, "LayerBlock")
        .def(py::init<>())
        .def(py::init([](const std::vector<std::shared_ptr<BaseLayer>> &layers) {
            return std::make_shared<LayerBlock>(layers);
        }))
        .def("add_layer", &LayerBlock::add_layer)
        .def("switch_to_cuda", &LayerBlock::switch_to_cuda)
        .def_readwrite("layers", &LayerBlock::layers);
    py::class_<ResNetBlock, BaseLayer, std::shared_ptr<ResNetBlock>>(m, "ResNetBlock")
        .def(py::init<std::shared_ptr<BaseLayer>, std::shared_ptr<BaseLayer>>(),
             py::arg("main_block"), py::arg("shortcut") = nullptr)
        .def_readwrite("main_block", &ResNetBlock::main_block)
        .def_readwrite("shortcut", &ResNetBlock::shortcut)
        .def_readwrite("input_z", &ResNetBlock::input_z)
        .def_readwrite("input_delta_z", &ResNetBlock::input_delta_z)
        .def_readwrite("shortcut_output_z", &ResNetBlock::shortcut_output_z)
        .def_readwrite("shortcut_output_delta_z", &ResNetBlock::shortcut_output_delta_z);

    py::class_<OutputUpdater, std::shared_ptr<OutputUpdater>>(m, "OutputUpdater")
        .def(py::init<const std::string>())
        // float32 / int32 numpy arrays are read in place; anything else (lists, as in
        // the reference's binding, or arrays of another type) goes through std::vector
        .def("update",
             [](OutputUpdater &self, BaseHiddenStates &out, const FloatArray &mu,
                const FloatArray &var, BaseDeltaStates &delta) {
                 if (mu.size() != var.size())
                     throw std::runtime_error("Observation size does not fit the output buffers");
                 self.update_raw(out, mu.data(), var.data(), (size_t)mu.size(), delta);
             },
             py::arg("output_states"), py::arg("mu_obs").noconvert(),
             py::arg("var_obs").noconvert(), py::arg("delta_states"))
        .def("update", &OutputUpdater::update, py::arg("output_states"), py::arg("mu_obs"),
             py::arg("var_obs"), py::arg("delta_states"))
        .def("update_using_indices",
             [](OutputUpdater &self, BaseHiddenStates &out, const FloatArray &mu,
                const FloatArray &var, const IntArray &idx, BaseDeltaStates &delta) {
                 if (mu.size() != var.size() || mu.size() != idx.size())
                     throw std::runtime_error("Observations, variances and indices must have "
                                              "one size, a multiple of the batch size");
                 self.update_using_indices_raw(out, mu.data(), var.data(), idx.data(),
                                               (size_t)mu.size(), delta);
             },
             py::arg("output_states"), py::arg("mu_obs").noconvert(),
             py::arg("var_obs").noconvert(), py::arg("selected_idx").noconvert(),
             py::arg("delta_states"))
        .def("update_using_indices", &OutputUpdater::update_using_indices,
             py::arg("output_states"), py::arg("mu_obs"), py::arg("var_obs"),
             py::arg("selected_idx"), py::arg("delta_states"))
        .def("update_heteros",
             [](OutputUpdater &self, BaseHiddenStates &out, const FloatArray &mu,
                BaseDeltaStates &delta) {
                 self.update_heteros_raw(out, mu.data(), (size_t)mu.size(), delta);
             },
             py::arg("output_states"), py::arg("mu_obs").noconvert(), py::arg("delta_states"))
        .def("update_heteros", &OutputUpdater::update_heteros, py::arg("output_states"),
             py::arg("mu_obs"), py::arg("delta_states"))
        .def_readwrite("device", &OutputUpdater::device);

    py::class_<Sequential, std::shared_ptr<Sequential>>(m, "Sequential")
        .def(py::init<>())
        .def(py::init([](const std::vector<std::shared_ptr<BaseLayer>> &layers) {
            auto seq = std::make_shared<Sequential>();
            for (const auto &layer : layers) seq->add_layer(layer);
            seq->add_layers();
            return seq;
        }))
        .def_readwrite("layers", &Sequential::layers)
        .def_readwrite("output_z_buffer", &Sequential::output_z_buffer)
        .def_readwrite("input_delta_z_buffer", &Sequential::input_delta_z_buffer)
        .def_readwrite("output_delta_z_buffer", &Sequential::output_delta_z_buffer)
        .def_readwrite("z_buffer_size", &Sequential::z_buffer_size)
        .def_readwrite("z_buffer_block_size", &Sequential::z_buffer_block_size)
        .def_readwrite("input_size", &Sequential::input_size)
        .def_readwrite("num_samples", &Sequential::num_samples)
        .def_readwrite("training", &Sequential::training)
        .def_readwrite("param_update", &Sequential::param_update)
        .def_readwrite("device", &Sequential::device)
        .def_readwrite("input_state_update", &Sequential::input_state_update)
        .def_readwrite("num_threads", &Sequential::num_threads)
        .def("to_device", &Sequential::to_device)
        .def("params_to_host", &Sequential::params_to_host)
        .def("params_to_device", &Sequential::params_to_device)
        .def("set_threads", &Sequential::set_threads)
        .def("train", &Sequential::train)
        .def("eval", &Sequential::eval)
        .def("forward",
             [](Sequential &self, py::object arg1, py::object arg2) {
                 if (py::isinstance<BaseHiddenStates>(arg1)) {
                     self.forward(arg1.cast<BaseHiddenStates &>());
                     return;
                 }
                 // numpy memory goes to the device as it is (no intermediate vector)
                 using Arr = py::array_t<float, py::array::c_style | py::array::forcecast>;
                 Arr mu = arg1.cast<Arr>();
                 if (arg2.is_none()) {
                     self.forward(mu.data(), nullptr, (size_t)mu.size());
                 } else {
                     Arr var = arg2.cast<Arr>();
                     if (var.size() != mu.size())
                         throw std::runtime_error("Input mean and variance differ in size");
                     self.forward(mu.data(), var.data(), (size_t)mu.size());
                 }
             },
             py::arg("mu_x"), py::arg("var_x") = py::none())
        .def("backward", &Sequential::backward)
        .def("step", &Sequential::step)
        // not in the reference: record the launches of a forward / backward pass into HIP
        // graphs and replay them (see Sequential::enable_graphs)
        .def("enable_graphs", &Sequential::enable_graphs, py::arg("on") = true)
        .def("graphs_enabled", &Sequential::graphs_enabled)
        .def("graphs_captured", &Sequential::graphs_captured)
        .def("output_to_host", &Sequential::output_to_host)
        .def("delta_z_to_host", &Sequential::delta_z_to_host)
        .def("set_delta_z",
             [](Sequential &self, py::array_t<float, py::array::c_style | py::array::forcecast> mu,
                py::array_t<float, py::array::c_style | py::array::forcecast> var) {
                 auto m_ = to_vec(mu), v_ = to_vec(var);
                 self.set_delta_z(m_, v_);
             },
             py::arg("delta_mu"), py::arg("delta_var"))
        .def("get_layer_stack_info", &Sequential::get_layer_stack_info)
        .def("preinit_layer", &Sequential::preinit_layer)
        .def("get_neg_var_w_counter", &Sequential::get_neg_var_w_counter)
        .def("save", &Sequential::save)
        .def("load", &Sequential::load)
        .def("save_csv", &Sequential::save_csv)
        .def("get_norm_mean_var", &Sequential::get_norm_mean_var)
        .def("load_csv", &Sequential::load_csv)
        .def("params_from", &Sequential::params_from)
        .def("parameters", &Sequential::parameters)
        .def("state_dict", &Sequential::state_dict)
        .def("load_state_dict", &Sequential::load_state_dict)
        .def("get_outputs",
             [](Sequential &self) {
                 auto r = self.get_outputs_vec();
                 return std::make_tuple(to_np(std::get<0>(r)), to_np(std::get<1>(r)));
             })
        .def("get_input_states", [](Sequential &self) {
            auto r = self.get_input_states_vec();
            return std::make_tuple(to_np(std::get<0>(r)), to_np(std::get<1>(r)));
        });

    m.def("manual_seed", &manual_seed);
    // not in the reference: ReLU / MixtureReLU after a Linear / Conv2d layer run in that
    // layer's kernel by default; False gives every layer its own launch again
    m.def("set_fused_activations", &set_fused_activations, py::arg("on"));
    m.def("is_cuda_available", &is_cuda_available);
    m.def("get_cuda_device_count", &get_cuda_device_count);
    m.def("get_cuda_current_device", &get_current_cuda_device);
    m.def("set_cuda_device", &set_cuda_device);
    m.def("is_cuda_device_available", &is_cuda_device_available);
    m.def("is_nccl_available", &is_nccl_available);
    m.def("get_cuda_device_properties", &get_cuda_device_properties);
    // (free, total) in bytes; the reference's binding of the reference-argument
    // form is what pytagi.cuda.get_device_memory documents as this pair
    m.def("get_cuda_device_memory", [](int device_index) {
        size_t free_memory = 0, total_memory = 0;
        if (!get_cuda_device_memory(device_index, free_memory, total_memory))
            throw std::runtime_error("could not query the device memory");
        return std::make_tuple(free_memory, total_memory);
    });
}
