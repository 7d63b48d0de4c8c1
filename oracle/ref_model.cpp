// Model-level runner over the reference's own drivers: builds a network of the
// reference's layer classes from a small text description, loads given
// parameters, and runs training steps through the reference's
// Sequential::forward -> OutputUpdater -> Sequential::backward -> Sequential::step
// (src/sequential.cpp:279-448, src/layer_block.cpp:150-218,
// src/resnet_block.cpp:188-277, src/base_output_updater.cpp:269-386) on the CPU.
// TEST INFRASTRUCTURE ONLY: compiled by oracle/Makefile into
// oracle/_ref/libtagi_ref.so together with the reference sources where they lie;
// used to write tests/golden/models.npz. No reference source is copied here.
//
// Description grammar (tokens separated by blanks):
//   net    := [ "input" W H C ] layer*
//   layer  := "Linear" K N bias
//           | "Conv2d" fi fo k bias stride pad pad_type in_w in_h
//           | "ReLU" | "MixtureReLU"
//           | "BatchNorm2d" C eps momentum bias
//           | "AvgPool2d" k stride pad pad_type
//           | "LayerBlock" "[" layer* "]"
//           | "ResNetBlock" "[" layer* "]" "[" layer* "]"    (second list empty: identity shortcut)
// "input W H C" writes in_width / in_height / in_channels of the first layer, which a
// network that starts with a block needs (its block cannot infer them).
// Parameter order ("leaf order"): layers in reading order of the description,
// blocks expanded in place (main before shortcut); per layer mu_w, var_w, mu_b,
// var_b and, for BatchNorm2d, mu_ra, var_ra.
#include <cstring>
#include <memory>
#include <sstream>
#include <stdexcept>
#include <string>
#include <vector>

#include "activation.h"
#include "base_layer.h"
#include "base_output_updater.h"
#include "batchnorm_layer.h"
#include "conv2d_layer.h"
#include "layer_block.h"
#include "linear_layer.h"
#include "pooling_layer.h"
#include "resnet_block.h"
#include "sequential.h"

namespace {

struct Parser {
    std::vector<std::string> tok;
    size_t pos = 0;
    std::vector<BaseLayer *> leaves;  // layers that own parameters, in leaf order

    explicit Parser(const char *text) {
        std::istringstream in(text);
        std::string t;
        while (in >> t) tok.push_back(t);
    }
    bool done() const { return pos >= tok.size(); }
    const std::string &peek() const { return tok.at(pos); }
    std::string next() { return tok.at(pos++); }
    int num() { return std::stoi(next()); }
    float real() { return std::stof(next()); }
    void expect(const char *s) {
        if (next() != s) throw std::runtime_error(std::string("expected ") + s);
    }

    std::shared_ptr<LayerBlock> block() {
        expect("[");
        auto b = std::make_shared<LayerBlock>();
        int n = 0;
        while (peek() != "]") {
            b->add_layer(layer());
            n++;
        }
        expect("]");
        if (n == 0) return nullptr;
        b->add_layers();
        return b;
    }

    std::shared_ptr<BaseLayer> layer() {
        const std::string name = next();
        std::shared_ptr<BaseLayer> l;
        if (name == "Linear") {
            int K = num(), N = num(), bias = num();
            l = std::make_shared<Linear>(K, N, bias != 0);
            leaves.push_back(l.get());
        } else if (name == "Conv2d") {
            int fi = num(), fo = num(), k = num(), bias = num(), s = num(), p = num(), pt = num(),
                w = num(), h = num();
            l = std::make_shared<Conv2d>(fi, fo, k, bias != 0, s, p, pt, w, h);
            leaves.push_back(l.get());
        } else if (name == "ReLU") {
            l = std::make_shared<ReLU>();
        } else if (name == "MixtureReLU") {
            l = std::make_shared<MixtureReLU>();
        } else if (name == "BatchNorm2d") {
            int C = num();
            float eps = real(), mom = real();
            int bias = num();
            l = std::make_shared<BatchNorm2d>(C, eps, mom, bias != 0);
            leaves.push_back(l.get());
        } else if (name == "AvgPool2d") {
            int k = num(), s = num(), p = num(), pt = num();
            l = std::make_shared<AvgPool2d>(k, s, p, pt);
        } else if (name == "LayerBlock") {
            l = block();
            if (!l) throw std::runtime_error("empty LayerBlock");
        } else if (name == "ResNetBlock") {
            auto main = block();
            auto shortcut = block();
            if (!main) throw std::runtime_error("empty main block");
            if (shortcut)
                l = std::make_shared<ResNetBlock>(main, shortcut);
            else
                l = std::make_shared<ResNetBlock>(main);
        } else {
            throw std::runtime_error("unknown layer " + name);
        }
        return l;
    }
};

struct Model {
    Sequential net;
    std::vector<BaseLayer *> leaves;
};

std::vector<std::vector<float> *> arrays_of(BaseLayer *l) {
    std::vector<std::vector<float> *> a = {&l->mu_w, &l->var_w, &l->mu_b, &l->var_b};
    if (auto *bn = dynamic_cast<BatchNorm2d *>(l)) {
        a.push_back(&bn->mu_ra);
        a.push_back(&bn->var_ra);
    }
    return a;
}

// The way the reference's Python binding builds a Sequential from a list
// (src/bindings/sequential_bindings.cpp: add_layer per element, then add_layers).
void build(Model &m, const char *spec, int threads) {
    Parser p(spec);
    int iw = 0, ih = 0, ic = 0;
    if (!p.done() && p.peek() == "input") {
        p.next();
        iw = p.num();
        ih = p.num();
        ic = p.num();
    }
    bool first = true;
    while (!p.done()) {
        auto l = p.layer();
        if (first && iw > 0) {
            l->in_width = iw;
            l->in_height = ih;
            l->in_channels = ic;
        }
        first = false;
        m.net.add_layer(l);
    }
    m.net.add_layers();
    m.net.set_threads(threads);
    m.net.preinit_layer();
    m.leaves = p.leaves;
    // Conv2d::preinit_layer (src/conv2d_layer.cpp:260-269) creates the parameters but
    // not their innovation vectors, and Conv2d::forward then skips its lazy branch
    // (128-132) because num_weights is set: allocate them the way that branch does
    for (auto *l : m.leaves)
        if (l->delta_mu_w.size() != l->mu_w.size()) l->allocate_param_delta();
}

size_t count_params(Model &m) {
    size_t n = 0;
    for (auto *l : m.leaves)
        for (auto *a : arrays_of(l)) n += a->size();
    return n;
}

void write_params(Model &m, float *out) {
    for (auto *l : m.leaves)
        for (auto *a : arrays_of(l)) {
            std::memcpy(out, a->data(), a->size() * sizeof(float));
            out += a->size();
        }
}

}  // namespace

extern "C" {

// Sizes of the parameter arrays in leaf order (4 per layer, 6 for BatchNorm2d).
// Returns the number of arrays, or -1 (description does not parse / capacity).
int ref_model_param_sizes(const char *spec, int *sizes, int capacity) {
    try {
        Model m;
        build(m, spec, 1);
        int n = 0;
        for (auto *l : m.leaves)
            for (auto *a : arrays_of(l)) {
                if (n >= capacity) return -1;
                sizes[n++] = (int)a->size();
            }
        return n;
    } catch (const std::exception &) {
        return -1;
    }
}

// Runs `steps` training steps and, with eval_forward != 0, one more forward in
// eval mode on the last batch.
//   params          : every parameter in leaf order (ref_model_param_sizes)
//   mu_x, var_x     : [steps][B*n_in]; var_x may be null (forward with means only)
//   update_mode     : 0 = OutputUpdater::update (y, var_y: [steps][B*n_out]),
//                     1 = update_using_indices (y, var_y: [steps][B*n_enc], sel 1-based),
//                     2 = update_heteros (y: [steps][B*n_out/2])
//   out_mu, out_var : [steps (+1 with eval_forward)][B*n_out] network outputs
//   in_dmu, in_dvar : [steps][B*n_in] input innovations (written when input_state_update)
//   params_out      : [steps][P] every parameter after each step
//   neg_counts      : [steps][top-level layers] BaseLayer::get_neg_var_w_counter
// Returns n_out, or -1 when the reference throws.
int ref_model_run(const char *spec, int threads, int input_state_update, const float *params,
                  int steps, int B, int n_in, const float *mu_x, const float *var_x,
                  int update_mode, int n_enc, const float *y, const float *var_y, const int *sel,
                  int eval_forward, float *out_mu, float *out_var, float *in_dmu, float *in_dvar,
                  float *params_out, int *neg_counts) {
    try {
        Model m;
        build(m, spec, threads);
        m.net.input_state_update = input_state_update != 0;
        for (auto *l : m.leaves)
            for (auto *a : arrays_of(l)) {
                std::memcpy(a->data(), params, a->size() * sizeof(float));
                params += a->size();
            }
        const size_t P = count_params(m);
        OutputUpdater updater(m.net.device);
        int n_out = 0;
        const size_t nx = (size_t)B * n_in;
        size_t ny = 0;
        for (int s = 0; s < steps; s++) {
            std::vector<float> mx(mu_x + s * nx, mu_x + (s + 1) * nx);
            std::vector<float> vx;
            if (var_x) vx.assign(var_x + s * nx, var_x + (s + 1) * nx);
            m.net.forward(mx, vx);
            auto &o = *m.net.output_z_buffer;
            n_out = (int)o.actual_size;
            const size_t no = (size_t)B * n_out;
            std::memcpy(out_mu + s * no, o.mu_a.data(), no * sizeof(float));
            std::memcpy(out_var + s * no, o.var_a.data(), no * sizeof(float));
            ny = update_mode == 1 ? (size_t)B * n_enc : update_mode == 2 ? no / 2 : no;
            std::vector<float> obs(y + s * ny, y + (s + 1) * ny);
            if (update_mode == 0) {
                std::vector<float> vobs(var_y + s * ny, var_y + (s + 1) * ny);
                updater.update(o, obs, vobs, *m.net.input_delta_z_buffer);
            } else if (update_mode == 1) {
                std::vector<float> vobs(var_y + s * ny, var_y + (s + 1) * ny);
                std::vector<int> idx(sel + s * ny, sel + (s + 1) * ny);
                updater.update_using_indices(o, obs, vobs, idx, *m.net.input_delta_z_buffer);
            } else {
                updater.update_heteros(o, obs, *m.net.input_delta_z_buffer);
            }
            m.net.backward();
            if (input_state_update) {
                auto &d = *m.net.output_delta_z_buffer;
                std::memcpy(in_dmu + s * nx, d.delta_mu.data(), nx * sizeof(float));
                std::memcpy(in_dvar + s * nx, d.delta_var.data(), nx * sizeof(float));
            }
            m.net.step();
            write_params(m, params_out + s * P);
            for (size_t i = 0; i < m.net.layers.size(); i++)
                neg_counts[s * m.net.layers.size() + i] = m.net.layers[i]->get_neg_var_w_counter();
        }
        if (eval_forward) {
            m.net.eval();
            std::vector<float> mx(mu_x + (steps - 1) * nx, mu_x + steps * nx);
            std::vector<float> vx;
            if (var_x) vx.assign(var_x + (steps - 1) * nx, var_x + steps * nx);
            m.net.forward(mx, vx);
            auto &o = *m.net.output_z_buffer;
            const size_t no = (size_t)B * n_out;
            std::memcpy(out_mu + steps * no, o.mu_a.data(), no * sizeof(float));
            std::memcpy(out_var + steps * no, o.var_a.data(), no * sizeof(float));
        }
        return n_out;
    } catch (const std::exception &) {
        return -1;
    }
}

}  // extern "C"
