#include "layers.h"

#include <algorithm>
#include <cmath>
#include <random>
#include <stdexcept>

namespace nebula {

namespace {

void read_floats(std::fstream &f, std::vector<float> &v) {
    f.read(reinterpret_cast<char*>(v.data()), (std::streamsize)(v.size() * sizeof(float)));
    if(!f) throw std::runtime_error("Error: weight file is shorter than the network needs");
}

void write_floats(std::fstream &f, const std::vector<float> &v) {
    f.write(reinterpret_cast<const char*>(v.data()), (std::streamsize)(v.size() * sizeof(float)));
}

[[noreturn]] void inference_only(const char *what) {
    throw std::runtime_error(std::string("Error: ") + what + " is not part of the inference-only build");
}

}  // namespace

// ---- layer_t ---------------------------------------------------------------------------------------
layer_t::layer_t(network_t *m_network, layer_t *m_prev_layer, layer_type_t m_layer_type) :
    layer_type(m_layer_type), activation_type(UNDEFINED_ACTIVATION),
    input_height(1), input_width(1), input_channel(1), input_size(1),
    output_height(1), output_width(1), output_channel(1), output_size(0),
    output_data(NULL), output_data_pinned(false), delta(NULL),
    padding(0), num_filters(1), filter_size(1), stride(1), group(1),
    prev_layer(m_prev_layer), next_layer(NULL),
    output_data_dev(NULL), delta_dev(NULL),
    num_threads(m_network->num_threads), network(m_network), owns_output(false) {
    if(m_prev_layer) m_prev_layer->next_layer = this;
}

layer_t::~layer_t() {
    if(owns_output && output_data_dev && network->ctx) nbl_free(network->ctx, output_data_dev);
    if(output_data_pinned) nbl_free_host(network->ctx, output_data);
    else delete [] output_data;
}

void layer_t::backward() { inference_only("backward()"); }
void layer_t::update() { inference_only("update()"); }
void layer_t::_backward_() { inference_only("_backward_()"); }
void layer_t::_update_() { inference_only("_update_()"); }

void layer_t::read_activation(section_config_t &m_section_config) {
    std::string activation_str;
    if(m_section_config.get_setting("activation", &activation_str)) {
        const unsigned id = lookup_type(activation_type_str, NUM_ACTIVATION_TYPES, activation_str);
        // the reference stores an out-of-range id and fails in activate(); fail at init instead
        if(id == UNDEFINED_ACTIVATION || id >= NUM_ACTIVATION_TYPES)
            throw std::runtime_error("Error: undefined activation type " + activation_str);
        activation_type = (activation_type_t)id;
    }
}

const float *layer_t::input_dev() const {
    return prev_layer ? prev_layer->output_data_dev : network->input_data_dev;
}

void layer_t::alloc_output() {
    if(!network->ctx) return;          // dry-run network: shapes only
    const size_t bytes = sizeof(float) * (size_t)output_size * network->batch_size;
    nbl_check(network->ctx, nbl_malloc(network->ctx, (void**)&output_data_dev, bytes), "nbl_malloc(output)");
    nbl_check(network->ctx, nbl_fill_zero(network->ctx, output_data_dev, bytes), "nbl_fill_zero(output)");
    owns_output = true;
}

// ---- convolutional ---------------------------------------------------------------------------------
convolutional_layer_t::convolutional_layer_t(network_t *m_network, layer_t *m_prev_layer, layer_type_t m_layer_type) :
    layer_t(m_network, m_prev_layer, m_layer_type), batch_normalize(false), weight_size(0), plan(NULL),
    fused_shortcut(NULL) {}

convolutional_layer_t::~convolutional_layer_t() {
    if(plan) nbl_conv2d_plan_destroy(network->ctx, plan);
}

void convolutional_layer_t::init(section_config_t m_section_config) {
    m_section_config.get_setting("filters", &num_filters);
    m_section_config.get_setting("size", &filter_size);
    m_section_config.get_setting("batch_normalize", &batch_normalize);
    m_section_config.get_setting("padding", &padding);
    m_section_config.get_setting("stride", &stride);
    read_activation(m_section_config);
    if(activation_type == UNDEFINED_ACTIVATION)
        throw std::runtime_error("Error: undefined activation type undefined_activation");

    input_size    = prev_layer ? prev_layer->output_size    : network->input_size;
    input_height  = prev_layer ? prev_layer->output_height  : network->input_height;
    input_width   = prev_layer ? prev_layer->output_width   : network->input_width;
    input_channel = prev_layer ? prev_layer->output_channel : network->input_channel;
    if(!stride || !filter_size || !num_filters || input_height + 2 * padding < filter_size ||
       input_width + 2 * padding < filter_size)
        throw std::runtime_error("Error: invalid convolution geometry");

    output_height  = nbl_conv_out_dim(input_height, filter_size, stride, padding);
    output_width   = nbl_conv_out_dim(input_width, filter_size, stride, padding);
    output_channel = num_filters;
    output_size    = output_height * output_width * output_channel;
    weight_size    = input_channel * num_filters * filter_size * filter_size;

    bias.assign(num_filters, 0.0f);
    weight.assign(weight_size, 0.0f);
    if(batch_normalize) {
        scale.assign(num_filters, 1.0f);
        rolling_mean.assign(num_filters, 0.0f);
        rolling_variance.assign(num_filters, 0.0f);
    }
    alloc_output();
}

// .wgh order: bias[F], weight[F][C][k][k], then scale, rolling_mean, rolling_variance when normalized.
void convolutional_layer_t::init_weight(std::fstream &m_weight_file) {
    read_floats(m_weight_file, bias);
    read_floats(m_weight_file, weight);
    if(batch_normalize) {
        read_floats(m_weight_file, scale);
        read_floats(m_weight_file, rolling_mean);
        read_floats(m_weight_file, rolling_variance);
    }
    pack();
}

void convolutional_layer_t::init_weight() {
    std::minstd_rand rng(1 + weight_size);
    std::normal_distribution<float> dist(0.0f, 1.0f);
    const float sigma = (float)std::sqrt(2.0 / (filter_size * filter_size * input_channel));
    for(unsigned i = 0; i < weight_size; i++) weight[i] = sigma * dist(rng);
    if(batch_normalize) rolling_variance.assign(num_filters, 1.0f);
    pack();
}

void convolutional_layer_t::store_weight(std::fstream &m_weight_file) {
    write_floats(m_weight_file, bias);
    write_floats(m_weight_file, weight);
    if(batch_normalize) {
        write_floats(m_weight_file, scale);
        write_floats(m_weight_file, rolling_mean);
        write_floats(m_weight_file, rolling_variance);
    }
}

void convolutional_layer_t::pack() {
    if(!network->ctx) return;          // dry-run network
    if(plan) { nbl_conv2d_plan_destroy(network->ctx, plan); plan = NULL; }
    nbl_check(network->ctx,
              nbl_conv2d_pack(network->ctx, weight.data(), bias.data(),
                              batch_normalize ? scale.data() : NULL,
                              batch_normalize ? rolling_mean.data() : NULL,
                              batch_normalize ? rolling_variance.data() : NULL,
                              input_channel, input_height, input_width, num_filters,
                              filter_size, stride, padding, (int)activation_type, &plan),
              "nbl_conv2d_pack");
    if(network->conv_split >= 0)
        nbl_check(network->ctx, nbl_conv2d_plan_set_split(plan, network->conv_split ? 1 : 0), "nbl_conv2d_plan_set_split");
}

bool convolutional_layer_t::fuse_with(shortcut_layer_t *m_shortcut) {
    if(!m_shortcut || m_shortcut->prev_layer != this || fused_shortcut) return false;
    layer_t *conn = m_shortcut->connection;
    if(!conn || conn == this || output_width / conn->output_width > 1) return false;
    if(owns_output && output_data_dev && network->ctx) nbl_free(network->ctx, output_data_dev);
    owns_output = false;
    output_data_dev = m_shortcut->output_data_dev;      // alias: nothing may read a stale buffer
    fused_shortcut = m_shortcut;
    m_shortcut->fused = true;
    return true;
}

void convolutional_layer_t::_forward_() {
    if(!plan) throw std::runtime_error("Error: convolutional layer has no weights (init_weight not called)");
    if(fused_shortcut) {
        layer_t *conn = fused_shortcut->connection;
        nbl_check(network->ctx,
                  nbl_conv2d_shortcut_fwd(network->ctx, plan, input_dev(), conn->output_data_dev, conn->output_channel,
                                          conn->output_height, conn->output_width, fused_shortcut->output_data_dev,
                                          network->batch_size, (int)fused_shortcut->activation_type),
                  "nbl_conv2d_shortcut_fwd");
        return;
    }
    nbl_check(network->ctx, nbl_conv2d_fwd(network->ctx, plan, input_dev(), output_data_dev, network->batch_size),
              "nbl_conv2d_fwd");
}

void convolutional_layer_t::last_launch(int *variant, int *slices) const {
    if(!plan) throw std::runtime_error("Error: convolutional layer has no weights (init_weight not called)");
    nbl_check(network->ctx, nbl_conv2d_plan_last_launch(plan, variant, slices), "nbl_conv2d_plan_last_launch");
}

int convolutional_layer_t::launch_source() const {
    if(!plan) throw std::runtime_error("Error: convolutional layer has no weights (init_weight not called)");
    return nbl_conv2d_plan_launch_source(plan);
}

void convolutional_layer_t::pin_launch(int variant, int split) {
    if(!plan) throw std::runtime_error("Error: convolutional layer has no weights (init_weight not called)");
    nbl_check(network->ctx, nbl_conv2d_plan_set_variant(plan, variant), "nbl_conv2d_plan_set_variant");
    nbl_check(network->ctx, nbl_conv2d_plan_set_split(plan, split), "nbl_conv2d_plan_set_split");
}

void convolutional_layer_t::weight_fields(std::vector<weight_field_t> &out) const {
    const unsigned fan_in = input_channel * filter_size * filter_size;
    out.push_back(weight_field_t{ WEIGHT_BIAS, num_filters, fan_in });
    out.push_back(weight_field_t{ WEIGHT_MATRIX, weight_size, fan_in });
    if(batch_normalize) {
        out.push_back(weight_field_t{ WEIGHT_BN_SCALE, num_filters, fan_in });
        out.push_back(weight_field_t{ WEIGHT_BN_MEAN, num_filters, fan_in });
        out.push_back(weight_field_t{ WEIGHT_BN_VARIANCE, num_filters, fan_in });
    }
}

double convolutional_layer_t::flop_per_image() const {
    return 2.0 * num_filters * output_height * output_width * input_channel * filter_size * filter_size;
}

// ---- connected -------------------------------------------------------------------------------------
connected_layer_t::connected_layer_t(network_t *m_network, layer_t *m_prev_layer, layer_type_t m_layer_type) :
    layer_t(m_network, m_prev_layer, m_layer_type), batch_normalize(false), weight_size(0),
    allocate_output(true), plan(NULL) {}

connected_layer_t::~connected_layer_t() {
    if(plan) nbl_fc_plan_destroy(network->ctx, plan);
}

void connected_layer_t::init(section_config_t m_section_config) {
    m_section_config.get_setting("output", &output_size);
    m_section_config.get_setting("batch_normalize", &batch_normalize);
    read_activation(m_section_config);
    if(activation_type == UNDEFINED_ACTIVATION)
        throw std::runtime_error("Error: undefined activation type undefined_activation");
    // an LSTM sets input_size itself before calling init()
    if(allocate_output) input_size = prev_layer ? prev_layer->output_size : network->input_size;
    if(!output_size || !input_size) throw std::runtime_error("Error: connected layer with zero size");
    weight_size = input_size * output_size;
    bias.assign(output_size, 0.0f);
    weight.assign(weight_size, 0.0f);
    if(batch_normalize) {
        scale.assign(output_size, 1.0f);
        rolling_mean.assign(output_size, 0.0f);
        rolling_variance.assign(output_size, 0.0f);
    }
    if(allocate_output) alloc_output();
}

// .wgh order: bias[O], weight[O][I], then scale, rolling_mean, rolling_variance when normalized.
void connected_layer_t::init_weight(std::fstream &m_weight_file) {
    read_floats(m_weight_file, bias);
    read_floats(m_weight_file, weight);
    if(batch_normalize) {
        read_floats(m_weight_file, scale);
        read_floats(m_weight_file, rolling_mean);
        read_floats(m_weight_file, rolling_variance);
    }
    if(allocate_output) pack();
}

void connected_layer_t::init_weight() {
    std::minstd_rand rng(7 + weight_size);
    std::uniform_real_distribution<float> dist(-1.0f, 1.0f);
    const float amp = (float)std::sqrt(2.0 / input_size);
    for(unsigned i = 0; i < weight_size; i++) weight[i] = amp * dist(rng);
    if(batch_normalize) rolling_variance.assign(output_size, 1.0f);
    if(allocate_output) pack();
}

void connected_layer_t::store_weight(std::fstream &m_weight_file) {
    write_floats(m_weight_file, bias);
    write_floats(m_weight_file, weight);
    if(batch_normalize) {
        write_floats(m_weight_file, scale);
        write_floats(m_weight_file, rolling_mean);
        write_floats(m_weight_file, rolling_variance);
    }
}

void connected_layer_t::weight_fields(std::vector<weight_field_t> &out) const {
    out.push_back(weight_field_t{ WEIGHT_BIAS, output_size, input_size });
    out.push_back(weight_field_t{ WEIGHT_MATRIX, weight_size, input_size });
    if(batch_normalize) {
        out.push_back(weight_field_t{ WEIGHT_BN_SCALE, output_size, input_size });
        out.push_back(weight_field_t{ WEIGHT_BN_MEAN, output_size, input_size });
        out.push_back(weight_field_t{ WEIGHT_BN_VARIANCE, output_size, input_size });
    }
}

void connected_layer_t::pack() {
    if(!network->ctx) return;          // dry-run network
    if(plan) { nbl_fc_plan_destroy(network->ctx, plan); plan = NULL; }
    nbl_check(network->ctx,
              nbl_fc_pack(network->ctx, weight.data(), bias.data(),
                          batch_normalize ? scale.data() : NULL,
                          batch_normalize ? rolling_mean.data() : NULL,
                          batch_normalize ? rolling_variance.data() : NULL,
                          input_size, output_size, (int)activation_type, &plan),
              "nbl_fc_pack");
}

void connected_layer_t::_forward_() {
    if(!plan) throw std::runtime_error("Error: connected layer has no weights (init_weight not called)");
    nbl_check(network->ctx, nbl_fc_fwd(network->ctx, plan, input_dev(), output_data_dev, network->batch_size),
              "nbl_fc_fwd");
}

// ---- pooling ---------------------------------------------------------------------------------------
pooling_layer_t::pooling_layer_t(network_t *m_network, layer_t *m_prev_layer, layer_type_t m_layer_type) :
    layer_t(m_network, m_prev_layer, m_layer_type), index_dev(NULL) {}

pooling_layer_t::~pooling_layer_t() {
    if(index_dev) nbl_free(network->ctx, index_dev);
}

void pooling_layer_t::init(section_config_t m_section_config) {
    if(layer_type != MAXPOOL_LAYER && layer_type != AVGPOOL_LAYER)
        throw std::runtime_error("undefined pooling layer type ");
    m_section_config.get_setting("stride", &stride);
    filter_size = stride;                       // window defaults to the stride ...
    m_section_config.get_setting("size", &filter_size);
    padding = (filter_size - 1) / 2;            // ... and padding to (size - 1) / 2
    m_section_config.get_setting("padding", &padding);
    if(!stride || !filter_size) throw std::runtime_error("Error: invalid pooling geometry");

    input_height  = prev_layer ? prev_layer->output_height  : network->input_height;
    input_width   = prev_layer ? prev_layer->output_width   : network->input_width;
    input_channel = prev_layer ? prev_layer->output_channel : network->input_channel;
    input_size    = prev_layer ? prev_layer->output_size    : network->input_size;

    output_height  = nbl_pool_out_dim(input_height, stride, padding);    // (in + 2*pad) / stride
    output_width   = nbl_pool_out_dim(input_width, stride, padding);
    output_channel = input_channel;
    output_size    = output_height * output_width * output_channel;
    alloc_output();
    if(layer_type == MAXPOOL_LAYER && network->ctx && network->pool_index) {
        const size_t bytes = sizeof(unsigned) * (size_t)output_size * network->batch_size;
        nbl_check(network->ctx, nbl_malloc(network->ctx, (void**)&index_dev, bytes), "nbl_malloc(index)");
        nbl_check(network->ctx, nbl_fill_zero(network->ctx, index_dev, bytes), "nbl_fill_zero(index)");
    }
}

void pooling_layer_t::_forward_() {
    nbl_check(network->ctx,
              nbl_pool_fwd(network->ctx, input_dev(), output_data_dev, index_dev, network->batch_size,
                           input_channel, input_height, input_width, filter_size, stride, padding,
                           layer_type == MAXPOOL_LAYER ? NBL_POOL_MAX : NBL_POOL_AVG),
              "nbl_pool_fwd");
}

// ---- shortcut --------------------------------------------------------------------------------------
shortcut_layer_t::shortcut_layer_t(network_t *m_network, layer_t *m_prev_layer, layer_type_t m_layer_type) :
    layer_t(m_network, m_prev_layer, m_layer_type), connection(NULL), fused(false), in_place(false), hops(0) {}

shortcut_layer_t::~shortcut_layer_t() {}

void shortcut_layer_t::init(section_config_t m_section_config) {
    m_section_config.get_setting("hops", &hops);
    read_activation(m_section_config);
    if(activation_type == UNDEFINED_ACTIVATION)
        throw std::runtime_error("Error: undefined activation type undefined_activation");
    // walk `hops` layers back, counting this layer as the start (so hops=4 after three convs reaches
    // the layer that fed the first of them)
    connection = this;
    for(unsigned i = 0; i < hops; i++) connection = connection ? connection->prev_layer : NULL;
    if(!connection || connection == this || !prev_layer)
        throw std::runtime_error("Error: shortcut hops do not reach an earlier layer");

    input_height  = connection->output_height;
    input_width   = connection->output_width;
    input_channel = connection->output_channel;
    output_height  = prev_layer->output_height;
    output_width   = prev_layer->output_width;
    output_channel = prev_layer->output_channel;
    output_size = output_height * output_width * output_channel;
    input_size = output_size;
    alloc_output();
}

void shortcut_layer_t::write_over_connection() {
    if(!fused || in_place || !connection || !prev_layer) return;
    if(owns_output && output_data_dev && network->ctx) nbl_free(network->ctx, output_data_dev);
    owns_output = false;
    output_data_dev = connection->output_data_dev;
    prev_layer->output_data_dev = output_data_dev;      // the fused convolution aliases this layer's tensor
    in_place = true;
}

void shortcut_layer_t::_forward_() {
    if(fused) return;          // already written by the preceding convolution
    nbl_check(network->ctx,
              nbl_shortcut_fwd(network->ctx, prev_layer->output_data_dev, connection->output_data_dev, output_data_dev,
                               network->batch_size, input_channel, input_height, input_width,
                               output_channel, output_height, output_width, (int)activation_type),
              "nbl_shortcut_fwd");
}

// ---- softmax ---------------------------------------------------------------------------------------
softmax_layer_t::softmax_layer_t(network_t *m_network, layer_t *m_prev_layer, layer_type_t m_layer_type) :
    layer_t(m_network, m_prev_layer, m_layer_type), copy_to_host(true) {}

softmax_layer_t::~softmax_layer_t() {}

void softmax_layer_t::init(section_config_t) {
    input_size = prev_layer ? prev_layer->output_size : network->input_size;
    output_size = input_size;
    const size_t count = (size_t)output_size * network->batch_size;
    if(network->ctx) {      // page-locked, so the per-forward copy of the probabilities needs no staging
        nbl_check(network->ctx, nbl_malloc_host(network->ctx, (void**)&output_data, count * sizeof(float)), "nbl_malloc_host(softmax)");
        output_data_pinned = true;
        std::fill(output_data, output_data + count, 0.0f);
    } else {
        output_data = new float[count]();
    }
    alloc_output();
}

void softmax_layer_t::_forward_() {
    nbl_check(network->ctx, nbl_softmax_fwd(network->ctx, input_dev(), output_data_dev, network->batch_size, input_size),
              "nbl_softmax_fwd");
    if(copy_to_host) {
        const size_t bytes = sizeof(float) * (size_t)output_size * network->batch_size;
        if(network->defer_host_copy) nbl_check(network->ctx, nbl_d2h_async(network->ctx, output_data, output_data_dev, bytes), "nbl_d2h_async(softmax)");
        else nbl_check(network->ctx, nbl_d2h(network->ctx, output_data, output_data_dev, bytes), "nbl_d2h(softmax)");
    }
}

// ---- dropout / cost --------------------------------------------------------------------------------
dropout_layer_t::dropout_layer_t(network_t *m_network, layer_t *m_prev_layer, layer_type_t m_layer_type) :
    layer_t(m_network, m_prev_layer, m_layer_type), probability(0.0f) {}

void dropout_layer_t::init(section_config_t m_section_config) {
    m_section_config.get_setting("probability", &probability);
    if(!prev_layer) throw std::runtime_error("Error: dropout cannot be the first layer");
    input_size = prev_layer->output_size;
    output_size = input_size;
    output_data_dev = prev_layer->output_data_dev;      // alias, never freed here
}

cost_layer_t::cost_layer_t(network_t *m_network, layer_t *m_prev_layer, layer_type_t m_layer_type) :
    layer_t(m_network, m_prev_layer, m_layer_type) {}

void cost_layer_t::init(section_config_t) {
    input_size = prev_layer ? prev_layer->output_size : network->input_size;
    output_size = input_size;
    output_data_dev = prev_layer ? prev_layer->output_data_dev : network->input_data_dev;   // alias
}

// ---- LSTM ------------------------------------------------------------------------------------------
lstm_layer_t::lstm_layer_t(network_t *m_network, layer_t *m_prev_layer, layer_type_t m_layer_type) :
    layer_t(m_network, m_prev_layer, m_layer_type), batch_normalize(false),
    input_gate_W(NULL), forget_gate_W(NULL), cell_gate_W(NULL), output_gate_W(NULL),
    input_gate_U(NULL), forget_gate_U(NULL), cell_gate_U(NULL), output_gate_U(NULL), plan(NULL) {}

lstm_layer_t::~lstm_layer_t() {
    if(plan) nbl_lstm_plan_destroy(network->ctx, plan);
    delete input_gate_W; delete forget_gate_W; delete cell_gate_W; delete output_gate_W;
    delete input_gate_U; delete forget_gate_U; delete cell_gate_U; delete output_gate_U;
}

void lstm_layer_t::init(section_config_t m_section_config) {
    m_section_config.get_setting("output", &output_size);
    m_section_config.get_setting("batch_normalize", &batch_normalize);
    read_activation(m_section_config);
    if(activation_type == UNDEFINED_ACTIVATION)
        throw std::runtime_error("Error: undefined activation type undefined_activation");
    input_size = prev_layer ? prev_layer->output_size : network->input_size;
    if(!network->time_step || network->batch_size % network->time_step)
        throw std::runtime_error("Error: batch size is not a multiple of time_steps");

    // Eight parameter holders initialised from the same section (so they share output=, activation=
    // and batch_normalize=): W reads the hidden state (fan-in = output size), U reads the input.
    connected_layer_t **slots[8] = { &input_gate_W, &forget_gate_W, &cell_gate_W, &output_gate_W,
                                     &input_gate_U, &forget_gate_U, &cell_gate_U, &output_gate_U };
    layer_t *saved_next = prev_layer ? prev_layer->next_layer : NULL;
    for(int s = 0; s < 8; s++) {
        connected_layer_t *sub = new connected_layer_t(network, NULL, CONNECTED_LAYER);
        sub->allocate_output = false;
        sub->input_size = s < 4 ? output_size : input_size;
        sub->init(m_section_config);
        *slots[s] = sub;
    }
    if(prev_layer) prev_layer->next_layer = saved_next;
    alloc_output();
}

// File order (not member order): W of input, forget, OUTPUT, CELL gate, then the same four for U.
void lstm_layer_t::init_weight(std::fstream &m_weight_file) {
    input_gate_W->init_weight(m_weight_file);
    forget_gate_W->init_weight(m_weight_file);
    output_gate_W->init_weight(m_weight_file);
    cell_gate_W->init_weight(m_weight_file);
    input_gate_U->init_weight(m_weight_file);
    forget_gate_U->init_weight(m_weight_file);
    output_gate_U->init_weight(m_weight_file);
    cell_gate_U->init_weight(m_weight_file);
    pack();
}

void lstm_layer_t::init_weight() {
    connected_layer_t *order[8] = { input_gate_W, forget_gate_W, output_gate_W, cell_gate_W,
                                    input_gate_U, forget_gate_U, output_gate_U, cell_gate_U };
    for(int s = 0; s < 8; s++) order[s]->init_weight();
    pack();
}

void lstm_layer_t::store_weight(std::fstream &m_weight_file) {
    connected_layer_t *order[8] = { input_gate_W, forget_gate_W, output_gate_W, cell_gate_W,
                                    input_gate_U, forget_gate_U, output_gate_U, cell_gate_U };
    for(int s = 0; s < 8; s++) order[s]->store_weight(m_weight_file);
}

void lstm_layer_t::weight_fields(std::vector<weight_field_t> &out) const {
    const connected_layer_t *order[8] = { input_gate_W, forget_gate_W, output_gate_W, cell_gate_W,
                                          input_gate_U, forget_gate_U, output_gate_U, cell_gate_U };
    for(int s = 0; s < 8; s++) order[s]->weight_fields(out);
}

void lstm_layer_t::pack() {
    if(!network->ctx) return;          // dry-run network
    if(plan) { nbl_lstm_plan_destroy(network->ctx, plan); plan = NULL; }
    connected_layer_t *order[8] = { input_gate_W, forget_gate_W, output_gate_W, cell_gate_W,
                                    input_gate_U, forget_gate_U, output_gate_U, cell_gate_U };
    const float *w[8], *b[8], *sc[8], *mu[8], *var[8];
    for(int s = 0; s < 8; s++) {
        w[s] = order[s]->weight.data(); b[s] = order[s]->bias.data();
        sc[s] = batch_normalize ? order[s]->scale.data() : NULL;
        mu[s] = batch_normalize ? order[s]->rolling_mean.data() : NULL;
        var[s] = batch_normalize ? order[s]->rolling_variance.data() : NULL;
    }
    nbl_check(network->ctx,
              nbl_lstm_pack(network->ctx, w, b, batch_normalize ? sc : NULL, batch_normalize ? mu : NULL,
                            batch_normalize ? var : NULL, input_size, output_size, (int)activation_type, &plan),
              "nbl_lstm_pack");
    carry_state(network->carry_state);
}

void lstm_layer_t::carry_state(bool on) {
    if(plan) nbl_check(network->ctx, nbl_lstm_plan_carry_state(network->ctx, plan, on ? 1 : 0), "nbl_lstm_plan_carry_state");
}

void lstm_layer_t::reset_state() {
    if(plan) nbl_check(network->ctx, nbl_lstm_plan_reset_state(network->ctx, plan), "nbl_lstm_plan_reset_state");
}

// network->batch_size counts every (time step, sequence) row; rows are time-major.
void lstm_layer_t::_forward_() {
    if(!plan) throw std::runtime_error("Error: lstm layer has no weights (init_weight not called)");
    if(!prev_layer && network->input_tokens_dev) {      // one-hot input rows given as token indices
        nbl_check(network->ctx,
                  nbl_lstm_fwd_tokens(network->ctx, plan, network->input_tokens_dev, output_data_dev, NULL,
                                      network->time_step, network->batch_size / network->time_step),
                  "nbl_lstm_fwd_tokens");
        return;
    }
    nbl_check(network->ctx,
              nbl_lstm_fwd(network->ctx, plan, input_dev(), output_data_dev, NULL,
                           network->time_step, network->batch_size / network->time_step),
              "nbl_lstm_fwd");
}

// ---- rnn ------------------------------------------------------------------------------------------
rnn_layer_t::rnn_layer_t(network_t *m_network, layer_t *m_prev_layer, layer_type_t m_layer_type) :
    layer_t(m_network, m_prev_layer, m_layer_type), batch_normalize(false),
    input_gate(NULL), hidden_gate(NULL), output_gate(NULL), plan(NULL) {}

rnn_layer_t::~rnn_layer_t() {
    if(plan) nbl_rnn_plan_destroy(network->ctx, plan);
    delete input_gate; delete hidden_gate; delete output_gate;
}

void rnn_layer_t::init(section_config_t m_section_config) {
    m_section_config.get_setting("output", &output_size);
    m_section_config.get_setting("batch_normalize", &batch_normalize);
    read_activation(m_section_config);
    if(activation_type == UNDEFINED_ACTIVATION)
        throw std::runtime_error("Error: undefined activation type undefined_activation");
    input_size = prev_layer ? prev_layer->output_size : network->input_size;
    if(!network->time_step || network->batch_size % network->time_step)
        throw std::runtime_error("Error: batch size is not a multiple of time_steps");
    // parameter holders: the input gate reads the layer's input, the other two the layer's own width
    connected_layer_t **slots[3] = { &input_gate, &hidden_gate, &output_gate };
    layer_t *saved_next = prev_layer ? prev_layer->next_layer : NULL;
    for(int s = 0; s < 3; s++) {
        connected_layer_t *sub = new connected_layer_t(network, NULL, CONNECTED_LAYER);
        sub->allocate_output = false;
        sub->input_size = s == 0 ? input_size : output_size;
        sub->init(m_section_config);
        *slots[s] = sub;
    }
    if(prev_layer) prev_layer->next_layer = saved_next;
    alloc_output();
}

void rnn_layer_t::init_weight(std::fstream &m_weight_file) {
    input_gate->init_weight(m_weight_file);
    hidden_gate->init_weight(m_weight_file);
    output_gate->init_weight(m_weight_file);
    pack();
}

void rnn_layer_t::init_weight() {
    input_gate->init_weight(); hidden_gate->init_weight(); output_gate->init_weight();
    pack();
}

void rnn_layer_t::store_weight(std::fstream &m_weight_file) {
    input_gate->store_weight(m_weight_file);
    hidden_gate->store_weight(m_weight_file);
    output_gate->store_weight(m_weight_file);
}

void rnn_layer_t::weight_fields(std::vector<weight_field_t> &out) const {
    input_gate->weight_fields(out); hidden_gate->weight_fields(out); output_gate->weight_fields(out);
}

void rnn_layer_t::pack() {
    if(!network->ctx) return;          // dry-run network
    if(plan) { nbl_rnn_plan_destroy(network->ctx, plan); plan = NULL; }
    connected_layer_t *order[3] = { input_gate, hidden_gate, output_gate };
    const float *w[3], *b[3], *sc[3], *mu[3], *var[3];
    for(int s = 0; s < 3; s++) {
        w[s] = order[s]->weight.data(); b[s] = order[s]->bias.data();
        sc[s] = batch_normalize ? order[s]->scale.data() : NULL;
        mu[s] = batch_normalize ? order[s]->rolling_mean.data() : NULL;
        var[s] = batch_normalize ? order[s]->rolling_variance.data() : NULL;
    }
    nbl_check(network->ctx,
              nbl_rnn_pack(network->ctx, w, b, batch_normalize ? sc : NULL, batch_normalize ? mu : NULL,
                           batch_normalize ? var : NULL, input_size, output_size, (int)activation_type, &plan),
              "nbl_rnn_pack");
}

void rnn_layer_t::_forward_() {
    if(!plan) throw std::runtime_error("Error: rnn layer has no weights (init_weight not called)");
    if(!prev_layer && network->input_tokens_dev) {      // one-hot input rows given as token indices
        nbl_check(network->ctx,
                  nbl_rnn_fwd_tokens(network->ctx, plan, network->input_tokens_dev, output_data_dev, network->time_step,
                                     network->batch_size / network->time_step),
                  "nbl_rnn_fwd_tokens");
        return;
    }
    nbl_check(network->ctx,
              nbl_rnn_fwd(network->ctx, plan, input_dev(), output_data_dev, network->time_step,
                          network->batch_size / network->time_step),
              "nbl_rnn_fwd");
}

// ---- rbm ------------------------------------------------------------------------------------------
rbm_layer_t::rbm_layer_t(network_t *m_network, layer_t *m_prev_layer, layer_type_t m_layer_type) :
    connected_layer_t(m_network, m_prev_layer, m_layer_type) {}

// rbm_layer.cc:69-90 reads output, k_step and activation; there is no batch_normalize key for it to honour
void rbm_layer_t::init(section_config_t m_section_config) {
    connected_layer_t::init(m_section_config);
    if(batch_normalize) {
        batch_normalize = false;
        scale.clear(); rolling_mean.clear(); rolling_variance.clear();
    }
}

}  // namespace nebula
