// The layer classes of the forward path.  Same virtual surface, public fields, cfg keys and .wgh
// field order as the reference's models/layers/*.h; each _forward_() is a call into the C ABI
// (include/nebula_hip.h) instead of a chain of CUDA kernels and cuBLAS calls.
#ifndef NEBULA_HOST_LAYERS_H
#define NEBULA_HOST_LAYERS_H

#include <fstream>
#include <vector>

#include "config.h"
#include "def.h"
#include "network.h"

namespace nebula {

// One array of a layer's slice of the .wgh stream.
enum weight_kind_t { WEIGHT_BIAS = 0, WEIGHT_MATRIX, WEIGHT_BN_SCALE, WEIGHT_BN_MEAN, WEIGHT_BN_VARIANCE };
struct weight_field_t { weight_kind_t kind; unsigned count; unsigned fan_in; };

// models/layers/layer.h:11-85
class layer_t {
public:
    layer_t(network_t *m_network, layer_t *m_prev_layer, layer_type_t m_layer_type = UNDEFINED_LAYER);
    virtual ~layer_t();

    virtual void init(section_config_t m_section_config) = 0;
    virtual void init_weight(std::fstream &m_weight_file) = 0;   // from a .wgh stream
    virtual void init_weight() = 0;                              // from scratch (random)
    virtual void store_weight(std::fstream &m_weight_file) = 0;
    // The arrays init_weight(fstream&) reads, in file order (empty for weightless layers).
    virtual void weight_fields(std::vector<weight_field_t> &) const {}
    // GPU forward.  forward() is the same path: this build has no CPU implementation.
    virtual void _forward_() = 0;
    virtual void forward() { _forward_(); }
    // inference-only build
    virtual void backward();
    virtual void update();
    virtual void _backward_();
    virtual void _update_();

    layer_type_t layer_type;
    activation_type_t activation_type;

    unsigned input_height, input_width, input_channel, input_size;
    unsigned output_height, output_width, output_channel, output_size;

    float *output_data;        // host copy; only the softmax layer fills it (as the reference's GPU path)
    bool output_data_pinned;            // output_data came from nbl_malloc_host
    float *delta;              // never allocated (training)

    unsigned padding, num_filters, filter_size, stride, group;

    layer_t *prev_layer, *next_layer;

    float *output_data_dev;    // [batch_size][output_size]
    float *delta_dev;          // never allocated (training)

protected:
    // activation= of the section -> activation_type; throws on an unknown name
    void read_activation(section_config_t &m_section_config);
    // device input of this layer: previous layer's output or the network input
    const float *input_dev() const;
    void alloc_output();       // output_data_dev = batch_size * output_size floats
    unsigned num_threads;
    network_t *network;
    bool owns_output;
};

// models/layers/convolutional_layer.h
class convolutional_layer_t : public layer_t {
public:
    convolutional_layer_t(network_t *m_network, layer_t *m_prev_layer, layer_type_t m_layer_type);
    ~convolutional_layer_t();
    void init(section_config_t m_section_config);
    void init_weight(std::fstream &m_weight_file);
    void init_weight();
    void store_weight(std::fstream &m_weight_file);
    void _forward_();
    void weight_fields(std::vector<weight_field_t> &out) const;
    double flop_per_image() const;
    // Take over the [shortcut] layer that follows: this layer's kernel then adds the residual and applies
    // the shortcut's activation in its epilogue and writes the shortcut's buffer; this layer's own output
    // pointer becomes an alias of that buffer.  Returns false (and changes nothing) when the pair cannot
    // be fused (up-sampling shortcut, or a shortcut whose source is this very layer).
    bool fuse_with(class shortcut_layer_t *m_shortcut);
    // Tile shape and k-split of the kernel: what the most recent forward used, and a way to pin both
    // (variant < 0: from the launch table, or searched on first use; split as nbl_conv2d_plan_set_split).
    void last_launch(int *variant, int *slices) const;
    int launch_source() const;          // nbl_launch_source of the most recent launch
    void pin_launch(int variant, int split);
    bool is_fused() const { return fused_shortcut != NULL; }
    const class shortcut_layer_t *shortcut_fused() const { return fused_shortcut; }
private:
    void pack();
    bool batch_normalize;
    unsigned weight_size;
    std::vector<float> bias, weight, scale, rolling_mean, rolling_variance;
    nbl_conv_plan *plan;
    class shortcut_layer_t *fused_shortcut;
};

// models/layers/connected_layer.h
class connected_layer_t : public layer_t {
public:
    connected_layer_t(network_t *m_network, layer_t *m_prev_layer, layer_type_t m_layer_type);
    ~connected_layer_t();
    void init(section_config_t m_section_config);
    void init_weight(std::fstream &m_weight_file);
    void init_weight();
    void store_weight(std::fstream &m_weight_file);
    void _forward_();
    void weight_fields(std::vector<weight_field_t> &out) const;
    // host arrays, for the LSTM layer that owns eight of these as parameter holders
    bool batch_normalize;
    unsigned weight_size;
    std::vector<float> bias, weight, scale, rolling_mean, rolling_variance;
    bool allocate_output;      // false for LSTM sub-layers (they never run on their own)
private:
    void pack();
    nbl_fc_plan *plan;
};

// models/layers/pooling_layer.h (MAXPOOL_LAYER / AVGPOOL_LAYER)
class pooling_layer_t : public layer_t {
public:
    pooling_layer_t(network_t *m_network, layer_t *m_prev_layer, layer_type_t m_layer_type);
    ~pooling_layer_t();
    void init(section_config_t m_section_config);
    void init_weight(std::fstream &) {}
    void init_weight() {}
    void store_weight(std::fstream &) {}
    void _forward_();
    unsigned *index_dev;       // maxpool argmax: flat offsets into the input tensor (NULL unless [net] pool_index=1)
};

// models/layers/shortcut_layer.h
class shortcut_layer_t : public layer_t {
public:
    shortcut_layer_t(network_t *m_network, layer_t *m_prev_layer, layer_type_t m_layer_type);
    ~shortcut_layer_t();
    void init(section_config_t m_section_config);
    void init_weight(std::fstream &) {}
    void init_weight() {}
    void store_weight(std::fstream &) {}
    void _forward_();
    layer_t *connection;       // the layer `hops` back whose output is added
    bool fused;                // computed by the preceding convolution's epilogue; _forward_() does nothing
    // Give up this layer's own buffer and write the result over the connection's tensor (same shape, fused only):
    // this layer's output pointer, and the fused convolution's, become aliases of the connection's.
    void write_over_connection();
    bool in_place;
private:
    unsigned hops;
};

// models/layers/softmax_layer.h
class softmax_layer_t : public layer_t {
public:
    softmax_layer_t(network_t *m_network, layer_t *m_prev_layer, layer_type_t m_layer_type);
    ~softmax_layer_t();
    void init(section_config_t m_section_config);
    void init_weight(std::fstream &) {}
    void init_weight() {}
    void store_weight(std::fstream &) {}
    void _forward_();          // also copies the probabilities to output_data (softmax_layer.cu:38-39)
    bool copy_to_host;
};

// models/layers/dropout_layer.h: identity at inference, aliases the previous layer's buffers
class dropout_layer_t : public layer_t {
public:
    dropout_layer_t(network_t *m_network, layer_t *m_prev_layer, layer_type_t m_layer_type);
    void init(section_config_t m_section_config);
    void init_weight(std::fstream &) {}
    void init_weight() {}
    void store_weight(std::fstream &) {}
    void _forward_() {}
private:
    float probability;
};

// models/layers/cost_layer.h: follows the logits, training signal only; a shape-preserving no-op here
class cost_layer_t : public layer_t {
public:
    cost_layer_t(network_t *m_network, layer_t *m_prev_layer, layer_type_t m_layer_type);
    void init(section_config_t m_section_config);
    void init_weight(std::fstream &) {}
    void init_weight() {}
    void store_weight(std::fstream &) {}
    void _forward_() {}
};

// models/layers/lstm_layer.h
class lstm_layer_t : public layer_t {
public:
    lstm_layer_t(network_t *m_network, layer_t *m_prev_layer, layer_type_t m_layer_type);
    ~lstm_layer_t();
    void init(section_config_t m_section_config);
    void init_weight(std::fstream &m_weight_file);
    void init_weight();
    void store_weight(std::fstream &m_weight_file);
    void _forward_();
    void weight_fields(std::vector<weight_field_t> &out) const;
    // hidden_state / cell_state between forward() calls (network_t::carry_state): kept, or cleared for a new stream
    void carry_state(bool on);
    void reset_state();
private:
    void pack();
    bool batch_normalize;
    // parameter holders in the reference's member order; file order is i, f, o, c for W then U
    connected_layer_t *input_gate_W, *forget_gate_W, *cell_gate_W, *output_gate_W;
    connected_layer_t *input_gate_U, *forget_gate_U, *cell_gate_U, *output_gate_U;
    nbl_lstm_plan *plan;
};

// models/layers/rnn_layer.h: three connected sub-layers (input, hidden, output gate) sharing the section's
// output size, activation and batch_normalize
class rnn_layer_t : public layer_t {
public:
    rnn_layer_t(network_t *m_network, layer_t *m_prev_layer, layer_type_t m_layer_type);
    ~rnn_layer_t();
    void init(section_config_t m_section_config);
    void init_weight(std::fstream &m_weight_file);
    void init_weight();
    void store_weight(std::fstream &m_weight_file);
    void _forward_();
    void weight_fields(std::vector<weight_field_t> &out) const;
private:
    void pack();
    bool batch_normalize;
    connected_layer_t *input_gate, *hidden_gate, *output_gate;    // file order
    nbl_rnn_plan *plan;
};

// models/layers/rbm_layer.h at inference: forward() is a connected layer without batchnorm
// (rbm_layer.cc:345-374); the file holds hidden_bias[O] then weight[O][I] (:150-153).
class rbm_layer_t : public connected_layer_t {
public:
    rbm_layer_t(network_t *m_network, layer_t *m_prev_layer, layer_type_t m_layer_type);
    void init(section_config_t m_section_config);
};

}  // namespace nebula
#endif
