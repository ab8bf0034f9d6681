// network_t: the caller of the forward path (the reference's models/networks/network.h:19-96 surface,
// inference half) and inference_net_t, a driver that builds either kind of shipped network
// (image nets and recurrent nets) from a network.cfg and feeds it tensors instead of datasets.
//
// Where the reference prints to std::cerr and calls exit(1), this code throws std::runtime_error
// with the same text; a command-line driver may turn that back into exit(1).
#ifndef NEBULA_HOST_NETWORK_H
#define NEBULA_HOST_NETWORK_H

#include <istream>
#include <string>
#include <vector>

#include "def.h"
#include "nebula_hip.h"

namespace nebula {

class layer_t;

class network_t {
public:
    network_t();
    virtual ~network_t();

    // Forward propagation: layers[i]->_forward_() in cfg order (models/networks/network.cc:57-63).
    void forward();
    // Training is outside this build.
    void backward();
    void update();
    // run type, network.cfg, data.cfg (unused by inference_net_t), weight file
    void init(const std::string m_run_type, const std::string m_network_config,
              const std::string m_data_config, const std::string m_input_weight = "");
    virtual void run(const std::string m_output_weight = "") = 0;

    run_type_t run_type;
    unsigned num_threads;               // kept for cfg compatibility; the GPU path does not use it

    float learning_rate, momentum, decay, cost;   // parsed, unused at inference

    unsigned input_height, input_width, input_channel, input_size;
    unsigned batch_size;                // already multiplied by time_step for recurrent nets
    unsigned time_step;

    float *input_data;                  // host staging buffer [batch_size][input_size]
    float *input_label;                 // unused at inference
    float *input_data_dev;              // device input [batch_size][input_size]

    nbl_ctx *ctx;                       // takes the place of cublas_handle / cudnn_handle
    // Recurrent nets fed by set_input_tokens(): position of the 1 in each one-hot input row, [T*B] time-major
    // (NULL while the dense input_data_dev is the input).  The first layer, if an LSTM, gathers instead of multiplying.
    unsigned *input_tokens_dev;
    // [net] key `conv_split` (a key the reference ignores): 0 = convolutions never split their sum over
    // the patch rows between blocks, 1 = wherever the cost model says so; absent = measured per layer on
    // first use.  With 0 a convolution's result does not depend on the tile shape the search picks.
    int conv_split;
    // [net] key `pool_index=1` (a key the reference ignores): max-pooling layers also store the argmax table the
    // reference's forward writes for its backward pass (models/layers/pooling_layer.cc:132,140).  Inference never
    // reads it, so by default it is neither allocated nor written (a third of a max-pool's memory traffic).
    bool pool_index;
    // [net] key `carry_state=1` (see inference_net_t::set_carry_state): [lstm] layers keep their state between passes
    bool carry_state;
    // Set while inference_net_t::forward() records or replays a HIP graph: a layer that copies to the host queues
    // the copy on the stream instead of waiting for it, and forward() waits once at its end.
    bool defer_host_copy;

    // Opens the headerless fp32 .wgh stream and lets every layer read its fields in cfg order
    // (models/networks/network.cc:99-122).
    void init_weight(const std::string m_input_weight);
    void store_weight(const std::string m_output_weight);

    std::vector<layer_t*> layers;
    std::vector<int> output_tensor;      // per layer: index of the layer that owns the tensor its output pointer refers to
    layer_t *input_layer, *output_layer;
    unsigned num_layers;

protected:
    virtual void init_network(const std::string m_network_config) = 0;
    virtual void init_data(const std::string m_data_config) = 0;
    virtual void load_data(const unsigned m_batch_index) = 0;
    virtual void print_results() = 0;
};

class inference_net_t : public network_t {
public:
    // device: HIP device ordinal.  batch_override > 0 replaces `batch=` of the [net] section.
    explicit inference_net_t(int device = 0, unsigned batch_override = 0);
    ~inference_net_t();

    // Build from cfg text instead of a file.
    void init_from_stream(std::istream &cfg, const std::string m_input_weight = "");
    // Copy a host tensor [batch_size][input_size] to the device input.
    void set_input(const float *host, size_t count);
    // `images` 8-bit interleaved images [height][width][input_channel] (channel order B, G, R as decoded) ->
    // network input, as convolutional_t::load_data() prepares it (resize, / 255, planes 0 and 2 swapped).
    void set_input_images(const unsigned char *host, unsigned images, unsigned height, unsigned width);
    // The recurrent driver's load_data() (models/networks/recurrent.cc:179-204) without materialising the one-hot
    // matrix: tokens[T*B] time-major, each the index of the 1.0 of its input row.  A later set_input() switches back.
    void set_input_tokens(const unsigned *host, size_t count);
    // recurrent_t::print_results(), test branch (recurrent.cc:239-247): adds sum_rows probability(label token) of
    // the output layer to cumulative_cost and returns exp(-log2(cumulative_cost / rows seen so far)).
    float accumulate_perplexity(const unsigned *label_tokens_host, size_t count);
    float cumulative_cost; size_t rows_seen;
    // convolutional_t::print_results(), test branch (convolutional.cc:428-447): running count of rows whose label
    // is among the output layer's k largest entries.
    unsigned accumulate_topk(const unsigned *labels_host, size_t count, unsigned k);
    unsigned topk_matches;
    void run(const std::string m_output_weight = "");
    bool recurrent() const { return is_recurrent; }

    // network_t::forward(), plus the `last_step_only` option below.
    void forward();
    // forward() with a HIP event between layers; ms[i] = time of layer i.
    void forward_timed(std::vector<float> &ms);
    // Recurrent nets only, [net] key `last_step_only=1` (a key the reference ignores): the layers after
    // the last LSTM see only the rows of the final time step (B rows instead of T*B), i.e. the output
    // projection and softmax are computed for the last step alone.
    bool last_step_only;
    // [net] key `fuse_shortcut=1` (a key the reference ignores): a convolution directly followed by a
    // [shortcut] computes the residual add and the shortcut's activation in its own epilogue.  Same float
    // operations in the same order; the convolution's pre-shortcut output is then never materialised.
    bool fuse_shortcut;
    // [net] key `shortcut_in_place=1` (with fuse_shortcut; a key the reference ignores): a fused shortcut whose
    // connection has the output's shape writes its result over the connection's tensor instead of into a buffer of
    // its own, wherever every other reader of that tensor runs before the fused convolution.  Each element is read
    // and written by the same lane, so the values are the same; what changes is that the connection layer's output
    // no longer exists after the pass (nbl_net_layer_output of it returns the shortcut's tensor) and that the
    // memory system sees one address stream for residual and result (a 64x256x56x56 residual layer: 106 -> 84 us).
    bool shortcut_in_place;
    // [net] key `hip_graph=1` (a key the reference ignores): forward() records the launches of one pass into a
    // HIP graph and replays it from then on, so a pass costs one launch on the host instead of one per kernel
    // (recurrent nets launch a kernel per layer and time step).  The first pass of a configuration runs
    // eagerly (tile search, workspaces grow), the second is recorded, later ones replay.  Anything that changes
    // what a pass launches (weights, token vs. dense input, last_step_only, the softmax copy) makes the next
    // pass start over; call invalidate_graph() after changing a layer behind the network's back.
    bool use_graph;
    // [net] key `carry_state=1` of a recurrent net (a key the reference ignores): [lstm] layers start a pass from the
    // hidden and cell state their previous pass ended with, as lstm_layer_t's never-cleared hidden_state / cell_state
    // do between the batches of one token stream; reset_state() starts a new stream.  Such passes run eagerly.
    void set_carry_state(bool on);
    void reset_state();
    void invalidate_graph();
    bool graph_active() const { return graph_exec != NULL; }   // true once a recorded pass is being replayed
    void forward_eager();

protected:
    void init_network(const std::string m_network_config);
    void init_data(const std::string m_data_config);
    void load_data(const unsigned m_batch_index);
    void print_results();

private:
    void build(class config_t &config);
    void run_layer(unsigned i);
    int first_after_lstm;      // index of the first layer after the last LSTM, -1 if none
    unsigned batch_override;
    bool is_recurrent;
    unsigned char *image_staging_dev;   // device copy of the last byte-image batch
    unsigned *tokens_dev, *labels_dev; float *cost_dev;   // token input, label tokens and the device-side sum
    size_t image_staging_bytes;
    std::vector<void*> events;
    void *graph_exec;                   // hipGraphExec_t of the recorded pass, NULL if none
    unsigned long long graph_key, warm_key;   // configuration the graph was recorded for / the last eager pass ran with
    unsigned graph_epoch;               // bumped by invalidate_graph()
    bool graph_unusable;                // recording failed once: stay eager
    unsigned long long pass_key() const;
};

// Throws std::runtime_error(nbl_last_error) when an ABI call fails.
void nbl_check(nbl_ctx *ctx, int rc, const char *what);

}  // namespace nebula
#endif
