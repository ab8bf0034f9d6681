#include "network.h"

#include <cmath>

#include <hip/hip_runtime_api.h>

#include <fstream>
#include <sstream>
#include <stdexcept>

#include "config.h"
#include "layers.h"

namespace nebula {

void nbl_check(nbl_ctx *ctx, int rc, const char *what) {
    if(rc == NBL_OK) return;
    std::ostringstream msg;
    msg << "Error: " << what << " failed (" << rc << "): " << nbl_last_error(ctx);
    throw std::runtime_error(msg.str());
}

network_t::network_t() :
    run_type(UNDEFINED_RUN), num_threads(1),
    learning_rate(0.001f), momentum(0.9f), decay(0.0001f), cost(0.0f),
    input_height(1), input_width(1), input_channel(1), input_size(0), batch_size(1), time_step(1),
    input_data(NULL), input_label(NULL), input_data_dev(NULL), ctx(NULL), input_tokens_dev(NULL), conv_split(-1), pool_index(false), carry_state(false), defer_host_copy(false),
    input_layer(NULL), output_layer(NULL), num_layers(0) {}

network_t::~network_t() {}

void network_t::forward() {
    for(unsigned i = 0; i < num_layers; i++) layers[i]->_forward_();
}

void network_t::backward() { throw std::runtime_error("Error: backward() is not part of the inference-only build"); }
void network_t::update() { throw std::runtime_error("Error: update() is not part of the inference-only build"); }

void network_t::init(const std::string m_run_type, const std::string m_network_config,
                     const std::string m_data_config, const std::string m_input_weight) {
    run_type = (run_type_t)lookup_type(run_type_str, NUM_RUN_TYPES, m_run_type);
    if(run_type != TEST_RUN) throw std::runtime_error("Error: only the `test` (inference) run type is supported");
    init_network(m_network_config);
    init_data(m_data_config);
    init_weight(m_input_weight);
}

void network_t::init_weight(const std::string m_input_weight) {
    if(m_input_weight.size()) {
        std::fstream weight_file(m_input_weight.c_str(), std::fstream::in | std::fstream::binary);
        if(!weight_file.is_open()) throw std::runtime_error("Error: failed to open " + m_input_weight);
        for(size_t i = 0; i < layers.size(); i++) layers[i]->init_weight(weight_file);
    } else {
        if(run_type == TEST_RUN)
            throw std::runtime_error(std::string("Error: missing input weight for ") + run_type_str[run_type]);
        for(size_t i = 0; i < layers.size(); i++) layers[i]->init_weight();
    }
}

void network_t::store_weight(const std::string m_output_weight) {
    if(!m_output_weight.size()) return;
    std::fstream weight_file(m_output_weight.c_str(), std::fstream::out | std::fstream::binary);
    if(!weight_file.is_open()) throw std::runtime_error("Error: failed to open " + m_output_weight);
    for(size_t i = 0; i < layers.size(); i++) layers[i]->store_weight(weight_file);
}

// ---- inference_net_t -------------------------------------------------------------------------------
inference_net_t::inference_net_t(int device, unsigned m_batch_override) :
    cumulative_cost(0.0f), rows_seen(0), topk_matches(0), last_step_only(false), fuse_shortcut(false), shortcut_in_place(false), use_graph(false),
    first_after_lstm(-1), batch_override(m_batch_override), is_recurrent(false), image_staging_dev(NULL),
    tokens_dev(NULL), labels_dev(NULL), cost_dev(NULL), image_staging_bytes(0),
    graph_exec(NULL), graph_key(0), warm_key(0), graph_epoch(1), graph_unusable(false) {
    run_type = TEST_RUN;
    if(device < 0) return;            // dry run: shapes, cfg and .wgh handling only; no device, no forward
    int rc = nbl_ctx_create(device, &ctx);
    if(rc != NBL_OK) {
        std::ostringstream msg;
        msg << "Error: cannot create a device context (" << rc << "): " << nbl_last_error(NULL);
        throw std::runtime_error(msg.str());
    }
}

inference_net_t::~inference_net_t() {
    if(graph_exec) { if(ctx) nbl_sync(ctx); (void)hipGraphExecDestroy((hipGraphExec_t)graph_exec); }
    for(size_t i = layers.size(); i > 0; i--) delete layers[i - 1];
    for(size_t i = 0; i < events.size(); i++) (void)hipEventDestroy((hipEvent_t)events[i]);
    if(input_data_dev && ctx) nbl_free(ctx, input_data_dev);
    if(image_staging_dev && ctx) nbl_free(ctx, image_staging_dev);
    if(ctx) { nbl_free(ctx, tokens_dev); nbl_free(ctx, labels_dev); nbl_free(ctx, cost_dev); }
    delete [] input_data;
    if(ctx) nbl_ctx_destroy(ctx);
}

void inference_net_t::init_network(const std::string m_network_config) {
    config_t config;
    config.parse(m_network_config);
    build(config);
}

void inference_net_t::init_from_stream(std::istream &cfg, const std::string m_input_weight) {
    config_t config;
    config.parse_stream(cfg);
    build(config);
    init_data("");
    if(m_input_weight.size()) init_weight(m_input_weight);
}

// One pass over the sections, as the reference's two drivers do
// (models/networks/convolutional.cc:52-122 for image nets, recurrent.cc:115-175 for recurrent nets;
// a [net] section holding time_steps= selects the recurrent reading).
void inference_net_t::build(config_t &config) {
    if(config.sections.empty() || config.sections[0].name != "net")
        throw std::runtime_error("Error: network config must start with a [net] section");
    num_layers = (unsigned)config.sections.size() - 1;
    layers.reserve(num_layers);
    for(size_t i = 0; i < config.sections.size(); i++) {
        section_config_t sc = config.sections[i];
        if(sc.name == "net") {
            sc.get_setting("num_threads", &num_threads);
            sc.get_setting("learning_rate", &learning_rate);
            sc.get_setting("momentum", &momentum);
            sc.get_setting("decay", &decay);
            sc.get_setting("height", &input_height);
            sc.get_setting("width", &input_width);
            sc.get_setting("channels", &input_channel);
            sc.get_setting("batch", &batch_size);
            sc.get_setting("fuse_shortcut", &fuse_shortcut);
            sc.get_setting("shortcut_in_place", &shortcut_in_place);
            sc.get_setting("hip_graph", &use_graph);
            sc.get_setting("pool_index", &pool_index);
            if(sc.exists("conv_split")) { unsigned v = 0; sc.get_setting("conv_split", &v); conv_split = v ? 1 : 0; }
            if(batch_override) batch_size = batch_override;
            input_size = input_height * input_width * input_channel;
            if(sc.exists("time_steps")) {
                is_recurrent = true;
                sc.get_setting("input_size", &input_size);
                sc.get_setting("time_steps", &time_step);
                sc.get_setting("last_step_only", &last_step_only);
                sc.get_setting("carry_state", &carry_state);
                batch_size *= time_step;                 // rows = time steps x sequences, time-major
            }
            if(!batch_size || !input_size) throw std::runtime_error("Error: [net] gives an empty input");
            continue;
        }
        layer_t *prev = layers.size() ? layers.back() : NULL;
        layer_t *layer = NULL;
        if(sc.name == "convolutional")   layer = new convolutional_layer_t(this, prev, CONVOLUTIONAL_LAYER);
        else if(sc.name == "connected")  layer = new connected_layer_t(this, prev, CONNECTED_LAYER);
        else if(sc.name == "dropout")    layer = new dropout_layer_t(this, prev, DROPOUT_LAYER);
        else if(sc.name == "maxpool")    layer = new pooling_layer_t(this, prev, MAXPOOL_LAYER);
        else if(sc.name == "avgpool")    layer = new pooling_layer_t(this, prev, AVGPOOL_LAYER);
        else if(sc.name == "shortcut")   layer = new shortcut_layer_t(this, prev, SHORTCUT_LAYER);
        else if(sc.name == "softmax")  { layer = new softmax_layer_t(this, prev, SOFTMAX_LAYER); output_layer = layer; }
        else if(sc.name == "cost")       layer = new cost_layer_t(this, prev, COST_LAYER);
        else if(sc.name == "lstm")       layer = new lstm_layer_t(this, prev, LSTM_LAYER);
        else if(sc.name == "rnn")        layer = new rnn_layer_t(this, prev, RNN_LAYER);
        else if(sc.name == "rbm")        layer = new rbm_layer_t(this, prev, RBM_LAYER);
        else throw std::runtime_error("Error: unknown layer type " + sc.name);
        if(layers.empty()) input_layer = layer;
        layers.push_back(layer);            // owned from here on, also if init() throws
        layer->init(sc);
    }
    num_layers = (unsigned)layers.size();
    if(!output_layer && !layers.empty()) output_layer = layers.back();
    // The layer whose kernel writes the tensor a layer's output pointer refers to, before any fusion: dropout and cost
    // layers alias their producer.  (Indices, not pointers: a dry-run network has no buffers to compare.)
    std::vector<int> producer(num_layers);
    for(unsigned i = 0; i < num_layers; i++) {
        producer[i] = (int)i;
        if((layers[i]->layer_type == DROPOUT_LAYER || layers[i]->layer_type == COST_LAYER) && i > 0) producer[i] = producer[i - 1];
    }
    auto index_of = [&](const layer_t *l) { for(unsigned i = 0; i < num_layers; i++) if(layers[i] == l) return (int)i; return -1; };
    if(fuse_shortcut)
        for(unsigned i = 1; i < num_layers; i++)
            if(layers[i]->layer_type == SHORTCUT_LAYER && layers[i - 1]->layer_type == CONVOLUTIONAL_LAYER) {
                // A fused convolution never writes its own (pre-add) output.  That is only safe when nothing but the
                // shortcut behind it reads that output: a later shortcut whose `hops` land on this convolution (or
                // on an alias of it) needs the pre-add tensor, so the pair stays unfused.
                bool read_elsewhere = false;
                for(unsigned j = i + 1; j < num_layers && !read_elsewhere; j++)
                    if(layers[j]->layer_type == SHORTCUT_LAYER) {
                        const int conn = index_of(static_cast<shortcut_layer_t*>(layers[j])->connection);
                        read_elsewhere = conn >= 0 && producer[conn] == (int)i - 1;
                    }
                if(!read_elsewhere)
                    static_cast<convolutional_layer_t*>(layers[i - 1])->fuse_with(static_cast<shortcut_layer_t*>(layers[i]));
            }
    if(fuse_shortcut && shortcut_in_place) {
        for(unsigned i = 1; i < num_layers; i++) {
            if(layers[i]->layer_type != SHORTCUT_LAYER) continue;
            shortcut_layer_t *sc = static_cast<shortcut_layer_t*>(layers[i]);
            if(!sc->fused) continue;
            const int conn = index_of(sc->connection);
            if(conn < 0) continue;
            const layer_t *c = layers[conn];
            if(c->output_channel != sc->output_channel || c->output_height != sc->output_height || c->output_width != sc->output_width) continue;
            const int tensor = producer[conn];
            // every other reader of that tensor must run before the fused convolution (layer i - 1) starts writing
            bool safe = true;
            for(unsigned j = 0; j < num_layers && safe; j++) {
                if(j == i) continue;
                const bool reads_as_input = j > 0 && producer[j - 1] == tensor && producer[j] == (int)j;
                const bool reads_as_connection = layers[j]->layer_type == SHORTCUT_LAYER &&
                                                 index_of(static_cast<shortcut_layer_t*>(layers[j])->connection) >= 0 &&
                                                 producer[index_of(static_cast<shortcut_layer_t*>(layers[j])->connection)] == tensor;
                if((reads_as_input || reads_as_connection) && j >= i - 1) safe = false;
            }
            if(layers[tensor] == output_layer) safe = false;
            if(safe) sc->write_over_connection();
        }
    }
    // Dropout and cost layers copied their producer's output pointer when they were initialised; a fusion or an in-place
    // shortcut above has since freed or replaced some of those tensors, so every alias is taken again, in layer order.
    for(unsigned i = 1; i < num_layers; i++)
        if(layers[i]->layer_type == DROPOUT_LAYER || layers[i]->layer_type == COST_LAYER)
            layers[i]->output_data_dev = layers[i - 1]->output_data_dev;
    // Which tensor every layer's output pointer refers to (the index of the layer that owns it): dropout and cost layers
    // share their producer's, a fused convolution its shortcut's, an in-place shortcut its connection's.
    output_tensor.assign(num_layers, 0);
    for(unsigned i = 0; i < num_layers; i++) {
        int t = (int)i;
        if((layers[i]->layer_type == DROPOUT_LAYER || layers[i]->layer_type == COST_LAYER) && i > 0) t = output_tensor[i - 1];
        if(layers[i]->layer_type == SHORTCUT_LAYER) {
            const shortcut_layer_t *sc = static_cast<const shortcut_layer_t*>(layers[i]);
            if(sc->in_place)
                for(unsigned j = 0; j < i; j++) if(layers[j] == sc->connection) t = output_tensor[j];
            if(sc->fused && i > 0) output_tensor[i - 1] = t;
        }
        output_tensor[i] = t;
    }
    for(unsigned i = 0; i < num_layers; i++)
        if(layers[i]->layer_type == LSTM_LAYER || layers[i]->layer_type == RNN_LAYER) first_after_lstm = i + 1 < num_layers ? (int)i + 1 : -1;
}

void inference_net_t::init_data(const std::string) {
    if(input_data_dev || input_data) return;
    const size_t count = (size_t)batch_size * input_size;
    input_data = new float[count]();
    if(!ctx) return;
    nbl_check(ctx, nbl_malloc(ctx, (void**)&input_data_dev, count * sizeof(float)), "nbl_malloc(input)");
    nbl_check(ctx, nbl_fill_zero(ctx, input_data_dev, count * sizeof(float)), "nbl_fill_zero(input)");
    // the first layer captured the (then NULL) input pointer lazily through input_dev(), nothing to patch
}

void inference_net_t::set_input(const float *host, size_t count) {
    if(!ctx) throw std::runtime_error("Error: no device (dry-run network)");
    if(count != (size_t)batch_size * input_size) throw std::runtime_error("Error: input tensor has the wrong size");
    nbl_check(ctx, nbl_h2d(ctx, input_data_dev, host, count * sizeof(float)), "nbl_h2d(input)");
    input_tokens_dev = NULL;
}

void inference_net_t::set_input_tokens(const unsigned *host, size_t count) {
    if(!ctx) throw std::runtime_error("Error: no device (dry-run network)");
    if(!is_recurrent) throw std::runtime_error("Error: token input on a network without time_steps");
    if(count != (size_t)batch_size) throw std::runtime_error("Error: token input has the wrong size");
    if(layers.empty() || (layers[0]->layer_type != LSTM_LAYER && layers[0]->layer_type != RNN_LAYER))
        throw std::runtime_error("Error: token input needs an lstm or rnn layer first");
    if(!tokens_dev) nbl_check(ctx, nbl_malloc(ctx, (void**)&tokens_dev, (size_t)batch_size * sizeof(unsigned)), "nbl_malloc(tokens)");
    nbl_check(ctx, nbl_h2d(ctx, tokens_dev, host, count * sizeof(unsigned)), "nbl_h2d(tokens)");
    input_tokens_dev = tokens_dev;
}

float inference_net_t::accumulate_perplexity(const unsigned *label_tokens_host, size_t count) {
    if(!ctx) throw std::runtime_error("Error: no device (dry-run network)");
    if(!output_layer) throw std::runtime_error("Error: network has no layers");
    // rows the output layer holds: every (time step, sequence) row, or the last step's with last_step_only
    const size_t rows = last_step_only && is_recurrent ? batch_size / time_step : batch_size;
    if(count != rows) throw std::runtime_error("Error: label tokens have the wrong size");
    if(!labels_dev) nbl_check(ctx, nbl_malloc(ctx, (void**)&labels_dev, (size_t)batch_size * sizeof(unsigned)), "nbl_malloc(labels)");
    if(!cost_dev) nbl_check(ctx, nbl_malloc(ctx, (void**)&cost_dev, 16), "nbl_malloc(cost)");
    nbl_check(ctx, nbl_h2d(ctx, labels_dev, label_tokens_host, count * sizeof(unsigned)), "nbl_h2d(labels)");
    nbl_check(ctx, nbl_target_prob_sum(ctx, output_layer->output_data_dev, labels_dev, (unsigned)rows, output_layer->output_size,
                                       cost_dev), "nbl_target_prob_sum");
    float sum = 0.0f;
    nbl_check(ctx, nbl_d2h(ctx, &sum, cost_dev, sizeof(float)), "nbl_d2h(cost)");
    cumulative_cost += sum;
    rows_seen += rows;
    return std::exp(-1.0f * std::log2(cumulative_cost / (float)rows_seen));
}

// The image driver's load_data() contract (models/networks/convolutional.cc:384-412) with the resize,
// scaling and plane reordering done on the device: the batch crosses PCIe as bytes.
void inference_net_t::set_input_images(const unsigned char *host, unsigned images, unsigned height, unsigned width) {
    if(!ctx) throw std::runtime_error("Error: no device (dry-run network)");
    if(is_recurrent) throw std::runtime_error("Error: image input on a recurrent network");
    if(images != batch_size) throw std::runtime_error("Error: input batch has the wrong number of images");
    const size_t bytes = (size_t)images * height * width * input_channel;
    if(bytes > image_staging_bytes) {
        nbl_check(ctx, nbl_free(ctx, image_staging_dev), "nbl_free(image staging)");
        image_staging_dev = NULL; image_staging_bytes = 0;
        nbl_check(ctx, nbl_malloc(ctx, (void**)&image_staging_dev, bytes), "nbl_malloc(image staging)");
        image_staging_bytes = bytes;
    }
    nbl_check(ctx, nbl_h2d(ctx, image_staging_dev, host, bytes), "nbl_h2d(images)");
    nbl_check(ctx, nbl_image_to_input(ctx, image_staging_dev, images, height, width, input_channel, input_data_dev,
                                      input_height, input_width), "nbl_image_to_input");
}

unsigned inference_net_t::accumulate_topk(const unsigned *labels_host, size_t count, unsigned k) {
    if(!ctx) throw std::runtime_error("Error: no device (dry-run network)");
    if(!output_layer) throw std::runtime_error("Error: network has no layers");
    const size_t rows = last_step_only && is_recurrent ? batch_size / time_step : batch_size;
    if(count != rows) throw std::runtime_error("Error: labels have the wrong size");
    if(!labels_dev) nbl_check(ctx, nbl_malloc(ctx, (void**)&labels_dev, (size_t)batch_size * sizeof(unsigned)), "nbl_malloc(labels)");
    if(!cost_dev) nbl_check(ctx, nbl_malloc(ctx, (void**)&cost_dev, 16), "nbl_malloc(cost)");
    nbl_check(ctx, nbl_h2d(ctx, labels_dev, labels_host, count * sizeof(unsigned)), "nbl_h2d(labels)");
    nbl_check(ctx, nbl_topk_matches(ctx, output_layer->output_data_dev, labels_dev, (unsigned)rows, output_layer->output_size, k,
                                    reinterpret_cast<unsigned*>(cost_dev)), "nbl_topk_matches");
    unsigned found = 0;
    nbl_check(ctx, nbl_d2h(ctx, &found, cost_dev, sizeof(unsigned)), "nbl_d2h(matches)");
    topk_matches += found;
    return topk_matches;
}

void inference_net_t::load_data(const unsigned) {}
void inference_net_t::print_results() {}

void inference_net_t::run(const std::string) {
    forward();
    nbl_check(ctx, nbl_sync(ctx), "nbl_sync");
}

// Layer i, with the rows narrowed to the final time step behind the last recurrent layer when last_step_only is
// set.  A layer there that reads the recurrent layer's T*B rows -- directly, or through layers that only alias
// their producer's buffer (dropout, cost) -- is pointed at the last B rows for the duration of its call; every
// layer behind the recurrent layer works on B rows.  Pointer and row count are restored right after the call.
void inference_net_t::run_layer(unsigned i) {
    const bool narrow = last_step_only && is_recurrent && time_step > 1 && first_after_lstm >= 0 &&
                        (int)i >= first_after_lstm;
    if(!narrow) { layers[i]->_forward_(); return; }
    const unsigned rows = batch_size, seqs = batch_size / time_step;
    layer_t *src = layers[i]->prev_layer;       // the layer whose output pointer layer i reads
    const layer_t *real = src;                  // ... and the layer that wrote the rows behind that pointer
    while(real && (real->layer_type == DROPOUT_LAYER || real->layer_type == COST_LAYER)) real = real->prev_layer;
    const bool reads_all_steps = real != NULL && real == layers[first_after_lstm - 1];
    float *saved = src ? src->output_data_dev : NULL;
    if(reads_all_steps) src->output_data_dev += (size_t)(time_step - 1) * seqs * src->output_size;
    batch_size = seqs;
    try { layers[i]->_forward_(); }
    catch(...) { batch_size = rows; if(src) src->output_data_dev = saved; throw; }
    batch_size = rows;
    if(src) src->output_data_dev = saved;
}

void inference_net_t::forward_eager() {
    if(!ctx) throw std::runtime_error("Error: no device (dry-run network)");
    for(unsigned i = 0; i < num_layers; i++) run_layer(i);
}

void inference_net_t::set_carry_state(bool on) {
    carry_state = on;
    for(size_t i = 0; i < layers.size(); i++)
        if(layers[i]->layer_type == LSTM_LAYER) static_cast<lstm_layer_t*>(layers[i])->carry_state(on);
}

void inference_net_t::reset_state() {
    for(size_t i = 0; i < layers.size(); i++)
        if(layers[i]->layer_type == LSTM_LAYER) static_cast<lstm_layer_t*>(layers[i])->reset_state();
}

void inference_net_t::invalidate_graph() {
    ++graph_epoch;
    if(graph_exec) {
        if(ctx) nbl_sync(ctx);
        (void)hipGraphExecDestroy((hipGraphExec_t)graph_exec);
        graph_exec = NULL;
    }
}

// What a pass launches depends on: the rows per pass, dense or token input, last_step_only, which softmax layers
// copy to the host, and everything invalidate_graph() stands for (weights, plans).  Never 0.
unsigned long long inference_net_t::pass_key() const {
    unsigned long long k = 1469598103934665603ull;
    const unsigned long long parts[] = { batch_size, time_step, (unsigned long long)last_step_only, graph_epoch,
                                         (unsigned long long)(size_t)input_tokens_dev, (unsigned long long)(size_t)input_data_dev };
    for(size_t i = 0; i < sizeof(parts) / sizeof(parts[0]); i++) k = (k ^ parts[i]) * 1099511628211ull;
    for(unsigned i = 0; i < num_layers; i++)
        if(layers[i]->layer_type == SOFTMAX_LAYER)
            k = (k ^ (static_cast<const softmax_layer_t*>(layers[i])->copy_to_host ? 2u : 1u)) * 1099511628211ull;
    return k ? k : 1;
}

void inference_net_t::forward() {
    if(!ctx) throw std::runtime_error("Error: no device (dry-run network)");
    if(!use_graph || graph_unusable || carry_state) { forward_eager(); return; }
    hipStream_t stream = (hipStream_t)nbl_ctx_stream(ctx);
    const unsigned long long key = pass_key();
    if(graph_exec && key != graph_key) invalidate_graph();      // (bumps the epoch: the key is taken again below)
    const unsigned long long now = pass_key();
    if(!graph_exec) {
        if(warm_key != now) {          // first pass of this configuration: tile search, workspaces, lazily built tables
            forward_eager();
            warm_key = now;
            return;
        }
        // second pass: record.  Nothing below may wait for the stream or allocate; a layer that does makes the
        // recording fail, and the network stays on eager passes.
        hipGraph_t graph = NULL;
        if(hipStreamBeginCapture(stream, hipStreamCaptureModeThreadLocal) != hipSuccess) {
            (void)hipGetLastError(); graph_unusable = true; forward_eager(); return;
        }
        defer_host_copy = true;
        bool recorded = true;
        try { for(unsigned i = 0; i < num_layers; i++) run_layer(i); }
        catch(...) { recorded = false; }
        defer_host_copy = false;
        if(hipStreamEndCapture(stream, &graph) != hipSuccess || !graph) recorded = false;
        hipGraphExec_t exec = NULL;
        if(recorded && hipGraphInstantiate(&exec, graph, NULL, NULL, 0) != hipSuccess) recorded = false;
        if(graph) (void)hipGraphDestroy(graph);
        if(!recorded) {
            (void)hipGetLastError();
            graph_unusable = true;
            forward_eager();
            return;
        }
        graph_exec = (void*)exec;
        graph_key = now;
    }
    if(hipGraphLaunch((hipGraphExec_t)graph_exec, stream) != hipSuccess)
        throw std::runtime_error("Error: hipGraphLaunch failed");
    // the recorded pass queues its host copies instead of waiting for each: wait once, as an eager pass ending in
    // a softmax layer does
    nbl_check(ctx, nbl_sync(ctx), "nbl_sync");
}

void inference_net_t::forward_timed(std::vector<float> &ms) {
    if(!ctx) throw std::runtime_error("Error: no device (dry-run network)");
    hipStream_t stream = (hipStream_t)nbl_ctx_stream(ctx);
    while(events.size() < (size_t)num_layers + 1) {
        hipEvent_t e;
        if(hipEventCreate(&e) != hipSuccess) throw std::runtime_error("Error: hipEventCreate failed");
        events.push_back((void*)e);
    }
    for(unsigned i = 0; i < num_layers; i++) {
        if(hipEventRecord((hipEvent_t)events[i], stream) != hipSuccess) throw std::runtime_error("Error: hipEventRecord failed");
        run_layer(i);
    }
    if(hipEventRecord((hipEvent_t)events[num_layers], stream) != hipSuccess) throw std::runtime_error("Error: hipEventRecord failed");
    if(hipEventSynchronize((hipEvent_t)events[num_layers]) != hipSuccess) throw std::runtime_error("Error: hipEventSynchronize failed");
    ms.assign(num_layers, 0.0f);
    for(unsigned i = 0; i < num_layers; i++)
        if(hipEventElapsedTime(&ms[i], (hipEvent_t)events[i], (hipEvent_t)events[i + 1]) != hipSuccess)
            throw std::runtime_error("Error: hipEventElapsedTime failed");
}

}  // namespace nebula
