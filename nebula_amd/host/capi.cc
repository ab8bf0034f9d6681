// C entry points over the C++ layer framework (include/nebula_layers.h).
#include "nebula_layers.h"

#include <cstring>
#include <sstream>
#include <stdexcept>
#include <string>
#include <vector>

#include "layers.h"
#include "network.h"

using namespace nebula;

struct nbl_net { inference_net_t *net; };

static thread_local std::string g_error;

#define NBL_NET_TRY(body) \
    try { body; return 0; } \
    catch(const std::exception &e) { g_error = e.what(); return -1; } \
    catch(...) { g_error = "unknown C++ exception"; return -1; }

static layer_t *layer_at(nbl_net *n, int i) {
    if(!n || i < 0 || (size_t)i >= n->net->layers.size()) throw std::runtime_error("Error: layer index out of range");
    return n->net->layers[(size_t)i];
}

extern "C" {

const char *nbl_net_last_error(void) { return g_error.c_str(); }

int nbl_net_create(const char *cfg, int is_text, unsigned batch_override, int device,
                   const char *weight_path, nbl_net **out) {
    if(!out || !cfg) { g_error = "nbl_net_create: NULL argument"; return -1; }
    *out = NULL;
    inference_net_t *net = NULL;
    try {
        net = new inference_net_t(device, batch_override);
        const std::string w = weight_path ? weight_path : "";
        if(is_text) {
            std::istringstream in(cfg);
            net->init_from_stream(in, w);
        } else if(w.size()) {
            net->init("test", cfg, "", w);
        } else {
            std::ifstream in(cfg);
            if(!in.is_open()) throw std::runtime_error(std::string("Error: failed to open ") + cfg);
            net->init_from_stream(in, "");
        }
        *out = new nbl_net{ net };
        return 0;
    } catch(const std::exception &e) {
        g_error = e.what();
        delete net;
        return -1;
    }
}

int nbl_net_destroy(nbl_net *n) {
    if(!n) return -1;
    delete n->net;
    delete n;
    return 0;
}

int nbl_net_load_weights(nbl_net *n, const char *weight_path) {
    NBL_NET_TRY(if(!n || !weight_path) throw std::runtime_error("NULL argument"); n->net->invalidate_graph(); n->net->init_weight(weight_path));
}

int nbl_net_store_weights(nbl_net *n, const char *weight_path) {
    NBL_NET_TRY(if(!n || !weight_path) throw std::runtime_error("NULL argument"); n->net->store_weight(weight_path));
}

int nbl_net_weight_layout(nbl_net *n, unsigned *fields, size_t capacity, size_t *num_fields) {
    NBL_NET_TRY(
        if(!n || !num_fields) throw std::runtime_error("NULL argument");
        size_t count = 0;
        for(size_t i = 0; i < n->net->layers.size(); i++) {
            std::vector<weight_field_t> f;
            n->net->layers[i]->weight_fields(f);
            for(size_t j = 0; j < f.size(); j++, count++) {
                if(fields && count < capacity) {
                    unsigned *dst = fields + 4 * count;
                    dst[0] = (unsigned)i; dst[1] = (unsigned)f[j].kind; dst[2] = f[j].count; dst[3] = f[j].fan_in;
                }
            }
        }
        *num_fields = count);
}

int nbl_net_dims(nbl_net *n, unsigned *d) {
    if(!n || !d) return -1;
    d[0] = n->net->batch_size; d[1] = n->net->time_step; d[2] = n->net->input_size;
    d[3] = n->net->input_height; d[4] = n->net->input_width; d[5] = n->net->input_channel;
    return 0;
}

int nbl_net_num_layers(nbl_net *n) { return n ? (int)n->net->layers.size() : -1; }

int nbl_net_layer_info(nbl_net *n, int i, unsigned *info) {
    NBL_NET_TRY(
        layer_t *l = layer_at(n, i);
        info[0] = l->layer_type; info[1] = l->activation_type; info[2] = l->output_channel;
        info[3] = l->output_height; info[4] = l->output_width; info[5] = l->output_size;
        info[6] = l->input_size; info[7] = l->padding);
}

int nbl_net_layer_flop(nbl_net *n, int i, double *flop) {
    NBL_NET_TRY(
        layer_t *l = layer_at(n, i);
        *flop = 0.0;
        if(l->layer_type == CONVOLUTIONAL_LAYER) *flop = static_cast<convolutional_layer_t*>(l)->flop_per_image();
        else if(l->layer_type == CONNECTED_LAYER || l->layer_type == RBM_LAYER) *flop = 2.0 * l->input_size * l->output_size;
        else if(l->layer_type == RNN_LAYER) *flop = 2.0 * (l->input_size + 2.0 * l->output_size) * l->output_size;
        else if(l->layer_type == LSTM_LAYER) *flop = 2.0 * (l->input_size + (double)l->output_size) * 4.0 * l->output_size);
}

int nbl_net_set_input(nbl_net *n, const float *host, size_t count) {
    NBL_NET_TRY(if(!n || !host) throw std::runtime_error("NULL argument"); n->net->set_input(host, count));
}

int nbl_net_set_input_images(nbl_net *n, const unsigned char *host, unsigned images, unsigned height, unsigned width) {
    NBL_NET_TRY(if(!n || !host) throw std::runtime_error("NULL argument"); n->net->set_input_images(host, images, height, width));
}

int nbl_net_set_input_tokens(nbl_net *n, const unsigned *host, size_t count) {
    NBL_NET_TRY(if(!n || !host) throw std::runtime_error("NULL argument"); n->net->set_input_tokens(host, count));
}

int nbl_net_accumulate_perplexity(nbl_net *n, const unsigned *label_tokens, size_t count, float *perplexity) {
    NBL_NET_TRY(
        if(!n || !label_tokens || !perplexity) throw std::runtime_error("NULL argument");
        *perplexity = n->net->accumulate_perplexity(label_tokens, count));
}

int nbl_net_accumulate_topk(nbl_net *n, const unsigned *labels, size_t count, unsigned k, unsigned *matches) {
    NBL_NET_TRY(
        if(!n || !labels || !matches) throw std::runtime_error("NULL argument");
        *matches = n->net->accumulate_topk(labels, count, k));
}

int nbl_net_forward(nbl_net *n) {
    NBL_NET_TRY(if(!n) throw std::runtime_error("NULL argument"); n->net->forward());
}

int nbl_net_sync(nbl_net *n) {
    NBL_NET_TRY(if(!n) throw std::runtime_error("NULL argument"); nbl_check(n->net->ctx, nbl_sync(n->net->ctx), "nbl_sync"));
}

int nbl_net_forward_timed(nbl_net *n, float *ms) {
    NBL_NET_TRY(
        if(!n || !ms) throw std::runtime_error("NULL argument");
        std::vector<float> v;
        n->net->forward_timed(v);
        memcpy(ms, v.data(), v.size() * sizeof(float)));
}

int nbl_net_layer_output(nbl_net *n, int i, float *host, size_t count) {
    NBL_NET_TRY(
        layer_t *l = layer_at(n, i);
        if(count != (size_t)l->output_size * n->net->batch_size) throw std::runtime_error("Error: output buffer has the wrong size");
        nbl_check(n->net->ctx, nbl_d2h(n->net->ctx, host, l->output_data_dev, count * sizeof(float)), "nbl_d2h"));
}

int nbl_net_layer_output_writer(nbl_net *n, int i, int *writer) {
    NBL_NET_TRY(
        layer_t *l = layer_at(n, i);
        if(!writer) throw std::runtime_error("Error: writer is NULL");
        // the last layer with a kernel of its own that writes the tensor this layer's output pointer refers to
        (void)l;
        const std::vector<layer_t*> &layers = n->net->layers;
        // a dropout or cost layer has no kernel: its values are its producer's
        int own = i;
        while(own > 0 && (layers[own]->layer_type == DROPOUT_LAYER || layers[own]->layer_type == COST_LAYER)) own--;
        *writer = own;
        const std::vector<int> &tensor = n->net->output_tensor;
        for(int j = i + 1; j < (int)layers.size() && j < (int)tensor.size(); j++) {
            const layer_type_t t = layers[j]->layer_type;
            if(t == DROPOUT_LAYER || t == COST_LAYER) continue;
            if(tensor[j] == tensor[i]) *writer = j;
        });
}

int nbl_net_pool_index(nbl_net *n, int i, unsigned *host, size_t count) {
    NBL_NET_TRY(
        layer_t *l = layer_at(n, i);
        if(l->layer_type != MAXPOOL_LAYER) throw std::runtime_error("Error: not a maxpool layer");
        if(count != (size_t)l->output_size * n->net->batch_size) throw std::runtime_error("Error: index buffer has the wrong size");
        if(!static_cast<pooling_layer_t*>(l)->index_dev) throw std::runtime_error("Error: the argmax table is not kept (set pool_index=1 in [net])");
        nbl_check(n->net->ctx, nbl_d2h(n->net->ctx, host, static_cast<pooling_layer_t*>(l)->index_dev,
                                       count * sizeof(unsigned)), "nbl_d2h"));
}

int nbl_net_conv_last_launch(nbl_net *n, int i, int *variant, int *slices) {
    NBL_NET_TRY(
        layer_t *l = layer_at(n, i);
        if(l->layer_type != CONVOLUTIONAL_LAYER) throw std::runtime_error("Error: not a convolutional layer");
        static_cast<convolutional_layer_t*>(l)->last_launch(variant, slices));
}

int nbl_net_conv_problem(nbl_net *n, int i, unsigned *key) {
    NBL_NET_TRY(
        layer_t *l = layer_at(n, i);
        if(l->layer_type != CONVOLUTIONAL_LAYER) throw std::runtime_error("Error: not a convolutional layer");
        if(!key) throw std::runtime_error("Error: key is NULL");
        const convolutional_layer_t *c = static_cast<convolutional_layer_t*>(l);
        key[0] = c->input_channel; key[1] = c->input_height; key[2] = c->input_width; key[3] = c->num_filters;
        key[4] = c->filter_size; key[5] = c->stride; key[6] = c->padding; key[7] = n->net->batch_size;
        key[8] = key[9] = key[10] = key[11] = 0;
        if(c->shortcut_fused()) {
            const layer_t *conn = c->shortcut_fused()->connection;
            key[8] = conn->output_channel; key[9] = conn->output_height; key[10] = conn->output_width;
            key[11] = c->shortcut_fused()->in_place ? 1u : 0u;
        });
}

int nbl_net_conv_launch_source(nbl_net *n, int i, int *source) {
    NBL_NET_TRY(
        layer_t *l = layer_at(n, i);
        if(l->layer_type != CONVOLUTIONAL_LAYER) throw std::runtime_error("Error: not a convolutional layer");
        if(!source) throw std::runtime_error("Error: source is NULL");
        *source = static_cast<convolutional_layer_t*>(l)->launch_source());
}

int nbl_net_conv_pin_launch(nbl_net *n, int i, int variant, int split) {
    NBL_NET_TRY(
        layer_t *l = layer_at(n, i);
        if(l->layer_type != CONVOLUTIONAL_LAYER) throw std::runtime_error("Error: not a convolutional layer");
        n->net->invalidate_graph();
        static_cast<convolutional_layer_t*>(l)->pin_launch(variant, split));
}

int nbl_net_softmax_copy(nbl_net *n, int enabled) {
    if(!n) return -1;
    for(size_t i = 0; i < n->net->layers.size(); i++)
        if(n->net->layers[i]->layer_type == SOFTMAX_LAYER)
            static_cast<softmax_layer_t*>(n->net->layers[i])->copy_to_host = enabled != 0;
    return 0;
}

int nbl_net_set_graph(nbl_net *n, int enabled) {
    if(!n) return -1;
    n->net->invalidate_graph();
    n->net->use_graph = enabled != 0;
    return 0;
}

int nbl_net_set_carry_state(nbl_net *n, int enabled) {
    NBL_NET_TRY(if(!n) throw std::runtime_error("NULL argument"); n->net->set_carry_state(enabled != 0));
}

int nbl_net_reset_state(nbl_net *n) {
    NBL_NET_TRY(if(!n) throw std::runtime_error("NULL argument"); n->net->reset_state());
}

int nbl_net_graph_active(nbl_net *n) { return n ? (n->net->graph_active() ? 1 : 0) : -1; }

void *nbl_net_ctx(nbl_net *n) { return n ? (void*)n->net->ctx : NULL; }

}  // extern "C"
