// TEST INFRASTRUCTURE ONLY -- never linked into, or called by, the product.
//
// A C-callable harness around the *unmodified* Nebula reference sources.  It is
// compiled together with the reference's own .cc files (see oracle/Makefile,
// target `ref`) straight from where they lie under /root/reference, with
// -DCUSTOM_BLAS so that the reference's hand-written threaded GEMM
// (common/gemm.h:108-147) is used and no external BLAS header is needed.
// The resulting library, oracle/_ref/libnebula_ref.so, exists only in the
// authoring container; it validates the C restatement in nebula_oracle.c and
// produces the golden vectors under tests/golden/.
//
// Nothing of the reference is copied here: the harness only *includes* the
// reference headers and drives the reference classes the way
// models/networks/convolutional.cc:52-122 and models/networks/recurrent.cc:115-175
// do (those two drivers cannot be compiled here because they need OpenCV).

#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <fstream>
#include <string>
#include <vector>

#include "config.h"
#include "def.h"
#include "utils.h"
#include "gemm.h"
#include "batchnorm.h"
#include "activations.h"
#include "network.h"
#include "layer.h"
#include "convolutional_layer.h"
#include "connected_layer.h"
#include "dropout_layer.h"
#include "shortcut_layer.h"
#include "softmax_layer.h"
#include "cost_layer.h"
#include "lstm_layer.h"
#include "rnn_layer.h"
#include "rbm_layer.h"
// The maxpool argmax table is a private member of the reference class; the
// harness has to read it, so access control (only) is lifted for this header.
#define private public
#include "pooling_layer.h"
#undef private

using namespace nebula;

namespace {

// network_t has five pure virtuals that belong to the dataset drivers; the
// harness feeds tensors directly, so they are empty here.
struct probe_net_t : public network_t {
    void run(const std::string) {}
    void init_network(const std::string m_cfg) {
        config_t config;
        config.parse(m_cfg);
        num_layers = config.sections.size() - 1;
        layers.reserve(num_layers);
        for(size_t i = 0; i < config.sections.size(); i++) {
            section_config_t sc = config.sections[i];
            if(sc.name == "net") {
                sc.get_setting("num_threads", &num_threads);
                sc.get_setting("height", &input_height);
                sc.get_setting("width", &input_width);
                sc.get_setting("channels", &input_channel);
                sc.get_setting("batch", &batch_size);
                input_size = input_height * input_width * input_channel;
                // Recurrent nets: models/networks/recurrent.cc:129-139.
                if(sc.exists("time_steps")) {
                    sc.get_setting("input_size", &input_size);
                    sc.get_setting("time_steps", &time_step);
                    batch_size *= time_step;
                }
                continue;
            }
            layer_t *prev = layers.size() ? layers[layers.size() - 1] : NULL;
            layer_t *layer = NULL;
            if(sc.name == "convolutional") layer = new convolutional_layer_t(this, prev, CONVOLUTIONAL_LAYER);
            else if(sc.name == "connected") layer = new connected_layer_t(this, prev, CONNECTED_LAYER);
            else if(sc.name == "dropout") layer = new dropout_layer_t(this, prev, DROPOUT_LAYER);
            else if(sc.name == "maxpool") layer = new pooling_layer_t(this, prev, MAXPOOL_LAYER);
            else if(sc.name == "avgpool") layer = new pooling_layer_t(this, prev, AVGPOOL_LAYER);
            else if(sc.name == "shortcut") layer = new shortcut_layer_t(this, prev, SHORTCUT_LAYER);
            else if(sc.name == "softmax") { layer = new softmax_layer_t(this, prev, SOFTMAX_LAYER); output_layer = layer; }
            else if(sc.name == "cost") layer = new cost_layer_t(this, prev, COST_LAYER);
            else if(sc.name == "lstm") layer = new lstm_layer_t(this, prev, LSTM_LAYER);
            else if(sc.name == "rnn") layer = new rnn_layer_t(this, prev, RNN_LAYER);
            else if(sc.name == "rbm") layer = new rbm_layer_t(this, prev, RBM_LAYER);
            else { fprintf(stderr, "ref_harness: unknown section %s\n", sc.name.c_str()); exit(1); }
            if(!layers.size()) input_layer = layer;
            layer->init(sc);
            layers.push_back(layer);
        }
    }
    void load_data(const unsigned) {}
    void print_results() {}
    void init_data(const std::string) {
        input_data = new float[(size_t)input_size * batch_size]();
    }
    void load_weights(const std::string &path) { init_weight(path); }
    std::vector<layer_t*> &get_layers() { return layers; }
};

}  // namespace

extern "C" {

void *ref_net_create(const char *cfg_path) {
    probe_net_t *net = new probe_net_t();
    net->run_type = TEST_RUN;
    net->init_network(cfg_path);
    net->init_data("");
    return net;
}

unsigned ref_net_num_layers(void *h) { return (unsigned)((probe_net_t*)h)->get_layers().size(); }

// out[0..2] = batch_size (already multiplied by time_step for recurrent nets), time_step, input_size
void ref_net_dims(void *h, unsigned *out) {
    probe_net_t *net = (probe_net_t*)h;
    out[0] = net->batch_size; out[1] = net->time_step; out[2] = net->input_size;
}

// out[0..7] = layer_type, activation_type, output_height, output_width, output_channel, output_size, input_size, padding
void ref_net_layer_dims(void *h, unsigned i, unsigned *out) {
    layer_t *l = ((probe_net_t*)h)->get_layers()[i];
    out[0] = l->layer_type; out[1] = l->activation_type;
    out[2] = l->output_height; out[3] = l->output_width; out[4] = l->output_channel;
    out[5] = l->output_size; out[6] = l->input_size; out[7] = l->padding;
}

void ref_net_load_weights(void *h, const char *path) { ((probe_net_t*)h)->load_weights(path); }

// One forward pass in cfg order (models/networks/network.cc:57-63), cost layers skipped
// (they read labels, not part of inference).  For nets holding an LSTM only the first
// call on a fresh net is meaningful (state persists and sub-layer pointers are not rewound).
void ref_net_forward(void *h, const float *input) {
    probe_net_t *net = (probe_net_t*)h;
    memcpy(net->input_data, input, sizeof(float) * (size_t)net->input_size * net->batch_size);
    std::vector<layer_t*> &layers = net->get_layers();
    for(size_t i = 0; i < layers.size(); i++) {
        if(layers[i]->layer_type == COST_LAYER) continue;
        layers[i]->forward();
    }
}

const float *ref_net_output(void *h, unsigned i) { return ((probe_net_t*)h)->get_layers()[i]->output_data; }

const unsigned *ref_net_pool_index(void *h, unsigned i) {
    layer_t *l = ((probe_net_t*)h)->get_layers()[i];
    if(l->layer_type != MAXPOOL_LAYER) return NULL;
    return ((pooling_layer_t*)l)->index;
}

// ---- primitives (common/) -------------------------------------------------------------
void ref_im2col(float *im, unsigned c, unsigned hgt, unsigned wid, unsigned k, unsigned s, unsigned p,
                float *col, unsigned nthreads) { im2col(im, c, hgt, wid, k, s, p, col, nthreads); }

void ref_gemm(int ta, int tb, unsigned M, unsigned N, unsigned K, float alpha, float *A, unsigned lda,
              float *B, unsigned ldb, float beta, float *C, unsigned ldc, unsigned nthreads) {
    gemm<float>(ta, tb, M, N, K, alpha, A, lda, B, ldb, beta, C, ldc, nthreads);
}

void ref_forward_bias(unsigned nthreads, float *out, float *bias, unsigned channel, unsigned size, unsigned batch) {
    forward_bias(nthreads, out, bias, channel, size, batch);
}

void ref_batchnorm_normalize(unsigned nthreads, float *out, float *mean, float *var,
                             unsigned channel, unsigned size, unsigned batch) {
    batchnorm_normalize(nthreads, out, mean, var, channel, size, batch);
}

void ref_batchnorm_scale_down(unsigned nthreads, float *out, float *scale,
                              unsigned channel, unsigned size, unsigned batch) {
    batchnorm_scale_down(nthreads, out, scale, channel, size, batch);
}

void ref_shortcut(unsigned nthreads, unsigned iw, unsigned ih, unsigned ic, float *in,
                  unsigned ow, unsigned oh, unsigned oc, float *out, unsigned batch) {
    shortcut(nthreads, iw, ih, ic, in, ow, oh, oc, out, batch);
}

// id = activation_type_t value (common/def.h:62-78); returns -1 for ids layer_t::activate rejects.
int ref_activation(unsigned id, float *x, unsigned n) {
    switch(id) {
        case ELU_ACTIVATION: elu_activation(x, n); break;
        case HARDTAN_ACTIVATION: hardtan_activation(x, n); break;
        case LEAKY_ACTIVATION: leaky_activation(x, n); break;
        case LHTAN_ACTIVATION: lhtan_activation(x, n); break;
        case LINEAR_ACTIVATION: break;
        case LOGGY_ACTIVATION: loggy_activation(x, n); break;
        case LOGISTIC_ACTIVATION: logistic_activation(x, n); break;
        case PLSE_ACTIVATION: plse_activation(x, n); break;
        case RAMP_ACTIVATION: ramp_activation(x, n); break;
        case RELIE_ACTIVATION: relie_activation(x, n); break;
        case RELU_ACTIVATION: relu_activation(x, n); break;
        case STAIR_ACTIVATION: stair_activation(x, n); break;
        case TANH_ACTIVATION: tanh_activation(x, n); break;
        default: return -1;
    }
    return 0;
}

}  // extern "C"
