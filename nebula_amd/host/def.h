// Enumerations and their cfg spellings.  The numeric values and the strings are part of the
// network.cfg / C-ABI contract of the reference (common/def.h:14-115): activation ids cross the
// C ABI as integers and the names are what a cfg file says after `activation=`.
#ifndef NEBULA_HOST_DEF_H
#define NEBULA_HOST_DEF_H

#include <string>

namespace nebula {

enum run_type_t { UNDEFINED_RUN = 0, TEST_RUN, TRAIN_RUN, NUM_RUN_TYPES };

enum layer_type_t {
    UNDEFINED_LAYER = 0, CONNECTED_LAYER, CONVOLUTIONAL_LAYER, COST_LAYER, DROPOUT_LAYER, AVGPOOL_LAYER,
    MAXPOOL_LAYER, SHORTCUT_LAYER, SOFTMAX_LAYER, RNN_LAYER, LSTM_LAYER, RBM_LAYER, NUM_LAYER_TYPES
};

enum activation_type_t {
    UNDEFINED_ACTIVATION = 0, ELU_ACTIVATION, HARDTAN_ACTIVATION, LEAKY_ACTIVATION, LHTAN_ACTIVATION,
    LINEAR_ACTIVATION, LOGGY_ACTIVATION, LOGISTIC_ACTIVATION, PLSE_ACTIVATION, RAMP_ACTIVATION,
    RELIE_ACTIVATION, RELU_ACTIVATION, STAIR_ACTIVATION, TANH_ACTIVATION, NUM_ACTIVATION_TYPES
};

extern const char *const run_type_str[NUM_RUN_TYPES + 1];
extern const char *const layer_type_str[NUM_LAYER_TYPES + 1];
extern const char *const activation_type_str[NUM_ACTIVATION_TYPES + 1];

// Index of `name` in a NULL-free table of `count + 1` strings; `count` when absent (the reference's
// get_type macro, common/def.h:120-121, yields the end position for an unknown string).
unsigned lookup_type(const char *const *table, unsigned count, const std::string &name);

}  // namespace nebula
#endif
