/*
 * nebula_layers.h -- C entry points of libnebula_layers.so, the C++ layer framework
 * (nebula_amd/host: network_t / layer_t classes with the reference's surface) driven from C,
 * Python (ctypes) or any other FFI.  The classes themselves are the drop-in for
 * models/layers/ and models/networks/network.{h,cc}; these functions stand in for the 38-line
 * benchmark mains (benchmarks/<net>_<size>/main.cc:28-34: construct, init(), run()) and for the
 * dataset drivers' load_data()/print_results() (models/networks/convolutional.cc:263-483,
 * recurrent.cc:179-247), which feed tensors and read results.
 *
 * Every function returns 0 on success and a negative value on failure; nbl_net_last_error() then
 * holds the message the reference would have printed before exit(1).
 */
#ifndef NEBULA_LAYERS_H
#define NEBULA_LAYERS_H

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct nbl_net nbl_net;

/* cfg: path of a network.cfg (is_text = 0) or its contents (is_text = 1).  batch_override > 0 replaces
 * the [net] section's batch=.  weight_path may be NULL or "" (load later with nbl_net_load_weights).
 * device < 0 builds a dry-run network: cfg parsing, shape inference, .wgh reading/writing and the
 * queries below work without a GPU; anything that would compute fails with an error. */
int nbl_net_create(const char *cfg, int is_text, unsigned batch_override, int device,
                   const char *weight_path, nbl_net **out);
int nbl_net_destroy(nbl_net *net);
const char *nbl_net_last_error(void);
/* network_t::init_weight(path): the headerless fp32 .wgh stream, layer by layer in cfg order. */
int nbl_net_load_weights(nbl_net *net, const char *weight_path);
int nbl_net_store_weights(nbl_net *net, const char *weight_path);
/* The arrays of the .wgh stream in file order.  Each field is four unsigneds: layer index, kind
 * (0 bias, 1 weight matrix, 2 batchnorm scale, 3 rolling mean, 4 rolling variance), element count, fan-in.
 * Writes at most `capacity` fields to `fields` (may be NULL) and the total number to *num_fields. */
int nbl_net_weight_layout(nbl_net *net, unsigned *fields, size_t capacity, size_t *num_fields);
/* dims[0..5] = batch_size (rows, including time steps), time_step, input_size, input_h, input_w, input_c */
int nbl_net_dims(nbl_net *net, unsigned *dims);
int nbl_net_num_layers(nbl_net *net);
/* info[0..7] = layer_type, activation_type, output_channel, output_height, output_width, output_size,
 * input_size, padding */
int nbl_net_layer_info(nbl_net *net, int layer, unsigned *info);
/* per input row: 2*F*OH*OW*C*k*k for a convolutional layer, 2*I*O for a connected / rbm one, 2*(I+2*O)*O for an
 * rnn layer, 2*(I+H)*4H for an lstm layer, 0 otherwise */
int nbl_net_layer_flop(nbl_net *net, int layer, double *flop_per_row);
/* host -> device input, [batch_size][input_size] floats */
int nbl_net_set_input(nbl_net *net, const float *host, size_t count);
/* The image driver's load_data() (models/networks/convolutional.cc:384-412) with the preprocessing on the
 * device: `images` (= batch size) 8-bit interleaved images [height][width][channels] in decoded channel
 * order (B, G, R) are copied as bytes, resized to the network's input size if they differ (8-bit
 * INTER_LINEAR), scaled by 1/255 and stored as planes with planes 0 and 2 swapped. */
int nbl_net_set_input_images(nbl_net *net, const unsigned char *host, unsigned images, unsigned height, unsigned width);
/* recurrent_t::load_data() (models/networks/recurrent.cc:179-204) without the one-hot matrix: tokens[T*B]
 * (time-major; = batch_size entries) name the position of the 1.0 in each input row.  Needs an [lstm] or an
 * [rnn] as the first layer, which then gathers weight columns instead of multiplying.  nbl_net_set_input switches back. */
int nbl_net_set_input_tokens(nbl_net *net, const unsigned *host, size_t count);
/* recurrent_t::print_results(), test branch (recurrent.cc:239-247): after a forward, adds the output layer's
 * probabilities of the label tokens (one per output row) to the running sum and returns the driver's figure
 * exp(-log2(sum / rows seen)). */
int nbl_net_accumulate_perplexity(nbl_net *net, const unsigned *label_tokens, size_t count, float *perplexity);
/* convolutional_t::print_results(), test branch (models/networks/convolutional.cc:428-447): after a forward,
 * adds the number of rows whose label is among the output layer's k largest entries to a running count of
 * matches and returns that count (the reference's static `matches`).  labels: one class index per output row. */
int nbl_net_accumulate_topk(nbl_net *net, const unsigned *labels, size_t count, unsigned k, unsigned *matches);
/* network_t::forward(); asynchronous unless the net ends in a softmax (which copies to the host) */
int nbl_net_forward(nbl_net *net);
int nbl_net_sync(nbl_net *net);
/* forward with a HIP event between layers: ms[i] = duration of layer i (num_layers entries) */
int nbl_net_forward_timed(nbl_net *net, float *ms);
/* device -> host copy of layer's output ([batch_size][output_size]).  A convolution fused with the [shortcut] behind
 * it (fuse_shortcut=1) has no buffer of its own: its output is the shortcut's (the sum, activated). */
int nbl_net_layer_output(nbl_net *net, int layer, float *host, size_t count);
/* Whose values nbl_net_layer_output(layer) returns after a pass: *writer = layer itself for a layer with a tensor of
 * its own; the producing layer for a [dropout] or [cost] layer (they share its tensor); the [shortcut] behind it for a fused convolution; with shortcut_in_place=1 the last shortcut that wrote its
 * result over this layer's tensor (a ResNet stage then shares one tensor between its blocks and only the last block's
 * output survives the pass). */
int nbl_net_layer_output_writer(nbl_net *net, int layer, int *writer);
/* The max-pool argmax table the reference's forward keeps for its backward pass (pooling_layer.cc:132,140):
 * flat offsets into the layer's input tensor.  Kept only when the [net] section says pool_index=1 (a key the
 * reference ignores); inference never reads the table, so by default it is not written. */
int nbl_net_pool_index(nbl_net *net, int layer, unsigned *host, size_t count);
/* Convolutional layers: tile shape index and number of k slices (1 = unsplit) of the layer's most recent launch
 * (nbl_conv2d_plan_last_launch), and a way to pin both (variant < 0: from the launch table, or searched on first use; split: -1 likewise,
 * 0 never, 1 cost model, 2..8 that many slices) so that a run can be repeated with exactly the launches of another. */
int nbl_net_conv_last_launch(nbl_net *net, int layer, int *variant, int *slices);
int nbl_net_conv_pin_launch(nbl_net *net, int layer, int variant, int split);
/* Where the layer's most recent launch took its tile shape and k-split from: an nbl_launch_source value of
 * include/nebula_hip.h (2 = the launch table file, 3 = measured in this process, 1 = pinned, 4 = cost model). */
int nbl_net_conv_launch_source(nbl_net *net, int layer, int *source);
/* The launch-table key of a convolutional layer at the network's batch size, twelve numbers in the order of a table
 * line: C H W F size stride padding batch, then channels, height, width of the residual a fused shortcut adds and 1
 * when the result is written over it (four zeros without a fused shortcut).  Works on dry-run networks. */
int nbl_net_conv_problem(nbl_net *net, int layer, unsigned *key);
/* the softmax layer skips its device->host copy when enabled = 0 (throughput measurement) */
int nbl_net_softmax_copy(nbl_net *net, int enabled);
/* enabled = 1 (also the [net] key hip_graph=1, which the reference ignores): nbl_net_forward records the
 * launches of one pass into a HIP graph and replays it from then on: one launch on the host per pass instead
 * of one per kernel (a recurrent net launches a kernel per layer and time step).  The first pass of a
 * configuration runs eagerly (tile search, workspace growth), the second is recorded, later ones replay; a
 * pass then always ends with a wait for the stream.  Loading weights, switching between token and dense
 * input or toggling the softmax copy starts over.  The reference has no counterpart (its launches are eager).
 * nbl_net_graph_active: 1 while passes are replays of a recorded graph, 0 otherwise (also when recording was
 * not possible and the network stayed eager). */
int nbl_net_set_graph(nbl_net *net, int enabled);
/* enabled = 1 (also the [net] key carry_state=1, which the reference ignores): every [lstm] layer starts a pass
 * from the hidden and cell state its previous pass ended with (nbl_lstm_plan_carry_state), as the reference's
 * layers do between the batches of one token stream (lstm_layer.cu:15-140 never clears them); the default starts
 * every pass from zero.  Passes of a carrying network are never recorded into a HIP graph (what a pass reads
 * depends on the pass before it).  nbl_net_reset_state: the next pass starts from zero again (a new stream). */
int nbl_net_set_carry_state(nbl_net *net, int enabled);
int nbl_net_reset_state(nbl_net *net);
int nbl_net_graph_active(nbl_net *net);
/* the nbl_ctx* of the network (include/nebula_hip.h), e.g. for nbl_timer_start/stop */
void *nbl_net_ctx(nbl_net *net);

#ifdef __cplusplus
}
#endif
#endif
