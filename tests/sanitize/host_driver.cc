// Sanitizer driver for the host-side layer framework (nebula_amd/host/*.cc), built by tests/test_sanitizers.py with
// -fsanitize=address,undefined.  Dry-run networks only (device < 0): cfg parsing, shape inference, the .wgh
// reader/writer and the error paths, i.e. all host logic that runs without a GPU.
//
//   host_driver <network.cfg> <weights.wgh> <scratch.wgh>
//
// Exit code 0 and "ok <layers> <floats>" on stdout when every step behaved; anything else is a failure.
#include <cstdio>
#include <cstring>
#include <fstream>
#include <sstream>
#include <stdexcept>
#include <string>
#include <vector>

#include "nebula_layers.h"

static int fail(const char *what) {
    std::fprintf(stderr, "host_driver: %s: %s\n", what, nbl_net_last_error());
    return 1;
}

int main(int argc, char **argv) {
    if(argc != 4) { std::fprintf(stderr, "usage: host_driver cfg wgh scratch\n"); return 2; }
    nbl_net *net = NULL;
    // from a file path, weights given at creation
    if(nbl_net_create(argv[1], 0, 0, -1, argv[2], &net) != 0) return fail("create(path, weights)");
    const int layers = nbl_net_num_layers(net);
    unsigned dims[6];
    if(nbl_net_dims(net, dims) != 0) return fail("dims");
    size_t nf = 0;
    if(nbl_net_weight_layout(net, NULL, 0, &nf) != 0) return fail("weight_layout(count)");
    std::vector<unsigned> fields(4 * nf + 4);
    if(nbl_net_weight_layout(net, fields.data(), nf, &nf) != 0) return fail("weight_layout");
    size_t floats = 0;
    for(size_t i = 0; i < nf; i++) floats += fields[4 * i + 2];
    for(int i = 0; i < layers; i++) {
        unsigned info[8]; double flop = 0.0;
        if(nbl_net_layer_info(net, i, info) != 0 || nbl_net_layer_flop(net, i, &flop) != 0) return fail("layer_info");
    }
    unsigned info[8];
    if(nbl_net_layer_info(net, layers, info) == 0) { std::fprintf(stderr, "layer index past the end accepted\n"); return 1; }
    if(nbl_net_layer_info(net, -1, info) == 0) { std::fprintf(stderr, "negative layer index accepted\n"); return 1; }
    // round trip of the weight stream
    if(nbl_net_store_weights(net, argv[3]) != 0) return fail("store_weights");
    {
        std::ifstream a(argv[2], std::ios::binary), b(argv[3], std::ios::binary);
        std::stringstream sa, sb; sa << a.rdbuf(); sb << b.rdbuf();
        if(sa.str().size() != floats * sizeof(float) || sa.str() != sb.str()) { std::fprintf(stderr, "weight round trip differs\n"); return 1; }
    }
    // compute entry points must refuse a network without a device, not crash
    std::vector<float> x((size_t)dims[0] * dims[2], 0.5f);
    if(nbl_net_set_input(net, x.data(), x.size()) == 0 || nbl_net_forward(net) == 0) {
        std::fprintf(stderr, "dry-run network accepted a forward pass\n"); return 1;
    }
    // a truncated weight file is reported
    {
        std::ofstream t(argv[3], std::ios::binary | std::ios::trunc);
        if(floats > 1) { std::vector<float> half(floats / 2, 1.0f); t.write((const char*)half.data(), (std::streamsize)(half.size() * sizeof(float))); }
    }
    if(floats > 1 && nbl_net_load_weights(net, argv[3]) == 0) { std::fprintf(stderr, "short weight file accepted\n"); return 1; }
    if(nbl_net_load_weights(net, "/nonexistent/weights.wgh") == 0 && floats) { std::fprintf(stderr, "missing weight file accepted\n"); return 1; }
    if(nbl_net_destroy(net) != 0) return fail("destroy");

    // the same network from cfg text, with a batch override, weights loaded afterwards
    std::ifstream cf(argv[1]);
    std::stringstream text; text << cf.rdbuf();
    if(nbl_net_create(text.str().c_str(), 1, 3, -1, NULL, &net) != 0) return fail("create(text)");
    if(nbl_net_load_weights(net, argv[2]) != 0) return fail("load_weights");
    if(nbl_net_destroy(net) != 0) return fail("destroy");

    // malformed configurations are errors, not crashes
    const char *bad[] = {
        "", "[convolutional]\nfilters=2\n", "[net]\nbatch=1\nheight\n", "[net]\nbatch=1\nheight=4\nwidth=4\nchannels=1\n[bogus]\nx=1\n",
        "[net]\nbatch=1\nheight=4\nwidth=4\nchannels=1\n[convolutional]\nfilters=2\nsize=9\nactivation=relu\n",
        "[net]\nbatch=1\nheight=4\nwidth=4\nchannels=1\n[convolutional]\nfilters=2\nsize=3\nactivation=swish\n",
        "[net]\nbatch=1\nheight=4\nwidth=4\nchannels=1\n[shortcut]\nhops=3\nactivation=linear\n",
        "[net]\nbatch=3\ninput_size=4\ntime_steps=0\n[lstm]\noutput=4\nactivation=linear\n",
        "[net]\nbatch=0\nheight=4\nwidth=4\nchannels=1\n[softmax]\n",
    };
    for(size_t i = 0; i < sizeof(bad) / sizeof(bad[0]); i++) {
        net = NULL;
        if(nbl_net_create(bad[i], 1, 0, -1, NULL, &net) == 0) { std::fprintf(stderr, "bad cfg %zu accepted\n", i); return 1; }
    }
    std::printf("ok %d %zu\n", layers, floats);
    return 0;
}
