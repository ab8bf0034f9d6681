#include "config.h"

#include <algorithm>
#include <cctype>
#include <fstream>
#include <stdexcept>

#include "def.h"

namespace nebula {

const char *const run_type_str[NUM_RUN_TYPES + 1] = { "undefined_run", "test", "train", "num_run_types" };

const char *const layer_type_str[NUM_LAYER_TYPES + 1] = {
    "undefined_layer", "connected_layer", "convolutional_layer", "cost_layer", "dropout_layer", "avgpool_layer",
    "maxpool_layer", "shortcut_layer", "softmax_layer", "rnn_layer", "lstm_layer", "rbm_layer", "num_layer_types" };

const char *const activation_type_str[NUM_ACTIVATION_TYPES + 1] = {
    "undefined_activation", "elu", "hardtan", "leaky", "lhtan", "linear", "loggy", "logistic", "plse", "ramp",
    "relie", "relu", "stair", "tanh", "num_activation_types" };

unsigned lookup_type(const char *const *table, unsigned count, const std::string &name) {
    // the reference searches the whole table including the trailing "num_*" entry
    for(unsigned i = 0; i <= count; i++) if(name == table[i]) return i;
    return count + 1;
}

std::string &lowercase(std::string &s) {
    std::transform(s.begin(), s.end(), s.begin(), [](unsigned char c) { return (char)std::tolower(c); });
    return s;
}

section_config_t::section_config_t(std::string m_name) : name(m_name) {}

void section_config_t::add_setting(std::string m_key, std::string m_value) {
    settings.insert(std::make_pair(lowercase(m_key), lowercase(m_value)));   // insert: first one wins
}

const std::string *section_config_t::find(std::string &m_key) const {
    const std::map<std::string, std::string>::const_iterator at = settings.find(lowercase(m_key));
    return at == settings.end() ? NULL : &at->second;
}

bool section_config_t::exists(std::string m_key) { return find(m_key) != NULL; }

void config_t::parse(std::string m_config_name) {
    std::ifstream in(m_config_name.c_str());
    if(!in.is_open()) throw std::runtime_error("Error: failed to open " + m_config_name);
    parse_stream(in);
}

void config_t::parse_stream(std::istream &in) {
    std::string line;
    while(std::getline(in, line)) {
        line.erase(std::remove(line.begin(), line.end(), ' '), line.end());
        if(line.empty() || line[0] == '#') continue;
        if(line[0] == '[') {
            sections.push_back(section_config_t(line.substr(1, line.size() - 2)));
            continue;
        }
        const size_t eq = line.find('=');
        if(eq == std::string::npos) throw std::runtime_error("Error: invalid config\n" + line);
        if(sections.empty()) throw std::runtime_error("Error: invalid config (setting before any section)\n" + line);
        sections.back().add_setting(line.substr(0, eq), line.substr(eq + 1));
    }
}

}  // namespace nebula
