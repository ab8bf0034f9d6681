// network.cfg reader with the reference's exact quirks (common/config.cc:22-24,44-75):
// spaces (only spaces) are removed, lines starting with '#' are comments, "[name]" opens a section,
// "key=value" is stored lower-cased on both sides, the first occurrence of a key wins, unknown
// keys are kept and ignored, and values are converted with operator>> (so bools are 0/1).
#ifndef NEBULA_HOST_CONFIG_H
#define NEBULA_HOST_CONFIG_H

#include <istream>
#include <map>
#include <sstream>
#include <string>
#include <vector>

namespace nebula {

std::string &lowercase(std::string &s);

// One "[name]" block of a cfg file: its key=value lines.
class section_config_t {
public:
    std::string name;

    explicit section_config_t(std::string m_name);
    void add_setting(std::string m_key, std::string m_value);
    bool exists(std::string m_key);
    // *m_var = the value of m_key read with operator>>; false (and *m_var untouched) when the key is absent
    template <typename T>
    bool get_setting(std::string m_key, T *m_var) {
        const std::string *text = find(m_key);
        if(!text) return false;
        std::istringstream in(*text);
        in >> *m_var;
        return true;
    }

private:
    const std::string *find(std::string &m_key) const;     // lower-cases m_key first, as every access does
    std::map<std::string, std::string> settings;
};

class config_t {
public:
    // Throws std::runtime_error where the reference prints and exits.
    void parse(std::string m_config_name);          // from a file
    void parse_stream(std::istream &in);            // from any stream (tests, embedded cfgs)
    std::vector<section_config_t> sections;
};

}  // namespace nebula
#endif
