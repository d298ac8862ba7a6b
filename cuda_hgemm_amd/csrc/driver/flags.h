// Minimal "-name=value" command-line flags (the reference uses gflags, src/main.cu:35-45,
// which this image does not ship).  Accepts -name=value, --name=value, -name value and,
// for booleans, a bare -name.
#pragma once

#include <stdlib.h>
#include <string.h>

#include <map>
#include <string>
#include <vector>

#include "../common.h"

namespace hgemm {

class Flags {
public:
    void define(const std::string &name, const std::string &default_value, const std::string &help) {
        m_values[name] = default_value;
        m_help.push_back(name + " (default " + default_value + "): " + help);
    }

    void parse(int argc, char **argv) {
        for (int i = 1; i < argc; ++i) {
            std::string arg = argv[i];
            if (arg == "-help" || arg == "--help" || arg == "-h") {
                for (const auto &line : m_help) fprintf(stderr, "  -%s\n", line.c_str());
                exit(EXIT_SUCCESS);
            }
            HGEMM_CHECK_MSG(arg.size() > 1 && arg[0] == '-', "unexpected argument '%s'", arg.c_str());
            arg = arg.substr(arg[1] == '-' ? 2 : 1);
            std::string name = arg, value;
            const size_t eq = arg.find('=');
            if (eq != std::string::npos) {
                name = arg.substr(0, eq);
                value = arg.substr(eq + 1);
            } else if (i + 1 < argc && argv[i + 1][0] != '-') {
                value = argv[++i];
            } else {
                value = "true";
            }
            HGEMM_CHECK_MSG(m_values.count(name) == 1, "unknown flag -%s", name.c_str());
            m_values[name] = value;
        }
    }

    const std::string &str(const std::string &name) const {
        auto it = m_values.find(name);
        HGEMM_CHECK_MSG(it != m_values.end(), "flag -%s was never defined", name.c_str());
        return it->second;
    }
    size_t u64(const std::string &name) const {
        const std::string &v = str(name);
        char *end = nullptr;
        const unsigned long long x = strtoull(v.c_str(), &end, 10);
        HGEMM_CHECK_MSG(end && *end == '\0' && !v.empty() && v[0] != '-', "flag -%s: '%s' is not a count",
                        name.c_str(), v.c_str());
        return (size_t)x;
    }
    bool boolean(const std::string &name) const {
        const std::string &v = str(name);
        if (v == "true" || v == "1" || v == "yes") return true;
        if (v == "false" || v == "0" || v == "no") return false;
        HGEMM_CHECK_MSG(false, "flag -%s: '%s' is not a boolean", name.c_str(), v.c_str());
        return false;
    }

private:
    std::map<std::string, std::string> m_values;
    std::vector<std::string> m_help;
};

}  // namespace hgemm
