// cli_options.h -- the small command-line reader shared by the drivers that mirror the reference's
// boost::program_options front ends: "--name value", "--name=value", multi-token values, "-T" for
// --num_threads, required options, defaults, and the same wording for the usual mistakes.
#pragma once
#include <sys/stat.h>

#include <cctype>
#include <cstddef>
#include <iostream>
#include <map>
#include <string>
#include <vector>

namespace cli {

struct Option {
    const char* name;
    bool required;
    bool multitoken;
    const char* fallback;  // nullptr: no default
    const char* help;
};

using Values = std::map<std::string, std::vector<std::string>>;

inline void usage(const Option* options, size_t count) {
    std::cout << "Arguments:\n  -h [ --help ]  Print information on arguments\n";
    for (size_t i = 0; i < count; ++i) {
        const Option& o = options[i];
        std::cout << "  --" << o.name << (o.fallback ? std::string(" arg (=") + o.fallback + ")" : " arg") << "  "
                  << o.help << "\n";
    }
}

inline const Option* find_option(const Option* options, size_t count, const std::string& name) {
    for (size_t i = 0; i < count; ++i)
        if (name == options[i].name) return options + i;
    return nullptr;
}

// returns false (after printing what is wrong) on a malformed command line
inline bool parse(const Option* options, size_t count, int argc, char** argv, Values& out, bool* help) {
    *help = false;
    for (int i = 1; i < argc; ++i) {
        std::string a = argv[i];
        if (a == "-h" || a == "--help") {
            *help = true;
            return true;
        }
        std::string name, value;
        bool has_value = false;
        if (a == "-T") {
            name = "num_threads";
        } else if (a.rfind("--", 0) == 0) {
            const size_t eq = a.find('=');
            name = a.substr(2, eq == std::string::npos ? std::string::npos : eq - 2);
            if (eq != std::string::npos) value = a.substr(eq + 1), has_value = true;
        } else {
            std::cerr << "too many positional options have been specified on the command line\n";
            return false;
        }
        const Option* o = find_option(options, count, name);
        if (!o) {
            std::cerr << "unrecognised option '" << a << "'\n";
            return false;
        }
        std::vector<std::string>& vals = out[name];
        if (has_value) {
            vals.push_back(value);
        } else if (o->multitoken) {
            while (i + 1 < argc && !(argv[i + 1][0] == '-' && !std::isdigit((unsigned char)argv[i + 1][1])))
                vals.push_back(argv[++i]);
            if (vals.empty()) {
                std::cerr << "the required argument for option '--" << name << "' is missing\n";
                return false;
            }
        } else {
            if (i + 1 >= argc) {
                std::cerr << "the required argument for option '--" << name << "' is missing\n";
                return false;
            }
            vals.assign(1, argv[++i]);
        }
    }
    for (size_t i = 0; i < count; ++i) {
        const Option& o = options[i];
        if (out.count(o.name)) continue;
        if (o.required) {
            std::cerr << "the option '--" << o.name << "' is required but missing\n";
            return false;
        }
        if (o.fallback) out[o.name].assign(1, o.fallback);
    }
    return true;
}

inline void make_dirs(const std::string& path) {
    for (size_t p = 1; p <= path.size(); ++p)
        if (p == path.size() || path[p] == '/') mkdir(path.substr(0, p).c_str(), 0755);
}

}  // namespace cli
