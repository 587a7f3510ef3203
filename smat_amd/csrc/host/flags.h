// Minimal command-line flags in the style the reference binary is driven with
// (`hgemm -n_mult=32 -filename=a.mtx`, src/run_smat.sh:16-18): -name=value,
// --name=value, -name value; booleans also accept a bare -name.
#pragma once
#include <cstdlib>
#include <cstring>
#include <map>
#include <string>

class Flags {
public:
    Flags(int argc, char **argv)
    {
        for (int i = 1; i < argc; i++) {
            std::string a = argv[i];
            if (a.size() < 2 || a[0] != '-') { positional_ += a + " "; continue; }
            a = a.substr(a[1] == '-' ? 2 : 1);
            const size_t eq = a.find('=');
            if (eq != std::string::npos) values_[a.substr(0, eq)] = a.substr(eq + 1);
            else if (i + 1 < argc && argv[i + 1][0] != '-') values_[a] = argv[++i];
            else values_[a] = "true";
        }
    }
    bool has(const std::string &k) const { return values_.count(k) != 0; }
    std::string str(const std::string &k, const std::string &d) const { return has(k) ? values_.at(k) : d; }
    long num(const std::string &k, long d) const { return has(k) ? std::strtol(values_.at(k).c_str(), nullptr, 10) : d; }
    double real(const std::string &k, double d) const { return has(k) ? std::strtod(values_.at(k).c_str(), nullptr) : d; }
    bool flag(const std::string &k, bool d) const
    {
        if (!has(k)) return d;
        const std::string &v = values_.at(k);
        return !(v == "false" || v == "0" || v == "no");
    }

private:
    std::map<std::string, std::string> values_;
    std::string positional_;
};
