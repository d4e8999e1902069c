// Tuning cache: which row of the tile-config table a convolution runs on, measured once and kept in a JSON file.
//
// The counterpart of the reference's auto-tuner (kernel_selector/core/auto_tuner.cpp:27-112: cache file
// { "<compute units>": { "<hash of the kernel's parameters>": ["<implementation name>", <tune index>] } },
// kernel_selector/core/kernel_selector.cpp GetAutoTuneBestKernel, the build option cldnn_build_option_tuning_config
// with the modes tuning_use_cache / tuning_tune_and_cache).  The file has the same shape here: the key is a readable
// signature of the convolution descriptor, the value the tile row's name and index; index -1 = the built-in table's
// own choice was the fastest.  An entry whose name no longer matches the row of that index is ignored.
#include <cctype>
#include <cstdio>
#include <fstream>
#include <sstream>

#include "impl.h"

namespace host {

namespace {

struct parser {
    const std::string& s;
    size_t i = 0;
    void skip()
    {
        while (i < s.size() && std::isspace((unsigned char)s[i])) ++i;
    }
    bool eat(char c)
    {
        skip();
        if (i < s.size() && s[i] == c) {
            ++i;
            return true;
        }
        return false;
    }
    void need(char c)
    {
        if (!eat(c)) throw api_error(CLDNN_ERROR, std::string("tuning cache: expected '") + c + "' at offset " + std::to_string(i));
    }
    std::string str()
    {
        need('"');
        std::string r;
        while (i < s.size() && s[i] != '"') {
            if (s[i] == '\\' && i + 1 < s.size()) ++i;
            r += s[i++];
        }
        need('"');
        return r;
    }
    int num()
    {
        skip();
        size_t j = i;
        if (j < s.size() && (s[j] == '-' || s[j] == '+')) ++j;
        while (j < s.size() && std::isdigit((unsigned char)s[j])) ++j;
        if (j == i) throw api_error(CLDNN_ERROR, "tuning cache: number expected at offset " + std::to_string(i));
        const int v = std::stoi(s.substr(i, j - i));
        i = j;
        return v;
    }
};

std::string quoted(const std::string& s)
{
    std::string r = "\"";
    for (char c : s) {
        if (c == '"' || c == '\\') r += '\\';
        r += c;
    }
    return r + "\"";
}

}  // namespace

void tuning_cache::load(const std::string& file, int tuning_mode)
{
    path = file, mode = tuning_mode, entries.clear(), dirty = false;
    std::ifstream f(path);
    if (!f.good()) {
        // reference auto_tuner.cpp:40-46
        if (mode == cldnn_tuning_use_cache)
            throw api_error(CLDNN_ERROR, "Tuning file: " + path + " could not be read! Must provide a valid cache file in USE_CACHE mode.");
        return;
    }
    std::stringstream buf;
    buf << f.rdbuf();
    const std::string text = buf.str();
    parser p{text};
    p.skip();
    if (p.i == text.size()) return;  // an empty file is an empty cache
    p.need('{');
    if (p.eat('}')) return;
    do {
        const std::string units = p.str();
        p.need(':');
        p.need('{');
        if (!p.eat('}')) {
            do {
                const std::string key = p.str();
                p.need(':');
                p.need('[');
                const std::string name = p.str();
                p.need(',');
                const int index = p.num();
                p.need(']');
                entries[units][key] = {name, index};
            } while (p.eat(','));
            p.need('}');
        }
    } while (p.eat(','));
    p.need('}');
}

bool tuning_cache::find(uint32_t compute_units, const std::string& key, std::string* name, int* index) const
{
    auto u = entries.find(std::to_string(compute_units));
    if (u == entries.end()) return false;
    auto e = u->second.find(key);
    if (e == u->second.end()) return false;
    *name = e->second.first, *index = e->second.second;
    return true;
}

void tuning_cache::store(uint32_t compute_units, const std::string& key, const std::string& name, int index)
{
    entries[std::to_string(compute_units)][key] = {name, index};
    dirty = true;
}

void tuning_cache::save()
{
    if (!dirty) return;
    std::ofstream f(path, std::ofstream::out | std::ofstream::trunc);
    if (!f.good()) throw api_error(CLDNN_ERROR, "Tuning file: " + path + " could not be written.");
    f << "{\n";
    bool first_units = true;
    for (auto& u : entries) {
        f << (first_units ? "" : ",\n") << "  " << quoted(u.first) << ": {\n";
        first_units = false;
        bool first = true;
        for (auto& e : u.second) {
            f << (first ? "" : ",\n") << "    " << quoted(e.first) << ": [" << quoted(e.second.first) << ", " << e.second.second << "]";
            first = false;
        }
        f << "\n  }";
    }
    f << "\n}\n";
    dirty = false;
}

// Everything of the descriptor that decides which kernel runs and how long it takes; the values of the factors are not
// part of it (the reference hashes the kernel parameters the same way, kernel_selector/core/kernel_selector_params.cpp
// to_string()).
std::string conv_signature(const cldnn_hip_conv_desc& d)
{
    auto tensor = [](const cldnn_hip_tensor& t) {
        std::ostringstream o;
        o << "t" << t.dtype << "f" << t.format << ":" << t.b << "x" << t.f << "x" << t.y << "x" << t.x << "+" << t.pad_lo_y << "," << t.pad_lo_x << ","
          << t.pad_hi_y << "," << t.pad_hi_x;
        return o.str();
    };
    std::ostringstream o;
    o << "conv;in=" << tensor(d.input) << ";out=" << tensor(d.output) << ";w=" << d.weights_dtype << ":" << d.ofm << "x" << d.ifm << "x" << d.fy << "x"
      << d.fx << ";s=" << d.stride_y << "," << d.stride_x << ";d=" << d.dilation_y << "," << d.dilation_x << ";p=" << d.pad_y << "," << d.pad_x << "+"
      << d.pad_end_delta_y << "," << d.pad_end_delta_x << ";g=" << d.groups << ";bias=" << d.bias_dtype << ";q=" << d.has_wqf << d.has_calib
      << ";act=" << d.activation << ";fc=" << d.fully_connected << ";even=" << d.round_to_even;
    if (d.sibling_split) o << ";pair=" << d.sibling_split << "," << d.sibling_activation;  // two convolutions of one input in one launch
    if (d.fused)
        o << ";eltw=" << (d.second_input_in_output ? std::string("inplace") : tensor(d.eltw)) << ";es=" << d.eltw_stride_y << "," << d.eltw_stride_x
          << ";eact=" << d.eltw_activation << ";ecal=" << d.has_eltw_calib << ";scale1=" << (d.non_conv_scale == 1.0f) << ";csat=" << d.conv_saturate;
    return o.str();
}

}  // namespace host
