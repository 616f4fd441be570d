// Leela Zero weights files: the text format the engine reads in
// Network::load_network_file / load_v1_network (reference src/Network.cpp:225-405) and the
// preparation Network::initialize applies before handing the weights to the pipe
// (:540-576): Winograd transform of the 3x3 filters, 1/sqrt(var + eps), conv biases folded
// into the batch-norm means.
#include "weights_file.h"

#include <zlib.h>

#include <cstdlib>
#include <cstring>
#include <stdexcept>

#include "lzhip.h"

namespace lzhip {

namespace {

// gzopen reads plain files as they are (reference src/Network.cpp:353-375).
std::string read_all(const std::string& path) {
    gzFile f = gzopen(path.c_str(), "rb");
    if (!f) throw std::invalid_argument("Could not open weights file: " + path);
    std::string buf;
    std::vector<char> chunk(64 * 1024);
    for (;;) {
        const int n = gzread(f, chunk.data(), (unsigned)chunk.size());
        if (n == 0) break;
        if (n < 0) {
            gzclose(f);
            throw std::invalid_argument("Failed to decompress or read: " + path);
        }
        buf.append(chunk.data(), (size_t)n);
    }
    gzclose(f);
    return buf;
}

std::vector<std::string> split_lines(const std::string& text) {
    std::vector<std::string> lines;
    size_t pos = 0;
    while (pos < text.size()) {
        size_t nl = text.find('\n', pos);
        if (nl == std::string::npos) nl = text.size();
        lines.emplace_back(text, pos, nl - pos);
        pos = nl + 1;
    }
    return lines;
}

// Whitespace-separated floats; false when anything else is on the line.
bool parse_floats(const std::string& line, std::vector<float>& out) {
    out.clear();
    const char* p = line.c_str();
    const char* end = p + line.size();
    for (;;) {
        while (p < end && (*p == ' ' || *p == '\t' || *p == '\r')) p++;
        if (p >= end) return true;
        char* q = nullptr;
        const float v = std::strtof(p, &q);
        if (q == p) return false;
        out.push_back(v);
        p = q;
    }
}

void bn_var(std::vector<float>& w) { lzhip_process_bn_var(w.data(), (int)w.size()); }

void need(bool ok, const char* what) {
    if (!ok) throw std::invalid_argument(what);
}

}  // namespace

WeightsFile load_weights_file(const std::string& path) {
    const std::string text = read_all(path);
    std::vector<std::string> lines = split_lines(text);
    // First line: the format version (reference src/Network.cpp:378-401).
    int version = -1;
    if (!lines.empty()) {
        char* q = nullptr;
        const long v = std::strtol(lines[0].c_str(), &q, 10);
        if (q != lines[0].c_str()) version = (int)v;
    }
    need(version == 1 || version == 2, "Weights file is the wrong version.");

    WeightsFile wf;
    wf.value_head_not_stm = version == 2;
    // 1 format id, 1 input layer (4 lines), 14 lines of heads; the rest are residual
    // blocks of 8 lines each (reference src/Network.cpp:250-258).
    const long total = (long)lines.size();
    const long residual_lines = total - (1 + 4 + 14);
    need(residual_lines >= 0 && residual_lines % 8 == 0,
         "Inconsistent number of weights in the file.");
    wf.blocks = (int)(residual_lines / 8);
    const int n_layers = 1 + 2 * wf.blocks;

    std::vector<std::vector<float>> rows((size_t)total - 1);
    for (long i = 1; i < total; i++)
        if (!parse_floats(lines[(size_t)i], rows[(size_t)i - 1])) {
            throw std::invalid_argument("Failed to parse weight file. Error on line " +
                                        std::to_string(i + 1) + ".");
        }
    // The second parameter line holds the biases of the input convolution: one per filter.
    const int F = (int)rows[1].size();
    need(F >= 1, "Inconsistent number of weights in the file.");
    wf.filters = F;

    wf.U.resize((size_t)n_layers);
    wf.bn_mean.resize((size_t)n_layers);
    wf.bn_scale.resize((size_t)n_layers);
    for (int l = 0; l < n_layers; l++) {
        const int C = l == 0 ? LZHIP_INPUT_CHANNELS : F;
        std::vector<float>& w = rows[(size_t)l * 4 + 0];
        std::vector<float>& b = rows[(size_t)l * 4 + 1];
        std::vector<float>& mean = rows[(size_t)l * 4 + 2];
        std::vector<float>& var = rows[(size_t)l * 4 + 3];
        need(w.size() == (size_t)F * C * 9 && b.size() == (size_t)F && mean.size() == (size_t)F &&
                 var.size() == (size_t)F,
             "Inconsistent number of weights in the file.");
        wf.U[(size_t)l].resize((size_t)36 * C * F);
        lzhip_winograd_transform_f(w.data(), F, C, wf.U[(size_t)l].data());
        for (int k = 0; k < F; k++) mean[(size_t)k] -= b[(size_t)k];   // bias into the mean
        bn_var(var);
        wf.bn_mean[(size_t)l] = std::move(mean);
        wf.bn_scale[(size_t)l] = std::move(var);
    }
    std::vector<float>* hd = &rows[(size_t)n_layers * 4];
    need(hd[0].size() == (size_t)2 * F && hd[1].size() == 2 && hd[2].size() == 2 &&
             hd[3].size() == 2 && hd[6].size() == (size_t)F && hd[7].size() == 1 &&
             hd[8].size() == 1 && hd[9].size() == 1,
         "Inconsistent number of weights in the file.");
    need(hd[4].size() == (size_t)LZHIP_MOVES * 2 * LZHIP_NPTS,
         "The weights file is not for 19x19 boards.");
    need(hd[5].size() == (size_t)LZHIP_MOVES &&
             hd[10].size() == (size_t)LZHIP_VALUE_LAYER * LZHIP_NPTS &&
             hd[11].size() == (size_t)LZHIP_VALUE_LAYER &&
             hd[12].size() == (size_t)LZHIP_VALUE_LAYER && hd[13].size() == 1,
         "Inconsistent number of weights in the file.");
    wf.conv_pol_w = hd[0];
    wf.bn_pol_mean = hd[2];
    for (int i = 0; i < 2; i++) wf.bn_pol_mean[(size_t)i] -= hd[1][(size_t)i];
    wf.bn_pol_scale = hd[3];
    bn_var(wf.bn_pol_scale);
    wf.ip_pol_w = std::move(hd[4]);
    wf.ip_pol_b = std::move(hd[5]);
    wf.conv_val_w = hd[6];
    wf.bn_val_mean = hd[8];
    wf.bn_val_mean[0] -= hd[7][0];
    wf.bn_val_scale = hd[9];
    bn_var(wf.bn_val_scale);
    wf.ip1_val_w = std::move(hd[10]);
    wf.ip1_val_b = std::move(hd[11]);
    wf.ip2_val_w = std::move(hd[12]);
    wf.ip2_val_b = std::move(hd[13]);
    return wf;
}

}  // namespace lzhip
