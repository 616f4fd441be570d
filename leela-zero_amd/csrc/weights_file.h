// Reader of Leela Zero weights files (reference src/Network.cpp:225-405), with the
// preparation of Network::initialize (:540-576) applied: what comes back is what
// ForwardPipe::push_weights and the head arithmetic take.
#ifndef LZHIP_WEIGHTS_FILE_H
#define LZHIP_WEIGHTS_FILE_H

#include <string>
#include <vector>

namespace lzhip {

struct WeightsFile {
    int filters = 0, blocks = 0;
    bool value_head_not_stm = false;             // format 2
    std::vector<std::vector<float>> U;           // [layer]: [36][C_in][filters]
    std::vector<std::vector<float>> bn_mean;     // conv bias folded in
    std::vector<std::vector<float>> bn_scale;    // 1/sqrt(var + 1e-5)
    std::vector<float> conv_pol_w, conv_val_w;   // [2][filters], [filters]
    std::vector<float> bn_pol_mean, bn_pol_scale, ip_pol_w, ip_pol_b;
    std::vector<float> bn_val_mean, bn_val_scale, ip1_val_w, ip1_val_b, ip2_val_w, ip2_val_b;
};

// Plain or gzip-compressed, format 1 or 2.  Throws std::invalid_argument with the
// engine's own wording for a file it would refuse.
WeightsFile load_weights_file(const std::string& path);

}  // namespace lzhip
#endif
