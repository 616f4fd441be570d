// Engine-side adapter over the C ABI of lz-hip (include/lzhip.h): a ForwardPipe that a
// Leela Zero build can construct where it constructs OpenCLScheduler today (reference
// src/Network.cpp:578-597), without sharing any C++ class layout with the library.
// Compiles inside the engine tree: "ForwardPipe.h" and "Network.h" are the engine's own
// (reference src/ForwardPipe.h:38-71, src/Network.h:66-67).
#ifndef HIPPIPEADAPTER_H_INCLUDED
#define HIPPIPEADAPTER_H_INCLUDED

#include <memory>
#include <stdexcept>
#include <vector>

#include "ForwardPipe.h"
#include "Network.h"  // NetworkHaltException
#include "lzhip.h"

class HIPPipeAdapter : public ForwardPipe {
public:
    HIPPipeAdapter(int precision, int max_batch, int device)
        : m_precision(precision), m_max_batch(max_batch), m_device(device) {}
    ~HIPPipeAdapter() override { lzhip_destroy(m_handle); }

    void initialize(const int channels) override {
        if (lzhip_create(channels, m_precision, m_max_batch, m_device, &m_handle) != LZHIP_OK)
            throw std::runtime_error(lzhip_last_error());
    }
    void push_weights(unsigned int /*filter_size*/, unsigned int /*channels*/,
                      unsigned int /*outputs*/,
                      std::shared_ptr<const ForwardPipeWeights> weights) override {
        const size_t n = weights->m_conv_weights.size();
        std::vector<const float*> U(n), mean(n), scale(n);
        for (size_t l = 0; l < n; l++) {
            U[l] = weights->m_conv_weights[l].data();
            mean[l] = weights->m_batchnorm_means[l].data();
            scale[l] = weights->m_batchnorm_stddevs[l].data();
        }
        if (lzhip_push_weights(m_handle, static_cast<int>(n), U.data(), mean.data(), scale.data(),
                               weights->m_conv_pol_w.data(),
                               weights->m_conv_val_w.data()) != LZHIP_OK)
            throw std::runtime_error(lzhip_last_error());
    }
    void forward(const std::vector<float>& input, std::vector<float>& output_pol,
                 std::vector<float>& output_val) override {
        const int rc = lzhip_forward(m_handle, input.data(), output_pol.data(), output_val.data());
        if (rc == LZHIP_EHALT) throw NetworkHaltException();
        if (rc != LZHIP_OK) throw std::runtime_error(lzhip_last_error());
    }
    void drain() override { lzhip_drain(m_handle); }
    void resume() override { lzhip_resume(m_handle); }

private:
    lzhip_handle* m_handle = nullptr;
    int m_precision, m_max_batch, m_device;
};

#endif
