// HIPPipe: the device executor behind the scheduler.  One instance owns the
// weights, activation buffers and stream of one network on one GPU.
#pragma once
#include <cstddef>
#include <memory>
#include <mutex>
#include <string>
#include <vector>

#include "forward_pipe.h"

namespace lzhip {

// a rounded up to a multiple of b (Utils::ceilMultiple, reference src/Utils.cpp:208-215):
// what the pipe pads its channel and tile counts with.
inline size_t ceil_multiple(size_t a, size_t b) {
    if (b == 0 || a % b == 0) return a;
    return a + (b - a % b);
}


struct HeadWeightsHost {
    const float *bn_pol_mean, *bn_pol_scale, *ip_pol_w, *ip_pol_b;
    const float *bn_val_mean, *bn_val_scale, *ip1_val_w, *ip1_val_b, *ip2_val_w, *ip2_val_b;
};

class HIPPipe : public BatchExecutor {
public:
    ~HIPPipe() override = default;

    // ForwardPipe::push_weights with plain pointers (layouts: include/lzhip.h).
    virtual void push_weights(int n_layers, const float* const* U, const float* const* bn_mean,
                              const float* const* bn_scale, const float* pol_w,
                              const float* val_w) = 0;
    // Asynchronous forward on device-resident buffers (fp32 in/out), enqueued on one of
    // the pipe's lanes (a stream with its own working buffers); forwards on different
    // lanes run side by side.  sync() waits for every lane; stream() is lane 0's.
    virtual int lanes() const = 0;
    virtual void forward_device(int lane, int n, const float* d_in, float* d_pol,
                                float* d_val) = 0;
    // forward_device on lane 0's stream with the working buffers in a static device array
    // (no allocation anywhere on the way); small batches and nets only, see lzhip.h.
    virtual void forward_device_static(int n, const float* d_in, float* d_pol,
                                       float* d_val) = 0;
    virtual void sync() = 0;
    virtual void* stream() = 0;

    virtual void push_heads(const HeadWeightsHost& hw) = 0;
    virtual void evaluate_batch(int n, const float* in, float temperature, float* policy,
                                float* value, float* logits, float* pol, float* val) = 0;

    // `reps` evaluations of one batch, one after the other on lane 0, each of them the
    // copy of the planes from pinned host memory, the tower, the heads and the copy of
    // policy and value back to pinned host memory; returns the milliseconds between two
    // events recorded on that stream around all of them.
    virtual float timed_evaluations(int n, int reps, const float* in, float temperature,
                                    float* policy, float* value) = 0;

    virtual void debug_layer(int layer, int n, const float* act_in, const float* res, float* V,
                             float* M, float* Y) = 0;
    virtual void profile_forward(int n, const float* d_in, float* d_pol, float* d_val,
                                 float* ms, int* launches) = 0;
    virtual std::vector<float> act_scales() const = 0;
    virtual int filters() const = 0;
    virtual int precision() const = 0;
};

// Throws std::runtime_error when the device or runtime is unusable.
std::unique_ptr<HIPPipe> create_hip_pipe(int device, int precision, int max_batch, int filters);

}  // namespace lzhip
