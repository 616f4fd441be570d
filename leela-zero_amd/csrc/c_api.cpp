// extern "C" surface declared in include/lzhip.h.  Every function converts
// C++ exceptions into return codes; the message of the last failure is kept
// per calling thread.
#include <cmath>
#include <cstring>
#include <memory>
#include <stdexcept>
#include <string>

#include "forward_pipe.h"
#include "hip_pipe.h"
#include "lzhip.h"

using namespace lzhip;

struct lzhip_handle {
    std::unique_ptr<HIPScheduler> sched;
    HIPPipe* pipe = nullptr;  // owned by sched
};

static thread_local std::string g_err;

static int fail(int code, const char* what) {
    g_err = what ? what : "";
    return code;
}

#define GUARD_BEGIN try {
#define GUARD_END                                              \
    }                                                          \
    catch (const std::invalid_argument& e) {                   \
        return fail(LZHIP_EINVAL, e.what());                   \
    }                                                          \
    catch (const std::logic_error& e) {                        \
        return fail(LZHIP_EINVAL, e.what());                   \
    }                                                          \
    catch (const std::bad_alloc& e) {                          \
        return fail(LZHIP_ENOMEM, e.what());                   \
    }                                                          \
    catch (const std::exception& e) {                          \
        return fail(LZHIP_EDEVICE, e.what());                  \
    }                                                          \
    catch (...) {                                              \
        return fail(LZHIP_EDEVICE, "unknown failure");         \
    }

extern "C" {

const char* lzhip_last_error(void) { return g_err.c_str(); }
const char* lzhip_version(void) { return "lzhip 0.1 (gfx950)"; }

int lzhip_create(int filters, int precision, int max_batch, int device, lzhip_handle** out) {
    if (!out) return fail(LZHIP_EINVAL, "out is null");
    *out = nullptr;
    GUARD_BEGIN
    auto pipe = create_hip_pipe(device, precision, max_batch, filters);
    HIPPipe* raw = pipe.get();
    auto h = std::make_unique<lzhip_handle>();
    h->sched = std::make_unique<HIPScheduler>(std::unique_ptr<BatchExecutor>(pipe.release()));
    h->pipe = raw;
    *out = h.release();
    return LZHIP_OK;
    GUARD_END
}

int lzhip_destroy(lzhip_handle* h) {
    if (!h) return LZHIP_OK;
    GUARD_BEGIN
    delete h;
    return LZHIP_OK;
    GUARD_END
}

int lzhip_push_weights(lzhip_handle* h, int n_layers, const float* const* U,
                       const float* const* bn_mean, const float* const* bn_scale,
                       const float* pol_w, const float* val_w) {
    if (!h || !U || !bn_mean || !bn_scale || !pol_w || !val_w)
        return fail(LZHIP_EINVAL, "null argument");
    GUARD_BEGIN
    h->pipe->push_weights(n_layers, U, bn_mean, bn_scale, pol_w, val_w);
    return LZHIP_OK;
    GUARD_END
}

int lzhip_forward(lzhip_handle* h, const float* in, float* pol, float* val) {
    if (!h || !in || !pol || !val) return fail(LZHIP_EINVAL, "null argument");
    GUARD_BEGIN
    const int rc = h->sched->forward_raw(in, pol, val);
    if (rc == LZHIP_EHALT) return fail(LZHIP_EHALT, "halted by drain");
    return rc;
    GUARD_END
}

int lzhip_forward_batch(lzhip_handle* h, int n, const float* in, float* pol, float* val) {
    if (!h || !in || !pol || !val) return fail(LZHIP_EINVAL, "null argument");
    GUARD_BEGIN
    h->pipe->forward_batch(n, in, pol, val);
    return LZHIP_OK;
    GUARD_END
}

int lzhip_forward_batch_device(lzhip_handle* h, int n, const void* d_in, void* d_pol,
                               void* d_val) {
    if (!h || !d_in || !d_pol || !d_val) return fail(LZHIP_EINVAL, "null argument");
    GUARD_BEGIN
    h->pipe->forward_device(n, static_cast<const float*>(d_in), static_cast<float*>(d_pol),
                            static_cast<float*>(d_val));
    return LZHIP_OK;
    GUARD_END
}

int lzhip_sync(lzhip_handle* h) {
    if (!h) return fail(LZHIP_EINVAL, "null handle");
    GUARD_BEGIN
    h->pipe->sync();
    return LZHIP_OK;
    GUARD_END
}

void* lzhip_stream(lzhip_handle* h) { return h ? h->pipe->stream() : nullptr; }

int lzhip_drain(lzhip_handle* h) {
    if (!h) return fail(LZHIP_EINVAL, "null handle");
    GUARD_BEGIN
    h->sched->drain();
    return LZHIP_OK;
    GUARD_END
}

int lzhip_resume(lzhip_handle* h) {
    if (!h) return fail(LZHIP_EINVAL, "null handle");
    GUARD_BEGIN
    h->sched->resume();
    return LZHIP_OK;
    GUARD_END
}

int lzhip_get_stats(lzhip_handle* h, lzhip_stats* out) {
    if (!h || !out) return fail(LZHIP_EINVAL, "null argument");
    GUARD_BEGIN
    *out = h->sched->stats();
    return LZHIP_OK;
    GUARD_END
}

int lzhip_reset_stats(lzhip_handle* h) {
    if (!h) return fail(LZHIP_EINVAL, "null handle");
    GUARD_BEGIN
    h->sched->reset_stats();
    return LZHIP_OK;
    GUARD_END
}

int lzhip_push_heads(lzhip_handle* h, const float* bn_pol_mean, const float* bn_pol_scale,
                     const float* ip_pol_w, const float* ip_pol_b, const float* bn_val_mean,
                     const float* bn_val_scale, const float* ip1_val_w,
                     const float* ip1_val_b, const float* ip2_val_w, const float* ip2_val_b) {
    if (!h || !bn_pol_mean || !bn_pol_scale || !ip_pol_w || !ip_pol_b || !bn_val_mean ||
        !bn_val_scale || !ip1_val_w || !ip1_val_b || !ip2_val_w || !ip2_val_b)
        return fail(LZHIP_EINVAL, "null argument");
    GUARD_BEGIN
    HeadWeightsHost hw{bn_pol_mean, bn_pol_scale, ip_pol_w,  ip_pol_b,  bn_val_mean,
                       bn_val_scale, ip1_val_w,   ip1_val_b, ip2_val_w, ip2_val_b};
    h->pipe->push_heads(hw);
    return LZHIP_OK;
    GUARD_END
}

int lzhip_evaluate_batch(lzhip_handle* h, int n, const float* in, float temperature,
                         float* policy, float* value, float* logits, float* pol, float* val) {
    if (!h || !in || !policy || !value) return fail(LZHIP_EINVAL, "null argument");
    GUARD_BEGIN
    h->pipe->evaluate_batch(n, in, temperature, policy, value, logits, pol, val);
    return LZHIP_OK;
    GUARD_END
}

// Network::winograd_transform_f (reference src/Network.cpp:159-223):
// U = G f G^T for every (output, channel) filter, written position-major with
// the output channel fastest: U[(xi*6+nu)][c][o].
int lzhip_winograd_transform_f(const float* f, int outputs, int channels, float* U) {
    if (!f || !U || outputs < 1 || channels < 1) return fail(LZHIP_EINVAL, "bad argument");
    const float s2 = 1.4142135623730951f;
    const float G[6][3] = {{1.0f, 0.0f, 0.0f},
                           {-2.0f / 3.0f, -s2 / 3.0f, -1.0f / 3.0f},
                           {-2.0f / 3.0f, s2 / 3.0f, -1.0f / 3.0f},
                           {1.0f / 6.0f, s2 / 6.0f, 1.0f / 3.0f},
                           {1.0f / 6.0f, -s2 / 6.0f, 1.0f / 3.0f},
                           {0.0f, 0.0f, 1.0f}};
    const size_t plane = (size_t)channels * outputs;
    for (int o = 0; o < outputs; o++)
        for (int c = 0; c < channels; c++) {
            const float* g = f + ((size_t)o * channels + c) * 9;
            float Gg[6][3];
            for (int i = 0; i < 6; i++)
                for (int j = 0; j < 3; j++) {
                    float acc = 0.0f;
                    for (int k = 0; k < 3; k++) acc += G[i][k] * g[k * 3 + j];
                    Gg[i][j] = acc;
                }
            float* dst = U + (size_t)c * outputs + o;
            for (int xi = 0; xi < 6; xi++)
                for (int nu = 0; nu < 6; nu++) {
                    float acc = 0.0f;
                    for (int k = 0; k < 3; k++) acc += Gg[xi][k] * G[nu][k];
                    dst[(size_t)(xi * 6 + nu) * plane] = acc;
                }
        }
    return LZHIP_OK;
}

int lzhip_process_bn_var(float* w, int n) {
    if (!w || n < 0) return fail(LZHIP_EINVAL, "bad argument");
    for (int i = 0; i < n; i++) w[i] = 1.0f / std::sqrt(w[i] + 1e-5f);
    return LZHIP_OK;
}

int lzhip_debug_layer(lzhip_handle* h, int layer, int n, const float* act_in, const float* res,
                      float* V, float* M, float* Y) {
    if (!h || !act_in) return fail(LZHIP_EINVAL, "null argument");
    GUARD_BEGIN
    h->pipe->debug_layer(layer, n, act_in, res, V, M, Y);
    return LZHIP_OK;
    GUARD_END
}

int lzhip_get_act_scales(lzhip_handle* h, float* out, int n) {
    if (!h || !out) return fail(LZHIP_EINVAL, "null argument");
    GUARD_BEGIN
    const auto s = h->pipe->act_scales();
    if ((int)s.size() != n) return fail(LZHIP_EINVAL, "n must be n_layers + 1");
    std::memcpy(out, s.data(), sizeof(float) * s.size());
    return LZHIP_OK;
    GUARD_END
}

int lzhip_profile_forward(lzhip_handle* h, int n, const void* d_in, void* d_pol, void* d_val,
                          float* ms, int* launches) {
    if (!h || !d_in || !d_pol || !d_val || !ms || !launches)
        return fail(LZHIP_EINVAL, "null argument");
    GUARD_BEGIN
    h->pipe->profile_forward(n, static_cast<const float*>(d_in), static_cast<float*>(d_pol),
                             static_cast<float*>(d_val), ms, launches);
    return LZHIP_OK;
    GUARD_END
}

}  // extern "C"
