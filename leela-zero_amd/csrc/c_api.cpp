// extern "C" surface declared in include/lzhip.h.  Every function converts
// C++ exceptions into return codes; the message of the last failure is kept
// per calling thread.
#include <algorithm>
#include <atomic>
#include <chrono>
#include <cmath>
#include <cstring>
#include <memory>
#include <mutex>
#include <stdexcept>
#include <string>
#include <thread>
#include <vector>

#include "forward_pipe.h"
#include "hip_pipe.h"
#include "lzhip.h"
#include "lzhip_search.h"
#include "search.h"
#include "weights_file.h"

using namespace lzhip;

struct lzhip_handle {
    std::unique_ptr<HIPScheduler> sched;
    HIPPipe* pipe = nullptr;  // owned by sched
    // host-side copy of what lzhip_push_heads received, for the entry points
    // that run the heads on the calling thread with `heads == NULL`
    std::shared_ptr<const HeadWeights> host_heads;
    std::mutex heads_mu;
    // Network::m_value_head_not_stm: set by the caller that read a format-2 weights file
    std::atomic<bool> value_not_stm{false};
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

int lzhip_create_from_file(const char* path, int precision, int max_batch, int device,
                           lzhip_handle** out, int* filters, int* blocks) {
    if (!path || !out) return fail(LZHIP_EINVAL, "null argument");
    *out = nullptr;
    GUARD_BEGIN
    const WeightsFile wf = load_weights_file(path);   // before any device is touched
    if (filters) *filters = wf.filters;
    if (blocks) *blocks = wf.blocks;
    lzhip_handle* raw = nullptr;
    int rc = lzhip_create(wf.filters, precision, max_batch, device, &raw);
    if (rc != LZHIP_OK) return rc;
    // owned until everything has succeeded: an exception below (e.g. bad_alloc in the
    // pointer tables) must not leave the handle behind
    struct Destroy {
        void operator()(lzhip_handle* p) const { delete p; }
    };
    std::unique_ptr<lzhip_handle, Destroy> owner(raw);
    lzhip_handle* h = raw;
    const size_t nl = wf.U.size();
    std::vector<const float*> U(nl), mean(nl), scale(nl);
    for (size_t l = 0; l < nl; l++) {
        U[l] = wf.U[l].data();
        mean[l] = wf.bn_mean[l].data();
        scale[l] = wf.bn_scale[l].data();
    }
    rc = lzhip_push_weights(h, (int)nl, U.data(), mean.data(), scale.data(), wf.conv_pol_w.data(),
                            wf.conv_val_w.data());
    if (rc == LZHIP_OK)
        rc = lzhip_push_heads(h, wf.bn_pol_mean.data(), wf.bn_pol_scale.data(), wf.ip_pol_w.data(),
                              wf.ip_pol_b.data(), wf.bn_val_mean.data(), wf.bn_val_scale.data(),
                              wf.ip1_val_w.data(), wf.ip1_val_b.data(), wf.ip2_val_w.data(),
                              wf.ip2_val_b.data());
    if (rc != LZHIP_OK) {
        const std::string keep = g_err;
        owner.reset();
        g_err = keep;
        return rc;
    }
    owner.release();
    h->value_not_stm.store(wf.value_head_not_stm);
    *out = h;
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
    h->pipe->forward_device(0, n, static_cast<const float*>(d_in), static_cast<float*>(d_pol),
                            static_cast<float*>(d_val));
    return LZHIP_OK;
    GUARD_END
}

int lzhip_lanes(lzhip_handle* h) { return h ? h->pipe->lanes() : 0; }

int lzhip_forward_batch_device_lane(lzhip_handle* h, int lane, int n, const void* d_in,
                                    void* d_pol, void* d_val) {
    if (!h || !d_in || !d_pol || !d_val) return fail(LZHIP_EINVAL, "null argument");
    GUARD_BEGIN
    h->pipe->forward_device(lane, n, static_cast<const float*>(d_in),
                            static_cast<float*>(d_pol), static_cast<float*>(d_val));
    return LZHIP_OK;
    GUARD_END
}

int lzhip_forward_batch_device_noalloc(lzhip_handle* h, int n, const void* d_in, void* d_pol,
                                       void* d_val) {
    if (!h || !d_in || !d_pol || !d_val) return fail(LZHIP_EINVAL, "null argument");
    GUARD_BEGIN
    h->pipe->forward_device_static(n, static_cast<const float*>(d_in),
                                   static_cast<float*>(d_pol), static_cast<float*>(d_val));
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

int lzhip_process_batch_stats(uint64_t out[4]) {
    if (!out) return fail(LZHIP_EINVAL, "null argument");
    out[0] = lzhip::batch_stats.single_evals.load();
    out[1] = lzhip::batch_stats.batch_evals.load();
    out[2] = lzhip::batch_stats.positions.load();
    out[3] = lzhip::batch_stats.slots.load();
    return LZHIP_OK;
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
    const lzhip_head_weights c{bn_pol_mean, bn_pol_scale, ip_pol_w,  ip_pol_b,  bn_val_mean,
                               bn_val_scale, ip1_val_w,   ip1_val_b, ip2_val_w, ip2_val_b};
    auto host = std::make_shared<const HeadWeights>(c);
    std::lock_guard<std::mutex> lk(h->heads_mu);
    h->host_heads = std::move(host);
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

int lzhip_timed_evaluations(lzhip_handle* h, int n, int reps, const float* in,
                            float temperature, float* policy, float* value, float* ms) {
    if (!h || !in || !policy || !value || !ms) return fail(LZHIP_EINVAL, "null argument");
    GUARD_BEGIN
    *ms = h->pipe->timed_evaluations(n, reps, in, temperature, policy, value);
    return LZHIP_OK;
    GUARD_END
}

int lzhip_forward_eval(lzhip_handle* h, const float* in, float temperature, float* policy,
                       float* value) {
    if (!h || !in || !policy || !value) return fail(LZHIP_EINVAL, "null argument");
    GUARD_BEGIN
    const int rc = h->sched->evaluate_raw(in, temperature, policy, value);
    if (rc == LZHIP_EHALT) return fail(LZHIP_EHALT, "halted by drain");
    return rc;
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

size_t lzhip_ceil_multiple(size_t a, size_t b) { return lzhip::ceil_multiple(a, b); }

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

// ---- callers above forward(): planes, one evaluation, search driver ---------

static bool heads_complete(const lzhip_head_weights* w) {
    return w && w->bn_pol_mean && w->bn_pol_scale && w->ip_pol_w && w->ip_pol_b && w->bn_val_mean &&
           w->bn_val_scale && w->ip1_val_w && w->ip1_val_b && w->ip2_val_w && w->ip2_val_b;
}

// The head parameters an entry point works with: the caller's, or, for NULL,
// the ones lzhip_push_heads stored.
static std::shared_ptr<const HeadWeights> resolve_heads(lzhip_handle* h,
                                                        const lzhip_head_weights* heads) {
    if (heads) {
        if (!heads_complete(heads)) throw std::invalid_argument("head parameters contain a null pointer");
        return std::make_shared<const HeadWeights>(*heads);
    }
    std::lock_guard<std::mutex> lk(h->heads_mu);
    if (!h->host_heads) throw std::invalid_argument("heads is NULL and lzhip_push_heads was not called");
    return h->host_heads;
}

int lzhip_symmetry_index(int symmetry, int idx) { return symmetry_index(symmetry, idx); }

int lzhip_gather_features(const uint8_t* boards, int n_boards, int to_move, int symmetry,
                          float* out) {
    if (!boards || !out) return fail(LZHIP_EINVAL, "null argument");
    if (n_boards < 1 || n_boards > go::kHistory || (to_move != LZHIP_BLACK && to_move != LZHIP_WHITE) ||
        symmetry < 0 || symmetry >= 8)
        return fail(LZHIP_EINVAL, "n_boards in 1..8, to_move 0/1, symmetry 0..7");
    const uint8_t* ptr[go::kHistory];
    for (int h = 0; h < n_boards; h++) ptr[h] = boards + (size_t)h * go::kPoints;
    gather_features(ptr, n_boards, to_move, symmetry, out);
    return LZHIP_OK;
}

int lzhip_get_output(lzhip_handle* h, const lzhip_head_weights* heads, const uint8_t* boards,
                     int n_boards, int to_move, int symmetry, float softmax_temp, float* policy,
                     float* winrate) {
    if (!h || !boards || !policy || !winrate) return fail(LZHIP_EINVAL, "null argument");
    if (!(softmax_temp > 0.0f)) return fail(LZHIP_EINVAL, "softmax_temp must be positive");
    GUARD_BEGIN
    const auto hw = resolve_heads(h, heads);
    std::vector<float> in(LZHIP_INPUT_SIZE), pol(LZHIP_POL_SIZE), val(LZHIP_VAL_SIZE);
    const int rc = lzhip_gather_features(boards, n_boards, to_move, symmetry, in.data());
    if (rc != LZHIP_OK) return rc;
    const int frc = h->sched->forward_raw(in.data(), pol.data(), val.data());
    if (frc == LZHIP_EHALT) return fail(LZHIP_EHALT, "halted by drain");
    float p[go::kPoints + 1];
    heads_on_host(*hw, pol.data(), val.data(), softmax_temp, p, winrate);
    for (int i = 0; i < go::kPoints; i++) policy[symmetry_index(symmetry, i)] = p[i];
    policy[go::kPoints] = p[go::kPoints];
    if (h->value_not_stm.load() && to_move == go::WHITE) *winrate = 1.0f - *winrate;
    return LZHIP_OK;
    GUARD_END
}

int lzhip_netbench(lzhip_handle* h, const lzhip_head_weights* heads, const uint8_t* boards,
                   int n_boards, int to_move, int threads, int iterations, uint64_t seed,
                   int* evaluations, double* seconds) {
    if (!h || !boards || !evaluations || !seconds) return fail(LZHIP_EINVAL, "null argument");
    if (threads < 1 || threads > 4096 || iterations < 1)
        return fail(LZHIP_EINVAL, "threads and iterations must be positive");
    GUARD_BEGIN
    const auto hw = resolve_heads(h, heads);
    {   // the arguments are checked once, here, not in every thread
        std::vector<float> probe(LZHIP_INPUT_SIZE);
        const int rc = lzhip_gather_features(boards, n_boards, to_move, 0, probe.data());
        if (rc != LZHIP_OK) return rc;
    }
    std::atomic<int> runcount{0}, halted{0};
    std::mutex err_mu;
    std::string err;
    const auto t0 = std::chrono::steady_clock::now();
    std::vector<std::thread> pool;
    for (int t = 0; t < threads; t++)
        pool.emplace_back([&, t] {
            std::vector<float> in(LZHIP_INPUT_SIZE), pol(LZHIP_POL_SIZE), val(LZHIP_VAL_SIZE);
            uint64_t st = seed + 0x9E3779B97F4A7C15ull * (uint64_t)(t + 1);
            float p[go::kPoints + 1], win;
            try {
                while (runcount.load() < iterations && halted.load() == 0) {
                    runcount++;
                    st = st * 6364136223846793005ull + 1442695040888963407ull;
                    const int sym = (int)(st >> 61);
                    lzhip_gather_features(boards, n_boards, to_move, sym, in.data());
                    if (h->sched->forward_raw(in.data(), pol.data(), val.data()) == LZHIP_EHALT) {
                        halted++;
                        break;
                    }
                    heads_on_host(*hw, pol.data(), val.data(), 1.0f, p, &win);
                }
            } catch (const std::exception& e) {
                std::lock_guard<std::mutex> lk(err_mu);
                err = e.what();
                halted++;
            }
        });
    for (auto& th : pool) th.join();
    *seconds = std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count();
    *evaluations = runcount.load();
    if (!err.empty()) throw std::runtime_error(err);
    if (halted.load()) return fail(LZHIP_EHALT, "halted by drain");
    return LZHIP_OK;
    GUARD_END
}

int lzhip_get_output_average(lzhip_handle* h, const lzhip_head_weights* heads,
                             const uint8_t* boards, int n_boards, int to_move,
                             float softmax_temp, float* policy, float* winrate) {
    if (!h || !boards || !policy || !winrate) return fail(LZHIP_EINVAL, "null argument");
    if (!(softmax_temp > 0.0f)) return fail(LZHIP_EINVAL, "softmax_temp must be positive");
    GUARD_BEGIN
    const auto hw = resolve_heads(h, heads);
    constexpr int S = 8;
    std::vector<float> in((size_t)S * LZHIP_INPUT_SIZE), pol((size_t)S * LZHIP_POL_SIZE),
        val((size_t)S * LZHIP_VAL_SIZE);
    for (int sym = 0; sym < S; sym++) {
        const int rc = lzhip_gather_features(boards, n_boards, to_move, sym,
                                             in.data() + (size_t)sym * LZHIP_INPUT_SIZE);
        if (rc != LZHIP_OK) return rc;
    }
    const int step = std::min(S, h->pipe->max_batch());
    for (int s0 = 0; s0 < S; s0 += step) {
        const int n = std::min(step, S - s0);
        h->pipe->forward_batch(n, in.data() + (size_t)s0 * LZHIP_INPUT_SIZE,
                               pol.data() + (size_t)s0 * LZHIP_POL_SIZE,
                               val.data() + (size_t)s0 * LZHIP_VAL_SIZE);
    }
    for (int i = 0; i <= go::kPoints; i++) policy[i] = 0.0f;
    float win = 0.0f;
    for (int sym = 0; sym < S; sym++) {
        float p[go::kPoints + 1], w;
        heads_on_host(*hw, pol.data() + (size_t)sym * LZHIP_POL_SIZE,
                      val.data() + (size_t)sym * LZHIP_VAL_SIZE, softmax_temp, p, &w);
        for (int i = 0; i < go::kPoints; i++) policy[symmetry_index(sym, i)] += p[i] / (float)S;
        policy[go::kPoints] += p[go::kPoints] / (float)S;
        win += w / (float)S;
    }
    *winrate = (h->value_not_stm.load() && to_move == go::WHITE) ? 1.0f - win : win;
    return LZHIP_OK;
    GUARD_END
}

int lzhip_set_value_head_not_stm(lzhip_handle* h, int on) {
    if (!h) return fail(LZHIP_EINVAL, "null handle");
    h->value_not_stm.store(on != 0);
    return LZHIP_OK;
}

int lzhip_search_default_config(lzhip_search_config* cfg) {
    if (!cfg) return fail(LZHIP_EINVAL, "null argument");
    std::memset(cfg, 0, sizeof(*cfg));
    cfg->threads = 16;
    cfg->visits = 1600;
    cfg->moves = 20;
    cfg->cache_size = 150000;
    cfg->reuse_tree = 1;
    cfg->random_moves = 0;
    cfg->virtual_loss = 3;
    cfg->device_heads = 0;
    cfg->puct = 0.5f;
    cfg->logpuct = 0.015f;
    cfg->logconst = 1.7f;
    cfg->fpu_reduction = 0.25f;
    cfg->fpu_root_reduction = cfg->fpu_reduction;
    cfg->softmax_temp = 1.0f;
    cfg->komi = 7.5f;
    cfg->seed = 1;
    return LZHIP_OK;
}

int lzhip_selfplay(lzhip_handle* h, const lzhip_head_weights* heads,
                   const lzhip_search_config* cfg, lzhip_search_result* result, int* moves_out,
                   int moves_cap) {
    if (!h || !cfg || !result) return fail(LZHIP_EINVAL, "null argument");
    if (cfg->threads < 1 || cfg->threads > 4096 || cfg->visits < 1 || cfg->moves < 0 ||
        !(cfg->softmax_temp > 0.0f))
        return fail(LZHIP_EINVAL, "threads in 1..4096, visits >= 1, moves >= 0, softmax_temp > 0");
    GUARD_BEGIN
    selfplay(*h->sched, resolve_heads(h, heads), *cfg, *result, moves_out,
             moves_out ? moves_cap : 0, h->value_not_stm.load());
    return LZHIP_OK;
    GUARD_END
}

int lzhip_board_replay(const int* moves, int n_moves, float komi, uint8_t* stones, uint8_t* legal,
                       int* ko_point, int* superko, float* score) {
    if (n_moves < 0 || (n_moves > 0 && !moves)) return fail(LZHIP_EINVAL, "bad move list");
    GUARD_BEGIN
    go::Position pos;
    bool repeated = false;
    for (int i = 0; i < n_moves; i++) {
        const int mv = moves[i];
        if (mv < 0 || mv > go::kPass || !pos.legal_slow(pos.to_move(), mv))
            return fail(LZHIP_EINVAL, "illegal move in the list");
        pos.play(mv);
        repeated = (mv != go::kPass) && pos.superko();
    }
    if (stones) std::memcpy(stones, pos.stones().data(), go::kPoints);
    if (legal) {
        go::GroupInfo g;
        pos.analyze(g);
        for (int v = 0; v <= go::kPass; v++) legal[v] = pos.legal(g, pos.to_move(), v) ? 1 : 0;
    }
    if (ko_point) *ko_point = pos.ko_point();
    if (superko) *superko = repeated ? 1 : 0;
    if (score) *score = pos.area_score(komi);
    return LZHIP_OK;
    GUARD_END
}

}  // extern "C"
