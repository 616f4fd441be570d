// The C++ drop-in path on a real device, as the engine would use it: construct
// lzhip::HIPScheduler as a ForwardPipe (reference src/Network.cpp:578-597),
// initialize(channels), push_weights(6, 18, channels, shared_ptr<ForwardPipeWeights>)
// (src/Network.cpp:407-414), then forward() from several threads, drain()/resume().
// Results must be bit-identical to the C-ABI path on the same weights (both run
// the same executor), and a halted call must throw NetworkHaltException.
// Built by the package's build step into csrc/engine_path_test; run on a GPU box.
#include <atomic>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <memory>
#include <random>
#include <thread>
#include <vector>

#include "forward_pipe.h"
#include "lzhip.h"

#define CHECK(cond)                                                                 \
    do {                                                                            \
        if (!(cond)) {                                                              \
            std::fprintf(stderr, "FAILED %s:%d: %s\n", __FILE__, __LINE__, #cond); \
            std::exit(1);                                                           \
        }                                                                           \
    } while (0)

int main() {
    const int F = 64, blocks = 2, nl = 1 + 2 * blocks, B = 4;
    std::mt19937 rng(123);
    std::normal_distribution<float> nd(0.0f, 1.0f);
    std::uniform_real_distribution<float> ud(0.5f, 1.5f);

    // Winograd-domain filters straight from the library's own host transform.
    auto w = std::make_shared<ForwardPipe::ForwardPipeWeights>();
    for (int l = 0; l < nl; l++) {
        const int cin = l == 0 ? 18 : F;
        std::vector<float> f((size_t)F * cin * 9), U((size_t)36 * cin * F);
        const float sd = std::sqrt(2.0f / (9.0f * cin));
        for (auto& v : f) v = nd(rng) * sd;
        CHECK(lzhip_winograd_transform_f(f.data(), F, cin, U.data()) == LZHIP_OK);
        w->m_conv_weights.push_back(U);
        w->m_conv_biases.emplace_back(F, 0.0f);
        std::vector<float> mean(F), var(F);
        for (auto& v : mean) v = 0.1f * nd(rng);
        for (auto& v : var) v = ud(rng);
        CHECK(lzhip_process_bn_var(var.data(), F) == LZHIP_OK);
        w->m_batchnorm_means.push_back(mean);
        w->m_batchnorm_stddevs.push_back(var);
    }
    w->m_conv_pol_w.resize(2 * F);
    w->m_conv_val_w.resize(F);
    for (auto& v : w->m_conv_pol_w) v = nd(rng) * std::sqrt(2.0f / F);
    for (auto& v : w->m_conv_val_w) v = nd(rng) * std::sqrt(2.0f / F);
    w->m_conv_pol_b.assign(2, 0.0f);
    w->m_conv_val_b.assign(1, 0.0f);

    const int N = 12;
    std::vector<std::vector<float>> in(N, std::vector<float>(LZHIP_INPUT_SIZE, 0.0f));
    std::uniform_real_distribution<float> u01(0.0f, 1.0f);
    for (auto& x : in) {
        for (int h = 0; h < 8; h++)
            for (int p = 0; p < 361; p++) {
                const float u = u01(rng);
                if (u < 0.2f) x[h * 361 + p] = 1.0f;
                else if (u < 0.4f) x[(8 + h) * 361 + p] = 1.0f;
            }
        for (int p = 0; p < 361; p++) x[16 * 361 + p] = 1.0f;
    }

    for (int precision : {LZHIP_FP32, LZHIP_FP16}) {
        // the C-ABI path
        lzhip_handle* h = nullptr;
        if (lzhip_create(F, precision, B, 0, &h) != LZHIP_OK) {
            std::fprintf(stderr, "lzhip_create: %s\n", lzhip_last_error());
            return 2;
        }
        std::vector<const float*> U(nl), mean(nl), scale(nl);
        for (int l = 0; l < nl; l++) {
            U[l] = w->m_conv_weights[l].data();
            mean[l] = w->m_batchnorm_means[l].data();
            scale[l] = w->m_batchnorm_stddevs[l].data();
        }
        CHECK(lzhip_push_weights(h, nl, U.data(), mean.data(), scale.data(),
                                 w->m_conv_pol_w.data(), w->m_conv_val_w.data()) == LZHIP_OK);
        std::vector<std::vector<float>> rpol(N, std::vector<float>(LZHIP_POL_SIZE)),
            rval(N, std::vector<float>(LZHIP_VAL_SIZE));
        for (int i = 0; i < N; i++)
            CHECK(lzhip_forward(h, in[i].data(), rpol[i].data(), rval[i].data()) == LZHIP_OK);
        CHECK(lzhip_destroy(h) == LZHIP_OK);

        // the engine-facing class, through the base-class pointer
        std::unique_ptr<ForwardPipe> pipe = std::make_unique<lzhip::HIPScheduler>(precision, B, 0);
        CHECK(!pipe->needs_autodetect());
        pipe->initialize(F);
        pipe->push_weights(6, 18, F, w);
        std::atomic<int> ok{0};
        std::vector<std::thread> th;
        for (int t = 0; t < 6; t++)
            th.emplace_back([&, t] {
                std::vector<float> pol(LZHIP_POL_SIZE), val(LZHIP_VAL_SIZE);
                for (int i = t; i < N; i += 6) {
                    pipe->forward(in[i], pol, val);
                    CHECK(std::memcmp(pol.data(), rpol[i].data(), sizeof(float) * LZHIP_POL_SIZE) == 0);
                    CHECK(std::memcmp(val.data(), rval[i].data(), sizeof(float) * LZHIP_VAL_SIZE) == 0);
                    for (float v : pol) CHECK(std::isfinite(v));
                    ok++;
                }
            });
        for (auto& t : th) t.join();
        CHECK(ok == N);
        pipe->drain();
        bool halted = false;
        try {
            std::vector<float> pol(LZHIP_POL_SIZE), val(LZHIP_VAL_SIZE);
            pipe->forward(in[0], pol, val);
        } catch (const NetworkHaltException&) {
            halted = true;
        }
        CHECK(halted);
        pipe->resume();
        {
            std::vector<float> pol(LZHIP_POL_SIZE), val(LZHIP_VAL_SIZE);
            pipe->forward(in[0], pol, val);
            CHECK(std::memcmp(pol.data(), rpol[0].data(), sizeof(float) * LZHIP_POL_SIZE) == 0);
        }
        // wrong shapes are refused as the reference's asserts would
        bool threw = false;
        try {
            pipe->push_weights(3, 18, F, w);
        } catch (const std::exception&) {
            threw = true;
        }
        CHECK(threw);
        std::printf("precision %d: engine path matches the C ABI bit for bit\n", precision);
    }
    std::printf("engine path ok\n");
    return 0;
}
