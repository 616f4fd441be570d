// Compile-only check, built with -fsyntax-only against the engine's real headers
// (-I<reference>/src -DLZHIP_ENGINE_BUILD): the two drop-in classes override the engine's
// own ForwardPipe (reference src/ForwardPipe.h:38-71) signature for signature -- every
// `override` below is checked by the compiler against that header -- and throw the
// engine's NetworkHaltException (reference src/Network.h:66-67).
#include <memory>
#include <vector>

#include "forward_pipe.h"       // lzhip::HIPScheduler, on top of the engine's ForwardPipe.h
#include "HIPPipeAdapter.h"     // the C-ABI adapter

static std::unique_ptr<ForwardPipe>&& init_like_the_engine(int channels,
                                                           std::unique_ptr<ForwardPipe>&& pipe) {
    // the call sequence of Network::init_net (reference src/Network.cpp:407-414)
    auto weights = std::make_shared<ForwardPipe::ForwardPipeWeights>();
    pipe->initialize(channels);
    pipe->push_weights(6, 18, channels, weights);
    return std::move(pipe);
}

int main() {
    std::unique_ptr<ForwardPipe> a =
        init_like_the_engine(256, std::make_unique<lzhip::HIPScheduler>(LZHIP_FP16, 64, 0));
    std::unique_ptr<ForwardPipe> b =
        init_like_the_engine(256, std::make_unique<HIPPipeAdapter>(LZHIP_FP16, 64, 0));
    std::vector<float> in(LZHIP_INPUT_SIZE), pol(LZHIP_POL_SIZE), val(LZHIP_VAL_SIZE);
    try {
        a->forward(in, pol, val);
        b->forward(in, pol, val);
    } catch (const NetworkHaltException&) {
    }
    a->drain();
    a->resume();
    return a->needs_autodetect() || b->needs_autodetect();
}
