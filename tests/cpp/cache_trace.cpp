// Runs a script of cache operations through the search driver's EvalCache and prints
// the outcome of every lookup, in the format oracle/ref_cache_shim.cpp uses for the
// reference's NNCache (reference src/NNCache.cpp:47-80), so that the two can be compared
// line by line.  Input: capacity, then "i <hash> <winrate>" / "l <hash>" lines.
#include <cstdint>
#include <cstdio>
#include <iostream>
#include <stdexcept>
#include <string>

#include "search.h"

namespace lzhip {
std::unique_ptr<BatchExecutor> make_hip_pipe(int, int, int, int) {
    throw std::runtime_error("no device in this tool");
}
}  // namespace lzhip

int main() {
    int size;
    if (!(std::cin >> size)) return 1;
    lzhip::EvalCache cache((size_t)size);
    std::string op;
    while (std::cin >> op) {
        std::uint64_t hash;
        std::cin >> hash;
        if (op == "i") {
            float w;
            std::cin >> w;
            lzhip::Netresult r;
            r.winrate = w;
            cache.insert(hash, r);
        } else {
            lzhip::Netresult r;
            if (cache.lookup(hash, r)) std::printf("1 %.3f\n", r.winrate);
            else std::printf("0\n");
        }
    }
    return 0;
}
