// TEST INFRASTRUCTURE ONLY -- not part of the product path.
//
// Drives the reference's evaluation cache (NNCache, compiled from the reference tree by
// oracle/Makefile, target `ref`) with a script of operations, so that the replacement
// policy of the search driver's cache can be compared with it operation by operation.
// Protocol (stdin): first line the capacity; then one operation per line,
// "i <hash> <winrate>" (insert) or "l <hash>" (lookup).  Every lookup answers one line:
// "0" for a miss or "1 <winrate>" for a hit.
#include <cstdint>
#include <cstdio>
#include <iostream>
#include <string>

#include "NNCache.h"

int main() {
    int size;
    if (!(std::cin >> size)) return 1;
    NNCache cache(size);
    std::string op;
    while (std::cin >> op) {
        std::uint64_t hash;
        std::cin >> hash;
        if (op == "i") {
            float w;
            std::cin >> w;
            NNCache::Netresult r;
            r.winrate = w;
            cache.insert(hash, r);
        } else {
            NNCache::Netresult r;
            if (cache.lookup(hash, r)) std::printf("1 %.3f\n", r.winrate);
            else std::printf("0\n");
        }
    }
    return 0;
}
