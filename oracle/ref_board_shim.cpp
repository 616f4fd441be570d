// TEST INFRASTRUCTURE ONLY -- not part of the product path.
//
// Drives the reference's own board code (FullBoard / FastBoard, compiled from the
// reference tree by oracle/Makefile, target `ref`) so that the Go rules the search
// driver plays by, and their plain-Python restatement, can be checked against the real
// thing.  This file is a caller of the reference, not a copy of it: it replays a move
// list with FullBoard::update_board (reference src/FullBoard.cpp:139-210) and reports
// what FastState::is_move_legal would answer (src/FastState.cpp:76-83: not the ko
// vertex, empty, not suicide), the ko vertex, the area score
// (src/FastBoard.cpp:292-296) and whether the stones repeat an earlier position (what
// KoState::superko decides through hashes, src/KoState.cpp:51-58; compared here on the
// stones themselves, because the hash tables need the engine's random generator and
// configuration globals, which do not build in this image).
//
// Protocol (stdin -> stdout, one game per line): "n m1 m2 ... mn" with moves 0..360 =
// y*19+x, 361 = pass; answer: "ok <ko> <superko> <score> <361 stones 0/1/2> <362 legal
// 0/1>" or "illegal <index>".
#include <cstdio>
#include <iostream>
#include <sstream>
#include <string>
#include <vector>

#include "FullBoard.h"

static int vertex_of(const FullBoard& b, int mv) { return b.get_vertex(mv % 19, mv / 19); }

int main() {
    std::string line;
    while (std::getline(std::cin, line)) {
        std::istringstream in(line);
        int n;
        if (!(in >> n)) break;
        std::vector<int> moves(n);
        for (auto& m : moves) in >> m;
        FullBoard b;
        b.reset_board(19);
        int color = FastBoard::BLACK, komove = FastBoard::NO_VERTEX;
        std::vector<std::string> seen;
        auto stones_of = [&]() {
            std::string s(361, '2');
            for (int i = 0; i < 361; i++) {
                const auto st = b.get_state(i % 19, i / 19);
                s[i] = st == FastBoard::BLACK ? '0' : (st == FastBoard::WHITE ? '1' : '2');
            }
            return s;
        };
        auto legal = [&](int mv) {
            if (mv == 361) return true;
            const int v = vertex_of(b, mv);
            return v != komove && b.get_state(v) == FastBoard::EMPTY && !b.is_suicide(v, color);
        };
        seen.push_back(stones_of());
        int bad = -1;
        bool repeated = false;
        for (int i = 0; i < n; i++) {
            if (moves[i] < 0 || moves[i] > 361 || !legal(moves[i])) {
                bad = i;
                break;
            }
            if (moves[i] == 361) {
                komove = FastBoard::NO_VERTEX;
                repeated = false;
            } else {
                komove = b.update_board(color, vertex_of(b, moves[i]));
                const std::string now = stones_of();
                repeated = false;
                for (const auto& s : seen) repeated = repeated || s == now;
            }
            seen.push_back(stones_of());
            color = !color;
        }
        if (bad >= 0) {
            std::printf("illegal %d\n", bad);
            continue;
        }
        int ko = -1;
        if (komove != FastBoard::NO_VERTEX) {
            const auto xy = b.get_xy(komove);
            ko = xy.second * 19 + xy.first;
        }
        std::string leg(362, '0');
        for (int mv = 0; mv <= 361; mv++) leg[mv] = legal(mv) ? '1' : '0';
        std::printf("ok %d %d %.1f %s %s\n", ko, repeated ? 1 : 0, b.area_score(7.5f),
                    stones_of().c_str(), leg.c_str());
    }
    return 0;
}
