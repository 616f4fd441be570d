// Compact 19x19 Go rules for the search driver: stones, captures, simple ko,
// positional superko, passes, area scoring and an 8-position history for the
// network's input planes.  It provides what the search asks of the reference's
// board classes (FastBoard::is_suicide src/FastBoard.cpp:168-195,
// FullBoard::update_board src/FullBoard.cpp:150-210, FastState::is_move_legal
// src/FastState.cpp:76-83, FastState::play_move :89-110, KoState::superko
// src/KoState.cpp:51-58, FastBoard::area_score src/FastBoard.cpp:260-296,
// GameState::get_past_board) with a different
// design: no incremental string bookkeeping; groups and liberties are found by
// flood fill, once per position for move generation and locally for captures.
#ifndef LZHIP_GOBOARD_H_INCLUDED
#define LZHIP_GOBOARD_H_INCLUDED

#include <array>
#include <cstdint>
#include <cstring>
#include <vector>

namespace lzhip {
namespace go {

constexpr int kSize = 19;
constexpr int kPoints = kSize * kSize;
constexpr int kPass = kPoints;  // move index 0..360 = y*19+x, 361 = pass
constexpr int kHistory = 8;

enum : uint8_t { BLACK = 0, WHITE = 1, EMPTY = 2 };

struct Tables {
    int8_t n_nbr[kPoints];
    int16_t nbr[kPoints][4];
    uint64_t zob[2][kPoints];
    uint64_t zob_ko[kPoints + 1];
    uint64_t zob_pass[4];
    uint64_t zob_white_to_move;
    Tables();
};
const Tables& tables();

using Stones = std::array<uint8_t, kPoints>;

// Per-position group map used by move generation.
struct GroupInfo {
    int16_t id[kPoints];    // group index of a stone, -1 on empty points
    int16_t libs[kPoints];  // liberties of group index g (first n_groups valid)
    int n_groups = 0;
};

class Position {
public:
    Position();

    int to_move() const { return m_to_move; }
    int passes() const { return m_passes; }
    int movenum() const { return m_movenum; }
    int ko_point() const { return m_ko; }
    uint8_t at(int v) const { return m_sq[v]; }
    const Stones& stones() const { return m_sq; }
    // Stones `h` moves ago (h = 0 is the present), h < min(movenum()+1, 8).
    const Stones& past(int h) const { return m_hist[(m_hist_head + kHistory - h) % kHistory]; }

    // Key of the cache: stones, side to move, ko point and pass count
    // (the reference's FastBoard hash covers the same state).
    uint64_t hash() const;
    uint64_t stone_hash() const { return m_stone_hash; }
    // hash() of the position in which every point v has moved to map[v]
    // (reference FullBoard::calc_symmetry_hash, src/FullBoard.cpp:111-122).
    uint64_t mapped_hash(const int16_t* map) const;

    void analyze(GroupInfo& g) const;
    // Empty, not the ko point, not suicide (needs analyze() of this position).
    bool legal(const GroupInfo& g, int color, int v) const;
    bool legal_slow(int color, int v) const;

    // Plays for the side to move; `move` must be legal or kPass.
    void play(int move);
    // True when the stones now on the board repeat an earlier position.
    bool superko() const;
    // Black minus white area (stones plus empty points reached only through
    // empty points), minus komi.
    float area_score(float komi) const;

private:
    bool has_liberty(int v) const;
    int remove_group(int v, int* last_removed);

    Stones m_sq;
    int m_to_move = BLACK;
    int m_ko = -1;
    int m_passes = 0;
    int m_movenum = 0;
    uint64_t m_stone_hash = 0;
    std::array<Stones, kHistory> m_hist;
    int m_hist_head = 0;
    std::vector<uint64_t> m_seen;  // stone hashes of all earlier positions
};

}  // namespace go
}  // namespace lzhip
#endif
