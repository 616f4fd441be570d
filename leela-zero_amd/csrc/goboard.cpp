// Go rules for the search driver; see goboard.h for what each call stands for
// in the reference.
#include "goboard.h"

#include <algorithm>

namespace lzhip {
namespace go {

static uint64_t splitmix64(uint64_t& s) {
    uint64_t z = (s += 0x9E3779B97F4A7C15ull);
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}

Tables::Tables() {
    for (int v = 0; v < kPoints; v++) {
        const int x = v % kSize, y = v / kSize;
        int n = 0;
        if (x > 0) nbr[v][n++] = (int16_t)(v - 1);
        if (x < kSize - 1) nbr[v][n++] = (int16_t)(v + 1);
        if (y > 0) nbr[v][n++] = (int16_t)(v - kSize);
        if (y < kSize - 1) nbr[v][n++] = (int16_t)(v + kSize);
        n_nbr[v] = (int8_t)n;
        for (; n < 4; n++) nbr[v][n] = -1;
    }
    uint64_t s = 0x6c7a686970ull;
    for (int c = 0; c < 2; c++)
        for (int v = 0; v < kPoints; v++) zob[c][v] = splitmix64(s);
    for (int v = 0; v <= kPoints; v++) zob_ko[v] = splitmix64(s);
    for (int p = 0; p < 4; p++) zob_pass[p] = splitmix64(s);
    zob_white_to_move = splitmix64(s);
}

const Tables& tables() {
    static const Tables t;
    return t;
}

Position::Position() {
    m_sq.fill(EMPTY);
    for (auto& h : m_hist) h.fill(EMPTY);
    m_seen.reserve(64);
}

uint64_t Position::hash() const {
    const Tables& t = tables();
    uint64_t h = m_stone_hash;
    if (m_to_move == WHITE) h ^= t.zob_white_to_move;
    h ^= t.zob_ko[m_ko < 0 ? kPoints : m_ko];
    h ^= t.zob_pass[std::min(m_passes, 3)];
    return h;
}

uint64_t Position::mapped_hash(const int16_t* map) const {
    const Tables& t = tables();
    uint64_t h = 0;
    for (int v = 0; v < kPoints; v++)
        if (m_sq[v] != EMPTY) h ^= t.zob[m_sq[v]][map[v]];
    if (m_to_move == WHITE) h ^= t.zob_white_to_move;
    h ^= t.zob_ko[m_ko < 0 ? kPoints : map[m_ko]];
    h ^= t.zob_pass[std::min(m_passes, 3)];
    return h;
}

void Position::analyze(GroupInfo& g) const {
    const Tables& t = tables();
    std::memset(g.id, 0xff, sizeof(g.id));
    int16_t lib_mark[kPoints];
    std::memset(lib_mark, 0xff, sizeof(lib_mark));
    int16_t stack[kPoints];
    g.n_groups = 0;
    for (int s = 0; s < kPoints; s++) {
        if (m_sq[s] == EMPTY || g.id[s] >= 0) continue;
        const int16_t gid = (int16_t)g.n_groups++;
        const uint8_t color = m_sq[s];
        int libs = 0, sp = 0;
        stack[sp++] = (int16_t)s;
        g.id[s] = gid;
        while (sp) {
            const int v = stack[--sp];
            for (int k = 0; k < t.n_nbr[v]; k++) {
                const int n = t.nbr[v][k];
                if (m_sq[n] == EMPTY) {
                    if (lib_mark[n] != gid) {
                        lib_mark[n] = gid;
                        libs++;
                    }
                } else if (m_sq[n] == color && g.id[n] < 0) {
                    g.id[n] = gid;
                    stack[sp++] = (int16_t)n;
                }
            }
        }
        g.libs[gid] = (int16_t)libs;
    }
}

bool Position::legal(const GroupInfo& g, int color, int v) const {
    if (v == kPass) return true;
    if (m_sq[v] != EMPTY || v == m_ko) return false;
    const Tables& t = tables();
    for (int k = 0; k < t.n_nbr[v]; k++) {
        const int n = t.nbr[v][k];
        if (m_sq[n] == EMPTY) return true;
        const int libs = g.libs[g.id[n]];
        if (m_sq[n] == color) {
            if (libs >= 2) return true;   // keeps a liberty besides v
        } else if (libs == 1) {
            return true;                  // captures that group
        }
    }
    return false;
}

bool Position::legal_slow(int color, int v) const {
    GroupInfo g;
    analyze(g);
    return legal(g, color, v);
}

bool Position::has_liberty(int v) const {
    const Tables& t = tables();
    const uint8_t color = m_sq[v];
    bool seen[kPoints] = {false};
    int16_t stack[kPoints];
    int sp = 0;
    stack[sp++] = (int16_t)v;
    seen[v] = true;
    while (sp) {
        const int p = stack[--sp];
        for (int k = 0; k < t.n_nbr[p]; k++) {
            const int n = t.nbr[p][k];
            if (m_sq[n] == EMPTY) return true;
            if (m_sq[n] == color && !seen[n]) {
                seen[n] = true;
                stack[sp++] = (int16_t)n;
            }
        }
    }
    return false;
}

int Position::remove_group(int v, int* last_removed) {
    const Tables& t = tables();
    const uint8_t color = m_sq[v];
    int16_t stack[kPoints];
    int sp = 0, removed = 0;
    stack[sp++] = (int16_t)v;
    m_sq[v] = EMPTY;
    while (sp) {
        const int p = stack[--sp];
        m_stone_hash ^= t.zob[color][p];
        removed++;
        *last_removed = p;
        for (int k = 0; k < t.n_nbr[p]; k++) {
            const int n = t.nbr[p][k];
            if (m_sq[n] == color) {
                m_sq[n] = EMPTY;
                stack[sp++] = (int16_t)n;
            }
        }
    }
    return removed;
}

void Position::play(int move) {
    const Tables& t = tables();
    m_seen.push_back(m_stone_hash);
    const int color = m_to_move;
    if (move == kPass) {
        m_passes++;
        m_ko = -1;
    } else {
        m_passes = 0;
        m_sq[move] = (uint8_t)color;
        m_stone_hash ^= t.zob[color][move];
        const uint8_t opp = (uint8_t)(color ^ 1);
        int captured = 0, cap_point = -1;
        bool lone = true;  // no friendly neighbour
        for (int k = 0; k < t.n_nbr[move]; k++) {
            const int n = t.nbr[move][k];
            if (m_sq[n] == opp) {
                if (!has_liberty(n)) captured += remove_group(n, &cap_point);
            } else if (m_sq[n] == color) {
                lone = false;
            }
        }
        // Simple ko: one stone taken by a lone stone that is left with exactly
        // the vacated point as its liberty.
        m_ko = -1;
        if (captured == 1 && lone) {
            int libs = 0;
            for (int k = 0; k < t.n_nbr[move]; k++)
                if (m_sq[t.nbr[move][k]] == EMPTY) libs++;
            if (libs == 1) m_ko = cap_point;
        }
        if (captured == 0 && !has_liberty(move)) {
            int dummy;
            remove_group(move, &dummy);  // only reachable with an illegal move
        }
    }
    m_to_move = color ^ 1;
    m_movenum++;
    m_hist_head = (m_hist_head + 1) % kHistory;
    m_hist[m_hist_head] = m_sq;
}

bool Position::superko() const {
    for (size_t i = 0; i < m_seen.size(); i++)
        if (m_seen[i] == m_stone_hash) return true;
    return false;
}

float Position::area_score(float komi) const {
    const Tables& t = tables();
    int reach[2] = {0, 0};
    for (int c = 0; c < 2; c++) {
        bool seen[kPoints] = {false};
        int16_t stack[kPoints];
        int sp = 0;
        for (int v = 0; v < kPoints; v++)
            if (m_sq[v] == c) {
                seen[v] = true;
                stack[sp++] = (int16_t)v;
                reach[c]++;
            }
        while (sp) {
            const int p = stack[--sp];
            for (int k = 0; k < t.n_nbr[p]; k++) {
                const int n = t.nbr[p][k];
                if (m_sq[n] == EMPTY && !seen[n]) {
                    seen[n] = true;
                    reach[c]++;
                    stack[sp++] = (int16_t)n;
                }
            }
        }
    }
    return (float)(reach[BLACK] - reach[WHITE]) - komi;
}

}  // namespace go
}  // namespace lzhip
