// Search-side caller of the network backend: the pieces of the engine that sit
// directly above ForwardPipe::forward, rebuilt so that the call pattern of a
// real search (many threads, one blocking single-position request each, halt at
// the end of every move) can be driven and measured against the HIP backend.
//
//   input planes + symmetries   Network::gather_features / get_symmetry
//                               (reference src/Network.cpp:913-993, :518-531)
//   heads on the calling thread Network::get_output_internal (:811-864)
//   evaluation cache            NNCache (src/NNCache.cpp:47-80)
//   get_output                  Network::get_output (:744-809), RANDOM_SYMMETRY
//   tree search                 UCTSearch::play_simulation (src/UCTSearch.cpp:237-286),
//                               UCTNode::create_children / uct_select_child /
//                               update / get_raw_eval (src/UCTNode.cpp:62-155,
//                               :306-362, :207-218, :270-282), virtual loss 3
//                               (src/UCTNode.h:51), halt at stop
//                               (src/UCTSearch.cpp:828-832)
//
// Not rebuilt: time management, LCB move choice, Dirichlet noise, pondering,
// GTP, SGF, training output.
#ifndef LZHIP_SEARCH_H_INCLUDED
#define LZHIP_SEARCH_H_INCLUDED

#include <array>
#include <atomic>
#include <condition_variable>
#include <cstdint>
#include <deque>
#include <memory>
#include <mutex>
#include <string>
#include <thread>
#include <unordered_map>
#include <vector>

#include "forward_pipe.h"
#include "goboard.h"
#include "lzhip_search.h"

namespace lzhip {

// symmetry_index(s, idx): the board index that NN index `idx` reads under
// symmetry s (reference symmetry_nn_idx_table, src/Network.cpp:518-531).
int symmetry_index(int symmetry, int idx);

// boards: n_boards stone arrays, newest first, values go::BLACK/WHITE/EMPTY.
void gather_features(const uint8_t* const* boards, int n_boards, int to_move, int symmetry,
                     float* out /* [18][361] */);
void gather_features(const go::Position& pos, int symmetry, float* out);

struct Netresult {
    std::array<float, go::kPoints> policy{};
    float policy_pass = 0.0f;
    float winrate = 0.0f;
};

// Head parameters, laid out for the host loops (FC weights input-major).
struct HeadWeights {
    explicit HeadWeights(const lzhip_head_weights& w);
    float bn_pol_mean[2], bn_pol_scale[2], bn_val_mean, bn_val_scale;
    std::vector<float> ip_pol_wt;   // [722][362]
    std::vector<float> ip_pol_b;    // [362]
    std::vector<float> ip1_val_wt;  // [361][256]
    std::vector<float> ip1_val_b;   // [256]
    std::vector<float> ip2_val_w;   // [256]
    float ip2_val_b;
};

// BN+ReLU, FC, softmax / FC, ReLU, FC, tanh on raw head planes; policy comes
// back in NN index order (no symmetry un-rotation).
void heads_on_host(const HeadWeights& w, const float* pol /*[2][361]*/,
                   const float* val /*[361]*/, float softmax_temp, float* policy /*[362]*/,
                   float* winrate);

class EvalCache {
public:
    explicit EvalCache(size_t size) : m_size(size) {}
    bool lookup(uint64_t hash, Netresult& out);
    void insert(uint64_t hash, const Netresult& r);
    void clear();
    uint64_t lookups() const { return m_lookups; }
    uint64_t hits() const { return m_hits; }

private:
    std::mutex m_mutex;
    size_t m_size;
    std::unordered_map<uint64_t, std::unique_ptr<const Netresult>> m_map;
    std::deque<uint64_t> m_order;
    uint64_t m_lookups = 0, m_hits = 0;
};

// The slice of `Network` the search needs.
class NetworkFacade {
public:
    NetworkFacade(ForwardPipe& pipe, std::shared_ptr<const HeadWeights> heads, size_t cache_size,
                  float softmax_temp);
    NetworkFacade(ForwardPipe& pipe, const lzhip_head_weights& heads, size_t cache_size,
                  float softmax_temp)
        : NetworkFacade(pipe, std::make_shared<const HeadWeights>(heads), cache_size, softmax_temp) {}
    // symmetry in 0..7, or -1 for a random one drawn from `rng_state`.
    Netresult get_output(const go::Position& pos, int symmetry, uint64_t& rng_state,
                         bool use_cache = true);
    Netresult get_output_internal(const go::Position& pos, int symmetry);
    // Cache lookup as Network::probe_cache (reference src/Network.cpp:717-742):
    // the position itself, then, during the first 30 moves and when enabled,
    // its seven symmetric images (their cached policy is mapped back).
    bool probe_cache(const go::Position& pos, Netresult& out);
    void set_symmetry_probe(bool on) { m_symmetry_probe = on; }
    // Let the backend compute the heads (the pipe must be a HIPScheduler whose
    // executor has them); the calling thread then only gathers planes and
    // rotates the policy back.
    void set_device_heads(bool on);
    // Networks of file format 2 give the value for black, not for the side to move
    // (reference src/Network.cpp:395-400, :797-802): get_output then turns it round
    // when white is to move.
    void set_value_head_not_stm(bool on) { m_value_not_stm = on; }
    void drain() { m_pipe.drain(); }
    void resume() { m_pipe.resume(); }
    EvalCache& cache() { return m_cache; }
    uint64_t evals() const { return m_evals.load(); }
    // get_output calls that consulted the cache, and those it answered
    // (directly or through a symmetric image).
    uint64_t cache_lookups() const { return m_probes.load(); }
    uint64_t cache_hits() const { return m_probe_hits.load(); }

private:
    ForwardPipe& m_pipe;
    std::shared_ptr<const HeadWeights> m_heads;
    EvalCache m_cache;
    float m_temp;
    bool m_symmetry_probe = true;
    bool m_value_not_stm = false;
    HIPScheduler* m_sched_heads = nullptr;   // set when the backend computes the heads
    std::atomic<uint64_t> m_evals{0}, m_probes{0}, m_probe_hits{0};
};

struct SearchStats {
    uint64_t playouts = 0;      // simulations that ended with a value
    uint64_t wasted = 0;        // simulations that ran into a node under expansion
    uint64_t halted = 0;        // simulations cut short by the halt at stop
    uint64_t nodes = 0;
};

struct Node;
struct Child;

// The arithmetic of child selection on plain numbers, as UCTNode::uct_select_child and
// UCTNode::get_raw_eval do it (reference src/UCTNode.cpp:306-362, :270-282); the tree code
// below calls exactly these, and the host tests pin them on hand-worked nodes.
//
// Mean value of a node for `tomove` with `virtual_loss` visits in progress counted as
// lost: blackevals / (visits + vl) for black; for white the pending visits count as black
// wins before the value is turned round.  0.5 for a node without visits.
float puct_eval_for(int tomove, double blackevals, int visits, int virtual_loss);
// What the parent contributes: the exploration numerator sqrt(N ln(logpuct N + logconst))
// over the children's visits N, and the value given to children without visits, the
// parent's own mean for the side to move less fpu_reduction * sqrt(priors of the visited)
// (fpu_root_reduction when the parent is the root, reference src/UCTNode.cpp:322-324).
struct PuctParent {
    double numerator;
    float fpu_reduction;
    float fpu_eval;
};
PuctParent puct_parent(const lzhip_search_config& cfg, bool is_root, size_t children_visits,
                       float visited_policy, float parent_eval_for_color);
// Selection value of one child: its mean (fpu_eval without visits, -1 - fpu_reduction
// while another thread expands it) + puct * prior * numerator / (1 + visits).
double puct_value(const lzhip_search_config& cfg, const PuctParent& parent, float prior,
                  int visits, bool expanding, float child_eval_for_color);

class UCTSearch {
public:
    UCTSearch(NetworkFacade& net, const lzhip_search_config& cfg);
    ~UCTSearch();
    // Searches from `root` until its visit count reaches cfg.visits and returns
    // the chosen move (most visited child).
    int think(const go::Position& root);
    // Moves the tree to the position after `move` (keeps that subtree when
    // cfg.reuse_tree is set).
    void advance(int move);
    const SearchStats& stats() const { return m_stats; }
    int root_visits() const;
    // (move, visits) of the root's children after think().
    std::vector<std::pair<int, int>> root_children() const;
    // (move, prior) of the root's children, best first.
    std::vector<std::pair<int, float>> root_priors() const;
    // Consistency of the idle tree: pending virtual losses and nodes left in
    // the expanding state (both must be 0), and whether every expanded node
    // holds visits == 1 + sum of its children's visits.
    struct TreeCheck {
        long virtual_loss = 0;
        long expanding = 0;
        long visit_mismatch = 0;
        long nodes = 0;
    };
    TreeCheck check_tree() const;

private:
    struct Result {
        bool valid = false;
        float eval = 0.0f;
    };
    Result play_simulation(go::Position& pos, Node* node, bool is_root, uint64_t& rng);
    bool create_children(Node* node, const go::Position& pos, float& eval, uint64_t& rng);
    Child* select_child(Node* node, int color, bool is_root);
    void worker(const go::Position* root, uint64_t seed);
    void pool_thread();

    NetworkFacade& m_net;
    lzhip_search_config m_cfg;
    Node* m_root = nullptr;
    std::atomic<bool> m_run{false}, m_failed{false};
    std::mutex m_fail_mutex;
    std::string m_failure;
    std::atomic<uint64_t> m_playouts{0}, m_wasted{0}, m_halted{0}, m_nodes{0};
    SearchStats m_stats;
    uint64_t m_seed;
    // persistent search threads, woken once per move
    std::vector<std::thread> m_pool;
    std::mutex m_pool_mu;
    std::condition_variable m_pool_cv, m_done_cv;
    uint64_t m_generation = 0;
    int m_active = 0;
    bool m_quit = false;
    const go::Position* m_root_pos = nullptr;
    std::thread m_reaper;   // frees the part of the tree a move left behind
};

// Plays cfg.moves moves of self-play from the empty board; fills `out` and, if
// given, the move list.
void selfplay(ForwardPipe& pipe, std::shared_ptr<const HeadWeights> heads,
              const lzhip_search_config& cfg, lzhip_search_result& out, int* moves, int moves_cap,
              bool value_head_not_stm = false);
inline void selfplay(ForwardPipe& pipe, const lzhip_head_weights& heads,
                     const lzhip_search_config& cfg, lzhip_search_result& out, int* moves,
                     int moves_cap) {
    selfplay(pipe, std::make_shared<const HeadWeights>(heads), cfg, out, moves, moves_cap);
}

}  // namespace lzhip
#endif
