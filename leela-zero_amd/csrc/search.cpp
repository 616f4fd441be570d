// Search-side caller of the backend; search.h lists which part of the
// reference each piece stands for.
#include "search.h"

#include <algorithm>
#include <chrono>
#include <cmath>
#include <cstring>
#include <limits>
#include <stdexcept>
#include <thread>

namespace lzhip {

using go::kPass;
using go::kPoints;
using go::kSize;

// ---------------------------------------------------------------------------
// symmetries and input planes
// ---------------------------------------------------------------------------

namespace {

struct SymTable {
    int16_t idx[8][kPoints];
    SymTable() {
        for (int s = 0; s < 8; s++)
            for (int v = 0; v < kPoints; v++) {
                int x = v % kSize, y = v / kSize;
                if (s & 4) std::swap(x, y);
                if (s & 2) x = kSize - 1 - x;
                if (s & 1) y = kSize - 1 - y;
                idx[s][v] = (int16_t)(y * kSize + x);
            }
    }
};

const SymTable& sym_table() {
    static const SymTable t;
    return t;
}

uint64_t next_rand(uint64_t& s) {
    // xorshift64*
    s ^= s >> 12;
    s ^= s << 25;
    s ^= s >> 27;
    return s * 0x2545F4914F6CDD1Dull;
}

}  // namespace

int symmetry_index(int symmetry, int idx) {
    if (symmetry < 0 || symmetry >= 8 || idx < 0 || idx >= kPoints) return -1;
    return sym_table().idx[symmetry][idx];
}

void gather_features(const uint8_t* const* boards, int n_boards, int to_move, int symmetry,
                     float* out) {
    std::memset(out, 0, sizeof(float) * LZHIP_INPUT_SIZE);
    const int16_t* map = sym_table().idx[symmetry];
    const int n = std::min(n_boards, go::kHistory);
    float* own = out;
    float* opp = out + go::kHistory * kPoints;
    for (int h = 0; h < n; h++) {
        const uint8_t* b = boards[h];
        float* o = own + h * kPoints;
        float* p = opp + h * kPoints;
        for (int i = 0; i < kPoints; i++) {
            const uint8_t c = b[map[i]];
            if (c == to_move) o[i] = 1.0f;
            else if (c == (to_move ^ 1)) p[i] = 1.0f;
        }
    }
    float* stm = out + (2 * go::kHistory + (to_move == go::BLACK ? 0 : 1)) * kPoints;
    for (int i = 0; i < kPoints; i++) stm[i] = 1.0f;
}

void gather_features(const go::Position& pos, int symmetry, float* out) {
    const uint8_t* boards[go::kHistory];
    const int n = std::min(pos.movenum() + 1, go::kHistory);
    for (int h = 0; h < n; h++) boards[h] = pos.past(h).data();
    gather_features(boards, n, pos.to_move(), symmetry, out);
}

// ---------------------------------------------------------------------------
// heads on the calling thread
// ---------------------------------------------------------------------------

HeadWeights::HeadWeights(const lzhip_head_weights& w) {
    for (int c = 0; c < 2; c++) {
        bn_pol_mean[c] = w.bn_pol_mean[c];
        bn_pol_scale[c] = w.bn_pol_scale[c];
    }
    bn_val_mean = w.bn_val_mean[0];
    bn_val_scale = w.bn_val_scale[0];
    const int pin = 2 * kPoints, pout = kPoints + 1;
    ip_pol_wt.resize((size_t)pin * pout);
    for (int o = 0; o < pout; o++)
        for (int i = 0; i < pin; i++) ip_pol_wt[(size_t)i * pout + o] = w.ip_pol_w[(size_t)o * pin + i];
    ip_pol_b.assign(w.ip_pol_b, w.ip_pol_b + pout);
    ip1_val_wt.resize((size_t)kPoints * 256);
    for (int o = 0; o < 256; o++)
        for (int i = 0; i < kPoints; i++) ip1_val_wt[(size_t)i * 256 + o] = w.ip1_val_w[(size_t)o * kPoints + i];
    ip1_val_b.assign(w.ip1_val_b, w.ip1_val_b + 256);
    ip2_val_w.assign(w.ip2_val_w, w.ip2_val_w + 256);
    ip2_val_b = w.ip2_val_b[0];
}

void heads_on_host(const HeadWeights& w, const float* pol, const float* val, float softmax_temp,
                   float* policy, float* winrate) {
    constexpr int pout = kPoints + 1;
    float logits[pout];
    for (int o = 0; o < pout; o++) logits[o] = w.ip_pol_b[o];
    for (int c = 0; c < 2; c++)
        for (int i = 0; i < kPoints; i++) {
            const float x = w.bn_pol_scale[c] * (pol[c * kPoints + i] - w.bn_pol_mean[c]);
            if (x <= 0.0f) continue;
            const float* row = &w.ip_pol_wt[(size_t)(c * kPoints + i) * pout];
            for (int o = 0; o < pout; o++) logits[o] += x * row[o];
        }
    float alpha = logits[0];
    for (int o = 1; o < pout; o++) alpha = std::max(alpha, logits[o]);
    float denom = 0.0f;
    for (int o = 0; o < pout; o++) {
        policy[o] = std::exp((logits[o] - alpha) / softmax_temp);
        denom += policy[o];
    }
    for (int o = 0; o < pout; o++) policy[o] /= denom;

    float hid[256];
    for (int o = 0; o < 256; o++) hid[o] = w.ip1_val_b[o];
    for (int i = 0; i < kPoints; i++) {
        const float x = w.bn_val_scale * (val[i] - w.bn_val_mean);
        if (x <= 0.0f) continue;
        const float* row = &w.ip1_val_wt[(size_t)i * 256];
        for (int o = 0; o < 256; o++) hid[o] += x * row[o];
    }
    float out = w.ip2_val_b;
    for (int o = 0; o < 256; o++) out += std::max(hid[o], 0.0f) * w.ip2_val_w[o];
    *winrate = (1.0f + std::tanh(out)) / 2.0f;
}

// ---------------------------------------------------------------------------
// evaluation cache
// ---------------------------------------------------------------------------

bool EvalCache::lookup(uint64_t hash, Netresult& out) {
    std::lock_guard<std::mutex> lk(m_mutex);
    m_lookups++;
    auto it = m_map.find(hash);
    if (it == m_map.end()) return false;
    m_hits++;
    out = *it->second;
    return true;
}

void EvalCache::insert(uint64_t hash, const Netresult& r) {
    if (m_size == 0) return;
    std::lock_guard<std::mutex> lk(m_mutex);
    if (m_map.find(hash) != m_map.end()) return;
    m_map.emplace(hash, std::make_unique<const Netresult>(r));
    m_order.push_back(hash);
    if (m_order.size() > m_size) {
        m_map.erase(m_order.front());
        m_order.pop_front();
    }
}

void EvalCache::clear() {
    std::lock_guard<std::mutex> lk(m_mutex);
    m_map.clear();
    m_order.clear();
}

// ---------------------------------------------------------------------------
// network facade
// ---------------------------------------------------------------------------

NetworkFacade::NetworkFacade(ForwardPipe& pipe, std::shared_ptr<const HeadWeights> heads,
                             size_t cache_size, float softmax_temp)
    : m_pipe(pipe), m_heads(std::move(heads)), m_cache(cache_size), m_temp(softmax_temp) {}

void NetworkFacade::set_device_heads(bool on) {
    m_sched_heads = nullptr;
    if (!on) return;
    m_sched_heads = dynamic_cast<HIPScheduler*>(&m_pipe);
    if (!m_sched_heads) throw std::invalid_argument("device heads need a HIPScheduler backend");
}

Netresult NetworkFacade::get_output_internal(const go::Position& pos, int symmetry) {
    thread_local std::vector<float> in(LZHIP_INPUT_SIZE), pol(LZHIP_POL_SIZE), val(LZHIP_VAL_SIZE);
    gather_features(pos, symmetry, in.data());
    m_evals++;
    float policy[kPoints + 1], winrate;
    if (m_sched_heads) {
        float value;
        if (m_sched_heads->evaluate_raw(in.data(), m_temp, policy, &value) == LZHIP_EHALT)
            throw NetworkHaltException();
        winrate = (1.0f + value) / 2.0f;
    } else {
        m_pipe.forward(in, pol, val);  // may throw NetworkHaltException
        heads_on_host(*m_heads, pol.data(), val.data(), m_temp, policy, &winrate);
    }
    Netresult r;
    const int16_t* map = sym_table().idx[symmetry];
    for (int i = 0; i < kPoints; i++) r.policy[map[i]] = policy[i];
    r.policy_pass = policy[kPoints];
    r.winrate = winrate;
    return r;
}

bool NetworkFacade::probe_cache(const go::Position& pos, Netresult& out) {
    if (m_cache.lookup(pos.hash(), out)) return true;
    // opening_moves(19) / 2 = (361 / 6) / 2 (reference src/TimeControl.cpp:300-304)
    if (!m_symmetry_probe || pos.movenum() >= (kPoints / 6) / 2) return false;
    for (int sym = 1; sym < 8; sym++) {
        const int16_t* map = sym_table().idx[sym];
        Netresult cached;
        if (m_cache.lookup(pos.mapped_hash(map), cached)) {
            for (int i = 0; i < kPoints; i++) out.policy[i] = cached.policy[map[i]];
            out.policy_pass = cached.policy_pass;
            out.winrate = cached.winrate;
            return true;
        }
    }
    return false;
}

Netresult NetworkFacade::get_output(const go::Position& pos, int symmetry, uint64_t& rng_state,
                                    bool use_cache) {
    Netresult r;
    const uint64_t key = pos.hash();
    if (use_cache) {
        m_probes++;
        if (probe_cache(pos, r)) {
            m_probe_hits++;
            return r;
        }
    }
    if (symmetry < 0) symmetry = (int)(next_rand(rng_state) >> 61);
    r = get_output_internal(pos, symmetry);
    if (m_value_not_stm && pos.to_move() == go::WHITE) r.winrate = 1.0f - r.winrate;
    if (use_cache) m_cache.insert(key, r);
    return r;
}

// ---------------------------------------------------------------------------
// tree
// ---------------------------------------------------------------------------

enum : uint8_t { ST_INITIAL = 0, ST_EXPANDING = 1, ST_EXPANDED = 2 };

struct Child {
    std::atomic<Node*> node{nullptr};
    float prior = 0.0f;
    int16_t move = 0;
    std::atomic<bool> valid{true};
};

struct Node {
    std::atomic<int> visits{0};
    std::atomic<int> vloss{0};
    std::atomic<double> blackevals{0.0};
    std::atomic<uint8_t> state{ST_INITIAL};
    float net_eval = 0.0f;
    std::unique_ptr<Child[]> children;
    int n_children = 0;

    void update(float eval) {
        visits.fetch_add(1);
        double cur = blackevals.load();
        while (!blackevals.compare_exchange_weak(cur, cur + (double)eval)) {
        }
    }
    // Mean value for `tomove` with `vl` pending visits counted as losses.
    float raw_eval(int tomove, int vl) const {
        return puct_eval_for(tomove, blackevals.load(), visits.load(), vl);
    }
    bool expanded() const { return state.load(std::memory_order_acquire) == ST_EXPANDED; }
};

float puct_eval_for(int tomove, double blackevals, int visits, int virtual_loss) {
    const int v = visits + virtual_loss;
    double be = blackevals;
    if (tomove == go::WHITE) be += (double)virtual_loss;
    float e = v > 0 ? (float)(be / (double)v) : 0.5f;
    if (tomove == go::WHITE) e = 1.0f - e;
    return e;
}

PuctParent puct_parent(const lzhip_search_config& cfg, bool is_root, size_t children_visits,
                       float visited_policy, float parent_eval_for_color) {
    PuctParent p;
    p.numerator = std::sqrt((double)children_visits *
                            std::log((double)cfg.logpuct * (double)children_visits +
                                     (double)cfg.logconst));
    p.fpu_reduction =
        (is_root ? cfg.fpu_root_reduction : cfg.fpu_reduction) * std::sqrt(visited_policy);
    p.fpu_eval = parent_eval_for_color - p.fpu_reduction;
    return p;
}

double puct_value(const lzhip_search_config& cfg, const PuctParent& parent, float prior,
                  int visits, bool expanding, float child_eval_for_color) {
    float winrate = parent.fpu_eval;
    if (expanding)
        winrate = -1.0f - parent.fpu_reduction;  // someone is waiting for its evaluation
    else if (visits > 0)
        winrate = child_eval_for_color;
    const double puct =
        (double)cfg.puct * (double)prior * (parent.numerator / (1.0 + (double)visits));
    return (double)winrate + puct;
}

static void free_tree(Node* n) {
    if (!n) return;
    for (int i = 0; i < n->n_children; i++) free_tree(n->children[i].node.load());
    delete n;
}

namespace {
struct VirtualLoss {
    Node* n;
    int k;
    VirtualLoss(Node* node, int count) : n(node), k(count) { n->vloss.fetch_add(k); }
    ~VirtualLoss() { n->vloss.fetch_sub(k); }
};
}  // namespace

UCTSearch::UCTSearch(NetworkFacade& net, const lzhip_search_config& cfg)
    : m_net(net), m_cfg(cfg), m_seed(cfg.seed * 0x9E3779B97F4A7C15ull + 0x1234567ull) {
    if (cfg.threads < 1 || cfg.visits < 1 || cfg.virtual_loss < 0)
        throw std::invalid_argument("search config: threads, visits >= 1, virtual_loss >= 0");
}

UCTSearch::~UCTSearch() {
    {
        std::lock_guard<std::mutex> lk(m_pool_mu);
        m_quit = true;
    }
    m_pool_cv.notify_all();
    for (auto& th : m_pool) th.join();
    if (m_reaper.joinable()) m_reaper.join();
    free_tree(m_root);
}

// Search threads live as long as the search object: every move wakes them with
// a new generation number instead of creating them again.
void UCTSearch::pool_thread() {
    uint64_t seen = 0;
    std::unique_lock<std::mutex> lk(m_pool_mu);
    for (;;) {
        m_pool_cv.wait(lk, [&] { return m_quit || m_generation != seen; });
        if (m_quit) return;
        seen = m_generation;
        const go::Position* root = m_root_pos;
        const uint64_t seed = next_rand(m_seed);
        lk.unlock();
        worker(root, seed);
        lk.lock();
        if (--m_active == 0) m_done_cv.notify_all();
    }
}

int UCTSearch::root_visits() const { return m_root ? m_root->visits.load() : 0; }

std::vector<std::pair<int, int>> UCTSearch::root_children() const {
    std::vector<std::pair<int, int>> out;
    if (!m_root || !m_root->expanded()) return out;
    for (int i = 0; i < m_root->n_children; i++) {
        const Child& c = m_root->children[i];
        Node* n = c.node.load();
        out.emplace_back((int)c.move, (n && c.valid.load()) ? n->visits.load() : 0);
    }
    return out;
}

std::vector<std::pair<int, float>> UCTSearch::root_priors() const {
    std::vector<std::pair<int, float>> out;
    if (!m_root || !m_root->expanded()) return out;
    for (int i = 0; i < m_root->n_children; i++)
        out.emplace_back((int)m_root->children[i].move, m_root->children[i].prior);
    return out;
}

static void check_node(const Node* n, bool terminal_ok, UCTSearch::TreeCheck& c) {
    c.nodes++;
    c.virtual_loss += n->vloss.load();
    if (n->state.load() == ST_EXPANDING) c.expanding++;
    if (n->state.load() != ST_EXPANDED) return;
    long sum = 0;
    for (int i = 0; i < n->n_children; i++) {
        const Node* ch = n->children[i].node.load();
        if (!ch) continue;
        sum += ch->visits.load();
        check_node(ch, terminal_ok, c);
    }
    if (n->visits.load() != 1 + sum) c.visit_mismatch++;
}

UCTSearch::TreeCheck UCTSearch::check_tree() const {
    TreeCheck c;
    if (m_root) check_node(m_root, true, c);
    return c;
}

bool UCTSearch::create_children(Node* node, const go::Position& pos, float& eval, uint64_t& rng) {
    if (pos.passes() >= 2) return false;
    uint8_t expected = ST_INITIAL;
    if (!node->state.compare_exchange_strong(expected, ST_EXPANDING)) return false;

    Netresult net;
    try {
        net = m_net.get_output(pos, -1, rng);
    } catch (...) {
        node->state.store(ST_INITIAL, std::memory_order_release);  // expansion cancelled
        throw;
    }

    const int to_move = pos.to_move();
    const float stm_eval = net.winrate;
    node->net_eval = (to_move == go::WHITE) ? 1.0f - stm_eval : stm_eval;
    eval = node->net_eval;

    go::GroupInfo groups;
    pos.analyze(groups);
    std::vector<std::pair<float, int>> list;
    list.reserve(kPoints + 1);
    float legal_sum = 0.0f;
    for (int v = 0; v < kPoints; v++)
        if (pos.legal(groups, to_move, v)) {
            list.emplace_back(net.policy[v], v);
            legal_sum += net.policy[v];
        }
    // Passing is offered when few points are left, or when the side to move is
    // far ahead by the network and not behind on the board.
    bool allow_pass = (int)list.size() <= std::max(5, kSize);
    if (!allow_pass && stm_eval > 0.8f) {
        const float rel = (to_move == go::BLACK ? 1.0f : -1.0f) * pos.area_score(m_cfg.komi);
        if (rel >= 0.0f) allow_pass = true;
    }
    if (allow_pass) {
        list.emplace_back(net.policy_pass, kPass);
        legal_sum += net.policy_pass;
    }
    if (legal_sum > std::numeric_limits<float>::min()) {
        for (auto& e : list) e.first /= legal_sum;
    } else {
        const float u = 1.0f / (float)list.size();
        for (auto& e : list) e.first = u;
    }
    std::stable_sort(list.rbegin(), list.rend());

    node->n_children = (int)list.size();
    node->children.reset(new Child[list.size()]);
    for (size_t i = 0; i < list.size(); i++) {
        node->children[i].prior = list[i].first;
        node->children[i].move = (int16_t)list[i].second;
    }
    m_nodes += list.size();
    if (node->visits.load() == 0) node->update(eval);
    node->state.store(ST_EXPANDED, std::memory_order_release);
    return true;
}

Child* UCTSearch::select_child(Node* node, int color, bool is_root) {
    float total_visited_policy = 0.0f;
    size_t parentvisits = 0;
    for (int i = 0; i < node->n_children; i++) {
        const Child& c = node->children[i];
        if (!c.valid.load(std::memory_order_relaxed)) continue;
        Node* n = c.node.load(std::memory_order_acquire);
        const int v = n ? n->visits.load(std::memory_order_relaxed) : 0;
        parentvisits += (size_t)v;
        if (v > 0) total_visited_policy += c.prior;
    }
    const PuctParent parent =
        puct_parent(m_cfg, is_root, parentvisits, total_visited_policy, node->raw_eval(color, 0));

    Child* best = nullptr;
    double best_value = std::numeric_limits<double>::lowest();
    for (int i = 0; i < node->n_children; i++) {
        Child& c = node->children[i];
        if (!c.valid.load(std::memory_order_relaxed)) continue;
        Node* n = c.node.load(std::memory_order_acquire);
        const int v = n ? n->visits.load(std::memory_order_relaxed) : 0;
        const bool expanding = n && n->state.load(std::memory_order_relaxed) == ST_EXPANDING;
        const float child_eval =
            (v > 0 && !expanding) ? n->raw_eval(color, n->vloss.load(std::memory_order_relaxed))
                                  : 0.0f;
        const double value = puct_value(m_cfg, parent, c.prior, v, expanding, child_eval);
        if (value > best_value) {
            best_value = value;
            best = &c;
        }
    }
    if (!best) return nullptr;
    Node* n = best->node.load(std::memory_order_acquire);
    if (!n) {
        Node* fresh = new Node();
        if (!best->node.compare_exchange_strong(n, fresh, std::memory_order_acq_rel))
            delete fresh;  // another thread created it first
    }
    return best;
}

UCTSearch::Result UCTSearch::play_simulation(go::Position& pos, Node* node, bool is_root,
                                             uint64_t& rng) {
    const int color = pos.to_move();
    Result result;
    bool new_node = false;
    VirtualLoss guard(node, m_cfg.virtual_loss);

    if (!node->expanded()) {
        if (pos.passes() >= 2) {
            const float score = pos.area_score(m_cfg.komi);
            result.valid = true;
            result.eval = score > 0.0f ? 1.0f : (score < 0.0f ? 0.0f : 0.5f);
        } else {
            float eval = 0.0f;
            if (create_children(node, pos, eval, rng)) {
                result.valid = true;
                result.eval = eval;
                new_node = true;
            }
        }
    }

    if (node->expanded() && !result.valid) {
        Child* picked = select_child(node, color, is_root);
        if (picked) {
            Node* next = picked->node.load(std::memory_order_acquire);
            pos.play(picked->move);
            if (picked->move != kPass && pos.superko()) {
                picked->valid.store(false);
            } else {
                result = play_simulation(pos, next, false, rng);
            }
        }
    }

    if (result.valid && !new_node) node->update(result.eval);
    return result;
}

void UCTSearch::worker(const go::Position* root, uint64_t seed) {
    uint64_t rng = seed | 1;
    try {
        while (m_run.load(std::memory_order_relaxed) &&
               m_root->visits.load(std::memory_order_relaxed) < m_cfg.visits) {
            go::Position pos = *root;
            const Result r = play_simulation(pos, m_root, true, rng);
            if (r.valid) m_playouts++;
            else m_wasted++;
        }
    } catch (const NetworkHaltException&) {
        m_halted++;
    } catch (const std::exception& e) {
        std::lock_guard<std::mutex> lk(m_fail_mutex);
        if (m_failure.empty()) m_failure = e.what()[0] ? e.what() : "search thread failed";
        m_failed = true;
    }
}

int UCTSearch::think(const go::Position& root) {
    if (!m_root) m_root = new Node();
    uint64_t rng = next_rand(m_seed) | 1;
    if (!m_root->expanded() && root.passes() < 2) {
        float eval;
        create_children(m_root, root, eval, rng);
    }
    if (!m_root->expanded() || m_root->n_children == 0) return kPass;

    if (m_root->visits.load() < m_cfg.visits) {
        m_run = true;
        {
            std::lock_guard<std::mutex> lk(m_pool_mu);
            m_root_pos = &root;
            m_active = m_cfg.threads;
            m_generation++;
            while ((int)m_pool.size() < m_cfg.threads)
                m_pool.emplace_back(&UCTSearch::pool_thread, this);
        }
        m_pool_cv.notify_all();
        // A position in which no simulation can end with a value (every child
        // ruled out by superko) must not spin forever.
        const uint64_t wasted_limit = m_wasted.load() + 1000ull * (uint64_t)m_cfg.visits;
        while (m_root->visits.load(std::memory_order_relaxed) < m_cfg.visits && !m_failed.load() &&
               m_wasted.load(std::memory_order_relaxed) < wasted_limit)
            std::this_thread::sleep_for(std::chrono::microseconds(50));
        // Stop: no new simulations, requests still waiting in the backend are
        // released with a halt, and the backend is re-opened once all threads
        // are out.
        m_run = false;
        m_net.drain();
        {
            std::unique_lock<std::mutex> lk(m_pool_mu);
            m_done_cv.wait(lk, [&] { return m_active == 0; });
        }
        m_net.resume();
        if (m_failed.load()) throw std::runtime_error(m_failure);
    }

    m_stats.playouts = m_playouts.load();
    m_stats.wasted = m_wasted.load();
    m_stats.halted = m_halted.load();
    m_stats.nodes = m_nodes.load();

    // Most visited child; before cfg.random_moves, in proportion to visits.
    int best = -1, best_visits = -1;
    uint64_t total = 0;
    for (int i = 0; i < m_root->n_children; i++) {
        const Child& c = m_root->children[i];
        Node* n = c.node.load();
        const int v = (n && c.valid.load()) ? n->visits.load() : 0;
        total += (uint64_t)v;
        if (v > best_visits) {
            best_visits = v;
            best = i;
        }
    }
    if (root.movenum() < m_cfg.random_moves && total > 0) {
        uint64_t pick = next_rand(rng) % total;
        for (int i = 0; i < m_root->n_children; i++) {
            const Child& c = m_root->children[i];
            Node* n = c.node.load();
            const uint64_t v = (n && c.valid.load()) ? (uint64_t)n->visits.load() : 0;
            if (pick < v) {
                best = i;
                break;
            }
            pick -= v;
        }
    }
    return best >= 0 ? (int)m_root->children[best].move : kPass;
}

void UCTSearch::advance(int move) {
    Node* keep = nullptr;
    if (m_root && m_cfg.reuse_tree && m_root->expanded()) {
        for (int i = 0; i < m_root->n_children; i++) {
            Child& c = m_root->children[i];
            if (c.move == move && c.valid.load()) {
                keep = c.node.exchange(nullptr);
                break;
            }
        }
    }
    // The discarded part of the tree is freed while the next search is already running.
    if (m_reaper.joinable()) m_reaper.join();
    Node* old = m_root;
    m_root = keep;
    if (old) m_reaper = std::thread([old] { free_tree(old); });
}

// ---------------------------------------------------------------------------
// self-play driver
// ---------------------------------------------------------------------------

void selfplay(ForwardPipe& pipe, std::shared_ptr<const HeadWeights> heads,
              const lzhip_search_config& cfg, lzhip_search_result& out, int* moves, int moves_cap,
              bool value_head_not_stm) {
    std::memset(&out, 0, sizeof(out));
    auto* sched = dynamic_cast<HIPScheduler*>(&pipe);
    lzhip_stats before{};
    if (sched) before = sched->stats();

    NetworkFacade net(pipe, std::move(heads), (size_t)std::max(cfg.cache_size, 0), cfg.softmax_temp);
    net.set_symmetry_probe(cfg.random_moves == 0);  // as the reference: not in randomised self-play
    net.set_device_heads(cfg.device_heads != 0);
    net.set_value_head_not_stm(value_head_not_stm);
    UCTSearch search(net, cfg);
    go::Position pos;
    const auto t0 = std::chrono::steady_clock::now();
    int played = 0;
    for (; played < cfg.moves && pos.passes() < 2; played++) {
        const int mv = search.think(pos);
        pos.play(mv);
        search.advance(mv);
        if (moves && played < moves_cap) moves[played] = mv;
    }
    const auto t1 = std::chrono::steady_clock::now();

    const SearchStats& st = search.stats();
    out.playouts = st.playouts;
    out.wasted = st.wasted;
    out.halted = st.halted;
    out.nodes = st.nodes;
    out.evals = net.evals();
    out.cache_lookups = net.cache_lookups();
    out.cache_hits = net.cache_hits();
    out.seconds = std::chrono::duration<double>(t1 - t0).count();
    out.visits_per_s = out.seconds > 0 ? (double)out.playouts / out.seconds : 0.0;
    out.moves_played = played;
    out.passes_at_end = pos.passes();
    out.final_score = pos.area_score(cfg.komi);
    if (sched) {
        const lzhip_stats after = sched->stats();
        out.sched.requests = after.requests - before.requests;
        out.sched.batches = after.batches - before.batches;
        out.sched.batch_slots = after.batch_slots - before.batch_slots;
        out.sched.halted = after.halted - before.halted;
        out.sched.max_batch_seen = after.max_batch_seen;
        out.sched.max_batch = after.max_batch;
    }
}

}  // namespace lzhip
