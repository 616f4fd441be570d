// Host-only test of the search driver against a stand-in executor behind the
// real batching scheduler; meant to be built plainly and with -fsanitize=thread.
// The stand-in "network" is equivariant under the eight board symmetries, so a
// wrong rotation or un-rotation of planes or policy shows up as a wrong prior.
//
// Checked, after the call pattern of the reference's search
// (src/UCTSearch.cpp:237-286, :757-850; src/UCTNode.cpp:62-155, :306-362):
//   * priors come back in board order for every symmetry;
//   * every move played is legal, visit budgets are met, and when the threads
//     have left no virtual loss or half-expanded node remains and every
//     expanded node holds 1 + the visits of its children;
//   * requests still queued at the end of a move are released by the halt and
//     the scheduler answers again afterwards;
//   * one thread with one seed plays the same game twice;
//   * the evaluation cache answers repeated positions, and in the opening also
//     the seven symmetric images of a cached position, with the policy mapped
//     back to the asking position's board order;
//   * a finished game (two passes) is not searched;
//   * with the heads computed behind the pipe (requests of that kind are batched
//     among themselves) the search plays the same single-thread game as with the
//     heads on the calling thread;
//   * an executor failure reaches the caller as an exception.
#include <atomic>
#include <chrono>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <stdexcept>
#include <thread>
#include <vector>

#include "forward_pipe.h"
#include "search.h"

using namespace lzhip;
using go::kPass;
using go::kPoints;

namespace lzhip {
std::unique_ptr<BatchExecutor> make_hip_pipe(int, int, int, int) {
    throw std::runtime_error("no device in the search test");
}
}  // namespace lzhip

#define CHECK(cond)                                                                 \
    do {                                                                            \
        if (!(cond)) {                                                              \
            std::fprintf(stderr, "FAILED %s:%d: %s\n", __FILE__, __LINE__, #cond); \
            std::exit(1);                                                           \
        }                                                                           \
    } while (0)

// pol plane 0 at i = 3 * (opponent stones of the newest board next to i);
// val plane at i = 1 + own stone - opponent stone at i (newest board).
class NeighbourNet : public BatchExecutor {
public:
    NeighbourNet(int mb, int delay_us) : m_mb(mb), m_delay(delay_us) {}
    int max_batch() const override { return m_mb; }
    void forward_batch(int n, const float* in, float* pol, float* val) override {
        if (fail.load()) throw std::runtime_error("injected failure");
        if (m_delay) std::this_thread::sleep_for(std::chrono::microseconds(m_delay));
        for (int b = 0; b < n; b++) {
            const float* x = in + (size_t)b * LZHIP_INPUT_SIZE;
            const float* own = x;
            const float* opp = x + 8 * kPoints;
            float* p = pol + (size_t)b * LZHIP_POL_SIZE;
            float* v = val + (size_t)b * LZHIP_VAL_SIZE;
            for (int i = 0; i < kPoints; i++) {
                const int xx = i % 19, yy = i / 19;
                float s = 0.0f;
                if (xx > 0) s += opp[i - 1];
                if (xx < 18) s += opp[i + 1];
                if (yy > 0) s += opp[i - 19];
                if (yy < 18) s += opp[i + 19];
                p[i] = 3.0f * s;
                p[kPoints + i] = 0.0f;
                v[i] = own[i] - opp[i] + 1.0f;
            }
        }
        batches++;
        positions += n;
    }
    // the heads behind the pipe: same arithmetic as the search threads would do
    bool has_heads() const override { return host_heads != nullptr; }
    void evaluate_heads_batch(int n, const float* in, float temperature, float* policy,
                              float* value) override {
        if (!host_heads) throw std::logic_error("no heads");
        std::vector<float> pol((size_t)n * LZHIP_POL_SIZE), val((size_t)n * LZHIP_VAL_SIZE);
        forward_batch(n, in, pol.data(), val.data());
        for (int b = 0; b < n; b++) {
            float win;
            heads_on_host(*host_heads, pol.data() + (size_t)b * LZHIP_POL_SIZE,
                          val.data() + (size_t)b * LZHIP_VAL_SIZE, temperature,
                          policy + (size_t)b * 362, &win);
            value[b] = 2.0f * win - 1.0f;
        }
        head_batches++;
    }
    std::atomic<bool> fail{false};
    std::atomic<long> batches{0}, positions{0}, head_batches{0};
    std::shared_ptr<const HeadWeights> host_heads;

private:
    int m_mb, m_delay;
};

// Heads: logit[o] = pol plane 0 at o (pass logit 0); value = tanh(0.05 * stone
// difference) for differences above -10 -> the side with more stones is ahead.
struct Heads {
    std::vector<float> bn_pol_mean{0, 0}, bn_pol_scale{1, 1}, ip_pol_w, ip_pol_b, bn_val_mean{0},
        bn_val_scale{1}, ip1_val_w, ip1_val_b, ip2_val_w, ip2_val_b{0};
    lzhip_head_weights c{};
    Heads() {
        ip_pol_w.assign((size_t)362 * 722, 0.0f);
        for (int o = 0; o < kPoints; o++) ip_pol_w[(size_t)o * 722 + o] = 1.0f;
        ip_pol_b.assign(362, 0.0f);
        ip1_val_w.assign((size_t)256 * kPoints, 0.0f);
        for (int i = 0; i < kPoints; i++) ip1_val_w[i] = 1.0f;
        ip1_val_b.assign(256, 0.0f);
        ip1_val_b[0] = -351.0f;  // hidden unit 0 = relu(10 + own - opp)
        ip2_val_w.assign(256, 0.0f);
        ip2_val_w[0] = 0.05f;
        ip2_val_b[0] = -0.5f;
        c.bn_pol_mean = bn_pol_mean.data();
        c.bn_pol_scale = bn_pol_scale.data();
        c.ip_pol_w = ip_pol_w.data();
        c.ip_pol_b = ip_pol_b.data();
        c.bn_val_mean = bn_val_mean.data();
        c.bn_val_scale = bn_val_scale.data();
        c.ip1_val_w = ip1_val_w.data();
        c.ip1_val_b = ip1_val_b.data();
        c.ip2_val_w = ip2_val_w.data();
        c.ip2_val_b = ip2_val_b.data();
    }
};

static lzhip_search_config config(int threads, int visits, int moves) {
    lzhip_search_config c{};
    c.threads = threads;
    c.visits = visits;
    c.moves = moves;
    c.cache_size = 20000;
    c.reuse_tree = 1;
    c.random_moves = 0;
    c.virtual_loss = 3;
    c.puct = 0.5f;
    c.logpuct = 0.015f;
    c.logconst = 1.7f;
    c.fpu_reduction = 0.25f;
    c.fpu_root_reduction = 0.25f;
    c.softmax_temp = 1.0f;
    c.komi = 7.5f;
    c.seed = 7;
    return c;
}

static void test_unrotation() {
    HIPScheduler sched(std::make_unique<NeighbourNet>(4, 0));
    Heads heads;
    NetworkFacade net(sched, heads.c, 0, 1.0f);
    go::Position pos;
    const int stone = 5 * 19 + 2;  // (2,5): off every symmetry axis
    pos.play(stone);               // black; white to move sees one opponent stone
    uint64_t rng = 99;
    for (int sym = 0; sym < 8; sym++) {
        const Netresult r = net.get_output(pos, sym, rng, false);
        // the four neighbours of the stone share the top prior, in board order
        const float top = r.policy[stone - 1];
        CHECK(top > 0.04f);
        CHECK(std::fabs(r.policy[stone + 1] - top) < 1e-6f);
        CHECK(std::fabs(r.policy[stone - 19] - top) < 1e-6f);
        CHECK(std::fabs(r.policy[stone + 19] - top) < 1e-6f);
        int above = 0;
        for (int i = 0; i < kPoints; i++)
            if (r.policy[i] > top * 0.5f) above++;
        CHECK(above == 4);
        CHECK(r.winrate < 0.5f);  // the side to move is a stone behind
        float sum = r.policy_pass;
        for (int i = 0; i < kPoints; i++) sum += r.policy[i];
        CHECK(std::fabs(sum - 1.0f) < 1e-4f);
    }
}

// Format-2 networks give the value for black: get_output turns it round for white, also in
// what it puts into the cache (reference src/Network.cpp:797-807).
static void test_value_head_not_stm() {
    HIPScheduler sched(std::make_unique<NeighbourNet>(4, 0));
    Heads heads;
    NetworkFacade plain(sched, heads.c, 0, 1.0f), flipped(sched, heads.c, 10, 1.0f);
    flipped.set_value_head_not_stm(true);
    go::Position pos;
    uint64_t rng = 5;
    const Netresult b0 = plain.get_output(pos, 0, rng, false);      // black to move
    const Netresult b1 = flipped.get_output(pos, 0, rng, true);
    CHECK(b0.winrate == b1.winrate);
    pos.play(5 * 19 + 2);                                             // white to move
    const Netresult w0 = plain.get_output(pos, 3, rng, false);
    const Netresult w1 = flipped.get_output(pos, 3, rng, true);
    CHECK(std::fabs(w1.winrate - (1.0f - w0.winrate)) < 1e-7f);
    CHECK(std::fabs(w0.winrate - 0.5f) > 0.01f);                     // the flip is visible
    for (int i = 0; i < kPoints; i++) CHECK(w0.policy[i] == w1.policy[i]);
    const Netresult w2 = flipped.get_output(pos, 3, rng, true);      // from the cache
    CHECK(flipped.cache_hits() == 1 && w2.winrate == w1.winrate);
}

static void test_symmetric_cache_probe() {
    HIPScheduler sched(std::make_unique<NeighbourNet>(4, 0));
    Heads heads;
    NetworkFacade net(sched, heads.c, 100, 1.0f);
    uint64_t rng = 5;
    // black (2,5), white (9,3): no symmetry of its own
    go::Position a;
    a.play(5 * 19 + 2);
    a.play(3 * 19 + 9);
    const Netresult ra = net.get_output(a, 0, rng);
    CHECK(net.evals() == 1 && net.cache_hits() == 0);
    for (int sym = 1; sym < 8; sym++) {
        // the same game seen through symmetry `sym`
        go::Position b;
        b.play(symmetry_index(sym, 5 * 19 + 2));
        b.play(symmetry_index(sym, 3 * 19 + 9));
        const Netresult direct = net.get_output(b, 0, rng, /*use_cache=*/false);
        const uint64_t evals_before = net.evals();
        const Netresult cached = net.get_output(b, 0, rng);
        CHECK(net.evals() == evals_before);           // answered from a's entry
        CHECK(net.cache_hits() == (uint64_t)sym);
        for (int i = 0; i < kPoints; i++) CHECK(std::fabs(cached.policy[i] - direct.policy[i]) < 1e-6f);
        CHECK(std::fabs(cached.winrate - direct.winrate) < 1e-6f);
        CHECK(std::fabs(cached.winrate - ra.winrate) < 1e-6f);
    }
    // switched off, or after the opening, the images are not consulted
    net.set_symmetry_probe(false);
    go::Position c;
    c.play(symmetry_index(3, 5 * 19 + 2));
    c.play(symmetry_index(3, 3 * 19 + 9));
    const uint64_t evals_before = net.evals();
    net.get_output(c, 0, rng);
    CHECK(net.evals() == evals_before + 1);
}

static std::vector<int> play_game(int threads, int visits, int moves, int delay_us, int max_batch,
                                  lzhip_search_result* res_out, int reuse = 1) {
    HIPScheduler sched(std::make_unique<NeighbourNet>(max_batch, delay_us));
    Heads heads;
    lzhip_search_config cfg = config(threads, visits, moves);
    cfg.reuse_tree = reuse;
    NetworkFacade net(sched, heads.c, (size_t)cfg.cache_size, 1.0f);
    UCTSearch search(net, cfg);
    go::Position pos;
    std::vector<int> game;
    for (int m = 0; m < moves && pos.passes() < 2; m++) {
        const int before = search.root_visits();
        const int mv = search.think(pos);
        CHECK(search.root_visits() >= visits);
        CHECK(search.root_visits() >= before);
        const auto tc = search.check_tree();
        CHECK(tc.virtual_loss == 0);
        CHECK(tc.expanding == 0);
        CHECK(tc.visit_mismatch == 0);
        CHECK(mv == kPass || pos.legal_slow(pos.to_move(), mv));
        // the chosen move is the most visited child
        int best = -1;
        for (auto& cv : search.root_children()) best = std::max(best, cv.second);
        for (auto& cv : search.root_children())
            if (cv.first == mv) CHECK(cv.second == best);
        pos.play(mv);
        CHECK(!(mv != kPass && pos.superko()));
        search.advance(mv);
        game.push_back(mv);
    }
    // the backend answers again after the halts
    std::vector<float> in(LZHIP_INPUT_SIZE, 0.0f), pol(LZHIP_POL_SIZE), val(LZHIP_VAL_SIZE);
    sched.forward(in, pol, val);
    if (res_out) {
        res_out->playouts = search.stats().playouts;
        res_out->halted = search.stats().halted;
        res_out->wasted = search.stats().wasted;
        res_out->evals = net.evals();
        res_out->cache_hits = net.cache_hits();
        res_out->cache_lookups = net.cache_lookups();
        res_out->sched = sched.stats();
    }
    return game;
}

static void test_heads_behind_the_pipe() {
    Heads heads;
    std::vector<int> games[2];
    for (int mode = 0; mode < 2; mode++) {
        auto exec = std::make_unique<NeighbourNet>(4, 0);
        exec->host_heads = std::make_shared<const HeadWeights>(heads.c);
        NeighbourNet* raw = exec.get();
        HIPScheduler sched(std::move(exec));
        lzhip_search_config cfg = config(1, 80, 5);
        cfg.device_heads = mode;
        lzhip_search_result res;
        int moves[5];
        selfplay(sched, heads.c, cfg, res, moves, 5);
        games[mode].assign(moves, moves + res.moves_played);
        CHECK((raw->head_batches.load() > 0) == (mode == 1));
    }
    CHECK(games[0] == games[1]);
    // several threads, both kinds of request in the queue at once
    auto exec = std::make_unique<NeighbourNet>(8, 100);
    exec->host_heads = std::make_shared<const HeadWeights>(heads.c);
    HIPScheduler sched(std::move(exec));
    std::atomic<int> ok{0};
    std::vector<std::thread> th;
    for (int t = 0; t < 8; t++)
        th.emplace_back([&, t] {
            std::vector<float> in(LZHIP_INPUT_SIZE, 0.0f), pol(LZHIP_POL_SIZE), val(LZHIP_VAL_SIZE);
            in[8 * kPoints + 40 + t] = 1.0f;   // one opponent stone
            for (int r = 0; r < 20; r++) {
                if ((t + r) & 1) {
                    float policy[362], value;
                    CHECK(sched.evaluate_raw(in.data(), 1.0f, policy, &value) == LZHIP_OK);
                    float sum = 0.0f;
                    for (float p : policy) sum += p;
                    CHECK(std::fabs(sum - 1.0f) < 1e-4f);
                    CHECK(policy[40 + t + 1] > 0.04f && value < 0.0f);
                } else {
                    sched.forward(in, pol, val);
                    CHECK(pol[40 + t + 1] == 3.0f);
                }
                ok++;
            }
        });
    for (auto& t : th) t.join();
    CHECK(ok == 160);
}

static void test_single_thread_deterministic() {
    lzhip_search_result a{}, b{};
    const auto g1 = play_game(1, 120, 6, 0, 4, &a);
    const auto g2 = play_game(1, 120, 6, 0, 4, &b);
    CHECK(g1 == g2);
    CHECK(g1.size() == 6);
    CHECK(a.playouts == b.playouts);
    CHECK(a.halted <= 6);  // one thread: at most the request in flight at each stop
    // with the neighbour prior white's first reply touches black's first stone
    const int d = std::abs(g1[1] - g1[0]);
    CHECK(d == 1 || d == 19);
}

static void test_many_threads() {
    lzhip_search_result r{};
    const auto g = play_game(12, 300, 5, 150, 8, &r);
    CHECK(g.size() == 5);
    CHECK(r.playouts >= 5 * 200);
    CHECK(r.sched.max_batch_seen <= 8);
    CHECK(r.sched.max_batch_seen >= 2);  // concurrent requests were batched
    CHECK(r.sched.requests + r.sched.halted >= r.evals);
    std::printf("  12 threads: playouts %llu evals %llu halted %llu wasted %llu batches %llu max %u\n",
                (unsigned long long)r.playouts, (unsigned long long)r.evals,
                (unsigned long long)r.halted, (unsigned long long)r.wasted,
                (unsigned long long)r.sched.batches, r.sched.max_batch_seen);
}

static void test_cache_hits_without_tree_reuse() {
    lzhip_search_result r{};
    play_game(2, 150, 3, 0, 4, &r, /*reuse=*/0);
    CHECK(r.cache_hits > 50);  // the second and third searches revisit known positions
    CHECK(r.evals + r.cache_hits == r.cache_lookups);
}

static void test_finished_game_is_not_searched() {
    HIPScheduler sched(std::make_unique<NeighbourNet>(4, 0));
    Heads heads;
    lzhip_search_config cfg = config(2, 50, 1);
    NetworkFacade net(sched, heads.c, 100, 1.0f);
    UCTSearch search(net, cfg);
    go::Position pos;
    pos.play(kPass);
    pos.play(kPass);
    CHECK(search.think(pos) == kPass);
    CHECK(net.evals() == 0);
}

static void test_selfplay_entry_and_failure() {
    Heads heads;
    {
        HIPScheduler sched(std::make_unique<NeighbourNet>(8, 50));
        lzhip_search_config cfg = config(6, 100, 4);
        lzhip_search_result res;
        int moves[4] = {-1, -1, -1, -1};
        selfplay(sched, heads.c, cfg, res, moves, 4);
        CHECK(res.moves_played == 4);
        CHECK(res.playouts > 0 && res.seconds > 0 && res.visits_per_s > 0);
        CHECK(res.sched.batches > 0 && res.sched.batch_slots == res.sched.batches * 8);
        CHECK(res.sched.requests <= res.evals);
        for (int m : moves) CHECK(m >= 0 && m <= kPass);
    }
    {
        auto exec = std::make_unique<NeighbourNet>(4, 0);
        exec->fail = true;
        HIPScheduler sched(std::move(exec));
        lzhip_search_config cfg = config(3, 50, 2);
        lzhip_search_result res;
        bool threw = false;
        try {
            selfplay(sched, heads.c, cfg, res, nullptr, 0);
        } catch (const std::runtime_error&) {
            threw = true;
        }
        CHECK(threw);
    }
    {
        HIPScheduler sched(std::make_unique<NeighbourNet>(4, 0));
        lzhip_search_config cfg = config(0, 50, 2);
        lzhip_search_result res;
        bool threw = false;
        try {
            selfplay(sched, heads.c, cfg, res, nullptr, 0);
        } catch (const std::invalid_argument&) {
            threw = true;
        }
        CHECK(threw);
    }
}

// Child selection on a hand-worked node (reference src/UCTNode.cpp:306-362, get_raw_eval
// :270-282, defaults src/GTP.cpp:346-350: puct 0.5, logpuct 0.015, logconst 1.7, fpu
// reduction 0.25; virtual loss 3, src/UCTNode.h:51).
//
// Parent: mean for black 0.55.  Children (prior, visits, sum of black values):
//   c0 0.40, 6, 3.30      c1 0.30, 3, 1.95      c2 0.20, 0      c3 0.10, 0
// N = 9 visits below the parent, priors of the visited children 0.70.
//   numerator     = sqrt(9 * ln(0.015 * 9 + 1.7)) = sqrt(9 * 0.607045) = 2.337392
//   fpu_reduction = 0.25 * sqrt(0.70) = 0.209165
// Black to move: fpu_eval = 0.55 - 0.209165 = 0.340835
//   c0  3.30/6 = 0.55   + 0.5 * 0.40 * 2.337392 / 7 = 0.55 + 0.066783 = 0.616783
//   c1  1.95/3 = 0.65   + 0.5 * 0.30 * 2.337392 / 4 = 0.65 + 0.087652 = 0.737652   <- chosen
//   c2  0.340835        + 0.5 * 0.20 * 2.337392 / 1 =                   0.574574
//   c3  0.340835        + 0.5 * 0.10 * 2.337392 / 1 =                   0.457705
//   Without the reduction c2 would read 0.55 + 0.233739 = 0.783739 and be chosen (and with
//   the reduction added instead of subtracted, 0.992904): the reduction decides.
// White to move: parent mean 0.45, fpu_eval = 0.240835; the children's means turn round
//   c0  0.45 + 0.066783 = 0.516783   <- chosen     c1  0.35 + 0.087652 = 0.437652
//   c2  0.240835 + 0.233739 = 0.474574             c3  0.240835 + 0.116870 = 0.357705
// Virtual loss, black to move, another thread inside c1 (3 pending visits counted as lost):
//   c1  1.95/(3+3) = 0.325 + 0.087652 = 0.412652, so c0 (0.616783) is chosen instead;
//   seen from white the three pending visits count as black wins: 1 - (1.95+3)/6 = 0.175.
// A child under expansion reads -1 - 0.209165 + its exploration term and is never chosen
// while another child is there.
static void test_puct_arithmetic() {
    lzhip_search_config cfg = config(1, 10, 1);
    CHECK(cfg.puct == 0.5f && cfg.logpuct == 0.015f && cfg.logconst == 1.7f);
    CHECK(cfg.fpu_reduction == 0.25f && cfg.virtual_loss == 3);
    const float prior[4] = {0.40f, 0.30f, 0.20f, 0.10f};
    const int visits[4] = {6, 3, 0, 0};
    const double blackevals[4] = {3.30, 1.95, 0.0, 0.0};
    auto near = [](double a, double b) { return std::fabs(a - b) < 2e-6; };
    auto pick = [&](const lzhip_search_config& c, int color, const int* vloss, int expanding,
                    double* values, bool is_root = false) {
        size_t n = 0;
        float visited = 0.0f;
        for (int i = 0; i < 4; i++) {
            n += (size_t)visits[i];
            if (visits[i] > 0) visited += prior[i];
        }
        const float parent_eval = puct_eval_for(color, 5.5, 10, 0);
        const PuctParent par = puct_parent(c, is_root, n, visited, parent_eval);
        int best = -1;
        double best_value = -1e300;
        for (int i = 0; i < 4; i++) {
            const float e = puct_eval_for(color, blackevals[i], visits[i], vloss ? vloss[i] : 0);
            values[i] = puct_value(c, par, prior[i], visits[i], i == expanding, e);
            if (values[i] > best_value) {
                best_value = values[i];
                best = i;
            }
        }
        return best;
    };
    double v[4];
    {
        const PuctParent par = puct_parent(cfg, false, 9, 0.70f, 0.55f);
        CHECK(near(par.numerator, 2.337392) && near(par.fpu_reduction, 0.209165) &&
              near(par.fpu_eval, 0.340835));
    }
    CHECK(pick(cfg, go::BLACK, nullptr, -1, v) == 1);
    CHECK(near(v[0], 0.616783) && near(v[1], 0.737652) && near(v[2], 0.574574) &&
          near(v[3], 0.457705));
    lzhip_search_config no_fpu = cfg;
    no_fpu.fpu_reduction = 0.0f;
    CHECK(pick(no_fpu, go::BLACK, nullptr, -1, v) == 2 && near(v[2], 0.783739));
    // the root has a reduction of its own (reference src/UCTNode.cpp:322-324): with none at
    // the root and 0.25 below it the same node picks child 2 as the root and child 1 elsewhere
    lzhip_search_config root_cfg = cfg;
    CHECK(root_cfg.fpu_root_reduction == 0.25f);
    root_cfg.fpu_root_reduction = 0.0f;
    CHECK(pick(root_cfg, go::BLACK, nullptr, -1, v, true) == 2 && near(v[2], 0.783739));
    CHECK(pick(root_cfg, go::BLACK, nullptr, -1, v, false) == 1 && near(v[2], 0.574574));
    CHECK(pick(cfg, go::WHITE, nullptr, -1, v) == 0);
    CHECK(near(v[0], 0.516783) && near(v[1], 0.437652) && near(v[2], 0.474574) &&
          near(v[3], 0.357705));
    const int vloss[4] = {0, 3, 0, 0};
    CHECK(pick(cfg, go::BLACK, vloss, -1, v) == 0 && near(v[1], 0.412652));
    CHECK(near(puct_eval_for(go::WHITE, 1.95, 3, 3), 0.175));
    CHECK(near(puct_eval_for(go::BLACK, 0.0, 0, 0), 0.5));
    CHECK(pick(cfg, go::BLACK, nullptr, 1, v) == 0 && near(v[1], -1.0 - 0.209165 + 0.087652));
    std::printf("puct arithmetic pinned\n");
}

int main() {
    test_puct_arithmetic();
    std::printf("unrotation\n");
    test_unrotation();
    test_value_head_not_stm();
    std::printf("symmetric cache probe\n");
    test_symmetric_cache_probe();
    std::printf("heads behind the pipe\n");
    test_heads_behind_the_pipe();
    std::printf("single thread\n");
    test_single_thread_deterministic();
    std::printf("many threads\n");
    test_many_threads();
    std::printf("cache\n");
    test_cache_hits_without_tree_reuse();
    std::printf("finished game\n");
    test_finished_game_is_not_searched();
    std::printf("selfplay entry\n");
    test_selfplay_entry_and_failure();
    std::printf("search tests passed\n");
    return 0;
}
