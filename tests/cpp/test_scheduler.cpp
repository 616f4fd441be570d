// Host-only test of the batching scheduler with a stand-in executor, meant to be
// built with -fsanitize=thread.  Checks the invariants the reference's scheduler
// promises its callers (reference src/OpenCLScheduler.cpp:256-441):
//   * every request is answered exactly once, with its own position's data;
//   * a batch never exceeds max_batch;
//   * drain() releases every waiter with a halt, later calls halt at once,
//     resume() needs an empty queue and re-opens the pipe;
//   * destruction with idle and with blocked callers ends cleanly;
//   * an executor failure reaches the caller as an exception;
//   * with an executor that accepts two or three batches at a time, that many are in
//     flight together and all of the above still holds;
//   * planes that hold only 0 and 1 reach an executor that takes bits one bit per
//     value, any other value sends the whole batch down the float path, and both give
//     each caller the result of its own planes;
//   * a steady population of callers smaller than max_batch ends up in one
//     batch per round instead of two alternating partial ones.
#include <atomic>
#include <chrono>
#include <condition_variable>
#include <cstdio>
#include <cstdlib>
#include <mutex>
#include <stdexcept>
#include <thread>
#include <vector>

#include "forward_pipe.h"

using namespace lzhip;

// The scheduler's translation unit refers to the device factory; no device here.
namespace lzhip {
std::unique_ptr<BatchExecutor> make_hip_pipe(int, int, int, int) {
    throw std::runtime_error("no device in the scheduler test");
}
}  // namespace lzhip

#define CHECK(cond)                                                        \
    do {                                                                   \
        if (!(cond)) {                                                     \
            std::fprintf(stderr, "FAILED %s:%d: %s\n", __FILE__, __LINE__, #cond); \
            std::exit(1);                                                  \
        }                                                                  \
    } while (0)

// pol[i] = in[0] + i, val[i] = in[1] - i : each answer identifies its own request.
class FakeExec : public BatchExecutor {
public:
    FakeExec(int mb, int delay_us, int concurrency = 1)
        : m_mb(mb), m_delay(delay_us), m_conc(concurrency) {}
    int max_batch() const override { return m_mb; }
    int max_concurrency() const override { return m_conc; }
    void forward_batch(int n, const float* in, float* pol, float* val) override {
        struct InFlight {
            FakeExec* e;
            explicit InFlight(FakeExec* x) : e(x) {
                const int now = ++e->inside;
                int seen = e->max_inside.load();
                while (now > seen && !e->max_inside.compare_exchange_weak(seen, now)) {}
            }
            ~InFlight() { --e->inside; }
        } in_flight(this);
        if (n < 1 || n > m_mb) { oversize = true; }
        if (fail_next.exchange(false)) throw std::runtime_error("injected failure");
        {   // a closed gate keeps every batch inside the executor until the test opens it
            std::unique_lock<std::mutex> lk(m_gate_mu);
            m_gate_cv.wait(lk, [&] { return m_gate_open; });
        }
        std::this_thread::sleep_for(std::chrono::microseconds(m_delay));
        for (int b = 0; b < n; b++) {
            const float* x = in + (size_t)b * LZHIP_INPUT_SIZE;
            for (int i = 0; i < LZHIP_POL_SIZE; i++) pol[(size_t)b * LZHIP_POL_SIZE + i] = x[0] + i;
            for (int i = 0; i < LZHIP_VAL_SIZE; i++) val[(size_t)b * LZHIP_VAL_SIZE + i] = x[1] - i;
        }
        calls++;
        positions += n;
    }
    void set_gate(bool open) {
        {
            std::lock_guard<std::mutex> lk(m_gate_mu);
            m_gate_open = open;
        }
        m_gate_cv.notify_all();
    }
    std::atomic<bool> oversize{false}, fail_next{false};
    std::atomic<int> calls{0}, positions{0}, inside{0}, max_inside{0};
private:
    int m_mb, m_delay, m_conc;
    std::mutex m_gate_mu;
    std::condition_variable m_gate_cv;
    bool m_gate_open = true;
};

// Takes bit-packed planes; the answer depends on every input value:
// pol[i] = sum_k (k % 7 + 1) * x[k] + i, val[i] = x[i] (first 361 values).
class BitsExec : public BatchExecutor {
public:
    explicit BitsExec(int mb) : m_mb(mb) {}
    int max_batch() const override { return m_mb; }
    int max_concurrency() const override { return 2; }
    bool accepts_bits() const override { return true; }
    static float digest(const float* x) {
        double s = 0.0;
        for (int k = 0; k < LZHIP_INPUT_SIZE; k++) s += (double)(k % 7 + 1) * x[k];
        return (float)s;
    }
    void forward_batch(int n, const float* in, float* pol, float* val) override {
        std::this_thread::sleep_for(std::chrono::microseconds(100));
        for (int b = 0; b < n; b++) {
            const float* x = in + (size_t)b * LZHIP_INPUT_SIZE;
            const float d = digest(x);
            for (int i = 0; i < LZHIP_POL_SIZE; i++) pol[(size_t)b * LZHIP_POL_SIZE + i] = d + i;
            for (int i = 0; i < LZHIP_VAL_SIZE; i++) val[(size_t)b * LZHIP_VAL_SIZE + i] = x[i];
        }
        float_batches++;
    }
    void run_bits(int n, const uint32_t* bits, bool heads, float, float* a, float* b) override {
        CHECK(!heads);
        std::vector<float> in((size_t)n * LZHIP_INPUT_SIZE);
        for (int p = 0; p < n; p++)
            for (int k = 0; k < LZHIP_INPUT_SIZE; k++)
                in[(size_t)p * LZHIP_INPUT_SIZE + k] =
                    (float)((bits[(size_t)p * kInputWords + (k >> 5)] >> (k & 31)) & 1u);
        forward_batch(n, in.data(), a, b);
        float_batches--;
        bit_batches++;
    }
    std::atomic<int> float_batches{0}, bit_batches{0};
private:
    int m_mb;
};

static void test_bit_packed_requests() {
    auto* be = new BitsExec(8);
    HIPScheduler s{std::unique_ptr<BatchExecutor>(be)};
    std::atomic<int> ok{0};
    std::vector<std::thread> th;
    for (int t = 0; t < 10; t++)
        th.emplace_back([&, t] {
            std::vector<float> in(LZHIP_INPUT_SIZE), pol(LZHIP_POL_SIZE), val(LZHIP_VAL_SIZE);
            uint64_t st = 1234567 + 977 * t;
            for (int r = 0; r < 30; r++) {
                for (auto& v : in) {
                    st = st * 6364136223846793005ull + 1442695040888963407ull;
                    v = (st >> 62) == 0 ? 1.0f : 0.0f;
                }
                in[LZHIP_INPUT_SIZE - 1] = 1.0f;                 // the last, partial word
                if (t == 3 && r % 4 == 0) in[100 + r] = 0.5f;    // not a 0/1 plane
                if (t == 5 && r % 7 == 0) in[7] = -0.0f;         // nor is a negative zero
                s.forward(in, pol, val);
                const float d = BitsExec::digest(in.data());
                for (int i = 0; i < LZHIP_POL_SIZE; i++) CHECK(pol[i] == d + i);
                for (int i = 0; i < LZHIP_VAL_SIZE; i++) CHECK(val[i] == in[i]);
                ok++;
            }
        });
    for (auto& t : th) t.join();
    CHECK(ok == 300);
    CHECK(be->bit_batches > 0 && be->float_batches > 0);
    std::printf("bit-packed: %d batches as bits, %d as floats\n", be->bit_batches.load(),
                be->float_batches.load());
}

static void one_call(HIPScheduler& s, float a, float b, std::atomic<int>& ok,
                     std::atomic<int>& halted) {
    std::vector<float> in(LZHIP_INPUT_SIZE, 0.0f), pol(LZHIP_POL_SIZE), val(LZHIP_VAL_SIZE);
    in[0] = a;
    in[1] = b;
    try {
        s.forward(in, pol, val);
        for (int i = 0; i < LZHIP_POL_SIZE; i++) CHECK(pol[i] == a + i);
        for (int i = 0; i < LZHIP_VAL_SIZE; i++) CHECK(val[i] == b - i);
        ok++;
    } catch (const NetworkHaltException&) {
        halted++;
    }
}

static void test_concurrent(int threads, int mb, int reps, int concurrency = 1) {
    auto* fe = new FakeExec(mb, 200, concurrency);
    HIPScheduler s{std::unique_ptr<BatchExecutor>(fe)};
    std::atomic<int> ok{0}, halted{0};
    std::vector<std::thread> th;
    // the process-wide counters the engine prints after a search (no other scheduler is
    // running during this test, so their growth is this scheduler's)
    const size_t g_single = batch_stats.single_evals, g_batch = batch_stats.batch_evals,
                 g_pos = batch_stats.positions, g_slots = batch_stats.slots;
    for (int t = 0; t < threads; t++)
        th.emplace_back([&, t] {
            for (int r = 0; r < reps; r++) one_call(s, (float)(t * 1000 + r), (float)(r - t), ok, halted);
        });
    for (auto& t : th) t.join();
    CHECK(ok == threads * reps && halted == 0);
    {
        const lzhip_stats st = s.stats();
        const size_t singles = batch_stats.single_evals - g_single;
        const size_t multis = batch_stats.batch_evals - g_batch;
        CHECK(singles + multis == st.batches);
        CHECK(batch_stats.positions - g_pos == st.requests);
        CHECK(batch_stats.slots - g_slots == st.batch_slots);
        if (threads == 1) CHECK(multis == 0 && singles == st.requests);
    }
    CHECK(!fe->oversize);
    CHECK(fe->positions == threads * reps);
    const lzhip_stats st = s.stats();
    CHECK(st.requests == (uint64_t)threads * reps);
    CHECK(st.max_batch_seen <= (uint32_t)mb);
    CHECK(st.batches == (uint64_t)fe->calls.load());
    if (threads >= 2 * mb) CHECK(st.batches < (uint64_t)threads * reps);  // it did batch
    CHECK(fe->max_inside <= concurrency);
    if (concurrency >= 2 && threads >= 4 * mb) CHECK(fe->max_inside == concurrency);  // batches overlapped
    std::printf("concurrent threads=%d mb=%d: %llu batches for %llu requests, max %u\n", threads,
                mb, (unsigned long long)st.batches, (unsigned long long)st.requests,
                st.max_batch_seen);
}

// 12 callers that come straight back after each answer, max batch 32: once the
// scheduler has seen the population it waits for all of them, so the mean
// batch approaches 12 instead of the 6+6 of two alternating groups.
static void test_population_batches(int concurrency) {
    auto* fe = new FakeExec(32, 2000, concurrency);
    HIPScheduler s{std::unique_ptr<BatchExecutor>(fe)};
    std::atomic<int> ok{0}, halted{0};
    std::vector<std::thread> th;
    const int threads = 12, reps = 40;
    for (int t = 0; t < threads; t++)
        th.emplace_back([&, t] {
            for (int r = 0; r < reps; r++) {
                one_call(s, (float)t, (float)r, ok, halted);
                std::this_thread::sleep_for(std::chrono::microseconds(100 + 20 * t));  // host work
            }
        });
    for (auto& t : th) t.join();
    const lzhip_stats st = s.stats();
    CHECK(ok == threads * reps);
    const double mean = (double)st.requests / (double)st.batches;
    std::printf("population (executor concurrency %d): %llu batches, mean batch %.1f of %d callers\n",
                concurrency, (unsigned long long)st.batches, mean, threads);
    CHECK(mean >= 9.0);
}

// drain() while batches sit inside the executor and requests wait in the queue.  The
// executor is held on a gate, so "queued while a batch is inside" is a state the test
// waits for, not a guess about timing: with `concurrency` batches inside and the spare
// worker holding at most one assembled batch more, at most (concurrency + 1) * max_batch
// of the 32 requests have left the queue when drain() runs; all others must halt.
static void test_drain_resume(int concurrency) {
    const int mb = 4, callers = 32;
    auto* fe = new FakeExec(mb, 100, concurrency);
    HIPScheduler s{std::unique_ptr<BatchExecutor>(fe)};
    s.set_max_wait_us(0);
    fe->set_gate(false);
    std::atomic<int> ok{0}, halted{0};
    std::vector<std::thread> th;
    for (int t = 0; t < callers; t++)
        th.emplace_back([&, t] { one_call(s, (float)t, 1.0f, ok, halted); });
    while (s.outstanding() < callers || fe->inside < concurrency) std::this_thread::yield();
    s.drain();
    // a call made while drained halts at once, also with batches still inside the executor
    one_call(s, 1.0f, 2.0f, ok, halted);
    CHECK(ok == 0 && halted >= 1);
    fe->set_gate(true);
    for (auto& t : th) t.join();
    CHECK(ok + halted == callers + 1);
    CHECK(ok >= 1 && ok <= (concurrency + 1) * mb);
    CHECK(halted >= callers + 1 - (concurrency + 1) * mb);
    CHECK(fe->max_inside == concurrency);
    const int halted_before = halted;
    s.resume();
    one_call(s, 3.0f, 4.0f, ok, halted);
    CHECK(halted == halted_before);
    CHECK(s.stats().halted == (uint64_t)halted_before);
    std::printf("drain/resume: %d served, %d halted\n", ok.load(), halted.load());
}

static void test_destroy_with_waiters(int concurrency) {
    std::atomic<int> ok{0}, halted{0};
    std::vector<std::thread> th;
    {
        auto* fe = new FakeExec(2, 30000, concurrency);
        auto s = std::make_unique<HIPScheduler>(std::unique_ptr<BatchExecutor>(fe));
        s->set_max_wait_us(0);
        for (int t = 0; t < 8; t++) th.emplace_back([&, t, p = s.get()] { one_call(*p, (float)t, 0.0f, ok, halted); });
        std::this_thread::sleep_for(std::chrono::milliseconds(5));
        s->drain();  // callers must be out of forward() before the object may die
        for (auto& t : th) t.join();
    }
    CHECK(ok + halted == 8);
    { HIPScheduler idle{std::unique_ptr<BatchExecutor>(new FakeExec(2, 10, concurrency))}; }
    std::printf("destroy: %d served, %d halted\n", ok.load(), halted.load());
}

static void test_executor_failure(int concurrency) {
    auto* fe = new FakeExec(4, 10, concurrency);
    HIPScheduler s{std::unique_ptr<BatchExecutor>(fe)};
    fe->fail_next = true;
    std::vector<float> in(LZHIP_INPUT_SIZE, 0.0f), pol(LZHIP_POL_SIZE), val(LZHIP_VAL_SIZE);
    bool threw = false;
    try {
        s.forward(in, pol, val);
    } catch (const std::runtime_error& e) {
        threw = std::string(e.what()) == "injected failure";
    }
    CHECK(threw);
    std::atomic<int> ok{0}, halted{0};
    one_call(s, 5.0f, 6.0f, ok, halted);  // the pipe keeps working afterwards
    CHECK(ok == 1);
    bool bad = false;
    try {
        std::vector<float> small(3);
        s.forward(small, pol, val);
    } catch (const std::invalid_argument&) {
        bad = true;
    }
    CHECK(bad);
    std::printf("executor failure propagated\n");
}

int main() {
    test_concurrent(1, 4, 20);
    test_concurrent(16, 32, 30);   // fewer callers than max_batch: must still batch, never stall
    test_concurrent(48, 8, 20);
    test_concurrent(48, 8, 20, 2);  // two batches in flight
    test_concurrent(5, 8, 20, 2);
    test_concurrent(48, 8, 20, 3);  // three
    test_concurrent(9, 8, 20, 3);
    test_bit_packed_requests();
    test_population_batches(1);
    test_population_batches(2);
    test_population_batches(3);
    for (int c = 1; c <= 3; c++) {
        test_drain_resume(c);
        test_destroy_with_waiters(c);
        test_executor_failure(c);
    }
    std::printf("scheduler tests passed\n");
    return 0;
}
