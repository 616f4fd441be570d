// HIPScheduler: request queue + one worker thread that forms batches for the
// device executor.  Host-only C++ (no HIP calls here), so the queueing logic
// can be unit-tested on a CPU with a stand-in executor under -fsanitize=thread.
//
// Behaviour it keeps from the reference scheduler (src/OpenCLScheduler.cpp):
//  * forward() blocks the calling search thread until its own result is in
//    its own buffers (:256-277, :392-403);
//  * drain() empties the queue and makes every waiting and every later
//    forward() end with NetworkHaltException until resume() (:411-441);
//  * the destructor stops the worker and releases waiters (:134-144).
#include <algorithm>
#include <chrono>
#include <cstring>
#include <stdexcept>
#include <string>

#include "forward_pipe.h"
#include "hip_pipe.h"

namespace lzhip {

batch_stats_t batch_stats;

static constexpr int kInSize = LZHIP_INPUT_SIZE;
static constexpr int kPolSize = LZHIP_POL_SIZE;
static constexpr int kValSize = LZHIP_VAL_SIZE;

HIPScheduler::HIPScheduler(int precision, int max_batch, int device)
    : m_precision(precision), m_max_batch(max_batch), m_device(device) {}

HIPScheduler::HIPScheduler(std::unique_ptr<BatchExecutor> exec) : m_exec(std::move(exec)) {
    m_max_batch = m_exec->max_batch();
    start_worker();
}

HIPScheduler::~HIPScheduler() {
    {
        std::lock_guard<std::mutex> lk(m_mutex);
        m_running = false;
    }
    m_cv.notify_all();
    for (auto& w : m_workers)
        if (w.joinable()) w.join();
    // Anything still queued is released as halted.
    std::deque<std::shared_ptr<Request>> rest;
    {
        std::lock_guard<std::mutex> lk(m_mutex);
        rest.swap(m_queue);
    }
    for (auto& r : rest) {
        {
            std::lock_guard<std::mutex> lk(r->mu);
            r->state = 2;
        }
        r->cv.notify_all();
    }
    delete m_fail_msg;
}

void HIPScheduler::start_worker() {
    std::lock_guard<std::mutex> lk(m_mutex);
    if (m_running) return;
    m_running = true;
    // One worker per batch the executor runs side by side, and one more: handing 64 results
    // back (a wake-up per caller) takes a few hundred microseconds, during which that
    // worker's share of the device would sit idle; the spare worker has the next full
    // batch assembled by then and submits it the moment the executor is free.
    m_lanes = std::max(1, std::min(3, m_exec->max_concurrency()));
    const int n = m_lanes + 1;
    for (int i = 0; i < n; i++) m_workers.emplace_back(&HIPScheduler::worker, this);
}

// ForwardPipe::initialize (reference src/OpenCLScheduler.cpp:108-132): create
// the device pipe for `channels` filters and start the batching worker.
void HIPScheduler::initialize(int channels) {
    if (!m_exec) m_exec = make_hip_pipe(m_device, m_precision, m_max_batch, channels);
    m_max_batch = m_exec->max_batch();
    start_worker();
}

// ForwardPipe::push_weights (reference src/OpenCLScheduler.cpp:223-254).
// filter_size is the Winograd alpha (6) and channels the input plane count
// (18), as passed by Network::init_net (src/Network.cpp:411).
void HIPScheduler::push_weights(unsigned int filter_size, unsigned int channels,
                                unsigned int outputs,
                                std::shared_ptr<const ForwardPipeWeights> weights) {
    auto* pipe = dynamic_cast<HIPPipe*>(m_exec.get());
    if (!pipe) throw std::runtime_error("push_weights: executor is not a device pipe");
    if (filter_size != 6 || channels != LZHIP_INPUT_CHANNELS)
        throw std::invalid_argument("push_weights: expected Winograd alpha 6 and 18 input planes");
    const size_t nl = weights->m_conv_weights.size();
    if (nl == 0 || weights->m_batchnorm_means.size() != nl ||
        weights->m_batchnorm_stddevs.size() != nl)
        throw std::invalid_argument("push_weights: inconsistent layer counts");
    std::vector<const float*> U(nl), mean(nl), scale(nl);
    for (size_t l = 0; l < nl; l++) {
        const size_t cin = l == 0 ? channels : outputs;
        if (weights->m_conv_weights[l].size() != 36 * cin * outputs ||
            weights->m_batchnorm_means[l].size() != outputs ||
            weights->m_batchnorm_stddevs[l].size() != outputs)
            throw std::invalid_argument("push_weights: layer has the wrong size");
        U[l] = weights->m_conv_weights[l].data();
        mean[l] = weights->m_batchnorm_means[l].data();
        scale[l] = weights->m_batchnorm_stddevs[l].data();
    }
    if (weights->m_conv_pol_w.size() != 2 * (size_t)outputs ||
        weights->m_conv_val_w.size() != (size_t)outputs)
        throw std::invalid_argument("push_weights: head convolutions have the wrong size");
    pipe->push_weights((int)nl, U.data(), mean.data(), scale.data(),
                       weights->m_conv_pol_w.data(), weights->m_conv_val_w.data());
}

void HIPScheduler::forward(const std::vector<float>& input, std::vector<float>& output_pol,
                           std::vector<float>& output_val) {
    if (input.size() != (size_t)kInSize || output_pol.size() != (size_t)kPolSize ||
        output_val.size() != (size_t)kValSize)
        throw std::invalid_argument("forward: wrong vector sizes");
    if (forward_raw(input.data(), output_pol.data(), output_val.data()) == LZHIP_EHALT)
        throw NetworkHaltException();
}

int HIPScheduler::forward_raw(const float* in, float* pol, float* val) {
    auto req = std::make_shared<Request>();
    req->in = in;
    req->pol = pol;
    req->val = val;
    return submit(req);
}

int HIPScheduler::evaluate_raw(const float* in, float temperature, float* policy, float* value) {
    if (!(temperature > 0.0f)) throw std::invalid_argument("temperature must be positive");
    if (!m_exec || !m_exec->has_heads())
        throw std::invalid_argument("the executor holds no head parameters (push_heads)");
    auto req = std::make_shared<Request>();
    req->in = in;
    req->pol = policy;
    req->val = value;
    req->heads = true;
    req->temperature = temperature;
    return submit(req);
}

// Packs planes that hold only +0.0f and 1.0f, one bit per value; false (and `bits`
// unspecified) as soon as any other value shows up.
static bool pack_planes(const float* in, uint32_t* bits) {
    static_assert(sizeof(float) == sizeof(uint32_t), "float size");
    constexpr uint32_t kOne = 0x3f800000u;
    uint32_t word = 0, other = 0;
    int w = 0;
    for (int i = 0; i < kInSize; i++) {
        uint32_t v;
        std::memcpy(&v, in + i, sizeof(v));
        other |= (v != 0u && v != kOne) ? 1u : 0u;
        word |= (uint32_t)(v == kOne) << (i & 31);
        if ((i & 31) == 31) {
            bits[w++] = word;
            word = 0;
        }
    }
    if (kInSize & 31) bits[w] = word;
    return other == 0;
}

int HIPScheduler::submit(const std::shared_ptr<Request>& req) {
    if (m_draining.load()) {
        m_halted++;
        return LZHIP_EHALT;
    }
    req->packed = m_exec && m_exec->accepts_bits() && pack_planes(req->in, req->bits);
    m_outstanding++;
    bool wake;
    {
        std::lock_guard<std::mutex> lk(m_mutex);
        if (!m_running) {
            m_outstanding--;
            throw std::runtime_error("forward: scheduler is not initialised");
        }
        // drain() may have started between the check above and here
        if (m_draining.load()) {
            m_outstanding--;
            m_halted++;
            return LZHIP_EHALT;
        }
        m_queue.push_back(req);
        // The collecting worker sleeps until the queue has the length it waits for (or its
        // grace period ends, or the device comes free: others notify it of those); waking
        // every worker for every request in between only makes them queue up for this mutex.
        wake = !m_collecting || m_queue.size() >= m_wake_at;
    }
    if (wake) m_cv.notify_all();  // the collecting worker and an idle one share this condition
    int state;
    {
        std::unique_lock<std::mutex> lk(req->mu);
        req->cv.wait(lk, [&] { return req->state != 0; });
        state = req->state;
    }
    m_outstanding--;
    if (state == 1) {
        m_requests++;
        return LZHIP_OK;
    }
    if (state == 2) {
        m_halted++;
        return LZHIP_EHALT;
    }
    std::string msg;
    {
        std::lock_guard<std::mutex> lk(m_mutex);
        msg = m_fail_msg ? *m_fail_msg : std::string("executor failure");
    }
    throw std::runtime_error(msg);
}

// Batch pickup.  The worker sleeps until a request exists, then grants a
// grace period for the batch to grow towards the number of callers seen around
// the previous batches (those that were queued or in flight when a batch
// finished: the threads just answered come back after their host-side work).
// A forward of a few positions costs about as much as one of a full batch, so
// waiting a fraction of a batch time for the stragglers beats launching two
// alternating half batches.  The grace period is bounded by half the measured
// execution time of a batch (or the fixed value set_max_wait_us gave); an
// estimate of the callers that is too high costs at most that much per batch
// and decays by one caller per batch.
void HIPScheduler::worker() {
    std::vector<float> in, pol, val;
    std::vector<uint32_t> bits((size_t)m_max_batch * BatchExecutor::kInputWords);
    in.resize((size_t)m_max_batch * kInSize);
    pol.resize((size_t)m_max_batch * kPolSize);
    val.resize((size_t)m_max_batch * kValSize);
    std::vector<std::shared_ptr<Request>> batch;
    for (;;) {
        batch.clear();
        {
            std::unique_lock<std::mutex> lk(m_mutex);
            m_cv.wait(lk, [&] { return !m_running || (!m_collecting && !m_queue.empty()); });
            if (!m_running) return;
            // Only one worker assembles a batch at a time; it hands the role on
            // when it leaves this block.
            m_collecting = true;
            struct Handover {
                HIPScheduler* s;
                ~Handover() {
                    s->m_collecting = false;
                    s->m_wake_at = 1;
                    s->m_cv.notify_all();
                }
            } handover{this};
            const int cap_us = m_max_wait_us >= 0
                                   ? m_max_wait_us
                                   : std::max(50, std::min(5000, (int)(m_exec_us * 0.5)));
            // Every executor slot taken: only a full batch is worth assembling ahead of
            // time; otherwise wait for a slot and decide then.
            if (m_exec_busy >= m_lanes) {
                m_wake_at = (size_t)m_max_batch;
                m_cv.wait(lk, [&] {
                    return !m_running || m_queue.empty() || m_exec_busy < m_lanes ||
                           (int)m_queue.size() >= m_max_batch;
                });
                if (!m_running) return;
            }
            // Callers known to exist: those seen around recent batches, or inside
            // forward() right now.  If they all fit one batch, a second batch next
            // to the one in flight would only split them into two small ones that
            // cost a full forward each: wait for the device first.  Otherwise the
            // callers not in flight are the ones this batch can hope for.
            const int pop = std::max(m_population, m_outstanding.load());
            size_t target;
            if (pop <= m_max_batch) {
                target = (size_t)std::max(1, pop);
                m_wake_at = target;
                if (cap_us > 0)
                    m_cv.wait(lk, [&] {
                        return !m_running || m_queue.empty() || m_inflight == 0 ||
                               m_queue.size() >= target;
                    });
                if (!m_running) return;
            } else {
                target = (size_t)std::max(1, std::min(m_max_batch, pop - m_inflight));
            }
            m_wake_at = target;
            if (m_queue.size() < target && cap_us > 0) {
                // system_clock: waits on it map to pthread_cond_timedwait, which thread
                // sanitizers model; the grace period is far too short for clock steps
                // to matter.
                const auto deadline =
                    std::chrono::system_clock::now() + std::chrono::microseconds(cap_us);
                m_cv.wait_until(lk, deadline, [&] {
                    return !m_running || m_queue.empty() || m_queue.size() >= target;
                });
                if (!m_running) return;
            }
            // drain() may have emptied the queue while we waited
            // a batch holds requests of one kind (raw planes, or heads at one temperature)
            while (!m_queue.empty() && (int)batch.size() < m_max_batch) {
                const Request& f = *m_queue.front();
                if (!batch.empty() && (f.heads != batch[0]->heads ||
                                       (f.heads && f.temperature != batch[0]->temperature)))
                    break;
                batch.push_back(std::move(m_queue.front()));
                m_queue.pop_front();
            }
            m_inflight += (int)batch.size();
        }
        if (batch.empty()) continue;
        const int n = (int)batch.size();  // m_inflight was raised under the lock above
        bool all_packed = true;
        for (int i = 0; i < n; i++) all_packed = all_packed && batch[i]->packed;
        if (all_packed) {
            for (int i = 0; i < n; i++)
                std::memcpy(bits.data() + (size_t)i * BatchExecutor::kInputWords, batch[i]->bits,
                            sizeof(uint32_t) * BatchExecutor::kInputWords);
        } else {
            for (int i = 0; i < n; i++)
                std::memcpy(in.data() + (size_t)i * kInSize, batch[i]->in, sizeof(float) * kInSize);
        }
        {
            // the executor takes m_lanes batches at a time
            std::unique_lock<std::mutex> lk(m_mutex);
            m_cv.wait(lk, [&] { return m_exec_busy < m_lanes; });
            m_exec_busy++;
        }
        int outcome = 1;
        const auto t0 = std::chrono::steady_clock::now();
        try {
            if (all_packed)
                m_exec->run_bits(n, bits.data(), batch[0]->heads, batch[0]->temperature,
                                 pol.data(), val.data());
            else if (batch[0]->heads)
                m_exec->evaluate_heads_batch(n, in.data(), batch[0]->temperature, pol.data(),
                                             val.data());
            else
                m_exec->forward_batch(n, in.data(), pol.data(), val.data());
        } catch (const std::exception& e) {
            outcome = 3;
            std::lock_guard<std::mutex> lk(m_mutex);
            delete m_fail_msg;
            m_fail_msg = new std::string(e.what());
        }
        {
            const double us =
                std::chrono::duration<double, std::micro>(std::chrono::steady_clock::now() - t0).count();
            std::lock_guard<std::mutex> lk(m_mutex);
            m_exec_us = m_exec_us > 0.0 ? 0.75 * m_exec_us + 0.25 * us : us;
            // callers in flight plus those that queued up meanwhile; forgets slowly
            m_population = std::max(m_outstanding.load(), m_population - 1);
            m_inflight -= n;
            m_exec_busy--;
        }
        m_cv.notify_all();  // a collector may be waiting for the device to come free
        m_batches++;
        (n == 1 ? batch_stats.single_evals : batch_stats.batch_evals)++;
        batch_stats.positions += (size_t)n;
        batch_stats.slots += (size_t)m_max_batch;
        uint32_t seen = m_max_seen.load();
        while ((uint32_t)n > seen && !m_max_seen.compare_exchange_weak(seen, (uint32_t)n)) {}
        for (int i = 0; i < n; i++) {
            Request& r = *batch[i];
            if (outcome == 1 && r.heads) {
                std::memcpy(r.pol, pol.data() + (size_t)i * 362, sizeof(float) * 362);
                *r.val = val[i];
            } else if (outcome == 1) {
                std::memcpy(r.pol, pol.data() + (size_t)i * kPolSize, sizeof(float) * kPolSize);
                std::memcpy(r.val, val.data() + (size_t)i * kValSize, sizeof(float) * kValSize);
            }
            {
                std::lock_guard<std::mutex> lk(r.mu);
                r.state = outcome;
            }
            r.cv.notify_all();
        }
    }
}

// ForwardPipe::drain (reference src/OpenCLScheduler.cpp:411-433): requests
// still queued are released as halted; a batch already on the device
// completes normally.
void HIPScheduler::drain() {
    m_draining.store(true);
    std::deque<std::shared_ptr<Request>> taken;
    {
        std::lock_guard<std::mutex> lk(m_mutex);
        taken.swap(m_queue);
    }
    m_cv.notify_all();
    for (auto& r : taken) {
        {
            std::lock_guard<std::mutex> lk(r->mu);
            r->state = 2;
        }
        r->cv.notify_all();
    }
}

// ForwardPipe::resume (reference src/OpenCLScheduler.cpp:435-441).  The
// caller has joined its search threads, so the queue is empty.
void HIPScheduler::resume() {
    {
        std::lock_guard<std::mutex> lk(m_mutex);
        if (!m_queue.empty()) throw std::logic_error("resume: requests are still queued");
    }
    m_draining.store(false);
}

void HIPScheduler::set_max_wait_us(int us) {
    std::lock_guard<std::mutex> lk(m_mutex);
    m_max_wait_us = us < 0 ? -1 : us;
}

lzhip_stats HIPScheduler::stats() {
    lzhip_stats s;
    s.requests = m_requests.load();
    s.batches = m_batches.load();
    s.batch_slots = s.batches * (uint64_t)m_max_batch;
    s.halted = m_halted.load();
    s.max_batch_seen = m_max_seen.load();
    s.max_batch = (uint32_t)m_max_batch;
    return s;
}

void HIPScheduler::reset_stats() {
    m_requests = 0;
    m_batches = 0;
    m_halted = 0;
    m_max_seen = 0;
}

}  // namespace lzhip
