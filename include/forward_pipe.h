// C++ side of the boundary: the abstract network backend the engine programs
// against, and the two classes this library adds behind it.
//
// `ForwardPipe` / `ForwardPipeWeights` re-declare, member for member, the
// interface of the reference (src/ForwardPipe.h:38-71) so that
// `Network::init_net` (src/Network.cpp:407-414) can be handed a HIPScheduler
// where it is handed an OpenCLScheduler today (src/Network.cpp:578-597).
// Inside the engine the engine's own header is used and `LZHIP_ENGINE_BUILD`
// makes this file skip the re-declaration.
#ifndef LZHIP_FORWARD_PIPE_H_INCLUDED
#define LZHIP_FORWARD_PIPE_H_INCLUDED

#include <atomic>
#include <condition_variable>
#include <cstdint>
#include <deque>
#include <exception>
#include <memory>
#include <mutex>
#include <stdexcept>
#include <string>
#include <thread>
#include <vector>

#include "lzhip.h"

#ifdef LZHIP_ENGINE_BUILD
#include "ForwardPipe.h"  // the engine's own declarations
#include "Network.h"      // NetworkHaltException
#else
// Thrown out of forward() when the request was woken by drain()
// (reference src/Network.h:66-67).
class NetworkHaltException : public std::exception {};

class ForwardPipe {
public:
    // Weights as the network facade hands them over (src/ForwardPipe.h:40-54):
    // Winograd-domain 3x3 filters, BN means with the conv bias folded in,
    // BN 1/sqrt(var+eps), and the two 1x1 head convolutions.
    class ForwardPipeWeights {
    public:
        std::vector<std::vector<float>> m_conv_weights;
        std::vector<std::vector<float>> m_conv_biases;
        std::vector<std::vector<float>> m_batchnorm_means;
        std::vector<std::vector<float>> m_batchnorm_stddevs;
        std::vector<float> m_conv_pol_w;
        std::vector<float> m_conv_pol_b;
        std::vector<float> m_conv_val_w;
        std::vector<float> m_conv_val_b;
    };

    virtual ~ForwardPipe() = default;
    virtual void initialize(int channels) = 0;
    virtual bool needs_autodetect() { return false; }
    virtual void forward(const std::vector<float>& input, std::vector<float>& output_pol,
                         std::vector<float>& output_val) = 0;
    virtual void push_weights(unsigned int filter_size, unsigned int channels,
                              unsigned int outputs,
                              std::shared_ptr<const ForwardPipeWeights> weights) = 0;
    virtual void drain() {}
    virtual void resume() {}
};
#endif  // LZHIP_ENGINE_BUILD

namespace lzhip {

// Process-wide batch counters of every HIPScheduler: the place of the reference's global
// batch_stats (reference src/OpenCLScheduler.h:43-49, counted at .cpp:367-373, printed
// after every search by src/UCTSearch.cpp:855-860).  single_evals / batch_evals count
// device batches of one position / of more, as there; positions and slots (batches x
// max_batch) give the batch fill ratio.  Always counted (the reference: debug builds).
struct batch_stats_t {
    std::atomic<size_t> single_evals{0};
    std::atomic<size_t> batch_evals{0};
    std::atomic<size_t> positions{0};
    std::atomic<size_t> slots{0};
};
extern batch_stats_t batch_stats;

// What the scheduler drives: something that evaluates up to max_batch()
// positions held in host memory and blocks until the results are back.
// HIPPipe is the device implementation; the scheduler's unit tests plug in a
// host-side stand-in so that the queueing logic can run under a thread
// sanitizer without a GPU.
class BatchExecutor {
public:
    virtual ~BatchExecutor() = default;
    virtual int max_batch() const = 0;
    // How many forward_batch calls may run at the same time.  The scheduler never
    // has more than that many (at most three) inside the executor; it starts one
    // worker thread more, which assembles the next batch meanwhile.
    virtual int max_concurrency() const { return 1; }
    // in [n][18*361] -> pol [n][722], val [n][361]; throws std::runtime_error.
    virtual void forward_batch(int n, const float* in, float* pol, float* val) = 0;
    // Input planes that hold only 0 and 1 (what the engine's feature planes are) may be
    // handed over one bit per value: kInputWords 32-bit words per position, bit
    // (c*361 + pt) = plane c at point pt.  run_bits does what forward_batch (heads ==
    // false: out_a = pol planes, out_b = val plane) or evaluate_heads_batch (heads ==
    // true: out_a = policy, out_b = value) does.  Executors that do not take bits say so.
    static constexpr int kInputWords = (LZHIP_INPUT_SIZE + 31) / 32;
    virtual bool accepts_bits() const { return false; }
    virtual void run_bits(int /*n*/, const uint32_t* /*bits*/, bool /*heads*/,
                          float /*temperature*/, float* /*out_a*/, float* /*out_b*/) {
        throw std::logic_error("this executor does not take bit-packed planes");
    }
    // Whether evaluate_heads_batch can be served (head parameters are on board).
    virtual bool has_heads() const { return false; }
    // Tower + heads for n positions: policy [n][362] (softmax at `temperature`),
    // value [n] (tanh output).  Executors without heads on board refuse.
    virtual void evaluate_heads_batch(int /*n*/, const float* /*in*/, float /*temperature*/,
                                      float* /*policy*/, float* /*value*/) {
        throw std::logic_error("this executor does not compute the heads");
    }
};

// Device executor: owns the weights and activation buffers of one network on
// one GPU and runs the residual tower + 1x1 heads for a batch.  Takes the
// place of OpenCL<net_t> + OpenCL_Network<net_t> (reference src/OpenCL.h:86-226);
// there is no tuner, tile shapes are fixed for gfx950.
class HIPPipe;
std::unique_ptr<BatchExecutor> make_hip_pipe(int device, int precision, int max_batch,
                                             int filters);

// Batching scheduler: takes the place of OpenCLScheduler<net_t>
// (reference src/OpenCLScheduler.h:51-118, .cpp:256-441) for one GPU.
// Differences that are deliberate:
//  * a request waits on a per-request done flag (the reference waits on a
//    condition variable without a predicate, .cpp:272);
//  * the worker launches whatever is queued, up to max_batch, after a short
//    adaptive grace period, instead of "full batch or exactly one"
//    (.cpp:311-353), so that fewer search threads than max_batch still batch.
//    The batch it waits for is the number of callers seen around the previous
//    batches (capped at max_batch); the grace period is bounded by half the
//    measured execution time of a batch, because at these sizes a forward
//    costs about the same for 8 positions as for 32.
class HIPScheduler : public ForwardPipe {
public:
    // The engine-facing constructor: device pipe created in initialize().
    HIPScheduler(int precision, int max_batch, int device = 0);
    // Test/bring-up constructor: drive an arbitrary executor.
    explicit HIPScheduler(std::unique_ptr<BatchExecutor> exec);
    ~HIPScheduler() override;

    void initialize(int channels) override;
    void forward(const std::vector<float>& input, std::vector<float>& output_pol,
                 std::vector<float>& output_val) override;
    void push_weights(unsigned int filter_size, unsigned int channels, unsigned int outputs,
                      std::shared_ptr<const ForwardPipeWeights> weights) override;
    void drain() override;
    void resume() override;

    // Pointer form of forward() used by the C ABI; returns LZHIP_OK/LZHIP_EHALT
    // and throws std::runtime_error on executor failure.
    int forward_raw(const float* in, float* pol, float* val);
    // One position through the queue with the heads computed by the executor
    // (Network::get_output_internal's arithmetic, reference src/Network.cpp:833-851,
    // moved behind the pipe): policy [362], *value = tanh output.  Requests of this
    // kind are batched among themselves.  Same return codes as forward_raw.
    int evaluate_raw(const float* in, float temperature, float* policy, float* value);

    BatchExecutor* executor() { return m_exec.get(); }
    // Callers inside forward() right now (queued, in a batch, or about to return).
    int outstanding() const { return m_outstanding.load(); }
    lzhip_stats stats();
    void reset_stats();
    // Upper bound, in microseconds, of the grace period the worker grants a
    // partial batch: 0 = launch immediately, negative = automatic (half the
    // measured execution time of a batch; the default).
    void set_max_wait_us(int us);

private:
    struct Request {
        const float* in;
        float* pol;   // raw policy planes [722], or policy [362] when heads are asked for
        float* val;   // raw value plane [361], or the value scalar
        bool heads = false;
        float temperature = 1.0f;
        // the planes one bit per value, filled by the calling thread when every value is
        // exactly 0 or 1 (then `packed`); 32 times less to gather and to send to the device
        bool packed = false;
        uint32_t bits[BatchExecutor::kInputWords];
        std::mutex mu;
        std::condition_variable cv;
        int state = 0;  // 0 pending, 1 done, 2 halted, 3 failed
    };
    void start_worker();
    void worker();
    int submit(const std::shared_ptr<Request>& req);

    int m_precision = LZHIP_FP32, m_max_batch = 1, m_device = 0;
    std::unique_ptr<BatchExecutor> m_exec;
    std::mutex m_mutex;
    std::condition_variable m_cv;
    std::deque<std::shared_ptr<Request>> m_queue;
    std::vector<std::thread> m_workers;
    bool m_collecting = false;  // one worker at a time assembles a batch
    size_t m_wake_at = 1;       // queue length at which the collecting worker wants to be woken
    bool m_running = false;
    std::atomic<bool> m_draining{false};
    std::atomic<int> m_outstanding{0};  // callers currently inside forward()
    int m_max_wait_us = -1;   // < 0: automatic
    int m_population = 1;     // callers seen around recent batches
    int m_inflight = 0;       // positions in batches assembled and not yet answered
    int m_lanes = 1;          // batches the executor runs side by side
    int m_exec_busy = 0;      // batches inside the executor right now
    double m_exec_us = 0.0;   // smoothed execution time of a batch
    std::string* m_fail_msg = nullptr;
    // statistics
    std::atomic<uint64_t> m_requests{0}, m_batches{0}, m_halted{0};
    std::atomic<uint32_t> m_max_seen{0};
};

}  // namespace lzhip
#endif
