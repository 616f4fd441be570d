// HIPPipe implementation: buffer management, weight upload, the layer loop
// (the role of OpenCL_Network::forward, reference src/OpenCL.cpp:142-329)
// and the fp16 activation-scale calibration.
#include "hip_pipe.h"

#include <hip/hip_runtime.h>

#include <atomic>
#include <cmath>
#include <cstdlib>
#include <condition_variable>
#include <cstring>
#include <map>
#include <tuple>
#include <stdexcept>

#include "kernels.h"

namespace lzhip {

typedef _Float16 half_t;

#define HIP_CHECK(expr)                                                                     \
    do {                                                                                    \
        hipError_t e_ = (expr);                                                             \
        if (e_ != hipSuccess) {                                                             \
            throw std::runtime_error(std::string("HIP error: ") + hipGetErrorString(e_) +   \
                                     " at " + __FILE__ + ":" + std::to_string(__LINE__) +   \
                                     " (" #expr ")");                                       \
        }                                                                                   \
    } while (0)


// Working memory of the entry point that allocates nothing (forward_device_static):
// the buffers a lane otherwise gets from hipMalloc -- packed input planes, three
// activation planes, V and M -- for up to kStaticMaxBatch positions of a net with up
// to kStaticMaxFp filters (padded count) in the wider storage type (fp32):
//   V, M   2 x 36 x 256 x 256 x 4 B = 18 874 368
//   act0   8 x 361 x 64 x 4 B       =    739 328
//   act[3] 3 x 8 x 361 x 256 x 4 B  =  8 871 936      total 28 485 632 B (27.2 MiB)
// Every GPU the library runs on holds its own copy from module load to process end.
// In host code `scratch` is only a handle for hipGetSymbolAddress: the address kernels
// may use is the one resolved per device in static_scratch().
constexpr int kStaticMaxBatch = 8;
constexpr int kStaticMaxFp = 256;
constexpr int kStaticTp = 256;   // 8 x 25 tiles rounded up to kTileRowPad
constexpr size_t kStaticTileBytes = (size_t)kPos * kStaticTp * kStaticMaxFp * 4;
constexpr size_t kStaticAct0Bytes = (size_t)kStaticMaxBatch * kPts * 64 * 4;
constexpr size_t kStaticActBytes = (size_t)kStaticMaxBatch * kPts * kStaticMaxFp * 4;
constexpr size_t kStaticBytes = 2 * kStaticTileBytes + kStaticAct0Bytes + 3 * kStaticActBytes;
static_assert(kStaticTileBytes % 256 == 0 && kStaticAct0Bytes % 256 == 0 &&
              kStaticActBytes % 256 == 0, "sub-buffers keep the 256-byte alignment");
static __device__ __align__(256) unsigned char scratch[kStaticBytes];

constexpr int kMaxDevices = 64;
static std::mutex g_scratch_mu;
static unsigned char* g_scratch_ptr[kMaxDevices] = {};
// One event per device, recorded behind every forward that uses the device's array and
// waited for by the next one, whichever handle and stream it comes from: forwards of
// different handles on one GPU then follow one another on the device instead of
// overwriting each other's tiles.  g_scratch_order_mu makes "wait, enqueue, record" one
// step, so the order of the records is the order of the waits.
static hipEvent_t g_scratch_event[kMaxDevices] = {};
static std::mutex g_scratch_order_mu;

// Device address of this device's copy of `scratch`; resolved once per device, with
// that device current (called from the pipe's constructor, i.e. from lzhip_create).
static unsigned char* static_scratch(int device) {
    if (device < 0 || device >= kMaxDevices) throw std::invalid_argument("device ordinal out of range");
    std::lock_guard<std::mutex> lk(g_scratch_mu);
    if (!g_scratch_ptr[device]) {
        HIP_CHECK(hipSetDevice(device));
        unsigned char* ptr = nullptr;
        HIP_CHECK(hipGetSymbolAddress(reinterpret_cast<void**>(&ptr), HIP_SYMBOL(scratch)));
        if (!ptr) throw std::runtime_error("hipGetSymbolAddress returned a null address");
        HIP_CHECK(hipEventCreateWithFlags(&g_scratch_event[device], hipEventDisableTiming));
        g_scratch_ptr[device] = ptr;
    }
    return g_scratch_ptr[device];
}

template <typename T> struct DevBuf {
    T* p = nullptr;
    size_t count = 0;
    void alloc(size_t n) {
        release();
        if (n == 0) return;
        HIP_CHECK(hipMalloc(reinterpret_cast<void**>(&p), n * sizeof(T)));
        HIP_CHECK(hipMemset(p, 0, n * sizeof(T)));
        count = n;
    }
    void release() {
        if (p) (void)hipFree(p);
        p = nullptr;
        count = 0;
    }
    ~DevBuf() { release(); }
    DevBuf() = default;
    DevBuf(const DevBuf&) = delete;
    DevBuf& operator=(const DevBuf&) = delete;
    DevBuf(DevBuf&& o) noexcept : p(o.p), count(o.count) { o.p = nullptr; o.count = 0; }
};

template <typename T> struct PinnedBuf {
    T* p = nullptr;
    void alloc(size_t n) {
        release();
        HIP_CHECK(hipHostMalloc(reinterpret_cast<void**>(&p), n * sizeof(T), hipHostMallocDefault));
    }
    void release() {
        if (p) (void)hipHostFree(p);
        p = nullptr;
    }
    ~PinnedBuf() { release(); }
};

template <typename P> constexpr int precision_of();
template <> constexpr int precision_of<float>() { return LZHIP_FP32; }
template <> constexpr int precision_of<half_t>() { return LZHIP_FP16; }

template <typename P>
class HIPPipeImpl final : public HIPPipe {
public:
    HIPPipeImpl(int device, int max_batch, int filters)
        : m_device(device), m_max_batch(max_batch), m_filters(filters) {
        if (max_batch < 1 || max_batch > 4096) throw std::invalid_argument("max_batch out of range");
        if (filters < 1 || filters > 4096) throw std::invalid_argument("filters out of range");
        int count = 0;
        HIP_CHECK(hipGetDeviceCount(&count));
        if (device < 0 || device >= count) throw std::runtime_error("no such HIP device");
        HIP_CHECK(hipSetDevice(device));
        hipDeviceProp_t prop;
        HIP_CHECK(hipGetDeviceProperties(&prop, device));
        if (std::strncmp(prop.gcnArchName, "gfx950", 6) != 0)
            throw std::runtime_error(std::string("device is ") + prop.gcnArchName +
                                     ", this library contains gfx950 code only");
        // Small batches leave more of the device idle at every kernel boundary: a third
        // lane pays up to batch 48 (40x256 fp16: +1..30 % up to 32, +7 % at 40, +4 % at 48) and
        // no longer from 52 (-2 % there, -6 % at 64).
        m_n_lanes = max_batch <= 48 ? 3 : 2;
        if (const char* e = std::getenv("LZHIP_LANES")) {   // measurement knob: 1..3 lanes
            const int v = std::atoi(e);
            if (v >= 1 && v <= kLanes) m_n_lanes = v;
        }
        // Every refusal comes before the first stream, event or allocation is made: a
        // constructor that throws runs no destructor.
        m_Fp = (int)ceil_multiple((size_t)filters, 64);
        if (!gemm_supports_channels<P>(m_Fp))
            throw std::invalid_argument(
                "unsupported filter count: after rounding up to a multiple of 64, fp16 takes up "
                "to 512 and 640, 768, 896, 1024; fp32 takes up to 512");
        m_C0p = 64;
        m_Tp = (int)ceil_multiple((size_t)max_batch * kTilesPerBoard, kTileRowPad);
        // The transform kernels address V and M through 32-bit buffer offsets.
        if ((size_t)kPos * m_Tp * m_Fp * sizeof(P) >= ((size_t)1 << 31))
            throw std::invalid_argument(
                "max_batch x filters too large: the Winograd tile buffers would exceed 2 GiB");
        m_static = static_scratch(device);
        struct Unwind {   // releases what the body below has created if it throws
            HIPPipeImpl* self;
            bool armed = true;
            ~Unwind() { if (armed) self->release_device_objects(); }
        } unwind{this};
        for (int i = 0; i < m_n_lanes; i++) {
            HIP_CHECK(hipStreamCreate(&m_lane[i].stream));
            HIP_CHECK(hipEventCreateWithFlags(&m_lane[i].last, hipEventDisableTiming));
        }
        const size_t B = (size_t)max_batch;
        m_din.alloc(B * kInPlanes * kPts);
        m_dpol.alloc(B * 2 * kPts);
        m_dval.alloc(B * kPts);
        for (int i = 0; i < m_n_lanes; i++) {
            IoSlot& sl = m_slot[i];
            sl.hin.alloc(B * kInPlanes * kPts);
            sl.hpol.alloc(B * 2 * kPts);
            sl.hval.alloc(B * kPts);
            sl.din.alloc(B * kInPlanes * kPts);
            sl.dpol.alloc(B * 2 * kPts);
            sl.dval.alloc(B * kPts);
            sl.hbits.alloc(B * kInputWords);
            HIP_CHECK(hipEventCreateWithFlags(&sl.done, hipEventDisableTiming));
        }
        for (int i = 0; i < m_n_lanes; i++) {
            Lane& ln = m_lane[i];
            ln.act0.alloc(B * kPts * m_C0p);
            for (auto& a : ln.act) a.alloc(B * kPts * m_Fp);
            ln.V.alloc((size_t)kPos * m_Tp * m_Fp);
            ln.M.alloc((size_t)kPos * m_Tp * m_Fp);
            ln.flags.alloc(B * kFusedFlagsPerBoard);    // zeroed: no launch has epoch 0
        }
        m_gave_up.alloc(1);
        *m_gave_up.p = 0;
        // measurement knobs.  LZHIP_FUSE: 0 never, 1 where it pays (the default), 2 wherever a
        // fused launch exists; LZHIP_SLAB=0: tile arrays row by row at every batch
        if (const char* e = std::getenv("LZHIP_FUSE")) m_fuse = std::atoi(e);
        if (const char* e = std::getenv("LZHIP_INPLACE")) m_in_place = std::atoi(e) != 0;
        if (const char* e = std::getenv("LZHIP_SLAB")) m_slab = std::atoi(e) != 0;
        m_scalar.alloc(4);
        for (int i = 0; i < kTimerPool; i++) {
            HIP_CHECK(hipEventCreate(&m_ev_start[i]));
            HIP_CHECK(hipEventCreate(&m_ev_stop[i]));
        }
        unwind.armed = false;
    }

    ~HIPPipeImpl() override { release_device_objects(); }

    // Streams and events (the buffers free themselves).  Also run by the constructor
    // when it fails half way.
    void release_device_objects() {
        (void)hipSetDevice(m_device);
        for (auto& ln : m_lane)
            if (ln.stream) (void)hipStreamSynchronize(ln.stream);
        clear_graphs();
        for (int i = 0; i < kTimerPool; i++) {
            if (m_ev_start[i]) (void)hipEventDestroy(m_ev_start[i]);
            if (m_ev_stop[i]) (void)hipEventDestroy(m_ev_stop[i]);
            m_ev_start[i] = m_ev_stop[i] = nullptr;
        }
        for (auto& sl : m_slot) {
            if (sl.done) (void)hipEventDestroy(sl.done);
            sl.done = nullptr;
        }
        for (auto& ln : m_lane) {
            if (ln.last) (void)hipEventDestroy(ln.last);
            ln.last = nullptr;
            if (ln.stream) (void)hipStreamDestroy(ln.stream);
            ln.stream = nullptr;
        }
    }

    int max_batch() const override { return m_max_batch; }
    int max_concurrency() const override { return m_n_lanes; }
    bool has_heads() const override { return m_heads_ready; }
    int filters() const override { return m_filters; }
    int precision() const override { return precision_of<P>(); }
    void* stream() override { return m_lane[0].stream; }
    int lanes() const override { return m_n_lanes; }
    std::vector<float> act_scales() const override { return m_s; }

    // -------------------------------------------------------------------
    // All or nothing: a failure anywhere below (an allocation, a copy, the calibration)
    // leaves the handle as it was before the call -- no layers, forwards refused, and a
    // later push_weights accepted.
    void push_weights(int n_layers, const float* const* U, const float* const* bn_mean,
                      const float* const* bn_scale, const float* pol_w,
                      const float* val_w) override {
        Lane& ln = m_lane[0];
        std::lock_guard<std::mutex> lk(ln.mu);
        if (n_layers < 1 || (n_layers % 2) != 1)
            throw std::invalid_argument("n_layers must be 1 + 2*blocks");
        if (m_ready || !m_layers.empty()) throw std::invalid_argument("push_weights called twice");
        HIP_CHECK(hipSetDevice(m_device));
        try {
            build_layers(n_layers, U, bn_mean, bn_scale, pol_w, val_w);
        } catch (...) {
            (void)hipStreamSynchronize(ln.stream);
            m_layers.clear();
            m_w3.release();
            m_s.clear();
            throw;
        }
        m_ready = true;
    }

    void build_layers(int n_layers, const float* const* U, const float* const* bn_mean,
                      const float* const* bn_scale, const float* pol_w, const float* val_w) {
        auto& ln = m_lane[0];
        const int F = m_filters;
        m_layers.resize(n_layers);
        // Filters are laid out on the host in fp32; an fp16 net converts them on the device.
        std::vector<float> tmp;
        DevBuf<float> stage;
        auto upload = [&](DevBuf<P>& d) {
            d.alloc(tmp.size());
            if constexpr (sizeof(P) == 4) {
                HIP_CHECK(hipMemcpy(d.p, tmp.data(), tmp.size() * sizeof(float),
                                    hipMemcpyHostToDevice));
            } else {
                if (stage.count < tmp.size()) stage.alloc(tmp.size());
                HIP_CHECK(hipMemcpy(stage.p, tmp.data(), tmp.size() * sizeof(float),
                                    hipMemcpyHostToDevice));
                convert_filters(stage.p, d.p, tmp.size(), ln.stream);
                HIP_CHECK(hipGetLastError());
                HIP_CHECK(hipStreamSynchronize(ln.stream));
            }
        };
        for (int l = 0; l < n_layers; l++) {
            Layer& L = m_layers[l];
            L.C = l == 0 ? kInPlanes : F;
            L.Cp = l == 0 ? m_C0p : m_Fp;
            tmp.assign((size_t)kPos * m_Fp * L.Cp, 0.0f);
            // One copy of the filters, in the order the GEMM of this width and precision
            // reads them.  Whether that is the streaming kernel does not depend on the batch
            // of a forward (only on the handle's limit), so a network holds either the
            // fragment order or the row order, never both.
            if (gemm_stream_shape(kTilesPerBoard, L.Cp, m_Fp, (int)sizeof(P)) &&
                gemm_stream_prefers(m_Fp, (int)sizeof(P), m_max_batch)) {
                build_stream_filters(U[l], L.C, F, L.Cp, m_Fp, (int)sizeof(P), tmp.data());
                upload(L.Uf);
            } else {
                // reference layout [36][C][F] (F fastest)  ->  [36][Fp][Cp] (C fastest),
                // zero padded (the role of zeropad_U, reference src/OpenCLScheduler.cpp:60-82)
                for (int p = 0; p < kPos; p++)
                    for (int c = 0; c < L.C; c++) {
                        const float* src = U[l] + ((size_t)p * L.C + c) * F;
                        for (int k = 0; k < F; k++)
                            tmp[((size_t)p * m_Fp + k) * L.Cp + c] = src[k];
                    }
                upload(L.U);
            }
            L.mean.assign(bn_mean[l], bn_mean[l] + F);
            L.scale.assign(bn_scale[l], bn_scale[l] + F);
            L.d_mean.alloc(m_Fp);
            L.d_scale.alloc(m_Fp);
        }
        std::vector<float> w3((size_t)3 * m_Fp, 0.0f);
        for (int c = 0; c < F; c++) {
            w3[c] = pol_w[c];
            w3[m_Fp + c] = pol_w[F + c];
            w3[2 * m_Fp + c] = val_w[c];
        }
        m_w3.alloc(w3.size());
        HIP_CHECK(hipMemcpy(m_w3.p, w3.data(), w3.size() * sizeof(float), hipMemcpyHostToDevice));

        m_s.assign(n_layers + 1, 1.0f);
        for (int l = 0; l < n_layers; l++) upload_bn(l);
        if (precision_of<P>() == LZHIP_FP16) calibrate();
        HIP_CHECK(hipStreamSynchronize(ln.stream));
    }

    // -------------------------------------------------------------------
    void forward_device(int lane, int n, const float* d_in, float* d_pol, float* d_val) override {
        if (lane < 0 || lane >= m_n_lanes) throw std::invalid_argument("no such lane");
        Lane& ln = m_lane[lane];
        std::lock_guard<std::mutex> lk(ln.mu);
        check_ready(n);
        HIP_CHECK(hipSetDevice(m_device));
        run_forward(ln, n, d_in, nullptr, d_pol, d_val);
        HIP_CHECK(hipGetLastError());
    }

    // The same forward with every working buffer taken from the device's static
    // `scratch` array instead of the lane's allocations: kernel launches only, no
    // allocation of any kind.  Enqueued on lane 0's stream.  All calls on one GPU share
    // the array (whatever the handle): each waits on the device for the one enqueued
    // before it (one event per device, see g_scratch_event), so calls from different
    // handles or threads of this process run one after the other on the device.  While
    // the stream is being captured into a graph no event is recorded or waited for (the
    // captured launches are then ordered by the graph's own dependencies, and replays
    // that overlap with other users of the array race).  Nothing in the array has to
    // start at zero: every element a kernel reads for a real tile is written earlier in
    // the same call (rows of V past the last tile feed only rows of M that no kernel reads).
    void forward_device_static(int n, const float* d_in, float* d_pol, float* d_val) override {
        Lane& ln = m_lane[0];
        std::lock_guard<std::mutex> lk(ln.mu);
        if (!m_ready) throw std::invalid_argument("push_weights has not been called");
        if (n < 1 || n > kStaticMaxBatch || n > m_max_batch)
            throw std::invalid_argument(
                "the no-allocation forward takes 1..8 positions (and at most max_batch): its "
                "static working memory is sized for 8");
        if (m_Fp > kStaticMaxFp)
            throw std::invalid_argument(
                "the no-allocation forward takes networks of up to 256 filters: its static "
                "working memory is sized for that");
        HIP_CHECK(hipSetDevice(m_device));
        unsigned char* base = m_static;
        Work w;
        w.stream = ln.stream;
        w.Tp = kStaticTp;
        w.V = reinterpret_cast<P*>(base);
        w.M = reinterpret_cast<P*>(base + kStaticTileBytes);
        w.act0 = reinterpret_cast<P*>(base + 2 * kStaticTileBytes);
        for (int i = 0; i < 3; i++)
            w.act[i] = reinterpret_cast<P*>(base + 2 * kStaticTileBytes + kStaticAct0Bytes +
                                            (size_t)i * kStaticActBytes);
        hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
        HIP_CHECK(hipStreamIsCapturing(ln.stream, &cap));
        const bool ordered = cap == hipStreamCaptureStatusNone;
        std::lock_guard<std::mutex> order(g_scratch_order_mu);
        hipEvent_t ev = g_scratch_event[m_device];
        if (ordered) HIP_CHECK(hipStreamWaitEvent(ln.stream, ev, 0));
        enqueue_forward(w, n, d_in, nullptr, d_pol, d_val, false);
        HIP_CHECK(hipGetLastError());
        if (ordered) HIP_CHECK(hipEventRecord(ev, ln.stream));
    }

    void sync() override {
        HIP_CHECK(hipSetDevice(m_device));
        for (int i = 0; i < m_n_lanes; i++) HIP_CHECK(hipStreamSynchronize(m_lane[i].stream));
        check_waits();
    }

    // A fused launch whose work-groups gave up waiting for each other has produced nothing
    // usable; it says so through a word in mapped host memory.
    void check_waits() {
        if (__atomic_load_n(m_gave_up.p, __ATOMIC_RELAXED) != 0)
            throw std::runtime_error(
                "a fused transform + GEMM launch ran into its wait limit: the results of this "
                "handle are invalid (LZHIP_FUSE=0 runs the two kernels as separate launches)");
    }

    // Host-buffer forward.  Up to kIoSlots callers may be inside at once: each
    // copies into its own pinned staging, enqueues copy-in, forward and copy-out
    // on the stream under the pipe lock, and waits for its own event outside
    // the lock, so that the next batch is queued on the device while this one
    // runs and host-side copies overlap device work.
    void forward_batch(int n, const float* in, float* pol, float* val) override {
        run_host_batch(n, in, nullptr, false, 1.0f, pol, val);
    }

    // Bit-packed planes: 816 bytes per position travel instead of 26 KB; the first kernel
    // expands them.  Results are those of the float path on the same 0/1 planes.
    bool accepts_bits() const override { return true; }
    void run_bits(int n, const uint32_t* bits, bool heads, float temperature, float* out_a,
                  float* out_b) override {
        if (heads && !m_heads_ready) throw std::invalid_argument("push_heads has not been called");
        if (heads && !(temperature > 0.0f))
            throw std::invalid_argument("temperature must be positive");
        run_host_batch(n, nullptr, bits, heads, temperature, out_a, out_b);
    }

    // The same path with the heads computed on the device: policy [n][362] and the
    // tanh value [n] come back instead of the raw planes.
    void evaluate_heads_batch(int n, const float* in, float temperature, float* policy,
                              float* value) override {
        if (!m_heads_ready) throw std::invalid_argument("push_heads has not been called");
        if (!(temperature > 0.0f)) throw std::invalid_argument("temperature must be positive");
        run_host_batch(n, in, nullptr, true, temperature, policy, value);
    }

    void run_host_batch(int n, const float* in, const uint32_t* bits, bool heads,
                        float temperature, float* out_a, float* out_b) {
        check_ready(n);
        HIP_CHECK(hipSetDevice(m_device));
        IoSlot* sl = nullptr;
        {
            std::unique_lock<std::mutex> lk(m_slot_mu);
            m_slot_cv.wait(lk, [&] {
                for (int i = 0; i < m_n_lanes; i++)
                    if (!m_slot[i].busy) return true;
                return false;
            });
            for (int i = 0; i < m_n_lanes && !sl; i++)
                if (!m_slot[i].busy) sl = &m_slot[i];
            sl->busy = true;
        }
        struct Release {
            HIPPipeImpl* self;
            IoSlot* sl;
            ~Release() {
                {
                    std::lock_guard<std::mutex> lk(self->m_slot_mu);
                    sl->busy = false;
                }
                self->m_slot_cv.notify_all();
            }
        } release{this, sl};
        // sizes of the two results per position, both written by the device into hpol / hval
        const size_t na = heads ? 362 : 2 * kPts, nb = heads ? 1 : kPts;
        if (bits)
            std::memcpy(sl->hbits.p, bits, sizeof(uint32_t) * (size_t)n * kInputWords);
        else
            std::memcpy(sl->hin.p, in, sizeof(float) * (size_t)n * kInPlanes * kPts);
        {
            // each staging slot has a lane of its own: two batches run side by side
            Lane& ln = m_lane[sl - m_slot];
            std::lock_guard<std::mutex> lk(ln.mu);
            // Pinned host memory is mapped into the device's address space: the first
            // kernel reads the packed planes and the last ones write the results straight
            // through it, so that no copy command sits between this batch's kernels and
            // the next batch's (each one is a bubble of tens of microseconds on the
            // stream).  Float planes, 32 times larger, still go by copy.
            float* out_a_dev = heads ? sl->dpol.p : sl->hpol.p;   // raw planes: straight to host
            float* out_b_dev = heads ? sl->dval.p : sl->hval.p;
            if (bits) {
                run_forward(ln, n, nullptr, sl->hbits.p, out_a_dev, out_b_dev);
            } else {
                HIP_CHECK(hipMemcpyAsync(sl->din.p, sl->hin.p,
                                         sizeof(float) * (size_t)n * kInPlanes * kPts,
                                         hipMemcpyHostToDevice, ln.stream));
                run_forward(ln, n, sl->din.p, nullptr, out_a_dev, out_b_dev);
            }
            if (heads) {
                HeadParams hp{m_h[0].p, m_h[1].p, m_h[2].p, m_h[3].p, m_h[4].p,
                              m_h[5].p, m_h[6].p, m_h[7].p, m_h[8].p, m_h[9].p};
                launch_heads(sl->dpol.p, sl->dval.p, hp, temperature, sl->hpol.p, nullptr,
                             sl->hval.p, sl->dwork.p, n, ln.stream);
            }
            HIP_CHECK(hipGetLastError());
            HIP_CHECK(hipEventRecord(sl->done, ln.stream));
        }
        HIP_CHECK(hipEventSynchronize(sl->done));
        check_waits();
        std::memcpy(out_a, sl->hpol.p, sizeof(float) * (size_t)n * na);
        std::memcpy(out_b, sl->hval.p, sizeof(float) * (size_t)n * nb);
    }

    // -------------------------------------------------------------------
    void push_heads(const HeadWeightsHost& hw) override {
        Lane& ln = m_lane[0];
        std::lock_guard<std::mutex> lk(ln.mu);
        HIP_CHECK(hipSetDevice(m_device));
        auto up = [&](DevBuf<float>& d, const float* src, size_t n) {
            d.alloc(n);
            HIP_CHECK(hipMemcpy(d.p, src, n * sizeof(float), hipMemcpyHostToDevice));
        };
        up(m_h[0], hw.bn_pol_mean, 2);
        up(m_h[1], hw.bn_pol_scale, 2);
        {   // FC matrices go up in the operand order of the matrix instruction
            std::vector<float> t(head_fc_fragment_count(true));
            head_fc_fragments(hw.ip_pol_w, true, t.data());
            up(m_h[2], t.data(), t.size());
            t.assign(head_fc_fragment_count(false), 0.0f);
            head_fc_fragments(hw.ip1_val_w, false, t.data());
            up(m_h[6], t.data(), t.size());
        }
        up(m_h[3], hw.ip_pol_b, 362);
        up(m_h[4], hw.bn_val_mean, 1);
        up(m_h[5], hw.bn_val_scale, 1);
        up(m_h[7], hw.ip1_val_b, 256);
        up(m_h[8], hw.ip2_val_w, 256);
        up(m_h[9], hw.ip2_val_b, 1);
        const size_t B = (size_t)m_max_batch;
        m_dpolicy.alloc(B * 362);
        m_dlogits.alloc(B * 362);
        m_dvalue.alloc(B);
        m_dwork.alloc(B * (362 + 256));
        for (int i = 0; i < m_n_lanes; i++) m_slot[i].dwork.alloc(B * (362 + 256));
        m_heads_ready = true;
    }

    void evaluate_batch(int n, const float* in, float temperature, float* policy, float* value,
                        float* logits, float* pol, float* val) override {
        Lane& ln = m_lane[0];
        std::lock_guard<std::mutex> lk(ln.mu);
        check_ready(n);
        if (!m_heads_ready) throw std::invalid_argument("push_heads has not been called");
        if (!(temperature > 0.0f)) throw std::invalid_argument("temperature must be positive");
        HIP_CHECK(hipSetDevice(m_device));
        HIP_CHECK(hipMemcpyAsync(m_din.p, in, sizeof(float) * (size_t)n * kInPlanes * kPts,
                                 hipMemcpyHostToDevice, ln.stream));
        run_forward(ln, n, m_din.p, nullptr, m_dpol.p, m_dval.p);
        HeadParams hp{m_h[0].p, m_h[1].p, m_h[2].p, m_h[3].p, m_h[4].p,
                      m_h[5].p, m_h[6].p, m_h[7].p, m_h[8].p, m_h[9].p};
        launch_heads(m_dpol.p, m_dval.p, hp, temperature, m_dpolicy.p, m_dlogits.p, m_dvalue.p,
                     m_dwork.p, n, ln.stream);
        HIP_CHECK(hipGetLastError());
        HIP_CHECK(hipStreamSynchronize(ln.stream));
        HIP_CHECK(hipMemcpy(policy, m_dpolicy.p, sizeof(float) * (size_t)n * 362, hipMemcpyDeviceToHost));
        HIP_CHECK(hipMemcpy(value, m_dvalue.p, sizeof(float) * (size_t)n, hipMemcpyDeviceToHost));
        if (logits)
            HIP_CHECK(hipMemcpy(logits, m_dlogits.p, sizeof(float) * (size_t)n * 362, hipMemcpyDeviceToHost));
        if (pol)
            HIP_CHECK(hipMemcpy(pol, m_dpol.p, sizeof(float) * (size_t)n * 2 * kPts, hipMemcpyDeviceToHost));
        if (val)
            HIP_CHECK(hipMemcpy(val, m_dval.p, sizeof(float) * (size_t)n * kPts, hipMemcpyDeviceToHost));
    }

    float timed_evaluations(int n, int reps, const float* in, float temperature, float* policy,
                            float* value) override {
        Lane& ln = m_lane[0];
        std::lock_guard<std::mutex> lk(ln.mu);
        check_ready(n);
        if (!m_heads_ready) throw std::invalid_argument("push_heads has not been called");
        if (!(temperature > 0.0f)) throw std::invalid_argument("temperature must be positive");
        if (reps < 1 || reps > 100000) throw std::invalid_argument("reps out of range");
        HIP_CHECK(hipSetDevice(m_device));
        const size_t in_count = (size_t)n * kInPlanes * kPts;
        PinnedBuf<float> hin, hpolicy, hvalue;
        hin.alloc(in_count);
        hpolicy.alloc((size_t)n * 362);
        hvalue.alloc((size_t)n);
        std::memcpy(hin.p, in, in_count * sizeof(float));
        HeadParams hp{m_h[0].p, m_h[1].p, m_h[2].p, m_h[3].p, m_h[4].p,
                      m_h[5].p, m_h[6].p, m_h[7].p, m_h[8].p, m_h[9].p};
        HIP_CHECK(hipStreamSynchronize(ln.stream));
        HIP_CHECK(hipEventRecord(m_ev_start[0], ln.stream));
        for (int r = 0; r < reps; r++) {
            HIP_CHECK(hipMemcpyAsync(m_din.p, hin.p, in_count * sizeof(float),
                                     hipMemcpyHostToDevice, ln.stream));
            run_forward(ln, n, m_din.p, nullptr, m_dpol.p, m_dval.p);
            launch_heads(m_dpol.p, m_dval.p, hp, temperature, m_dpolicy.p, nullptr, m_dvalue.p,
                         m_dwork.p, n, ln.stream);
            HIP_CHECK(hipMemcpyAsync(hpolicy.p, m_dpolicy.p, sizeof(float) * (size_t)n * 362,
                                     hipMemcpyDeviceToHost, ln.stream));
            HIP_CHECK(hipMemcpyAsync(hvalue.p, m_dvalue.p, sizeof(float) * (size_t)n,
                                     hipMemcpyDeviceToHost, ln.stream));
        }
        HIP_CHECK(hipGetLastError());
        HIP_CHECK(hipEventRecord(m_ev_stop[0], ln.stream));
        HIP_CHECK(hipEventSynchronize(m_ev_stop[0]));
        float ms = 0.0f;
        HIP_CHECK(hipEventElapsedTime(&ms, m_ev_start[0], m_ev_stop[0]));
        std::memcpy(policy, hpolicy.p, sizeof(float) * (size_t)n * 362);
        std::memcpy(value, hvalue.p, sizeof(float) * (size_t)n);
        return ms;
    }

    // -------------------------------------------------------------------
    void debug_layer(int layer, int n, const float* act_in, const float* res, float* Vout,
                     float* Mout, float* Yout) override {
        Lane& ln = m_lane[0];
        std::lock_guard<std::mutex> lk(ln.mu);
        check_ready(n);
        if (layer < 0 || layer >= (int)m_layers.size()) throw std::invalid_argument("bad layer");
        HIP_CHECK(hipSetDevice(m_device));
        Layer& L = m_layers[layer];
        const int F = m_filters, C = L.C, Cp = L.Cp;
        const int Tu = n * kTilesPerBoard;
        // stage fp32 NCHW planes through the V buffer's tail?  No: use a scratch buffer.
        DevBuf<float> d_planes, d_res, d_sc, d_mn;
        d_planes.alloc((size_t)n * C * kPts);
        HIP_CHECK(hipMemcpy(d_planes.p, act_in, sizeof(float) * (size_t)n * C * kPts, hipMemcpyHostToDevice));
        P* a_in = (layer == 0) ? ln.act0.p : ln.act[0].p;
        launch_pack_input<P>(d_planes.p, a_in, n, C, Cp, ln.stream, nullptr);
        const P* r = nullptr;
        if (res) {
            d_res.alloc((size_t)n * F * kPts);
            HIP_CHECK(hipMemcpy(d_res.p, res, sizeof(float) * (size_t)n * F * kPts, hipMemcpyHostToDevice));
            launch_pack_input<P>(d_res.p, ln.act[1].p, n, F, m_Fp, ln.stream, nullptr);
            r = ln.act[1].p;
        }
        std::vector<float> sc(m_Fp, 0.0f), mn(m_Fp, 0.0f);
        for (int k = 0; k < F; k++) { sc[k] = L.scale[k]; mn[k] = L.mean[k]; }
        d_sc.alloc(m_Fp); d_mn.alloc(m_Fp);
        HIP_CHECK(hipMemcpy(d_sc.p, sc.data(), sizeof(float) * m_Fp, hipMemcpyHostToDevice));
        HIP_CHECK(hipMemcpy(d_mn.p, mn.data(), sizeof(float) * m_Fp, hipMemcpyHostToDevice));
        launch_in_transform<P>(a_in, ln.V.p, n, Cp, m_Tp, ln.stream, nullptr);
        // The layout a forward of n boards keeps its tiles in: the GEMM and the output
        // transform run as they do there.  In a forward a tower layer's V comes slab by slab
        // from the fused transform; here the input transform's rows are re-laid on the host.
        int slab = 0;
        if constexpr (sizeof(P) == 2) {
            if (m_slab && L.Uf.p != nullptr && gemm_stream_shape(Tu, Cp, m_Fp, 2))
                slab = tile_slab(n, m_Fp, 2, true);
        }
        std::vector<P> v_rows;
        if (Vout || (slab != 0 && Cp != 64)) {
            v_rows.resize((size_t)kPos * m_Tp * Cp);
            HIP_CHECK(hipStreamSynchronize(ln.stream));
            HIP_CHECK(hipMemcpy(v_rows.data(), ln.V.p, v_rows.size() * sizeof(P), hipMemcpyDeviceToHost));
        }
        if (slab != 0 && Cp != 64) {
            std::vector<P> g(v_rows.size());
            for (int p = 0; p < kPos; p++)
                for (int t = 0; t < m_Tp; t++)
                    for (int c = 0; c < Cp; c++)
                        g[(((size_t)p * (Cp / slab) + c / slab) * m_Tp + t) * slab + c % slab] =
                            v_rows[((size_t)p * m_Tp + t) * Cp + c];
            HIP_CHECK(hipMemcpy(ln.V.p, g.data(), g.size() * sizeof(P), hipMemcpyHostToDevice));
        }
        launch_gemm<P>(ln.V.p, L.U.p, L.Uf.p, ln.M.p, Tu, m_Tp, Cp, m_Fp, ln.stream, nullptr, slab);
        launch_out_transform<P>(ln.M.p, r, ln.act[2].p, d_sc.p, d_mn.p, 1.0f, n, m_Fp, m_Tp,
                                ln.stream, nullptr, slab);
        HIP_CHECK(hipGetLastError());
        HIP_CHECK(hipStreamSynchronize(ln.stream));
        const int T = n * kTilesPerBoard;
        if (Vout) {
            const std::vector<P>& h = v_rows;
            for (int t = 0; t < T; t++)
                for (int p = 0; p < kPos; p++)
                    for (int c = 0; c < C; c++)
                        Vout[(((size_t)(t / 25) * kPos + p) * C + c) * 25 + t % 25] =
                            (float)h[((size_t)p * m_Tp + t) * Cp + c];
        }
        if (Mout) {
            std::vector<P> h((size_t)kPos * m_Tp * m_Fp);
            HIP_CHECK(hipMemcpy(h.data(), ln.M.p, h.size() * sizeof(P), hipMemcpyDeviceToHost));
            for (int t = 0; t < T; t++)
                for (int p = 0; p < kPos; p++)
                    for (int k = 0; k < F; k++)
                        Mout[(((size_t)(t / 25) * kPos + p) * F + k) * 25 + t % 25] = (float)
                            (slab != 0 ? h[(((size_t)p * (m_Fp / slab) + k / slab) * m_Tp + t) * slab + k % slab]
                                       : h[((size_t)p * m_Tp + t) * m_Fp + k]);
        }
        if (Yout) {
            std::vector<P> h((size_t)n * kPts * m_Fp);
            HIP_CHECK(hipMemcpy(h.data(), ln.act[2].p, h.size() * sizeof(P), hipMemcpyDeviceToHost));
            for (int b = 0; b < n; b++)
                for (int pt = 0; pt < kPts; pt++)
                    for (int k = 0; k < F; k++)
                        Yout[((size_t)b * F + k) * kPts + pt] =
                            (float)h[((size_t)b * kPts + pt) * m_Fp + k];
        }
    }

    // -------------------------------------------------------------------
    void profile_forward(int n, const float* d_in, float* d_pol, float* d_val, float* ms,
                         int* launches) override {
        Lane& ln = m_lane[0];
        std::lock_guard<std::mutex> lk(ln.mu);
        check_ready(n);
        HIP_CHECK(hipSetDevice(m_device));
        if ((int)m_layers.size() * 3 + 2 > kTimerPool)
            throw std::invalid_argument("network too deep for the timer pool");
        m_timer_used = 0;
        enqueue_forward(ln, n, d_in, nullptr, d_pol, d_val, true);
        HIP_CHECK(hipGetLastError());
        HIP_CHECK(hipStreamSynchronize(ln.stream));
        for (int k = 0; k < LZHIP_K_COUNT; k++) { ms[k] = 0.0f; launches[k] = 0; }
        for (int i = 0; i < m_timer_used; i++) {
            float t = 0.0f;
            HIP_CHECK(hipEventElapsedTime(&t, m_ev_start[i], m_ev_stop[i]));
            ms[m_timer_class[i]] += t;
            launches[m_timer_class[i]]++;
        }
    }

private:
    typedef std::tuple<int, const void*, float*, float*> GraphKey;
    // A lane is a stream with the working buffers of one forward.  Two batches on two
    // lanes run side by side on the device: each kernel's start-up and tail overlap with
    // the other lane's work, which a single chain of dependent kernels cannot do.
    // Lane 0 also serves calibration, profiling and the single-batch entry points.
    struct Lane {
        hipStream_t stream = nullptr;
        std::mutex mu;  // serialises enqueues on this lane
        DevBuf<P> act0, act[3], V, M;
        DevBuf<unsigned long long> flags;   // fused launches: one word per (board, channel group)
        unsigned long long epoch = 0;       // grows by one per fused launch (under mu)
        hipEvent_t last = nullptr;          // recorded behind the lane's latest forward
        std::map<GraphKey, hipGraphExec_t> graphs;
    };
    static constexpr int kLanes = 3;   // upper bound; m_n_lanes are in use

    // The working buffers of one forward as plain pointers: a lane's own allocations
    // or the static array.  Tp = rows of V and M per Winograd position.
    struct Work {
        hipStream_t stream = nullptr;
        P *act0 = nullptr, *act[3] = {nullptr, nullptr, nullptr}, *V = nullptr, *M = nullptr;
        int Tp = 0;
        // what a fused transform + GEMM launch synchronises through; null: separate launches
        unsigned long long* flags = nullptr;
        unsigned long long* epoch = nullptr;
        bool alone = false;   // no other lane had work on the device when this one was enqueued
    };
    Work work_of(Lane& ln) const {
        Work w;
        w.stream = ln.stream;
        w.act0 = ln.act0.p;
        for (int i = 0; i < 3; i++) w.act[i] = ln.act[i].p;
        w.V = ln.V.p;
        w.M = ln.M.p;
        w.Tp = m_Tp;
        w.flags = ln.flags.p;
        w.epoch = &ln.epoch;
        // (an event that was never recorded reads as complete)
        w.alone = true;
        for (int i = 0; i < m_n_lanes; i++)
            if (&m_lane[i] != &ln && hipEventQuery(m_lane[i].last) != hipSuccess) w.alone = false;
        (void)hipGetLastError();   // hipErrorNotReady is an answer, not a failure
        return w;
    }

    struct Layer {
        int C = 0, Cp = 0;
        DevBuf<P> U;
        DevBuf<P> Uf;                         // fragment order (streaming GEMM), may be empty
        std::vector<float> mean, scale;       // as pushed (unscaled)
        DevBuf<float> d_mean, d_scale;        // with activation scales folded in
        float rfac = 1.0f;
    };

    void check_ready(int n) const {
        if (!m_ready) throw std::invalid_argument("push_weights has not been called");
        if (n < 1 || n > m_max_batch) throw std::invalid_argument("batch size out of range");
    }

    // BN parameters of layer l for stored activations x/s:
    //   out/s_out = relu(scale*s_in/s_out * (conv(x/s_in) - mean/s_in) + (s_res/s_out) * res/s_res)
    void upload_bn(int l) {
        Layer& L = m_layers[l];
        const float s_in = m_s[l], s_out = m_s[l + 1];
        std::vector<float> sc(m_Fp, 0.0f), mn(m_Fp, 0.0f);
        for (int k = 0; k < m_filters; k++) {
            sc[k] = L.scale[k] * (s_in / s_out);
            mn[k] = L.mean[k] / s_in;
        }
        const bool second = l >= 2 && (l % 2) == 0;
        L.rfac = second ? m_s[l - 1] / s_out : 1.0f;
        HIP_CHECK(hipMemcpy(L.d_scale.p, sc.data(), sizeof(float) * m_Fp, hipMemcpyHostToDevice));
        HIP_CHECK(hipMemcpy(L.d_mean.p, mn.data(), sizeof(float) * m_Fp, hipMemcpyHostToDevice));
    }

    LaunchTimer* timer(bool timed, int cls) {
        if (!timed) return nullptr;
        const int i = m_timer_used++;
        m_timer_class[i] = cls;
        m_timer.start = m_ev_start[i];
        m_timer.stop = m_ev_stop[i];
        return &m_timer;
    }

    // Activation buffer roles rotate: cur = block input, mid, nxt = block output.
    void run_conv(Lane& ln, int l, int n, const P* in, const P* res, P* out, bool timed) {
        Layer& L = m_layers[l];
        const int Tu = n * kTilesPerBoard;
        launch_in_transform<P>(in, ln.V.p, n, L.Cp, m_Tp, ln.stream, timer(timed, LZHIP_K_IN));
        launch_gemm<P>(ln.V.p, L.U.p, L.Uf.p, ln.M.p, Tu, m_Tp, L.Cp, m_Fp, ln.stream,
                       timer(timed, LZHIP_K_GEMM));
        launch_out_transform<P>(ln.M.p, res, out, L.d_scale.p, L.d_mean.p, L.rfac, n, m_Fp, m_Tp,
                                ln.stream, timer(timed, LZHIP_K_OUT));
    }

    // With LZHIP_GRAPH=1 the 165 launches of a forward are captured once per
    // (batch size, buffers) into a HIP graph and replayed, which takes the launch
    // work off the host thread.  Only kernel nodes are captured (no memsets or
    // copies).  On the device the replay measured no faster than stream launches
    // (the gaps between these kernels are drain and cache write-back, not launch
    // latency), so plain stream launches are the default.
    void clear_graphs(Lane& ln) {
        for (auto& kv : ln.graphs) (void)hipGraphExecDestroy(kv.second);
        ln.graphs.clear();
    }
    void clear_graphs() {
        for (auto& ln : m_lane) clear_graphs(ln);
    }
    // d_in: fp32 planes, or, when null, d_bits: the planes one bit per value
    void run_forward(Lane& ln, int n, const float* d_in, const uint32_t* d_bits, float* d_pol,
                     float* d_val) {
        if (!m_use_graph) {
            enqueue_forward(ln, n, d_in, d_bits, d_pol, d_val, false);
            return;
        }
        const GraphKey key(n, d_in ? (const void*)d_in : (const void*)d_bits, d_pol, d_val);
        auto it = ln.graphs.find(key);
        if (it == ln.graphs.end()) {
            if (ln.graphs.size() >= 64) clear_graphs(ln);
            hipGraph_t g = nullptr;
            hipGraphExec_t ge = nullptr;
            HIP_CHECK(hipStreamBeginCapture(ln.stream, hipStreamCaptureModeThreadLocal));
            enqueue_forward(ln, n, d_in, d_bits, d_pol, d_val, false);
            HIP_CHECK(hipStreamEndCapture(ln.stream, &g));
            const hipError_t e = hipGraphInstantiate(&ge, g, nullptr, nullptr, 0);
            (void)hipGraphDestroy(g);
            HIP_CHECK(e);
            it = ln.graphs.emplace(key, ge).first;
        }
        HIP_CHECK(hipGraphLaunch(it->second, ln.stream));
    }

    // Layer loop.  Every layer but the last ends in the fused kernel that turns
    // M_l straight into V_{l+1}; the spatial activation is written only where a
    // later layer adds it back as a skip connection (layer 0 and every block
    // output), and by the last layer for the 1x1 heads.
    void enqueue_forward(Lane& ln, int n, const float* d_in, const uint32_t* d_bits,
                         float* d_pol, float* d_val, bool timed) {
        enqueue_forward(work_of(ln), n, d_in, d_bits, d_pol, d_val, timed);
        hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
        HIP_CHECK(hipStreamIsCapturing(ln.stream, &cap));
        if (cap == hipStreamCaptureStatusNone) HIP_CHECK(hipEventRecord(ln.last, ln.stream));
    }
    void enqueue_forward(const Work& w, int n, const float* d_in, const uint32_t* d_bits,
                         float* d_pol, float* d_val, bool timed) {
        const int nl = (int)m_layers.size();
        const int Tu = n * kTilesPerBoard;
        if (d_in)
            launch_pack_input<P>(d_in, w.act0, n, kInPlanes, m_C0p, w.stream,
                                 timer(timed, LZHIP_K_PACK));
        else
            launch_pack_input_bits<P>(d_bits, w.act0, n, kInPlanes, m_C0p, w.stream,
                                      timer(timed, LZHIP_K_PACK));
        launch_in_transform<P>(w.act0, w.V, n, m_C0p, w.Tp, w.stream, timer(timed, LZHIP_K_IN));
        // Small batches of fp16 towers (xform_gemm_shape) keep their tile arrays slab by slab
        // (tile_slab) from the first GEMM's output to the last transform's input -- nothing
        // outside this function sees them -- and send the transform of layer l and the GEMM
        // of layer l + 1 as one launch where xform_gemm_pays says that is faster: the fused
        // launch shortens a chain of dependent kernels, but its waiting work-groups hold
        // compute units that another lane's kernels could use, so the answer depends on
        // whether this forward has the device to itself.  All ways give the same bits.  No
        // fused launches under graph capture (the launch carries a number that has to differ
        // from launch to launch), when every launch is timed, or on the static working memory.
        int slab = 0;
        if constexpr (sizeof(P) == 2) {
            if (m_slab && m_layers.size() > 1 && m_layers[1].Uf.p != nullptr &&
                gemm_stream_shape(Tu, m_Fp, m_Fp, 2))
                slab = tile_slab(n, m_Fp, 2, w.alone);
        }
        bool fused = false;
        if constexpr (sizeof(P) == 2) {
            fused = m_fuse > 0 && !timed && !m_use_graph && w.flags != nullptr &&
                    xform_gemm_shape(n, m_Fp, 2) &&
                    (m_fuse > 1 || xform_gemm_pays(n, m_Fp, slab, w.alone));
        }
        // With the streaming GEMM the tower's layers work in place: M_l is written over V_l
        // and V_{l+1} over M_l (see the kernels), so a lane's tiles are one array instead of
        // two and the lanes' working sets (2 or 3 x 33 MB of tiles less at 64 boards) fit the
        // 256 MB memory-side cache.  Layer 0 reads 64 padded planes and keeps its own output.
        P* tiles = w.M;
        const bool in_place = m_in_place && !fused && m_layers.size() > 1 &&
                              gemm_stream_shape(Tu, m_Fp, m_Fp, (int)sizeof(P)) &&
                              m_layers[1].Uf.p != nullptr;
        int cur = 0, nxt = 1;  // block input (skip) / block output
        launch_gemm<P>(w.V, m_layers[0].U.p, m_layers[0].Uf.p, w.M, Tu, w.Tp, m_layers[0].Cp, m_Fp,
                       w.stream, timer(timed, LZHIP_K_GEMM), slab);
        for (int l = 0; l < nl; l++) {
            Layer& L = m_layers[l];
            const bool block_end = (l % 2) == 0;      // layer 0 and second convs
            const P* res = (block_end && l >= 2) ? w.act[cur] : nullptr;
            P* out = l == 0 ? w.act[cur] : w.act[nxt];
            if (l == nl - 1) {
                launch_out_transform<P>(tiles, res, out, L.d_scale.p, L.d_mean.p, L.rfac, n, m_Fp,
                                        w.Tp, w.stream, timer(timed, LZHIP_K_OUT), slab);
                launch_head_conv<P>(out, m_w3.p, m_s[nl], d_pol, d_val, n, m_Fp, w.stream,
                                    timer(timed, LZHIP_K_HEAD));
            } else {
                Layer& N = m_layers[l + 1];
                bool done = false;
                if constexpr (sizeof(P) == 2) {
                    if (fused) {
                        launch_xform_gemm(w.M, res, block_end ? out : nullptr, w.M, L.d_scale.p,
                                          L.d_mean.p, L.rfac, n, m_Fp, w.Tp, N.Uf.p, w.flags,
                                          ++*w.epoch, m_gave_up.p, w.stream, slab);
                        done = true;
                    }
                }
                if (!done) {
                    launch_out_in_transform<P>(tiles, res, block_end ? out : nullptr, w.V,
                                               L.d_scale.p, L.d_mean.p, L.rfac, n, m_Fp, w.Tp,
                                               w.stream, timer(timed, LZHIP_K_OUTIN), slab);
                    if (in_place) tiles = w.V;
                    launch_gemm<P>(w.V, N.U.p, N.Uf.p, tiles, Tu, w.Tp, N.Cp, m_Fp, w.stream,
                                   timer(timed, LZHIP_K_GEMM), slab);
                }
            }
            if (block_end && l >= 2) { const int o = cur; cur = nxt; nxt = o; }
        }
    }

    float absmax(const P* x, size_t count) {
        Lane& ln = m_lane[0];
        HIP_CHECK(hipMemsetAsync(m_scalar.p, 0, sizeof(float), ln.stream));
        launch_absmax<P>(x, count, m_scalar.p, ln.stream);
        float v = 0.0f;
        HIP_CHECK(hipMemcpyAsync(&v, m_scalar.p, sizeof(float), hipMemcpyDeviceToHost, ln.stream));
        HIP_CHECK(hipStreamSynchronize(ln.stream));
        return v;
    }

    // fp16 storage needs every stored activation to sit well inside the
    // half-precision range, also after the up-to-20x growth of the input
    // transform.  Convolution, ReLU and the residual add commute with positive
    // scaling, so layer l stores x_l / s_l with s_l a power of two chosen here
    // from a forward pass over synthetic positions; the scales are folded
    // into the batch-norm parameters and undone in the 1x1 heads, which is
    // exact in real arithmetic.  Trained networks keep |x| small and get
    // s_l = 1 (plain fp16 storage, as the reference's half pipeline).
    void calibrate() {
        Lane& ln = m_lane[0];
        const int n = m_max_batch < 8 ? m_max_batch : 8;
        std::vector<float> in((size_t)n * kInPlanes * kPts, 0.0f);
        uint64_t st = 0x9E3779B97F4A7C15ull;
        auto rnd = [&]() {
            st = st * 6364136223846793005ull + 1442695040888963407ull;
            return (double)(st >> 11) * (1.0 / 9007199254740992.0);
        };
        for (int b = 0; b < n; b++) {
            float* x = in.data() + (size_t)b * kInPlanes * kPts;
            for (int h = 0; h < 8; h++)
                for (int pt = 0; pt < kPts; pt++) {
                    const double u = rnd();
                    if (u < 0.2) x[h * kPts + pt] = 1.0f;
                    else if (u < 0.4) x[(8 + h) * kPts + pt] = 1.0f;
                }
            for (int pt = 0; pt < kPts; pt++) x[16 * kPts + pt] = 1.0f;
        }
        HIP_CHECK(hipMemcpy(m_din.p, in.data(), in.size() * sizeof(float), hipMemcpyHostToDevice));
        launch_pack_input<P>(m_din.p, ln.act0.p, n, kInPlanes, m_C0p, ln.stream, nullptr);

        const float target = 16.0f;
        const int nl = (int)m_layers.size();
        const size_t cnt = (size_t)n * kPts * m_Fp;
        int cur = 0, mid = 1, nxt = 2;
        auto settle = [&](int l, const P* src, const P* res, P* dst) {
            // provisional: keep the incoming scale, then correct from the measured range
            m_s[l + 1] = m_s[l];
            bool adjusted = false;
            for (int attempt = 0; attempt < 8; attempt++) {
                upload_bn(l);
                if (attempt == 0) {
                    run_conv(ln, l, n, src, res, dst, false);
                } else {
                    Layer& L = m_layers[l];
                    launch_out_transform<P>(ln.M.p, res, dst, L.d_scale.p, L.d_mean.p, L.rfac, n,
                                            m_Fp, m_Tp, ln.stream, nullptr);
                }
                const float mx = absmax(dst, cnt);
                if (!(mx < kActStoreMax)) {  // at the storage clamp (or NaN): coarser scale, try again
                    m_s[l + 1] *= 256.0f;
                    adjusted = false;
                    continue;
                }
                if (adjusted) return;  // re-run with the corrected scale is in range
                const float true_max = mx * m_s[l + 1];
                float want = 1.0f;
                if (true_max > target) want = std::exp2(std::ceil(std::log2(true_max / target)));
                if (want == m_s[l + 1]) return;
                m_s[l + 1] = want;
                adjusted = true;
            }
            throw std::runtime_error("activation-scale calibration did not converge");
        };
        settle(0, ln.act0.p, nullptr, ln.act[cur].p);
        for (int l = 1; l + 1 < nl; l += 2) {
            settle(l, ln.act[cur].p, nullptr, ln.act[mid].p);
            settle(l + 1, ln.act[mid].p, ln.act[cur].p, ln.act[nxt].p);
            const int o = cur; cur = nxt; nxt = o;
        }
    }

    static constexpr int kTimerPool = 512;
    int m_device, m_max_batch, m_filters;
    int m_Fp = 0, m_C0p = 0, m_Tp = 0;
    unsigned char* m_static = nullptr;   // this device's copy of the static working memory
    Lane m_lane[kLanes];
    int m_n_lanes = 2;
    DevBuf<float> m_din, m_dpol, m_dval, m_w3, m_scalar;  // evaluate_batch / calibration
    // Staging of forward_batch: kIoSlots batches may be between "copied in" and
    // "copied out" at once, slot i on lane i.
    struct IoSlot {
        PinnedBuf<float> hin, hpol, hval;
        PinnedBuf<uint32_t> hbits;
        DevBuf<float> din, dpol, dval;
        DevBuf<float> dwork;   // heads: logits and hidden units between the two kernels
        hipEvent_t done = nullptr;
        bool busy = false;
    };
    static constexpr int kIoSlots = kLanes;
    IoSlot m_slot[kIoSlots];
    std::mutex m_slot_mu;
    std::condition_variable m_slot_cv;
    std::vector<Layer> m_layers;
    std::atomic<bool> m_ready{false};   // set by a push_weights that ran to its end
    std::vector<float> m_s;  // activation scales, m_s[0] = input
    DevBuf<float> m_h[10], m_dpolicy, m_dlogits, m_dvalue, m_dwork;
    bool m_heads_ready = false;
    hipEvent_t m_ev_start[kTimerPool] = {}, m_ev_stop[kTimerPool] = {};
    int m_timer_class[kTimerPool] = {};
    int m_timer_used = 0;
    LaunchTimer m_timer;
    // LZHIP_GRAPH=1 (any value but 0): forwards replay a captured graph
    bool m_use_graph = [] {
        const char* e = std::getenv("LZHIP_GRAPH");
        return e != nullptr && std::atoi(e) != 0;
    }();
    int m_fuse = 1;                      // fused transform + GEMM launches (see enqueue_forward)
    bool m_in_place = true;              // tower layers keep V and M in one array (see enqueue_forward)
    bool m_slab = true;                  // small batches keep the tile arrays slab by slab (tile_slab)
    PinnedBuf<unsigned> m_gave_up;       // set by a fused launch whose wait ran into its limit
};

std::unique_ptr<HIPPipe> create_hip_pipe(int device, int precision, int max_batch, int filters) {
    if (precision == LZHIP_FP32)
        return std::unique_ptr<HIPPipe>(new HIPPipeImpl<float>(device, max_batch, filters));
    if (precision == LZHIP_FP16)
        return std::unique_ptr<HIPPipe>(new HIPPipeImpl<half_t>(device, max_batch, filters));
    throw std::invalid_argument("precision must be LZHIP_FP32 or LZHIP_FP16");
}

std::unique_ptr<BatchExecutor> make_hip_pipe(int device, int precision, int max_batch,
                                             int filters) {
    return create_hip_pipe(device, precision, max_batch, filters);
}

}  // namespace lzhip
