/*
 * lzhip.h -- C ABI of the MI355X (gfx950) network-forward backend for Leela Zero.
 *
 * The reference engine has no C ABI of its own: its backends are C++ classes
 * behind the abstract `ForwardPipe` (reference src/ForwardPipe.h:38-71).  Every
 * entry point below names the reference interface it stands in for, so that a
 * maintainer can bind it from the engine (see include/forward_pipe.h for the
 * C++ classes HIPScheduler / HIPPipe built on the same core).
 *
 * Conventions: plain pointers and sizes only; all functions return 0 on success
 * and a negative LZHIP_E* code on failure; no C++ exception crosses this
 * boundary; `lzhip_last_error()` returns a thread-local message for the last
 * failure on the calling thread.  Host pointers unless a name says `_device`.
 */
#ifndef LZHIP_H_INCLUDED
#define LZHIP_H_INCLUDED

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define LZHIP_OK 0
#define LZHIP_EINVAL (-1)   /* bad argument / wrong call order                       */
#define LZHIP_EDEVICE (-2)  /* HIP runtime error (message in lzhip_last_error)        */
#define LZHIP_EHALT (-3)    /* request woken by drain(): NetworkHaltException,        */
                            /* reference src/Network.h:66-67, OpenCLScheduler.cpp:274 */
#define LZHIP_ENOMEM (-4)

#define LZHIP_FP32 0 /* reference OpenCLScheduler<float>                              */
#define LZHIP_FP16 1 /* reference OpenCLScheduler<half>: fp16 storage, fp32 accumulate */

/* Fixed sizes of the boundary (reference src/config.h:48-53, src/Network.h:87-91). */
#define LZHIP_BOARD 19
#define LZHIP_NPTS 361
#define LZHIP_INPUT_CHANNELS 18
#define LZHIP_INPUT_SIZE (18 * 361) /* one position, NCHW, fp32                       */
#define LZHIP_POL_SIZE (2 * 361)    /* raw policy 1x1-conv planes                     */
#define LZHIP_VAL_SIZE 361          /* raw value 1x1-conv plane                       */
#define LZHIP_MOVES 362             /* 361 points + pass                              */
#define LZHIP_VALUE_LAYER 256

typedef struct lzhip_handle lzhip_handle;

/* Counters of the batching scheduler.  Replaces the reference's debug-only
 * batch_stats (src/OpenCLScheduler.h:43-49). */
typedef struct lzhip_stats {
    uint64_t requests;     /* forward() calls answered with a result                 */
    uint64_t batches;      /* device batches launched by the scheduler               */
    uint64_t batch_slots;  /* batches * max_batch : denominator of the fill ratio    */
    uint64_t halted;       /* forward() calls answered with LZHIP_EHALT              */
    uint32_t max_batch_seen;
    uint32_t max_batch;
} lzhip_stats;

/* ---- life cycle ------------------------------------------------------- */

/* Stands in for constructing the backend + ForwardPipe::initialize(channels)
 * (reference src/ForwardPipe.h:58, src/OpenCLScheduler.cpp:84-132,
 * src/Network.cpp:407-414).  `filters` = residual-tower width, `precision` =
 * LZHIP_FP32 / LZHIP_FP16 (reference cfg_precision, src/GTP.h:104-107),
 * `max_batch` = reference cfg_batch_size, `device` = HIP device ordinal
 * (reference --gpu).  Fails with LZHIP_EDEVICE when no gfx950 device or the
 * HIP runtime is unavailable: there is no CPU fallback. */
int lzhip_create(int filters, int precision, int max_batch, int device, lzhip_handle** out);

/* Network::initialize from a weights file (reference src/Network.cpp:351-405
 * load_network_file, :225-349 load_v1_network, :540-576 preparation): reads a
 * Leela Zero weights file (text, plain or gzip, format 1 or 2), detects filters and
 * residual blocks from it as the engine does, applies the Winograd transform of the
 * filters, 1/sqrt(var + 1e-5) and the folding of the conv biases into the batch-norm
 * means, creates the handle and pushes tower weights and head parameters
 * (lzhip_push_heads); format 2 sets lzhip_set_value_head_not_stm.  A file the
 * engine would refuse gives LZHIP_EINVAL with the engine's message ("Weights file is
 * the wrong version.", "Inconsistent number of weights in the file.", "Failed to
 * parse weight file. Error on line N.", "The weights file is not for 19x19 boards.",
 * "Could not open weights file: ...") before any device is touched.  filters and
 * blocks may be NULL. */
int lzhip_create_from_file(const char* path, int precision, int max_batch, int device,
                           lzhip_handle** out, int* filters, int* blocks);

/* Destructor of the backend (reference src/OpenCLScheduler.cpp:134-144):
 * wakes and joins the worker, pending requests finish with LZHIP_EHALT. */
int lzhip_destroy(lzhip_handle* h);

/* ForwardPipe::push_weights (reference src/ForwardPipe.h:65-67; contents of
 * ForwardPipeWeights src/ForwardPipe.h:40-54; call site src/Network.cpp:411).
 * U[l]        Winograd-domain filters [36][C_in][filters], filters fastest,
 *             C_in = 18 for l = 0 and `filters` otherwise (src/Network.cpp:215)
 * bn_mean[l]  [filters], conv bias already folded in   (src/Network.cpp:554-566)
 * bn_scale[l] [filters], already 1/sqrt(var + 1e-5)    (src/Network.cpp:151-157)
 * pol_w [2][filters], val_w [filters]  1x1 head convolutions, biases are zero
 * n_layers = 1 + 2 * residual blocks.  Data is copied; call exactly once. */
int lzhip_push_weights(lzhip_handle* h, int n_layers, const float* const* U,
                       const float* const* bn_mean, const float* const* bn_scale,
                       const float* pol_w, const float* val_w);

/* ---- evaluation ------------------------------------------------------- */

/* ForwardPipe::forward (reference src/ForwardPipe.h:62-64, scheduler
 * implementation src/OpenCLScheduler.cpp:256-277): one position, blocking,
 * callable from many threads at once; requests are batched on the device.
 * in[6498] -> pol[722], val[361] (raw 1x1 outputs, caller-allocated,
 * src/Network.cpp:819-829).  Returns LZHIP_EHALT if woken by lzhip_drain. */
int lzhip_forward(lzhip_handle* h, const float* in, float* pol, float* val);

/* Batch executor under the scheduler: OpenCL_Network::forward(batch)
 * (reference src/OpenCL.cpp:142-329).  n <= max_batch positions, host
 * buffers, blocking (H2D + tower + 1x1 heads + D2H).  Thread-safe: as many
 * callers as the handle has lanes are served side by side, further ones
 * wait.  Does not go through the request queue. */
int lzhip_forward_batch(lzhip_handle* h, int n, const float* in, float* pol, float* val);

/* Same executor on buffers that already live in device memory (the reference
 * keeps them in its OpenCLContext, src/OpenCL.h:64-84).  d_in fp32
 * [n][18][361], d_pol fp32 [n][722], d_val fp32 [n][361].  Enqueues on the
 * handle's stream and returns without waiting; lzhip_sync waits. */
int lzhip_forward_batch_device(lzhip_handle* h, int n, const void* d_in, void* d_pol,
                               void* d_val);
/* The handle owns lzhip_lanes(h) lanes: a stream each, with the working buffers of
 * one forward, as each batch worker of the reference owns an OpenCLContext with its
 * command queue and buffers (src/OpenCL.h:64-84, src/OpenCLScheduler.cpp:113-130,
 * :291).  Forwards enqueued on different lanes run side by side on the device, and
 * since a chain of dependent kernels leaves the device partly idle at every kernel
 * boundary, two batches on two lanes finish sooner than the same two on one.
 * A handle has two lanes, three when its max_batch is at most 48 (small batches leave
 * more of the device idle).  lzhip_forward_batch_device is lane 0; lzhip_forward_batch
 * and the request queue use one lane per batch in flight. */
int lzhip_lanes(lzhip_handle* h);
int lzhip_forward_batch_device_lane(lzhip_handle* h, int lane, int n, const void* d_in,
                                    void* d_pol, void* d_val);
/* No counterpart in the reference.  For callers that cannot allocate device memory at
 * the time of the call -- code under HIP graph capture, tight serving loops, harnesses
 * that forbid hipMalloc: lzhip_forward_batch_device (lane 0's stream, same arguments,
 * same results bit for bit) with every working buffer of the forward (packed planes,
 * activations, the Winograd tile arrays V and M) in a static device array of
 * 28 485 632 bytes that each GPU holds from library load to process end, instead of
 * the lane's allocated buffers.  The call launches kernels and nothing else.
 * Limits: 1 <= n <= LZHIP_NOALLOC_MAX_BATCH (and <= max_batch), networks of up to
 * LZHIP_NOALLOC_MAX_FILTERS filters; anything larger returns LZHIP_EINVAL with a
 * message.  All calls on one GPU share the array, from whatever handle: the library
 * orders them on the device (each call's kernels wait, through one event per GPU, for
 * the kernels of the call enqueued before it), so calls from several handles or threads
 * of one process do not overwrite each other's tiles; they do not run side by side
 * either.  While the lane's stream is being captured into a graph that ordering is left
 * out (no event is recorded into the capture): replays of such a graph that overlap
 * with other users of the array race.  Two processes on one GPU each hold their own
 * copy of the array.  Returns without waiting; lzhip_sync waits. */
#define LZHIP_NOALLOC_MAX_BATCH 8
#define LZHIP_NOALLOC_MAX_FILTERS 256
int lzhip_forward_batch_device_noalloc(lzhip_handle* h, int n, const void* d_in, void* d_pol,
                                       void* d_val);
/* Waits for the work enqueued on every lane. */
int lzhip_sync(lzhip_handle* h);
/* The hipStream_t of lane 0 (for callers that record events). */
void* lzhip_stream(lzhip_handle* h);

/* ForwardPipe::drain / resume (reference src/ForwardPipe.h:69-70,
 * src/OpenCLScheduler.cpp:411-441, callers src/UCTSearch.cpp:828-832). */
int lzhip_drain(lzhip_handle* h);
int lzhip_resume(lzhip_handle* h);

int lzhip_get_stats(lzhip_handle* h, lzhip_stats* out);
int lzhip_reset_stats(lzhip_handle* h);
/* The reference's global batch_stats (src/OpenCLScheduler.h:43-49, printed after every
 * search, src/UCTSearch.cpp:855-860), over every handle of the process since it started:
 * out[0] = device batches of one position (single_evals), out[1] = batches of more
 * (batch_evals), out[2] = positions in all batches, out[3] = batches x max_batch. */
int lzhip_process_batch_stats(uint64_t out[4]);

/* ---- heads computed on the device (reference computes them on the host,
 * src/Network.cpp:833-851) ------------------------------------------------ */

/* Head parameters as Network holds them (reference src/Network.h:166-183),
 * after the same preprocessing as src/Network.cpp:351-352,568-576:
 * bn_*_scale = 1/sqrt(var+1e-5), 1x1 conv biases folded into bn_*_mean.
 * ip_pol_w [362][722], ip1_val_w [256][361], ip2_val_w [256].  The arrays are
 * copied; call it while no evaluation that uses the heads is in flight. */
int lzhip_push_heads(lzhip_handle* h, const float* bn_pol_mean, const float* bn_pol_scale,
                     const float* ip_pol_w, const float* ip_pol_b, const float* bn_val_mean,
                     const float* bn_val_scale, const float* ip1_val_w,
                     const float* ip1_val_b, const float* ip2_val_w, const float* ip2_val_b);

/* forward_batch + the arithmetic of Network::get_output_internal
 * (reference src/Network.cpp:833-851, without the symmetry un-rotation):
 * policy[n][362] = softmax(FC(relu(bn(pol))) / temperature),
 * value[n] = tanh(FC(relu(FC(relu(bn(val)))))) -- winrate is (1+value)/2.
 * Optional outputs may be NULL: logits[n][362], pol[n][722], val[n][361]. */
int lzhip_evaluate_batch(lzhip_handle* h, int n, const float* in, float temperature,
                         float* policy, float* value, float* logits, float* pol, float* val);

/* Measurement: `reps` evaluations of the same n positions one after the other on lane 0,
 * each of them host-to-device copy of the planes (from pinned memory), tower, heads on
 * the device, device-to-host copy of policy [n][362] and value [n] (to pinned memory),
 * bracketed by two events on that stream; *ms = time between the events.  policy and
 * value receive the last evaluation's results.  The counterpart of timing
 * OpenCL_Network::forward from its first enqueueWriteBuffer to the end of its blocking
 * read (reference src/OpenCL.cpp:208-216,312-318), heads included.  Needs lzhip_push_heads. */
int lzhip_timed_evaluations(lzhip_handle* h, int n, int reps, const float* in,
                            float temperature, float* policy, float* value, float* ms);

/* One position through the batching queue with the heads computed on the
 * device: the whole of Network::get_output_internal's arithmetic (reference
 * src/Network.cpp:824-851) except the symmetry un-rotation, as one blocking,
 * thread-safe call.  policy [362] (index 361 = pass), *value = tanh output
 * (winrate = (1 + value) / 2).  Requests of this kind are batched among
 * themselves; needs lzhip_push_heads.  Returns LZHIP_EHALT while drained. */
int lzhip_forward_eval(lzhip_handle* h, const float* in, float temperature, float* policy,
                       float* value);

/* ---- weight preparation on the host (no device needed) ----------------- */

/* Network::winograd_transform_f (reference src/Network.cpp:159-223):
 * f [outputs][channels][3][3] -> U [36][channels][outputs]. */
int lzhip_winograd_transform_f(const float* f, int outputs, int channels, float* U);
/* process_bn_var (reference src/Network.cpp:151-157), in place. */
int lzhip_process_bn_var(float* w, int n);
/* Utils::ceilMultiple (reference src/Utils.cpp:208-215): a rounded up to a multiple of b
 * (b > 0), the helper the reference pads its GEMM dimensions with (src/OpenCL.cpp:380-382).
 * This library pads with it too: filters to 64 channels, tile rows to 256; b == 0 returns a. */
size_t lzhip_ceil_multiple(size_t a, size_t b);

/* ---- introspection used by the parity tests and the bench --------------- */

/* Runs conv layer `layer` alone on n positions and returns every stage in the
 * reference's own layouts (src/CPUPipe.cpp:164-174, :196-202, :273-280):
 * act_in [n][C_in][361] (C_in = 18 for layer 0) -> V [n][36][C_in][25],
 * M [n][36][filters][25], Y [n][filters][361] after BN (+res) + ReLU.
 * res [n][filters][361] or NULL.  Activation scaling is off in this call. */
int lzhip_debug_layer(lzhip_handle* h, int layer, int n, const float* act_in, const float* res,
                      float* V, float* M, float* Y);

/* Per-layer activation scales chosen for fp16 storage (all 1 in fp32):
 * out[n_layers + 1]; out[0] is the input scale, out[l + 1] that of layer l. */
int lzhip_get_act_scales(lzhip_handle* h, float* out, int n);

/* Kernel classes of the tower, for timing. */
#define LZHIP_K_PACK 0      /* NCHW fp32 input -> channels-last storage type   */
#define LZHIP_K_IN 1        /* Winograd input transform                        */
#define LZHIP_K_GEMM 2      /* 36-way batched MFMA GEMM                        */
#define LZHIP_K_OUT 3       /* output transform + BN + residual + ReLU         */
#define LZHIP_K_HEAD 4      /* 1x1 policy/value convolutions                   */
#define LZHIP_K_OUTIN 5     /* output transform fused with the next input one  */
#define LZHIP_K_COUNT 6

/* One forward of n device-resident positions with every kernel launch timed
 * individually by the device's own begin/end timestamps.  ms[LZHIP_K_COUNT]
 * receives the summed duration per class, launches[...] the launch counts. */
int lzhip_profile_forward(lzhip_handle* h, int n, const void* d_in, void* d_pol, void* d_val,
                          float* ms, int* launches);

const char* lzhip_last_error(void);
const char* lzhip_version(void);

#ifdef __cplusplus
}
#endif
#endif
