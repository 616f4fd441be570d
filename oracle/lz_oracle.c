/*
 * lz_oracle.c -- TEST INFRASTRUCTURE, NOT PRODUCT CODE.
 *
 * A plain-C, CPU-only restatement of the algorithm of Leela Zero's CPU network
 * pipe and of the head arithmetic that sits directly above it.  It exists to
 * check the HIP path and to provide a CPU timing baseline.  Only the tests,
 * the smoke check and the bench's CPU-baseline leg may load it; the GPU
 * library never calls into this file.
 *
 * Each function names the reference lines whose arithmetic it follows
 * (paths are relative to the reference tree's src/ directory).  The code is
 * written from that arithmetic, batch-1 and per-call scratch like the
 * reference, but with its own structure.
 *
 * How each function is pinned (the reference ships no numeric test vectors
 * for this path, and its CPUPipe.cpp cannot be compiled in this image without
 * writing a stand-in cblas.h / Eigen, so it is treated as unbuildable):
 *   lzo_winograd_transform_f, lzo_transform_in, lzo_sgemm, lzo_transform_out:
 *       the chain must equal a direct zero-padded 3x3 correlation computed in
 *       float64 (tests/test_oracle.py), on random data, including the 19x19
 *       clipping of the last tile row/column;  the U / V / M index layouts
 *       are additionally pinned element-by-element against dense matrix
 *       products with the literal G, B^T, A^T matrices.
 *   lzo_batchnorm, lzo_convolve1, lzo_innerproduct, lzo_softmax, lzo_heads:
 *       textbook closed forms in numpy float64.
 *   lzo_forward: layer wiring checked against an independent float64 network
 *       built from direct convolutions (tests/test_oracle.py).
 *   Bit-exact agreement with the reference's BLAS/Eigen summation order is
 *   NOT claimed anywhere ("parity unpinned" at the last-ulp level); parity is
 *   claimed only to the tolerances written in the tests.
 */
#include <dlfcn.h>
#include <math.h>
#include <pthread.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <time.h>

#define BOARD 19
#define NPTS 361           /* config.h:48-53 NUM_INTERSECTIONS            */
#define MOVES 362          /* config.h:53 POTENTIAL_MOVES                 */
#define WM 4               /* Network.h:58 WINOGRAD_M                     */
#define ALPHA 6            /* Network.h:59 WINOGRAD_ALPHA                 */
#define WTILES 5           /* Network.h:60-61                             */
#define NTILE 36           /* Network.h:62 WINOGRAD_TILE                  */
#define NP 25              /* Network.h:63 WINOGRAD_P                     */
#define IN_CH 18           /* Network.h:88 INPUT_CHANNELS                 */
#define VALUE_LAYER 256    /* Network.h:91                                */
static const float SQ2 = 1.4142135623730951f; /* Network.h:64 */

/* ------------------------------------------------------------------ */
/* optional real BLAS: scipy's bundled OpenBLAS, found at run time      */
typedef void (*sgemm_fn)(int order, int ta, int tb, int m, int n, int k,
                         float alpha, const float* a, int lda, const float* b,
                         int ldb, float beta, float* c, int ldc);
static sgemm_fn g_sgemm = NULL;
static char g_blas_name[256] = "builtin";

/* Try to bind cblas_sgemm from a shared library given by path.
 * Returns 1 on success.  The reference pins OpenBLAS to one thread per call
 * (Network.cpp:499); we do the same if the setter is exported. */
int lzo_use_blas(const char* path) {
    void* h = dlopen(path, RTLD_NOW | RTLD_LOCAL);
    if (!h) return 0;
    const char* names[] = {"scipy_cblas_sgemm", "cblas_sgemm", NULL};
    const char* setters[] = {"scipy_openblas_set_num_threads",
                             "openblas_set_num_threads", NULL};
    for (int i = 0; names[i]; i++) {
        void* f = dlsym(h, names[i]);
        if (f) {
            g_sgemm = (sgemm_fn)f;
            for (int j = 0; setters[j]; j++) {
                void (*st)(int) = (void (*)(int))dlsym(h, setters[j]);
                if (st) { st(1); break; }
            }
            snprintf(g_blas_name, sizeof g_blas_name, "%s", names[i]);
            return 1;
        }
    }
    return 0;
}
void lzo_use_builtin(void) { g_sgemm = NULL; snprintf(g_blas_name, sizeof g_blas_name, "builtin"); }
const char* lzo_blas_name(void) { return g_blas_name; }

/* ------------------------------------------------------------------ */
/* Network.cpp:151-157  var -> 1/sqrt(var + 1e-5)                       */
void lzo_process_bn_var(float* w, int n) {
    const float eps = 1e-5f;
    for (int i = 0; i < n; i++) w[i] = 1.0f / sqrtf(w[i] + eps);
}

/* Network.cpp:159-223  U = G f G^T per (o, c); output index
 * U[(xi*6+nu)][c][o] (o fastest).  f is [o][c][3][3]. */
void lzo_winograd_transform_f(const float* f, int outputs, int channels, float* U) {
    const float G[ALPHA][3] = {
        {1.0f, 0.0f, 0.0f},
        {-2.0f / 3.0f, -SQ2 / 3.0f, -1.0f / 3.0f},
        {-2.0f / 3.0f, SQ2 / 3.0f, -1.0f / 3.0f},
        {1.0f / 6.0f, SQ2 / 6.0f, 1.0f / 3.0f},
        {1.0f / 6.0f, -SQ2 / 6.0f, 1.0f / 3.0f},
        {0.0f, 0.0f, 1.0f}};
    for (int c = 0; c < channels; c++) {
        for (int o = 0; o < outputs; o++) {
            const float* g = f + ((size_t)o * channels + c) * 9;
            float t[ALPHA][3];
            for (int i = 0; i < ALPHA; i++)
                for (int j = 0; j < 3; j++) {
                    float acc = 0.0f;
                    for (int k = 0; k < 3; k++) acc += G[i][k] * g[k * 3 + j];
                    t[i][j] = acc;
                }
            for (int xi = 0; xi < ALPHA; xi++)
                for (int nu = 0; nu < ALPHA; nu++) {
                    float acc = 0.0f;
                    for (int k = 0; k < 3; k++) acc += t[xi][k] * G[nu][k];
                    U[((size_t)(xi * ALPHA + nu) * channels + c) * outputs + o] = acc;
                }
        }
    }
}

/* CPUPipe.cpp:88-106  one 6-point 1-D input transform, o = B^T i       */
static inline void bt6(const float i[6], float o[6]) {
    float a = i[1] * -SQ2 + i[3] * (SQ2 / 2.0f);
    float b = i[2] * -2.0f + i[4] * 1.0f;
    o[0] = i[0] + i[2] * (-5.0f / 2.0f) + i[4];
    o[1] = a + b;
    o[2] = -a + b;
    float c = i[3] * SQ2 + i[1] * (-SQ2 / 2.0f);
    float d = i[2] * (-1.0f / 2.0f) + i[4];
    o[3] = c + d;
    o[4] = -c + d;
    o[5] = i[1] + i[3] * (-5.0f / 2.0f) + i[5];
}

/* CPUPipe.cpp:63-183  in [C][361] -> V[36][C][25], tile = by*5+bx.
 * Plane padded to 22x22 with a one-point zero halo at the top/left
 * (CPUPipe.cpp:70-74,111); tile (by,bx) starts at padded (4by,4bx). */
void lzo_transform_in(const float* in, float* V, int C) {
    enum { WP = 2 + WM * WTILES };
    for (int ch = 0; ch < C; ch++) {
        float pad[WP][WP];
        memset(pad, 0, sizeof pad);
        for (int y = 0; y < BOARD; y++)
            for (int x = 0; x < BOARD; x++) pad[y + 1][x + 1] = in[ch * NPTS + y * BOARD + x];
        for (int by = 0; by < WTILES; by++)
            for (int bx = 0; bx < WTILES; bx++) {
                float t1[ALPHA][ALPHA]; /* t1[row'][col] = (B^T d)          */
                for (int x = 0; x < ALPHA; x++) {
                    float col[6], o[6];
                    for (int y = 0; y < ALPHA; y++) col[y] = pad[WM * by + y][WM * bx + x];
                    bt6(col, o);
                    for (int y = 0; y < ALPHA; y++) t1[y][x] = o[y];
                }
                for (int y = 0; y < ALPHA; y++) { /* (B^T d) B, row by row   */
                    float o[6];
                    bt6(t1[y], o);
                    for (int x = 0; x < ALPHA; x++)
                        V[((size_t)(y * ALPHA + x) * C + ch) * NP + by * WTILES + bx] = o[x];
                }
            }
    }
}

/* CPUPipe.cpp:185-210  for each of the 36 positions:
 * M_b[K][25] = U_b^T (U_b is [C][K]) * V_b [C][25]. */
void lzo_sgemm(const float* U, const float* V, float* M, int C, int K) {
    for (int b = 0; b < NTILE; b++) {
        const float* u = U + (size_t)b * K * C;
        const float* v = V + (size_t)b * C * NP;
        float* m = M + (size_t)b * K * NP;
        if (g_sgemm) { /* RowMajor=101, Trans=112, NoTrans=111 */
            g_sgemm(101, 112, 111, K, NP, C, 1.0f, u, K, v, NP, 0.0f, m, NP);
            continue;
        }
        memset(m, 0, sizeof(float) * K * NP);
        for (int c = 0; c < C; c++) {
            const float* vr = v + c * NP;
            const float* ur = u + (size_t)c * K;
            for (int k = 0; k < K; k++) {
                const float w = ur[k];
                float* mr = m + k * NP;
                for (int p = 0; p < NP; p++) mr[p] += w * vr[p];
            }
        }
    }
}

/* CPUPipe.cpp:225-238  one 6->4 1-D output transform, o = A^T i        */
static inline void at6(const float i[6], float o[4]) {
    float t1p2 = (i[1] + i[2]) * (1.0f / 2.0f);
    float t1m2 = (i[1] - i[2]) * (SQ2 / 4.0f);
    float t3p4 = i[3] + i[4];
    float t3m4 = (i[3] - i[4]) * SQ2;
    o[0] = i[0] + t1p2 + t1p2 + t3p4;
    o[1] = t1m2 + t1m2 + t3m4;
    o[2] = t1p2 + t3p4 + t3p4;
    o[3] = t1m2 + t3m4 + t3m4 + i[5];
}

/* CPUPipe.cpp:212-284  M[36][K][25] -> Y[K][361]; tile (by,bx) writes the
 * 4x4 block at board (4by,4bx), clipped to 19x19 (CPUPipe.cpp:273-280). */
void lzo_transform_out(const float* M, float* Y, int K) {
    for (int k = 0; k < K; k++)
        for (int by = 0; by < WTILES; by++)
            for (int bx = 0; bx < WTILES; bx++) {
                const int b = by * WTILES + bx;
                float m[ALPHA][ALPHA], t[WM][ALPHA], o[WM][WM];
                for (int xi = 0; xi < ALPHA; xi++)
                    for (int nu = 0; nu < ALPHA; nu++)
                        m[xi][nu] = M[((size_t)(xi * ALPHA + nu) * K + k) * NP + b];
                for (int j = 0; j < ALPHA; j++) {
                    float col[6], r[4];
                    for (int i = 0; i < ALPHA; i++) col[i] = m[i][j];
                    at6(col, r);
                    for (int i = 0; i < WM; i++) t[i][j] = r[i];
                }
                for (int i = 0; i < WM; i++) at6(t[i], o[i]);
                for (int i = 0; i < WM; i++)
                    for (int j = 0; j < WM; j++) {
                        const int y = WM * by + i, x = WM * bx + j;
                        if (y < BOARD && x < BOARD) Y[k * NPTS + y * BOARD + x] = o[i][j];
                    }
            }
}

/* CPUPipe.cpp:352-377 and Network.cpp:639-664:
 * y = max(0, s*(y-mean) [+ res]).  ReLU always applied. */
void lzo_batchnorm(int channels, float* data, const float* means, const float* scales,
                   const float* eltwise) {
    for (int c = 0; c < channels; c++) {
        const float mean = means[c], s = scales[c];
        float* a = data + c * NPTS;
        if (!eltwise) {
            for (int b = 0; b < NPTS; b++) a[b] = fmaxf(0.0f, s * (a[b] - mean));
        } else {
            const float* r = eltwise + c * NPTS;
            for (int b = 0; b < NPTS; b++) a[b] = fmaxf(0.0f, (s * (a[b] - mean)) + r[b]);
        }
    }
}

/* CPUPipe.cpp:301-350 with filter_size 1 (Im2Col.h:82-88 is a copy):
 * out[o][p] = sum_c w[o][c] * in[c][p] + bias[o]. */
void lzo_convolve1(int outputs, int C, const float* in, const float* w, const float* bias,
                   float* out) {
    for (int o = 0; o < outputs; o++) {
        float* y = out + o * NPTS;
        for (int p = 0; p < NPTS; p++) y[p] = 0.0f;
        for (int c = 0; c < C; c++) {
            const float wv = w[o * C + c];
            const float* x = in + c * NPTS;
            for (int p = 0; p < NPTS; p++) y[p] += wv * x[p];
        }
        const float bv = bias ? bias[o] : 0.0f;
        for (int p = 0; p < NPTS; p++) y[p] += bv;
    }
}

/* The weights a pipe receives (ForwardPipe.h:40-54), as plain pointers.
 * U[l] is Winograd-domain [36][C_in][F] (l = 0: C_in = 18), bn_scale is
 * already 1/sqrt(var+eps), conv biases already folded into bn_mean. */
typedef struct {
    int filters;
    int n_layers; /* 1 + 2*blocks */
    const float* const* U;
    const float* const* bn_mean;
    const float* const* bn_scale;
    const float* pol_w; /* [2][F] */
    const float* val_w; /* [1][F] */
} lzo_net;

/* CPUPipe.cpp:379-428.  in [18][361] -> pol [2][361], val [361].
 * If trace != NULL it receives the activation after every conv layer
 * ([n_layers][F][361]) -- used only to calibrate/diagnose. */
void lzo_forward_trace(const lzo_net* net, const float* input, float* pol, float* val,
                       float* trace) {
    const int F = net->filters;
    const int cmax = F > IN_CH ? F : IN_CH;
    float* V = (float*)malloc(sizeof(float) * NTILE * cmax * NP);
    float* M = (float*)malloc(sizeof(float) * NTILE * F * NP);
    float* a = (float*)malloc(sizeof(float) * F * NPTS); /* current activation */
    float* t = (float*)malloc(sizeof(float) * F * NPTS); /* mid-block          */
    float* n = (float*)malloc(sizeof(float) * F * NPTS); /* block output       */

    lzo_transform_in(input, V, IN_CH);
    lzo_sgemm(net->U[0], V, M, IN_CH, F);
    lzo_transform_out(M, a, F);
    lzo_batchnorm(F, a, net->bn_mean[0], net->bn_scale[0], NULL);
    if (trace) memcpy(trace, a, sizeof(float) * F * NPTS);

    for (int l = 1; l + 1 < net->n_layers; l += 2) {
        lzo_transform_in(a, V, F);
        lzo_sgemm(net->U[l], V, M, F, F);
        lzo_transform_out(M, t, F);
        lzo_batchnorm(F, t, net->bn_mean[l], net->bn_scale[l], NULL);
        if (trace) memcpy(trace + (size_t)l * F * NPTS, t, sizeof(float) * F * NPTS);

        lzo_transform_in(t, V, F);
        lzo_sgemm(net->U[l + 1], V, M, F, F);
        lzo_transform_out(M, n, F);
        lzo_batchnorm(F, n, net->bn_mean[l + 1], net->bn_scale[l + 1], a);
        if (trace) memcpy(trace + (size_t)(l + 1) * F * NPTS, n, sizeof(float) * F * NPTS);
        float* sw = a; a = n; n = sw;
    }
    lzo_convolve1(2, F, a, net->pol_w, NULL, pol);
    lzo_convolve1(1, F, a, net->val_w, NULL, val);
    free(V); free(M); free(a); free(t); free(n);
}

void lzo_forward(const lzo_net* net, const float* input, float* pol, float* val) {
    lzo_forward_trace(net, input, pol, val, NULL);
}

/* Convenience for callers that cannot build the struct (ctypes). */
void lzo_forward_flat(int filters, int n_layers, const float* const* U,
                      const float* const* bn_mean, const float* const* bn_scale,
                      const float* pol_w, const float* val_w, const float* input, float* pol,
                      float* val, float* trace) {
    lzo_net net = {filters, n_layers, U, bn_mean, bn_scale, pol_w, val_w};
    lzo_forward_trace(&net, input, pol, val, trace);
}

/* Network.cpp:609-637  out = W[outputs][inputs] * in + b, optional ReLU. */
void lzo_innerproduct(int inputs, int outputs, int relu, const float* in, const float* W,
                      const float* b, float* out) {
    for (int o = 0; o < outputs; o++) {
        float acc = 0.0f;
        const float* w = W + (size_t)o * inputs;
        for (int i = 0; i < inputs; i++) acc += w[i] * in[i];
        float v = b[o] + acc;
        if (relu) v = fmaxf(0.0f, v);
        out[o] = v;
    }
}

/* Network.cpp:693-712 */
void lzo_softmax(const float* in, int n, float temperature, float* out) {
    float alpha = in[0];
    for (int i = 1; i < n; i++) alpha = in[i] > alpha ? in[i] : alpha;
    float denom = 0.0f;
    for (int i = 0; i < n; i++) {
        out[i] = expf((in[i] - alpha) / temperature);
        denom += out[i];
    }
    for (int i = 0; i < n; i++) out[i] /= denom;
}

/* Head parameters (Network.h:166-183).  bn_*_scale already 1/sqrt(var+eps);
 * 1x1 conv biases already folded into the means (Network.cpp:568-576). */
typedef struct {
    const float* bn_pol_mean;  /* [2]        */
    const float* bn_pol_scale; /* [2]        */
    const float* ip_pol_w;     /* [362][722] */
    const float* ip_pol_b;     /* [362]      */
    const float* bn_val_mean;  /* [1]        */
    const float* bn_val_scale; /* [1]        */
    const float* ip1_val_w;    /* [256][361] */
    const float* ip1_val_b;    /* [256]      */
    const float* ip2_val_w;    /* [256]      */
    const float* ip2_val_b;    /* [1]        */
} lzo_heads_w;

/* Network.cpp:833-851 (without the symmetry un-rotation, :855-861).
 * pol/val are the raw pipe outputs and are not modified.
 * Writes policy[362] (softmax), logits[362] (optional), value_tanh,
 * winrate = (1+tanh)/2, and the pre-tanh scalar. */
void lzo_heads(const lzo_heads_w* h, const float* pol, const float* val, float temperature,
               float* policy, float* logits, float* value_tanh, float* winrate,
               float* value_pre) {
    float p[2 * NPTS], v[NPTS], lg[MOVES], h1[VALUE_LAYER], o;
    memcpy(p, pol, sizeof p);
    memcpy(v, val, sizeof v);
    lzo_batchnorm(2, p, h->bn_pol_mean, h->bn_pol_scale, NULL);
    lzo_innerproduct(2 * NPTS, MOVES, 0, p, h->ip_pol_w, h->ip_pol_b, lg);
    lzo_softmax(lg, MOVES, temperature, policy);
    if (logits) memcpy(logits, lg, sizeof lg);
    lzo_batchnorm(1, v, h->bn_val_mean, h->bn_val_scale, NULL);
    lzo_innerproduct(NPTS, VALUE_LAYER, 1, v, h->ip1_val_w, h->ip1_val_b, h1);
    lzo_innerproduct(VALUE_LAYER, 1, 0, h1, h->ip2_val_w, h->ip2_val_b, &o);
    if (value_pre) *value_pre = o;
    const float th = tanhf(o);
    if (value_tanh) *value_tanh = th;
    if (winrate) *winrate = (1.0f + th) / 2.0f;
}

void lzo_heads_flat(const float* bn_pol_mean, const float* bn_pol_scale, const float* ip_pol_w,
                    const float* ip_pol_b, const float* bn_val_mean, const float* bn_val_scale,
                    const float* ip1_val_w, const float* ip1_val_b, const float* ip2_val_w,
                    const float* ip2_val_b, const float* pol, const float* val,
                    float temperature, float* policy, float* logits, float* value_tanh,
                    float* winrate, float* value_pre) {
    lzo_heads_w h = {bn_pol_mean, bn_pol_scale, ip_pol_w, ip_pol_b, bn_val_mean,
                     bn_val_scale, ip1_val_w, ip1_val_b, ip2_val_w, ip2_val_b};
    lzo_heads(&h, pol, val, temperature, policy, logits, value_tanh, winrate, value_pre);
}

/* ------------------------------------------------------------------ */
/* Timing harness shaped like Network::benchmark (Network.cpp:128-149):
 * `threads` workers pull evaluations from a shared counter until `total`
 * single-position forwards are done.  Returns wall seconds. */
typedef struct {
    const lzo_net* net;
    const float* inputs; /* [n_inputs][18][361] */
    int n_inputs, total;
    volatile int next;
    pthread_mutex_t mu;
    float* pol_out; /* optional [total][722] */
    float* val_out; /* optional [total][361] */
} bench_ctx;

static void* bench_worker(void* arg) {
    bench_ctx* c = (bench_ctx*)arg;
    float pol[2 * NPTS], val[NPTS];
    for (;;) {
        pthread_mutex_lock(&c->mu);
        int i = c->next;
        if (i < c->total) c->next = i + 1;
        pthread_mutex_unlock(&c->mu);
        if (i >= c->total) break;
        lzo_forward(c->net, c->inputs + (size_t)(i % c->n_inputs) * IN_CH * NPTS, pol, val);
        if (c->pol_out) memcpy(c->pol_out + (size_t)i * 2 * NPTS, pol, sizeof pol);
        if (c->val_out) memcpy(c->val_out + (size_t)i * NPTS, val, sizeof val);
    }
    return NULL;
}

double lzo_benchmark(int filters, int n_layers, const float* const* U,
                     const float* const* bn_mean, const float* const* bn_scale,
                     const float* pol_w, const float* val_w, const float* inputs, int n_inputs,
                     int total, int threads, float* pol_out, float* val_out) {
    lzo_net net = {filters, n_layers, U, bn_mean, bn_scale, pol_w, val_w};
    bench_ctx c;
    c.net = &net; c.inputs = inputs; c.n_inputs = n_inputs; c.total = total; c.next = 0;
    c.pol_out = pol_out; c.val_out = val_out;
    pthread_mutex_init(&c.mu, NULL);
    if (threads < 1) threads = 1;
    pthread_t* th = (pthread_t*)malloc(sizeof(pthread_t) * threads);
    struct timespec t0, t1;
    clock_gettime(CLOCK_MONOTONIC, &t0);
    for (int i = 0; i < threads; i++) pthread_create(&th[i], NULL, bench_worker, &c);
    for (int i = 0; i < threads; i++) pthread_join(th[i], NULL);
    clock_gettime(CLOCK_MONOTONIC, &t1);
    free(th);
    pthread_mutex_destroy(&c.mu);
    return (double)(t1.tv_sec - t0.tv_sec) + 1e-9 * (double)(t1.tv_nsec - t0.tv_nsec);
}
