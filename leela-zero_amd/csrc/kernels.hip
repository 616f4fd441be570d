// gfx950 (CDNA4) kernels of the Winograd F(4x4,3x3) residual tower.
//
// Arithmetic follows the reference CPU pipe (reference src/CPUPipe.cpp:63-284,
// :352-377) and its OpenCL twins (src/kernels/convolve3.opencl:47-79); the
// decomposition, layouts and launch shapes are this library's own.
#include "kernels.h"

#include <cstdlib>
#include <stdexcept>
#include <type_traits>

#include <hip/hip_ext.h>

namespace lzhip {

typedef _Float16 half_t;
typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef _Float16 half8v __attribute__((ext_vector_type(8)));
typedef float float4v __attribute__((ext_vector_type(4)));
typedef float float16v __attribute__((ext_vector_type(16)));
typedef int int4v __attribute__((ext_vector_type(4)));

#define SQ2 1.4142135623730951f
// Timeline hook for measurement builds (a harness that includes this file defines it to
// record a timestamp); expands to nothing in the library.
#ifndef LZ_STAMP
#define LZ_STAMP(i)
#endif
constexpr int kStoreThrough = 17;  // cache policy of a raw buffer store: sc0 | sc1 (write-through)

// ---------------------------------------------------------------------------
// Per-lane channel vector: how many consecutive channels one lane owns in the
// bandwidth-bound kernels (4 bytes per lane and access for both types).
template <typename P> struct ChanVec;
template <> struct ChanVec<float> {
    static constexpr int N = 1;
    static __device__ __forceinline__ void load(const float* p, float* o) { o[0] = *p; }
    static __device__ __forceinline__ void store(float* p, const float* v) { *p = v[0]; }
};
template <> struct ChanVec<half_t> {
    static constexpr int N = 2;
    static __device__ __forceinline__ void load(const half_t* p, float* o) {
        const half2v h = *reinterpret_cast<const half2v*>(p);
        o[0] = (float)h.x;
        o[1] = (float)h.y;
    }
    // Saturating: a value beyond the fp16 range is stored as +-65504, not inf.
    static __device__ __forceinline__ void store(half_t* p, const float* v) {
        half2v h;
        h.x = (half_t)fminf(fmaxf(v[0], -65504.0f), 65504.0f);
        h.y = (half_t)fminf(fmaxf(v[1], -65504.0f), 65504.0f);
        *reinterpret_cast<half2v*>(p) = h;
    }
};

template <typename P> __device__ __forceinline__ P to_storage(float v);
// Four consecutive storage elements as one LDS/global access.
template <typename P> struct Quad;
template <> struct Quad<float> { typedef float type __attribute__((ext_vector_type(4))); };
template <> struct Quad<_Float16> { typedef _Float16 type __attribute__((ext_vector_type(4))); };

template <> __device__ __forceinline__ float to_storage<float>(float v) { return v; }
template <> __device__ __forceinline__ half_t to_storage<half_t>(float v) {
    return (half_t)fminf(fmaxf(v, -65504.0f), 65504.0f);
}

// Stored activations are kept at or below kActStoreMax = 2040 < 65504 / 30.6 (30.6 = largest
// absolute row sum of B^T (x) B^T), so the input transform of a stored activation cannot
// leave the half-precision range and V needs no clamp of its own.  Every kernel that
// stores an activation (fused and unfused output transform) goes through this one clamp,
// and the activation-scale calibration measures through it.
template <typename P> __device__ __forceinline__ float act_clamp(float v);
template <> __device__ __forceinline__ float act_clamp<float>(float v) { return v; }
template <> __device__ __forceinline__ float act_clamp<half_t>(float v) {
    return fminf(v, kActStoreMax);
}
template <typename P> __device__ __forceinline__ P act_to_storage(float v) {
    return (P)act_clamp<P>(v);
}

// o = B^T i for one 6-vector (reference src/CPUPipe.cpp:88-106).
__device__ __forceinline__ void bt6(const float i0, const float i1, const float i2,
                                    const float i3, const float i4, const float i5, float& o0,
                                    float& o1, float& o2, float& o3, float& o4, float& o5) {
    const float a = i1 * -SQ2 + i3 * (SQ2 / 2.0f);
    const float b = i2 * -2.0f + i4;
    o0 = i0 + i2 * (-5.0f / 2.0f) + i4;
    o1 = a + b;
    o2 = -a + b;
    const float c = i3 * SQ2 + i1 * (-SQ2 / 2.0f);
    const float d = i2 * (-1.0f / 2.0f) + i4;
    o3 = c + d;
    o4 = -c + d;
    o5 = i1 + i3 * (-5.0f / 2.0f) + i5;
}

// o = A^T i for one 6-vector (reference src/CPUPipe.cpp:225-238; the same sums,
// associated so that they take twelve operations).
__device__ __forceinline__ void at6(const float i0, const float i1, const float i2,
                                    const float i3, const float i4, const float i5, float& o0,
                                    float& o1, float& o2, float& o3) {
    const float s12 = i1 + i2, d12 = i1 - i2;
    const float s34 = i3 + i4, d34 = i3 - i4;
    o0 = (i0 + s12) + s34;
    o1 = fmaf(d34, SQ2, d12 * (SQ2 / 2.0f));
    o2 = fmaf(s34, 2.0f, s12 * 0.5f);
    o3 = fmaf(d34, 2.0f * SQ2, fmaf(d12, SQ2 / 4.0f, i5));
}

// ---------------------------------------------------------------------------
template <typename K, typename... Args>
static inline void launch(K kernel, dim3 grid, dim3 block, hipStream_t s, LaunchTimer* t,
                          Args... args) {
    if (t && t->start) {
        hipExtLaunchKernelGGL(kernel, grid, block, 0, s, t->start, t->stop, 0, args...);
    } else {
        hipLaunchKernelGGL(kernel, grid, block, 0, s, args...);
    }
}

// ---------------------------------------------------------------------------
// Planes NCHW fp32 [n][C][361] -> channels-last storage type [n][361][Cp],
// channels C..Cp-1 zero.
template <typename P>
__global__ __launch_bounds__(256) void pack_input_k(const float* __restrict__ in,
                                                    P* __restrict__ act, int n, int C, int Cp) {
    const size_t gid = (size_t)blockIdx.x * 256 + threadIdx.x;
    const size_t total = (size_t)n * kPts * Cp;
    if (gid >= total) return;
    const int c = (int)(gid % Cp);
    const size_t bp = gid / Cp;
    const int pt = (int)(bp % kPts);
    const size_t b = bp / kPts;
    float v = 0.0f;
    if (c < C) v = in[(b * C + c) * kPts + pt];
    act[gid] = to_storage<P>(v);
}

template <typename P>
void launch_pack_input(const float* in, P* act, int n, int C, int Cp, hipStream_t s,
                       LaunchTimer* t) {
    const size_t total = (size_t)n * kPts * Cp;
    launch(pack_input_k<P>, dim3((unsigned)((total + 255) / 256)), dim3(256), s, t, in, act, n, C,
           Cp);
}

// The same from bit-packed planes: bit (c*361 + pt) of a board's kInputWords words is
// plane c at point pt (planes that hold only 0 and 1, which is what the engine feeds).
template <typename P>
__global__ __launch_bounds__(256) void pack_input_bits_k(const uint32_t* __restrict__ bits,
                                                         P* __restrict__ act, int n, int C,
                                                         int Cp) {
    const size_t gid = (size_t)blockIdx.x * 256 + threadIdx.x;
    const size_t total = (size_t)n * kPts * Cp;
    if (gid >= total) return;
    const int c = (int)(gid % Cp);
    const size_t bp = gid / Cp;
    const int pt = (int)(bp % kPts);
    const size_t b = bp / kPts;
    float v = 0.0f;
    if (c < C) {
        const int bit = c * kPts + pt;
        v = (float)((bits[b * kInputWords + (bit >> 5)] >> (bit & 31)) & 1u);
    }
    act[gid] = to_storage<P>(v);
}

template <typename P>
void launch_pack_input_bits(const uint32_t* bits, P* act, int n, int C, int Cp, hipStream_t s,
                            LaunchTimer* t) {
    const size_t total = (size_t)n * kPts * Cp;
    launch(pack_input_bits_k<P>, dim3((unsigned)((total + 255) / 256)), dim3(256), s, t, bits, act,
           n, C, Cp);
}

// ---------------------------------------------------------------------------
// Winograd input transform V = B^T d B (reference src/CPUPipe.cpp:63-183).
// One lane owns one tile and ChanVec<P>::N consecutive channels; consecutive
// lanes own consecutive channels, so every load and store of a wave covers a
// contiguous run of the channels-last arrays.  The 6x6 patch starts one point
// above/left of board point (4by, 4bx); points off the board read as zero.
// (At most four wavefronts per SIMD are asked for: aiming at eight, the compiler keeps the
// kernel within 64 registers by waiting for each of the 36 loads before it issues the next.)
template <typename P>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 4))) void in_transform_k(const P* __restrict__ act,
                                                      P* __restrict__ V, int T, int Cp,
                                                      int Tp) {
    constexpr int VN = ChanVec<P>::N;
    const int lpt = Cp / VN;  // lanes per tile
    const int gid = blockIdx.x * 256 + threadIdx.x;
    const int t = gid / lpt;
    if (t >= T) return;
    const int c = (gid - t * lpt) * VN;
    const int b = t / kTilesPerBoard;
    const int j = t - b * kTilesPerBoard;
    const int by = j / 5, bx = j - by * 5;
    const int y0 = 4 * by - 1, x0 = 4 * bx - 1;
    const P* base = act + (size_t)b * kPts * Cp + c;

    float d[VN][36];
#pragma unroll
    for (int yy = 0; yy < 6; yy++) {
#pragma unroll
        for (int xx = 0; xx < 6; xx++) {
            const int y = y0 + yy, x = x0 + xx;
            // clamped address + select instead of a branch: all 36 loads stay in flight
            const bool inb = (unsigned)y < (unsigned)kBoard && (unsigned)x < (unsigned)kBoard;
            const int pt = inb ? y * kBoard + x : 0;
            float tmp[VN];
            ChanVec<P>::load(base + (size_t)pt * Cp, tmp);
#pragma unroll
            for (int v = 0; v < VN; v++) d[v][yy * 6 + xx] = inb ? tmp[v] : 0.0f;
        }
    }
#pragma unroll
    for (int v = 0; v < VN; v++) {
        float t1[36];
#pragma unroll
        for (int xx = 0; xx < 6; xx++)  // columns: along y
            bt6(d[v][0 + xx], d[v][6 + xx], d[v][12 + xx], d[v][18 + xx], d[v][24 + xx],
                d[v][30 + xx], t1[0 + xx], t1[6 + xx], t1[12 + xx], t1[18 + xx], t1[24 + xx],
                t1[30 + xx]);
#pragma unroll
        for (int yy = 0; yy < 6; yy++)  // rows: along x
            bt6(t1[yy * 6 + 0], t1[yy * 6 + 1], t1[yy * 6 + 2], t1[yy * 6 + 3], t1[yy * 6 + 4],
                t1[yy * 6 + 5], d[v][yy * 6 + 0], d[v][yy * 6 + 1], d[v][yy * 6 + 2],
                d[v][yy * 6 + 3], d[v][yy * 6 + 4], d[v][yy * 6 + 5]);
    }
    P* vout = V + (size_t)t * Cp + c;
    const size_t pstride = (size_t)Tp * Cp;
#pragma unroll
    for (int p = 0; p < 36; p++) {
        float tmp[VN];
#pragma unroll
        for (int v = 0; v < VN; v++) tmp[v] = d[v][p];
        ChanVec<P>::store(vout + p * pstride, tmp);
    }
}

template <typename P>
void launch_in_transform(const P* act, P* V, int n, int Cp, int Tp, hipStream_t s,
                         LaunchTimer* t) {
    const int T = n * kTilesPerBoard;
    const int lanes = T * (Cp / ChanVec<P>::N);
    launch(in_transform_k<P>, dim3((lanes + 255) / 256), dim3(256), s, t, act, V, T, Cp, Tp);
}

// ---------------------------------------------------------------------------
// Output transform Y = A^T m A fused with batch-norm scale/shift, residual add
// and ReLU (reference src/CPUPipe.cpp:212-284 + :352-377; the reference GPU
// path fuses the same way, src/kernels/convolve3.opencl:218-318).
// out = max(0, scale*(y - mean) + rfac*res); rfac carries the ratio of the
// activation scales of the skip connection and of this layer (1 in fp32).
template <typename P>
__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const P* base, size_t bytes);

template <typename P>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 3))) void out_transform_k(
    const P* __restrict__ M, const P* __restrict__ res, P* __restrict__ out,
    const float* __restrict__ bn_scale, const float* __restrict__ bn_mean, float rfac, int T,
    int Kp, int Tp, int slab) {
    constexpr int VN = ChanVec<P>::N;
    const int lpt = Kp / VN;
    const int gid = blockIdx.x * 256 + threadIdx.x;
    const int t = gid / lpt;
    if (t >= T) return;
    const int c = (gid - t * lpt) * VN;
    const int b = t / kTilesPerBoard;
    const int j = t - b * kTilesPerBoard;
    const int by = j / 5, bx = j - by * 5;

    float m[VN][36];
    // slab > 0: M lies slab by slab, [36][Kp / slab][Tp][slab]
    const P* msrc = slab > 0 ? M + ((size_t)(c / slab) * Tp + t) * slab + c % slab
                             : M + (size_t)t * Kp + c;
    const size_t pstride = (size_t)Tp * Kp;
#pragma unroll
    for (int p = 0; p < 36; p++) {
        float tmp[VN];
        ChanVec<P>::load(msrc + p * pstride, tmp);
#pragma unroll
        for (int v = 0; v < VN; v++) m[v][p] = tmp[v];
    }
    float o[VN][16];
#pragma unroll
    for (int v = 0; v < VN; v++) {
        float t1[24];  // [4][6]
#pragma unroll
        for (int xx = 0; xx < 6; xx++)
            at6(m[v][0 + xx], m[v][6 + xx], m[v][12 + xx], m[v][18 + xx], m[v][24 + xx],
                m[v][30 + xx], t1[0 + xx], t1[6 + xx], t1[12 + xx], t1[18 + xx]);
#pragma unroll
        for (int i = 0; i < 4; i++)
            at6(t1[i * 6 + 0], t1[i * 6 + 1], t1[i * 6 + 2], t1[i * 6 + 3], t1[i * 6 + 4],
                t1[i * 6 + 5], o[v][i * 4 + 0], o[v][i * 4 + 1], o[v][i * 4 + 2],
                o[v][i * 4 + 3]);
    }
    float sc[VN], mn[VN];
#pragma unroll
    for (int v = 0; v < VN; v++) {
        sc[v] = bn_scale[c + v];
        mn[v] = bn_mean[c + v];
    }
    const size_t bbase = (size_t)b * kPts * Kp + c;
    const __amdgpu_buffer_rsrc_t rO =
        make_rsrc(out, (size_t)((T + kTilesPerBoard - 1) / kTilesPerBoard) * kPts * Kp * sizeof(P));
    float r[VN][16];
    if (res != nullptr) {  // uniform; clamped addresses keep the 16 loads free of branches
#pragma unroll
        for (int i = 0; i < 4; i++) {
#pragma unroll
            for (int jj = 0; jj < 4; jj++) {
                const int y = min(4 * by + i, kBoard - 1), x = min(4 * bx + jj, kBoard - 1);
                float tmp[VN];
                ChanVec<P>::load(res + bbase + (size_t)(y * kBoard + x) * Kp, tmp);
#pragma unroll
                for (int v = 0; v < VN; v++) r[v][i * 4 + jj] = tmp[v];
            }
        }
    } else {
#pragma unroll
        for (int v = 0; v < VN; v++)
#pragma unroll
            for (int q = 0; q < 16; q++) r[v][q] = 0.0f;
    }
#pragma unroll
    for (int i = 0; i < 4; i++) {
#pragma unroll
        for (int jj = 0; jj < 4; jj++) {
            const int y = 4 * by + i, x = 4 * bx + jj;
            float val[VN];
#pragma unroll
            for (int v = 0; v < VN; v++)
                val[v] = act_clamp<P>(
                    fmaxf(0.0f, sc[v] * (o[v][i * 4 + jj] - mn[v]) + rfac * r[v][i * 4 + jj]));
            // Unconditional store through a buffer descriptor: points off the board get an
            // offset outside it and are dropped by the hardware (a branch around each store
            // makes the compiler wait for the store before it).
            const unsigned off = (y < kBoard && x < kBoard)
                                     ? (unsigned)((bbase + (size_t)(y * kBoard + x) * Kp) * sizeof(P))
                                     : 0xfffffff0u;
            if constexpr (sizeof(P) == 4) {
                __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, val[0]), rO, off,
                                                      0, 0);
            } else {
                half2v h;
                h.x = (half_t)fminf(fmaxf(val[0], -65504.0f), 65504.0f);
                h.y = (half_t)fminf(fmaxf(val[1], -65504.0f), 65504.0f);
                __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, h), rO, off, 0,
                                                      0);
            }
        }
    }
}

template <typename P>
void launch_out_transform(const P* M, const P* res, P* out, const float* bn_scale,
                          const float* bn_mean, float rfac, int n, int Kp, int Tp,
                          hipStream_t s, LaunchTimer* t, int slab) {
    const int T = n * kTilesPerBoard;
    const int lanes = T * (Kp / ChanVec<P>::N);
    if (slab != 0 && (slab % ChanVec<P>::N != 0 || Kp % slab != 0))
        throw std::invalid_argument("out_transform: slab width does not fit");
    launch(out_transform_k<P>, dim3((lanes + 255) / 256), dim3(256), s, t, M, res, out,
           bn_scale, bn_mean, rfac, T, Kp, Tp, slab);
}

// ---------------------------------------------------------------------------
// Output transform of layer l fused with the input transform of layer l+1
// (the reference fuses the same pair for batch 1 only,
// src/kernels/convolve3.opencl:320-452).  Phase 1 turns the 25 M tiles of a
// board into the 19x19 activation plane (BN, residual, ReLU, rounded to the
// storage type exactly as the unfused kernel stores it) and keeps it in LDS;
// phase 2 reads the 6x6 patches back from LDS and writes the next layer's V.
// The activation itself goes to memory only when a later layer needs it as a
// skip connection.
//
// Raw buffer access: address = buffer base + scalar byte offset + per-lane byte
// offset.  Everything that selects a board, a tile pair or a Winograd position
// is wavefront-uniform and lives in the scalar offset, stepped with scalar
// adds; the per-lane offset never changes, so the global accesses need no
// vector address arithmetic, and accesses past the end of a buffer are benign.
template <typename P> struct BufIO;
template <> struct BufIO<float> {
    static __device__ __forceinline__ float load(__amdgpu_buffer_rsrc_t r, unsigned voff,
                                                 unsigned soff) {
        return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(r, voff, soff, 0));
    }
    static __device__ __forceinline__ void store(float v, __amdgpu_buffer_rsrc_t r, unsigned voff,
                                                 unsigned soff) {
        __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, v), r, voff, soff, 0);
    }
};
template <> struct BufIO<half_t> {
    static __device__ __forceinline__ half_t load(__amdgpu_buffer_rsrc_t r, unsigned voff,
                                                  unsigned soff) {
        return __builtin_bit_cast(half_t, __builtin_amdgcn_raw_buffer_load_b16(r, voff, soff, 0));
    }
    static __device__ __forceinline__ void store(half_t v, __amdgpu_buffer_rsrc_t r, unsigned voff,
                                                 unsigned soff) {
        __builtin_amdgcn_raw_buffer_store_b16(__builtin_bit_cast(unsigned short, v), r, voff, soff,
                                              0);
    }
};
// Two consecutive channels per access (4 bytes in fp16, 8 in fp32).
template <typename P> struct BufIO2;
template <> struct BufIO2<float> {
    typedef float pair_t __attribute__((ext_vector_type(2)));
    static __device__ __forceinline__ void load(__amdgpu_buffer_rsrc_t r, unsigned voff,
                                                unsigned soff, float& a, float& b) {
        // two 4-byte loads: this compiler lowers the 8-byte raw buffer load builtin
        // to a single dword load
        a = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(r, voff, soff, 0));
        b = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(r, voff + 4, soff, 0));
    }
    template <int AUX = 0>
    static __device__ __forceinline__ void store(pair_t v, __amdgpu_buffer_rsrc_t r, unsigned voff,
                                                 unsigned soff) {
        typedef unsigned u2 __attribute__((ext_vector_type(2)));
        __builtin_amdgcn_raw_buffer_store_b64(__builtin_bit_cast(u2, v), r, voff, soff, AUX);
    }
    // the pair as stored, no conversion (so that nothing has to wait for the data yet)
    static __device__ __forceinline__ pair_t load_raw(__amdgpu_buffer_rsrc_t r, unsigned voff,
                                                      unsigned soff) {
        float a, b;
        load(r, voff, soff, a, b);
        pair_t v;
        v.x = a;
        v.y = b;
        return v;
    }
};
template <> struct BufIO2<half_t> {
    typedef half2v pair_t;
    static __device__ __forceinline__ void load(__amdgpu_buffer_rsrc_t r, unsigned voff,
                                                unsigned soff, float& a, float& b) {
        const half2v h =
            __builtin_bit_cast(half2v, __builtin_amdgcn_raw_buffer_load_b32(r, voff, soff, 0));
        a = (float)h.x;
        b = (float)h.y;
    }
    template <int AUX = 0>
    static __device__ __forceinline__ void store(pair_t v, __amdgpu_buffer_rsrc_t r, unsigned voff,
                                                 unsigned soff) {
        __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, v), r, voff, soff, AUX);
    }
    static __device__ __forceinline__ pair_t load_raw(__amdgpu_buffer_rsrc_t r, unsigned voff,
                                                      unsigned soff) {
        return __builtin_bit_cast(pair_t, __builtin_amdgcn_raw_buffer_load_b32(r, voff, soff, 0));
    }
};

template <typename P>
__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const P* base, size_t bytes) {
    // untyped 32-bit-element descriptor for gfx9-family raw buffer instructions
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<P*>(base), 0, (int)bytes, 0x00020000);
}

// One workgroup owns one board and 64 channels.  A lane owns two consecutive
// channels (one 4- or 8-byte access instead of two), a half-wave owns a tile,
// so a wavefront handles two neighbouring tiles at once and the 13 wavefronts
// cover the 25 tiles in a single pass: every wavefront issues its 36 M loads
// once, up front, instead of walking through several tiles with a full memory
// latency each, and the number of memory instructions (which bounded the
// one-channel-per-lane version) is halved.  The two tiles of a wavefront are
// adjacent rows of M and V, so the half-wave only adds a constant to the lane
// offset.  The LDS plane carries a zero halo: the 6x6 patch reads need no
// bounds handling.  Loads that fall outside the board (clipped tiles) read
// neighbouring memory or, past the end of the buffer, zero (raw buffer
// semantics); their results are never stored.
//
// CG = channels per workgroup.  64 (a half-wave per tile, 13 wavefronts) moves
// whole 128-byte runs and is the choice when there are enough boards to give
// every compute unit a workgroup; with few boards the kernel is bound by the
// arithmetic of the one compute unit a workgroup runs on, and 32 or 16 channels
// per workgroup (4 or 8 tiles per wavefront, 7 or 4 wavefronts) spread a board
// over more compute units.
// Cache policy of the fused transform's stores.  With 64 channels per work-group every
// store instruction writes whole 128-byte lines (64 channels of one tile row or board
// point), and nothing in the kernel reads them again: written through (sc0 sc1) they leave
// for memory while the kernel runs instead of staying behind as dirty lines that the end
// of the kernel has to flush (measured at 64 boards, 256 filters: 15.2 -> 14.0 us per
// launch).  The narrower work-groups write half and quarter lines, which written through
// cost twice the time (32 channels at 64 boards: 16.4 us against 12.9): they stay write-back.
template <int CG> constexpr int xform_store_policy() { return CG == 64 ? kStoreThrough : 0; }
constexpr int kPlane = 22;       // LDS plane: 19 points + 1 zero halo before + 2 after
// Strides of the plane in channel pairs.  A store or load instruction of the transform
// touches the same cell of every tile in the wavefront, CG / 2 consecutive pairs each, and
// tiles lie 4 cells (and 4 rows) apart: with cells of exactly CG / 2 pairs the narrow shapes
// put all their tiles on the same banks (16 channels: 8 tiles on 8 of 32 banks, measured
// 237 k conflict cycles in 351 k active ones per launch).  Padded so that four cells and
// four rows both advance the bank by CG / 2, consecutive tiles take consecutive groups of
// banks (7.7 k conflict cycles left, the halo; the launch takes as long as before: LDS was
// not what it waited for).  The 64-channel shape (one tile per 32 lanes) needs no padding.
constexpr int plane_cell_pairs(int cg) { return cg == 16 ? 10 : cg == 32 ? 20 : cg / 2; }
constexpr int plane_row_pairs(int cg) {
    return cg == 16 ? kPlane * 10 + 6 : cg == 32 ? kPlane * 20 + 4 : kPlane * (cg / 2);
}
constexpr int plane_pairs(int cg) { return kPlane * plane_row_pairs(cg); }
constexpr int fuse_waves(int cg) { return (kTilesPerBoard + 128 / cg - 1) / (128 / cg); }

// The body of the kernel, for work-group `wg` of the launch's transform work-groups, with
// the LDS plane handed in (plane_pairs(CG) channel pairs); returns the work item
// (board * channel groups + channel group) it processed, or -1 if `wg` had none.
// VPOL = cache policy of the stores of V.  VSLAB / MSLAB: V is written / M is read channel
// group by channel group, [36][Kp / CG][Tp][CG], instead of [36][Tp][Kp] (tile_slab): the 25
// tiles of this work-group's board and channel group are then one contiguous run per
// Winograd position (whole lines, which is also what makes write-through stores cheap).
template <typename P, int CG, int VPOL, bool VSLAB = false, bool MSLAB = false>
__device__ __forceinline__ int out_in_transform_body(
    typename BufIO2<P>::pair_t* ybuf, unsigned wg, const P* M, const P* res, P* act_out, P* Vn,
    const float* __restrict__ bn_scale, const float* __restrict__ bn_mean, float rfac, int n,
    int Kp, int Tp) {
    typedef typename BufIO2<P>::pair_t pair_t;
    constexpr int CP = CG / 2;        // channel pairs per plane cell = lanes per tile
    constexpr int CS = plane_cell_pairs(CG), RS = plane_row_pairs(CG);   // plane strides
    constexpr int TPW = 64 / CP;      // tiles per wavefront
    constexpr int WAVES = fuse_waves(CG);
    // Work-group w runs on die w % 8, each die with its own L2.  The narrow shapes share
    // 128-byte lines between the work-groups of neighbouring channel groups, so the items
    // (board, channel group) are cut into 8 contiguous segments and work-group w takes item
    // w / 8 of segment w % 8: the sharers then sit on one die and a line comes from memory
    // once, instead of once for each die that holds a piece of it.
    const int ncg = Kp / CG;
    const int per_die = (n * ncg + 7) >> 3;
    const int item = (int)(wg & 7) * per_die + (int)(wg >> 3);
    if (item >= n * ncg) return -1;
    const int b = item / ncg;
    const int cg = item - b * ncg;

    const unsigned lane = threadIdx.x & 63;
    const unsigned cl = lane % CP, sub = lane / CP;    // channel pair, tile within the wavefront
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const unsigned esz = (unsigned)sizeof(P);
    const int j = TPW * wave + (int)sub;               // this lane's tile
    const bool valid = j < kTilesPerBoard;
    const int jc = valid ? j : kTilesPerBoard - 1;
    const int by = jc / 5, bx = jc - by * 5;
    const int ny = min(4, kBoard - 4 * by), nx = min(4, kBoard - 4 * bx);

    const unsigned pstride = (unsigned)Tp * (unsigned)Kp * esz;   // bytes between positions
    const size_t tile_bytes = (size_t)kPos * Tp * Kp * esz;
    const size_t act_bytes = (size_t)n * kPts * Kp * esz;
    const __amdgpu_buffer_rsrc_t rM = make_rsrc(M, tile_bytes);
    const __amdgpu_buffer_rsrc_t rV = make_rsrc(Vn, tile_bytes);
    const __amdgpu_buffer_rsrc_t rR = make_rsrc(res != nullptr ? res : M, act_bytes);
    const __amdgpu_buffer_rsrc_t rA = make_rsrc(act_out != nullptr ? act_out : Vn, act_bytes);
    // per-lane byte offsets: channel pair (+ the tile's row within the wavefront) / tile origin
    unsigned voff_t = cl * 2 * esz + (valid ? sub : 0u) * (unsigned)Kp * esz;
    unsigned voff_a = cl * 2 * esz + (unsigned)((4 * by) * kBoard + 4 * bx) * (unsigned)Kp * esz;
    // Pin both offsets into registers here: computed later, between the two groups of
    // loads, their arithmetic waits for the first group's data (a register-reuse hazard).
    asm volatile("" : "+v"(voff_t), "+v"(voff_a));
    // uniform byte offsets of the wavefront's first tile / of the board
    const unsigned soff_t =
        ((unsigned)(b * kTilesPerBoard + TPW * wave) * (unsigned)Kp + cg * CG) * esz;
    const unsigned soff_a = ((unsigned)(b * kPts) * (unsigned)Kp + cg * CG) * esz;
    float sc[2], nb[2];   // scale * (y - mean) = y * scale + nb
#pragma unroll
    for (int v = 0; v < 2; v++) {
        sc[v] = bn_scale[cg * CG + cl * 2 + v];
        nb[v] = -sc[v] * bn_mean[cg * CG + cl * 2 + v];
    }

    // All loads of the pass go out before any arithmetic.  M's go first, column by
    // column of the 6x6 position grid: loads return in issue order at the rate the
    // memory system delivers them, and the first transform pass works on columns, so it
    // can start on the first six while the rest are still arriving.  The skip
    // connection (needed last) follows, left as stored: converting it here would wait
    // for it.  The scheduling barrier keeps the compiler from sinking those loads behind
    // the first arithmetic on M.
    pair_t m[36];   // as stored; converted where used
    // the same two offsets in the slab layout, [36][Kp / CG][Tp][CG]
    unsigned voff_s = cl * 2 * esz + (valid ? sub : 0u) * (unsigned)CG * esz;
    asm volatile("" : "+v"(voff_s));
    const unsigned soff_s =
        ((unsigned)cg * (unsigned)Tp + (unsigned)(b * kTilesPerBoard + TPW * wave)) *
        (unsigned)CG * esz;
#pragma unroll
    for (int xx = 0; xx < 6; xx++) {
        unsigned so = (MSLAB ? soff_s : soff_t) + (unsigned)xx * pstride;
#pragma unroll
        for (int row = 0; row < 6; row++) {
            m[row * 6 + xx] = BufIO2<P>::load_raw(rM, MSLAB ? voff_s : voff_t, so);
            so += 6u * pstride;
        }
        __builtin_amdgcn_sched_barrier(0);   // keep the columns in this order
    }
    pair_t r[16];
    if (res != nullptr) {
#pragma unroll
        for (int i = 0; i < 4; i++)
#pragma unroll
            for (int jj = 0; jj < 4; jj++)
                r[i * 4 + jj] = BufIO2<P>::load_raw(
                    rR, voff_a, soff_a + (unsigned)(i * kBoard + jj) * (unsigned)Kp * esz);
    } else {
#pragma unroll
        for (int q = 0; q < 16; q++) {
            r[q].x = (P)0.0f;
            r[q].y = (P)0.0f;
        }
    }
    __builtin_amdgcn_sched_barrier(0);

    LZ_STAMP(1);
    // zero the halo cells of the plane (rows and columns 0, 20, 21): 3 full rows
    // and 3 cells in each of the 19 rows between them; one cell per tile slot
    {
        pair_t zero;
        zero.x = (P)0.0f;
        zero.y = (P)0.0f;
        for (int q = TPW * wave + (int)sub; q < 3 * kPlane + 3 * kBoard; q += TPW * WAVES) {
            int cell;
            if (q < 3 * kPlane) {
                const int row = q < kPlane ? 0 : (q < 2 * kPlane ? kBoard + 1 : kBoard + 2);
                cell = row * RS + (q % kPlane) * CS;
            } else {
                const int e = q - 3 * kPlane, y = 1 + e / 3, c3 = e % 3;
                cell = y * RS + (c3 == 0 ? 0 : kBoard + c3) * CS;
            }
            ybuf[cell + cl] = zero;
        }
    }

    // ---- phase 1: A^T m A, BN (+ residual), ReLU -> LDS plane (+ memory)
    // plane cell of the tile's patch origin (board row 4by-1, column 4bx-1)
    pair_t* const origin = ybuf + (4 * by) * RS + (4 * bx) * CS + cl;
    pair_t keep[16];   // this tile's activations, written to memory after the barrier
    {
        float o[2][16];
        float t1[2][24];
        // column pass in the order the columns arrive (the barrier pins that order)
#pragma unroll
        for (int xx = 0; xx < 6; xx++) {
#pragma unroll
            for (int v = 0; v < 2; v++) {
                float c[6];
#pragma unroll
                for (int row = 0; row < 6; row++)
                    c[row] = (float)(v == 0 ? m[row * 6 + xx].x : m[row * 6 + xx].y);
                at6(c[0], c[1], c[2], c[3], c[4], c[5], t1[v][0 + xx], t1[v][6 + xx],
                    t1[v][12 + xx], t1[v][18 + xx]);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
#pragma unroll
        for (int v = 0; v < 2; v++)
#pragma unroll
            for (int i = 0; i < 4; i++)
                at6(t1[v][i * 6 + 0], t1[v][i * 6 + 1], t1[v][i * 6 + 2], t1[v][i * 6 + 3],
                    t1[v][i * 6 + 4], t1[v][i * 6 + 5], o[v][i * 4 + 0], o[v][i * 4 + 1],
                    o[v][i * 4 + 2], o[v][i * 4 + 3]);
#pragma unroll
        for (int i = 0; i < 4; i++) {
#pragma unroll
            for (int jj = 0; jj < 4; jj++) {
                pair_t sv;
                sv.x = act_to_storage<P>(fmaxf(
                    0.0f, fmaf((float)r[i * 4 + jj].x, rfac, fmaf(o[0][i * 4 + jj], sc[0], nb[0]))));
                sv.y = act_to_storage<P>(fmaxf(
                    0.0f, fmaf((float)r[i * 4 + jj].y, rfac, fmaf(o[1][i * 4 + jj], sc[1], nb[1]))));
                keep[i * 4 + jj] = sv;
                if (valid && i < ny && jj < nx) origin[(i + 1) * RS + (jj + 1) * CS] = sv;
            }
        }
    }
    LZ_STAMP(2);
    __syncthreads();
    LZ_STAMP(3);
    // The activation leaves only now: stores issued before the barrier would have to be
    // acknowledged before any wavefront may pass it; here they drain under phase 2.
    if (act_out != nullptr) {
#pragma unroll
        for (int i = 0; i < 4; i++)
#pragma unroll
            for (int jj = 0; jj < 4; jj++)
                if (valid && i < ny && jj < nx)
                    BufIO2<P>::template store<xform_store_policy<CG>()>(keep[i * 4 + jj], rA, voff_a,
                                     soff_a + (unsigned)(i * kBoard + jj) * (unsigned)Kp * esz);
    }

    // ---- phase 2: B^T d B of the next layer from the plane in LDS
    {
        pair_t raw[36];
#pragma unroll
        for (int yy = 0; yy < 6; yy++)
#pragma unroll
            for (int xx = 0; xx < 6; xx++) raw[yy * 6 + xx] = origin[yy * RS + xx * CS];
        pair_t outp[36];
#pragma unroll
        for (int v = 0; v < 2; v++) {
            float d[36], t1[36];
#pragma unroll
            for (int q = 0; q < 36; q++) d[q] = (float)(v == 0 ? raw[q].x : raw[q].y);
#pragma unroll
            for (int xx = 0; xx < 6; xx++)
                bt6(d[0 + xx], d[6 + xx], d[12 + xx], d[18 + xx], d[24 + xx], d[30 + xx],
                    t1[0 + xx], t1[6 + xx], t1[12 + xx], t1[18 + xx], t1[24 + xx], t1[30 + xx]);
#pragma unroll
            for (int yy = 0; yy < 6; yy++)
                bt6(t1[yy * 6 + 0], t1[yy * 6 + 1], t1[yy * 6 + 2], t1[yy * 6 + 3],
                    t1[yy * 6 + 4], t1[yy * 6 + 5], d[yy * 6 + 0], d[yy * 6 + 1], d[yy * 6 + 2],
                    d[yy * 6 + 3], d[yy * 6 + 4], d[yy * 6 + 5]);
#pragma unroll
            for (int q = 0; q < 36; q++) {
                if (v == 0) outp[q].x = (P)d[q];
                else outp[q].y = (P)d[q];
            }
        }
        LZ_STAMP(4);
        if (valid) {
            unsigned so = VSLAB ? soff_s : soff_t, vo = VSLAB ? voff_s : voff_t;
#pragma unroll
            for (int p = 0; p < 36; p++) {
                BufIO2<P>::template store<VPOL>(outp[p], rV, vo, so);
                so += pstride;
            }
        }
    }
    LZ_STAMP(5);
    return item;
}

// M and Vn may be one array (every value of M is in a register before the same lane writes
// the value of V that takes its place), so neither is declared free of aliases.
// SLAB: M and V lie slab by slab, [36][Kp / CG][Tp][CG] (see tile_slab); V's stores are then
// whole lines and go out write-through.
template <typename P, int CG, bool SLAB = false>
__global__ __launch_bounds__(fuse_waves(CG) * 64) void out_in_transform_k(
    const P* M, const P* __restrict__ res, P* __restrict__ act_out, P* Vn,
    const float* __restrict__ bn_scale, const float* __restrict__ bn_mean, float rfac, int n,
    int Kp, int Tp) {
    __shared__ typename BufIO2<P>::pair_t ybuf[plane_pairs(CG)];
    (void)out_in_transform_body<P, CG, SLAB ? kStoreThrough : xform_store_policy<CG>(), SLAB,
                                SLAB>(ybuf, blockIdx.x, M, res, act_out, Vn, bn_scale, bn_mean,
                                      rfac, n, Kp, Tp);
}

template <typename P>
void launch_out_in_transform(const P* M, const P* res, P* act_out, P* Vn, const float* bn_scale,
                             const float* bn_mean, float rfac, int n, int Kp, int Tp,
                             hipStream_t s, LaunchTimer* t, int slab) {
    // With few boards a narrow shape spreads a board's arithmetic over more compute units;
    // the 64-channel shape moves whole lines.  Measured at 256 filters with the layers working
    // in place (transform + GEMM per layer, us, with 16 / 32 / 64 channels per work-group):
    // 8 boards 11.7 / 12.8 / 14.0, 16 boards 14.6 / 15.3 / 15.4, 20 boards 17.3 / 16.5 / 16.6,
    // 24 boards 18.4 / 17.5 / 16.8, 32 boards 21.9 / 20.5 / 19.9, 40 boards 24.7 / 24.8 / 20.8.
    // The narrow shapes only pay with the die-aware item order of the kernel: dealt round-robin
    // over the dies, their work-groups fetch every line of M once per die that holds a piece
    // of it (16 channels at batch 16: 11.2 us per launch against 7.7).
    const int items64 = n * (Kp / 64);
    auto grid = [](int items) { return dim3((unsigned)(8 * ((items + 7) / 8))); };
    if (slab == 16)
        launch(out_in_transform_k<P, 16, true>, grid(items64 * 4), dim3(fuse_waves(16) * 64), s,
               t, M, res, act_out, Vn, bn_scale, bn_mean, rfac, n, Kp, Tp);
    else if (slab == 32)
        launch(out_in_transform_k<P, 32, true>, grid(items64 * 2), dim3(fuse_waves(32) * 64), s,
               t, M, res, act_out, Vn, bn_scale, bn_mean, rfac, n, Kp, Tp);
    else if (slab != 0)
        throw std::invalid_argument("out_in_transform: slabs are 16 or 32 channels wide");
    else if (items64 > 80)
        launch(out_in_transform_k<P, 64>, grid(items64), dim3(fuse_waves(64) * 64), s, t, M, res,
               act_out, Vn, bn_scale, bn_mean, rfac, n, Kp, Tp);
    else if (items64 > 64)
        launch(out_in_transform_k<P, 32>, grid(items64 * 2), dim3(fuse_waves(32) * 64), s, t, M,
               res, act_out, Vn, bn_scale, bn_mean, rfac, n, Kp, Tp);
    else
        launch(out_in_transform_k<P, 16>, grid(items64 * 4), dim3(fuse_waves(16) * 64), s, t, M,
               res, act_out, Vn, bn_scale, bn_mean, rfac, n, Kp, Tp);
}

// ---------------------------------------------------------------------------
// The 36 independent GEMMs M_p[t][k] = sum_c V_p[t][c] * U_p[k][c]
// (reference src/CPUPipe.cpp:185-210; GPU twin XgemmBatched).
//
// One workgroup = 4 wavefronts (2x2) computes a BM x BN tile of one position.
// Both operands are staged through LDS in 128-byte-per-row slices (64 halves
// or 32 floats of the contraction index), double buffered, rows padded by 16
// bytes so that the 16-byte-per-lane fragment reads are conflict free.
// Each lane feeds the matrix cores with 16 contiguous bytes of its row:
//   fp16: one v_mfma_f32_32x32x16_f16 per fragment pair (8 halves per lane)
//   fp32: four v_mfma_f32_32x32x2_f32 per fragment pair (one float each)
// Lane l supplies row (l & 31) of its 32-row block of either operand, and the
// upper half-wave supplies the other half of the k-slice; the assignment of k
// values to MFMA k-slots is the same for both operands, which is all the
// contraction needs.  Accumulation is fp32 for both storage types.
// Workgroups of different Winograd positions start their walk over the k-slices at
// different slices (the sum over k may run in any order): at any moment the
// 128-byte pieces being fetched then spread over whole 512-byte rows instead of
// all workgroups hitting the same quarter of every row, which would leave most
// memory channels idle.  The rotation depends on the position only, so a given
// board sees the same summation order whatever else is in the batch.
__device__ __forceinline__ int rotated_slice(int k, int rot, int nk) {
    const int kk = k + rot;
    return kk >= nk ? kk - nk : kk;
}

template <typename P> struct Mma;
template <> struct Mma<half_t> {
    static __device__ __forceinline__ float16v run(int4v a, int4v b, float16v c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8v, a),
                                                      __builtin_bit_cast(half8v, b), c, 0, 0, 0);
    }
};
template <> struct Mma<float> {
    static __device__ __forceinline__ float16v run(int4v a, int4v b, float16v c) {
        const float4v fa = __builtin_bit_cast(float4v, a);
        const float4v fb = __builtin_bit_cast(float4v, b);
        c = __builtin_amdgcn_mfma_f32_32x32x2f32(fa.x, fb.x, c, 0, 0, 0);
        c = __builtin_amdgcn_mfma_f32_32x32x2f32(fa.y, fb.y, c, 0, 0, 0);
        c = __builtin_amdgcn_mfma_f32_32x32x2f32(fa.z, fb.z, c, 0, 0, 0);
        c = __builtin_amdgcn_mfma_f32_32x32x2f32(fa.w, fb.w, c, 0, 0, 0);
        return c;
    }
};

// Work items are (position, row tile, column tile) triples, column tile fastest.
// The device hands workgroup b to accelerator die (XCD) b % 8, each die with its
// own L2, so the item list is cut into 8 contiguous segments and workgroup b
// takes item (b / 8) of segment (b % 8): all tiles of one position, and the
// column tiles that share a V row tile, then run on the same die, U_p and the
// V tile are fetched from memory once and the repeats hit that die's L2.
template <typename P, int BM, int BN, int NK>
__global__ __launch_bounds__(256) void wino_gemm_k(const P* __restrict__ V,
                                                   const P* __restrict__ U, P* __restrict__ M,
                                                   int Tp, int Cp, int Kp, int tiles_m,
                                                   int tiles_n, int seg) {
    constexpr int EPC = 16 / sizeof(P);   // elements per 16-byte chunk
    constexpr int BK = 128 / sizeof(P);   // contraction extent of one LDS stage
    // LDS rows: padded to 144 bytes, or (the 64-column tile) bare 128-byte rows whose
    // 16-byte chunks are permuted by the row number, which is just as conflict free for
    // the fragment reads (16 lanes = 16 rows: 8 chunk slots x 2 row parities = all 64
    // banks) and brings a stage pair under a third of the LDS, so that three
    // work-groups share a compute unit instead of two.
    constexpr bool SWZ = BN == 64 && sizeof(P) == 2;   // fp32 is bound by the matrix pipe: no gain
    constexpr int ROW = SWZ ? BK : BK + EPC;
    constexpr int WM = BM / 2, WN = BN / 2;
    constexpr int MB = WM / 32, NB = WN / 32;
    constexpr int A_CH = BM * 8 / 256, B_CH = BN * 8 / 256;  // chunks per thread and stage
    auto slot = [](int row, int chunk) { return SWZ ? (chunk ^ ((row >> 1) & 7)) : chunk; };
    constexpr int CROW = BN + EPC;        // padded row of the staged output tile
    constexpr int STAGE = (BM + BN) * ROW;
    constexpr int SMEM = (2 * STAGE > BM * CROW) ? 2 * STAGE : BM * CROW;
    static_assert(MB >= 1 && NB >= 1, "tile too small for a 2x2 wave grid");

    __shared__ __attribute__((aligned(16))) P smem[SMEM];

    const int n_items = kPos * tiles_m * tiles_n;
    const int xcd = blockIdx.x & 7;
    const int item = xcd * seg + (blockIdx.x >> 3);
    if ((int)(blockIdx.x >> 3) >= seg || item >= n_items) return;
    const int tn = item % tiles_n;
    const int rest = item / tiles_n;
    const int tm = rest % tiles_m;
    const int p = rest / tiles_m;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wy = wave >> 1, wx = wave & 1;
    const P* Ag = V + ((size_t)p * Tp + (size_t)tm * BM) * Cp;
    const P* Bg = U + ((size_t)p * Kp + (size_t)tn * BN) * Cp;

    float16v acc[MB][NB];
#pragma unroll
    for (int i = 0; i < MB; i++)
#pragma unroll
        for (int j = 0; j < NB; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0.0f;

    // Two register stages: the slice for step kt+2 is requested while step kt is
    // being multiplied, so two slices per workgroup are in flight.
    int4v ra[2][A_CH], rb[2][B_CH];
    (void)Cp;
    const int lrow = tid >> 3, lch = tid & 7;  // row / chunk of this thread's first chunk

    auto gload = [&](int st, int k0) {
#pragma unroll
        for (int i = 0; i < A_CH; i++)
            ra[st][i] = *reinterpret_cast<const int4v*>(Ag + (size_t)(lrow + i * 32) * Cp + k0 +
                                                        lch * EPC);
#pragma unroll
        for (int i = 0; i < B_CH; i++)
            rb[st][i] = *reinterpret_cast<const int4v*>(Bg + (size_t)(lrow + i * 32) * Cp + k0 +
                                                        lch * EPC);
    };
    auto lstore = [&](int st, int buf) {
        P* As = smem + buf * STAGE;
        P* Bs = As + BM * ROW;
#pragma unroll
        for (int i = 0; i < A_CH; i++)
            *reinterpret_cast<int4v*>(&As[(lrow + i * 32) * ROW + slot(lrow, lch) * EPC]) = ra[st][i];
#pragma unroll
        for (int i = 0; i < B_CH; i++)
            *reinterpret_cast<int4v*>(&Bs[(lrow + i * 32) * ROW + slot(lrow, lch) * EPC]) = rb[st][i];
    };

    // NK = Cp / BK is a template argument: the pipeline below is straight-line
    // code, so the compiler knows exactly which loads are outstanding at each
    // wait and the slice for step k+2 really stays in flight across step k.
    const int rot = p % NK;
    gload(0, rotated_slice(0, rot, NK) * BK);
    if (NK > 1) gload(1, rotated_slice(1, rot, NK) * BK);
    lstore(0, 0);
    __syncthreads();

    const int frow = lane & 31, fk = lane >> 5;   // tile offsets are multiples of 32 rows
#pragma unroll
    for (int k = 0; k < NK; k++) {
        const int h = k & 1;
        if (k + 2 < NK) {
            gload(h, rotated_slice(k + 2, rot, NK) * BK);
            __builtin_amdgcn_sched_barrier(0);  // request the slice before the math starts
        }
        const P* As = smem + h * STAGE;
        const P* Bs = As + BM * ROW;
#pragma unroll
        for (int kc = 0; kc < 4; kc++) {
            int4v fa[MB], fb[NB];
#pragma unroll
            for (int i = 0; i < MB; i++)
                fa[i] = *reinterpret_cast<const int4v*>(
                    &As[(wy * WM + i * 32 + frow) * ROW + slot(frow, kc * 2 + fk) * EPC]);
#pragma unroll
            for (int j = 0; j < NB; j++)
                fb[j] = *reinterpret_cast<const int4v*>(
                    &Bs[(wx * WN + j * 32 + frow) * ROW + slot(frow, kc * 2 + fk) * EPC]);
#pragma unroll
            for (int i = 0; i < MB; i++)
#pragma unroll
                for (int j = 0; j < NB; j++) acc[i][j] = Mma<P>::run(fb[j], fa[i], acc[i][j]);
        }
        if (k + 1 < NK) lstore(h ^ 1, h ^ 1);
        __syncthreads();
    }

    // The U block is the MFMA's row operand and the V block its column operand,
    // so register r of lane l holds output channel 8*(r/4) + 4*(l/32) + r%4 of
    // tile row l%32: four consecutive channels per lane, which go to the LDS
    // staging tile (all slices have been consumed) as one 8- or 16-byte write.
    // From there whole rows leave in 16-byte pieces.
    const int ccol = 4 * (lane >> 5), crow = lane & 31;
#pragma unroll
    for (int i = 0; i < MB; i++)
#pragma unroll
        for (int j = 0; j < NB; j++)
#pragma unroll
            for (int q = 0; q < 4; q++) {
                typename Quad<P>::type v;
#pragma unroll
                for (int e = 0; e < 4; e++) v[e] = to_storage<P>(acc[i][j][q * 4 + e]);
                *reinterpret_cast<typename Quad<P>::type*>(
                    &smem[(wy * WM + i * 32 + crow) * CROW + wx * WN + j * 32 + 8 * q + ccol]) = v;
            }
    __syncthreads();
    constexpr int CPR = BN / EPC;  // 16-byte chunks per output row
    P* Mg = M + ((size_t)p * Tp + (size_t)tm * BM) * Kp + (size_t)tn * BN;
#pragma unroll 4
    for (int q = tid; q < BM * CPR; q += 256) {
        const int row = q / CPR, ch = q - row * CPR;
        *reinterpret_cast<int4v*>(Mg + (size_t)row * Kp + ch * EPC) =
            *reinterpret_cast<const int4v*>(&smem[row * CROW + ch * EPC]);
    }
}

// Persistent variant for an even number of k-slices.  A workgroup walks
// through several work items of its die's segment; the global loads of the
// next item's first two slices are issued while the current item's last two
// slices are being multiplied, so every workgroup keeps two slices (64 KB at
// the 128x128 tile) in flight from its first to its last item instead of
// starting each tile with an empty pipeline.  The finished tile leaves through
// the LDS stage that the last slice has just vacated.
template <typename P, int BM, int BN, int NK>
__global__ __launch_bounds__(256, 2) void wino_gemm_persistent_k(
    const P* __restrict__ V, const P* __restrict__ U, P* __restrict__ M, int Tp, int Cp, int Kp,
    int tiles_m, int tiles_n, int seg, int wg_per_xcd) {
    static_assert(NK >= 2 && (NK % 2) == 0, "needs an even slice count");
    constexpr int EPC = 16 / sizeof(P);
    constexpr int BK = 128 / sizeof(P);
    constexpr int ROW = BK + EPC;
    constexpr int WM = BM / 2, WN = BN / 2;
    constexpr int MB = WM / 32, NB = WN / 32;
    constexpr int A_CH = BM * 8 / 256, B_CH = BN * 8 / 256;
    constexpr int CROW = BN + EPC;
    constexpr int STAGE = (BM + BN) * ROW;
    // output staging fits one vacated stage either whole or in two row halves
    constexpr int EP_PARTS = (BM * CROW > STAGE) ? 2 : 1;
    static_assert((BM / EP_PARTS) * CROW <= STAGE, "output staging does not fit a stage");
    static_assert(EP_PARTS == 1 || WM * 2 == BM, "row halves must coincide with the wave rows");

    __shared__ __attribute__((aligned(16))) P smem[2 * STAGE];

    const int n_items = kPos * tiles_m * tiles_n;
    const int xcd = blockIdx.x & 7, w = blockIdx.x >> 3;
    int item = xcd * seg + w;
    const int last = min(n_items, (xcd + 1) * seg);
    if (w >= wg_per_xcd || item >= last) return;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wy = wave >> 1, wx = wave & 1;
    const int lrow = tid >> 3, lch = tid & 7;
    const int frow = lane & 31, fk = (lane >> 5) * EPC;
    const int ccol = 4 * (lane >> 5), crow = lane & 31;
    (void)Cp;

    // rs = row stride of the operand loads; the look-ahead past a workgroup's last
    // item uses rs = 0 and one shared address, so that the loads stay
    // unconditional (the compiler can then count outstanding loads exactly)
    // without fetching anything real.
    struct Ptrs { const P* a; const P* b; P* m; size_t rs; int rot; };
    auto locate = [&](int it) {
        const int tn = it % tiles_n;
        const int rest = it / tiles_n;
        const int tm = rest % tiles_m;
        const int p = rest / tiles_m;
        Ptrs r;
        r.a = V + ((size_t)p * Tp + (size_t)tm * BM) * Cp + (size_t)lrow * Cp + lch * EPC;
        r.b = U + ((size_t)p * Kp + (size_t)tn * BN) * Cp + (size_t)lrow * Cp + lch * EPC;
        r.m = M + ((size_t)p * Tp + (size_t)tm * BM) * Kp + (size_t)tn * BN;
        r.rs = (size_t)Cp;
        r.rot = p % NK;
        return r;
    };

    int4v ra[2][A_CH], rb[2][B_CH];
    auto gload = [&](int st, const Ptrs& q, int k0) {
#pragma unroll
        for (int i = 0; i < A_CH; i++)
            ra[st][i] = *reinterpret_cast<const int4v*>(q.a + (size_t)(i * 32) * q.rs + k0);
#pragma unroll
        for (int i = 0; i < B_CH; i++)
            rb[st][i] = *reinterpret_cast<const int4v*>(q.b + (size_t)(i * 32) * q.rs + k0);
    };
    auto lstore = [&](int st, int buf) {
        P* As = smem + buf * STAGE;
        P* Bs = As + BM * ROW;
#pragma unroll
        for (int i = 0; i < A_CH; i++)
            *reinterpret_cast<int4v*>(&As[(lrow + i * 32) * ROW + lch * EPC]) = ra[st][i];
#pragma unroll
        for (int i = 0; i < B_CH; i++)
            *reinterpret_cast<int4v*>(&Bs[(lrow + i * 32) * ROW + lch * EPC]) = rb[st][i];
    };

    Ptrs cur = locate(item);
    gload(0, cur, rotated_slice(0, cur.rot, NK) * BK);
    gload(1, cur, rotated_slice(1, cur.rot, NK) * BK);
    lstore(0, 0);
    __syncthreads();

    for (;;) {
        const int nitem = item + wg_per_xcd;
        const bool has_next = nitem < last;  // uniform
        Ptrs nxt = locate(has_next ? nitem : item);
        if (!has_next) {
            nxt.a = V;
            nxt.b = U;
            nxt.rs = 0;
        }

        float16v acc[MB][NB];
#pragma unroll
        for (int i = 0; i < MB; i++)
#pragma unroll
            for (int j = 0; j < NB; j++)
#pragma unroll
                for (int r = 0; r < 16; r++) acc[i][j][r] = 0.0f;

#pragma unroll
        for (int k = 0; k < NK; k++) {
            const int h = k & 1;
            if (k + 2 < NK) {
                gload(h, cur, rotated_slice(k + 2, cur.rot, NK) * BK);
            } else {
                gload(h, nxt, rotated_slice(k + 2 - NK, nxt.rot, NK) * BK);
            }
            __builtin_amdgcn_sched_barrier(0);
            const P* As = smem + h * STAGE;
            const P* Bs = As + BM * ROW;
#pragma unroll
            for (int kc = 0; kc < 4; kc++) {
                int4v fa[MB], fb[NB];
#pragma unroll
                for (int i = 0; i < MB; i++)
                    fa[i] = *reinterpret_cast<const int4v*>(
                        &As[(wy * WM + i * 32 + frow) * ROW + kc * 2 * EPC + fk]);
#pragma unroll
                for (int j = 0; j < NB; j++)
                    fb[j] = *reinterpret_cast<const int4v*>(
                        &Bs[(wx * WN + j * 32 + frow) * ROW + kc * 2 * EPC + fk]);
#pragma unroll
                for (int i = 0; i < MB; i++)
#pragma unroll
                    for (int j = 0; j < NB; j++)
                        acc[i][j] = Mma<P>::run(fb[j], fa[i], acc[i][j]);
            }
            lstore(h ^ 1, h ^ 1);
            __syncthreads();
        }

        // The last slice sat in stage 1, which is free now (stage 0 already holds
        // the next item's first slice).
        P* stage = smem + STAGE;
        constexpr int CPR = BN / EPC;
        constexpr int PROWS = BM / EP_PARTS;
#pragma unroll
        for (int part = 0; part < EP_PARTS; part++) {
            if (EP_PARTS == 1 || wy == part) {
#pragma unroll
                for (int i = 0; i < MB; i++)
#pragma unroll
                    for (int j = 0; j < NB; j++)
#pragma unroll
                        for (int q = 0; q < 4; q++) {
                            typename Quad<P>::type v;
#pragma unroll
                            for (int e = 0; e < 4; e++) v[e] = to_storage<P>(acc[i][j][q * 4 + e]);
                            const int row = (EP_PARTS == 1 ? wy * WM : 0) + i * 32 + crow;
                            *reinterpret_cast<typename Quad<P>::type*>(
                                &stage[row * CROW + wx * WN + j * 32 + 8 * q + ccol]) = v;
                        }
            }
            __syncthreads();
#pragma unroll 4
            for (int q = tid; q < PROWS * CPR; q += 256) {
                const int row = q / CPR, ch = q - row * CPR;
                *reinterpret_cast<int4v*>(cur.m + (size_t)(part * PROWS + row) * Kp + ch * EPC) =
                    *reinterpret_cast<const int4v*>(&stage[row * CROW + ch * EPC]);
            }
            __syncthreads();
        }
        if (!has_next) break;
        item = nitem;
        cur = nxt;
    }
}

// Large-tile variant: one workgroup of 8 wavefronts (2 x 4) owns a 256 x 256
// tile, i.e. all output channels of 256 tiles when the network has 256
// filters.  Per multiply-add it moves half as many operand bytes from L2 to
// the compute unit as the 128 x 128 tile, which is what bounds this GEMM (its
// contraction is only 256 deep); at 64 boards the 7 x 36 tiles fill the 256
// compute units in a single round.
template <typename P, int NK>
__global__ __launch_bounds__(512) void wino_gemm_big_k(const P* __restrict__ V,
                                                       const P* __restrict__ U,
                                                       P* __restrict__ M, int T, int Tp, int Cp,
                                                       int Kp, int tiles_m, int tiles_n, int seg) {
    constexpr int BM = 256, BN = 256, NT = 512;
    constexpr int EPC = 16 / sizeof(P);
    constexpr int BK = 128 / sizeof(P);
    constexpr int ROW = BK + EPC;
    constexpr int WM = 128, WN = 64;       // per-wave tile, waves laid out 2 (rows) x 4 (columns)
    constexpr int MB = WM / 32, NB = WN / 32;
    constexpr int A_CH = BM * 8 / NT, B_CH = BN * 8 / NT;
    constexpr int CROW = BN + EPC;
    constexpr int STAGE = (BM + BN) * ROW;
    constexpr int EP_PARTS = sizeof(P) == 2 ? 2 : 4;   // output staged through one vacated stage
    constexpr int PROWS = BM / EP_PARTS;
    static_assert(PROWS * CROW <= STAGE, "output staging does not fit a stage");

    __shared__ __attribute__((aligned(16))) P smem[2 * STAGE];

    const int n_items = kPos * tiles_m * tiles_n;
    const int xcd = blockIdx.x & 7;
    const int item = xcd * seg + (blockIdx.x >> 3);
    if ((int)(blockIdx.x >> 3) >= seg || item >= n_items) return;
    const int tn = item % tiles_n;
    const int rest = item / tiles_n;
    const int tm = rest % tiles_m;
    const int p = rest / tiles_m;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wy = wave >> 2, wx = wave & 3;
    const int lrow = tid >> 3, lch = tid & 7;   // 64 rows per pass of the workgroup
    // Rows past the last real tile re-read row T-1 (their products are never stored).
    const P* Ag[A_CH];
#pragma unroll
    for (int i = 0; i < A_CH; i++) {
        const int row = min(tm * BM + lrow + i * 64, T - 1);
        Ag[i] = V + ((size_t)p * Tp + row) * Cp + lch * EPC;
    }
    const P* Bg = U + ((size_t)p * Kp + (size_t)tn * BN + lrow) * Cp + lch * EPC;

    float16v acc[MB][NB];
#pragma unroll
    for (int i = 0; i < MB; i++)
#pragma unroll
        for (int j = 0; j < NB; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0.0f;

    int4v ra[2][A_CH], rb[2][B_CH];
    auto gload = [&](int st, int k0) {
#pragma unroll
        for (int i = 0; i < A_CH; i++)
            ra[st][i] = *reinterpret_cast<const int4v*>(Ag[i] + k0);
#pragma unroll
        for (int i = 0; i < B_CH; i++)
            rb[st][i] = *reinterpret_cast<const int4v*>(Bg + (size_t)(i * 64) * Cp + k0);
    };
    auto lstore = [&](int st, int buf) {
        P* As = smem + buf * STAGE;
        P* Bs = As + BM * ROW;
#pragma unroll
        for (int i = 0; i < A_CH; i++)
            *reinterpret_cast<int4v*>(&As[(lrow + i * 64) * ROW + lch * EPC]) = ra[st][i];
#pragma unroll
        for (int i = 0; i < B_CH; i++)
            *reinterpret_cast<int4v*>(&Bs[(lrow + i * 64) * ROW + lch * EPC]) = rb[st][i];
    };

    const int rot = p % NK;
    gload(0, rotated_slice(0, rot, NK) * BK);
    if (NK > 1) gload(1, rotated_slice(1, rot, NK) * BK);
    lstore(0, 0);
    __syncthreads();

    const int frow = lane & 31, fk = (lane >> 5) * EPC;
#pragma unroll
    for (int k = 0; k < NK; k++) {
        const int h = k & 1;
        if (k + 2 < NK) {
            gload(h, rotated_slice(k + 2, rot, NK) * BK);
            __builtin_amdgcn_sched_barrier(0);
        }
        const P* As = smem + h * STAGE;
        const P* Bs = As + BM * ROW;
#pragma unroll
        for (int kc = 0; kc < 4; kc++) {
            int4v fa[MB], fb[NB];
#pragma unroll
            for (int i = 0; i < MB; i++)
                fa[i] = *reinterpret_cast<const int4v*>(
                    &As[(wy * WM + i * 32 + frow) * ROW + kc * 2 * EPC + fk]);
#pragma unroll
            for (int j = 0; j < NB; j++)
                fb[j] = *reinterpret_cast<const int4v*>(
                    &Bs[(wx * WN + j * 32 + frow) * ROW + kc * 2 * EPC + fk]);
#pragma unroll
            for (int i = 0; i < MB; i++)
#pragma unroll
                for (int j = 0; j < NB; j++) acc[i][j] = Mma<P>::run(fb[j], fa[i], acc[i][j]);
        }
        if (k + 1 < NK) lstore(h ^ 1, h ^ 1);
        __syncthreads();
    }

    // Output: PROWS rows at a time through LDS, then out in 16-byte pieces.
    const int ccol = 4 * (lane >> 5), crow = lane & 31;
    constexpr int CPR = BN / EPC;
    P* Mg = M + ((size_t)p * Tp + (size_t)tm * BM) * Kp + (size_t)tn * BN;
    const int real_rows = T - tm * BM;   // rows of this tile that hold tiles of a board
#pragma unroll
    for (int part = 0; part < EP_PARTS; part++) {
#pragma unroll
        for (int i = 0; i < MB; i++) {
            const int row0 = wy * WM + i * 32;      // first tile row of this MFMA block
            if (row0 / PROWS == part) {             // uniform per wave
#pragma unroll
                for (int j = 0; j < NB; j++)
#pragma unroll
                    for (int q = 0; q < 4; q++) {
                        typename Quad<P>::type v;
#pragma unroll
                        for (int e = 0; e < 4; e++) v[e] = to_storage<P>(acc[i][j][q * 4 + e]);
                        *reinterpret_cast<typename Quad<P>::type*>(
                            &smem[(row0 - part * PROWS + crow) * CROW + wx * WN + j * 32 + 8 * q +
                                  ccol]) = v;
                    }
            }
        }
        __syncthreads();
#pragma unroll 4
        for (int q = tid; q < PROWS * CPR; q += NT) {
            const int row = q / CPR, ch = q - row * CPR;
            if (part * PROWS + row < real_rows)   // padding rows are never read back
                *reinterpret_cast<int4v*>(Mg + (size_t)(part * PROWS + row) * Kp + ch * EPC) =
                    *reinterpret_cast<const int4v*>(&smem[row * CROW + ch * EPC]);
        }
        __syncthreads();
    }
}

template <typename P, int BN, int NK>
static void launch_gemm_nk(const P* V, const P* U, P* M, int tiles_m, int Tp, int Cp, int Kp,
                           hipStream_t s, LaunchTimer* t) {
    const int tiles_n = Kp / BN;
    const int n_items = kPos * tiles_m * tiles_n;
    int seg = (n_items + 7) / 8;
    seg = (seg + tiles_n - 1) / tiles_n * tiles_n;  // keep the column tiles of a row tile together
    if constexpr (NK >= 2 && (NK % 2) == 0 && BN == 128) {
        // two resident workgroups on each of a die's 32 compute units
        const int wg_per_xcd = seg < 64 ? seg : 64;
        launch(wino_gemm_persistent_k<P, kGemmBM, BN, NK>, dim3(8 * wg_per_xcd), dim3(256), s, t,
               V, U, M, Tp, Cp, Kp, tiles_m, tiles_n, seg, wg_per_xcd);
    } else {
        launch(wino_gemm_k<P, kGemmBM, BN, NK>, dim3(8 * seg), dim3(256), s, t, V, U, M, Tp, Cp,
               Kp, tiles_m, tiles_n, seg);
    }
}

// Channel counts are multiples of 64, so the number of 128-byte k-slices is
// Cp/64 for fp16 and Cp/32 for fp32; 1..8, 10, 12, 14 and 16 slices are instantiated
// (every width up to 512 channels in both types, 640..1024 by 128 in fp16).
template <typename P, int BN>
static void launch_gemm_bn(const P* V, const P* U, P* M, int tiles_m, int Tp, int Cp, int Kp,
                           hipStream_t s, LaunchTimer* t) {
    constexpr int BK = 128 / (int)sizeof(P);
    switch (Cp / BK) {
#define LZ_NK(N) case N: launch_gemm_nk<P, BN, N>(V, U, M, tiles_m, Tp, Cp, Kp, s, t); return;
        LZ_NK(1) LZ_NK(2) LZ_NK(3) LZ_NK(4) LZ_NK(5) LZ_NK(6) LZ_NK(7) LZ_NK(8)
        LZ_NK(10) LZ_NK(12) LZ_NK(14) LZ_NK(16)
#undef LZ_NK
        default: break;
    }
    // the pipe refuses such widths at creation (gemm_supports_channels)
    throw std::invalid_argument("no GEMM instantiated for this channel count");
}

// The 256 x 256 tile computed as two 128-row passes.  The stores of the first
// pass drain while the second pass streams its operands, so only half of the
// output is written with nothing else in flight; the price is that the U tile
// is read twice (the second time from L2).  The operand loads of the second
// pass are issued before the first pass's output leaves, and a second pass
// that holds only padding rows is skipped.
template <typename P, int NK, int HM>
__global__ __launch_bounds__(512) void wino_gemm_split_k(const P* __restrict__ V,
                                                         const P* __restrict__ U,
                                                         P* __restrict__ M, int T, int Tp, int Cp,
                                                         int Kp, int tiles_m, int tiles_n, int seg) {
    constexpr int BM = 256, BN = 256, NT = 512;
    constexpr int PASSES = BM / HM;
    constexpr int EPC = 16 / sizeof(P);
    constexpr int BK = 128 / sizeof(P);
    constexpr int ROW = BK + EPC;
    constexpr int WM = HM / 2, WN = 64;    // per-wave tile, waves laid out 2 (rows) x 4 (columns)
    constexpr int MB = WM / 32, NB = WN / 32;
    constexpr int A_CH = HM * 8 / NT, B_CH = BN * 8 / NT;
    constexpr int CROW = BN + EPC;
    constexpr int STAGE = (HM + BN) * ROW;
    constexpr int PROWS = sizeof(P) == 2 ? 64 : 32;
    constexpr int EP_PARTS = HM / PROWS;
    static_assert(PROWS * CROW <= STAGE, "output staging does not fit a stage");
    static_assert(HM % 64 == 0 && EP_PARTS >= 1, "pass height");

    __shared__ __attribute__((aligned(16))) P smem[2 * STAGE];

    const int n_items = kPos * tiles_m * tiles_n;
    const int xcd = blockIdx.x & 7;
    const int item = xcd * seg + (blockIdx.x >> 3);
    if ((int)(blockIdx.x >> 3) >= seg || item >= n_items) return;
    const int tn = item % tiles_n;
    const int rest = item / tiles_n;
    const int tm = rest % tiles_m;
    const int p = rest / tiles_m;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wy = wave >> 2, wx = wave & 3;
    const int lrow = tid >> 3, lch = tid & 7;   // 64 rows per pass of the workgroup
    const P* Bg = U + ((size_t)p * Kp + (size_t)tn * BN + lrow) * Cp + lch * EPC;
    const int rot = p % NK;
    const int frow = lane & 31, fk = (lane >> 5) * EPC;
    const int ccol = 4 * (lane >> 5), crow = lane & 31;
    constexpr int CPR = BN / EPC;

    int4v ra[2][A_CH], rb[2][B_CH];
    const P* Ag[A_CH];
    auto set_rows = [&](int half) {
#pragma unroll
        for (int i = 0; i < A_CH; i++) {
            const int row = min(tm * BM + half * HM + lrow + i * 64, T - 1);
            Ag[i] = V + ((size_t)p * Tp + row) * Cp + lch * EPC;
        }
    };
    auto gload = [&](int st, int k0) {
#pragma unroll
        for (int i = 0; i < A_CH; i++)
            ra[st][i] = *reinterpret_cast<const int4v*>(Ag[i] + k0);
#pragma unroll
        for (int i = 0; i < B_CH; i++)
            rb[st][i] = *reinterpret_cast<const int4v*>(Bg + (size_t)(i * 64) * Cp + k0);
    };
    auto lstore = [&](int st, int buf) {
        P* As = smem + buf * STAGE;
        P* Bs = As + HM * ROW;
#pragma unroll
        for (int i = 0; i < A_CH; i++)
            *reinterpret_cast<int4v*>(&As[(lrow + i * 64) * ROW + lch * EPC]) = ra[st][i];
#pragma unroll
        for (int i = 0; i < B_CH; i++)
            *reinterpret_cast<int4v*>(&Bs[(lrow + i * 64) * ROW + lch * EPC]) = rb[st][i];
    };

    const int real_rows = T - tm * BM;          // rows of the tile that belong to boards
    const int halves = min(PASSES, (real_rows + HM - 1) / HM);  // uniform over the workgroup

    set_rows(0);
    gload(0, rotated_slice(0, rot, NK) * BK);
    if (NK > 1) gload(1, rotated_slice(1, rot, NK) * BK);

#pragma unroll
    for (int half = 0; half < PASSES; half++) {
        if (half < halves) {
            float16v acc[MB][NB];
#pragma unroll
            for (int i = 0; i < MB; i++)
#pragma unroll
                for (int j = 0; j < NB; j++)
#pragma unroll
                    for (int r = 0; r < 16; r++) acc[i][j][r] = 0.0f;

            lstore(0, 0);
            __syncthreads();
#pragma unroll
            for (int k = 0; k < NK; k++) {
                const int h = k & 1;
                if (k + 2 < NK) {
                    gload(h, rotated_slice(k + 2, rot, NK) * BK);
                    __builtin_amdgcn_sched_barrier(0);
                } else if (half + 1 < halves) {
                    // the first slices of the next pass take the free register stages
                    if (k + 2 == NK) set_rows(half + 1);
                    gload(h, rotated_slice(k + 2 - NK, rot, NK) * BK);
                    __builtin_amdgcn_sched_barrier(0);
                }
                const P* As = smem + h * STAGE;
                const P* Bs = As + HM * ROW;
#pragma unroll
                for (int kc = 0; kc < 4; kc++) {
                    int4v fa[MB], fb[NB];
#pragma unroll
                    for (int i = 0; i < MB; i++)
                        fa[i] = *reinterpret_cast<const int4v*>(
                            &As[(wy * WM + i * 32 + frow) * ROW + kc * 2 * EPC + fk]);
#pragma unroll
                    for (int j = 0; j < NB; j++)
                        fb[j] = *reinterpret_cast<const int4v*>(
                            &Bs[(wx * WN + j * 32 + frow) * ROW + kc * 2 * EPC + fk]);
#pragma unroll
                    for (int i = 0; i < MB; i++)
#pragma unroll
                        for (int j = 0; j < NB; j++)
                            acc[i][j] = Mma<P>::run(fb[j], fa[i], acc[i][j]);
                }
                if (k + 1 < NK) lstore(h ^ 1, h ^ 1);
                __syncthreads();
            }

            // Output of this pass: PROWS rows at a time through LDS, out in 16-byte pieces.
            P* Mg = M + ((size_t)p * Tp + (size_t)tm * BM + half * HM) * Kp + (size_t)tn * BN;
            const int rows_here = real_rows - half * HM;
#pragma unroll
            for (int part = 0; part < EP_PARTS; part++) {
#pragma unroll
                for (int i = 0; i < MB; i++) {
                    const int row0 = wy * WM + i * 32;
                    if (row0 / PROWS == part) {     // uniform per wave
#pragma unroll
                        for (int j = 0; j < NB; j++)
#pragma unroll
                            for (int q = 0; q < 4; q++) {
                                typename Quad<P>::type v;
#pragma unroll
                                for (int e = 0; e < 4; e++)
                                    v[e] = to_storage<P>(acc[i][j][q * 4 + e]);
                                *reinterpret_cast<typename Quad<P>::type*>(
                                    &smem[(row0 - part * PROWS + crow) * CROW + wx * WN + j * 32 +
                                          8 * q + ccol]) = v;
                            }
                    }
                }
                __syncthreads();
#pragma unroll 4
                for (int q = tid; q < PROWS * CPR; q += NT) {
                    const int row = q / CPR, ch = q - row * CPR;
                    if (part * PROWS + row < rows_here)
                        *reinterpret_cast<int4v*>(Mg + (size_t)(part * PROWS + row) * Kp +
                                                  ch * EPC) =
                            *reinterpret_cast<const int4v*>(&smem[row * CROW + ch * EPC]);
                }
                __syncthreads();
            }
        }
    }
}

// ---------------------------------------------------------------------------
// Filter-stationary streaming GEMM (fp16 storage).  One work-group of NW wavefronts
// (8 at 256 filters, 6 / 4 / 2 at 192 / 128 / 64) owns one Winograd position and a run of
// consecutive 32-row blocks of V; wavefront w owns output channels 32w..32w+31 of a
// column tile of 32 NW channels and keeps its
// share of U_p -- 32 channels x Cp input channels -- in registers for the whole
// kernel (Cp/4 registers per lane), already in the order the matrix instruction
// wants it.  V streams through: a 32-row block (all Cp input channels, so the
// contraction of those rows completes in one step) is requested kStreamAhead steps
// ahead into registers and passes through a three-stage LDS ring, where all
// wavefronts read it as their column operand.  A step multiplies one block; the
// fragment reads of the block's second half and of the next block's first half are
// issued ahead of the matrix instructions that hide them, and one barrier ends the
// step.  Loads of later blocks, matrix instructions and stores of earlier blocks are
// in flight together from the first block to the last.
//
// Output: register r of lane l of a 32x32 accumulator holds row 8(r/4) + 4(l/32) + r%4
// of the row operand.  The row operand is U, and the host stores U's channels permuted
// (gemm_stream_channel) so that this lane's sixteen registers are the channels
// 16(r/8) + 8(l/32) + r%8 of the wavefront's 32, i.e. two 16-byte runs.  Those go into
// an LDS copy of the block's 32 x 32 NW result, and one step later (behind the barrier
// that is there anyway) every wavefront sends its share of the rows, 1 KiB per store
// instruction.  The stores are write-through (sc0 sc1): whole lines leave for memory
// while the kernel runs, instead of collecting as dirty lines in the L2 that the end
// of the kernel has to flush with nothing else in flight (measured at 64 boards and
// 256 filters: 14.2 -> 12.3 us per launch; in 32-byte pieces straight from the
// accumulators write-through is slower than write-back).
//
// Uf layout ("fragment order"): [36][Kp/32][Cp/16][64 lanes][8 halves]; lane l of
// fragment (p, wb, kc) holds U_p[32 wb + gemm_stream_channel(l % 32)][16 kc + 8 (l / 32) + 0..7],
// so every operand load of a wavefront is one contiguous KiB.
constexpr int kStreamBlocks = 16;  // most 32-row blocks per work-group (steps of the pipeline)
constexpr int kStreamAhead = 2;    // blocks requested ahead of the one being multiplied

__host__ __device__ constexpr int gemm_stream_channel(int i) {
    // i = 8q + 4h + e  ->  16 (q / 2) + 8 h + 4 (q % 2) + e
    return 16 * (i >> 4) + 8 * ((i >> 2) & 1) + 4 * ((i >> 3) & 1) + (i & 3);
}

// What a fused launch hands the GEMM's work-groups to wait on (see xform_gemm_k): one
// 64-bit word per (board, channel group) of the transform that produces V in the same
// launch, set to `epoch` when that work-group's stores have reached memory.
struct StreamWait {
    const unsigned long long* flags;
    unsigned long long epoch;
    unsigned* gave_up;     // set to 1 if a wait ran into its spin limit
    int ncg;               // channel groups per board
};
constexpr int kFlagSpinLimit = 1 << 18;   // polls of ~0.3 us each before a wait gives up

// LDS of the streaming GEMM in halves: the ring of V blocks (as many stages as the
// pipeline can use) and two copies of a block's result.
template <int NKC, int NBLK, int NW> constexpr int gemm_stream_lds_halves() {
    return (NBLK < 3 ? NBLK : 3) * 32 * (NKC * 16 + 8) + 2 * 32 * (32 * NW + 8);
}

// FUSED: the work-group is part of a fused launch (xform_gemm_k): it waits for the producers
// of its rows.  VSLAB / MSLAB > 0: V is read / M is written slab by slab,
// [Kp / SLAB][Tp][SLAB] per position, instead of row by row, [Tp][Kp] (the layout the narrow
// transform shapes work in, where a work-group's 25 tiles are one contiguous run).
template <int NKC, int NBLK, int NW, bool FUSED, int VSLAB = 0, int MSLAB = 0>
__device__ __forceinline__ void wino_gemm_stream_body(half_t* smem, unsigned wg, const half_t* V,
                                                      const half_t* __restrict__ Uf, half_t* M,
                                                      int T, int Tp, int Kp, int chunks,
                                                      int nblk_total, int tiles_n, int seg,
                                                      StreamWait wait) {
    constexpr int D = kStreamAhead;
    constexpr int NT = 64 * NW;                  // threads: NW wavefronts of 32 output channels
    constexpr int CW = 32 * NW;                  // width of the column tile
    constexpr int Cp = NKC * 16;
    constexpr int HK = NKC / 2;                  // fragments per half block
    constexpr int CPRW = Cp / 8;                 // 16-byte chunks per row
    constexpr int NCH = 32 * CPRW;               // chunks per block
    constexpr int CH = (NCH + NT - 1) / NT;      // chunk loads per thread and block
    constexpr bool FULL = NCH % NT == 0;         // every thread has all CH chunks
    constexpr int ROWE = Cp + 8;                 // padded LDS row (halves): conflict-free 16-byte reads
    constexpr int STAGE = 32 * ROWE;
    constexpr int OROW = CW + 8;                 // row of the output copy (halves)
    constexpr int OSTAGE = 32 * OROW;
    static_assert(NKC % 2 == 0 && D == 2, "pipeline shape");
    constexpr int SLAB = VSLAB;
    static_assert((VSLAB == 0 || VSLAB == 16 || VSLAB == 32) &&
                      (MSLAB == 0 || MSLAB == 16 || MSLAB == 32),
                  "slab widths");

    constexpr int NST = NBLK < 3 ? NBLK : 3;     // stages of the ring in use
    static_assert(NST * STAGE + 2 * OSTAGE == gemm_stream_lds_halves<NKC, NBLK, NW>(), "LDS size");
    half_t* const obuf = smem + NST * STAGE;

    const int n_items = kPos * chunks * tiles_n;
    const int xcd = wg & 7;
    const int item = xcd * seg + (int)(wg >> 3);
    if ((int)(wg >> 3) >= seg || item >= n_items) return;
    const int tn = item % tiles_n;
    const int rest = item / tiles_n;
    const int ch = rest % chunks;
    const int p = rest / chunks;
    // this work-group's real blocks: [blk0, blk1), at most NBLK of them
    const int blk0 = (ch * nblk_total) / chunks;
    const int blk1 = ((ch + 1) * nblk_total) / chunks;
    const int nreal = blk1 - blk0;

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int hh = lane >> 5, jrow = lane & 31;

    // chunk coordinates of this thread's loads within a block
    int lrow[CH], lcc[CH];
    bool lval[CH];
    unsigned lslab[CH];   // slab layout: byte offset of the chunk's slab and place in its row
#pragma unroll
    for (int i = 0; i < CH; i++) {
        const int idx = tid + i * NT;
        lval[i] = FULL || idx < NCH;
        if constexpr (SLAB > 0) {
            // a wavefront's 64 chunks are consecutive rows of one slab: one contiguous KiB
            constexpr int CPS = SLAB / 8;               // chunks per row of a slab
            const int g = idx / (32 * CPS), rem = idx % (32 * CPS);
            lrow[i] = rem / CPS;
            lcc[i] = g * CPS + rem % CPS;
            lslab[i] = ((unsigned)g * (unsigned)Tp * SLAB + (unsigned)(rem % CPS) * 8u) * 2u;
        } else {
            lrow[i] = (idx / CPRW) & 31;
            lcc[i] = idx % CPRW;
            lslab[i] = 0;
        }
    }
    const half_t* Vp = V + (size_t)p * Tp * Cp;

    int4v st[D][CH];
    // In a fused launch V has just been written by work-groups of the same launch on other
    // dies: its loads carry the device-scope policy (sc1), which takes them past this
    // die's caches to where those (written-through) stores went.
    const __amdgpu_buffer_rsrc_t rV = make_rsrc(Vp, (size_t)Tp * Cp * sizeof(half_t));
    auto gload = [&](int slot, int s) {
        // steps past the last real block re-read that block (cache hits, never stored)
        const int blk = blk0 + (s < nreal ? s : nreal - 1);
#pragma unroll
        for (int i = 0; i < CH; i++) {
            const int row = min(blk * 32 + lrow[i], T - 1);
            if (lval[i]) {
                if constexpr (SLAB > 0)
                    st[slot][i] = __builtin_amdgcn_raw_buffer_load_b128(
                        rV, lslab[i] + (unsigned)row * (unsigned)(SLAB * 2), 0, FUSED ? 16 : 0);
                else if constexpr (FUSED)
                    st[slot][i] = __builtin_amdgcn_raw_buffer_load_b128(
                        rV, (unsigned)(row * Cp + lcc[i] * 8) * 2u, 0, 16);
                else
                    st[slot][i] =
                        *reinterpret_cast<const int4v*>(Vp + (size_t)row * Cp + lcc[i] * 8);
            }
        }
    };
    auto lstore = [&](int slot, int buf) {
        half_t* S = smem + buf * STAGE;
#pragma unroll
        for (int i = 0; i < CH; i++)
            if (lval[i]) *reinterpret_cast<int4v*>(&S[lrow[i] * ROWE + lcc[i] * 8]) = st[slot][i];
    };

    // The first two blocks of V, then this wavefront's share of U in the order the
    // multiplication uses it.  (Completion is counted in issue order: the LDS stores below
    // wait for V only, and each matrix instruction of the first step only for the filter
    // fragments up to its own, so the first step starts while most of U is still arriving:
    // -0.5 us per launch at 64 boards against U first.)
    int4v u[NKC];
    const half_t* Up =
        Uf + ((((size_t)p * (Kp / 32) + (size_t)tn * NW + wave) * NKC) * 64 + lane) * 8;
    if constexpr (FUSED) {
        // The filters depend on nothing in this launch: they are requested first and
        // arrive while the transform work-groups are still producing V.  Then wait for the
        // transform work-groups of every board that has a tile among this work-group's rows.
#pragma unroll
        for (int kc = 0; kc < NKC; kc++)
            u[kc] = *reinterpret_cast<const int4v*>(Up + (size_t)kc * 64 * 8);
        LZ_STAMP(10);
        const int row_lo = blk0 * 32, row_hi = min(blk1 * 32, T);
        const int b_lo = row_lo / kTilesPerBoard, b_hi = (row_hi - 1) / kTilesPerBoard;
        const int nflags = (b_hi - b_lo + 1) * wait.ncg;
        const unsigned long long* f = wait.flags + (size_t)b_lo * wait.ncg;
        for (int i = tid; i < nflags; i += NT) {
            int polls = 0;
            while (__hip_atomic_load(f + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) !=
                   wait.epoch) {
                __builtin_amdgcn_s_sleep(2);
                if (++polls > kFlagSpinLimit) {   // never hang: report and go on
                    __hip_atomic_store(wait.gave_up, 1u, __ATOMIC_RELAXED,
                                       __HIP_MEMORY_SCOPE_SYSTEM);
                    break;
                }
            }
        }
        __syncthreads();
        LZ_STAMP(11);
        gload(0, 0);
        if (NBLK > 1) gload(1, 1);
    } else {
        gload(0, 0);
        if (NBLK > 1) gload(1, 1);
#pragma unroll
        for (int kc = 0; kc < NKC; kc++)
            u[kc] = *reinterpret_cast<const int4v*>(Up + (size_t)kc * 64 * 8);
    }
    lstore(0, 0);
    if (NBLK > 1) lstore(1, 1);
    __syncthreads();
    LZ_STAMP(12);

    // M goes out through a raw buffer whose extent is the T real rows of this position:
    // rows past the last tile, and the steps past this work-group's last block, get an
    // offset outside it and are dropped by the hardware, so the stores are unconditional
    // straight-line code (a branch around them would make the compiler wait for every
    // outstanding load behind it).
    const size_t m_bytes = (size_t)(MSLAB > 0 ? Tp : T) * Kp * sizeof(half_t);
    const __amdgpu_buffer_rsrc_t rM = make_rsrc(M + (size_t)p * Tp * Kp, m_bytes);
    const unsigned m_rowb = (unsigned)Kp * 2u;
    // The 32 x CW result leaves in 16-byte pieces, two per thread.  Eight wavefronts:
    // wavefront w sends rows 4w..4w+3, two whole 512-byte rows per store instruction.  Fewer:
    // the pieces are dealt to the threads in memory order (a row holds CW / 8 of them), so
    // that a store instruction still writes one contiguous KiB when the tile is the whole row.
    // Slabs: a slab's share of the block (32 rows x MSLAB channels) is contiguous, and the
    // pieces are dealt in that order, so a store instruction again writes one contiguous KiB.
    constexpr int PPR = CW / 8;
    auto send_rows = [&](int s) {
        const half_t* O = obuf + (s & 1) * OSTAGE;
#pragma unroll
        for (int i = 0; i < 2; i++) {
            int r, cc;
            if constexpr (MSLAB > 0) {
                constexpr int PR = MSLAB / 8;              // pieces per row of a slab
                const int piece = tid + i * NT;
                const int g = piece / (32 * PR), rem = piece - g * (32 * PR);
                r = rem / PR;
                cc = g * PR + (rem - r * PR);
            } else if constexpr (NW == 8) {
                r = wave * 4 + hh + 2 * i;
                cc = jrow;
            } else {
                const int piece = tid + i * NT;
                r = piece / PPR;
                cc = piece - r * PPR;
            }
            const int4v v = *reinterpret_cast<const int4v*>(O + r * OROW + cc * 8);
            const unsigned row = (unsigned)((blk0 + s) * 32 + r);
            unsigned vo;
            if constexpr (MSLAB > 0) {
                constexpr int PR = MSLAB / 8;
                const unsigned slab = (unsigned)(tn * (CW / MSLAB) + cc / PR);
                vo = (s < nreal && row < (unsigned)T)
                         ? ((slab * (unsigned)Tp + row) * (unsigned)MSLAB + (unsigned)(cc % PR) * 8u) * 2u
                         : 0x7ffffff0u;
            } else {
                vo = s < nreal ? row * m_rowb + (unsigned)(tn * CW + cc * 8) * 2u : 0x7ffffff0u;
            }
            __builtin_amdgcn_raw_buffer_store_b128(v, rM, vo, 0, kStoreThrough);
        }
    };

    const int frag = jrow * ROWE + hh * 8;
    int4v alo[HK], ahi[HK];
#pragma unroll
    for (int kc = 0; kc < HK; kc++) alo[kc] = *reinterpret_cast<const int4v*>(smem + frag + kc * 16);

    // Every work-group runs all NBLK steps; those past its last block multiply stale data and
    // store nothing.  (Leaving after nreal steps, with the blocks split evenly over 7
    // work-groups per position at every batch, was measured and is slower in this kernel,
    // which the stream bounds: one lane -1 % at 64 boards, -6 % at 96, +5 % at 40.)
#pragma unroll
    for (int s = 0; s < NBLK; s++) {
        if (s + D < NBLK) gload(s % D, s + D);
        if (s > 0) send_rows(s - 1);
        const half_t* S = smem + (s % 3) * STAGE + frag;
#pragma unroll
        for (int kc = 0; kc < HK; kc++)
            ahi[kc] = *reinterpret_cast<const int4v*>(S + (HK + kc) * 16);
        __builtin_amdgcn_sched_barrier(0);
        float16v acc;
#pragma unroll
        for (int r = 0; r < 16; r++) acc[r] = 0.0f;
#pragma unroll
        for (int kc = 0; kc < HK; kc++)
            acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8v, u[kc]),
                                                         __builtin_bit_cast(half8v, alo[kc]), acc,
                                                         0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
        if (s + 1 < NBLK) {
            const half_t* Sn = smem + ((s + 1) % 3) * STAGE + frag;
#pragma unroll
            for (int kc = 0; kc < HK; kc++)
                alo[kc] = *reinterpret_cast<const int4v*>(Sn + kc * 16);
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int kc = 0; kc < HK; kc++)
            acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8v, u[HK + kc]),
                                                         __builtin_bit_cast(half8v, ahi[kc]), acc,
                                                         0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
        if (s + 2 < NBLK) lstore((s + 2) % D, (s + 2) % 3);
        half8v o0, o1;
#pragma unroll
        for (int e = 0; e < 8; e++) {
            o0[e] = to_storage<half_t>(acc[e]);
            o1[e] = to_storage<half_t>(acc[8 + e]);
        }
        half_t* O = obuf + (s & 1) * OSTAGE + jrow * OROW + wave * 32 + hh * 8;
        *reinterpret_cast<half8v*>(O) = o0;
        *reinterpret_cast<half8v*>(O + 16) = o1;
        __syncthreads();
        LZ_STAMP(13 + s);
    }
    send_rows(NBLK - 1);
}

// V and M may be one array when the tile is the whole row of M (tiles_n == 1, as many input
// as output channels): a work-group has a block of V in LDS before it writes the block of M
// that takes its place, and no other work-group touches those rows.
template <int NKC, int NBLK, int NW, int VSLAB = 0, int MSLAB = 0>
__global__ __launch_bounds__(64 * NW) void wino_gemm_stream_k(const half_t* V,
                                                          const half_t* __restrict__ Uf,
                                                          half_t* M, int T, int Tp,
                                                          int Kp, int chunks, int nblk_total,
                                                          int tiles_n, int seg) {
    __shared__ __attribute__((aligned(16))) half_t smem[gemm_stream_lds_halves<NKC, NBLK, NW>()];
    wino_gemm_stream_body<NKC, NBLK, NW, false, VSLAB, MSLAB>(
        smem, blockIdx.x, V, Uf, M, T, Tp, Kp, chunks, nblk_total, tiles_n, seg, StreamWait{});
}

// ---------------------------------------------------------------------------
// One launch for the fused transform of layer l (M_l -> V_{l+1}) and the GEMM of layer l+1
// (V_{l+1} -> M_{l+1}), for small batches.  Two dependent launches cost a hand-over of
// ~2.4 us between them whatever their size, and a GEMM work-group spends its first ~2 us
// fetching 128 KiB of filters that depend on nothing: at 16 boards those two are a third of
// a layer.  Here the launch's first work-groups run the transform and the rest the GEMM.
// The GEMM work-groups request their filters at once, then wait, per board whose tiles
// they multiply, for a word that each transform work-group sets (to the launch's `epoch`,
// a number that grows with every fused launch of a lane, so nothing has to be cleared)
// after its stores of V -- written through, with the device-scope policy -- have been
// acknowledged; the GEMM work-groups read V with the same policy.  (Release and acquire
// fences in their place would write back and invalidate a die's whole L2 once per wavefront:
// measured 60 us per launch at 16 boards.)  With few boards the transform leaves compute
// units free, and the GEMM work-groups that start there have their filters by the time V
// is ready; from 16 boards they follow as the transform's work-groups retire, and the
// launch still saves the hand-over.
//
// Waiting is safe because the waiters never hold what the producers need: work-groups are
// dispatched in the order of their index, so every transform work-group is resident (or
// done) before the first GEMM work-group starts, and a transform work-group waits for
// nothing.  A wait is bounded all the same: after kFlagSpinLimit polls it reports through
// `gave_up` and goes on, so that the launch always ends.
//
// The buffers: the transform reads M and writes V, the GEMM reads V and writes M -- the
// same M.  A GEMM work-group writes rows of M only after every transform work-group of
// the boards those rows belong to has finished, i.e. after their last read.  V and M are
// normally one array, each stage overwriting its input, as the separate launches do.
// SLAB: both lie slab by slab, [36][Kp / CG][Tp][CG] (tile_slab), so that the transform reads
// and writes whole lines; row by row, its written-through 32- and 64-byte pieces of V land in
// lines that the die's L2 already holds from reading M.
template <int CG, int NBLK, int NW, bool SLAB>
__global__ __launch_bounds__(64 * (NW > fuse_waves(CG) ? NW : fuse_waves(CG))) void xform_gemm_k(
    half_t* M, const half_t* res, half_t* act_out, half_t* V, const float* __restrict__ bn_scale,
    const float* __restrict__ bn_mean, float rfac, int n, int Kp, int Tp,
    const half_t* __restrict__ Uf, int T, int chunks, int nblk_total, int tiles_n, int seg,
    unsigned n_xform_wg, unsigned long long* flags, unsigned long long epoch, unsigned* gave_up) {
    typedef BufIO2<half_t>::pair_t pair_t;
    constexpr int NKC = 2 * NW;      // tower layers: as many input as output channels
    constexpr int XBYTES = plane_pairs(CG) * (int)sizeof(pair_t);
    constexpr int GBYTES = gemm_stream_lds_halves<NKC, NBLK, NW>() * 2;
    // More than half of a compute unit's 160 KiB, whatever the roles need: two work-groups of
    // this launch never share a unit.  A GEMM work-group beside a transform work-group sends
    // its 128 KiB of filters through the memory pipeline that the transform -- which the
    // whole launch waits for -- is using (measured at 16 boards: 16.7 us per launch with
    // sharing, also with the filter requests spread out in time, 16.1 without).
    constexpr int ALONE = 82 * 1024;
    constexpr int NEED = XBYTES > GBYTES ? XBYTES : GBYTES;
    __shared__ __attribute__((aligned(16))) unsigned char lds[NEED > ALONE ? NEED : ALONE];
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    LZ_STAMP(0);
    if (blockIdx.x < n_xform_wg) {
        if (wave >= fuse_waves(CG)) return;    // the block is sized for the larger role
        const int item = out_in_transform_body<half_t, CG, kStoreThrough, SLAB, SLAB>(
            reinterpret_cast<pair_t*>(lds), blockIdx.x, M, res, act_out, V, bn_scale, bn_mean,
            rfac, n, Kp, Tp);
        if (item < 0) return;                  // uniform over the work-group
        // V was stored write-through: once a wavefront's stores are acknowledged they are in
        // memory, past every die's cache.  All wavefronts wait for that, then one word says so.
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        LZ_STAMP(6);
        __syncthreads();
        if (threadIdx.x == 0)
            __hip_atomic_store(flags + item, epoch, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        LZ_STAMP(7);
    } else {
        if (wave >= NW) return;
        wino_gemm_stream_body<NKC, NBLK, NW, true, SLAB ? CG : 0, SLAB ? CG : 0>(
            reinterpret_cast<half_t*>(lds), blockIdx.x - n_xform_wg, V, Uf, M, T, Tp, Kp, chunks,
            nblk_total, tiles_n, seg, StreamWait{flags, epoch, gave_up, Kp / CG});
    }
}

// ---------------------------------------------------------------------------
// The same filter-stationary structure in fp32 (v_mfma_f32_32x32x2_f32, a sixteenth of
// the fp16 matrix rate: this kernel is bound by the matrix pipe, not by the stream).
// Wavefront w keeps U_p for its 32 output channels in Cp/2 registers per lane; a step
// multiplies one 32-row block of V, 4 matrix instructions per 16-byte fragment read, so
// that nothing but the matrix pipe is busy for long.  The contraction index is dealt so
// that one 16-byte read serves four instructions: in instruction 4j + i, lanes 0..31
// hold input channel 8j + i and lanes 32..63 channel 8j + 4 + i, of U (rows) and of V
// (columns) alike.  The block's result goes through a single LDS copy (two barriers per
// step are little beside 128 matrix instructions) and leaves as whole rows, written
// through, as in the fp16 kernel.  (Stored straight from the accumulators instead, 64
// bytes per lane with write-back stores and one barrier per step, the kernel is slower:
// 87 against 83 us per launch at 64 boards and 256 filters, 28 against 24 at 128 filters.)
//
// Uf layout: [36][Kp/32][Cp/8][64 lanes][4 floats]; lane l of fragment (p, wb, j) holds
// U_p[32 wb + gemm_stream_channel(l % 32)][8 j + 4 (l / 32) + 0..3].

template <int NK8, int NBLK, int NW>
__global__ __launch_bounds__(64 * NW) void wino_gemm_stream32_k(const float* V,   // may be M
                                                                const float* __restrict__ Uf,
                                                                float* M, int T,
                                                                int Tp, int Kp, int chunks,
                                                                int nblk_total, int seg) {
    constexpr int D = kStreamAhead;
    constexpr int NT = 64 * NW;
    constexpr int CW = 32 * NW;
    constexpr int Cp = NK8 * 8;
    constexpr int CPRW = Cp / 4;                 // 16-byte chunks per row
    constexpr int NCH = 32 * CPRW;               // chunks per block
    constexpr int CH = (NCH + NT - 1) / NT;
    constexpr bool FULL = NCH % NT == 0;
    constexpr int ROWE = Cp + 4;                 // padded LDS row (floats)
    constexpr int STAGE = 32 * ROWE;
    constexpr int OROW = CW + 4;
    static_assert(D == 2, "pipeline shape");

    __shared__ __attribute__((aligned(16))) float smem[3 * STAGE + 32 * OROW];
    float* const obuf = smem + 3 * STAGE;

    const int n_items = kPos * chunks;
    const int xcd = blockIdx.x & 7;
    const int item = xcd * seg + (blockIdx.x >> 3);
    if ((int)(blockIdx.x >> 3) >= seg || item >= n_items) return;
    const int ch = item % chunks;
    const int p = item / chunks;
    const int blk0 = (ch * nblk_total) / chunks;
    const int blk1 = ((ch + 1) * nblk_total) / chunks;
    const int nreal = blk1 - blk0;

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int hh = lane >> 5, jrow = lane & 31;

    int lrow[CH], lcc[CH];
    bool lval[CH];
#pragma unroll
    for (int i = 0; i < CH; i++) {
        const int idx = tid + i * NT;
        lval[i] = FULL || idx < NCH;
        lrow[i] = (idx / CPRW) & 31;
        lcc[i] = idx % CPRW;
    }
    const float* Vp = V + (size_t)p * Tp * Cp;

    int4v st[D][CH];
    auto gload = [&](int slot, int s) {
        // requests past the last real block re-read that block (cache hits, never used)
        const int blk = blk0 + (s < nreal ? s : nreal - 1);
#pragma unroll
        for (int i = 0; i < CH; i++) {
            const int row = min(blk * 32 + lrow[i], T - 1);
            if (lval[i])
                st[slot][i] =
                    *reinterpret_cast<const int4v*>(Vp + (size_t)row * Cp + lcc[i] * 4);
        }
    };
    auto lstore = [&](int slot, int buf) {
        float* S = smem + buf * STAGE;
#pragma unroll
        for (int i = 0; i < CH; i++)
            if (lval[i]) *reinterpret_cast<int4v*>(&S[lrow[i] * ROWE + lcc[i] * 4]) = st[slot][i];
    };

    gload(0, 0);
    if (NBLK > 1) gload(1, 1);
    float4v u[NK8];
    {
        const float* Up = Uf + ((((size_t)p * (Kp / 32) + wave) * NK8) * 64 + lane) * 4;
#pragma unroll
        for (int j = 0; j < NK8; j++)
            u[j] = *reinterpret_cast<const float4v*>(Up + (size_t)j * 64 * 4);
    }
    lstore(0, 0);
    if (NBLK > 1) lstore(1, 1);
    __syncthreads();

    // rows past the last tile get an offset outside the buffer and are dropped
    const size_t m_bytes = (size_t)T * Kp * sizeof(float);
    const __amdgpu_buffer_rsrc_t rM = make_rsrc(M + (size_t)p * Tp * Kp, m_bytes);
    const unsigned m_rowb = (unsigned)Kp * 4u;
    constexpr int PPR = CW / 4;                  // 16-byte pieces per row
    auto send_rows = [&](int s) {
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int piece = tid + i * NT;
            const int r = piece / PPR;
            const int cc = piece - r * PPR;
            const int4v v = *reinterpret_cast<const int4v*>(obuf + r * OROW + cc * 4);
            const unsigned row = (unsigned)((blk0 + s) * 32 + r);
            __builtin_amdgcn_raw_buffer_store_b128(v, rM, row * m_rowb + (unsigned)cc * 16u, 0,
                                                   kStoreThrough);
        }
    };

    const int frag = jrow * ROWE + hh * 4;
    // NBLK bounds the steps; a work-group leaves after its own nreal (the same for all its
    // threads): a step costs 128 matrix instructions here, so the blocks of a position are
    // split evenly over the work-groups (gemm_stream_split) and none runs an idle step.
    int last = 0;
#pragma unroll
    for (int s = 0; s < NBLK; s++) {
        if (s >= nreal) break;
        last = s;
        if (s + D < NBLK) gload(s % D, s + D);
        if (s > 0) send_rows(s - 1);
        // the requests above stay above: left to itself the scheduler moves them down to the
        // LDS stores that consume them, and a step then ends in a wait for memory
        __builtin_amdgcn_sched_barrier(0);
        const float* S = smem + (s % 3) * STAGE + frag;
        float16v acc;
#pragma unroll
        for (int r = 0; r < 16; r++) acc[r] = 0.0f;
        // two fragment registers in turn: the read that refills one is issued behind the
        // four instructions that used it and has the other's four to arrive in
        static_assert(NK8 % 2 == 0, "fragments are read in pairs");
        float4v fa = *reinterpret_cast<const float4v*>(S);
        float4v fb = *reinterpret_cast<const float4v*>(S + 8);
#pragma unroll
        for (int j = 0; j < NK8; j += 2) {
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(u[j].x, fa.x, acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(u[j].y, fa.y, acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(u[j].z, fa.z, acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(u[j].w, fa.w, acc, 0, 0, 0);
            if (j + 2 < NK8) fa = *reinterpret_cast<const float4v*>(S + (j + 2) * 8);
            __builtin_amdgcn_sched_barrier(0);
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(u[j + 1].x, fb.x, acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(u[j + 1].y, fb.y, acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(u[j + 1].z, fb.z, acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(u[j + 1].w, fb.w, acc, 0, 0, 0);
            if (j + 3 < NK8) fb = *reinterpret_cast<const float4v*>(S + (j + 3) * 8);
            __builtin_amdgcn_sched_barrier(0);
        }
        if (s + 2 < NBLK) lstore((s + 2) % D, (s + 2) % 3);
        __syncthreads();   // every wavefront has sent the rows of the block before
        float* O = obuf + jrow * OROW + wave * 32 + hh * 8;
        *reinterpret_cast<float4v*>(O) = float4v{acc[0], acc[1], acc[2], acc[3]};
        *reinterpret_cast<float4v*>(O + 4) = float4v{acc[4], acc[5], acc[6], acc[7]};
        *reinterpret_cast<float4v*>(O + 16) = float4v{acc[8], acc[9], acc[10], acc[11]};
        *reinterpret_cast<float4v*>(O + 20) = float4v{acc[12], acc[13], acc[14], acc[15]};
        __syncthreads();
    }
    send_rows(last);
}

// Fragment-order copy of one layer's filters for the streaming kernels, built on the host
// in fp32 (fp16 nets convert on the device, convert_filters): src is the reference layout
// [36][C][F] (F fastest); dst is [36][Kp/32][Cp/16][64][8] for wino_gemm_stream_k
// (elem_bytes 2) and [36][Kp/32][Cp/8][64][4] for wino_gemm_stream32_k (elem_bytes 4), zero
// padded: a fragment is G consecutive input channels per lane, G = 16 / elem_bytes.
void build_stream_filters(const float* src, int C, int F, int Cp, int Kp, int elem_bytes,
                          float* dst) {
    const int G = 16 / elem_bytes;             // values per lane and fragment
    const int nfr = Cp / (2 * G), nwb = Kp / 32;
    for (int p = 0; p < kPos; p++)
        for (int wb = 0; wb < nwb; wb++)
            for (int fr = 0; fr < nfr; fr++)
                for (int l = 0; l < 64; l++) {
                    const int k = 32 * wb + gemm_stream_channel(l & 31);
                    for (int e = 0; e < G; e++) {
                        const int c = 2 * G * fr + G * (l >> 5) + e;
                        float v = 0.0f;
                        if (c < C && k < F) v = src[((size_t)p * C + c) * F + k];
                        dst[((((size_t)p * nwb + wb) * nfr + fr) * 64 + l) * G + e] = v;
                    }
                }
}

// fp32 -> storage type on the device (round to nearest even, as a host cast would): the
// filters of an fp16 net are laid out on the host in fp32 and converted here, which takes
// the conversion of 2 x 191 M values out of push_weights' host time for a 40 x 256 net.
__global__ __launch_bounds__(256) void convert_filters_k(const float* __restrict__ src,
                                                         half_t* __restrict__ dst, size_t n) {
    const size_t stride = (size_t)gridDim.x * 256;
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += stride)
        dst[i] = (half_t)src[i];
}

void convert_filters(const float* src, half_t* dst, size_t n, hipStream_t s) {
    const size_t blocks = (n + 255) / 256;
    hipLaunchKernelGGL(convert_filters_k, dim3((unsigned)(blocks < 2048 ? blocks : 2048)),
                       dim3(256), 0, s, src, dst, n);
}

// Blocks per work-group for T tile rows in the fp16 kernel: the fewest (a power of two up
// to kStreamBlocks) with which one round of work-groups covers the 256 compute units, so
// that a batch of 8 boards runs one block per work-group, 64 boards eight and 128 sixteen.
static int gemm_stream_blocks(int T, int Kp) {
    const int nblk = (T + 31) / 32;
    const int per_pos = 256 / (kPos * ((Kp + 255) / 256));   // work-groups per position in one round
    int nb = 1;
    while (nb < kStreamBlocks && (nblk + nb - 1) / nb > per_pos) nb *= 2;
    return nb;
}

// The fp32 kernel's split of a position's 32-row blocks over work-groups: as many work-groups per
// position as one round over the 256 compute units allows (7 at one column tile: 252
// work-groups), fewer when there are fewer blocks, more when a work-group would otherwise
// get more than kStreamBlocks.  A work-group takes floor or ceil of blocks / chunks and
// leaves after its own; the kernel is instantiated for the next power of two.
struct StreamSplit { int chunks, nb; };
static StreamSplit gemm_stream_split(int T, int Kp) {
    const int nblk = (T + 31) / 32;
    const int per_pos = 256 / (kPos * ((Kp + 255) / 256));
    int chunks = nblk < per_pos ? nblk : per_pos;
    const int least = (nblk + kStreamBlocks - 1) / kStreamBlocks;
    if (chunks < least) chunks = least;
    const int most = (nblk + chunks - 1) / chunks;   // blocks of the largest share
    int nb = 1;
    while (nb < most) nb *= 2;
    return {chunks, nb};
}

// Whether launch_gemm takes a streaming kernel for this shape when it is handed the
// fragment-order filters: input layer (64 padded planes) and tower layers, any batch, of nets
// of 128, 192 and 256 filters in both storage types (one column tile of Kp / 32 wavefronts;
// at 64 filters the tiled kernel is as fast: 3.0 against 3.5 us at 4 boards, 3.5 against 3.5 at
// 33).  fp32, tiled -> streaming: 256 filters 88 -> 79-83 us per launch at 64 boards, 78 -> 58 at
// 48, 22 -> 13 at 8; 128 filters 27 -> 23 at 64 boards.  At 192 filters in fp32 six wavefronts
// sit unevenly on four SIMDs: the streaming kernel is ahead up to 24 boards on one lane (15x192
// forwards +6 % at 1 board, +11 % at 8, +20 % at 16, +10 % at 24; all lanes +4 % at 8, +2 % at 16,
// -15 % at 24) and behind beyond (-4 % at 32, -8 % at 64): gemm_stream_prefers says which kernel
// family a handle of a given batch limit holds the filters for.  One family per handle keeps a
// position's result independent of the batch it is evaluated in.
bool gemm_stream_shape(int T, int Cp, int Kp, int elem_bytes) {
    (void)elem_bytes;
    if (T < 1 || !(Cp == 64 || Cp == Kp)) return false;
    return Kp == 128 || Kp == 256 || Kp == 192;
}
bool gemm_stream_prefers(int Kp, int elem_bytes, int max_batch) {
    return !(Kp == 192 && elem_bytes == 4 && max_batch > 16);
}

template <int NKC, int NW>
static void launch_gemm_stream_nkc(const half_t* V, const half_t* Uf, half_t* M, int T, int Tp,
                                   int Kp, hipStream_t s, LaunchTimer* t, int slab) {
    const int nblk = (T + 31) / 32;
    const int nb = gemm_stream_blocks(T, Kp);
    const int chunks = (nblk + nb - 1) / nb;
    const int tiles_n = Kp / (32 * NW);
    const int n_items = kPos * chunks * tiles_n;
    int seg = (n_items + 7) / 8;
    seg = (seg + tiles_n - 1) / tiles_n * tiles_n;
    const dim3 grid(8 * seg), block(64 * NW);
#define LZ_STREAM(NB, VS, MS)                                                                     \
    launch(wino_gemm_stream_k<NKC, NB, NW, VS, MS>, grid, block, s, t, V, Uf, M, T, Tp, Kp,      \
           chunks, nblk, tiles_n, seg)
    // slabs: the first layer reads its 64 input planes row by row (NKC == 4) and writes slabs;
    // the pairs (slab width, blocks per work-group) are those tile_slab hands out
    constexpr bool FIRST = NKC == 4;
    if (slab == 16) {
        switch (nb) {
            case 1: LZ_STREAM(1, FIRST ? 0 : 16, 16); return;
            case 2: LZ_STREAM(2, FIRST ? 0 : 16, 16); return;
            case 4: LZ_STREAM(4, FIRST ? 0 : 16, 16); return;
            default: break;
        }
    } else if (slab == 32) {
        switch (nb) {
            case 2: LZ_STREAM(2, FIRST ? 0 : 32, 32); return;
            case 4: LZ_STREAM(4, FIRST ? 0 : 32, 32); return;
            case 8: LZ_STREAM(8, FIRST ? 0 : 32, 32); return;
            default: break;
        }
    }
    if (slab != 0) throw std::invalid_argument("no slab-layout GEMM instantiated for this batch");
    switch (nb) {
        case 1: LZ_STREAM(1, 0, 0); break;
        case 2: LZ_STREAM(2, 0, 0); break;
        case 4: LZ_STREAM(4, 0, 0); break;
        case 8: LZ_STREAM(8, 0, 0); break;
        default: LZ_STREAM(16, 0, 0); break;
    }
#undef LZ_STREAM
}

// NW = Kp / 32 wavefronts per work-group; the first layer reads the 64 padded input planes.
template <int NW>
static void launch_gemm_stream_nw(const half_t* V, const half_t* Uf, half_t* M, int T, int Tp,
                                  int Cp, int Kp, hipStream_t s, LaunchTimer* t, int slab) {
    if (Cp == 64)
        launch_gemm_stream_nkc<4, NW>(V, Uf, M, T, Tp, Kp, s, t, slab);
    else
        launch_gemm_stream_nkc<2 * NW, NW>(V, Uf, M, T, Tp, Kp, s, t, slab);
}

static void launch_gemm_stream(const half_t* V, const half_t* Uf, half_t* M, int T, int Tp,
                               int Cp, int Kp, hipStream_t s, LaunchTimer* t, int slab) {
    switch (Kp) {
        case 256: launch_gemm_stream_nw<8>(V, Uf, M, T, Tp, Cp, Kp, s, t, slab); break;
        case 192: launch_gemm_stream_nw<6>(V, Uf, M, T, Tp, Cp, Kp, s, t, slab); break;
        default: launch_gemm_stream_nw<4>(V, Uf, M, T, Tp, Cp, Kp, s, t, slab); break;
    }
}

// The layout of the tile arrays for a forward of n boards: 0 = row by row, [36][Tp][Kp];
// 16 or 32 = slab by slab, [36][Kp / w][Tp][w], for the batches that take the transform
// shapes of that many channels per work-group (fp16 towers of 128, 192 and 256 filters).  A
// transform work-group (one board, w channels) then reads and writes its 25 tiles as one
// contiguous run of 25 w values per Winograd position instead of 25 pieces of 2 w bytes, and
// the GEMM reads and writes a slab's share of a 32-row block as one contiguous run: the same
// bytes in a quarter (an eighth) of the requests to the L2s.  Measured, transform alone at
// 256 filters, rows / slabs: 16 boards 7.0 / 6.0 us, 24 boards 9.2 (64-channel shape) / 7.3,
// 32 boards 9.3 / 7.8; from 40 boards the 64-channel shape (whole lines anyway) is level.
// Forwards, evaluations/s, rows -> slabs (best launch form each):
//   40x256 one lane: 1 board +6 %, 4 +10 %, 8 +9 %, 12 +8 %, 16 +10 %, 20 +2 %, 24 +3 %,
//          28 +6 %, 32 +6 %; three lanes: 12 +8 %, 16 +5 %, 20 +4 %, 24 -8 %, 28 -3 %, 32 -2 %
//   15x192 one lane: 1 to 4 +8 %, 8 +12 %, 16 +15 %, 21 +16 %, 26 +3 %, 32 +8 %, 42 0 %;
//          three lanes: 8 and 12 -3 %, 16 0 % (two lanes +13 %), 21 +11 %, 26 +14 %, 42 +4 %
//   10x128 one lane: 1 to 8 +3..6 %, 16 +10 %, 24 +8 %, 32 +15 %, 40 +4 %, 48 0 %, 64 -1 %;
//          three lanes: 16 -1 % (two lanes +9 %), 32 +2 %, 40 +8 %, 48 0 %, two lanes at 64 -5 %
// hence: every such batch at 192 filters, up to 44 boards at 128, and at 256 filters up to
// 20 boards, or up to 32 when the forward has the device to itself (`alone`).
int tile_slab(int n, int Kp, int elem_bytes, bool alone) {
    if (!xform_gemm_shape(n, Kp, elem_bytes)) return 0;
    if (Kp == 256 && n > 20 && !alone) return 0;
    if (Kp == 128 && n > 44) return 0;
    return n * (Kp / 64) <= 64 ? 16 : 32;
}

// Shapes served by the fused transform + GEMM launch: fp16 towers of 128, 192 and 256
// filters (the widths of the streaming GEMM) at batches that take the narrow transform
// shapes (up to 32 boards at 256 filters, 42 at 192, 64 at 128).
bool xform_gemm_shape(int n, int Kp, int elem_bytes) {
    return elem_bytes == 2 && (Kp == 128 || Kp == 192 || Kp == 256) && n >= 1 &&
           n * (Kp / 64) <= 128;
}

// Whether the fused launch is the faster way to run a forward of n boards whose tile arrays
// lie in slabs of `slab` channels (0: row by row), with the device to itself (`alone`) or
// shared with other lanes' forwards.  Measured (40x256 / 15x192 / 10x128, evaluations per
// second against separate launches):
//   alone, slabs: the launch pays where the transform's work-groups fill the device in one
//     round (n Kp / slab between 232 and 256), so that GEMM work-groups, which have fetched
//     their filters meanwhile, start as those retire instead of after a hand-over between
//     launches: 256 filters +3 % at 16 and 32 boards, 192 filters +4 % at 21 and +6 % at 42,
//     128 filters +5 % at 32; elsewhere -1..-10 % (256 filters: 8 to 12 boards -3..-6 %, 24
//     and 28 -4 %).  And at 256 filters up to 7 boards, where most of the device is free for
//     GEMM work-groups that fetch 128 KiB of filters each while the transform runs: +16 % at
//     1 board, +14 % at 2, +10 % at 3 and 4, +6 % at 5, +2 % at 6 (192 and 128 filters have a
//     half and a quarter of those bytes to hide: 0..-7 % up to 8 boards).
//   not alone, slabs: with few boards the device is mostly idle, and a lane's waiting GEMM
//     work-groups take nothing from the other lanes: three lanes, 256 filters +35 % at 3
//     boards, +19 % at 5, 0 % at 6, -17 % at 8; 192 filters +72 % at 1, +46 % at 2, +54 % at 4,
//     +12 % at 8, -10 % at 16; 128 filters +55 % at 1 to 4, +10 % at 8, -14 % at 16; two lanes
//     the same up to 4 or 5 boards (+7..37 %) and -1..-10 % at 8: taken up to 5 (256) or 6 boards.
//   rows (what is left of them: 128 filters from 45 boards, alone): +8 % at 48, +25 % at 64.
bool xform_gemm_pays(int n, int Kp, int slab, bool alone) {
    if (slab == 0) return alone && Kp == 128 && n >= 32;
    if (!alone) return n <= (Kp == 256 ? 5 : 6);
    const int groups = n * (Kp / slab);
    return (groups >= 232 && groups <= 256) || (Kp == 256 && n <= 7);
}

template <int CG, int NBLK, int NW, bool SLAB>
static void launch_xform_gemm_as(half_t* M, const half_t* res, half_t* act_out, half_t* V,
                                 const float* bn_scale, const float* bn_mean, float rfac, int n,
                                 int Kp, int Tp, const half_t* Uf, unsigned long long* flags,
                                 unsigned long long epoch, unsigned* gave_up, hipStream_t s) {
    const int T = n * kTilesPerBoard;
    const int nblk = (T + 31) / 32;
    const int chunks = (nblk + NBLK - 1) / NBLK;
    const int tiles_n = Kp / (32 * NW);
    const int seg = (kPos * chunks * tiles_n + 7) / 8;
    const unsigned n_xform_wg = 8u * (unsigned)((n * (Kp / CG) + 7) / 8);
    constexpr int WAVES = NW > fuse_waves(CG) ? NW : fuse_waves(CG);
    hipLaunchKernelGGL((xform_gemm_k<CG, NBLK, NW, SLAB>),
                       dim3(n_xform_wg + 8u * (unsigned)seg), dim3(64 * WAVES), 0, s, M, res,
                       act_out, V, bn_scale, bn_mean, rfac, n, Kp, Tp, Uf, T, chunks, nblk, tiles_n,
                       seg, n_xform_wg, flags, epoch, gave_up);
}

template <int NW>
static void launch_xform_gemm_nw(half_t* M, const half_t* res, half_t* act_out, half_t* V,
                                 const float* bn_scale, const float* bn_mean, float rfac, int n,
                                 int Kp, int Tp, const half_t* Uf, unsigned long long* flags,
                                 unsigned long long epoch, unsigned* gave_up, hipStream_t s,
                                 int slab) {
    const int nb = gemm_stream_blocks(n * kTilesPerBoard, Kp);
    const bool narrow = n * (Kp / 64) <= 64;     // 16-channel transform groups, else 32
#define LZ_FUSED(CG, NB, SLAB)                                                                  \
    launch_xform_gemm_as<CG, NB, NW, SLAB>(M, res, act_out, V, bn_scale, bn_mean, rfac, n, Kp,    \
                                           Tp, Uf, flags, epoch, gave_up, s)
    // the pairs that occur: 16-channel groups up to 64 / (Kp / 64) boards, i.e. up to 7, 14 or
    // (128 filters) 25 blocks of 32 rows per position; 32-channel groups up to twice that
    if (slab != 0) {   // both arrays slab by slab (they may be one)
        if (slab != (narrow ? 16 : 32))
            throw std::invalid_argument("fused launch: the slab width follows the batch");
        if (narrow && nb == 1) LZ_FUSED(16, 1, true);
        else if (narrow && nb == 2) LZ_FUSED(16, 2, true);
        else if (narrow && nb == 4) LZ_FUSED(16, 4, true);
        else if (!narrow && nb == 2) LZ_FUSED(32, 2, true);
        else if (!narrow && nb == 4) LZ_FUSED(32, 4, true);
        else if (!narrow && nb == 8) LZ_FUSED(32, 8, true);
        else throw std::invalid_argument("no fused launch instantiated for this batch");
        return;
    }
    if (V != M) throw std::invalid_argument("fused launch: row by row, V and M are one array");
    if (narrow && nb == 1) LZ_FUSED(16, 1, false);
    else if (narrow && nb == 2) LZ_FUSED(16, 2, false);
    else if (narrow && nb == 4) LZ_FUSED(16, 4, false);
    else if (!narrow && nb == 2) LZ_FUSED(32, 2, false);
    else if (!narrow && nb == 4) LZ_FUSED(32, 4, false);
    else if (!narrow && nb == 8) LZ_FUSED(32, 8, false);
    else throw std::invalid_argument("no fused launch instantiated for this batch");
#undef LZ_FUSED
}

// slab: 0 (V and M one array, row by row) or tile_slab's width (slab by slab; one array or two).
// flags: kFusedFlagsPerBoard words per board of the largest batch, zero before the first
// launch; epoch: a number no earlier launch on these flags has used (grows by one per launch).
void launch_xform_gemm(half_t* M, const half_t* res, half_t* act_out, half_t* V,
                       const float* bn_scale, const float* bn_mean, float rfac, int n, int Kp,
                       int Tp, const half_t* Uf, unsigned long long* flags,
                       unsigned long long epoch, unsigned* gave_up, hipStream_t s, int slab) {
    if (!xform_gemm_shape(n, Kp, 2)) throw std::invalid_argument("no fused launch for this shape");
    switch (Kp) {
        case 256: launch_xform_gemm_nw<8>(M, res, act_out, V, bn_scale, bn_mean, rfac, n, Kp, Tp, Uf, flags, epoch, gave_up, s, slab); break;
        case 192: launch_xform_gemm_nw<6>(M, res, act_out, V, bn_scale, bn_mean, rfac, n, Kp, Tp, Uf, flags, epoch, gave_up, s, slab); break;
        default: launch_xform_gemm_nw<4>(M, res, act_out, V, bn_scale, bn_mean, rfac, n, Kp, Tp, Uf, flags, epoch, gave_up, s, slab); break;
    }
}

template <int NK8, int NW>
static void launch_gemm_stream32_nk(const float* V, const float* Uf, float* M, int T, int Tp,
                                    int Kp, hipStream_t s, LaunchTimer* t) {
    const int nblk = (T + 31) / 32;
    const StreamSplit sp = gemm_stream_split(T, Kp);
    const int nb = sp.nb, chunks = sp.chunks;
    const int seg = (kPos * chunks + 7) / 8;
    const dim3 grid(8 * seg), block(64 * NW);
    switch (nb) {
        case 1: launch(wino_gemm_stream32_k<NK8, 1, NW>, grid, block, s, t, V, Uf, M, T, Tp, Kp, chunks, nblk, seg); break;
        case 2: launch(wino_gemm_stream32_k<NK8, 2, NW>, grid, block, s, t, V, Uf, M, T, Tp, Kp, chunks, nblk, seg); break;
        case 4: launch(wino_gemm_stream32_k<NK8, 4, NW>, grid, block, s, t, V, Uf, M, T, Tp, Kp, chunks, nblk, seg); break;
        case 8: launch(wino_gemm_stream32_k<NK8, 8, NW>, grid, block, s, t, V, Uf, M, T, Tp, Kp, chunks, nblk, seg); break;
        default: launch(wino_gemm_stream32_k<NK8, 16, NW>, grid, block, s, t, V, Uf, M, T, Tp, Kp, chunks, nblk, seg); break;
    }
}

template <int NW>
static void launch_gemm_stream32_nw(const float* V, const float* Uf, float* M, int T, int Tp,
                                    int Cp, int Kp, hipStream_t s, LaunchTimer* t) {
    if (Cp == 64)
        launch_gemm_stream32_nk<8, NW>(V, Uf, M, T, Tp, Kp, s, t);
    else
        launch_gemm_stream32_nk<4 * NW, NW>(V, Uf, M, T, Tp, Kp, s, t);
}

static void launch_gemm_stream(const float* V, const float* Uf, float* M, int T, int Tp, int Cp,
                               int Kp, hipStream_t s, LaunchTimer* t, int slab) {
    if (slab != 0) throw std::invalid_argument("the fp32 GEMM works row by row");
    if (Kp == 256)
        launch_gemm_stream32_nw<8>(V, Uf, M, T, Tp, Cp, Kp, s, t);
    else if (Kp == 192)
        launch_gemm_stream32_nw<6>(V, Uf, M, T, Tp, Cp, Kp, s, t);
    else
        launch_gemm_stream32_nw<4>(V, Uf, M, T, Tp, Cp, Kp, s, t);
}

template <typename P, int NK>
static void launch_gemm_big(const P* V, const P* U, P* M, int T, int tiles_m, int Tp, int Cp,
                            int Kp, hipStream_t s, LaunchTimer* t) {
    const int tiles_n = Kp / 256;
    const int n_items = kPos * tiles_m * tiles_n;
    int seg = (n_items + 7) / 8;
    seg = (seg + tiles_n - 1) / tiles_n * tiles_n;
    // Two 128-row passes wherever the k-pipeline has at least two slices to keep
    // the register stages busy across the pass boundary (measured 3 % faster than
    // one 256-row pass at 256 filters); the single-slice input layer keeps one pass,
    // and so do fp16 nets from 512 filters, where the GEMM is bound by the matrix and
    // LDS pipes and the 128 x 64 wave tile of the single pass reads less LDS per
    // instruction (measured 3 % faster at 512 filters, 6 % at 1024).
    if (NK >= 2 && !(sizeof(P) == 2 && NK >= 8))
        launch(wino_gemm_split_k<P, NK, 128>, dim3(8 * seg), dim3(512), s, t, V, U, M, T, Tp, Cp,
               Kp, tiles_m, tiles_n, seg);
    else
        launch(wino_gemm_big_k<P, NK>, dim3(8 * seg), dim3(512), s, t, V, U, M, T, Tp, Cp, Kp,
               tiles_m, tiles_n, seg);
}

// Channel counts (multiples of 64) for which a k-slice pipeline is instantiated:
// 1..8, 10, 12, 14 and 16 slices of 128 bytes.
template <typename P> bool gemm_supports_channels(int Cp) {
    constexpr int BK = 128 / (int)sizeof(P);
    if (Cp < 64 || Cp % 64 != 0) return false;
    const int nk = Cp / BK;
    return (nk >= 1 && nk <= 8) || nk == 10 || nk == 12 || nk == 14 || nk == 16;
}
template bool gemm_supports_channels<float>(int);
template bool gemm_supports_channels<half_t>(int);

// T = number of real tile rows (25 per board); Tp (the row count of V and M)
// must be a multiple of 256.
template <typename P>
void launch_gemm(const P* V, const P* U, const P* Uf, P* M, int T, int Tp, int Cp, int Kp,
                 hipStream_t s, LaunchTimer* t, int slab) {
    constexpr int BK = 128 / (int)sizeof(P);
    const int nk = Cp / BK;
    if (Uf != nullptr && gemm_stream_shape(T, Cp, Kp, (int)sizeof(P))) {
        launch_gemm_stream(V, Uf, M, T, Tp, Cp, Kp, s, t, slab);
        return;
    }
    if (slab != 0) throw std::invalid_argument("only the streaming GEMM works slab by slab");
    // The 256 x 256 tile pays off once its tiles can occupy most of the 256 compute units
    // (measured at 256 filters: from 6 row tiles = 216 work-groups, batch 52; with 5 = 180 the
    // 128 x 128 tiles are 2 % ahead; fp32 keeps the earlier hand-over at 160).
    const int big_rows = (T + 255) / 256;
    if (Kp % 256 == 0 && big_rows * (Kp / 256) * kPos >= (sizeof(P) == 2 ? 200 : 160)) {
        switch (nk) {
#define LZ_BIG(N) case N: launch_gemm_big<P, N>(V, U, M, T, big_rows, Tp, Cp, Kp, s, t); return;
            LZ_BIG(1) LZ_BIG(2) LZ_BIG(4) LZ_BIG(8) LZ_BIG(16)
#undef LZ_BIG
            default: break;
        }
    }
    const int tiles_m = (T + kGemmBM - 1) / kGemmBM;
    // Below the 256 x 256 tile, fp16: the 128 x 64 tile, three work-groups to a compute unit,
    // gives the chip the most independent pieces (measured at 256 filters: ahead of 128 x 128
    // tiles, two to a unit, at every batch up to 40, by 4 % at 21 and 1 % at 40); 128 x 128
    // tiles take over where that would be more than two rounds of the narrow ones.  fp32 (two
    // narrow work-groups to a unit): 128 x 128 once there are more than 320 of them.
    if (Kp % 128 == 0 && kPos * tiles_m * (Kp / 128) > (sizeof(P) == 2 ? 600 : 320))
        launch_gemm_bn<P, 128>(V, U, M, tiles_m, Tp, Cp, Kp, s, t);
    else
        launch_gemm_bn<P, 64>(V, U, M, tiles_m, Tp, Cp, Kp, s, t);
}

// ---------------------------------------------------------------------------
// 1x1 policy (2 planes) and value (1 plane) convolutions in one pass over the
// last activation (reference src/CPUPipe.cpp:424-427).  One wavefront per
// board point; lanes stride over channels, then a butterfly reduction.
template <typename P>
__global__ __launch_bounds__(256) void head_conv_k(const P* __restrict__ act,
                                                   const float* __restrict__ w3,
                                                   float out_scale, float* __restrict__ pol,
                                                   float* __restrict__ val, int n, int Cp) {
    const int gw = (blockIdx.x * 256 + threadIdx.x) >> 6;
    const int lane = threadIdx.x & 63;
    if (gw >= n * kPts) return;
    const int b = gw / kPts, pt = gw - b * kPts;
    const P* a = act + (size_t)gw * Cp;
    float s0 = 0.0f, s1 = 0.0f, s2 = 0.0f;
    for (int c = lane; c < Cp; c += 64) {
        const float x = (float)a[c];
        s0 += x * w3[c];
        s1 += x * w3[Cp + c];
        s2 += x * w3[2 * Cp + c];
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        s0 += __shfl_xor(s0, off);
        s1 += __shfl_xor(s1, off);
        s2 += __shfl_xor(s2, off);
    }
    if (lane == 0) {
        pol[(size_t)b * 2 * kPts + pt] = s0 * out_scale;
        pol[(size_t)b * 2 * kPts + kPts + pt] = s1 * out_scale;
        val[(size_t)b * kPts + pt] = s2 * out_scale;
    }
}

template <typename P>
void launch_head_conv(const P* act, const float* w3, float out_scale, float* pol, float* val,
                      int n, int Cp, hipStream_t s, LaunchTimer* t) {
    const int waves = n * kPts;
    launch(head_conv_k<P>, dim3((waves + 3) / 4), dim3(256), s, t, act, w3, out_scale, pol, val,
           n, Cp);
}

// ---------------------------------------------------------------------------
template <typename P>
__global__ __launch_bounds__(256) void absmax_k(const P* __restrict__ x, size_t count,
                                                float* out) {
    float m = 0.0f;
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < count;
         i += (size_t)gridDim.x * 256) {
        const float v = fabsf((float)x[i]);
        // NaN-propagating max so that a poisoned buffer is visible to the host.
        m = (v != v) ? INFINITY : fmaxf(m, v);
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) m = fmaxf(m, __shfl_xor(m, off));
    if ((threadIdx.x & 63) == 0) atomicMax(reinterpret_cast<int*>(out), __float_as_int(m));
}

template <typename P>
void launch_absmax(const P* x, size_t count, float* out, hipStream_t s) {
    size_t blocks = (count + 255) / 256;
    if (blocks > 2048) blocks = 2048;
    if (blocks == 0) blocks = 1;
    hipLaunchKernelGGL(absmax_k<P>, dim3((unsigned)blocks), dim3(256), 0, s, x, count, out);
}

// ---------------------------------------------------------------------------
// Head arithmetic above the pipe boundary (reference src/Network.cpp:833-851):
// policy: BN+ReLU on 2 planes -> FC 722->362 -> softmax(./temperature)
// value : BN+ReLU on 1 plane  -> FC 361->256 + ReLU -> FC 256->1 -> tanh
// One workgroup of 256 threads per position; FC rows are read by whole
// wavefronts (coalesced) and reduced with a butterfly.
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off);
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off));
    return v;
}

// The two large fully connected layers -- policy 722 -> 362 and value 361 -> 256 -- are
// matrix products over the batch, [n x K] . [K x N], and run on the matrix cores in fp32
// (v_mfma_f32_32x32x2_f32: fp32 operands, fp32 accumulate).  One work-group computes a
// 32-position x 32-output tile: the 32 input rows (batch norm and ReLU applied on the way)
// are staged in LDS once, the four wavefronts split the contraction index four ways, and
// their partial tiles meet in LDS.  The weights are held in the operand order of the
// instruction (head_fc_fragments): lane l of k-step s supplies W^T[2s + l/32][32 cb + l%32],
// four consecutive steps per 16-byte load, so a wavefront's load is one contiguous KiB.
// A second, small kernel finishes: softmax over the 362 logits, and FC 256 -> 1 + tanh.
constexpr int kHeadStepsPol = 92;   // k-steps (of 2) per wavefront: 4 * 92 * 2 = 736 >= 722
constexpr int kHeadStepsVal = 48;   // 4 * 48 * 2 = 384 >= 361
constexpr int kHeadColsPol = 12;    // 32-wide output blocks: 384 >= 362
constexpr int kHeadColsVal = 8;     // 256
constexpr int kHeadKPad = 4 * kHeadStepsPol * 2;   // staged row length of the wider layer

size_t head_fc_fragment_count(bool policy) {
    return (size_t)(policy ? kHeadColsPol * kHeadStepsPol : kHeadColsVal * kHeadStepsVal) * 4 *
           64;
}

// W [N][K] row-major (as the network facade holds it) -> fragment order
// [col block][wavefront 4][steps/4][lane 64][4 consecutive steps], zero padded.
void head_fc_fragments(const float* W, bool policy, float* dst) {
    const int K = policy ? 2 * kPts : kPts, N = policy ? 362 : 256;
    const int steps = policy ? kHeadStepsPol : kHeadStepsVal;
    const int cols = policy ? kHeadColsPol : kHeadColsVal;
    for (int cb = 0; cb < cols; cb++)
        for (int q = 0; q < 4; q++)
            for (int g = 0; g < steps / 4; g++)
                for (int l = 0; l < 64; l++)
                    for (int e = 0; e < 4; e++) {
                        const int step = q * steps + g * 4 + e;
                        const int k = 2 * step + (l >> 5), j = cb * 32 + (l & 31);
                        const float v = (k < K && j < N) ? W[(size_t)j * K + k] : 0.0f;
                        dst[((((size_t)cb * 4 + q) * (steps / 4) + g) * 64 + l) * 4 + e] = v;
                    }
}

// One layer's share of heads_fc_k.  Everything a work-group reads has been out of the caches
// since the last call (a tower of 81 layers ran in between) and the planes have just been
// written on other dies, so a round trip to memory takes ~2 us here: the wavefront's whole
// share of the weights (23 or 12 KiB) and, per thread, its 92 or 48 values of the planes are
// requested before the first is used.
template <bool POL>
__device__ __forceinline__ void heads_fc_body(float* xs, const float* __restrict__ src,
                                              const HeadParams& hp, float* __restrict__ out,
                                              int cb, int r0, int n) {
    constexpr int STEPS = POL ? kHeadStepsPol : kHeadStepsVal;
    constexpr int G = STEPS / 4;             // 16-byte weight loads per lane
    constexpr int KP = 4 * STEPS * 2;        // padded contraction length
    constexpr int KK = POL ? 2 * kPts : kPts;
    constexpr int N = POL ? 362 : 256;
    constexpr int ROW = kHeadKPad + 1;       // odd row length: conflict-free column reads
    const int tid = threadIdx.x, lane = tid & 63;
    const int q = __builtin_amdgcn_readfirstlane(tid >> 6);

    const float4v* wf = reinterpret_cast<const float4v*>(POL ? hp.ip_pol_wf : hp.ip1_val_wf) +
                        (((size_t)cb * 4 + q) * G) * 64 + lane;
    float4v w[G];
#pragma unroll
    for (int g = 0; g < G; g++) w[g] = wf[(size_t)g * 64];

    // 32 rows of the layer's input: batch norm + ReLU of the raw head planes, zero padded
    const float s0 = POL ? hp.bn_pol_scale[0] : hp.bn_val_scale[0];
    const float m0 = POL ? hp.bn_pol_mean[0] : hp.bn_val_mean[0];
    const float s1 = POL ? hp.bn_pol_scale[1] : s0;
    const float m1 = POL ? hp.bn_pol_mean[1] : m0;
    constexpr int U = KP / 8;                // 32 * KP values on 256 threads: all in one go
    for (int i0 = tid; i0 < 32 * KP; i0 += 256 * U) {
        float x[U];
#pragma unroll
        for (int u = 0; u < U; u++) {
            const int i = i0 + u * 256;
            const int r = i / KP, k = i - r * KP;
            x[u] = (i < 32 * KP && r0 + r < n && k < KK) ? src[(size_t)(r0 + r) * KK + k] : 0.0f;
        }
#pragma unroll
        for (int u = 0; u < U; u++) {
            const int i = i0 + u * 256;
            const int r = i / KP, k = i - r * KP;
            const bool second = POL && k >= kPts;
            float y = 0.0f;
            if (r0 + r < n && k < KK)
                y = fmaxf(0.0f, (second ? s1 : s0) * (x[u] - (second ? m1 : m0)));
            if (i < 32 * KP) xs[r * ROW + k] = y;
        }
    }
    __syncthreads();

    float16v acc;
#pragma unroll
    for (int r = 0; r < 16; r++) acc[r] = 0.0f;
    const float* xa = xs + (lane & 31) * ROW + q * STEPS * 2 + (lane >> 5);
#pragma unroll
    for (int g = 0; g < G; g++) {
        const float* x = xa + g * 8;
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(x[0], w[g].x, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(x[2], w[g].y, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(x[4], w[g].z, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(x[6], w[g].w, acc, 0, 0, 0);
    }
    __syncthreads();   // everyone is done with the staged rows: reuse them for the partial tiles

    // register r of lane l holds row 8(r/4) + 4(l/32) + r%4, column l%32
    float* red = xs + q * (32 * 33);
#pragma unroll
    for (int r = 0; r < 16; r++)
        red[(8 * (r >> 2) + 4 * (lane >> 5) + (r & 3)) * 33 + (lane & 31)] = acc[r];
    __syncthreads();
    const float* bias = POL ? hp.ip_pol_b : hp.ip1_val_b;
    for (int i = tid; i < 32 * 32; i += 256) {
        const int r = i >> 5, j = i & 31;
        const int col = cb * 32 + j;
        if (r0 + r < n && col < N) {
            const float v = xs[r * 33 + j] + xs[32 * 33 + r * 33 + j] +
                            xs[2 * 32 * 33 + r * 33 + j] + xs[3 * 32 * 33 + r * 33 + j];
            out[(size_t)(r0 + r) * N + col] = POL ? v + bias[col] : fmaxf(0.0f, v + bias[col]);
        }
    }
}

__global__ __launch_bounds__(256) void heads_fc_k(const float* __restrict__ pol,
                                                  const float* __restrict__ val, HeadParams hp,
                                                  float* __restrict__ logits,
                                                  float* __restrict__ hidden, int n) {
    __shared__ float xs[32 * (kHeadKPad + 1)];
    const int tasks = kHeadColsPol + kHeadColsVal;
    const int rb = blockIdx.x / tasks, task = blockIdx.x - rb * tasks;
    if (task < kHeadColsPol)
        heads_fc_body<true>(xs, pol, hp, logits, task, rb * 32, n);
    else
        heads_fc_body<false>(xs, val, hp, hidden, task - kHeadColsPol, rb * 32, n);
}

// One wavefront per position: softmax over the logits at `temperature`, and the value
// head's second layer + tanh (reference src/Network.cpp:693-712, :846-851).
__global__ __launch_bounds__(256) void heads_finish_k(const float* __restrict__ logits_in,
                                                      const float* __restrict__ hidden,
                                                      HeadParams hp, float temperature,
                                                      float* __restrict__ policy,
                                                      float* __restrict__ logits_out,
                                                      float* __restrict__ value, int n) {
    const int pos = blockIdx.x * 4 + (threadIdx.x >> 6);
    const int lane = threadIdx.x & 63;
    if (pos >= n) return;
    float l[6], m = -INFINITY;
#pragma unroll
    for (int qq = 0; qq < 6; qq++) {
        const int i = lane + 64 * qq;
        l[qq] = i < 362 ? logits_in[(size_t)pos * 362 + i] : -INFINITY;
        m = fmaxf(m, l[qq]);
    }
    m = wave_max(m);
    float e[6], s = 0.0f;
#pragma unroll
    for (int qq = 0; qq < 6; qq++) {
        e[qq] = lane + 64 * qq < 362 ? expf((l[qq] - m) / temperature) : 0.0f;
        s += e[qq];
    }
    s = wave_sum(s);
#pragma unroll
    for (int qq = 0; qq < 6; qq++) {
        const int i = lane + 64 * qq;
        if (i < 362) {
            policy[(size_t)pos * 362 + i] = e[qq] / s;
            if (logits_out != nullptr) logits_out[(size_t)pos * 362 + i] = l[qq];
        }
    }
    float acc = 0.0f;
    for (int i = lane; i < 256; i += 64) acc += hidden[(size_t)pos * 256 + i] * hp.ip2_val_w[i];
    acc = wave_sum(acc);
    if (lane == 0) value[pos] = tanhf(hp.ip2_val_b[0] + acc);
}

void launch_heads(const float* pol, const float* val, HeadParams hp, float temperature,
                  float* policy, float* logits, float* value, float* work, int n,
                  hipStream_t s) {
    // work: [n][362] logits followed by [n][256] hidden units
    float* wl = work;
    float* wh = work + (size_t)n * 362;
    const int rbs = (n + 31) / 32;
    hipLaunchKernelGGL(heads_fc_k, dim3(rbs * (kHeadColsPol + kHeadColsVal)), dim3(256), 0, s, pol,
                       val, hp, wl, wh, n);
    hipLaunchKernelGGL(heads_finish_k, dim3((n + 3) / 4), dim3(256), 0, s, wl, wh, hp, temperature,
                       policy, logits, value, n);
}

// ---------------------------------------------------------------------------
#define INSTANTIATE(P)                                                                         \
    template void launch_pack_input<P>(const float*, P*, int, int, int, hipStream_t,           \
                                       LaunchTimer*);                                          \
    template void launch_pack_input_bits<P>(const uint32_t*, P*, int, int, int, hipStream_t,   \
                                            LaunchTimer*);                                     \
    template void launch_in_transform<P>(const P*, P*, int, int, int, hipStream_t,             \
                                         LaunchTimer*);                                        \
    template void launch_gemm<P>(const P*, const P*, const P*, P*, int, int, int, int,         \
                                 hipStream_t, LaunchTimer*, int);                              \
    template void launch_out_transform<P>(const P*, const P*, P*, const float*, const float*,  \
                                          float, int, int, int, hipStream_t, LaunchTimer*,     \
                                          int);                                                \
    template void launch_out_in_transform<P>(const P*, const P*, P*, P*, const float*,         \
                                             const float*, float, int, int, int, hipStream_t,  \
                                             LaunchTimer*, int);                               \
    template void launch_head_conv<P>(const P*, const float*, float, float*, float*, int, int, \
                                      hipStream_t, LaunchTimer*);                              \
    template void launch_absmax<P>(const P*, size_t, float*, hipStream_t);
INSTANTIATE(float)
INSTANTIATE(half_t)

}  // namespace lzhip
