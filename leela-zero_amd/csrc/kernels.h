// Launch interface of the gfx950 kernels of the residual tower.
//
// Device data layouts (P = storage type: float or _Float16):
//   act  [n][361][Cp]        activations, channels fastest ("channels-last")
//   V    [36][Tp][Cp]        Winograd-domain input tiles, t = board*25 + by*5 + bx
//   U    [36][Kp][Cp]        Winograd-domain filters, input channel fastest
//   M    [36][Tp][Kp]        per-position GEMM results, output channel fastest
// Cp, Kp are the channel counts padded to a multiple of 64, Tp the tile count
// padded to a multiple of 256.  The contraction index (input channel) is the
// fastest-moving one of both GEMM operands, which is what the MFMA operand
// registers want: each lane fetches 16 contiguous bytes of one row.
#pragma once
#include <hip/hip_runtime.h>
#include <cstdint>

namespace lzhip {

constexpr int kBoard = 19;
constexpr int kPts = 361;
constexpr int kTilesPerBoard = 25;
constexpr int kPos = 36;       // 6x6 Winograd positions
constexpr int kInPlanes = 18;
constexpr int kGemmBM = 128;   // row extent of the standard GEMM tile
constexpr int kTileRowPad = 256;  // V and M row counts (Tp) are multiples of this
// Largest magnitude an activation is stored with in half precision (see act_clamp in
// kernels.hip); the calibration treats a measured maximum at this value as saturated.
constexpr float kActStoreMax = 2040.0f;

// Timing hook: when non-null every launch is bracketed by this event pair
// (device begin/end timestamps of that launch alone).
struct LaunchTimer {
    hipEvent_t start = nullptr, stop = nullptr;
};

// NCHW fp32 planes [n][C][361] -> act [n][361][Cp] (channels >= C zero).
// 32-bit words of one position's 18 x 361 input planes packed one bit per value.
constexpr int kInputWords = (18 * 361 + 31) / 32;

template <typename P>
void launch_pack_input_bits(const uint32_t* bits, P* act, int n, int C, int Cp, hipStream_t s,
                            LaunchTimer* t);
template <typename P>
void launch_pack_input(const float* in, P* act, int n, int C, int Cp, hipStream_t s,
                       LaunchTimer* t);

// act [n][361][Cp] -> V [36][Tp][Cp]
template <typename P>
void launch_in_transform(const P* act, P* V, int n, int Cp, int Tp, hipStream_t s,
                         LaunchTimer* t);

// Whether a GEMM pipeline exists for Cp channels (padded count, multiple of 64).
template <typename P> bool gemm_supports_channels(int Cp);

// M[p][t][k] = sum_c V[p][t][c] * U[p][k][c]
// T = real tile rows (25 per board); Tp = allocated rows, a multiple of kTileRowPad.
// Uf: the same filters in the fragment order of the streaming kernels (see
// build_stream_filters), or null; taken when gemm_stream_shape(T, Cp, Kp, sizeof(P)).
// slab (0, or tile_slab's 16 / 32; streaming shapes only): M is written slab by slab,
// [36][Kp / slab][Tp][slab], and V read that way too unless it is the first layer's (Cp == 64).
template <typename P>
void launch_gemm(const P* V, const P* U, const P* Uf, P* M, int T, int Tp, int Cp, int Kp,
                 hipStream_t s, LaunchTimer* t, int slab = 0);
bool gemm_stream_shape(int T, int Cp, int Kp, int elem_bytes);
// Whether a handle for batches up to max_batch should hold the streaming kernels' filters
// where gemm_stream_shape allows them (measured; see there).
bool gemm_stream_prefers(int Kp, int elem_bytes, int max_batch);
// Layout of the tile arrays that suits a forward of n boards: 0 row by row, else the slab width.
int tile_slab(int n, int Kp, int elem_bytes, bool alone);
// src [36][C][F] fp32 (F fastest) -> dst in the operand order of the streaming kernel for
// elements of elem_bytes (2: [36][Kp/32][Cp/16][64][8], 4: [36][Kp/32][Cp/8][64][4]), values
// in fp32, zero padded; convert_filters turns such an array into fp16 on the device.
void build_stream_filters(const float* src, int C, int F, int Cp, int Kp, int elem_bytes,
                          float* dst);
void convert_filters(const float* src, _Float16* dst, size_t n, hipStream_t s);

// M [36][Tp][Kp] (slab > 0: [36][Kp / slab][Tp][slab]) -> out [n][361][Kp]:
// max(0, scale*(A^T m A - mean) + rfac*res)
template <typename P>
void launch_out_transform(const P* M, const P* res, P* out, const float* bn_scale,
                          const float* bn_mean, float rfac, int n, int Kp, int Tp,
                          hipStream_t s, LaunchTimer* t, int slab = 0);

// Output transform of one layer fused with the input transform of the next:
// M [36][Tp][Kp] -> V_next [36][Tp][Kp]; the activation [n][361][Kp] is also
// written to act_out unless that is null.  Needs Kp to be a multiple of 64.  slab (0, 16 or
// 32): both tile arrays lie slab by slab and a work-group takes `slab` channels.
template <typename P>
void launch_out_in_transform(const P* M, const P* res, P* act_out, P* Vn, const float* bn_scale,
                             const float* bn_mean, float rfac, int n, int Kp, int Tp,
                             hipStream_t s, LaunchTimer* t, int slab = 0);

// launch_out_in_transform of one layer and launch_gemm of the next (filters Uf, in the
// streaming kernel's order) as one launch, for the shapes xform_gemm_shape accepts (fp16;
// 256 filters up to 32 boards, 192 up to 42, 128 up to 64).  M is read by the transform and
// rewritten by the GEMM; V is M (row by row: slab = 0) or M or a second array (slab by slab).
// flags: kFusedFlagsPerBoard 64-bit words per board (zero before the first launch); epoch: a
// value no earlier launch on these flags used; *gave_up is set to 1 if a wait inside the
// launch ran into its limit (the results are then invalid).
constexpr int kFusedFlagsPerBoard = 16;
bool xform_gemm_shape(int n, int Kp, int elem_bytes);
// Whether the fused launch is the faster way (measured) for a forward of n boards with the tile
// arrays in slabs of `slab` channels (0: rows) that has the device to itself or not.
bool xform_gemm_pays(int n, int Kp, int slab, bool alone);
void launch_xform_gemm(_Float16* M, const _Float16* res, _Float16* act_out, _Float16* V,
                       const float* bn_scale, const float* bn_mean, float rfac, int n, int Kp,
                       int Tp, const _Float16* Uf, unsigned long long* flags,
                       unsigned long long epoch, unsigned* gave_up, hipStream_t s, int slab = 0);

// 1x1 head convolutions: act [n][361][Cp] x w[3][Cp] -> pol [n][2][361], val [n][361],
// both multiplied by out_scale.
template <typename P>
void launch_head_conv(const P* act, const float* w3, float out_scale, float* pol, float* val,
                      int n, int Cp, hipStream_t s, LaunchTimer* t);

// max |x| over count elements -> *out (float, must be zeroed before).
template <typename P>
void launch_absmax(const P* x, size_t count, float* out, hipStream_t s);

// Head arithmetic above the pipe boundary: BN + ReLU, the two large fully connected layers
// on the matrix cores, softmax / FC + tanh.  Device pointers; the two large FC matrices are
// held in the operand order of the matrix instruction (head_fc_fragments).
struct HeadParams {
    const float *bn_pol_mean, *bn_pol_scale, *ip_pol_wf, *ip_pol_b;
    const float *bn_val_mean, *bn_val_scale, *ip1_val_wf, *ip1_val_b, *ip2_val_w, *ip2_val_b;
};
// Element count of the fragment-order copy of the policy (true) / value (false) matrix, and
// its construction from W [outputs][inputs] row-major.
size_t head_fc_fragment_count(bool policy);
void head_fc_fragments(const float* W, bool policy, float* dst);
// work: device scratch of n * (362 + 256) floats (logits and hidden units between the two
// kernels).  logits may be null.
void launch_heads(const float* pol, const float* val, HeadParams hp, float temperature,
                  float* policy, float* logits, float* value, float* work, int n,
                  hipStream_t s);

}  // namespace lzhip
