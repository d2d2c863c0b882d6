// A short causal convolution over time on each channel of the rows a sublayer reads:
//   out_t = x_t + sum_{j < taps} w[:, j] * x_{t - taps + 1 + j},  zeros before a request's start.
// x: the 32-bit rows of the step, a request's tokens in order. A source position inside the step's
// portion is read from the step's own rows; an earlier one from the request's history, `state`
// [slots, taps - 1, d] float32 with position p at ring place p % (taps - 1) (written by whoever
// updates the rows afterwards: liyab_gated_norm_add, or liyab_keep_rows). The sum is 32-bit and
// rounded once to the output type; `cast_out`, when given, gets x_t itself rounded the same way.
// Rows behind the step's tokens (padding: position 0 of the first request) read nothing of any
// history.
#include "common.h"
#include "launchers.h"

namespace liyab {

constexpr int kMaxTaps = 16;

typedef __attribute__((ext_vector_type(4))) float conv_f32x4;
__device__ __forceinline__ void conv_store4(float* dst, const conv_f32x4& v) { *reinterpret_cast<conv_f32x4*>(dst) = v; }
__device__ __forceinline__ void conv_store4(bf16_t* dst, const conv_f32x4& v) {
    uint2 packed;
    packed.x = static_cast<uint32_t>(float_to_bf16(v[0])) | (static_cast<uint32_t>(float_to_bf16(v[1])) << 16);
    packed.y = static_cast<uint32_t>(float_to_bf16(v[2])) | (static_cast<uint32_t>(float_to_bf16(v[3])) << 16);
    *reinterpret_cast<uint2*>(dst) = packed;
}

// VEC: four channels a thread; MAXT: the most taps this instance takes (its earlier inputs are loaded together)
template <typename T, bool VEC, int MAXT>
__global__ void __launch_bounds__(256)
causal_conv_kernel(T* __restrict__ out, T* __restrict__ cast_out, const float* __restrict__ x, const float* __restrict__ w, int taps,
                   const float* __restrict__ state, int n_slots, const int* __restrict__ tok_seq, const int* __restrict__ positions,
                   const int* __restrict__ seq_starts, const int* __restrict__ state_slots, int d) {
    const int t = blockIdx.x;
    const int s = tok_seq[t], p = positions[t];
    const int in_step = t - seq_starts[s];  // this token's place in its request's portion
    const int ring = taps - 1;
    int slot = state_slots[s];
    if (slot < 0 || slot >= n_slots) slot = -1;
    // where each earlier input comes from: a row of the step, a place of the ring, or nowhere
    const float* src[kMaxTaps];
#pragma unroll
    for (int m = 1; m < kMaxTaps; ++m) {
        src[m] = nullptr;
        if (m <= ring && p - m >= 0) {
            if (m <= in_step)
                src[m] = x + static_cast<int64_t>(t - m) * d;
            else if (state != nullptr && slot >= 0)
                src[m] = state + (static_cast<int64_t>(slot) * ring + (p - m) % ring) * d;
        }
    }
    const float* xr = x + static_cast<int64_t>(t) * d;
    if constexpr (VEC) {
        // Four channels a thread, 16 bytes a load (d a multiple of 4). Every earlier input is asked for before
        // any is used, in straight-line code (a load under a branch is waited for where the branch ends, three
        // trips to memory one after the other): one that does not exist reads this token's own row and counts
        // as nothing.
        typedef __attribute__((ext_vector_type(4))) float f32x4;
        for (int c = (blockIdx.y * 256 + threadIdx.x) * 4; c < d; c += gridDim.y * 1024) {
            const f32x4 xt = *reinterpret_cast<const f32x4*>(xr + c);
            const float* wc = w + static_cast<int64_t>(c) * taps;  // the taps of channels c .. c + 3, one after the other
            f32x4 xm[MAXT - 1];
            bool there[MAXT - 1];
#pragma unroll
            for (int m = 1; m < MAXT; ++m) {
                there[m - 1] = m <= ring && src[m] != nullptr;
                xm[m - 1] = *reinterpret_cast<const f32x4*>((there[m - 1] ? src[m] : xr) + c);
            }
            f32x4 acc;
#pragma unroll
            for (int e = 0; e < 4; ++e) acc[e] = wc[e * taps + taps - 1] * xt[e];
#pragma unroll
            for (int m = 1; m < MAXT; ++m)
#pragma unroll
                for (int e = 0; e < 4; ++e) acc[e] += there[m - 1] ? wc[e * taps + max(taps - 1 - m, 0)] * xm[m - 1][e] : 0.0f;
            f32x4 sum;
#pragma unroll
            for (int e = 0; e < 4; ++e) sum[e] = xt[e] + acc[e];
            conv_store4(out + static_cast<int64_t>(t) * d + c, sum);
            if (cast_out != nullptr) conv_store4(cast_out + static_cast<int64_t>(t) * d + c, xt);
        }
        return;
    }
    for (int c = blockIdx.y * 256 + threadIdx.x; c < d; c += gridDim.y * 256) {
        const float* wc = w + static_cast<int64_t>(c) * taps;
        const float xt = xr[c];
        float acc = wc[taps - 1] * xt;
#pragma unroll
        for (int m = 1; m < kMaxTaps; ++m)
            if (m <= ring && src[m] != nullptr) acc += wc[taps - 1 - m] * src[m][c];
        out[static_cast<int64_t>(t) * d + c] = from_float<T>(xt + acc);
        if (cast_out != nullptr) cast_out[static_cast<int64_t>(t) * d + c] = from_float<T>(xt);
    }
}

__global__ void __launch_bounds__(256)
keep_rows_kernel(float* __restrict__ state, int ring, int n_slots, const float* __restrict__ x, const int* __restrict__ tok_seq,
                 const int* __restrict__ positions, const int* __restrict__ context_lens, const int* __restrict__ state_slots,
                 const int* __restrict__ n_real, int d) {
    const int t = blockIdx.x;
    if (t >= *n_real) return;
    const int s = tok_seq[t], p = positions[t], slot = state_slots[s];
    if (p < context_lens[s] - ring || slot < 0 || slot >= n_slots) return;
    float* dst = state + (static_cast<int64_t>(slot) * ring + p % ring) * d;
    const float* xr = x + static_cast<int64_t>(t) * d;
    for (int i = threadIdx.x; i < d; i += 256) dst[i] = xr[i];
}

}  // namespace liyab

using namespace liyab;

extern "C" int liyab_causal_conv(void* out, void* cast_out, int dtype, const float* x, const float* w, int taps, const float* state,
                                 int n_slots, const int* tok_seq, const int* positions, const int* seq_starts, const int* state_slots,
                                 int n, int d, hipStream_t stream) {
    LIYAB_REQUIRE(out && x && w && tok_seq && positions && seq_starts && state_slots, "causal_conv: null pointer");
    LIYAB_REQUIRE(n >= 0 && d > 0, "causal_conv: bad sizes n=%d d=%d", n, d);
    LIYAB_REQUIRE(taps >= 1 && taps <= kMaxTaps, "causal_conv: %d taps; 1 to %d are taken", taps, kMaxTaps);
    LIYAB_REQUIRE(taps == 1 || (state != nullptr && n_slots > 0), "causal_conv: %d taps need the requests' history", taps);
    LIYAB_REQUIRE(dtype == kF32 || dtype == kBF16, "causal_conv: unknown dtype %d", dtype);
    if (n == 0) return 0;
    const bool vec = d % 4 == 0 && (reinterpret_cast<uintptr_t>(x) & 15) == 0 && (reinterpret_cast<uintptr_t>(out) & 15) == 0 &&
                     (cast_out == nullptr || (reinterpret_cast<uintptr_t>(cast_out) & 15) == 0) && (state == nullptr || (reinterpret_cast<uintptr_t>(state) & 15) == 0);
    const dim3 grid(n, vec ? std::min((d + 1023) / 1024, 16) : std::min((d + 255) / 256, 64));
#define LIYAB_CONV(T, V, MAXT)                                                                                                                  \
    causal_conv_kernel<T, V, MAXT><<<grid, 256, 0, stream>>>(static_cast<T*>(out), static_cast<T*>(cast_out), x, w, taps, state, n_slots, tok_seq, \
                                                             positions, seq_starts, state_slots, d)
    if (dtype == kF32) {
        if (!vec) LIYAB_CONV(float, false, kMaxTaps);
        else if (taps <= 4) LIYAB_CONV(float, true, 4);
        else LIYAB_CONV(float, true, kMaxTaps);
    } else {
        if (!vec) LIYAB_CONV(bf16_t, false, kMaxTaps);
        else if (taps <= 4) LIYAB_CONV(bf16_t, true, 4);
        else LIYAB_CONV(bf16_t, true, kMaxTaps);
    }
#undef LIYAB_CONV
    return check_launch("causal_conv");
}

// The step's rows that a later step's convolution reads (the last `ring` of each request) go to
// the requests' history, for callers whose row update does not keep them itself.
extern "C" int liyab_keep_rows(float* state, int ring, int n_slots, const float* x, const int* tok_seq, const int* positions,
                               const int* context_lens, const int* state_slots, const int* n_real, int n, int d, hipStream_t stream) {
    LIYAB_REQUIRE(state && x && tok_seq && positions && context_lens && state_slots && n_real, "keep_rows: null pointer");
    LIYAB_REQUIRE(n >= 0 && d > 0 && ring > 0 && n_slots > 0, "keep_rows: bad sizes");
    if (n == 0) return 0;
    keep_rows_kernel<<<n, 256, 0, stream>>>(state, ring, n_slots, x, tok_seq, positions, context_lens, state_slots, n_real, d);
    return check_launch("keep_rows");
}
