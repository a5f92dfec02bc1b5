// Shared device/host helpers for libmuon_amd (gfx950 only).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>

#include "../../include/muon_amd.h"

namespace muon_amd {

// ---- error reporting -------------------------------------------------------------------
void set_error(const char* fmt, ...);

#define MUON_REQUIRE(cond, ...)                      \
    do {                                             \
        if (!(cond)) {                               \
            ::muon_amd::set_error(__VA_ARGS__);      \
            return MUON_AMD_EINVAL;                  \
        }                                            \
    } while (0)

// Checks the launch that was just enqueued.
int check_launch(const char* what);

// ---- bf16 <-> fp32 -----------------------------------------------------------------------
// bf16 values are carried as uint16_t (upper half of the fp32 pattern).  The fp32 -> bf16
// conversion is round-to-nearest-even with NaN preserved (v_cvt_pk_bf16_f32 on gfx950).
__device__ __forceinline__ uint16_t f2bf(float f) {
    __bf16 b = static_cast<__bf16>(f);
    return __builtin_bit_cast(uint16_t, b);
}
__device__ __forceinline__ float bf2f(uint16_t h) {
    return __uint_as_float(static_cast<uint32_t>(h) << 16);
}
// fp32 value rounded through bf16.
__device__ __forceinline__ float round_bf(float f) { return bf2f(f2bf(f)); }

// Two fp32 values rounded to bf16 and packed (lo in bits 0-15): one v_cvt_pk_bf16_f32.
typedef float f32x2_t __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t pack2bf(float lo, float hi) {
    const f32x2_t v = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
}
// The halves of such a pair as fp32.
__device__ __forceinline__ float bf_lo(uint32_t p) { return __uint_as_float(p << 16); }
__device__ __forceinline__ float bf_hi(uint32_t p) { return __uint_as_float(p & 0xffff0000u); }

// torch's lerp (ATen/native/Lerp.h): two algebraically equal forms chosen by |weight|.
__device__ __forceinline__ float lerp_torch(float start, float end, float w) {
    const float diff = end - start;
    return (fabsf(w) < 0.5f) ? fmaf(w, diff, start) : end - diff * (1.0f - w);
}

// Largest s in [0, n) with prefix[s] <= b, for a non-decreasing prefix[0..n] with
// prefix[0] == 0 and b < prefix[n].
__device__ __forceinline__ int find_segment(const int32_t* __restrict__ prefix, int n, int b) {
    int lo = 0, hi = n;
    while (hi - lo > 1) {
        const int mid = (lo + hi) >> 1;
        if (prefix[mid] <= b) lo = mid; else hi = mid;
    }
    return lo;
}

// Sum over the 64 lanes of a wavefront; every lane gets the total.
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    return v;
}

}  // namespace muon_amd
