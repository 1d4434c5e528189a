// Shared host/device plumbing of the gfx950 routed-expert library: status codes and the
// thread-local error string behind the C ABI, launch checking, and the device primitives
// every kernel uses (nibble unpack, wave64 reductions, fp16 helpers).
#pragma once

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>

#include "../../include/aeon_mi355.h"

namespace aeon355 {

// ---- host: status + error text ------------------------------------------------------------

void set_error(const char* fmt, ...);

#define AEON_REQUIRE(cond, code, ...)            \
    do {                                         \
        if (!(cond)) {                           \
            ::aeon355::set_error(__VA_ARGS__);   \
            return (code);                       \
        }                                        \
    } while (0)

#define AEON_HIP(call)                                                                  \
    do {                                                                                \
        hipError_t aeon_hip_err_ = (call);                                              \
        if (aeon_hip_err_ != hipSuccess) {                                              \
            ::aeon355::set_error("%s failed: %s (%s:%d)", #call,                        \
                                 hipGetErrorString(aeon_hip_err_), __FILE__, __LINE__); \
            return AEON_ERR_HIP;                                                        \
        }                                                                               \
    } while (0)

// A launch is checked with hipGetLastError only: everything stays asynchronous on the
// caller's stream, as the reference's dispatchers are.
#define AEON_LAUNCH_CHECK() AEON_HIP(hipGetLastError())

inline hipStream_t as_stream(void* s) { return reinterpret_cast<hipStream_t>(s); }

// ---- device primitives ---------------------------------------------------------------------

typedef _Float16 half_t;
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));
typedef float float16_t __attribute__((ext_vector_type(16)));

// Pointers read out of a device-resident table are generic to the compiler, which then emits
// FLAT loads (they count against both memory counters and cannot be waited on in order).
// Every such pointer here is device global memory; saying so restores global_load and the
// in-order vmcnt pipelining the kernels are written for.
#define AEON_GLOBAL __attribute__((address_space(1)))
template <class T>
__device__ __forceinline__ const AEON_GLOBAL T* as_global(const T* p) {
    return (const AEON_GLOBAL T*)(p);
}
template <class T>
__device__ __forceinline__ const AEON_GLOBAL T* as_global(const void* p) {
    return (const AEON_GLOBAL T*)(p);
}

// A decode launch reads every weight once, while activations, scales (whose cache lines are
// shared between neighbouring row tiles), tables and expert lists are read again and again by
// other workgroups. The streaming ("non-temporal") hint on the weight loads keeps them from
// pushing the re-read data out of the caches: measured on the batch-64 decode step, 0.412 ->
// 0.371 ms with nothing else changed (with the hint on the scales as well: 0.375). Where
// weights ARE read again -- the prefill windows of a hot expert -- the hint costs (2.27 -> 2.39
// ms), so the grouped kernels load normally.
template <class T>
__device__ __forceinline__ T stream_load(const T* p) {
    return __builtin_nontemporal_load(p);
}
template <class T>
__device__ __forceinline__ T stream_load(const AEON_GLOBAL T* p) {
    return __builtin_nontemporal_load(p);
}
__device__ __forceinline__ uint4 stream_load(const uint4* p) {
    const u32x4_t v = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(p));
    return make_uint4(v[0], v[1], v[2], v[3]);
}
__device__ __forceinline__ uint2 stream_load(const uint2* p) {
    const u32x2_t v = __builtin_nontemporal_load(reinterpret_cast<const u32x2_t*>(p));
    return make_uint2(v[0], v[1]);
}

template <bool STREAM, class P>
__device__ __forceinline__ auto load_maybe_stream(P p) {
    if constexpr (STREAM) return stream_load(p);
    else return *p;
}

union Word2Half {
    uint32_t u;
    half2_t h;
};

// Eight int4 weights of one packed word -> four half2 holding (q - 8) exactly.
//
// Nibble order inside the word is the storage format's: column 2j sits in nibble j and
// column 2j+1 in nibble 4+j, so masking with 0x000F000F yields the pair (2j, 2j+1) for j=0
// directly. OR-ing 0x6400 makes the fp16 1024+q; a nibble left in bits 4..7 under 0x5400
// reads as 64+q (the fp16 ulp at 64 is 1/16), which saves two of the four shifts.
// (x & mask) | bits in one VALU instruction. The compiler emits v_and + v_or because a VOP3
// instruction cannot carry two literals on this target; with the constants held in registers
// the fused form applies.
__device__ __forceinline__ uint32_t and_or(uint32_t x, uint32_t mask, uint32_t bits) {
    uint32_t r;
    asm("v_and_or_b32 %0, %1, %2, %3" : "=v"(r) : "v"(x), "v"(mask), "v"(bits));
    return r;
}

__device__ __forceinline__ void unpack8(uint32_t w, half2_t out[4]) {
    Word2Half a, b, c, d;
    const uint32_t w8 = w >> 8;
    a.u = and_or(w, 0x000F000Fu, 0x64006400u);
    b.u = and_or(w, 0x00F000F0u, 0x54005400u);
    c.u = and_or(w8, 0x000F000Fu, 0x64006400u);
    d.u = and_or(w8, 0x00F000F0u, 0x54005400u);
    const half2_t k1032 = {(half_t)1032.0f, (half_t)1032.0f};
    const half2_t k72 = {(half_t)72.0f, (half_t)72.0f};
    out[0] = a.h - k1032;
    out[1] = b.h - k72;
    out[2] = c.h - k1032;
    out[3] = d.h - k72;
}

__device__ __forceinline__ half8_t unpack8_vec(uint32_t w) {
    half2_t p[4];
    unpack8(w, p);
    half8_t v = {p[0][0], p[0][1], p[1][0], p[1][1], p[2][0], p[2][1], p[3][0], p[3][1]};
    return v;
}

__device__ __forceinline__ float dot2(half2_t a, half2_t b, float c) {
    return __builtin_amdgcn_fdot2(a, b, c, false);
}

// dot of the 8 weights of one word (already unpacked) with 8 activations (a uint4 = 8 halves),
// fp32 accumulate.
__device__ __forceinline__ float dot8(const half2_t p[4], const uint4& x, float acc) {
    Word2Half x0, x1, x2, x3;
    x0.u = x.x; x1.u = x.y; x2.u = x.z; x3.u = x.w;
    acc = dot2(p[0], x0.h, acc);
    acc = dot2(p[1], x1.h, acc);
    acc = dot2(p[2], x2.h, acc);
    acc = dot2(p[3], x3.h, acc);
    return acc;
}

// the same from the packed word
__device__ __forceinline__ float dot8(uint32_t w, const uint4& x, float acc) {
    half2_t p[4];
    unpack8(w, p);
    return dot8(p, x, acc);
}

__device__ __forceinline__ float half_bits_to_float(uint16_t bits) {
    union { uint16_t u; half_t h; } v;
    v.u = bits;
    return (float)v.h;
}

__device__ __forceinline__ uint16_t float_to_half_bits(float x) {
    union { uint16_t u; half_t h; } v;
    v.h = (half_t)x;  // v_cvt_f16_f32, round to nearest even
    return v.u;
}

// silu(min(gate, L)) * clamp(up, -L, L): the gate is bounded only from above.
__device__ __forceinline__ float clamped_swiglu(float gate, float up, float limit) {
    gate = fminf(gate, limit);
    up = fminf(fmaxf(up, -limit), limit);
    return (gate / (1.0f + expf(-gate))) * up;
}

// xor-butterfly add across the 64 lanes of a wave, for the lane-id bits set in `mask_bits`
// (e.g. 0x30 sums lanes that differ in bits 4 and 5). Every lane must call it.
__device__ __forceinline__ float wave_xor_sum(float v, int mask_bits) {
#pragma unroll
    for (int offset = 32; offset > 0; offset >>= 1) {
        if (mask_bits & offset) v += __shfl_xor(v, offset, 64);
    }
    return v;
}

}  // namespace aeon355
