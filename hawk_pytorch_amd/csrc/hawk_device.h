// Device-side helpers shared by the RG-LRU scan, conv1d and decode-step kernels (gfx950).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace hawk {

constexpr int kWave = 64;
constexpr float kLog2e = 1.4426950408889634f;

// ---------------------------------------------------------------------------------------
// Element types.  Activations are either bf16 (stored as raw uint16_t) or fp32.
// ---------------------------------------------------------------------------------------
struct bf16_t {
    uint16_t bits;
};

typedef __bf16 bf16x2_native __attribute__((ext_vector_type(2)));
typedef float float2_native __attribute__((ext_vector_type(2)));
// Native vector types for raw register images (accepted by the nontemporal builtins).
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x8 __attribute__((ext_vector_type(8)));

// Two fp32 -> packed bf16 pair, round-to-nearest-even (one v_cvt_pk_bf16_f32 on gfx950).
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
    float2_native v = {lo, hi};
    bf16x2_native r = __builtin_convertvector(v, bf16x2_native);
    return __builtin_bit_cast(uint32_t, r);
}
__device__ __forceinline__ uint16_t to_bf16_bits(float f) {
    return __builtin_bit_cast(uint16_t, (__bf16)f);
}
__device__ __forceinline__ float bf16_lo(uint32_t w) { return __uint_as_float(w << 16); }
__device__ __forceinline__ float bf16_hi(uint32_t w) { return __uint_as_float(w & 0xffff0000u); }

// Two fp32 in [0,1] -> packed fp16 pair (one v_cvt_pkrtz_f16_f32) and back.  Used only for
// running products of alpha that scale a carry: their 2^-10 relative error lands on a
// correction term and is far below the bf16 rounding of the stored result.
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t pack_f16x2(float lo, float hi) {
    return __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(lo, hi));
}
__device__ __forceinline__ float f16_lo(uint32_t w) { return (float)__builtin_bit_cast(f16x2, w).x; }
__device__ __forceinline__ float f16_hi(uint32_t w) { return (float)__builtin_bit_cast(f16x2, w).y; }

// Raw register image of V consecutive elements of type ET.
template <typename ET, int V>
struct Raw;
template <>
struct Raw<bf16_t, 1> { typedef uint16_t type; };
template <>
struct Raw<bf16_t, 2> { typedef uint32_t type; };
template <>
struct Raw<bf16_t, 4> { typedef u32x2 type; };
template <>
struct Raw<bf16_t, 8> { typedef u32x4 type; };
template <>
struct Raw<float, 1> { typedef float type; };
template <>
struct Raw<float, 2> { typedef f32x2 type; };
template <>
struct Raw<float, 4> { typedef f32x4 type; };
template <>
struct Raw<float, 8> { typedef f32x8 type; };

__device__ __forceinline__ void unpack(uint16_t r, float (&o)[1]) { o[0] = __uint_as_float((uint32_t)r << 16); }
__device__ __forceinline__ void unpack(uint32_t r, float (&o)[2]) { o[0] = bf16_lo(r); o[1] = bf16_hi(r); }
__device__ __forceinline__ void unpack(u32x2 r, float (&o)[4]) {
    o[0] = bf16_lo(r.x); o[1] = bf16_hi(r.x); o[2] = bf16_lo(r.y); o[3] = bf16_hi(r.y);
}
__device__ __forceinline__ void unpack(u32x4 r, float (&o)[8]) {
    o[0] = bf16_lo(r.x); o[1] = bf16_hi(r.x); o[2] = bf16_lo(r.y); o[3] = bf16_hi(r.y);
    o[4] = bf16_lo(r.z); o[5] = bf16_hi(r.z); o[6] = bf16_lo(r.w); o[7] = bf16_hi(r.w);
}
__device__ __forceinline__ void unpack(float r, float (&o)[1]) { o[0] = r; }
__device__ __forceinline__ void unpack(f32x2 r, float (&o)[2]) { o[0] = r.x; o[1] = r.y; }
__device__ __forceinline__ void unpack(f32x4 r, float (&o)[4]) { o[0] = r.x; o[1] = r.y; o[2] = r.z; o[3] = r.w; }
__device__ __forceinline__ void unpack(f32x8 r, float (&o)[8]) {
#pragma unroll
    for (int k = 0; k < 8; ++k) o[k] = r[k];
}

__device__ __forceinline__ void pack(const float (&v)[1], uint16_t& r) { r = to_bf16_bits(v[0]); }
__device__ __forceinline__ void pack(const float (&v)[2], uint32_t& r) { r = pack_bf16x2(v[0], v[1]); }
__device__ __forceinline__ void pack(const float (&v)[4], u32x2& r) {
    r.x = pack_bf16x2(v[0], v[1]); r.y = pack_bf16x2(v[2], v[3]);
}
__device__ __forceinline__ void pack(const float (&v)[8], u32x4& r) {
    r.x = pack_bf16x2(v[0], v[1]); r.y = pack_bf16x2(v[2], v[3]);
    r.z = pack_bf16x2(v[4], v[5]); r.w = pack_bf16x2(v[6], v[7]);
}
__device__ __forceinline__ void pack(const float (&v)[1], float& r) { r = v[0]; }
__device__ __forceinline__ void pack(const float (&v)[2], f32x2& r) { r.x = v[0]; r.y = v[1]; }
__device__ __forceinline__ void pack(const float (&v)[4], f32x4& r) { r.x = v[0]; r.y = v[1]; r.z = v[2]; r.w = v[3]; }
__device__ __forceinline__ void pack(const float (&v)[8], f32x8& r) {
#pragma unroll
    for (int k = 0; k < 8; ++k) r[k] = v[k];
}

template <typename R>
__device__ __forceinline__ R raw_zero() {
    R r;
    __builtin_memset(&r, 0, sizeof(R));
    return r;
}

template <typename ET, int V>
__device__ __forceinline__ typename Raw<ET, V>::type load_raw(const ET* p) {
    return *reinterpret_cast<const typename Raw<ET, V>::type*>(p);
}
// Streaming store: the outputs are written once and not read again by this kernel.
template <typename ET, int V>
__device__ __forceinline__ void store_raw(ET* p, typename Raw<ET, V>::type r) {
    __builtin_nontemporal_store(r, reinterpret_cast<typename Raw<ET, V>::type*>(p));
}

// ---------------------------------------------------------------------------------------
// Buffer addressing.  A wave describes the slab of a tensor it works on with a buffer
// resource in scalar registers (base pointer + byte size); every access is then
// "resource + per-lane byte offset (one VGPR shared by all accesses) + scalar row offset",
// which costs no vector address arithmetic.  The hardware range check returns zero for
// loads and drops stores at or beyond the slab size, which is how ragged last tiles are
// handled.
// ---------------------------------------------------------------------------------------
typedef __amdgpu_buffer_rsrc_t rsrc_t;

__device__ __forceinline__ rsrc_t make_rsrc(const void* base, uint32_t bytes) {
    // raw buffer: stride 0, 32-bit untyped data format
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, (int)bytes, 0x00020000);
}

// Cache-policy bits of the buffer instructions.  Every tensor byte is touched exactly once
// per kernel, so both loads and stores are marked non-temporal ("nt"), which measurably
// raises streaming bandwidth on this part.
constexpr int kAuxDefault = 0;
constexpr int kAuxStream = 2;
#ifndef HAWK_LOAD_AUX
#define HAWK_LOAD_AUX kAuxStream
#endif

template <typename R>
__device__ __forceinline__ R buffer_load(rsrc_t r, uint32_t lane_bytes, uint32_t row_bytes) {
    if constexpr (sizeof(R) == 2) {
        return __builtin_bit_cast(R, __builtin_amdgcn_raw_buffer_load_b16(r, lane_bytes, row_bytes, HAWK_LOAD_AUX));
    } else if constexpr (sizeof(R) == 4) {
        return __builtin_bit_cast(R, __builtin_amdgcn_raw_buffer_load_b32(r, lane_bytes, row_bytes, HAWK_LOAD_AUX));
    } else if constexpr (sizeof(R) == 8) {
        return __builtin_bit_cast(R, __builtin_amdgcn_raw_buffer_load_b64(r, lane_bytes, row_bytes, HAWK_LOAD_AUX));
    } else {
        static_assert(sizeof(R) == 16, "unsupported access width");
        return __builtin_bit_cast(R, __builtin_amdgcn_raw_buffer_load_b128(r, lane_bytes, row_bytes, HAWK_LOAD_AUX));
    }
}

template <typename R>
__device__ __forceinline__ void buffer_store(R v, rsrc_t r, uint32_t lane_bytes, uint32_t row_bytes) {
    if constexpr (sizeof(R) == 2) {
        __builtin_amdgcn_raw_buffer_store_b16(__builtin_bit_cast(unsigned short, v), r, lane_bytes, row_bytes, kAuxStream);
    } else if constexpr (sizeof(R) == 4) {
        __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned int, v), r, lane_bytes, row_bytes, kAuxStream);
    } else if constexpr (sizeof(R) == 8) {
        __builtin_amdgcn_raw_buffer_store_b64(__builtin_bit_cast(u32x2, v), r, lane_bytes, row_bytes, kAuxStream);
    } else {
        static_assert(sizeof(R) == 16, "unsupported access width");
        __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, v), r, lane_bytes, row_bytes, kAuxStream);
    }
}

// ---------------------------------------------------------------------------------------
// Transcendentals: one hardware instruction each (v_exp_f32, v_rcp_f32, v_sqrt_f32,
// v_rsq_f32; about 1 ulp), which is what keeps the scan bandwidth-bound.
// ---------------------------------------------------------------------------------------
__device__ __forceinline__ float hw_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ float hw_rcp(float x) { return __builtin_amdgcn_rcpf(x); }
__device__ __forceinline__ float hw_sqrt(float x) { return __builtin_amdgcn_sqrtf(x); }
__device__ __forceinline__ float hw_rsq(float x) { return __builtin_amdgcn_rsqf(x); }

// logistic(x) = 1 / (1 + 2^(-x log2 e)); saturates cleanly to 0 and 1 at +-inf.
__device__ __forceinline__ float sigmoid_fast(float x) {
    return hw_rcp(1.0f + hw_exp2(-kLog2e * x));
}

// 1 - exp(y) for y <= 0 without cancellation: a degree-8 series for |y| < 1/4
// (truncation below 3e-9 relative), the direct form elsewhere (result >= 0.22).
__device__ __forceinline__ float one_minus_exp(float y) {
    float direct = 1.0f - hw_exp2(kLog2e * y);
    float p = 1.0f / 40320.0f;
    p = fmaf(p, y, 1.0f / 5040.0f);
    p = fmaf(p, y, 1.0f / 720.0f);
    p = fmaf(p, y, 1.0f / 120.0f);
    p = fmaf(p, y, 1.0f / 24.0f);
    p = fmaf(p, y, 1.0f / 6.0f);
    p = fmaf(p, y, 0.5f);
    p = fmaf(p, y, 1.0f);
    float series = -y * p;
    return (y > -0.25f) ? series : direct;
}

// softplus(x) = log(1 + e^x) to about 1e-6 relative accuracy over the whole range
// (Lambda is strongly negative at init, so relative accuracy for tiny results matters), in a
// dozen instructions: it is evaluated per lane per tile, so a library-grade routine would
// cost as much as several rows of the scan itself.
//   u = e^x;  u < 1/16: series u (1 - u/2 + u^2/3 - u^3/4 + u^4/5);  else ln2 * log2(1 + u);
//   x > 16: x + e^-x.
__device__ __forceinline__ float softplus_fast(float x) {
    const float u = hw_exp2(kLog2e * fminf(x, 16.0f));
    float p = 0.2f;
    p = fmaf(p, u, -0.25f);
    p = fmaf(p, u, 1.0f / 3.0f);
    p = fmaf(p, u, -0.5f);
    p = fmaf(p, u, 1.0f);
    const float small = u * p;
    const float mid = 0.6931471805599453f * __builtin_amdgcn_logf(1.0f + u);
    const float big = x + hw_exp2(-kLog2e * fmaxf(x, 16.0f));
    const float lo = (u < 0.0625f) ? small : mid;
    return (x > 16.0f) ? big : lo;
}

// Library-grade variants, for code that runs once per channel per launch.
__device__ __forceinline__ float softplus_precise(float x) {
    return x > 20.0f ? x : log1pf(expf(x));
}
__device__ __forceinline__ float sigmoid_precise(float x) {
    if (x >= 0.0f) return 1.0f / (1.0f + expf(-x));
    float e = expf(x);
    return e / (1.0f + e);
}

// Identity the optimiser cannot see through: stops it from keeping a value alive in a
// register across a long region when re-evaluating it later is the cheaper choice.
__device__ __forceinline__ float opaque(float x) {
    asm volatile("" : "+v"(x));
    return x;
}
__device__ __forceinline__ uint32_t opaque(uint32_t x) {
    asm volatile("" : "+v"(x));
    return x;
}
__device__ __forceinline__ uint16_t opaque(uint16_t x) {
    uint32_t w = x;
    asm volatile("" : "+v"(w));
    return (uint16_t)w;
}

__device__ __forceinline__ float clamp01(float z) { return fminf(fmaxf(z, 0.0f), 1.0f); }

// Standard normal CDF Phi(y) and e = exp(-y^2 / 2), the two pieces of the exact (erf) GELU:
//   gelu(y) = y Phi(y),   gelu'(y) = Phi(y) + y e / sqrt(2 pi).
//   PRECISE: Phi from erfc(|y| / sqrt 2) = t exp(-x^2 + P9(t)), t = 1 / (1 + x/2)  (Numerical
//            Recipes' erfcc; relative error 1.2e-7 in exact arithmetic, about 4e-6 in fp32,
//            also in the negative tail)
//   else:    erfc = t P4(t) exp(-x^2), t = 1 / (1 + 0.3275911 x)  (Abramowitz & Stegun 7.1.26;
//            absolute error of Phi 3e-7 in fp32, far below bf16 rounding), 14 instructions
template <bool PRECISE>
__device__ __forceinline__ void normal_cdf(float y, float& cdf, float& e) {
    if (PRECISE) {
        const float ax = fabsf(y) * 0.70710678118654752f;
        const float nx2 = -ax * ax;
        e = hw_exp2(nx2 * kLog2e);
        const float t = hw_rcp(fmaf(0.5f, ax, 1.0f));
        float p = 0.17087277f;
        p = fmaf(p, t, -0.82215223f);
        p = fmaf(p, t, 1.48851587f);
        p = fmaf(p, t, -1.13520398f);
        p = fmaf(p, t, 0.27886807f);
        p = fmaf(p, t, -0.18628806f);
        p = fmaf(p, t, 0.09678418f);
        p = fmaf(p, t, 0.37409196f);
        p = fmaf(p, t, 1.00002368f);
        p = fmaf(p, t, -1.26551223f);
        const float half_erfc = (0.5f * t) * hw_exp2((nx2 + p) * kLog2e);
        cdf = (y < 0.0f) ? half_erfc : 1.0f - half_erfc;
    } else {
        // u = |y| sqrt(log2(e) / 2), so that exp(-y^2 / 2) = 2^(-u^2); the constants of the
        // rational argument and the factor 1/2 are folded into the coefficients
        constexpr float kScale = 0.84932180028801904f;          // sqrt(log2(e) / 2)
        constexpr float kP = 0.3275911f * 0.83255461115769776f;   // p / sqrt(2) / kScale
        const float u = fabsf(y) * kScale;
        e = hw_exp2(-(u * u));
        const float t = hw_rcp(fmaf(kP, u, 1.0f));
        float p = 0.5f * 1.061405429f;
        p = fmaf(p, t, 0.5f * -1.453152027f);
        p = fmaf(p, t, 0.5f * 1.421413741f);
        p = fmaf(p, t, 0.5f * -0.284496736f);
        p = fmaf(p, t, 0.5f * 0.254829592f);
        const float half_erfc = (t * p) * e;
        // 1/2 + sign(y) (1/2 - half_erfc)
        cdf = 0.5f + __builtin_copysignf(0.5f - half_erfc, y);
    }
}
constexpr float kInvSqrt2Pi = 0.39894228040143268f;

// One decode step of the RG-LRU for one channel (hawk/hawk.py:137-151, :196 upstream):
//   h = alpha * state + sqrt(1 - alpha^2) * (sigmoid(xg) * x),  alpha = exp(-8 s sigmoid(ag)),
// with s = softplus(Lambda) evaluated by the caller.
__device__ __forceinline__ float rglru_step_value(float x, float xg, float ag, float s, float state) {
    const float i = sigmoid_fast(xg);
    const float r = sigmoid_fast(ag);
    const float alpha = hw_exp2(-8.0f * kLog2e * s * r);
    const float z = one_minus_exp(-16.0f * s * r);
    return fmaf(alpha, state, hw_sqrt(z) * (i * x));
}
// gelu(y) * h with the exact (erf) GELU (hawk/hawk.py:134-135 upstream).
__device__ __forceinline__ float gelu_times(float y, float h) {
    float cdf, e;
    normal_cdf<true>(y, cdf, e);
    return (y * cdf) * h;
}

}  // namespace hawk
