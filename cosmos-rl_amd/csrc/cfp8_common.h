// Shared device helpers and host-side error plumbing for libcosmosfp8 (gfx950 only).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "cosmos_fp8.h"

namespace cfp8 {

// ---- host side -----------------------------------------------------------
int set_error(int code, const char* fmt, ...);
int check_launch(const char* what);
int check_device();  // CFP8_OK when the current device is gfx950

static inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// ---- device side ---------------------------------------------------------
typedef uint32_t u32;
typedef unsigned short u16x2 __attribute__((ext_vector_type(2)));
typedef int i32x8 __attribute__((ext_vector_type(8)));
typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));

constexpr float kE4M3Max = 448.0f;
constexpr float kAmaxFloor = 1e-12f;
constexpr u32 kCanonNaN = 0x7FC00000u;

__device__ __forceinline__ float bf16_lo(u32 w) { return __uint_as_float(w << 16); }
__device__ __forceinline__ float bf16_hi(u32 w) { return __uint_as_float(w & 0xFFFF0000u); }

// max over |bf16| bit patterns, two lanes of 16 bits at a time.  Unsigned
// integer order equals numeric order for non-negative floats, and every NaN
// pattern (> 0x7F80) sorts above infinity, so NaN propagates by construction.
__device__ __forceinline__ u32 pk_absmax(u32 acc, u32 w) {
    u16x2 a = __builtin_bit_cast(u16x2, acc);
    u16x2 b = __builtin_bit_cast(u16x2, w & 0x7FFF7FFFu);
    return __builtin_bit_cast(u32, __builtin_elementwise_max(a, b));
}
__device__ __forceinline__ u32 pk_fold(u32 acc) {  // -> bf16 bits of the max, in the low half
    u32 lo = acc & 0xFFFFu, hi = acc >> 16;
    return lo > hi ? lo : hi;
}

template <int CTRL>
__device__ __forceinline__ u32 dpp(u32 v) {
    return (u32)__builtin_amdgcn_update_dpp(0, (int)v, CTRL, 0xF, 0xF, true);
}
__device__ __forceinline__ u32 umax(u32 a, u32 b) { return a > b ? a : b; }

// all-reduce max inside each aligned group of 16 lanes (one DPP row)
__device__ __forceinline__ u32 row16_max(u32 v) {
    v = umax(v, dpp<0xB1>(v));   // quad_perm [1,0,3,2]
    v = umax(v, dpp<0x4E>(v));   // quad_perm [2,3,0,1]
    v = umax(v, dpp<0x141>(v));  // row_half_mirror
    v = umax(v, dpp<0x140>(v));  // row_mirror
    return v;
}
// all-reduce max over the 64 lanes; the result is wave-uniform
__device__ __forceinline__ u32 wave_max(u32 v) {
    v = row16_max(v);
    u32 a = __builtin_amdgcn_readlane(v, 0), b = __builtin_amdgcn_readlane(v, 16);
    u32 c = __builtin_amdgcn_readlane(v, 32), d = __builtin_amdgcn_readlane(v, 48);
    return umax(umax(a, b), umax(c, d));
}

// amax bits (bf16 pattern in the low half) -> fp32 amax; NaN patterns stay NaN
__device__ __forceinline__ float amax_from_bits(u32 bits16) { return __uint_as_float(bits16 << 16); }

// scale = max(amax, 1e-12) / 448, NaN propagating and canonical
__device__ __forceinline__ float scale_from_amax(float amax) {
    if (amax != amax) return __uint_as_float(kCanonNaN);
    return fmaxf(amax, kAmaxFloor) / kE4M3Max;
}

// Per reduction set divider.  x / s is needed correctly rounded (the bytes must
// equal those of an IEEE fp32 division followed by a clamp to +-448 and an RNE cast).
// With r = 1/s correctly rounded, q0 = x*r, e = fma(q0, s, -x), q1 = fma(-e, r, q0) is
// the correctly rounded quotient wherever it is a normal number (Markstein); below
// 2^-11 every quotient rounds to a zero byte and only the sign matters, which this
// form of the residual keeps.  Non-finite scales (amax Inf or NaN) take the slow path.
struct Divider {
    float s, r;
    bool finite;
    __device__ __forceinline__ explicit Divider(float scale) {
        s = scale;
        finite = (__float_as_uint(scale) & 0x7F800000u) != 0x7F800000u;
        r = 1.0f / scale;
    }
    // The correctly rounded quotient x / s for finite x when `finite`, for the callers of this library: s is the
    // amax / 448 (amax floored at 1e-12) of a set that x belongs to, so |x / s| <= 448 * (1 + 2^-22) - the quotient
    // of the largest element is 448 or the fp32 value next to it - which is below 464 and which the conversion to
    // e4m3 rounds to at most 448 by itself: no clamp.  Reciprocal, product, residual, correction; the residual is
    // formed with the opposite sign, e = q0 * s - x, and subtracted, so that a zero keeps the sign of x without a
    // copysign (x = -0: q0 = -0, e = +0, (-e) * r + q0 = -0 + -0 = -0; x = +0: e = +0, -0 + +0 = +0; a q0 that
    // underflowed to a signed zero is met by (-e) * r = x * r of the same sign).
    __device__ __forceinline__ float fast(float x) const {
        float q0 = x * r;
        float e = __builtin_fmaf(q0, s, -x);
        return __builtin_fmaf(-e, r, q0);
    }
};

// Streaming (non-temporal) accesses: the quantisers read every input byte once and
// their output is consumed much later, so neither side should displace other data
// from L2 or the memory-side cache (and a no-allocate load never has to evict a
// dirty line first).
typedef u32 u32x4 __attribute__((ext_vector_type(4)));
typedef u32 u32x2 __attribute__((ext_vector_type(2)));
template <bool NT>
__device__ __forceinline__ uint4 ld16(const uint4* p) {
    if (NT) {
        const u32x4 v = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p));
        return make_uint4(v[0], v[1], v[2], v[3]);
    }
    return *p;
}
template <bool NT>
__device__ __forceinline__ void st8(uint2* p, uint2 o) {
    if (NT) {
        u32x2 v;
        v[0] = o.x;
        v[1] = o.y;
        __builtin_nontemporal_store(v, reinterpret_cast<u32x2*>(p));
    } else {
        *p = o;
    }
}
template <bool NT>
__device__ __forceinline__ void st16(uint4* p, uint4 o) {
    if (NT) {
        u32x4 v;
        v[0] = o.x; v[1] = o.y; v[2] = o.z; v[3] = o.w;
        __builtin_nontemporal_store(v, reinterpret_cast<u32x4*>(p));
    } else {
        *p = o;
    }
}

// two fp32 -> two OCP e4m3fn bytes (RNE) in the low or high half of `old`
template <bool HI>
__device__ __forceinline__ u32 cvt2(float a, float b, u32 old) {
    return (u32)__builtin_amdgcn_cvt_pk_fp8_f32(a, b, (int)old, HI);
}

// slow path byte for non-finite scales: NaN -> 0x7F, else clamp and convert
__device__ __forceinline__ u32 slow_byte(float x, float s) {
    float y = x / s;
    if (y != y) return 0x7Fu;
    y = __builtin_amdgcn_fmed3f(y, -kE4M3Max, kE4M3Max);
    return cvt2<false>(y, 0.0f, 0u) & 0xFFu;
}

// cast8 below for a finite scale only
__device__ __forceinline__ uint2 cast8_finite(const uint4& v, const Divider& d) {
    const u32 w[4] = {v.x, v.y, v.z, v.w};
    u32 o[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        u32 p = cvt2<false>(d.fast(bf16_lo(w[2 * i])), d.fast(bf16_hi(w[2 * i])), 0u);
        o[i] = cvt2<true>(d.fast(bf16_lo(w[2 * i + 1])), d.fast(bf16_hi(w[2 * i + 1])), p);
    }
    return make_uint2(o[0], o[1]);
}

// cast8 below for a scale that is +infinity or NaN, in integer arithmetic: x / NaN, NaN / s and inf / inf are NaN
// (byte 0x7F), a finite x over infinity is a zero with the sign of x
__device__ __forceinline__ uint2 cast8_nonfinite_scale(const uint4& v, float s) {
    const bool s_nan = s != s;
    const u32 w[4] = {v.x, v.y, v.z, v.w};
    u32 o[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        u32 bytes = 0;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const u32 h = (w[2 * i + (e >> 1)] >> ((e & 1) * 16)) & 0xFFFFu;  // bf16 bits
            const bool x_nonfinite = (h & 0x7F80u) == 0x7F80u;
            const u32 b = (s_nan || x_nonfinite) ? 0x7Fu : ((h >> 8) & 0x80u);
            bytes |= b << (8 * e);
        }
        o[i] = bytes;
    }
    return make_uint2(o[0], o[1]);
}

// 8 bf16 (one 16-byte vector) -> 8 fp8 bytes (uint2), element order preserved
__device__ __forceinline__ uint2 cast8(const uint4& v, const Divider& d) {
    const u32 w[4] = {v.x, v.y, v.z, v.w};
    u32 o[2];
    if (d.finite) {
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            u32 p = cvt2<false>(d.fast(bf16_lo(w[2 * i])), d.fast(bf16_hi(w[2 * i])), 0u);
            o[i] = cvt2<true>(d.fast(bf16_lo(w[2 * i + 1])), d.fast(bf16_hi(w[2 * i + 1])), p);
        }
    } else {
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            o[i] = slow_byte(bf16_lo(w[2 * i]), d.s) | (slow_byte(bf16_hi(w[2 * i]), d.s) << 8) |
                   (slow_byte(bf16_lo(w[2 * i + 1]), d.s) << 16) |
                   (slow_byte(bf16_hi(w[2 * i + 1]), d.s) << 24);
        }
    }
    return make_uint2(o[0], o[1]);
}

// cast8 for a scale that need not come from the data's own maximum: the quotient saturates at +-448 before the
// conversion, like the reference's clamp in front of its cast.  The decision is taken on the first product
// x * (1 / s): beyond 460 in magnitude (infinite included: a huge x over a small s, or x = +-inf, where the
// correction step would produce inf - inf) the result is +-448 with that sign; up to 460 the corrected quotient
// is below 464 and the conversion rounds it to at most 448 by itself.  A vector that holds a NaN is converted
// element by element, the NaN elements to the byte 0x7F (the hardware conversion of a NaN is not relied on).
__device__ __forceinline__ u32 absmax8(u32 acc, const uint4& v);
__device__ __forceinline__ uint2 cast8_clamped(const uint4& v, const Divider& d) {
    if (!d.finite) return cast8(v, d);
    const u32 w[4] = {v.x, v.y, v.z, v.w};
    auto q = [&](float x) {
        const float q0 = x * d.r;
        const float e = __builtin_fmaf(q0, d.s, -x);
        const float y = __builtin_fmaf(-e, d.r, q0);
        return __builtin_fabsf(q0) > 460.0f ? __builtin_copysignf(kE4M3Max, q0) : y;
    };
    u32 o[2];
    if (pk_fold(absmax8(0u, v)) > 0x7F80u) {
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            u32 bytes = 0;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const u32 word = w[2 * i + (e >> 1)];
                const float x = (e & 1) ? bf16_hi(word) : bf16_lo(word);
                const u32 b = x != x ? 0x7Fu : (cvt2<false>(q(x), 0.0f, 0u) & 0xFFu);
                bytes |= b << (8 * e);
            }
            o[i] = bytes;
        }
        return make_uint2(o[0], o[1]);
    }
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        u32 p = cvt2<false>(q(bf16_lo(w[2 * i])), q(bf16_hi(w[2 * i])), 0u);
        o[i] = cvt2<true>(q(bf16_lo(w[2 * i + 1])), q(bf16_hi(w[2 * i + 1])), p);
    }
    return make_uint2(o[0], o[1]);
}

__device__ __forceinline__ u32 absmax8(u32 acc, const uint4& v) {
    acc = pk_absmax(acc, v.x);
    acc = pk_absmax(acc, v.y);
    acc = pk_absmax(acc, v.z);
    return pk_absmax(acc, v.w);
}

// fp32 -> bf16 bits, round to nearest even, NaN kept quiet
__device__ __forceinline__ u32 f32_to_bf16_bits(float f) {
    u32 u = __float_as_uint(f);
    if ((u & 0x7FFFFFFFu) > 0x7F800000u) return (u >> 16) | 0x40u;
    return (u + 0x7FFFu + ((u >> 16) & 1u)) >> 16;
}
// two fp32 -> packed bf16 (round to nearest even) with the gfx950 conversion instruction
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ u32 pack_bf16x2(float a, float b) {
    f32x2 v;
    v[0] = a;
    v[1] = b;
    return __builtin_bit_cast(u32, __builtin_convertvector(v, bf16x2_t));
}

// exp(t) as a fixed sequence of IEEE fp32 operations (range reduction by ln2 in two parts, Taylor
// polynomial of degree 7 in Horner form with fused multiply-adds, exact scaling): every step is
// correctly rounded, so a CPU that runs the same sequence gets the same bits.  |error| < 2 ulp.
// t is clamped to [-104, 89]: below, the result is far under 2^-126 * 2^-24 and 1 + exp(t) == 1
// anyway; above, it overflows to infinity.  NaN is the caller's business.
__device__ __forceinline__ float exp32_det(float t) {
    t = t > 89.0f ? 89.0f : t;
    t = t < -104.0f ? -104.0f : t;
    const float n = __builtin_rintf(t * 1.44269502162933349609375f);
    float r = __builtin_fmaf(n, -0.693145751953125f, t);
    r = __builtin_fmaf(n, -1.428606765330187045037746429443359375e-06f, r);
    float p = 1.98412701138295233249664306640625e-04f;               // 1/5040
    p = __builtin_fmaf(p, r, 1.388888922519981861114501953125e-03f);  // 1/720
    p = __builtin_fmaf(p, r, 8.3333337679505348205566406250e-03f);    // 1/120
    p = __builtin_fmaf(p, r, 4.16666679084300994873046875e-02f);      // 1/24
    p = __builtin_fmaf(p, r, 0.16666667163372039794921875f);          // 1/6
    p = __builtin_fmaf(p, r, 0.5f);
    p = __builtin_fmaf(p, r, 1.0f);
    p = __builtin_fmaf(p, r, 1.0f);
    return __builtin_ldexpf(p, (int)n);
}

// SiLU of a bf16 value in fp32: x / (1 + exp(-x)), IEEE division; NaN stays NaN
__device__ __forceinline__ float silu32_det(float x) {
    if (x != x) return x;
    return x / (1.0f + exp32_det(-x));
}

// SiLU for results that are rounded to bf16 right away, four at a time.  The defining arithmetic is silu32_det (about 40
// VALU operations, most of them the IEEE division and the polynomial); what the caller keeps of it is the bf16
// rounding, 8 significant bits.  The hardware exponential and reciprocal (v_exp_f32, v_rcp_f32, one ulp each) give
// x / (1 + exp(-x)) in a fifth of the instructions, within a few fp32 ulps plus the rounding of the exponent
// t = -x log2(e), which weighs |t| ulps of t: measured over all bf16 inputs with |x| <= 16 the fast value is within
// 14 fp32 ulps of the defining one, within 1 for 99 % of them.  Two floats that close round to the same bf16 unless
// a rounding boundary of bf16 lies between them, i.e. unless the low 16 bits of the fast result are within
// 4 + |t| of 0x8000.  Only then - and for |x| > 16, infinities and NaN - the defining sequence runs: one wave-level
// test for the four values (the fast sequences of the four interleave, and the rare case lies out of line), then per
// flagged value.  That the bf16 result equals the defining one for every one of the 65536 bf16 inputs is checked
// exhaustively on the GPU by the test suite.
__device__ __forceinline__ void silu32x4_for_bf16(const float (&x)[4], float (&y)[4]) {
    bool redo[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const float t = x[i] * -1.44269502162933349609375f;
        y[i] = x[i] * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(t));
        const u32 margin = 4u + (u32)__builtin_fabsf(t);  // (the conversion saturates; NaN gives 0)
        const u32 low = __float_as_uint(y[i]) & 0xFFFFu;
        redo[i] = low - (0x8000u - margin) <= 2u * margin || !(__builtin_fabsf(x[i]) <= 16.0f);
    }
    if (__builtin_expect(redo[0] || redo[1] || redo[2] || redo[3], 0)) {
#pragma unroll
        for (int i = 0; i < 4; ++i)
            if (redo[i]) y[i] = silu32_det(x[i]);
    }
}

// four gate values (two words of two packed bf16) and four up values -> four packed bf16 of bf16(bf16(silu(g)) * u)
__device__ __forceinline__ void swiglu_quad(u32 g0, u32 g1, u32 u0, u32 u1, u32& h0, u32& h1) {
    const float x[4] = {bf16_lo(g0), bf16_hi(g0), bf16_lo(g1), bf16_hi(g1)};
    float y[4];
    silu32x4_for_bf16(x, y);
    const u32 s0 = pack_bf16x2(y[0], y[1]), s1 = pack_bf16x2(y[2], y[3]);
    h0 = pack_bf16x2(bf16_lo(s0) * bf16_lo(u0), bf16_hi(s0) * bf16_hi(u0));
    h1 = pack_bf16x2(bf16_lo(s1) * bf16_lo(u1), bf16_hi(s1) * bf16_hi(u1));
}

}  // namespace cfp8
