/* Scalar C restatement of the FP8 quantizers.  TEST INFRASTRUCTURE ONLY: it is
 * linked by tests/, smoke() and bench.py's cpu_baseline leg, never by the
 * shipped library.
 *
 * It shares no code with torch: the e4m3fn encoder below is an integer
 * round-to-nearest-even on the fp32 bit pattern, so agreement between this
 * file, torch's CPU cast and the known-answer table pins the cast three ways.
 *
 * Formula (one for all granularities; the reference call sites are
 * cosmos_rl/rollout/vllm_rollout/vllm_rollout.py:989-999 (rowwise),
 * cosmos_rl/utils/fp8/fp8_util.py:121-137 (tensorwise recipe),
 * cosmos_rl/policy/kernel/group_gemms.py:132,188-191 (128x128 / 1x128)):
 *     amax  = max |x|, scale = max(amax, 1e-12) / 448 (fp32 division),
 *     q     = e4m3fn_rne(clamp(x / scale, -448, 448)),
 * NaN in a reduction set -> scale 0x7FC00000 and bytes 0x7F.
 *
 * Build: gcc -O2 -fPIC -shared -ffp-contract=off -o libfp8ref.so fp8_ref.c -lm
 */
#include <math.h>
#include <stdint.h>
#include <string.h>

static inline float bf16_to_f32(uint16_t h) {
    uint32_t u = (uint32_t)h << 16;
    float f;
    memcpy(&f, &u, 4);
    return f;
}
static inline uint32_t f32_bits(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    return u;
}
static inline float bits_f32(uint32_t u) {
    float f;
    memcpy(&f, &u, 4);
    return f;
}

/* fp32 -> OCP e4m3fn, round to nearest even, no saturation: |v| >= 480 and
 * NaN/Inf give NaN.  e4m3fn: bias 7, 3 mantissa bits, subnormal step 2^-9,
 * largest finite 448 = 0x7E, NaN = 0x7F.  NaN is returned without sign. */
uint8_t fp8ref_e4m3_from_f32(float v) {
    uint32_t u = f32_bits(v);
    uint8_t sign = (uint8_t)((u >> 24) & 0x80);
    uint32_t a = u & 0x7FFFFFFFu;
    if (a >= 0x7F800000u) return 0x7F;                 /* Inf / NaN */
    int32_t e = (int32_t)(a >> 23) - 127;              /* unbiased exponent */
    uint32_t m = a & 0x7FFFFFu;
    uint32_t code;
    if (a == 0) return sign;
    if (e >= -6) {
        /* normal e4m3 candidate: keep 3 mantissa bits, RNE on the 20 dropped */
        uint32_t keep = m >> 20, rest = m & 0xFFFFFu, half = 0x80000u;
        code = ((uint32_t)(e + 7) << 3) | keep;
        if (rest > half || (rest == half && (keep & 1))) code += 1;  /* carries into exponent */
        if (code >= 0x7F) return 0x7F;                 /* >= 464 after rounding -> NaN */
    } else {
        /* subnormal target: value / 2^-9 rounded to an integer in 0..8 */
        if (e < -10 - 23) return sign;                 /* far below half the smallest step */
        uint32_t sig = (a >> 23) ? (m | 0x800000u) : m;/* fp32 subnormals have no hidden bit */
        int32_t ee = (a >> 23) ? e : -126;
        /* value = sig * 2^(ee-23); steps = value * 2^9 = sig * 2^(ee-14) ; ee <= -7 -> shift right */
        int32_t sh = 14 - ee;                          /* >= 21 */
        if (sh > 31) return sign;
        uint32_t q = sig >> sh, rest = sig & ((1u << sh) - 1u), half = 1u << (sh - 1);
        if (rest > half || (rest == half && (q & 1))) q += 1;
        code = q;                                      /* q == 8 is the smallest normal, 0x08 */
    }
    return (uint8_t)(sign | code);
}

float fp8ref_e4m3_to_f32(uint8_t b) {
    uint32_t e = (b >> 3) & 0xF, m = b & 7;
    float v;
    if ((b & 0x7F) == 0x7F) return NAN;
    if (e == 0) v = ldexpf((float)m, -9);
    else v = ldexpf((float)(8 + m), (int)e - 10);
    return (b & 0x80) ? -v : v;
}

static inline float scale_from_amax(float amax) {
    if (amax != amax) return bits_f32(0x7FC00000u);
    float a = amax < 1e-12f ? 1e-12f : amax;
    return a / 448.0f;
}

static inline uint8_t cast_one(float x, float scale) {
    float y = x / scale;
    if (y != y) return 0x7F;
    if (y > 448.0f) y = 448.0f;
    if (y < -448.0f) y = -448.0f;
    return fp8ref_e4m3_from_f32(y);
}

/* amax over a strided rectangle; NaN-propagating */
static float amax_rect(const uint16_t* x, int64_t ld, int64_t rows, int64_t cols) {
    float m = 0.0f;
    int nan = 0;
    for (int64_t r = 0; r < rows; ++r)
        for (int64_t c = 0; c < cols; ++c) {
            float v = fabsf(bf16_to_f32(x[r * ld + c]));
            if (v != v) nan = 1;
            else if (v > m) m = v;
        }
    return nan ? NAN : m;
}

void fp8ref_quant_rowwise(const uint16_t* x, int64_t R, int64_t C, uint8_t* q, float* s) {
    for (int64_t r = 0; r < R; ++r) {
        float sc = scale_from_amax(amax_rect(x + r * C, C, 1, C));
        s[r] = sc;
        for (int64_t c = 0; c < C; ++c) q[r * C + c] = cast_one(bf16_to_f32(x[r * C + c]), sc);
    }
}

/* fp32 -> bf16, round to nearest, ties to even, written as a search over the two neighbouring
 * bf16 values in double arithmetic (not the usual add-0x7FFF bit trick, so that it checks
 * torch's cast rather than repeating it); overflow rounds to infinity as IEEE 754 prescribes
 * (infinity stands for 2^128), NaN -> 0x7FC0.  This is `recv.to(torch.bfloat16)` at
 * cosmos_rl/policy/model/base.py:1068. */
uint16_t fp8ref_bf16_from_f32(float f) {
    if (f != f) return 0x7FC0u;
    const uint32_t u = f32_bits(f);
    const uint32_t lo = u & 0xFFFF0000u, hi = lo + 0x10000u;  /* hi is the neighbour farther from zero */
    if ((lo & 0x7F800000u) == 0x7F800000u) return (uint16_t)(lo >> 16);  /* infinity */
    const double x = fabs((double)f), a = fabs((double)bits_f32(lo));
    const double b = ((hi & 0x7FFFFFFFu) == 0x7F800000u) ? ldexp(1.0, 128) : fabs((double)bits_f32(hi));
    const double da = x - a, db = b - x;
    if (da < db) return (uint16_t)(lo >> 16);
    if (da > db) return (uint16_t)(hi >> 16);
    return (uint16_t)(((lo >> 16) & 1u) ? (hi >> 16) : (lo >> 16));
}

/* rowwise quantisation of fp32 input rounded to bf16 first (quant_rowwise_from in the torch oracle) */
void fp8ref_quant_rowwise_f32(const float* x, int64_t R, int64_t C, uint8_t* q, float* s) {
    for (int64_t r = 0; r < R; ++r) {
        float amax = 0.0f;
        int nan = 0;
        for (int64_t c = 0; c < C; ++c) {
            float v = fabsf(bf16_to_f32(fp8ref_bf16_from_f32(x[r * C + c])));
            if (v != v) nan = 1;
            else if (v > amax) amax = v;
        }
        float scale = nan ? bits_f32(0x7FC00000u) : scale_from_amax(amax);
        s[r] = scale;
        for (int64_t c = 0; c < C; ++c) q[r * C + c] = cast_one(bf16_to_f32(fp8ref_bf16_from_f32(x[r * C + c])), scale);
    }
}

void fp8ref_quant_tensorwise(const uint16_t* x, int64_t n, uint8_t* q, float* s) {
    float sc = scale_from_amax(amax_rect(x, n, 1, n));
    s[0] = sc;
    for (int64_t i = 0; i < n; ++i) q[i] = cast_one(bf16_to_f32(x[i]), sc);
}

/* scales: [ceil(R/128), ceil(C/128)] row-major (weight_mapper.py:236-243) */
void fp8ref_quant_block128(const uint16_t* x, int64_t R, int64_t C, uint8_t* q, float* s) {
    int64_t rb = (R + 127) / 128, cb = (C + 127) / 128;
    for (int64_t bi = 0; bi < rb; ++bi)
        for (int64_t bj = 0; bj < cb; ++bj) {
            int64_t r0 = bi * 128, c0 = bj * 128;
            int64_t nr = R - r0 < 128 ? R - r0 : 128, nc = C - c0 < 128 ? C - c0 : 128;
            float sc = scale_from_amax(amax_rect(x + r0 * C + c0, C, nr, nc));
            s[bi * cb + bj] = sc;
            for (int64_t r = 0; r < nr; ++r)
                for (int64_t c = 0; c < nc; ++c)
                    q[(r0 + r) * C + c0 + c] = cast_one(bf16_to_f32(x[(r0 + r) * C + c0 + c]), sc);
        }
}

/* scales: [M, ceil(K/128)] row-major (tests/test_deepep.py:85).
 * mode 0: build formula.  mode 1: tests/test_deepep.py:82-85 (multiply by
 * 448/clamp(amax,1e-4) - which torch evaluates as reciprocal(amax)*448 -, no
 * clamp before the cast, scale = amax/448). */
void fp8ref_quant_group128(const uint16_t* x, int64_t M, int64_t K, uint8_t* q, float* s, int mode) {
    int64_t kb = (K + 127) / 128;
    for (int64_t m = 0; m < M; ++m)
        for (int64_t b = 0; b < kb; ++b) {
            int64_t k0 = b * 128, nk = K - k0 < 128 ? K - k0 : 128;
            float amax = amax_rect(x + m * K + k0, K, 1, nk);
            if (mode == 0) {
                float sc = scale_from_amax(amax);
                s[m * kb + b] = sc;
                for (int64_t k = 0; k < nk; ++k)
                    q[m * K + k0 + k] = cast_one(bf16_to_f32(x[m * K + k0 + k]), sc);
            } else {
                if (amax != amax) {
                    s[m * kb + b] = bits_f32(0x7FC00000u);
                    for (int64_t k = 0; k < nk; ++k) q[m * K + k0 + k] = 0x7F;
                    continue;
                }
                float a = amax < 1e-4f ? 1e-4f : amax;
                float mul = (1.0f / a) * 448.0f; /* torch: scalar / tensor = reciprocal * scalar */
                s[m * kb + b] = a / 448.0f;
                for (int64_t k = 0; k < nk; ++k) {
                    float y = bf16_to_f32(x[m * K + k0 + k]) * mul;
                    q[m * K + k0 + k] = fp8ref_e4m3_from_f32(y);
                }
            }
        }
}

/* exp(t) as the fixed fp32 sequence the SwiGLU kernel uses: two-part ln2 reduction, Taylor
 * degree 7 in Horner form with fmaf, ldexpf.  Built with -ffp-contract=off, so every operation
 * below is exactly the one written. */
float fp8ref_exp32(float t) {
    t = t > 89.0f ? 89.0f : t;
    t = t < -104.0f ? -104.0f : t;
    const float n = rintf(t * 1.44269502162933349609375f);
    float r = fmaf(n, -0.693145751953125f, t);
    r = fmaf(n, -1.428606765330187045037746429443359375e-06f, r);
    float p = 1.98412701138295233249664306640625e-04f;
    p = fmaf(p, r, 1.388888922519981861114501953125e-03f);
    p = fmaf(p, r, 8.3333337679505348205566406250e-03f);
    p = fmaf(p, r, 4.16666679084300994873046875e-02f);
    p = fmaf(p, r, 0.16666667163372039794921875f);
    p = fmaf(p, r, 0.5f);
    p = fmaf(p, r, 1.0f);
    p = fmaf(p, r, 1.0f);
    return ldexpf(p, (int)n);
}

float fp8ref_silu32(float x) {
    if (x != x) return x;
    return x / (1.0f + fp8ref_exp32(-x));
}

/* h = bf16(bf16(silu(g)) * u): `self.activation_function(gate_proj_out) * up_proj_out` on bf16
 * tensors, cosmos_rl/policy/kernel/group_gemms.py:210 (SiLU), then the 1x128 quantiser of :213-218 */
void fp8ref_swiglu(const uint16_t* g, const uint16_t* u, int64_t n, uint16_t* h) {
    for (int64_t i = 0; i < n; ++i) {
        const uint16_t s = fp8ref_bf16_from_f32(fp8ref_silu32(bf16_to_f32(g[i])));
        h[i] = fp8ref_bf16_from_f32(bf16_to_f32(s) * bf16_to_f32(u[i]));
    }
}

/* Weighted combine of expert outputs into token order with bf16 rounding after every product and
 * every partial sum, starting from +0: `y = zeros_like(x)`, then per expert (ascending)
 * `y.scatter_add_(0, idx, expert_out * weights[idx, top, None])` on bf16 tensors,
 * cosmos_rl/policy/kernel/moe/moe.py:240-262.  row_map [T, topk] lists each token's source rows in
 * accumulation order (< 0: nothing).  mode 1: fp32 accumulator acc = fma(row, w, acc), one rounding
 * (cosmos_rl/policy/kernel/megatron_moe/permutation.py:370-424; w is fp32 there). */
void fp8ref_combine_rows(const uint16_t* rows, int64_t H, const int32_t* row_map, const uint16_t* w16, const float* w32,
                         int64_t T, int64_t topk, int mode, uint16_t* out) {
    for (int64_t t = 0; t < T; ++t)
        for (int64_t h = 0; h < H; ++h) {
            uint16_t y = 0;
            float acc = 0.0f;
            for (int64_t s = 0; s < topk; ++s) {
                const int32_t r = row_map[t * topk + s];
                if (r < 0) continue;
                const float x = bf16_to_f32(rows[(int64_t)r * H + h]);
                const float w = w32 ? w32[t * topk + s] : bf16_to_f32(w16[t * topk + s]);
                if (mode == 0) {
                    const uint16_t p = fp8ref_bf16_from_f32(x * w);
                    y = fp8ref_bf16_from_f32(bf16_to_f32(y) + bf16_to_f32(p));
                } else {
                    acc = fmaf(x, w, acc);
                }
            }
            out[t * H + h] = mode == 0 ? y : fp8ref_bf16_from_f32(acc);
        }
}

/* Division shortcut used by the kernels: r = 1/s (IEEE), q0 = x*r, e = fma(q0, s, -x),
 * q1 = fma(-e, r, q0), the byte is the e4m3 conversion of q1 WITHOUT a clamp.  The kernels only
 * divide by the scale of a set that x belongs to, so |x/s| <= 448 * (1 + 2^-22) there; every
 * finite bf16 x with an IEEE quotient in that range is checked.  Returns the number of (x, s)
 * pairs whose byte differs from the byte of the clamped IEEE quotient (signed zeros included:
 * the byte carries the sign).  *fp32_mismatch receives the count of pairs with
 * |x/s| >= 2^-11 - everywhere the quotient can still round to a non-zero byte - whose q1 is not
 * the IEEE quotient bit for bit. */
int64_t fp8ref_check_fast_div(const float* scales, int64_t n, int64_t* fp32_mismatch) {
    int64_t bad = 0, soft = 0;
    for (int64_t i = 0; i < n; ++i) {
        float s = scales[i];
        float r = 1.0f / s;
        for (uint32_t h = 0; h < 65536; ++h) {
            float x = bf16_to_f32((uint16_t)h);
            if (x != x || isinf(x)) continue;
            float want = x / s;
            if (!(fabsf(want) <= 448.0f * (1.0f + 0x1p-22f))) continue;
            float q0 = x * r;
            float e = fmaf(q0, s, -x);
            float q1 = fmaf(-e, r, q0);
            if (f32_bits(q1) != f32_bits(want) && fabsf(want) >= 0x1p-11f) ++soft;
            float a = want > 448.f ? 448.f : (want < -448.f ? -448.f : want);
            if (fp8ref_e4m3_from_f32(a) != fp8ref_e4m3_from_f32(q1)) ++bad;
        }
    }
    if (fp32_mismatch) *fp32_mismatch = soft;
    return bad;
}
