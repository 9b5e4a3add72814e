// MXFP4 weight quantisation: blocks of 32 consecutive elements of a row share one power-of-two
// scale (an e8m0 byte), every element becomes a 4-bit e2m1 code, two codes per byte (the element
// with the even index in the low nibble).
//
//   amax   = max |x| over the block
//   scale  = 2^ceil(log2(amax / 6))      as bits: ((amax / 6).bits + 0x007FFFFF) & 0x7F800000
//   code   = e2m1(x / scale), round to nearest, ties away from zero, |x / scale| <= 6 by construction
//
// Four lanes (one DPP quad) own a block, 16 bytes of bf16 each.  The hardware conversion
// v_cvt_scalef32_pk_fp4_f32 rounds ties to even, so the quotient is first multiplied by 1 + 2^-10:
// a bf16 value times a power of two has 8 significant bits, so a quotient that is not a tie is at
// least a factor 1 - 2^-9 away from the next tie above it and stays below it, while a tie moves
// up and rounds away from zero.  The product is exact in fp32 (8 + 11 bits).
// NaN and infinity in the input give unspecified codes.
#include "cfp8_common.h"

namespace cfp8 {

__global__ __launch_bounds__(256) void mxfp4_kernel(const uint4* __restrict__ x, int64_t ldx, unsigned nvec, unsigned total,
                                                    u32* __restrict__ q, int64_t ldq, uint8_t* __restrict__ scales,
                                                    int64_t lds) {
    uint4 v[4];
    unsigned row[4], col[4];
    bool ok[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        const unsigned idx = (blockIdx.x * 4 + k) * 256 + threadIdx.x;  // total < 2^31: no overflow
        ok[k] = idx < total;
        const unsigned i = ok[k] ? idx : 0;
        row[k] = i / nvec;
        col[k] = i - row[k] * nvec;
        v[k] = ld16<true>(x + (int64_t)row[k] * ldx + col[k]);
    }
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        u32 m = pk_fold(absmax8(0u, v[k]));
        m = umax(m, dpp<0xB1>(m));  // quad_perm [1,0,3,2]
        m = umax(m, dpp<0x4E>(m));  // quad_perm [2,3,0,1]
        const float dequant = amax_from_bits(m) / 6.0f;
        const u32 e = ((__float_as_uint(dequant) + 0x007FFFFFu) & 0x7F800000u) >> 23;  // e8m0 byte
        // 1 / 2^(e - 127); e = 0 (all-zero block) and e = 255 give 0, e = 254 a subnormal
        const float inv = e == 0u || e == 255u ? 0.f : __uint_as_float(e == 254u ? 0x00400000u : (254u - e) << 23);
        const float c = inv * 1.0009765625f;
        const u32 w[4] = {v[k].x, v[k].y, v[k].z, v[k].w};
        u32 out = 0;
        out = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(out, bf16_lo(w[0]) * c, bf16_hi(w[0]) * c, 1.0f, 0);
        out = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(out, bf16_lo(w[1]) * c, bf16_hi(w[1]) * c, 1.0f, 1);
        out = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(out, bf16_lo(w[2]) * c, bf16_hi(w[2]) * c, 1.0f, 2);
        out = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(out, bf16_lo(w[3]) * c, bf16_hi(w[3]) * c, 1.0f, 3);
        if (ok[k]) {
            __builtin_nontemporal_store(out, q + (int64_t)row[k] * ldq + col[k]);
            if ((threadIdx.x & 3) == 0) scales[(int64_t)row[k] * lds + (col[k] >> 2)] = (uint8_t)e;
        }
    }
}

}  // namespace cfp8

extern "C" int cfp8_quant_mxfp4(const void* x, int64_t rows, int64_t cols, int64_t ld_x, void* q, int64_t ld_q,
                                void* scales, int64_t ld_scales, void* stream) {
    using namespace cfp8;
    if (rows < 0 || cols < 0) return set_error(CFP8_EINVAL, "quant_mxfp4: negative shape");
    if (cols % 32) return set_error(CFP8_EINVAL, "quant_mxfp4: cols=%lld must be a multiple of 32", (long long)cols);
    if (rows == 0 || cols == 0) return CFP8_OK;
    if (!x || !q || !scales) return set_error(CFP8_EINVAL, "quant_mxfp4: null pointer");
    if (ld_x % 8 || ld_x < cols || ld_q % 4 || ld_q < cols / 2 || ld_scales < cols / 32)
        return set_error(CFP8_EINVAL, "quant_mxfp4: pitches: ld_x %% 8 == 0 and >= cols, ld_q %% 4 == 0 and >= cols / 2 (bytes), ld_scales >= cols / 32");
    if (!aligned16(x) || (reinterpret_cast<uintptr_t>(q) & 3u)) return set_error(CFP8_EINVAL, "quant_mxfp4: misaligned pointer (x 16 bytes, q 4 bytes)");
    const int64_t nvec = cols / 8;
    if (nvec >= (1ll << 30)) return set_error(CFP8_EINVAL, "quant_mxfp4: row too long");
    if (int rc = check_device()) return rc;
    hipStream_t st = static_cast<hipStream_t>(stream);
    // a launch covers fewer than 2^31 16-byte vectors: whole rows at a time
    const int64_t rows_per = ((1ll << 31) - 1024) / nvec;
    for (int64_t r0 = 0; r0 < rows; r0 += rows_per) {
        const int64_t nr = rows - r0 < rows_per ? rows - r0 : rows_per;
        const unsigned total = (unsigned)(nr * nvec);
        hipLaunchKernelGGL(mxfp4_kernel, dim3((total + 1023) / 1024), dim3(256), 0, st,
                           static_cast<const uint4*>(x) + r0 * (ld_x / 8), ld_x / 8, (unsigned)nvec, total,
                           static_cast<u32*>(q) + r0 * (ld_q / 4), ld_q / 4,
                           static_cast<uint8_t*>(scales) + r0 * ld_scales, ld_scales);
    }
    return check_launch("quant_mxfp4");
}
