// 128x128 block quantisation (weights), 1x128 group quantisation (activations)
// and the block dequantiser.  All three are HBM-bound streaming kernels.
#include "cfp8_common.h"

namespace cfp8 {

// ---------------------------------------------------------------------------
// 128x128 blocks.  One 256-thread workgroup per tile; thread (rg, cv) holds the
// 8 consecutive rows rg*8.. and the 8 consecutive columns cv*8.. of the tile as
// packed bf16 (32 VGPRs), so the tile is read from HBM once.  For every row,
// 16 lanes read 256 contiguous bytes.
// Plain output: 8-byte stores, 128 contiguous bytes per row.
// Transposed output ([cols, rows], the K-major operand of the block GEMM): the
// fp8 tile is turned in LDS (128 x 144 bytes) and leaves as 16-byte stores,
// 128 contiguous bytes per output row.
// ---------------------------------------------------------------------------
constexpr int kTStride = 144;  // bytes per LDS row of the transposed tile (16-byte aligned)

template <bool TRANSPOSE>
__global__ __launch_bounds__(256) void block128_kernel(const uint16_t* __restrict__ x, int64_t rows, int64_t cols,
                                                       uint8_t* __restrict__ q, float* __restrict__ scales,
                                                       int tiles_r, int tiles_c) {
    __shared__ u32 red[4];
    __shared__ __attribute__((aligned(16))) uint8_t tile[TRANSPOSE ? 128 * kTStride : 16];
    const int t = threadIdx.x;
    const int cv = t & 15, rg = t >> 4;
    const int64_t b = blockIdx.z;
    const int64_t r0 = (int64_t)blockIdx.y * 128, c0 = (int64_t)blockIdx.x * 128;
    const uint16_t* xb = x + b * rows * cols;
    const int64_t col = c0 + cv * 8;
    const bool col_ok = col < cols;  // cols % 8 == 0: a vector is inside or outside as a whole
    uint4 v[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const int64_t r = r0 + rg * 8 + i;
        v[i] = (col_ok && r < rows) ? ld16<true>(reinterpret_cast<const uint4*>(xb + r * cols + col)) : make_uint4(0, 0, 0, 0);
    }
    u32 m = 0;
#pragma unroll
    for (int i = 0; i < 8; ++i) m = absmax8(m, v[i]);
    m = wave_max(pk_fold(m));
    if ((t & 63) == 0) red[t >> 6] = m;
    __syncthreads();
    const float amax = amax_from_bits(umax(umax(red[0], red[1]), umax(red[2], red[3])));
    const float scale = scale_from_amax(amax);
    if (t == 0) scales[(b * tiles_r + blockIdx.y) * tiles_c + blockIdx.x] = scale;
    const Divider d(scale);
    if (!TRANSPOSE) {
        uint8_t* qb = q + b * rows * cols;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int64_t r = r0 + rg * 8 + i;
            if (col_ok && r < rows) st8<true>(reinterpret_cast<uint2*>(qb + r * cols + col), cast8(v[i], d));
        }
    } else {
        // bytes[i] = row i, 8 columns; regroup to 8 rows of one column (8 bytes) per LDS store
        uint2 bytes[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) bytes[i] = cast8(v[i], d);
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            u32 lo = 0, hi = 0;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const u32 wlo = j < 4 ? bytes[i].x : bytes[i].y;
                const u32 whi = j < 4 ? bytes[i + 4].x : bytes[i + 4].y;
                lo |= ((wlo >> (8 * (j & 3))) & 0xFFu) << (8 * i);
                hi |= ((whi >> (8 * (j & 3))) & 0xFFu) << (8 * i);
            }
            *reinterpret_cast<uint2*>(&tile[(cv * 8 + j) * kTStride + rg * 8]) = make_uint2(lo, hi);
        }
        __syncthreads();
        uint8_t* qb = q + b * rows * cols;  // [cols, rows]
        const int chunk = t & 7;            // 16 rows of the tile per chunk
#pragma unroll
        for (int p = 0; p < 4; ++p) {
            const int c = (t >> 3) + 32 * p;
            const int64_t oc = c0 + c, orow = r0 + chunk * 16;
            if (oc < cols && orow < rows)  // rows % 16 == 0: a chunk is inside or outside as a whole
                st16<true>(reinterpret_cast<uint4*>(qb + oc * rows + orow),
                           *reinterpret_cast<const uint4*>(&tile[c * kTStride + chunk * 16]));
        }
    }
}

// ---------------------------------------------------------------------------
// 1x128 groups.  16 lanes own one group (one 16-byte vector each), the max runs
// over the 16-lane DPP row.  Every thread handles 4 groups of 4 consecutive
// group-rows so that four loads are in flight per lane.
// ---------------------------------------------------------------------------
// With GATHER, output row r quantises input row src_rows[r] (a zero row where that is negative): the token
// gather in front of the grouped GEMM and the quantiser in one pass, without the gathered bf16 matrix.
// Groups are numbered row-major (row * ngroups + column) in 32 bits; a thread divides once and steps
// through its four consecutive groups.  Every load is unconditional on a clamped address (what must read
// as zero is cleared afterwards), so all four are in flight before the first is used.
template <int MODE, bool GATHER = false>
__global__ __launch_bounds__(256) void group128_kernel(const uint4* __restrict__ x, int nvec,
                                                       u32 ngroups, int64_t ldx, uint2* __restrict__ q, int64_t ldq,
                                                       float* __restrict__ scales, u32 rows, u32 total_groups,
                                                       const int32_t* __restrict__ src_rows = nullptr) {
    const int sub = threadIdx.x & 15;
    const u32 g0 = (blockIdx.x * 16u + (threadIdx.x >> 4)) * 4u;
    uint4 v[4];
    u32 row[4], gcol[4];
    bool ok[4];
    {
        u32 r = g0 / ngroups, c = g0 - r * ngroups;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            row[i] = r;
            gcol[i] = c;
            if (++c == ngroups) c = 0, ++r;
        }
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int vec = (int)gcol[i] * 16 + sub;
        ok[i] = g0 + i < total_groups && vec < nvec;
        const u32 rc = row[i] < rows ? row[i] : rows - 1;
        const int vc = vec < nvec ? vec : nvec - 1;
        if (GATHER) {
            const int32_t src = src_rows[rc];
            ok[i] = ok[i] && src >= 0;
            // tokens are read several times (once per expert they go to): leave them in the caches
            v[i] = ld16<false>(x + (int64_t)(src >= 0 ? src : 0) * ldx + vc);
        } else {
            v[i] = ld16<true>(x + (int64_t)rc * ldx + vc);
        }
    }
#pragma unroll
    for (int i = 0; i < 4; ++i)
        if (!ok[i]) v[i] = make_uint4(0, 0, 0, 0);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const u32 m = row16_max(pk_fold(absmax8(0u, v[i])));
        const float amax = amax_from_bits(m);
        uint2 out;
        float scale;
        if (MODE == CFP8_GROUP_MODE_DIV) {
            scale = scale_from_amax(amax);
            const Divider d(scale);
            out = cast8(v[i], d);
        } else {
            // x * (448 / clamp(amax, 1e-4)) as torch evaluates `448.0 / tensor`:
            // reciprocal first, then times 448.  No clamp before the cast: the product
            // exceeds 448 by at most a few fp32 roundings, far below the NaN threshold 464
            if (amax != amax) {
                scale = __uint_as_float(kCanonNaN);
                out = make_uint2(0x7F7F7F7Fu, 0x7F7F7F7Fu);
            } else {
                const float a = fmaxf(amax, 1e-4f);
                const float mul = (1.0f / a) * kE4M3Max;
                scale = a / kE4M3Max;
                const u32 w[4] = {v[i].x, v[i].y, v[i].z, v[i].w};
                u32 o[2];
#pragma unroll
                for (int k = 0; k < 2; ++k) {
                    u32 p = cvt2<false>(bf16_lo(w[2 * k]) * mul, bf16_hi(w[2 * k]) * mul, 0u);
                    o[k] = cvt2<true>(bf16_lo(w[2 * k + 1]) * mul, bf16_hi(w[2 * k + 1]) * mul, p);
                }
                out = make_uint2(o[0], o[1]);
            }
        }
        const int vec = (int)gcol[i] * 16 + sub;
        if (g0 + i < total_groups && vec < nvec) q[(int64_t)row[i] * ldq + vec] = out;
        if (sub == 0 && g0 + i < total_groups) scales[g0 + i] = scale;
    }
}

// ---------------------------------------------------------------------------
// block dequantiser: y[i, j] = fp8[i, j] * s[i / 128, j / 128]
// A thread owns one 8-column vector of four consecutive rows (one scale, four loads in flight); the block is
// BX vectors wide and 256 / BX row quads high, BX chosen by the host to fit the row length, so no index is divided.
// ---------------------------------------------------------------------------
template <bool F32>
__global__ __launch_bounds__(256) void dequant_block128_kernel(const uint8_t* __restrict__ q,
                                                               const float* __restrict__ s, int64_t rows,
                                                               int64_t cols, int nvec_row, int tiles_c, void* __restrict__ y) {
    const int cv = blockIdx.x * blockDim.x + threadIdx.x;
    if (cv >= nvec_row) return;
    // (one pass of this loop unless the matrix has more row quads than the grid's y extent can hold)
    for (int64_t r0 = ((int64_t)blockIdx.y * blockDim.y + threadIdx.y) * 4; r0 < rows;
         r0 += (int64_t)gridDim.y * blockDim.y * 4) {
        const float sc = s[(r0 >> 7) * tiles_c + (cv >> 4)];
        uint2 w[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const int64_t r = r0 + k < rows ? r0 + k : rows - 1;
            const u32x2 t = __builtin_nontemporal_load(reinterpret_cast<const u32x2*>(q + r * cols + (int64_t)cv * 8));
            w[k] = make_uint2(t[0], t[1]);
        }
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            if (r0 + k >= rows) break;
            float f[8];
            f32x2 p;
            p = __builtin_amdgcn_cvt_pk_f32_fp8((int)w[k].x, false); f[0] = p[0]; f[1] = p[1];
            p = __builtin_amdgcn_cvt_pk_f32_fp8((int)w[k].x, true);  f[2] = p[0]; f[3] = p[1];
            p = __builtin_amdgcn_cvt_pk_f32_fp8((int)w[k].y, false); f[4] = p[0]; f[5] = p[1];
            p = __builtin_amdgcn_cvt_pk_f32_fp8((int)w[k].y, true);  f[6] = p[0]; f[7] = p[1];
#pragma unroll
            for (int i = 0; i < 8; ++i) f[i] *= sc;
            const int64_t at = (r0 + k) * cols + (int64_t)cv * 8;
            if (F32) {
                uint4* o = reinterpret_cast<uint4*>(static_cast<float*>(y) + at);
                st16<true>(o, make_uint4(__float_as_uint(f[0]), __float_as_uint(f[1]), __float_as_uint(f[2]), __float_as_uint(f[3])));
                st16<true>(o + 1, make_uint4(__float_as_uint(f[4]), __float_as_uint(f[5]), __float_as_uint(f[6]), __float_as_uint(f[7])));
            } else {
                st16<true>(reinterpret_cast<uint4*>(static_cast<uint16_t*>(y) + at),
                           make_uint4(pack_bf16x2(f[0], f[1]), pack_bf16x2(f[2], f[3]), pack_bf16x2(f[4], f[5]), pack_bf16x2(f[6], f[7])));
            }
        }
    }
}

// ---------------------------------------------------------------------------
// 1x128 group dequantiser: y[i, j] = fp8[i, j] * s[i, j / 128], the inverse of group128_kernel.  The thread layout of
// the block dequantiser (one 8-column vector of four consecutive rows per thread), with a scale per row and group.
// E8M0: the scales are one exponent byte per group, value 2^(byte - 127) formed as the fp32 bit pattern byte << 23
// (byte 0 gives +0 and byte 255 +infinity, as that shift does).
// ---------------------------------------------------------------------------
template <bool F32, bool E8M0>
__global__ __launch_bounds__(256) void dequant_group128_kernel(const uint8_t* __restrict__ q, int64_t ld_q,
                                                               const void* __restrict__ s, int64_t ld_s, int64_t rows,
                                                               int nvec_row, void* __restrict__ y, int64_t ld_y) {
    const int cv = blockIdx.x * blockDim.x + threadIdx.x;
    if (cv >= nvec_row) return;
    for (int64_t r0 = ((int64_t)blockIdx.y * blockDim.y + threadIdx.y) * 4; r0 < rows;
         r0 += (int64_t)gridDim.y * blockDim.y * 4) {
        uint2 w[4];
        float sc[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const int64_t r = r0 + k < rows ? r0 + k : rows - 1;
            const u32x2 t = __builtin_nontemporal_load(reinterpret_cast<const u32x2*>(q + r * ld_q + (int64_t)cv * 8));
            w[k] = make_uint2(t[0], t[1]);
            if (E8M0) sc[k] = __uint_as_float((u32) static_cast<const uint8_t*>(s)[r * ld_s + (cv >> 4)] << 23);
            else sc[k] = static_cast<const float*>(s)[r * ld_s + (cv >> 4)];
        }
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            if (r0 + k >= rows) break;
            float f[8];
            f32x2 p;
            p = __builtin_amdgcn_cvt_pk_f32_fp8((int)w[k].x, false); f[0] = p[0]; f[1] = p[1];
            p = __builtin_amdgcn_cvt_pk_f32_fp8((int)w[k].x, true);  f[2] = p[0]; f[3] = p[1];
            p = __builtin_amdgcn_cvt_pk_f32_fp8((int)w[k].y, false); f[4] = p[0]; f[5] = p[1];
            p = __builtin_amdgcn_cvt_pk_f32_fp8((int)w[k].y, true);  f[6] = p[0]; f[7] = p[1];
#pragma unroll
            for (int i = 0; i < 8; ++i) f[i] *= sc[k];
            const int64_t at = (r0 + k) * ld_y + (int64_t)cv * 8;
            if (F32) {
                uint4* o = reinterpret_cast<uint4*>(static_cast<float*>(y) + at);
                st16<true>(o, make_uint4(__float_as_uint(f[0]), __float_as_uint(f[1]), __float_as_uint(f[2]), __float_as_uint(f[3])));
                st16<true>(o + 1, make_uint4(__float_as_uint(f[4]), __float_as_uint(f[5]), __float_as_uint(f[6]), __float_as_uint(f[7])));
            } else {
                st16<true>(reinterpret_cast<uint4*>(static_cast<uint16_t*>(y) + at),
                           make_uint4(pack_bf16x2(f[0], f[1]), pack_bf16x2(f[2], f[3]), pack_bf16x2(f[4], f[5]), pack_bf16x2(f[6], f[7])));
            }
        }
    }
}

// SwiGLU fused with the 1x128 quantiser: h = bf16(bf16(silu(g)) * u) is formed in registers from the
// two bf16 GEMM outputs and quantised like group128_kernel<DIV> does; h never exists in memory.
// The two roundings to bf16 are those of the unfused torch chain act(g) * u on bf16 tensors (swiglu_quad).

__global__ __launch_bounds__(256) void swiglu_group128_kernel(const uint4* __restrict__ gate, int64_t ldg,
                                                              const uint4* __restrict__ up, int64_t ldu, int nvec,
                                                              u32 ngroups, uint2* __restrict__ q, int64_t ldq,
                                                              float* __restrict__ scales, u32 rows, u32 total_groups) {
    const int sub = threadIdx.x & 15;
    const u32 g0 = (blockIdx.x * 16u + (threadIdx.x >> 4)) * 2u;
    uint4 vg[2], vu[2];
    u32 row[2], gcol[2];
    row[0] = g0 / ngroups;
    gcol[0] = g0 - row[0] * ngroups;
    gcol[1] = gcol[0] + 1 == ngroups ? 0 : gcol[0] + 1;
    row[1] = gcol[1] == 0 ? row[0] + 1 : row[0];
    bool ok[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int vec = (int)gcol[i] * 16 + sub;
        ok[i] = g0 + i < total_groups && vec < nvec;
        const int64_t rc = row[i] < rows ? row[i] : rows - 1;  // unconditional loads on clamped addresses
        const int vc = vec < nvec ? vec : nvec - 1;
        vg[i] = ld16<true>(gate + rc * ldg + vc);
        vu[i] = ld16<true>(up + rc * ldu + vc);
    }
#pragma unroll
    for (int i = 0; i < 2; ++i)
        if (!ok[i]) vg[i] = vu[i] = make_uint4(0, 0, 0, 0);
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        uint4 h;
        swiglu_quad(vg[i].x, vg[i].y, vu[i].x, vu[i].y, h.x, h.y);
        swiglu_quad(vg[i].z, vg[i].w, vu[i].z, vu[i].w, h.z, h.w);
        const u32 m = row16_max(pk_fold(absmax8(0u, h)));
        const float scale = scale_from_amax(amax_from_bits(m));
        const Divider d(scale);
        const uint2 out = cast8(h, d);
        if (ok[i]) st8<false>(q + (int64_t)row[i] * ldq + gcol[i] * 16 + sub, out);
        if (sub == 0 && g0 + i < total_groups) scales[g0 + i] = scale;
    }
}

// The gather-and-quantise pass turned round for a token matrix whose rows each feed several rows of the grouped
// matrix (top-k routing): a token's 1x128 groups are quantised once and the eight bytes a lane holds are stored to
// every row the token goes to, instead of reading and quantising the token once per destination.  The first
// blocks_tokens workgroups take the tokens (16 lanes per group of 128 columns, four groups per lane set as in
// group128_kernel), the rest write the rows of padding: zero bytes and the scale of an all-zero group.
__global__ __launch_bounds__(256) void scatter_group128_kernel(const uint4* __restrict__ x, int nvec, u32 ngroups, int64_t ldx,
                                                               u32 tokens, u32 token_groups, const int32_t* __restrict__ row_map,
                                                               int topk, const int32_t* __restrict__ src_rows, u32 rows_out,
                                                               uint2* __restrict__ q, int64_t ldq, float* __restrict__ scales,
                                                               u32 blocks_tokens) {
    const int sub = threadIdx.x & 15;
    if (blockIdx.x >= blocks_tokens) {
        // padding: one lane set per (row, group), four at a time
        const u32 total = rows_out * ngroups;
        const u32 g0 = ((blockIdx.x - blocks_tokens) * 16u + (threadIdx.x >> 4)) * 4u;
        u32 r = g0 / ngroups, c = g0 - r * ngroups;
        const float floor_scale = scale_from_amax(0.0f);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            if (g0 + i < total && src_rows[r] < 0) {
                const int vec = (int)c * 16 + sub;
                if (vec < nvec) q[(int64_t)r * ldq + vec] = make_uint2(0u, 0u);
                if (sub == 0) scales[(int64_t)r * ngroups + c] = floor_scale;
            }
            if (++c == ngroups) c = 0, ++r;
        }
        return;
    }
    const u32 g0 = (blockIdx.x * 16u + (threadIdx.x >> 4)) * 4u;
    uint4 v[4];
    u32 tok[4], gcol[4];
    bool ok[4];
    {
        u32 r = g0 / ngroups, c = g0 - r * ngroups;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            tok[i] = r;
            gcol[i] = c;
            if (++c == ngroups) c = 0, ++r;
        }
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int vec = (int)gcol[i] * 16 + sub;
        ok[i] = g0 + i < token_groups && vec < nvec;
        const u32 rc = tok[i] < tokens ? tok[i] : tokens - 1;
        const int vc = vec < nvec ? vec : nvec - 1;
        v[i] = ld16<true>(x + (int64_t)rc * ldx + vc);  // read once: streaming
    }
#pragma unroll
    for (int i = 0; i < 4; ++i)
        if (!ok[i]) v[i] = make_uint4(0, 0, 0, 0);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const u32 m = row16_max(pk_fold(absmax8(0u, v[i])));
        const float scale = scale_from_amax(amax_from_bits(m));
        const Divider d(scale);
        const uint2 out = cast8(v[i], d);
        if (g0 + i >= token_groups) continue;
        const int32_t* const dst = row_map + (int64_t)tok[i] * topk;
        for (int k0 = 0; k0 < topk; k0 += 8) {
            int32_t r[8];
#pragma unroll
            for (int k = 0; k < 8; ++k) r[k] = k0 + k < topk ? dst[k0 + k] : -1;
#pragma unroll
            for (int k = 0; k < 8; ++k) {
                if (r[k] < 0 || (u32)r[k] >= rows_out) continue;
                if (ok[i]) st8<false>(q + (int64_t)r[k] * ldq + gcol[i] * 16 + sub, out);
                if (sub == 0) scales[(int64_t)r[k] * ngroups + gcol[i]] = scale;
            }
        }
    }
}

// Groups are numbered in 32 bits, and a block's first group index must not wrap.
constexpr int64_t kMaxGroups = 0xFFFFFF00ll;

int launch_quant_group128(const void* x, int64_t rows, int64_t cols, int64_t ld_x, void* q, int64_t ld_q,
                          float* scales, int mode, hipStream_t st) {
    const int64_t ngroups = (cols + 127) / 128;
    const int64_t total = rows * ngroups;
    if (total > kMaxGroups) return set_error(CFP8_EINVAL, "quant_group128: too many groups for one launch");
    const unsigned blocks = (unsigned)((total + 63) / 64);
    const uint4* xv = static_cast<const uint4*>(x);
    uint2* qv = static_cast<uint2*>(q);
    if (mode == CFP8_GROUP_MODE_DIV)
        hipLaunchKernelGGL(group128_kernel<CFP8_GROUP_MODE_DIV>, dim3(blocks), dim3(256), 0, st, xv, (int)(cols / 8),
                           (u32)ngroups, ld_x / 8, qv, ld_q / 8, scales, (u32)rows, (u32)total, nullptr);
    else
        hipLaunchKernelGGL(group128_kernel<CFP8_GROUP_MODE_DEEPEP>, dim3(blocks), dim3(256), 0, st, xv, (int)(cols / 8),
                           (u32)ngroups, ld_x / 8, qv, ld_q / 8, scales, (u32)rows, (u32)total, nullptr);
    return check_launch("quant_group128");
}

}  // namespace cfp8

extern "C" int cfp8_quant_block128(const void* x, int64_t batch, int64_t rows, int64_t cols, void* q,
                                   float* scales, int transpose_out, void* stream) {
    using namespace cfp8;
    if (batch < 0 || rows < 0 || cols < 0) return set_error(CFP8_EINVAL, "quant_block128: negative shape");
    if (batch == 0 || rows == 0 || cols == 0) return CFP8_OK;
    if (!x || !q || !scales) return set_error(CFP8_EINVAL, "quant_block128: null pointer");
    if (cols % 8) return set_error(CFP8_EINVAL, "quant_block128: cols=%lld must be a multiple of 8", (long long)cols);
    if (transpose_out && rows % 16) return set_error(CFP8_EINVAL, "quant_block128: rows=%lld must be a multiple of 16 for the transposed output", (long long)rows);
    if (!aligned16(x) || (reinterpret_cast<uintptr_t>(q) & (transpose_out ? 15u : 7u)))
        return set_error(CFP8_EINVAL, "quant_block128: misaligned pointer");
    const int64_t tr = (rows + 127) / 128, tc = (cols + 127) / 128;
    if (tr > 65535 || batch > 65535 || tc > 0x7FFFFFFFll) return set_error(CFP8_EINVAL, "quant_block128: shape exceeds the grid limits");
    if (int rc = check_device()) return rc;
    hipStream_t st = static_cast<hipStream_t>(stream);
    dim3 grid((unsigned)tc, (unsigned)tr, (unsigned)batch);
    if (transpose_out)
        hipLaunchKernelGGL(block128_kernel<true>, grid, dim3(256), 0, st, static_cast<const uint16_t*>(x), rows, cols,
                           static_cast<uint8_t*>(q), scales, (int)tr, (int)tc);
    else
        hipLaunchKernelGGL(block128_kernel<false>, grid, dim3(256), 0, st, static_cast<const uint16_t*>(x), rows, cols,
                           static_cast<uint8_t*>(q), scales, (int)tr, (int)tc);
    return check_launch("quant_block128");
}

extern "C" int cfp8_quant_group128(const void* x, int64_t rows, int64_t cols, int64_t ld_x, void* q,
                                   int64_t ld_q, float* scales, int mode, void* stream) {
    using namespace cfp8;
    if (rows < 0 || cols < 0) return set_error(CFP8_EINVAL, "quant_group128: negative shape");
    if (rows == 0 || cols == 0) return CFP8_OK;
    if (!x || !q || !scales) return set_error(CFP8_EINVAL, "quant_group128: null pointer");
    if (mode != CFP8_GROUP_MODE_DIV && mode != CFP8_GROUP_MODE_DEEPEP) return set_error(CFP8_EINVAL, "quant_group128: unknown mode %d", mode);
    if (cols % 8 || ld_x % 8 || ld_q % 8 || ld_x < cols || ld_q < cols)
        return set_error(CFP8_EINVAL, "quant_group128: cols=%lld ld_x=%lld ld_q=%lld must be multiples of 8 with ld >= cols",
                         (long long)cols, (long long)ld_x, (long long)ld_q);
    if (!aligned16(x) || (reinterpret_cast<uintptr_t>(q) & 7u)) return set_error(CFP8_EINVAL, "quant_group128: misaligned pointer");
    if (int rc = check_device()) return rc;
    return launch_quant_group128(x, rows, cols, ld_x, q, ld_q, scales, mode, static_cast<hipStream_t>(stream));
}

extern "C" int cfp8_gather_quant_group128(const void* x, int64_t ld_x, const int32_t* src_rows, int64_t rows_out, int64_t cols,
                                          void* q, int64_t ld_q, float* scales, void* stream) {
    using namespace cfp8;
    if (rows_out < 0 || cols < 0) return set_error(CFP8_EINVAL, "gather_quant_group128: negative shape");
    if (rows_out == 0 || cols == 0) return CFP8_OK;
    if (!x || !src_rows || !q || !scales) return set_error(CFP8_EINVAL, "gather_quant_group128: null pointer");
    if (cols % 8 || ld_x % 8 || ld_q % 8 || ld_x < cols || ld_q < cols)
        return set_error(CFP8_EINVAL, "gather_quant_group128: cols=%lld ld_x=%lld ld_q=%lld must be multiples of 8 with ld >= cols",
                         (long long)cols, (long long)ld_x, (long long)ld_q);
    if (!aligned16(x) || (reinterpret_cast<uintptr_t>(q) & 7u)) return set_error(CFP8_EINVAL, "gather_quant_group128: misaligned pointer");
    const int64_t ngroups = (cols + 127) / 128, total = rows_out * ngroups;
    if (total > kMaxGroups) return set_error(CFP8_EINVAL, "gather_quant_group128: too many groups for one launch");
    if (int rc = check_device()) return rc;
    hipLaunchKernelGGL((group128_kernel<CFP8_GROUP_MODE_DIV, true>), dim3((unsigned)((total + 63) / 64)), dim3(256), 0,
                       static_cast<hipStream_t>(stream), static_cast<const uint4*>(x), (int)(cols / 8), (u32)ngroups, ld_x / 8,
                       static_cast<uint2*>(q), ld_q / 8, scales, (u32)rows_out, (u32)total, src_rows);
    return check_launch("gather_quant_group128");
}

extern "C" int cfp8_scatter_quant_group128(const void* x, int64_t ld_x, int64_t tokens, int64_t cols, const int32_t* row_map,
                                           int64_t topk, const int32_t* src_rows, int64_t rows_out, void* q, int64_t ld_q,
                                           float* scales, void* stream) {
    using namespace cfp8;
    if (tokens < 0 || cols < 0 || rows_out < 0 || topk < 0) return set_error(CFP8_EINVAL, "scatter_quant_group128: negative shape");
    if (rows_out == 0 || cols == 0) return CFP8_OK;
    if (!src_rows || !q || !scales || (tokens > 0 && topk > 0 && (!x || !row_map)))
        return set_error(CFP8_EINVAL, "scatter_quant_group128: null pointer");
    if (topk > 64) return set_error(CFP8_EINVAL, "scatter_quant_group128: topk=%lld is out of range (0..64)", (long long)topk);
    if (cols % 8 || ld_x % 8 || ld_q % 8 || ld_x < cols || ld_q < cols)
        return set_error(CFP8_EINVAL, "scatter_quant_group128: cols=%lld ld_x=%lld ld_q=%lld must be multiples of 8 with ld >= cols",
                         (long long)cols, (long long)ld_x, (long long)ld_q);
    if ((x && !aligned16(x)) || (reinterpret_cast<uintptr_t>(q) & 7u)) return set_error(CFP8_EINVAL, "scatter_quant_group128: misaligned pointer");
    const int64_t ngroups = (cols + 127) / 128;
    const int64_t token_groups = (topk > 0 ? tokens : 0) * ngroups, row_groups = rows_out * ngroups;
    if (token_groups > kMaxGroups || row_groups > kMaxGroups || tokens > 0x7FFFFFFFll || rows_out > 0x7FFFFFFFll)
        return set_error(CFP8_EINVAL, "scatter_quant_group128: too many groups for one launch");
    const int64_t blocks_tokens = (token_groups + 63) / 64, blocks_rows = (row_groups + 63) / 64;
    if (blocks_tokens + blocks_rows > 0x7FFFFFFFll) return set_error(CFP8_EINVAL, "scatter_quant_group128: too many groups for one launch");
    if (int rc = check_device()) return rc;
    hipLaunchKernelGGL(scatter_group128_kernel, dim3((unsigned)(blocks_tokens + blocks_rows)), dim3(256), 0, static_cast<hipStream_t>(stream),
                       static_cast<const uint4*>(x), (int)(cols / 8), (u32)ngroups, ld_x / 8, (u32)tokens, (u32)token_groups, row_map, (int)topk,
                       src_rows, (u32)rows_out, static_cast<uint2*>(q), ld_q / 8, scales, (u32)blocks_tokens);
    return check_launch("scatter_quant_group128");
}

extern "C" int cfp8_swiglu_quant_group128(const void* gate, int64_t ld_gate, const void* up, int64_t ld_up, int64_t rows,
                                          int64_t cols, void* q, int64_t ld_q, float* scales, void* stream) {
    using namespace cfp8;
    if (rows < 0 || cols < 0) return set_error(CFP8_EINVAL, "swiglu_quant_group128: negative shape");
    if (rows == 0 || cols == 0) return CFP8_OK;
    if (!gate || !up || !q || !scales) return set_error(CFP8_EINVAL, "swiglu_quant_group128: null pointer");
    if (cols % 8 || ld_gate % 8 || ld_up % 8 || ld_q % 8 || ld_gate < cols || ld_up < cols || ld_q < cols)
        return set_error(CFP8_EINVAL, "swiglu_quant_group128: cols=%lld ld_gate=%lld ld_up=%lld ld_q=%lld must be multiples of 8 with ld >= cols",
                         (long long)cols, (long long)ld_gate, (long long)ld_up, (long long)ld_q);
    if (!aligned16(gate) || !aligned16(up) || (reinterpret_cast<uintptr_t>(q) & 7u))
        return set_error(CFP8_EINVAL, "swiglu_quant_group128: misaligned pointer");
    const int64_t ngroups = (cols + 127) / 128, total = rows * ngroups;
    if (total > kMaxGroups) return set_error(CFP8_EINVAL, "swiglu_quant_group128: too many groups for one launch");
    if (int rc = check_device()) return rc;
    hipLaunchKernelGGL(swiglu_group128_kernel, dim3((unsigned)((total + 31) / 32)), dim3(256), 0, static_cast<hipStream_t>(stream),
                       static_cast<const uint4*>(gate), ld_gate / 8, static_cast<const uint4*>(up), ld_up / 8, (int)(cols / 8),
                       (u32)ngroups, static_cast<uint2*>(q), ld_q / 8, scales, (u32)rows, (u32)total);
    return check_launch("swiglu_quant_group128");
}

extern "C" int cfp8_dequant_block128(const void* q, const float* scales, int64_t rows, int64_t cols, void* y,
                                     int out_dtype, void* stream) {
    using namespace cfp8;
    if (rows < 0 || cols < 0) return set_error(CFP8_EINVAL, "dequant_block128: negative shape");
    if (rows == 0 || cols == 0) return CFP8_OK;
    if (!q || !scales || !y) return set_error(CFP8_EINVAL, "dequant_block128: null pointer");
    if (cols % 8) return set_error(CFP8_EINVAL, "dequant_block128: cols=%lld must be a multiple of 8", (long long)cols);
    if ((reinterpret_cast<uintptr_t>(q) & 7u) || !aligned16(y)) return set_error(CFP8_EINVAL, "dequant_block128: misaligned pointer");
    if (out_dtype != CFP8_OUT_BF16 && out_dtype != CFP8_OUT_F32) return set_error(CFP8_EINVAL, "dequant_block128: unknown out_dtype %d", out_dtype);
    const int64_t nvec_row = cols / 8;
    const int bx = nvec_row > 128 ? 256 : nvec_row > 64 ? 128 : 64, by = 256 / bx;
    int64_t gx = (nvec_row + bx - 1) / bx, gy = (rows + 4 * by - 1) / (4 * by);
    if (gx > 0x7FFFFFFFll) return set_error(CFP8_EINVAL, "dequant_block128: shape exceeds the grid limits");
    if (gy > 65535) gy = 65535;  // the kernel strides over the remaining row quads
    if (int rc = check_device()) return rc;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const int tc = (int)((cols + 127) / 128);
    const dim3 grid((unsigned)gx, (unsigned)gy), block(bx, by);
    if (out_dtype == CFP8_OUT_F32)
        hipLaunchKernelGGL(dequant_block128_kernel<true>, grid, block, 0, st, static_cast<const uint8_t*>(q), scales, rows, cols,
                           (int)nvec_row, tc, y);
    else
        hipLaunchKernelGGL(dequant_block128_kernel<false>, grid, block, 0, st, static_cast<const uint8_t*>(q), scales, rows, cols,
                           (int)nvec_row, tc, y);
    return check_launch("dequant_block128");
}

extern "C" int cfp8_dequant_group128(const void* q, int64_t ld_q, const void* scales, int64_t ld_scales, int scale_kind,
                                     int64_t rows, int64_t cols, void* y, int64_t ld_y, int out_dtype, void* stream) {
    using namespace cfp8;
    if (rows < 0 || cols < 0) return set_error(CFP8_EINVAL, "dequant_group128: negative shape");
    if (rows == 0 || cols == 0) return CFP8_OK;
    if (!q || !scales || !y) return set_error(CFP8_EINVAL, "dequant_group128: null pointer");
    if (out_dtype != CFP8_OUT_BF16 && out_dtype != CFP8_OUT_F32) return set_error(CFP8_EINVAL, "dequant_group128: unknown out_dtype %d", out_dtype);
    if (scale_kind != CFP8_SCALE_F32 && scale_kind != CFP8_SCALE_E8M0) return set_error(CFP8_EINVAL, "dequant_group128: unknown scale_kind %d", scale_kind);
    const int64_t ngroups = (cols + 127) / 128;
    if (cols % 8 || ld_q % 8 || ld_q < cols || ld_y < cols || ld_y % (out_dtype == CFP8_OUT_F32 ? 4 : 8) || ld_scales < ngroups)
        return set_error(CFP8_EINVAL, "dequant_group128: cols=%lld ld_q=%lld ld_y=%lld ld_scales=%lld: cols and ld_q must be multiples of 8, "
                         "rows of y 16-byte aligned, and every pitch at least its row", (long long)cols, (long long)ld_q, (long long)ld_y, (long long)ld_scales);
    if ((reinterpret_cast<uintptr_t>(q) & 7u) || !aligned16(y) || (scale_kind == CFP8_SCALE_F32 && (reinterpret_cast<uintptr_t>(scales) & 3u)))
        return set_error(CFP8_EINVAL, "dequant_group128: misaligned pointer");
    const int64_t nvec_row = cols / 8;
    const int bx = nvec_row > 128 ? 256 : nvec_row > 64 ? 128 : 64, by = 256 / bx;
    int64_t gx = (nvec_row + bx - 1) / bx, gy = (rows + 4 * by - 1) / (4 * by);
    if (gx > 0x7FFFFFFFll) return set_error(CFP8_EINVAL, "dequant_group128: shape exceeds the grid limits");
    if (gy > 65535) gy = 65535;  // the kernel strides over the remaining row quads
    if (int rc = check_device()) return rc;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const dim3 grid((unsigned)gx, (unsigned)gy), block(bx, by);
    const uint8_t* qp = static_cast<const uint8_t*>(q);
    const bool f32 = out_dtype == CFP8_OUT_F32, e8 = scale_kind == CFP8_SCALE_E8M0;
    if (f32 && e8) hipLaunchKernelGGL((dequant_group128_kernel<true, true>), grid, block, 0, st, qp, ld_q, scales, ld_scales, rows, (int)nvec_row, y, ld_y);
    else if (f32) hipLaunchKernelGGL((dequant_group128_kernel<true, false>), grid, block, 0, st, qp, ld_q, scales, ld_scales, rows, (int)nvec_row, y, ld_y);
    else if (e8) hipLaunchKernelGGL((dequant_group128_kernel<false, true>), grid, block, 0, st, qp, ld_q, scales, ld_scales, rows, (int)nvec_row, y, ld_y);
    else hipLaunchKernelGGL((dequant_group128_kernel<false, false>), grid, block, 0, st, qp, ld_q, scales, ld_scales, rows, (int)nvec_row, y, ld_y);
    return check_launch("dequant_group128");
}
