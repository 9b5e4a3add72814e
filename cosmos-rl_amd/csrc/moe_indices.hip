// Permutation indices for expert-grouped token layouts (the input side of the grouped GEMM).
//
// Tokens arrive grouped by (source rank, local expert); the grouped GEMM wants them grouped by
// expert, every group padded to a multiple of `alignment` rows.  Two launches on the caller's
// stream, no host round trip:
//   1. one workgroup scans the num_ranks * experts_per_rank counts: exclusive prefix sum (start
//      row of every (rank, expert) block), per-expert totals, padded sizes and their cumulative
//      ends;
//   2. one thread per output row finds its expert (binary search over the cumulative ends) and
//      its source rank (walk over at most num_ranks blocks) and writes the source row, or -1
//      for a padding row.
// Integer work, launch-bound at real sizes (a few hundred counts, ~10^5 rows).
#include "cfp8_common.h"

namespace cfp8 {

__global__ __launch_bounds__(1024) void permute_scan_kernel(const int64_t* __restrict__ counts, int experts, int ranks,
                                                            int64_t alignment, int64_t* __restrict__ start_index,
                                                            int32_t* __restrict__ m_sizes, int32_t* __restrict__ m_offsets) {
    __shared__ int64_t part[1024];
    const int t = threadIdx.x, n = experts * ranks;
    // exclusive prefix sum over the counts, rank-major: thread t owns a contiguous slice
    const int per = (n + 1023) / 1024;
    const int lo = t * per < n ? t * per : n, hi = (t + 1) * per < n ? (t + 1) * per : n;
    int64_t sum = 0;
    for (int i = lo; i < hi; ++i) sum += counts[i];
    part[t] = sum;
    __syncthreads();
    for (int off = 1; off < 1024; off <<= 1) {
        const int64_t v = t >= off ? part[t - off] : 0;
        __syncthreads();
        part[t] += v;
        __syncthreads();
    }
    int64_t run = part[t] - sum;
    for (int i = lo; i < hi; ++i) {
        start_index[i] = run;
        run += counts[i];
    }
    __syncthreads();
    // padded group sizes, then their inclusive prefix sum
    const int eper = (experts + 1023) / 1024;
    const int elo = t * eper < experts ? t * eper : experts, ehi = (t + 1) * eper < experts ? (t + 1) * eper : experts;
    int64_t esum = 0;
    for (int e = elo; e < ehi; ++e) {
        int64_t tot = 0;
        for (int r = 0; r < ranks; ++r) tot += counts[r * experts + e];
        tot = tot < alignment ? alignment : tot;
        tot = (tot + alignment - 1) / alignment * alignment;
        m_sizes[e] = (int32_t)tot;
        esum += tot;
    }
    part[t] = esum;
    __syncthreads();
    for (int off = 1; off < 1024; off <<= 1) {
        const int64_t v = t >= off ? part[t - off] : 0;
        __syncthreads();
        part[t] += v;
        __syncthreads();
    }
    int64_t erun = part[t] - esum;
    for (int e = elo; e < ehi; ++e) {
        erun += m_sizes[e];
        m_offsets[e] = (int32_t)erun;
    }
}

__global__ __launch_bounds__(256) void permute_fill_kernel(const int64_t* __restrict__ counts,
                                                           const int64_t* __restrict__ start_index,
                                                           const int32_t* __restrict__ m_sizes,
                                                           const int32_t* __restrict__ m_offsets, int experts, int ranks,
                                                           int32_t* __restrict__ out, int64_t capacity) {
    const int64_t p = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (p >= capacity) return;
    // first expert whose cumulative end lies beyond p
    int lo = 0, hi = experts;
    while (lo < hi) {
        const int mid = (lo + hi) >> 1;
        if ((int64_t)m_offsets[mid] > p) hi = mid;
        else lo = mid + 1;
    }
    int32_t v = -1;
    if (lo < experts) {
        int64_t local = p - ((int64_t)m_offsets[lo] - m_sizes[lo]);
        for (int r = 0; r < ranks; ++r) {
            const int64_t len = counts[r * experts + lo];
            if (local < len) {
                v = (int32_t)(start_index[r * experts + lo] + local);
                break;
            }
            local -= len;
        }
    }
    out[p] = v;
}

// out[i, :] = idx[i] >= 0 ? x[idx[i], :] : 0, 16 bytes per lane
__global__ __launch_bounds__(256) void gather_rows_kernel(const uint4* __restrict__ x, int64_t ldx,
                                                          const int32_t* __restrict__ idx, int64_t rows_out, int nvec,
                                                          uint4* __restrict__ out, int64_t ldo) {
    const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= rows_out) return;
    const int lane = threadIdx.x & 63;
    const int32_t src = idx[row];
    for (int v = lane; v < nvec; v += 64) {
        const uint4 d = src >= 0 ? ld16<true>(x + (int64_t)src * ldx + v) : make_uint4(0, 0, 0, 0);
        st16<false>(out + row * ldo + v, d);
    }
}

// Weighted combine of expert outputs back into token order: one wavefront per (token, 64 x 16-byte
// chunk of the row).  Lane s first fetches slot s of the token's row map and weight; the slots are
// then walked in order with lane-to-scalar reads, so every load of the walk has a uniform base.
// A slot whose row is negative (or not below num_rows) contributes an exact zero.
//   STEPS: every product and every partial sum is rounded to bf16, the arithmetic of
//          `y.scatter_add_(0, idx, expert_out * weights[idx, top, None])` on bf16 tensors;
//   else:  fp32 accumulator acc = fma(row, weight, acc), rounded to bf16 once.
template <bool STEPS, bool W32>
__global__ __launch_bounds__(256) void combine_rows_kernel(const uint4* __restrict__ rows, int64_t ldr,
                                                           int64_t num_rows, const int32_t* __restrict__ row_map,
                                                           const void* __restrict__ weights, int64_t tokens, int topk, int nvec, int chunks,
                                                           uint4* __restrict__ out, int64_t ldo) {
    const int64_t unit = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (unit >= tokens * chunks) return;  // whole wavefronts leave
    const int64_t t = unit / chunks;
    const int lane = threadIdx.x & 63;
    const int v = (int)(unit - t * chunks) * 64 + lane;
    const int vv = v < nvec ? v : nvec - 1;  // lanes past the row end re-read its last vector and store nothing
    int32_t src = -1;
    float w = 0.f;
    if (lane < topk) {
        src = row_map[t * topk + lane];
        if (W32) w = static_cast<const float*>(weights)[t * topk + lane];
        else w = __uint_as_float((u32) static_cast<const uint16_t*>(weights)[t * topk + lane] << 16);
    }
    if (src < 0 || src >= num_rows) {  // padding slot, or an index no source row has
        src = -1;
        w = 0.f;
    }
    u32 y[4] = {0u, 0u, 0u, 0u};
    float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll 4
    for (int s = 0; s < topk; ++s) {
        const int32_t r = __builtin_amdgcn_readlane(src, s);
        const float ws = __uint_as_float(__builtin_amdgcn_readlane(__float_as_uint(w), s));
        uint4 d = ld16<true>(rows + (int64_t)(r < 0 ? 0 : r) * ldr + vv);
        if (r < 0) d = make_uint4(0, 0, 0, 0);
        const u32 x[4] = {d.x, d.y, d.z, d.w};
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const float lo = __uint_as_float(x[e] << 16), hi = __uint_as_float(x[e] & 0xFFFF0000u);
            if (STEPS) {
                const u32 p = pack_bf16x2(lo * ws, hi * ws);
                y[e] = pack_bf16x2(__uint_as_float(y[e] << 16) + __uint_as_float(p << 16),
                                   __uint_as_float(y[e] & 0xFFFF0000u) + __uint_as_float(p & 0xFFFF0000u));
            } else {
                acc[2 * e] = __builtin_fmaf(lo, ws, acc[2 * e]);
                acc[2 * e + 1] = __builtin_fmaf(hi, ws, acc[2 * e + 1]);
            }
        }
    }
    if (!STEPS) {
#pragma unroll
        for (int e = 0; e < 4; ++e) y[e] = pack_bf16x2(acc[2 * e], acc[2 * e + 1]);
    }
    if (v < nvec) st16<true>(out + t * ldo + v, make_uint4(y[0], y[1], y[2], y[3]));
}

}  // namespace cfp8

extern "C" int cfp8_generate_permute_indices(const int64_t* tokens_per_expert_group, int experts_per_rank, int num_ranks,
                                             int64_t alignment, int32_t* permuted_indices, int64_t capacity,
                                             int32_t* m_sizes, int32_t* m_offsets, int64_t* start_index_values,
                                             void* stream) {
    using namespace cfp8;
    if (experts_per_rank <= 0 || num_ranks <= 0 || alignment <= 0 || capacity < 0)
        return set_error(CFP8_EINVAL, "generate_permute_indices: experts_per_rank=%d num_ranks=%d alignment=%lld capacity=%lld",
                         experts_per_rank, num_ranks, (long long)alignment, (long long)capacity);
    if ((int64_t)experts_per_rank * num_ranks > (1 << 20))
        return set_error(CFP8_EINVAL, "generate_permute_indices: more than 2^20 (rank, expert) pairs");
    if (!tokens_per_expert_group || !m_sizes || !m_offsets || !start_index_values || (capacity > 0 && !permuted_indices))
        return set_error(CFP8_EINVAL, "generate_permute_indices: null pointer");
    if (int rc = check_device()) return rc;
    hipStream_t st = static_cast<hipStream_t>(stream);
    hipLaunchKernelGGL(permute_scan_kernel, dim3(1), dim3(1024), 0, st, tokens_per_expert_group, experts_per_rank, num_ranks,
                       alignment, start_index_values, m_sizes, m_offsets);
    if (capacity > 0) {
        const int64_t blocks = (capacity + 255) / 256;
        if (blocks > 0x7FFFFFFFll) return set_error(CFP8_EINVAL, "generate_permute_indices: capacity too large");
        hipLaunchKernelGGL(permute_fill_kernel, dim3((unsigned)blocks), dim3(256), 0, st, tokens_per_expert_group,
                           start_index_values, m_sizes, m_offsets, experts_per_rank, num_ranks, permuted_indices, capacity);
    }
    return check_launch("generate_permute_indices");
}

extern "C" int cfp8_gather_rows(const void* x, int64_t ld_x_bytes, const int32_t* indices, int64_t rows_out,
                                int64_t row_bytes, void* out, int64_t ld_out_bytes, void* stream) {
    using namespace cfp8;
    if (rows_out < 0 || row_bytes < 0) return set_error(CFP8_EINVAL, "gather_rows: negative shape");
    if (rows_out == 0 || row_bytes == 0) return CFP8_OK;
    if (!x || !indices || !out) return set_error(CFP8_EINVAL, "gather_rows: null pointer");
    if (row_bytes % 16 || ld_x_bytes % 16 || ld_out_bytes % 16 || ld_x_bytes < row_bytes || ld_out_bytes < row_bytes)
        return set_error(CFP8_EINVAL, "gather_rows: row_bytes=%lld and the row pitches must be multiples of 16 with pitch >= row_bytes",
                         (long long)row_bytes);
    if (!aligned16(x) || !aligned16(out)) return set_error(CFP8_EINVAL, "gather_rows: misaligned pointer");
    const int64_t blocks = (rows_out + 3) / 4;
    if (blocks > 0x7FFFFFFFll || row_bytes / 16 > 0x7FFFFFFFll) return set_error(CFP8_EINVAL, "gather_rows: too large for one launch");
    if (int rc = check_device()) return rc;
    hipLaunchKernelGGL(gather_rows_kernel, dim3((unsigned)blocks), dim3(256), 0, static_cast<hipStream_t>(stream),
                       static_cast<const uint4*>(x), ld_x_bytes / 16, indices, rows_out, (int)(row_bytes / 16),
                       static_cast<uint4*>(out), ld_out_bytes / 16);
    return check_launch("gather_rows");
}

extern "C" int cfp8_combine_rows(const void* rows, int64_t ld_rows, int64_t num_rows, const int32_t* row_map,
                                 const void* weights, int weights_dtype, int64_t tokens, int topk, int64_t hidden,
                                 int mode, void* out, int64_t ld_out, void* stream) {
    using namespace cfp8;
    if (tokens < 0 || hidden < 0 || num_rows < 0) return set_error(CFP8_EINVAL, "combine_rows: negative shape");
    if (topk < 0 || topk > 64) return set_error(CFP8_EINVAL, "combine_rows: topk=%d must be in [0, 64]", topk);
    if (mode != CFP8_COMBINE_BF16_STEPS && mode != CFP8_COMBINE_F32) return set_error(CFP8_EINVAL, "combine_rows: unknown mode %d", mode);
    if (weights_dtype != CFP8_IN_BF16 && weights_dtype != CFP8_IN_F32)
        return set_error(CFP8_EINVAL, "combine_rows: weights must be bf16 or fp32");
    if (mode == CFP8_COMBINE_BF16_STEPS && weights_dtype != CFP8_IN_BF16)
        return set_error(CFP8_EINVAL, "combine_rows: the bf16-steps mode takes bf16 weights");
    if (tokens == 0 || hidden == 0) return CFP8_OK;
    if (!out || (topk > 0 && (!rows || !row_map || !weights))) return set_error(CFP8_EINVAL, "combine_rows: null pointer");
    if (topk > 0 && num_rows == 0) return set_error(CFP8_EINVAL, "combine_rows: no source rows");
    if (hidden % 8 || ld_rows % 8 || ld_out % 8 || ld_rows < hidden || ld_out < hidden)
        return set_error(CFP8_EINVAL, "combine_rows: hidden=%lld and the row pitches must be multiples of 8 with pitch >= hidden", (long long)hidden);
    if (!aligned16(rows) || !aligned16(out)) return set_error(CFP8_EINVAL, "combine_rows: misaligned pointer");
    const int64_t nvec = hidden / 8, chunks = (nvec + 63) / 64;
    if (nvec > 0x7FFFFFFFll || tokens > 0x7FFFFFFFFFFFll / chunks || (tokens * chunks + 3) / 4 > 0x7FFFFFFFll)
        return set_error(CFP8_EINVAL, "combine_rows: too large for one launch");
    if (int rc = check_device()) return rc;
    const dim3 grid((unsigned)((tokens * chunks + 3) / 4)), block(256);
    hipStream_t st = static_cast<hipStream_t>(stream);
    const uint4* r = static_cast<const uint4*>(rows);
    uint4* o = static_cast<uint4*>(out);
    if (mode == CFP8_COMBINE_BF16_STEPS)
        hipLaunchKernelGGL((combine_rows_kernel<true, false>), grid, block, 0, st, r, ld_rows / 8, num_rows, row_map, weights, tokens, topk, (int)nvec, (int)chunks, o, ld_out / 8);
    else if (weights_dtype == CFP8_IN_F32)
        hipLaunchKernelGGL((combine_rows_kernel<false, true>), grid, block, 0, st, r, ld_rows / 8, num_rows, row_map, weights, tokens, topk, (int)nvec, (int)chunks, o, ld_out / 8);
    else
        hipLaunchKernelGGL((combine_rows_kernel<false, false>), grid, block, 0, st, r, ld_rows / 8, num_rows, row_map, weights, tokens, topk, (int)nvec, (int)chunks, o, ld_out / 8);
    return check_launch("combine_rows");
}
