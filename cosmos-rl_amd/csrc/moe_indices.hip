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
