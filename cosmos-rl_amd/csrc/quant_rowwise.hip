// Rowwise dynamic FP8 quantisation: per row amax -> scale -> e4m3.
//
// HBM-bound: 2 bytes read and 1 byte written per element plus 4 bytes per row.
// Each row is read from HBM once: it is held in registers as packed bf16
// between the amax sweep and the cast sweep.
//   * rows of up to 4096 elements: one 64-lane wavefront per row, no LDS, no
//     barrier; four rows per 256-thread workgroup.
//   * rows of up to 32768 elements: one workgroup per row, cross-wave max
//     through LDS.
//   * longer rows: one workgroup per row, second sweep re-reads the row.
//
// The source may also be fp16 or fp32 (the dtype a weight is transferred in): it
// is rounded to bf16 first, exactly as `recv.to(torch.bfloat16)` would, and the
// row is still held as packed bf16, so the three sources share every kernel.
#include <hip/hip_fp16.h>

#include <type_traits>
#include <vector>

#include "cfp8_common.h"

namespace cfp8 {

// source element types; the values are the ABI's CFP8_IN_* codes
enum : int { kSrcBF16 = CFP8_IN_BF16, kSrcF16 = CFP8_IN_F16, kSrcF32 = CFP8_IN_F32 };
template <int SRC> struct SrcBytes { static constexpr int value = SRC == kSrcF32 ? 4 : 2; };

// 8 consecutive source elements -> 8 packed bf16 (round to nearest even).  `row` points at the
// first element of the row, `idx` counts groups of 8 elements.
template <int SRC, bool NT>
__device__ __forceinline__ uint4 ld8(const void* row, int64_t idx) {
    if (SRC == kSrcBF16) return ld16<NT>(static_cast<const uint4*>(row) + idx);
    if (SRC == kSrcF16) {
        const uint4 h = ld16<NT>(static_cast<const uint4*>(row) + idx);
        const u32 w[4] = {h.x, h.y, h.z, h.w};
        u32 o[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const __half2 hh = __builtin_bit_cast(__half2, w[i]);
            o[i] = pack_bf16x2(__low2float(hh), __high2float(hh));
        }
        return make_uint4(o[0], o[1], o[2], o[3]);
    }
    const uint4 a = ld16<NT>(static_cast<const uint4*>(row) + 2 * idx);
    const uint4 b = ld16<NT>(static_cast<const uint4*>(row) + 2 * idx + 1);
    return make_uint4(pack_bf16x2(__uint_as_float(a.x), __uint_as_float(a.y)), pack_bf16x2(__uint_as_float(a.z), __uint_as_float(a.w)),
                      pack_bf16x2(__uint_as_float(b.x), __uint_as_float(b.y)), pack_bf16x2(__uint_as_float(b.z), __uint_as_float(b.w)));
}

// ldx: bytes between rows of x; ldq: 8-byte units between rows of q
// One wavefront quantises row `row` (wave-uniform).
template <int V, bool NTS, int SRC>
__device__ __forceinline__ void rowwise_wave_body(const uint8_t* __restrict__ x, int64_t row, int nvec, int64_t ldx,
                                                  uint2* __restrict__ q, int64_t ldq, float* __restrict__ scales) {
    const int lane = threadIdx.x & 63;
    const uint8_t* xr = x + row * ldx;
    uint4 v[V];
#pragma unroll
    for (int i = 0; i < V; ++i) {
        int idx = lane + 64 * i;
        v[i] = idx < nvec ? ld8<SRC, true>(xr, idx) : make_uint4(0, 0, 0, 0);
    }
    u32 m = 0;
#pragma unroll
    for (int i = 0; i < V; ++i) m = absmax8(m, v[i]);
    const float amax = amax_from_bits(wave_max(pk_fold(m)));
    const float scale = scale_from_amax(amax);
    if (lane == 0) scales[row] = scale;
    const Divider d(scale);
    uint2* qr = q + row * ldq;
#pragma unroll
    for (int i = 0; i < V; ++i) {
        int idx = lane + 64 * i;
        if (idx < nvec) st8<NTS>(qr + idx, cast8(v[i], d));
    }
}

template <int V, bool NTS, int SRC>
__global__ __launch_bounds__(256) void rowwise_wave_kernel(const uint8_t* __restrict__ x, int64_t rows,
                                                           int nvec, int64_t ldx, uint2* __restrict__ q,
                                                           int64_t ldq, float* __restrict__ scales) {
    const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= rows) return;  // wave-uniform
    rowwise_wave_body<V, NTS, SRC>(x, row, nvec, ldx, q, ldq, scales);
}

__device__ __forceinline__ u32 block_max_256(u32 wave_val, u32* lds) {
    const int wave = threadIdx.x >> 6;
    if ((threadIdx.x & 63) == 0) lds[wave] = wave_val;
    __syncthreads();
    return umax(umax(lds[0], lds[1]), umax(lds[2], lds[3]));
}

// One workgroup quantises row `row`.
template <int V, bool NTS, int SRC>
__device__ __forceinline__ void rowwise_block_body(const uint8_t* __restrict__ x, int64_t row, int nvec, int64_t ldx,
                                                   uint2* __restrict__ q, int64_t ldq, float* __restrict__ scales,
                                                   u32* red) {
    const int t = threadIdx.x;
    const uint8_t* xr = x + row * ldx;
    uint4 v[V];
#pragma unroll
    for (int i = 0; i < V; ++i) {
        int idx = t + 256 * i;
        v[i] = idx < nvec ? ld8<SRC, true>(xr, idx) : make_uint4(0, 0, 0, 0);
    }
    u32 m = 0;
#pragma unroll
    for (int i = 0; i < V; ++i) m = absmax8(m, v[i]);
    const float amax = amax_from_bits(block_max_256(wave_max(pk_fold(m)), red));
    const float scale = scale_from_amax(amax);
    if (t == 0) scales[row] = scale;
    const Divider d(scale);
    uint2* qr = q + row * ldq;
#pragma unroll
    for (int i = 0; i < V; ++i) {
        int idx = t + 256 * i;
        if (idx < nvec) st8<NTS>(qr + idx, cast8(v[i], d));
    }
}

template <int V, bool NTS, int SRC>
__global__ __launch_bounds__(256) void rowwise_block_kernel(const uint8_t* __restrict__ x, int nvec,
                                                            int64_t ldx, uint2* __restrict__ q,
                                                            int64_t ldq, float* __restrict__ scales) {
    __shared__ u32 red[4];
    rowwise_block_body<V, NTS, SRC>(x, blockIdx.x, nvec, ldx, q, ldq, scales, red);
}

// ---- many weights in one launch --------------------------------------------------------------
// The weights of one flush group of a weight sync (rollout_control.py:1308-1319 runs the queued
// completions together) are a few dozen tensors of 13..140 MB: quantised one launch each, every one
// pays the ramp-up and the tail of a launch that lasts 8..70 us.  Here the table of tensors travels
// in the kernel arguments and a workgroup finds its tensor by a search over the prefix of workgroup
// counts, as in the tensorwise quantiser; all tensors of a launch share the kernel variant (vectors
// per lane), the source dtype and the store policy.
constexpr int kMaxRowBatch = 40;
struct RowTable {
    const uint8_t* x[kMaxRowBatch];
    uint2* q[kMaxRowBatch];
    float* scales[kMaxRowBatch];
    int64_t ldx[kMaxRowBatch], ldq[kMaxRowBatch];
    int64_t rows[kMaxRowBatch];
    int nvec[kMaxRowBatch];
    unsigned first_block[kMaxRowBatch + 1];
    int n;
};
__device__ __forceinline__ int find_row_tensor(const RowTable& tb, unsigned b) {
    int lo = 0, hi = tb.n - 1;
    while (lo < hi) {  // last t with first_block[t] <= b; uniform across the workgroup
        const int mid = (lo + hi + 1) >> 1;
        if (tb.first_block[mid] <= b) lo = mid;
        else hi = mid - 1;
    }
    return lo;
}

template <int V, bool NTS, int SRC>
__global__ __launch_bounds__(256) void rowwise_wave_multi_kernel(const RowTable tb) {
    const int t = find_row_tensor(tb, blockIdx.x);
    const int64_t row = (int64_t)(blockIdx.x - tb.first_block[t]) * 4 + (threadIdx.x >> 6);
    if (row >= tb.rows[t]) return;  // wave-uniform
    rowwise_wave_body<V, NTS, SRC>(tb.x[t], row, tb.nvec[t], tb.ldx[t], tb.q[t], tb.ldq[t], tb.scales[t]);
}

template <int V, bool NTS, int SRC>
__global__ __launch_bounds__(256) void rowwise_block_multi_kernel(const RowTable tb) {
    __shared__ u32 red[4];
    const int t = find_row_tensor(tb, blockIdx.x);
    rowwise_block_body<V, NTS, SRC>(tb.x[t], blockIdx.x - tb.first_block[t], tb.nvec[t], tb.ldx[t], tb.q[t], tb.ldq[t],
                                    tb.scales[t], red);
}

template <bool NTS, int SRC>
__global__ __launch_bounds__(256) void rowwise_stream_kernel(const uint8_t* __restrict__ x, int64_t nvec,
                                                             int64_t ldx, uint2* __restrict__ q,
                                                             int64_t ldq, float* __restrict__ scales) {
    __shared__ u32 red[4];
    const int64_t row = blockIdx.x;
    const int t = threadIdx.x;
    const uint8_t* xr = x + row * ldx;
    u32 m = 0;
    for (int64_t idx = t; idx < nvec; idx += 256) m = absmax8(m, ld8<SRC, false>(xr, idx));  // kept cacheable: re-read below
    const float amax = amax_from_bits(block_max_256(wave_max(pk_fold(m)), red));
    const float scale = scale_from_amax(amax);
    if (t == 0) scales[row] = scale;
    const Divider d(scale);
    uint2* qr = q + row * ldq;
    for (int64_t idx = t; idx < nvec; idx += 256) st8<NTS>(qr + idx, cast8(ld8<SRC, true>(xr, idx), d));
}

// Kernel variant for rows of nvec 16-byte vectors: vectors per lane of the one-wave-per-row kernel
// (1, 2, 4, 8: up to 4096 elements), vectors per thread of the one-workgroup-per-row kernel
// (4 .. 16, picked close to nvec / 256 so that few threads sit idle and few registers are held:
// 18944-element rows take 10, not 16), or 0 for the two-sweep kernel.
struct RowVariant {
    bool wave;
    int v;
};
static RowVariant row_variant(int64_t nvec) {
    if (nvec <= 64) return {true, 1};
    if (nvec <= 128) return {true, 2};
    if (nvec <= 256) return {true, 4};
    if (nvec <= 512) return {true, 8};
    for (int v : {4, 5, 6, 8, 10, 12, 16})
        if (nvec <= 256 * v) return {false, v};
    return {false, 0};
}

// Calls f(std::integral_constant<bool, wave>, std::integral_constant<int, V>) for the variant; false for the
// two-sweep kernel, which has no such form.
template <class F>
static bool with_row_variant(RowVariant rv, F&& f) {
#define CFP8_CASE(W, V)                                                               \
    if (rv.wave == W && rv.v == V) {                                                  \
        f(std::integral_constant<bool, W>{}, std::integral_constant<int, V>{});       \
        return true;                                                                  \
    }
    CFP8_CASE(true, 1) CFP8_CASE(true, 2) CFP8_CASE(true, 4) CFP8_CASE(true, 8)
    CFP8_CASE(false, 4) CFP8_CASE(false, 5) CFP8_CASE(false, 6) CFP8_CASE(false, 8)
    CFP8_CASE(false, 10) CFP8_CASE(false, 12) CFP8_CASE(false, 16)
#undef CFP8_CASE
    return false;
}

// streaming_out: write the fp8 bytes with non-temporal stores (weights, consumed much
// later); false keeps them cacheable (activations feeding the GEMM of the same call).
template <bool NTS, int SRC>
static void launch_rowwise_variant(const uint8_t* xv, int64_t rows, int64_t nvec, int64_t ldx, uint2* qv, int64_t ldq,
                                   float* scales, hipStream_t st) {
    const bool done = with_row_variant(row_variant(nvec), [&](auto wave, auto v) {
        constexpr int V = decltype(v)::value;
        if constexpr (decltype(wave)::value)
            hipLaunchKernelGGL((rowwise_wave_kernel<V, NTS, SRC>), dim3((unsigned)((rows + 3) / 4)), dim3(256), 0, st, xv,
                               rows, (int)nvec, ldx, qv, ldq, scales);
        else
            hipLaunchKernelGGL((rowwise_block_kernel<V, NTS, SRC>), dim3((unsigned)rows), dim3(256), 0, st, xv, (int)nvec,
                               ldx, qv, ldq, scales);
    });
    if (!done)
        hipLaunchKernelGGL((rowwise_stream_kernel<NTS, SRC>), dim3((unsigned)rows), dim3(256), 0, st, xv, nvec, ldx, qv, ldq, scales);
}

template <bool NTS, int SRC>
static void launch_rowwise_table(RowVariant rv, const RowTable& tb, unsigned blocks, hipStream_t st) {
    with_row_variant(rv, [&](auto wave, auto v) {
        constexpr int V = decltype(v)::value;
        if constexpr (decltype(wave)::value)
            hipLaunchKernelGGL((rowwise_wave_multi_kernel<V, NTS, SRC>), dim3(blocks), dim3(256), 0, st, tb);
        else
            hipLaunchKernelGGL((rowwise_block_multi_kernel<V, NTS, SRC>), dim3(blocks), dim3(256), 0, st, tb);
    });
}

template <int SRC>
static int launch_quant_rowwise_src(const void* x, int64_t rows, int64_t cols, int64_t ld_x, void* q, int64_t ld_q,
                                    float* scales, bool streaming_out, hipStream_t st) {
    const uint8_t* xv = static_cast<const uint8_t*>(x);
    uint2* qv = static_cast<uint2*>(q);
    const int64_t nvec = cols / 8, ldx = ld_x * SrcBytes<SRC>::value, ldq = ld_q / 8;
    if (streaming_out) launch_rowwise_variant<true, SRC>(xv, rows, nvec, ldx, qv, ldq, scales, st);
    else launch_rowwise_variant<false, SRC>(xv, rows, nvec, ldx, qv, ldq, scales, st);
    return check_launch("quant_rowwise");
}

int launch_quant_rowwise(const void* x, int64_t rows, int64_t cols, int64_t ld_x, void* q, int64_t ld_q,
                         float* scales, bool streaming_out, hipStream_t st) {
    return launch_quant_rowwise_src<kSrcBF16>(x, rows, cols, ld_x, q, ld_q, scales, streaming_out, st);
}

// argument checks shared by the single-tensor and the table entry points; rows == 0 is valid (and checked first)
static int check_rowwise_args(const void* x, int x_dtype, int64_t rows, int64_t cols, int64_t ld_x, const void* q,
                              int64_t ld_q, const float* scales) {
    if (rows < 0 || cols < 0) return set_error(CFP8_EINVAL, "quant_rowwise: negative shape");
    if (x_dtype != CFP8_IN_BF16 && x_dtype != CFP8_IN_F16 && x_dtype != CFP8_IN_F32)
        return set_error(CFP8_EINVAL, "quant_rowwise: unknown source dtype %d", x_dtype);
    if (rows == 0) return CFP8_OK;
    if (!x || !q || !scales) return set_error(CFP8_EINVAL, "quant_rowwise: null pointer");
    if (cols % 8 || ld_x % 8 || ld_q % 8 || ld_x < cols || ld_q < cols)
        return set_error(CFP8_EINVAL, "quant_rowwise: cols=%lld ld_x=%lld ld_q=%lld must be multiples of 8 with ld >= cols",
                         (long long)cols, (long long)ld_x, (long long)ld_q);
    if (!aligned16(x) || (reinterpret_cast<uintptr_t>(q) & 7u))
        return set_error(CFP8_EINVAL, "quant_rowwise: x must be 16-byte and q 8-byte aligned");
    if (rows > 0x7FFFFFFFll) return set_error(CFP8_EINVAL, "quant_rowwise: rows=%lld exceeds the grid limit", (long long)rows);
    return CFP8_OK;
}

static int quant_rowwise_entry(const void* x, int x_dtype, int64_t rows, int64_t cols, int64_t ld_x, void* q,
                               int64_t ld_q, float* scales, void* stream) {
    if (int rc = check_rowwise_args(x, x_dtype, rows, cols, ld_x, q, ld_q, scales)) return rc;
    if (rows == 0) return CFP8_OK;
    if (int rc = check_device()) return rc;
    // outputs of 32 MiB and more cannot stay cache resident anyway: stream them out
    const bool streaming = rows * cols >= (32ll << 20);
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (x_dtype == CFP8_IN_F32) return launch_quant_rowwise_src<kSrcF32>(x, rows, cols, ld_x, q, ld_q, scales, streaming, st);
    if (x_dtype == CFP8_IN_F16) return launch_quant_rowwise_src<kSrcF16>(x, rows, cols, ld_x, q, ld_q, scales, streaming, st);
    return launch_quant_rowwise_src<kSrcBF16>(x, rows, cols, ld_x, q, ld_q, scales, streaming, st);
}

// Table form: tensors are grouped by (kernel variant, source dtype, store policy); every group goes out in
// launches of at most kMaxRowBatch tensors.  Rows too long for a register-resident kernel take the
// single-tensor two-sweep kernel, one launch each.
static int quant_rowwise_multi_entry(const cfp8_rowwise_desc* descs, int64_t n, void* stream) {
    if (n < 0 || n > (1ll << 24)) return set_error(CFP8_EINVAL, "quant_rowwise_multi: bad tensor count");
    if (n == 0) return CFP8_OK;
    if (!descs) return set_error(CFP8_EINVAL, "quant_rowwise_multi: null descriptor table");
    for (int64_t i = 0; i < n; ++i) {
        const cfp8_rowwise_desc& d = descs[i];
        if (int rc = check_rowwise_args(d.x, d.x_dtype, d.rows, d.cols, d.ld_x, d.q, d.ld_q, d.scales)) return rc;
    }
    if (int rc = check_device()) return rc;
    hipStream_t st = static_cast<hipStream_t>(stream);
    // the store policy follows the bytes of the whole call: a sync's worth of weights does not stay in any cache
    int64_t total = 0;
    for (int64_t i = 0; i < n; ++i) total += descs[i].rows * descs[i].cols;
    const bool streaming = total >= (32ll << 20);
    std::vector<char> taken((size_t)n, 0);
    for (int64_t first = 0; first < n; ++first) {
        if (taken[(size_t)first]) continue;
        const cfp8_rowwise_desc& f = descs[first];
        if (f.rows == 0 || f.cols == 0) {
            taken[(size_t)first] = 1;
            if (f.rows && f.cols == 0)  // rows without elements still get their scale
                if (int rc = quant_rowwise_entry(f.x, f.x_dtype, f.rows, f.cols, f.ld_x, f.q, f.ld_q, f.scales, stream)) return rc;
            continue;
        }
        const RowVariant rv = row_variant(f.cols / 8);
        if (rv.v == 0) {
            taken[(size_t)first] = 1;
            if (int rc = quant_rowwise_entry(f.x, f.x_dtype, f.rows, f.cols, f.ld_x, f.q, f.ld_q, f.scales, stream)) return rc;
            continue;
        }
        RowTable tb;
        tb.n = 0;
        uint64_t blocks = 0;
        auto flush = [&]() {
            if (tb.n == 0) return;
            tb.first_block[tb.n] = (unsigned)blocks;
#define CFP8_GO(NTS)                                                                                              \
    if (f.x_dtype == CFP8_IN_F32) launch_rowwise_table<NTS, kSrcF32>(rv, tb, (unsigned)blocks, st);                \
    else if (f.x_dtype == CFP8_IN_F16) launch_rowwise_table<NTS, kSrcF16>(rv, tb, (unsigned)blocks, st);           \
    else launch_rowwise_table<NTS, kSrcBF16>(rv, tb, (unsigned)blocks, st);
            if (streaming) { CFP8_GO(true) } else { CFP8_GO(false) }
#undef CFP8_GO
            tb.n = 0;
            blocks = 0;
        };
        for (int64_t i = first; i < n; ++i) {
            const cfp8_rowwise_desc& d = descs[i];
            if (taken[(size_t)i] || d.rows == 0 || d.cols == 0 || d.x_dtype != f.x_dtype) continue;
            const RowVariant ri = row_variant(d.cols / 8);
            if (ri.wave != rv.wave || ri.v != rv.v) continue;
            const uint64_t nb = rv.wave ? (uint64_t)(d.rows + 3) / 4 : (uint64_t)d.rows;
            if (tb.n == kMaxRowBatch || blocks + nb > 0x7FFFFFFFull) flush();
            const int64_t eb = d.x_dtype == CFP8_IN_F32 ? 4 : 2;  // bytes per source element
            tb.x[tb.n] = static_cast<const uint8_t*>(d.x);
            tb.q[tb.n] = static_cast<uint2*>(d.q);
            tb.scales[tb.n] = d.scales;
            tb.ldx[tb.n] = d.ld_x * eb;
            tb.ldq[tb.n] = d.ld_q / 8;
            tb.rows[tb.n] = d.rows;
            tb.nvec[tb.n] = (int)(d.cols / 8);
            tb.first_block[tb.n] = (unsigned)blocks;
            blocks += nb;
            ++tb.n;
            taken[(size_t)i] = 1;
        }
        flush();
    }
    return check_launch("quant_rowwise_multi");
}

}  // namespace cfp8

extern "C" int cfp8_quant_rowwise_multi(const cfp8_rowwise_desc* descs, int64_t n, void* stream) {
    return cfp8::quant_rowwise_multi_entry(descs, n, stream);
}

extern "C" int cfp8_quant_rowwise(const void* x, int64_t rows, int64_t cols, int64_t ld_x, void* q,
                                  int64_t ld_q, float* scales, void* stream) {
    return cfp8::quant_rowwise_entry(x, CFP8_IN_BF16, rows, cols, ld_x, q, ld_q, scales, stream);
}

extern "C" int cfp8_quant_rowwise_from(const void* x, int x_dtype, int64_t rows, int64_t cols, int64_t ld_x, void* q,
                                       int64_t ld_q, float* scales, void* stream) {
    return cfp8::quant_rowwise_entry(x, x_dtype, rows, cols, ld_x, q, ld_q, scales, stream);
}
