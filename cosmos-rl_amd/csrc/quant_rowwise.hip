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
template <int V, bool NTS, int SRC>
__global__ __launch_bounds__(256) void rowwise_wave_kernel(const uint8_t* __restrict__ x, int64_t rows,
                                                           int nvec, int64_t ldx, uint2* __restrict__ q,
                                                           int64_t ldq, float* __restrict__ scales) {
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= rows) return;  // wave-uniform
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

__device__ __forceinline__ u32 block_max_256(u32 wave_val, u32* lds) {
    const int wave = threadIdx.x >> 6;
    if ((threadIdx.x & 63) == 0) lds[wave] = wave_val;
    __syncthreads();
    return umax(umax(lds[0], lds[1]), umax(lds[2], lds[3]));
}

template <int V, bool NTS, int SRC>
__global__ __launch_bounds__(256) void rowwise_block_kernel(const uint8_t* __restrict__ x, int nvec,
                                                            int64_t ldx, uint2* __restrict__ q,
                                                            int64_t ldq, float* __restrict__ scales) {
    __shared__ u32 red[4];
    const int64_t row = blockIdx.x;
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

// streaming_out: write the fp8 bytes with non-temporal stores (weights, consumed much
// later); false keeps them cacheable (activations feeding the GEMM of the same call).
template <bool NTS, int SRC>
static void launch_rowwise_variant(const uint8_t* xv, int64_t rows, int64_t nvec, int64_t ldx, uint2* qv, int64_t ldq,
                                   float* scales, hipStream_t st) {
#define CFP8_WAVE(V)                                                                                             \
    hipLaunchKernelGGL((rowwise_wave_kernel<V, NTS, SRC>), dim3((unsigned)((rows + 3) / 4)), dim3(256), 0, st, xv, \
                       rows, (int)nvec, ldx, qv, ldq, scales)
#define CFP8_BLOCK(V)                                                                                               \
    hipLaunchKernelGGL((rowwise_block_kernel<V, NTS, SRC>), dim3((unsigned)rows), dim3(256), 0, st, xv, (int)nvec, ldx, \
                       qv, ldq, scales)
    if (nvec <= 64) CFP8_WAVE(1);
    else if (nvec <= 128) CFP8_WAVE(2);
    else if (nvec <= 256) CFP8_WAVE(4);
    else if (nvec <= 512) CFP8_WAVE(8);
    else if (nvec <= 1024) CFP8_BLOCK(4);
    else if (nvec <= 2048) CFP8_BLOCK(8);
    else if (nvec <= 4096) CFP8_BLOCK(16);
    else
        hipLaunchKernelGGL((rowwise_stream_kernel<NTS, SRC>), dim3((unsigned)rows), dim3(256), 0, st, xv, nvec, ldx, qv, ldq, scales);
#undef CFP8_WAVE
#undef CFP8_BLOCK
}

template <int SRC>
static int launch_quant_rowwise_src(const void* x, int64_t rows, int64_t cols, int64_t ld_x, void* q, int64_t ld_q,
                                    float* scales, bool streaming_out, hipStream_t st) {
    const uint8_t* xv = static_cast<const uint8_t*>(x);
    uint2* qv = static_cast<uint2*>(q);
    const int64_t nvec = cols / 8, ldx = ld_x * SrcBytes<SRC>::value, ldq = ld_q / 8;
    if (rows > 0x7FFFFFFFll) return set_error(CFP8_EINVAL, "quant_rowwise: rows=%lld exceeds the grid limit", (long long)rows);
    if (streaming_out) launch_rowwise_variant<true, SRC>(xv, rows, nvec, ldx, qv, ldq, scales, st);
    else launch_rowwise_variant<false, SRC>(xv, rows, nvec, ldx, qv, ldq, scales, st);
    return check_launch("quant_rowwise");
}

int launch_quant_rowwise(const void* x, int64_t rows, int64_t cols, int64_t ld_x, void* q, int64_t ld_q,
                         float* scales, bool streaming_out, hipStream_t st) {
    return launch_quant_rowwise_src<kSrcBF16>(x, rows, cols, ld_x, q, ld_q, scales, streaming_out, st);
}

static int quant_rowwise_entry(const void* x, int x_dtype, int64_t rows, int64_t cols, int64_t ld_x, void* q,
                               int64_t ld_q, float* scales, void* stream) {
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
    if (int rc = check_device()) return rc;
    // outputs of 32 MiB and more cannot stay cache resident anyway: stream them out
    const bool streaming = rows * cols >= (32ll << 20);
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (x_dtype == CFP8_IN_F32) return launch_quant_rowwise_src<kSrcF32>(x, rows, cols, ld_x, q, ld_q, scales, streaming, st);
    if (x_dtype == CFP8_IN_F16) return launch_quant_rowwise_src<kSrcF16>(x, rows, cols, ld_x, q, ld_q, scales, streaming, st);
    return launch_quant_rowwise_src<kSrcBF16>(x, rows, cols, ld_x, q, ld_q, scales, streaming, st);
}

}  // namespace cfp8

extern "C" int cfp8_quant_rowwise(const void* x, int64_t rows, int64_t cols, int64_t ld_x, void* q,
                                  int64_t ld_q, float* scales, void* stream) {
    return cfp8::quant_rowwise_entry(x, CFP8_IN_BF16, rows, cols, ld_x, q, ld_q, scales, stream);
}

extern "C" int cfp8_quant_rowwise_from(const void* x, int x_dtype, int64_t rows, int64_t cols, int64_t ld_x, void* q,
                                       int64_t ld_q, float* scales, void* stream) {
    return cfp8::quant_rowwise_entry(x, x_dtype, rows, cols, ld_x, q, ld_q, scales, stream);
}
