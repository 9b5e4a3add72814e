// Tensorwise dynamic FP8 quantisation of many tensors: two launches per batch of
// up to 48 tensors (and a bounded number of bytes), no host round trip between them.
//
//   pass 1 (amax)  reads 2 B/element.  Every workgroup reduces a few contiguous
//                  chunks of one tensor and publishes its maximum with one
//                  fire-and-forget atomic max on the bit pattern (valid because
//                  |x| >= 0, and NaN patterns sort above infinity, so NaN
//                  propagates).  A tensor owns kAmaxSlots slots and a workgroup
//                  picks one by its index: thousands of co-resident workgroups
//                  hitting a single address serialise at the memory side.  Even
//                  so the 64 slots are two cache lines, and one atomic per 32 KiB
//                  holds a 1 GB tensor at 5.2 TB/s where the same loads without
//                  the atomic reach 6.9: a large launch therefore gives every
//                  workgroup up to 8 chunks (one atomic per 256 KiB).
//   pass 2 (cast)  reads 2 B and writes 1 B per element; every workgroup folds
//                  the tensor's slots and forms the scale on its own.
// The table of tensors travels in the kernel arguments (scalar loads), so the
// library needs no device-side descriptor buffer.

#include <mutex>

#include "cfp8_common.h"

namespace cfp8 {

constexpr int kMaxBatch = 48;
constexpr int kChunkVecs = 256 * 8;  // 16-byte vectors per workgroup: 32 KiB of bf16
constexpr int kAmaxSlots = CFP8_TENSORWISE_AMAX_SLOTS;  // one wavefront reads them in one load

struct TensorTable {
    const uint4* x[kMaxBatch];
    uint2* q[kMaxBatch];
    float* scale[kMaxBatch];
    int64_t nvec[kMaxBatch];
    u32* amax[kMaxBatch];  // kAmaxSlots slots each
    unsigned first_block[kMaxBatch + 1];  // exclusive prefix of workgroups per tensor
    int n;
    int per;  // chunks per workgroup (pass 1 only; pass 2 is one chunk per workgroup)
};

// Chunks per workgroup of pass 1 for a launch of `chunks` chunks in all: one while the launch is small (every
// chunk its own workgroup fills the GPU best), more once there are plenty.
static inline int amax_chunks_per_block(uint64_t chunks) {
    return chunks >= 32768 ? 8 : chunks >= 16384 ? 4 : chunks >= 8192 ? 2 : 1;
}

__device__ __forceinline__ int find_tensor(const TensorTable& tb, unsigned b) {
    int lo = 0, hi = tb.n - 1;
    while (lo < hi) {  // last t with first_block[t] <= b; uniform across the workgroup
        int mid = (lo + hi + 1) >> 1;
        if (tb.first_block[mid] <= b) lo = mid;
        else hi = mid - 1;
    }
    return lo;
}

__global__ __launch_bounds__(64) void tensorwise_zero_kernel(u32* slots, int64_t n) {
    const int64_t base = (int64_t)blockIdx.x * 64 * 1024;
    for (int64_t i = base + threadIdx.x; i < n && i < base + 64 * 1024; i += 64) slots[i] = 0u;
}

template <bool LDNT>
__global__ __launch_bounds__(256) void tensorwise_amax_kernel(const TensorTable tb) {
    __shared__ u32 red[4];
    const int t = find_tensor(tb, blockIdx.x);
    const unsigned local = blockIdx.x - tb.first_block[t];
    const int64_t nvec = tb.nvec[t];
    u32 m = 0;
    for (int c = 0; c < tb.per; ++c) {
        const int64_t base = ((int64_t)local * tb.per + c) * kChunkVecs;
        const int64_t left = nvec - base;
        if (left <= 0) break;  // uniform
        const uint4* x = tb.x[t] + base;
        uint4 v[8];
        if (left >= kChunkVecs) {
#pragma unroll
            for (int i = 0; i < 8; ++i) v[i] = ld16<LDNT>(x + threadIdx.x + 256 * i);
        } else {
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                int idx = threadIdx.x + 256 * i;
                v[i] = idx < left ? ld16<LDNT>(x + idx) : make_uint4(0, 0, 0, 0);
            }
        }
#pragma unroll
        for (int i = 0; i < 8; ++i) m = absmax8(m, v[i]);
    }
    m = wave_max(pk_fold(m));
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = m;
    __syncthreads();
    if (threadIdx.x == 0) {
        m = umax(umax(red[0], red[1]), umax(red[2], red[3])) << 16;  // fp32 bit pattern of the workgroup's amax
        if (m) atomicMax(tb.amax[t] + (local & (kAmaxSlots - 1)), m);  // result unused: the wave does not wait
    }
}

template <bool LDNT, bool STNT>
__global__ __launch_bounds__(256) void tensorwise_cast_kernel(const TensorTable tb) {
    const int t = find_tensor(tb, blockIdx.x);
    const unsigned local = blockIdx.x - tb.first_block[t];
    const int64_t base = (int64_t)local * kChunkVecs;
    const int64_t nvec = tb.nvec[t];
    const uint4* x = tb.x[t] + base;
    uint2* q = tb.q[t] + base;
    const int64_t left = nvec - base;
    static_assert(kAmaxSlots == 64, "one slot per lane");
    const float amax = __uint_as_float(wave_max(tb.amax[t][threadIdx.x & 63]));
    const float scale = scale_from_amax(amax);
    if (local == 0 && threadIdx.x == 0) *tb.scale[t] = scale;
    const Divider d(scale);
    uint4 v[8];
    if (left >= kChunkVecs) {
#pragma unroll
        for (int i = 0; i < 8; ++i) v[i] = ld16<LDNT>(x + threadIdx.x + 256 * i);
#pragma unroll
        for (int i = 0; i < 8; ++i) st8<STNT>(q + threadIdx.x + 256 * i, cast8(v[i], d));
    } else {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            int idx = threadIdx.x + 256 * i;
            if (idx < left) st8<STNT>(q + idx, cast8(ld16<LDNT>(x + idx), d));
        }
    }
}

enum : int { kPhaseAmax = 1, kPhaseCast = 2 };

static int run_tensorwise(const cfp8_tensor_desc* descs, int64_t n, float* amax_ws, void* stream, int phases) {
    if (n < 0 || n > (1ll << 24)) return set_error(CFP8_EINVAL, "quant_tensorwise: bad tensor count");
    if (n == 0) return CFP8_OK;
    if (!descs || !amax_ws) return set_error(CFP8_EINVAL, "quant_tensorwise: null descriptor table or amax workspace");
    for (int64_t i = 0; i < n; ++i) {
        const cfp8_tensor_desc& d = descs[i];
        if (d.numel < 0 || d.numel % 8) return set_error(CFP8_EINVAL, "quant_tensorwise: tensor %lld numel=%lld must be a non-negative multiple of 8", (long long)i, (long long)d.numel);
        if ((phases & kPhaseCast) && !d.scale) return set_error(CFP8_EINVAL, "quant_tensorwise: tensor %lld has a null scale pointer", (long long)i);
        if (d.numel && (!d.x || ((phases & kPhaseCast) && !d.q))) return set_error(CFP8_EINVAL, "quant_tensorwise: tensor %lld has a null data pointer", (long long)i);
        if (!aligned16(d.x) || (reinterpret_cast<uintptr_t>(d.q) & 7u)) return set_error(CFP8_EINVAL, "quant_tensorwise: tensor %lld is misaligned (x 16 bytes, q 8 bytes)", (long long)i);
        if ((d.numel / 8 + kChunkVecs - 1) / kChunkVecs > 0x3FFFFFFFll) return set_error(CFP8_EINVAL, "quant_tensorwise: tensor %lld is too large for one launch", (long long)i);
    }
    if (int rc = check_device()) return rc;
    hipStream_t st = static_cast<hipStream_t>(stream);
    u32* slots = reinterpret_cast<u32*>(amax_ws);
    if (phases & kPhaseAmax) {
        // zero every slot with a kernel (a memset node misbehaves under graph capture)
        const int64_t total = n * kAmaxSlots;
        const int64_t per = 64 * 1024;
        hipLaunchKernelGGL(tensorwise_zero_kernel, dim3((unsigned)((total + per - 1) / per)), dim3(64), 0, st, slots, total);
    }
    // Tensors are taken in batches of at most kMaxBatch entries; with both phases requested each
    // batch runs pass 1 then pass 2 back to back.  Every access streams past the caches (non-temporal
    // loads in both passes, non-temporal stores).  Measured on MI355X: few large launches with
    // streaming accesses beat small batches that would let pass 2 hit the 256 MiB memory-side cache,
    // because every launch pays a ramp-up and a tail.
    int64_t i = 0;
    while (i < n) {
        // the tensors of this batch: at most kMaxBatch, and few enough chunks for one grid
        const int64_t first = i;
        uint64_t chunks = 0;
        int count = 0;
        while (i < n && count < kMaxBatch) {
            uint64_t nc = (uint64_t)((descs[i].numel / 8 + kChunkVecs - 1) / kChunkVecs);
            if (nc == 0) nc = 1;  // a tensor with no element still owns one workgroup: it writes the scale
            if (count > 0 && chunks + nc > 0x7FFFFFFFull) break;
            chunks += nc;
            ++count;
            ++i;
        }
        // pass 1 gives a workgroup `per` chunks, pass 2 one: two tables that differ in the workgroup prefix
        for (int phase = kPhaseAmax; phase <= kPhaseCast; phase <<= 1) {
            if (!(phases & phase)) continue;
            TensorTable tb;
            tb.n = count;
            tb.per = phase == kPhaseAmax ? amax_chunks_per_block(chunks) : 1;
            unsigned blocks = 0;
            for (int k = 0; k < count; ++k) {
                const cfp8_tensor_desc& d = descs[first + k];
                const int64_t nvec = d.numel / 8;
                uint64_t nc = (uint64_t)((nvec + kChunkVecs - 1) / kChunkVecs);
                if (nc == 0) nc = 1;
                tb.x[k] = static_cast<const uint4*>(d.x);
                tb.q[k] = static_cast<uint2*>(d.q);
                tb.scale[k] = d.scale;
                tb.nvec[k] = nvec;
                tb.amax[k] = slots + (first + k) * kAmaxSlots;
                tb.first_block[k] = blocks;
                blocks += (unsigned)((nc + tb.per - 1) / tb.per);
            }
            tb.first_block[count] = blocks;
            if (phase == kPhaseAmax) hipLaunchKernelGGL(tensorwise_amax_kernel<true>, dim3(blocks), dim3(256), 0, st, tb);
            else hipLaunchKernelGGL((tensorwise_cast_kernel<true, true>), dim3(blocks), dim3(256), 0, st, tb);
        }
    }
    return check_launch("quant_tensorwise");
}

// ---- amax slots owned by the library, for callers that cannot allocate -------------------------
// One copy of this array lives on every GPU the library's code object is loaded on, at that GPU's
// own address.  In host code the name below is only a handle for hipGetSymbolAddress; kernels and
// every other use of the memory take the per-device pointer looked up in static_slots().
constexpr int kStaticMaxTensors = CFP8_TENSORWISE_STATIC_MAX_TENSORS;
static __device__ __align__(256) u32 scratch[kStaticMaxTensors * kAmaxSlots];

constexpr int kMaxDevices = 64;
static u32* g_static_slots[kMaxDevices];  // guarded by g_static_mutex; null until looked up
static std::mutex g_static_mutex;

// Device address of `scratch` on the current device, looked up once per device with that device
// current.
static int static_slots(u32** out) {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) {
        (void)hipGetLastError();
        return set_error(CFP8_EARCH, "quant_tensorwise_static: no current HIP device with an ordinal below %d", kMaxDevices);
    }
    std::lock_guard<std::mutex> lock(g_static_mutex);
    if (!g_static_slots[dev]) {
        u32* ptr = nullptr;
        hipError_t e = hipGetSymbolAddress(reinterpret_cast<void**>(&ptr), HIP_SYMBOL(scratch));
        if (e != hipSuccess || !ptr) {
            (void)hipGetLastError();
            return set_error(CFP8_ELAUNCH, "quant_tensorwise_static: hipGetSymbolAddress failed on device %d: %s", dev,
                             hipGetErrorString(e));
        }
        g_static_slots[dev] = ptr;
    }
    *out = g_static_slots[dev];
    return CFP8_OK;
}

}  // namespace cfp8

extern "C" int cfp8_quant_tensorwise_multi_static(const cfp8_tensor_desc* descs, int64_t n, void* stream) {
    using namespace cfp8;
    if (n < 0) return set_error(CFP8_EINVAL, "quant_tensorwise_static: bad tensor count");
    if (n > kStaticMaxTensors)
        return set_error(CFP8_EWORKSPACE,
                         "quant_tensorwise_static: %lld tensors exceed the %d the library's own amax slots hold; "
                         "split the call or use cfp8_quant_tensorwise_multi with a workspace",
                         (long long)n, kStaticMaxTensors);
    if (n == 0) return CFP8_OK;
    if (!descs) return set_error(CFP8_EINVAL, "quant_tensorwise_static: null descriptor table");
    if (int rc = check_device()) return rc;
    u32* slots = nullptr;
    if (int rc = static_slots(&slots)) return rc;
    // the amax phase clears the n * kAmaxSlots slots it uses with a fill kernel before pass 1
    return run_tensorwise(descs, n, reinterpret_cast<float*>(slots), stream, kPhaseAmax | kPhaseCast);
}

extern "C" int cfp8_quant_tensorwise_multi(const cfp8_tensor_desc* descs, int64_t n, float* amax_ws, void* stream) {
    return cfp8::run_tensorwise(descs, n, amax_ws, stream, cfp8::kPhaseAmax | cfp8::kPhaseCast);
}

extern "C" int cfp8_tensorwise_amax_multi(const cfp8_tensor_desc* descs, int64_t n, float* amax_ws, void* stream) {
    return cfp8::run_tensorwise(descs, n, amax_ws, stream, cfp8::kPhaseAmax);
}

extern "C" int cfp8_tensorwise_cast_multi(const cfp8_tensor_desc* descs, int64_t n, float* amax_ws, void* stream) {
    return cfp8::run_tensorwise(descs, n, amax_ws, stream, cfp8::kPhaseCast);
}

extern "C" int cfp8_quant_tensorwise(const void* x, int64_t numel, void* q, float* scale, float* amax_ws,
                                     void* stream) {
    cfp8_tensor_desc d{x, q, scale, numel};
    return cfp8_quant_tensorwise_multi(&d, 1, amax_ws, stream);
}
