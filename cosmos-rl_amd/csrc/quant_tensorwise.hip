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
//                  workgroup up to 8 chunks (one atomic per 256 KiB).  The maxima
//                  use slots 0 .. kAmaxSlots - 2; the last slot is the tensor's
//                  status word (see the resident kernel below), zero here.
//   pass 2 (cast)  reads 2 B and writes 1 B per element; every workgroup folds
//                  the tensor's slots and forms the scale on its own.
// The table of tensors travels in the kernel arguments (scalar loads), so the
// library needs no device-side descriptor buffer.

#include <atomic>
#include <mutex>

#include "cfp8_common.h"

namespace cfp8 {

constexpr int kMaxBatch = 48;
constexpr int kChunkVecs = 256 * 8;  // 16-byte vectors per workgroup: 32 KiB of bf16
constexpr int kAmaxSlots = CFP8_TENSORWISE_AMAX_SLOTS;  // one wavefront reads them in one load
constexpr int kMaxSlots = kAmaxSlots - 1;                // slots that hold maxima; slot kStatusSlot is the status word
constexpr int kStatusSlot = kAmaxSlots - 1;
constexpr int kMaxDevices = 64;  // device ordinals with per-device state of their own

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
        if (m) atomicMax(tb.amax[t] + local % (unsigned)kMaxSlots, m);  // result unused: the wave does not wait
    }
}

// CLAMP: the quotient is clamped to +-448 before the conversion.  The fused call needs no clamp (the scale comes
// from the maximum of the very data that is cast, so no quotient exceeds 448 by more than one fp32 step and the
// conversion rounds that to 448 by itself); the split-phase cast takes the caller's slots, which an all-reduce or
// a stale workspace may have left smaller than the tensor's own maximum, and saturates like the reference's cast.
template <bool LDNT, bool STNT, bool CLAMP>
__global__ __launch_bounds__(256) void tensorwise_cast_kernel(const TensorTable tb) {
    const int t = find_tensor(tb, blockIdx.x);
    const unsigned local = blockIdx.x - tb.first_block[t];
    const int64_t base = (int64_t)local * kChunkVecs;
    const int64_t nvec = tb.nvec[t];
    const uint4* x = tb.x[t] + base;
    uint2* q = tb.q[t] + base;
    const int64_t left = nvec - base;
    static_assert(kAmaxSlots == 64, "one slot per lane");
    const int slot = threadIdx.x & 63;
    const float amax = __uint_as_float(wave_max(slot < kMaxSlots ? tb.amax[t][slot] : 0u));
    const float scale = scale_from_amax(amax);
    if (local == 0 && threadIdx.x == 0) *tb.scale[t] = scale;
    const Divider d(scale);
    auto cast = [&](const uint4& v) { return CLAMP ? cast8_clamped(v, d) : cast8(v, d); };
    uint4 v[8];
    if (left >= kChunkVecs) {
#pragma unroll
        for (int i = 0; i < 8; ++i) v[i] = ld16<LDNT>(x + threadIdx.x + 256 * i);
#pragma unroll
        for (int i = 0; i < 8; ++i) st8<STNT>(q + threadIdx.x + 256 * i, cast(v[i]));
    } else {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            int idx = threadIdx.x + 256 * i;
            if (idx < left) st8<STNT>(q + idx, cast(ld16<LDNT>(x + idx)));
        }
    }
}

// ---------------------------------------------------------------------------
// Both passes in one launch, with the tensor kept on the chip in between (tensors of 106-141 MB: the MLP
// weights of a 7-8 B model; smaller ones several at a time, each held by a group of the CUs, see `groups` below).  One workgroup of twelve waves per CU (three per SIMD, 168 registers each, all of
// the CU's LDS): a lane keeps kResRegVecs 16-byte vectors in registers and kResLdsVecs in LDS, 256 CUs x 768
// lanes x 45 x 16 B = 141 MB.  Per tensor every wave loads its 1 KiB chunks (chunk c of the tensor goes to wave
// c mod waves, so that at any moment the GPU reads one compact window that moves through the tensor),
// reduces |x|, the workgroup publishes its maximum, the workgroups meet (below), and every wave casts what it holds
// with the tensor's scale and stores it: 2 B read and 1 B written per element instead of 2 + 2 + 1.  A slot that
// has been cast and stored is requested anew at once with the next tensor's chunk (register slots by loads into
// the same registers, LDS slots by direct-to-LDS loads), so one tensor's stores and the next one's loads are in
// flight together.  Every kept vector has its own registers, hence its own instructions: the code a wave runs per
// tensor is 30 KB of straight line, shared by the CU's twelve waves and small enough to stay in the instruction
// cache from one tensor to the next (with one wave per SIMD and all 512 registers it was 350 KB and the kernel
// spent its time fetching it).
// The meeting.  Every workgroup owns one word per side of a small array in device memory (tensors alternate
// sides); it writes tag << 16 | its maximum there with one atomic and then reads everybody's words until all carry
// the tensor's tag - at which point it also holds all the maxima.  While the workgroups meet nothing is in flight,
// so the meeting is the kernel's fixed cost per tensor; this form takes one trip to memory and one back (a counter
// took three dependent ones: publish the maximum, count the arrival, read the maxima - about 5 us more per tensor).
// The launch needs all its workgroups resident at once: the grid is one workgroup per CU and a workgroup takes a
// whole CU, so on a GPU that no other grid holds they are.  Where they are not (another stream's or process's
// kernel holds CUs, a second launch of this kind, a CU mask) the meeting cannot complete, so the wait is bounded
// by the wall clock and every wave leaves the kernel whatever happens.  A workgroup that gives up sets the status
// word (slot kStatusSlot of a tensor's amax slots) of the tensor it waited for and of every tensor behind it in
// the launch, marks its words of the meeting array so that the others stop waiting at once, and leaves; so does a
// workgroup that finds such a mark.  A workgroup may have seen the same meeting complete just before: it stores
// its part of that tensor with the right scale and gives up at the next meeting.  The two repair kernels that
// follow every resident launch on the same stream redo exactly the tensors whose status word is set, as two
// ordinary passes (a few microseconds when there is none), and what they write is what a complete launch writes,
// so the call's results are right either way; the status words stay set in the caller's workspace until its next
// use and cfp8_tensorwise_status counts them.
// The form is opt-in (cfp8_tensorwise_resident): a process switches it on when it has the GPU to itself while it
// quantises.
// ---------------------------------------------------------------------------
static std::atomic<int> g_resident_enabled{0};
static std::atomic<unsigned> g_resident_wait_us{20000};   // bound of a workgroup's wait at a tensor's meeting
static std::atomic<unsigned> g_resident_extra_arrivals{0};  // test hook: arrivals expected beyond the grid (never come)


constexpr int kResWaves = 12;     // per workgroup
constexpr int kResRegVecs = 32;
constexpr int kResLdsVecs = 13;
constexpr int kResVecs = kResRegVecs + kResLdsVecs;
constexpr int kResTouch = 2;      // chunks of the next tensor a wave touches while the workgroups meet
static_assert(kResLdsVecs <= kResRegVecs, "the LDS part passes through registers");
constexpr size_t kResLdsBytes = (size_t)kResWaves * kResLdsVecs * 64 * 16 + 64;
static_assert(kResLdsBytes <= 160 * 1024, "LDS of one CU");

// The meeting array: a word per workgroup and side (tensors alternate sides), tag << 16 | bf16 bits of the workgroup's
// maximum; cleared by a kernel in front of every resident launch.  A tag is the launch's number (10 bits, never all
// ones) and the tensor's number 1 .. kMaxBatch (6 bits); kMeetAbort in a word says that its workgroup has given the
// launch up.  Two such launches at once on one GPU cannot both have every CU and disturb each other's words; because
// their tags differ, neither can take a foreign word for an arrival: they run into the bound of the wait, and the
// repair kernels do the work.
constexpr int kMeetSlots = 1024;
constexpr u32 kMeetAbort = 0xFFFF0000u;
static __device__ __align__(256) u32 g_meet[2][kMeetSlots];

__global__ __launch_bounds__(256) void tensorwise_meet_clear_kernel() {
    for (int i = threadIdx.x; i < 2 * kMeetSlots; i += 256) (&g_meet[0][0])[i] = 0u;
}

struct ResidentTable {
    const uint4* x[kMaxBatch];
    uint2* q[kMaxBatch];
    float* scale[kMaxBatch];
    unsigned nchunks[kMaxBatch];  // 64-vector chunks (the tensor is a whole number of them)
    u32* amax[kMaxBatch];         // slots 1 .. 62: maxima (the repair kernels'), slot 63: status
    int n;
    unsigned wait_ticks;  // bound of the wait at a meeting, in ticks of the 100 MHz wall clock
    int groups;           // tensors held at the same time, each by group_wgs workgroups
    unsigned group_wgs;
    unsigned arrivals;    // words that must carry a tensor's tag: a group's size (a test asks for more, which never come)
    unsigned launch_tag;  // (launch number mod 1023) << 6: two launches that overlap on one GPU never take each other's words for theirs
};

__global__ __launch_bounds__(kResWaves * 64) __attribute__((amdgpu_waves_per_eu(3, 3))) void tensorwise_resident_kernel(const ResidentTable tb) {
    extern __shared__ __attribute__((aligned(16))) uint4 res_lds[];  // [waves][kResLdsVecs][64 lanes], then the give-up flag
    u32* const gave_up = reinterpret_cast<u32*>(res_lds + kResWaves * kResLdsVecs * 64);  // this tensor's outcome
    u32* const red = gave_up + 1;  // [kResWaves] maxima of the waves, then the tensor's maximum
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    // Groups: the launch's workgroups are cut into tb.groups equal groups, each of which holds one tensor at a time
    // (tensor r * groups + grp in round r) and meets only within itself: a tensor a fifth the size of the chip's
    // registers and LDS is held by a fifth of the CUs while the other four fifths hold four more.  Workgroups beyond
    // the last group have nothing to do.
    const unsigned grp = blockIdx.x / tb.group_wgs;
    if (grp >= (unsigned)tb.groups || (int)grp >= tb.n) return;  // (uniform; no barrier has been reached)
    const unsigned first_wg = grp * tb.group_wgs;  // the group's first workgroup = its first word of the meeting array
    const unsigned gw = (blockIdx.x - first_wg) * (unsigned)kResWaves + (unsigned)wave;  // the wave's number in its group
    const unsigned nw = tb.group_wgs * (unsigned)kResWaves;
    uint4* const my_lds = res_lds + wave * (kResLdsVecs * 64) + lane;
    if (threadIdx.x == 0) *gave_up = 0u;
    // Chunk i of the wave is chunk gw + i * nw of the tensor: at any moment the waves of a group read one compact
    // window that moves through the tensor, as a streaming kernel's workgroups do.  Every wave issues the same loads
    // and stores whatever its share: slots past its last chunk repeat that chunk (a wave without any repeats a chunk
    // of another wave), which changes neither the maximum nor a stored byte - branches around the loads would make
    // the compiler wait for every load in flight at each use of one.
    // Addresses are a scalar base (the tensor), a scalar offset (the slot's chunk) and one per-lane offset that is the
    // same for every slot of a tensor: buffer loads and stores, so that no slot needs address registers of its own.
    struct Geo {
        u32 lane_vec;  // vector index of the wave's chunk 0, plus the lane
        int lastc;     // index of the wave's last chunk
    };
    auto geo = [&](int t) {
        const unsigned nchunks = tb.nchunks[t];
        const int cnt = nchunks > gw ? (int)((nchunks - gw + nw - 1) / nw) : 0;
        const unsigned cb = gw < nchunks ? gw : gw % nchunks;
        return Geo{cb * 64u + (u32)lane, cnt > 0 ? cnt - 1 : 0};
    };
    const u32 stride = nw * 64u;  // vectors between two chunks of a wave
    auto slot_vec = [&](const Geo& g, int i) { return (u32)(i < g.lastc ? i : g.lastc) * stride; };  // scalar
    auto load = [&](__amdgpu_buffer_rsrc_t rx, const Geo& g, int i) {  // streaming 16-byte load of the wave's chunk i
        const u32x4 v = __builtin_amdgcn_raw_buffer_load_b128(rx, g.lane_vec * 16u, slot_vec(g, i) * 16u, 2);
        return make_uint4(v[0], v[1], v[2], v[3]);
    };
    auto store = [&](__amdgpu_buffer_rsrc_t rq, const Geo& g, int i, uint2 o) {
        u32x2 v;
        v[0] = o.x;
        v[1] = o.y;
        __builtin_amdgcn_raw_buffer_store_b64(v, rq, g.lane_vec * 8u, slot_vec(g, i) * 8u, 2);
    };
    auto rsrc = [&](const void* base) {
        return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, 0xFFFFFFFF, 0x00020000);
    };
    // Chunks 0 .. kResLdsVecs - 1 of the wave live in LDS and pass through the first register slots; chunk
    // kResLdsVecs + r lives in register slot r.
    // Direct-to-LDS loads of the next tensor and the reads of this one's LDS slots: the reads are written as
    // instructions of their own, which the compiler does not take for LDS accesses - behind a direct-to-LDS load it
    // would otherwise wait for every load in flight before each of them.
    typedef __attribute__((address_space(3))) void lds_void;
    uint8_t* const wave_lds = reinterpret_cast<uint8_t*>(res_lds + wave * (kResLdsVecs * 64));
    const u32 lds_lane = (u32) reinterpret_cast<uintptr_t>((lds_void*)my_lds);
    auto load_lds = [&](__amdgpu_buffer_rsrc_t rx, const Geo& g, int l) {  // the wave's chunk l, 16 bytes per lane, to its LDS slot l
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rx, (lds_void*)(wave_lds + l * 1024), 16, g.lane_vec * 16u, slot_vec(g, l) * 16u, 0, 2);
    };
    uint4 keep[kResRegVecs];
    Geo g = geo((int)grp);
    u32 m = 0;
    // ---- the first tensor's loads: kResDepth in flight per wave, issued in chunk order, straight into the registers
    // that keep them
    {
        constexpr int kResDepth = 8;
        const __amdgpu_buffer_rsrc_t rx = rsrc(tb.x[grp]);
#pragma unroll
        for (int l = 0; l < kResDepth; ++l) keep[l] = load(rx, g, l);
#pragma unroll
        for (int l = 0; l < kResLdsVecs; ++l) {
            m = absmax8(m, keep[l]);
            my_lds[l * 64] = keep[l];
            if (l + kResDepth < kResLdsVecs) keep[l + kResDepth] = load(rx, g, l + kResDepth);
        }
#pragma unroll
        for (int r = 0; r < kResDepth; ++r) keep[r] = load(rx, g, kResLdsVecs + r);
#pragma unroll
        for (int r = 0; r < kResRegVecs; ++r) {
            m = absmax8(m, keep[r]);
            if (r + kResDepth < kResRegVecs) keep[r + kResDepth] = load(rx, g, kResLdsVecs + r + kResDepth);
        }
    }
    for (int t = (int)grp, round = 0; t < tb.n; t += tb.groups, ++round) {
        // here the wave holds tensor t and m is the lane's maximum of it
        {
            const u32 w = wave_max(pk_fold(m));
            if (lane == 0) red[wave] = w;
        }
        // ---- while the workgroups meet, memory has nothing to do: every wave but the one that reads the meeting words
        // (whose reads would queue behind it) touches the lines of its first kResTouch chunks of the next tensor, one
        // dword per line, so that they are on their way into the caches during the meeting; the phase behind the meeting
        // asks for those chunks first.  (Through a descriptor of no bytes where there is nothing to touch.  A tensor that
        // takes this kernel has more chunks than its group has waves: chunk gw exists.)  Measured: 37.8 against 38.2 us
        // per 136 MB tensor with two chunks, nothing with one or three, slower with four and more.
        u32 touched;
        {
            const bool touch = wave != 0 && t + tb.groups < tb.n;
            const int tn = touch ? t + tb.groups : t;
            const u32 ci = (u32)(lane >> 3) < (u32)kResTouch ? (u32)(lane >> 3) : (u32)kResTouch - 1u;
            u32 c = gw + ci * nw;
            c = c < tb.nchunks[tn] ? c : gw;
            const __amdgpu_buffer_rsrc_t rt = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint4*>(tb.x[tn]), 0, touch ? 0xFFFFFFFF : 0, 0x00020000);
            touched = __builtin_amdgcn_raw_buffer_load_b32(rt, c * 1024u + (u32)(lane & 7) * 128u, 0, 0);
        }
        // ---- the meeting.  The workgroup's maximum goes, tagged with the tensor's number, to the workgroup's own word
        // of the meeting array (side t & 1) by one atomic whose result nobody waits for; the first wave then reads all
        // the workgroups' words until every one carries the tag, and has the tensor's maximum in hand when they do:
        // one trip to memory and one back, where a counter costs three in a row (publish, count, read the maxima).  All
        // of it by device-scope atomics, which act at the memory side of the XCDs' L2s, so no cache needs writing back or
        // invalidating (a release or acquire fence at device scope does both, tens of microseconds each).  A word is
        // reused two tensors later, when every workgroup has long read it: nobody reaches tensor t + 2 before all have
        // met at t + 1.
        __syncthreads();
        if (wave == 0) {
            u32 w = 0;
#pragma unroll
            for (int k = 0; k < kResWaves; ++k) w = umax(w, red[k]);
            const u32 tag = (tb.launch_tag | (u32)(t + 1)) << 16;  // this launch's number, then the tensor's
            u32* const side = &g_meet[round & 1][first_wg];  // the group's words
            if (lane == 0) {
                const u32 old = __hip_atomic_fetch_max(side + (blockIdx.x - first_wg), tag | w, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                (void)old;  // not used: the atomic is sent and forgotten
            }
            const uint64_t since = __builtin_amdgcn_s_memrealtime();
            bool met = false, lost = false;
            u32 mx = 0;
            for (;;) {
                // (words of workgroups that do not exist - a test asks for more arrivals than the grid has - never get a tag)
                bool all = true, any_abort = false;
                mx = 0;
                // (256 words per round of four loads that are in flight together: one trip for a GPU of 256 CUs; an
                // index past the last word reads the last word once more)
                for (unsigned base = 0; base < tb.arrivals; base += 256) {
                    u32 v[4];
#pragma unroll
                    for (int k = 0; k < 4; ++k) {
                        const unsigned i = base + (unsigned)(k * 64 + lane);
                        v[k] = __hip_atomic_load(side + (i < tb.arrivals ? i : tb.arrivals - 1), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    }
#pragma unroll
                    for (int k = 0; k < 4; ++k) {
                        all = all && (v[k] & 0xFFFF0000u) == tag;
                        any_abort = any_abort || (v[k] & 0xFFFF0000u) == kMeetAbort;
                        mx = umax(mx, v[k] & 0xFFFFu);
                    }
                }
                met = __builtin_amdgcn_ballot_w64(!all) == 0;
                lost = __builtin_amdgcn_ballot_w64(any_abort) != 0;
                if (met || lost) break;
                if (__builtin_amdgcn_s_memrealtime() - since > (uint64_t)tb.wait_ticks) {
                    lost = true;
                    break;
                }
            }
            if (met && !lost) {
                mx = wave_max(mx);
                if (lane == 0) red[kResWaves] = mx;  // (a word of its own: red[0] is written again before every wave has read this)
            } else {
                // Given up (by this workgroup's clock or because another workgroup says so): this tensor and the ones
                // behind it go to the repair kernels, the other workgroups are told through both sides of the meeting
                // array, and the workgroup leaves.  A workgroup that had already seen this meeting complete goes on to
                // store its part of the tensor - the same bytes the repair writes - and learns at the next meeting.
                if (lane == 0) {
                    *gave_up = 1u;
                    for (int u = t - (int)grp; u < tb.n; ++u)  // from the first tensor of this round on
                        __hip_atomic_store(tb.amax[u] + kStatusSlot, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    __hip_atomic_fetch_max(&g_meet[0][blockIdx.x], kMeetAbort, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    __hip_atomic_fetch_max(&g_meet[1][blockIdx.x], kMeetAbort, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                }
            }
        }
        __syncthreads();
        if (*gave_up != 0u) {
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // direct-to-LDS loads still on their way
            break;
        }
        // ---- cast what is held and store it; every slot that has been stored is requested anew at once with the next
        // tensor's chunk, so the stores of this tensor and the loads of the next share the memory system.  Behind the
        // last tensor the loads go through a descriptor of no bytes: they fetch nothing.
        // (Nothing is in flight here: the loads of this tensor were awaited before its maximum was formed.  Said with the
        // builtin, which the compiler takes into account - it cannot see the waits written as instructions, and would
        // otherwise put a wait for the kept registers' loads in front of every use of one, inside the phase below,
        // where it would bound the stores and loads in flight.)
        __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0), the other counters left alone
        asm volatile("" ::"v"(touched));         // (the touch load's register stays the wave's until it has landed)
        const float amax = amax_from_bits(red[kResWaves]);
        const float scale = scale_from_amax(amax);
        if (gw == 0 && lane == 0) *tb.scale[t] = scale;
        const Divider d(scale);
        const __amdgpu_buffer_rsrc_t rq = rsrc(tb.q[t]);
        const bool more = t + tb.groups < tb.n;
        const Geo gn = more ? geo(t + tb.groups) : g;
        const __amdgpu_buffer_rsrc_t rx =
            more ? rsrc(tb.x[t + tb.groups]) : __builtin_amdgcn_make_buffer_rsrc(const_cast<uint4*>(tb.x[t]), 0, 0, 0x00020000);
        auto lds_slot = [&](int l) {  // this tensor's LDS slot l, read before the slot is requested anew
            u32x4 v;
            asm volatile("ds_read_b128 %0, %1 offset:%2\n\ts_waitcnt lgkmcnt(0)" : "=v"(v) : "v"(lds_lane), "n"(l * 1024) : "memory");
            return make_uint4(v[0], v[1], v[2], v[3]);
        };
        // (slots past the wave's last chunk hold copies of it: not stored - a wave with no chunk of its own stores the
        // one it copied once more, the same bytes)
        int last_store = g.lastc;
        if (!d.finite) {
            // a scale that is infinite or NaN: the bytes are stored here, and the code below, which every other tensor
            // takes, only requests the next tensor (one definition of the kept registers: with a second one in this
            // branch the compiler spills most of them)
#pragma unroll
            for (int l = 0; l < kResLdsVecs; ++l)
                if (l <= g.lastc) store(rq, g, l, cast8_nonfinite_scale(my_lds[l * 64], scale));
#pragma unroll
            for (int r = 0; r < kResRegVecs; ++r)
                if (kResLdsVecs + r <= g.lastc) store(rq, g, kResLdsVecs + r, cast8_nonfinite_scale(keep[r], scale));
            last_store = -1;
        }
#pragma unroll
        for (int l = 0; l < kResLdsVecs; ++l) {
            const uint4 v = lds_slot(l);
            if (l <= last_store) store(rq, g, l, cast8_finite(v, d));
            load_lds(rx, gn, l);
            __builtin_amdgcn_sched_barrier(0);
        }
#pragma unroll
        for (int r = 0; r < kResRegVecs; ++r) {
            if (kResLdsVecs + r <= last_store) store(rq, g, kResLdsVecs + r, cast8_finite(keep[r], d));
            keep[r] = load(rx, gn, kResLdsVecs + r);
            __builtin_amdgcn_sched_barrier(0);
        }
        g = gn;
        if (!more) {
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // (the empty loads still write LDS: none is in flight when the wave ends)
            break;
        }
        // ---- the next tensor's maximum, slot by slot as the loads land (they return in order).  The LDS slots were
        // requested first: of the 2 x kResVecs stores and loads of the phase at most 63 are still in flight behind the
        // wait below, so the 2 x kResLdsVecs oldest - the LDS slots' - are done, and their part of the maximum is formed
        // while the register slots' loads are still landing (read by instructions written out, see lds_slot)
        static_assert(2 * kResVecs - 63 >= 2 * kResLdsVecs, "a wait for all but 63 operations covers the LDS slots");
        m = 0;
        asm volatile("s_waitcnt vmcnt(63)" ::: "memory");
#pragma unroll
        for (int l = 0; l < kResLdsVecs; ++l) m = absmax8(m, lds_slot(l));
#pragma unroll
        for (int r = 0; r < kResRegVecs; ++r) m = absmax8(m, keep[r]);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    }
}

// ---------------------------------------------------------------------------
// The two passes over exactly those tensors of a resident launch whose status word says that the launch gave them
// up.  Small fixed grids behind every resident launch: a workgroup reads the status words of the launch's tensors
// with one wave-wide load and leaves at once when none is set, which is the normal case.  Maxima go to slots
// 1 .. 62 of the tensor's amax slots (the resident kernel writes none of them: its maxima travel through the
// meeting array); slot 63 is the status word.
// ---------------------------------------------------------------------------
constexpr int kRepairBlocksPerCu = 8;

__device__ __forceinline__ uint64_t repair_mask(const ResidentTable& tb) {  // bit t: tensor t was given up
    const int lane = threadIdx.x & 63;
    u32 st = 0;
    if (lane < tb.n) st = tb.amax[lane][kStatusSlot];
    return __builtin_amdgcn_ballot_w64(st != 0u);
}

__global__ __launch_bounds__(256) void tensorwise_repair_amax_kernel(const ResidentTable tb) {
    __shared__ u32 red[4];
    uint64_t mask = repair_mask(tb);
    while (mask) {
        const int t = __builtin_ctzll(mask);
        mask &= mask - 1;
        const int64_t nvec = (int64_t)tb.nchunks[t] * 64;
        const uint4* const x = tb.x[t];
        u32 m = 0;
        for (int64_t base = (int64_t)blockIdx.x * kChunkVecs; base < nvec; base += (int64_t)gridDim.x * kChunkVecs) {
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const int64_t idx = base + threadIdx.x + 256 * i;
                if (idx < nvec) m = absmax8(m, ld16<true>(x + idx));
            }
        }
        m = wave_max(pk_fold(m));
        __syncthreads();  // red is free again
        if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = m;
        __syncthreads();
        if (threadIdx.x == 0) {
            m = umax(umax(red[0], red[1]), umax(red[2], red[3])) << 16;
            if (m) atomicMax(tb.amax[t] + 1 + blockIdx.x % (unsigned)(kMaxSlots - 1), m);
        }
    }
}

__global__ __launch_bounds__(256) void tensorwise_repair_cast_kernel(const ResidentTable tb) {
    uint64_t mask = repair_mask(tb);
    while (mask) {
        const int t = __builtin_ctzll(mask);
        mask &= mask - 1;
        const int slot = threadIdx.x & 63;
        const float amax = __uint_as_float(wave_max(slot >= 1 && slot < kStatusSlot ? tb.amax[t][slot] : 0u));
        const float scale = scale_from_amax(amax);
        if (blockIdx.x == 0 && threadIdx.x == 0) *tb.scale[t] = scale;
        const Divider d(scale);
        const int64_t nvec = (int64_t)tb.nchunks[t] * 64;
        const uint4* const x = tb.x[t];
        uint2* const q = tb.q[t];
        for (int64_t base = (int64_t)blockIdx.x * kChunkVecs; base < nvec; base += (int64_t)gridDim.x * kChunkVecs) {
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const int64_t idx = base + threadIdx.x + 256 * i;
                if (idx < nvec) st8<true>(q + idx, cast8(ld16<true>(x + idx), d));
            }
        }
    }
}

// how many of the n tensors of a workspace carry a set status word
__global__ __launch_bounds__(256) void tensorwise_status_kernel(const u32* slots, int64_t n, int32_t* out) {
    __shared__ int red[4];
    int c = 0;
    for (int64_t i = threadIdx.x; i < n; i += 256) c += slots[i * kAmaxSlots + kStatusSlot] != 0u;
    for (int off = 32; off; off >>= 1) c += __shfl_xor(c, off);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = c;
    __syncthreads();
    if (threadIdx.x == 0) *out = red[0] + red[1] + red[2] + red[3];
}

enum : int { kPhaseAmax = 1, kPhaseCast = 2 };

// Which tensors of a call a helper below takes: all of them, those that take the resident kernel, or the others.
enum : int { kTakeAll = 0, kTakeResident = 1, kTakeOthers = 2 };
static bool resident_fits(const cfp8_tensor_desc& d, int cus);
static inline bool taken(const cfp8_tensor_desc& d, int take, int cus) {
    return take == kTakeAll || resident_fits(d, cus) == (take == kTakeResident);
}

// pass 1 and / or pass 2 as launches of their own over the tensors of the call that `take` selects
static void two_pass(const cfp8_tensor_desc* descs, int64_t n, u32* slots, int phases, int take, int cus, hipStream_t st) {
    // Tensors are taken in batches of at most kMaxBatch entries; with both phases requested each
    // batch runs pass 1 then pass 2 back to back.  Every access streams past the caches (non-temporal
    // loads in both passes, non-temporal stores).  Measured on MI355X: few large launches with
    // streaming accesses beat small batches that would let pass 2 hit the 256 MiB memory-side cache,
    // because every launch pays a ramp-up and a tail.
    int64_t i = 0;
    while (i < n) {
        // the tensors of this batch: at most kMaxBatch, and few enough chunks for one grid
        int64_t idx[kMaxBatch];
        uint64_t chunks = 0;
        int count = 0;
        while (i < n && count < kMaxBatch) {
            if (!taken(descs[i], take, cus)) {
                ++i;
                continue;
            }
            uint64_t nc = (uint64_t)((descs[i].numel / 8 + kChunkVecs - 1) / kChunkVecs);
            if (nc == 0) nc = 1;  // a tensor with no element still owns one workgroup: it writes the scale
            if (count > 0 && chunks + nc > 0x7FFFFFFFull) break;
            chunks += nc;
            idx[count++] = i++;
        }
        if (count == 0) break;
        // pass 1 gives a workgroup `per` chunks, pass 2 one: two tables that differ in the workgroup prefix
        for (int phase = kPhaseAmax; phase <= kPhaseCast; phase <<= 1) {
            if (!(phases & phase)) continue;
            TensorTable tb;
            tb.n = count;
            tb.per = phase == kPhaseAmax ? amax_chunks_per_block(chunks) : 1;
            unsigned blocks = 0;
            for (int k = 0; k < count; ++k) {
                const cfp8_tensor_desc& d = descs[idx[k]];
                const int64_t nvec = d.numel / 8;
                uint64_t nc = (uint64_t)((nvec + kChunkVecs - 1) / kChunkVecs);
                if (nc == 0) nc = 1;
                tb.x[k] = static_cast<const uint4*>(d.x);
                tb.q[k] = static_cast<uint2*>(d.q);
                tb.scale[k] = d.scale;
                tb.nvec[k] = nvec;
                tb.amax[k] = slots + idx[k] * kAmaxSlots;
                tb.first_block[k] = blocks;
                blocks += (unsigned)((nc + tb.per - 1) / tb.per);
            }
            tb.first_block[count] = blocks;
            if (phase == kPhaseAmax) hipLaunchKernelGGL(tensorwise_amax_kernel<true>, dim3(blocks), dim3(256), 0, st, tb);
            else if (phases == kPhaseCast) hipLaunchKernelGGL((tensorwise_cast_kernel<true, true, true>), dim3(blocks), dim3(256), 0, st, tb);
            else hipLaunchKernelGGL((tensorwise_cast_kernel<true, true, false>), dim3(blocks), dim3(256), 0, st, tb);
        }
    }
}

// ---- the resident form: host side ---------------------------------------------------------------
static int resident_cus() {  // compute units of the current device, 0 if unknown
    static std::atomic<int> cached[kMaxDevices];
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) {
        (void)hipGetLastError();
        return 0;
    }
    int c = cached[dev].load(std::memory_order_relaxed);
    if (c > 0) return c;
    if (hipDeviceGetAttribute(&c, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || c <= 0 || c >= kMeetSlots) {
        (void)hipGetLastError();
        return 0;
    }
    static std::atomic<bool> raised[kMaxDevices];
    if (!raised[dev].load(std::memory_order_acquire)) {
        if (hipFuncSetAttribute(reinterpret_cast<const void*>(tensorwise_resident_kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                (int)kResLdsBytes) != hipSuccess) {
            (void)hipGetLastError();
            return 0;
        }
        raised[dev].store(true, std::memory_order_release);
    }
    cached[dev].store(c, std::memory_order_relaxed);
    return c;
}

// How many tensors like this one the chip holds at the same time (0: the tensor does not take the resident kernel).
// A tensor must be a whole number of 1 KiB chunks; G of them are resident together, each held by cus / G workgroups,
// for the largest G <= kResMaxGroups whose groups still hold the tensor, and the tensor must fill at least three
// quarters of its group: a round of G tensors costs the resident kernel about 5 us plus 0.52 us per million elements
// (every wave walks all its slots and the groups meet in the middle), the two launches 0.82 us per million.
constexpr int kResMaxGroups = 8;
static int resident_groups(const cfp8_tensor_desc& d, int cus) {
    if (d.numel <= 0 || d.numel % 512) return 0;
    const uint64_t nc = (uint64_t)(d.numel / 512);
    for (int g = kResMaxGroups; g >= 1; --g) {
        const uint64_t cap = (uint64_t)(cus / g) * kResWaves * kResVecs;
        if (cus / g >= 1 && nc <= cap) return nc * 4 >= cap * 3 ? g : 0;
    }
    return 0;
}
static bool resident_fits(const cfp8_tensor_desc& d, int cus) { return resident_groups(d, cus) != 0; }

// The tensors of the call that take the resident kernel: one class of group count after the other, kMaxBatch per launch
static void resident_all(const cfp8_tensor_desc* descs, int64_t n, u32* slots, int cus, hipStream_t st) {
    for (int groups = 1; groups <= kResMaxGroups; ++groups) {
        int64_t i = 0;
        while (i < n) {
            ResidentTable tb;
            int count = 0;
            for (; i < n && count < kMaxBatch; ++i) {
                const cfp8_tensor_desc& d = descs[i];
                if (resident_groups(d, cus) != groups) continue;
                tb.x[count] = static_cast<const uint4*>(d.x);
                tb.q[count] = static_cast<uint2*>(d.q);
                tb.scale[count] = d.scale;
                tb.nchunks[count] = (unsigned)(d.numel / 512);
                tb.amax[count] = slots + i * kAmaxSlots;
                ++count;
            }
            if (count == 0) break;
            tb.n = count;
            tb.groups = groups;
            tb.group_wgs = (unsigned)(cus / groups);
            tb.wait_ticks = g_resident_wait_us.load(std::memory_order_relaxed) * 100u;  // the wall clock runs at 100 MHz
            tb.arrivals = tb.group_wgs + g_resident_extra_arrivals.load(std::memory_order_relaxed);
            if (tb.arrivals > (unsigned)kMeetSlots) tb.arrivals = (unsigned)kMeetSlots;
            static std::atomic<unsigned> launches{0};
            tb.launch_tag = (launches.fetch_add(1, std::memory_order_relaxed) % 1023u) << 6;
            static_assert(kMaxBatch < 64, "a tensor's number fits six bits");
            // all workgroups must be resident together: one per CU, and a workgroup fills a CU (all of its LDS), so on a
            // GPU that no other grid holds they are
            hipLaunchKernelGGL(tensorwise_meet_clear_kernel, dim3(1), dim3(256), 0, st);
            hipLaunchKernelGGL(tensorwise_resident_kernel, dim3((unsigned)cus), dim3(kResWaves * 64), kResLdsBytes, st, tb);
            // tensors that the launch gave up (none, normally) are redone as two ordinary passes
            hipLaunchKernelGGL(tensorwise_repair_amax_kernel, dim3((unsigned)(cus * kRepairBlocksPerCu)), dim3(256), 0, st, tb);
            hipLaunchKernelGGL(tensorwise_repair_cast_kernel, dim3((unsigned)(cus * kRepairBlocksPerCu)), dim3(256), 0, st, tb);
        }
    }
}

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
    // Both passes requested: tensors that fit the chip (registers + LDS of all CUs) take the resident kernel, which
    // reads them once; the others take pass 1 and pass 2 as launches of their own.
    int cus = 0;
    if (phases == (kPhaseAmax | kPhaseCast) && g_resident_enabled.load(std::memory_order_relaxed)) cus = resident_cus();
    if (cus <= 0) {
        two_pass(descs, n, slots, phases, kTakeAll, 0, st);
        return check_launch("quant_tensorwise");
    }
    // (the order in which tensors are quantised is free: the large ones first, then the rest in full batches)
    resident_all(descs, n, slots, cus, st);
    two_pass(descs, n, slots, phases, kTakeOthers, cus, st);
    return check_launch("quant_tensorwise");
}

// ---- amax slots owned by the library, for callers that cannot allocate -------------------------
// One copy of this array lives on every GPU the library's code object is loaded on, at that GPU's
// own address.  In host code the name below is only a handle for hipGetSymbolAddress; kernels and
// every other use of the memory take the per-device pointer looked up in static_slots().
constexpr int kStaticMaxTensors = CFP8_TENSORWISE_STATIC_MAX_TENSORS;
static __device__ __align__(256) u32 scratch[kStaticMaxTensors * kAmaxSlots];

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

extern "C" int cfp8_tensorwise_resident(int enable) {
    if (enable < 0) return cfp8::g_resident_enabled.load(std::memory_order_relaxed);
    return cfp8::g_resident_enabled.exchange(enable ? 1 : 0, std::memory_order_relaxed);
}

extern "C" int cfp8_tensorwise_resident_tuning(int64_t wait_us, int extra_arrivals) {
    if (wait_us > 0) cfp8::g_resident_wait_us.store((unsigned)(wait_us < 30000000 ? wait_us : 30000000), std::memory_order_relaxed);
    if (extra_arrivals >= 0) cfp8::g_resident_extra_arrivals.store((unsigned)(extra_arrivals < 1024 ? extra_arrivals : 1024), std::memory_order_relaxed);
    return CFP8_OK;
}

extern "C" int cfp8_tensorwise_status(const float* amax_ws, int64_t n, int32_t* given_up, void* stream) {
    using namespace cfp8;
    if (n < 0 || n > (1ll << 24)) return set_error(CFP8_EINVAL, "tensorwise_status: bad tensor count");
    if (!given_up) return set_error(CFP8_EINVAL, "tensorwise_status: null pointer");
    if (int rc = check_device()) return rc;
    const u32* slots = reinterpret_cast<const u32*>(amax_ws);
    if (!slots) {  // the library's own slots, those of cfp8_quant_tensorwise_multi_static
        if (n > kStaticMaxTensors) return set_error(CFP8_EINVAL, "tensorwise_status: the library's own slots hold %d tensors", kStaticMaxTensors);
        u32* own = nullptr;
        if (int rc = static_slots(&own)) return rc;
        slots = own;
    }
    hipLaunchKernelGGL(tensorwise_status_kernel, dim3(1), dim3(256), 0, static_cast<hipStream_t>(stream), slots, n, given_up);
    return check_launch("tensorwise_status");
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
