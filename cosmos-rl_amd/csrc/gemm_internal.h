// What the GEMM translation units of libcosmosfp8 share: the argument block of every GEMM kernel, the launch
// record behind cfp8_gemm_dispatch_info, and a few device helpers.
#pragma once

#include <atomic>

#include "cfp8_common.h"

namespace cfp8 {

enum : int { kRowwise = 0, kBlock = 1, kGrouped = 2 };

struct GemmArgs {
    const uint8_t* a;   // activations fp8 [M, K]
    const uint8_t* b;   // weights fp8 [N, K] (grouped: [E, N, K])
    const float* sa;    // rowwise [M]; block [M, K/128]
    const float* sb;    // rowwise [N]; block: see strides
    const int32_t* m_indices;
    void* out;
    int64_t ld_a, ld_b, ld_out;
    int64_t sb_stride_n, sb_stride_k, sb_stride_e;
    int M, N, K;
    int tiles_m, tiles_n;
    // split-K (rowwise, at most 64 tokens): fp32 partial sums [k_slices, M, N] in caller-provided memory
    float* partial;
    size_t partial_bytes;
    int k_slices, slice_steps;
    // grouped GEMM with the SwiGLU + 1x128 quantisation epilogue: scales of the quantised product [M, N / 256]
    float* h_scales;
    int64_t ld_hs;
    // gemm_grouped_xres_kernel: pieces along N of the tile rows that are not whole-row units
    int unit_parts;
    // gemm_rowwise_256p_kernel: tiles of the last, at most half-full round, computed as quarter tiles by all workgroups
    int tail_tiles;
};

// ---- host side (gemm_fp8.hip) ---------------------------------------------
bool dry_run();                                                                   // launches are being recorded, not made
bool note_launch(const char* kernel, unsigned grid, unsigned block, size_t lds);  // true: launch for real
int raise_lds_limit(const void* fn, size_t lds, std::atomic<bool>& flag);         // once per (device, function)
int device_slot();                                                                // 0..63, 64 = not cached
int cu_count();                                                                   // compute units of the current device

// ---- units of the kernels in which a workgroup walks rows of tiles ----------
// The schedule for tiles_m tile rows of tiles_n tiles on `cus` workgroups: one workgroup per CU.  Tile rows beyond the
// last full round of whole rows (all of them, with fewer tile rows than CUs) are cut along N into `parts` pieces; a
// unit costs its tiles plus `unit_cost` tiles for starting it, and `parts` is the count with the shortest last round.  `fill` is the share of the run's tile slots (CUs x length of the longest workgroup's run) that hold tiles.
struct UnitPlan {
    int parts;
    int64_t blocks;
    double fill;
};
inline UnitPlan unit_plan(int tiles_m, int tiles_n, int cus, int unit_cost) {
    const int rem = tiles_m >= cus ? tiles_m % cus : tiles_m;
    int parts = 1;
    int64_t span = (int64_t)(tiles_m / cus) * (tiles_n + unit_cost);
    if (rem) {
        int64_t best = INT64_MAX;
        for (int q = 1; q <= tiles_n; ++q) {
            const int64_t rounds = ((int64_t)rem * q + cus - 1) / cus;
            const int64_t cost = rounds * ((tiles_n + q - 1) / q + unit_cost);
            if (cost < best) best = cost, parts = q;
        }
        span += best;
    }
    const int64_t units = (int64_t)(tiles_m - rem) + (int64_t)rem * parts;
    int64_t blocks = units < cus ? units : cus;
    // (the kernel takes tiles_m / gridDim.x * gridDim.x tile rows for whole-row units: with fewer tile rows than CUs
    // the grid must exceed the tile rows unless every unit is a whole row anyway)
    if (tiles_m < cus && parts == 1) blocks = tiles_m;
    return {parts, blocks, (double)tiles_m * tiles_n / ((double)cus * (double)span)};
}

// gemm_grouped_xres.hip
int launch_grouped_xres(GemmArgs& p, int out_dtype, hipStream_t st);
bool grouped_xres_pays(const GemmArgs& p);  // enough of the CUs' tile slots would hold tiles

// ---- device side ------------------------------------------------------------
#define CFP8_PHASE_END() __builtin_amdgcn_sched_barrier(0)
// Wait until at most `vm` of this wave's loads are outstanding and its LDS reads are done, then the workgroup barrier.
// Written out as instructions: in front of a barrier it knows of, the compiler waits for every load it has issued,
// including the direct-to-LDS loads that are meant to stay in flight across the barrier.
#define CFP8_WAIT_BARRIER(vm) asm volatile("s_waitcnt vmcnt(" #vm ") lgkmcnt(0)\n\ts_barrier" ::: "memory")

// One int of a table that no kernel writes, by a scalar load.  Behind the first store of a kernel the compiler turns
// such a read into a vector load, and then waits for every load in flight, the direct-to-LDS ones included.
__device__ __forceinline__ int scalar_table_load(const int32_t* table, int index) {
    const int32_t* const ptr = table + index;  // uniform
    int v;
    asm volatile("s_load_dword %0, %1, 0x0\n\ts_waitcnt lgkmcnt(0)" : "=s"(v) : "s"(ptr) : "memory");
    return v;
}

}  // namespace cfp8
