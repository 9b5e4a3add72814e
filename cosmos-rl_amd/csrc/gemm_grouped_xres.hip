// Grouped block-scaled FP8 GEMM for a short K with the activation fragments resident in registers.
// A translation unit of its own because it is compiled with -mllvm -amdgpu-mfma-vgpr-form: its kernel multiplies
// out of the accumulation-register half of the register file (the resident activation fragments live there) into
// ordinary vector registers (the products are consumed by VALU instructions, which cannot read the other half);
// the compiler's default for a kernel with all 512 registers is the opposite, and costs a register move per
// product register.
#include <stdio.h>
#include <stdlib.h>
#include <type_traits>

#include "gemm_internal.h"

namespace cfp8 {

// ---------------------------------------------------------------------------
// Grouped block-scaled GEMM for a short K (K / 128 = 5 or 6: the down projection of a MoE expert, K = the
// intermediate size), 128 x 256 tiles, FOUR wavefronts (one per SIMD, all 512 registers each).  With so few K steps a
// tile's activation rows fit in registers for the whole of K: a wave keeps the MFMA fragments of its 64 rows
// (4 x tiles x K / 128 steps x 8 registers, at most 192 - only the matrix instructions read them, so they can live in
// the accumulation-register half of the file) and reuses them for every tile of its unit, a run of tiles along N.
// Only the weight tiles pass through LDS: a third less traffic through the load path and half the fragment reads of
// the eight-wave kernel's 64 x 64 blocks (a wave tile is 64 x 128: the operand economy of the 256 x 256 rowwise
// kernel), which is what bounds that kernel at K = 768.
//
// Units.  One workgroup per CU walks units b, b + gridDim.x, ... (those that are not padding).  Loading a unit's
// fragments costs about as much as a tile (each lane fetches its own 32 bytes of 16 different rows: 16 cache lines
// per load instruction), so units are as long as the balance between the CUs allows: the first
// (tile rows / gridDim.x) * gridDim.x tile rows are whole rows of tiles, one unit each; the remaining tile rows are
// cut into `unit_parts` pieces along N, so that the last round of units covers (nearly) every CU with an equal share.
//
// The weight tiles of consecutive K steps, tiles and units form one stream of direct-to-LDS loads through a ring of
// four stages (a load has two K steps to land).  A K step is eight w tiles of four MFMAs each; the products of a w
// tile are folded into the accumulators (acc += product * activation scale * weight scale, VALU) under the MFMAs of
// the next one, the fragment of w tile i + 3 is read while w tile i is multiplied, and the workgroup's one barrier
// per step sits in the middle of the step: behind it the next step's stage has landed (its first fragments are read
// in the second half) and the stage that the step before used is free for the loads of three steps ahead.
//
// A tile has no epilogue of its own: its result leaves under the next tile's K steps, so that the conversions, the
// turn through LDS and the stores run under MFMAs instead of leaving the matrix pipe idle, and the stores reach memory
// spread over the run instead of in bursts from all CUs at once.  bf16: at its end a tile is packed into 64 registers;
// in the second half of K step j of the next tile (j = 0 .. 3) a wave writes the 16 rows of x tile j to its LDS buffer, at the
// beginning of step j + 1 it reads them back as row segments of 256 contiguous bytes, and it stores those two w tiles
// later, all in the half of a step that issues no weight loads (16 bytes per lane, 4 rows per store
// instruction - a store that touches 16 rows costs the address unit four times as much).  fp32: a lane owns 16
// contiguous bytes as it is, and the tile is stored from the accumulators during the first half of the next tile's
// first step, pair of w tiles by pair of w tiles, just ahead of that step's first writes to them (a tile's first step
// writes acc = product * scale).  Rows that do not belong to the unit's expert get an offset past the end of the
// buffer descriptor and the hardware drops their stores (the barriers count on a fixed number of stores); the very
// first tile "stores" a previous tile that does not exist in the same way.
//
// Results are the bits of the other block-scaled kernels: the same products in the same order of K.
// Requires M % 128 == 0, N % 256 == 0, weight scales contiguous along K.
// ---------------------------------------------------------------------------
// bf16: the stores that K step k issues for the tile before (x tile k - 1 in steps 1 .. 4); a negative k counts back from
// the end of the tile before
// bf16: the w tile (0 .. 7) of a store step at which each of its four stores is issued (behind that w tile's loads).
// (Measured: where in the step they sit makes no difference to the run time.)
constexpr int kXresStoreAt[4] = {2, 2, 3, 3};
// Is K step k (a negative k counts back from the end of the tile before) one of the four that store?
template <int KT>
constexpr bool xres_store_step(int k) {
    const int kk = ((k % KT) + KT) % KT;
    return kk >= 1 && kk <= 4;
}
// bf16: the vector-memory operations that may still be in flight behind the barrier of K step k (in front of w tile 4)
// once the stage requested two steps earlier has landed: the stores of step k - 2 behind its last load, all of
// step k - 1 (eight loads and its stores), and the stores of this step's first half.
template <int KT>
constexpr int xres_allowed(int k) {
    int n = 8;
    for (int r = 0; r < 4; ++r) {
        if (xres_store_step<KT>(k - 2) && kXresStoreAt[r] == 7) ++n;
        if (xres_store_step<KT>(k - 1)) ++n;
        if (xres_store_step<KT>(k) && kXresStoreAt[r] < 4) ++n;
    }
    return n;
}

template <int KT, bool OUT_F32>
__global__ __launch_bounds__(256) void gemm_grouped_xres_kernel(const GemmArgs p) {
    static_assert(KT >= 5 && KT <= 6, "5 or 6 K steps: the activation fragments stay in registers, and a tile leaves in four of the next tile's steps");
    constexpr int WS = 256 * 128;                  // one weight stage
    constexpr int S = 4;                           // weight stages: the stream's steps g, g + 1 (landed), g + 2, g + 3 (in flight)
    constexpr int NBASE = S * WS;                  // weight scales of the current and the next tile: [wave][2][64] floats
    constexpr int IBASE = NBASE + 4 * 2 * 64 * 4;  // the expert of every row of the current and the next unit: [2][128]
    constexpr int EBASE = IBASE + 2 * 128 * 4;     // bf16: per wave 16 rows of 256 bytes (+ 16) that turn a tile's rows into stores
    constexpr int EST = 272;
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    const int t = threadIdx.x, lane = t & 63;
    const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
    const int wm = wave & 1, wn = wave >> 1;  // rows wm * 64 .. + 63, columns wn * 128 .. + 127 of the tile
    const int lrow = lane & 15, quarter = lane >> 4;
    const int tiles_n = p.tiles_n;
    const int G = (int)gridDim.x;
    const int big = p.tiles_m / G * G;  // tile rows that are units of their own
    const int parts = p.unit_parts;     // pieces of each of the remaining tile rows
    const int units = big + (p.tiles_m - big) * parts;
    typedef __attribute__((address_space(3))) void lds_void;
    constexpr int kWaitVm0 = 0x0F70;  // s_waitcnt vmcnt(0), the other counters left alone

    // unit id -> tile row and range of tiles [t0, t1) along N.  Whole rows: every XCD (workgroup id mod 8) gets one
    // contiguous range of tile rows, so that the workgroups that run side by side on an XCD work on neighbouring rows,
    // mostly of one expert, and share its weight tiles in that XCD's L2.
    auto unit_of = [&](int pid, int& rb, int& t0, int& t1) {
        if (pid < big) {
            rb = (big & 7) == 0 ? (pid & 7) * (big >> 3) + (pid >> 3) : pid;
            t0 = 0;
            t1 = tiles_n;
        } else {
            const int v = pid - big, r = v / parts, piece = v - r * parts;
            rb = big + r;
            t0 = piece * tiles_n / parts;
            t1 = (piece + 1) * tiles_n / parts;
        }
    };
    auto unit_expert = [&](int pid) {
        int rb, t0, t1;
        unit_of(pid, rb, t0, t1);
        return scalar_table_load(p.m_indices, rb * 128);  // groups start on multiples of 128 rows
    };
    auto next_unit = [&](int pid) {  // the next unit of this workgroup that is not padding
        int q = pid + G;
        while (q < units && unit_expert(q) < 0) q += G;
        return q;
    };

    // weight tiles: global -> LDS directly, load i of a K step covers rows (wave + 4 i) * 8 .. + 7 of the tile
    // (row-major stage, 16-byte chunks XOR-ed by f(row), as in gemm_rowwise_256_kernel)
    uint32_t b_step = 32u * (uint32_t)p.ld_b;
    asm volatile("" : "+s"(b_step));
    const uint32_t chunk = (uint32_t)(((lane & 7) ^ ((wave & 1) * 4 + ((lane >> 4) & 1))) << 4);
    const uint32_t vb_lane = (uint32_t)(lane >> 3) * (uint32_t)p.ld_b + chunk;
    auto w_rsrc = [&](int expert, int n0) {
        const uint64_t bw = reinterpret_cast<uint64_t>(p.b) + ((uint64_t)expert * (uint64_t)p.N + (uint64_t)n0 + (uint64_t)wave * 8) * (uint64_t)p.ld_b;
        return __builtin_amdgcn_make_buffer_rsrc(reinterpret_cast<void*>(bw), 0, 0xFFFFFFFF, 0x00020000);
    };
    auto dma_w = [&](__amdgpu_buffer_rsrc_t r, int kt, int stage, int i) {
        __builtin_amdgcn_raw_ptr_buffer_load_lds(r, (lds_void*)(smem + stage * WS + (wave + 4 * i) * 1024), 16, vb_lane,
                                                 (uint32_t)i * b_step + ((uint32_t)kt << 7), 0, 0);
    };
    // the KT block scales of the wave's 128 weight rows of a tile, into the wave's scale slot `par` (4 bytes per lane;
    // lanes beyond KT repeat the last one)
    auto dma_sn = [&](int expert_, int n0_, int par) {
        const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc(
            const_cast<float*>(p.sb) + (int64_t)expert_ * p.sb_stride_e + (int64_t)((n0_ >> 7) + wn) * p.sb_stride_n, 0, 0xFFFFFFFF, 0x00020000);
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, (lds_void*)(smem + NBASE + ((wave * 2 + par) * 64) * 4), 4,
                                                 (uint32_t)(lane < KT ? lane : KT - 1) * 4u, 0, 0, 0);
    };
    const int fsw = ((lrow >> 1) & 1) | (((lrow >> 3) & 1) << 2);
    const int w_off = (wn * 128 + lrow) * 128 + (((2 * quarter) ^ fsw) << 4);
    const int w_off2 = (wn * 128 + lrow) * 128 + (((2 * quarter + 1) ^ fsw) << 4);
    auto frag = [&](int stage, int tile16) {
        const uint8_t* base = smem + stage * WS + tile16 * 2048;
        const i32x4 lo = *reinterpret_cast<const i32x4*>(base + w_off);
        const i32x4 hi = *reinterpret_cast<const i32x4*>(base + w_off2);
        i32x8 r;
        r[0] = lo[0]; r[1] = lo[1]; r[2] = lo[2]; r[3] = lo[3];
        r[4] = hi[0]; r[5] = hi[1]; r[6] = hi[2]; r[7] = hi[3];
        return r;
    };

    // what a wave keeps of its unit: the activation fragments of its 64 rows for every K step and their 1x128 scales
    // (row j * 16 + lrow of x tile j, K step k)
    i32x8 X[KT][4];
    float sm[4][KT];
    const uint32_t vx_lane = (uint32_t)(wm * 64 + lrow) * (uint32_t)p.ld_a + (uint32_t)quarter * 32u;
    uint32_t a_tile16 = 16u * (uint32_t)p.ld_a;
    asm volatile("" : "+s"(a_tile16));
    auto load_unit = [&](int m0, int par) {
        const __amdgpu_buffer_rsrc_t rx = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t*>(p.a) + (int64_t)m0 * p.ld_a, 0, 0xFFFFFFFF, 0x00020000);
#pragma unroll
        for (int k = 0; k < KT; ++k)
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const u32x4 lo = __builtin_amdgcn_raw_buffer_load_b128(rx, vx_lane, (uint32_t)j * a_tile16 + (uint32_t)k * 128u, 0);
                const u32x4 hi = __builtin_amdgcn_raw_buffer_load_b128(rx, vx_lane + 16u, (uint32_t)j * a_tile16 + (uint32_t)k * 128u, 0);
                X[k][j][0] = (int)lo[0]; X[k][j][1] = (int)lo[1]; X[k][j][2] = (int)lo[2]; X[k][j][3] = (int)lo[3];
                X[k][j][4] = (int)hi[0]; X[k][j][5] = (int)hi[1]; X[k][j][6] = (int)hi[2]; X[k][j][7] = (int)hi[3];
            }
        const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(p.sa) + (int64_t)m0 * KT, 0, 0xFFFFFFFF, 0x00020000);
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int k = 0; k < KT; ++k)
                sm[j][k] = __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(rs, (uint32_t)((wm * 64 + j * 16 + lrow) * KT) * 4u, (uint32_t)k * 4u, 0));
        // which rows belong to the unit's expert: the row indices go to LDS (waves 0 and 1, 64 rows each) and are
        // turned into the lanes' row flags at the end of the unit's first tile, several barriers later - consumed
        // here, they would make the wave wait for everything it has just requested
        if (wave < 2) {
            const __amdgpu_buffer_rsrc_t ri = __builtin_amdgcn_make_buffer_rsrc(const_cast<int32_t*>(p.m_indices) + m0 + wave * 64, 0, 0xFFFFFFFF, 0x00020000);
            __builtin_amdgcn_raw_ptr_buffer_load_lds(ri, (lds_void*)(smem + IBASE + (par * 128 + wave * 64) * 4), 4, (uint32_t)lane * 4u, 0, 0, 0);
        }
    };
    // the lane's row flags of the unit whose row indices lie in slot par.  fp32: bit j = row j * 16 + lrow of the wave's
    // 64; bf16: bit 4 j + r = row j * 16 + r * 4 + (lane >> 4), the rows the lane stores after the turn through LDS
    auto row_flags = [&](int par, int expert) {
        const uint32_t ia = (uint32_t) reinterpret_cast<uintptr_t>((lds_void*)(smem + IBASE + (par * 128 + wm * 64 + (OUT_F32 ? lrow : (lane >> 4))) * 4));
        u32 kp = 0;
#pragma unroll
        for (int g4 = 0; g4 < (OUT_F32 ? 1 : 4); ++g4) {
            int idx[4];
            if constexpr (OUT_F32)
                asm volatile("ds_read_b32 %0, %4\n\tds_read_b32 %1, %4 offset:64\n\tds_read_b32 %2, %4 offset:128\n\tds_read_b32 %3, %4 offset:192\n\t"
                             "s_waitcnt lgkmcnt(0)" : "=&v"(idx[0]), "=&v"(idx[1]), "=&v"(idx[2]), "=&v"(idx[3]) : "v"(ia) : "memory");
            else
                asm volatile("ds_read_b32 %0, %4\n\tds_read_b32 %1, %4 offset:16\n\tds_read_b32 %2, %4 offset:32\n\tds_read_b32 %3, %4 offset:48\n\t"
                             "s_waitcnt lgkmcnt(0)" : "=&v"(idx[0]), "=&v"(idx[1]), "=&v"(idx[2]), "=&v"(idx[3]) : "v"(ia + (uint32_t)g4 * 64u) : "memory");
#pragma unroll
            for (int e = 0; e < 4; ++e) kp |= (idx[e] == expert ? 1u : 0u) << (g4 * 4 + e);
        }
        return kp;
    };

    int pid = blockIdx.x;
    while (pid < units && unit_expert(pid) < 0) pid += G;
    if (pid >= units) return;  // nothing but padding for this workgroup (uniform)
    int rb, tn, tn_end;
    unit_of(pid, rb, tn, tn_end);
    int m0 = rb * 128, expert = scalar_table_load(p.m_indices, m0);
    __amdgpu_buffer_rsrc_t rw = w_rsrc(expert, tn * 256);
    int ws = 0;     // stage of the stream's current step
    int snpar = 0;  // scale slot of the current tile
    // The workgroup's next unit is looked up when a unit begins, while its activation fragments are on their way: the
    // scalar loads of the lookup (more than one round trip when units of padding are skipped) cost nothing there.
    int nu_pid = units, nu_m0 = 0, nu_expert = 0, nu_tn = 0, nu_tn_end = 0;
    auto find_next_unit = [&](int from) {
        nu_pid = next_unit(from);
        if (nu_pid < units) {
            int rbn;
            unit_of(nu_pid, rbn, nu_tn, nu_tn_end);
            nu_m0 = rbn * 128;
            nu_expert = scalar_table_load(p.m_indices, nu_m0);
        }
    };
#pragma unroll
    for (int k = 0; k < 3; ++k)
#pragma unroll
        for (int i = 0; i < 8; ++i) dma_w(rw, k, k, i);
    dma_sn(expert, tn * 256, 0);
    load_unit(m0, 0);
    find_next_unit(pid);
    __builtin_amdgcn_s_waitcnt(kWaitVm0);
    __syncthreads();
    u32 keep = row_flags(0, expert);  // which of the rows this lane stores belong to the unit's expert
    int upar = 0;                     // slot of the current unit's row indices
    bool fresh = false;               // the row flags of the current unit are still to be formed
    i32x8 Wf[4];                      // window of weight fragments: w tile i of the stream lives in Wf[i & 3]
#pragma unroll
    for (int i = 0; i < 3; ++i) Wf[i] = frag(0, i);
    CFP8_PHASE_END();

    f32x4 acc[8][4], P[2][4];  // [w tile][x tile]; raw products of two w tiles
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};
    // The tile that is waiting to be stored (fp32: in `acc`; bf16: packed in Pk): its output rows as a buffer, the
    // lane's byte offset in it, and the lane's row flags.  No tile is waiting at the start: no flag set.
    __amdgpu_buffer_rsrc_t ro_p = __builtin_amdgcn_make_buffer_rsrc(p.out, 0, 0x80000000u, 0x00020000);
    uint32_t off_p = 0;
    u32 keep_p = 0;
    uint32_t ld_out_b = (uint32_t)p.ld_out * (OUT_F32 ? 4u : 2u);  // output row pitch in bytes
    asm volatile("" : "+s"(ld_out_b));
    constexpr uint32_t kDropped = 0xFFFF0000u;  // an offset beyond every output buffer
    // fp32: the stores of w tiles 2 m and 2 m + 1 of the waiting tile, from the accumulators
    auto store_pair = [&](int m) {
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const f32x4 v = acc[2 * m + h][j];
                __builtin_amdgcn_raw_buffer_store_b128(u32x4{__float_as_uint(v[0]), __float_as_uint(v[1]), __float_as_uint(v[2]), __float_as_uint(v[3])}, ro_p,
                                                       ((keep_p >> j) & 1u) ? off_p : kDropped, (uint32_t)(j * 16) * ld_out_b + (uint32_t)(2 * m + h) * 64u, 0);
            }
    };
    // bf16: the waiting tile, packed: Pk[j][i] = the lane's four columns of w tile i in row j * 16 + lrow
    u32 Pk[4][8][2];
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int i = 0; i < 8; ++i) Pk[j][i][0] = Pk[j][i][1] = 0u;
    uint8_t* const ebuf = smem + EBASE + wave * (16 * EST);
    const int rd_row = lane >> 4, rd_chunk = lane & 15;
    const uint32_t ebuf_wr = (uint32_t) reinterpret_cast<uintptr_t>((lds_void*)(ebuf + lrow * EST + quarter * 8));
    auto turn_write = [&](int j) {  // x tile j of the waiting tile into the wave's buffer
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            // written as an instruction: in front of an LDS store it knows of, the compiler waits for the weight
            // loads that are on their way into other parts of LDS
            const uint64_t two = (uint64_t)Pk[j][i][0] | ((uint64_t)Pk[j][i][1] << 32);
            asm volatile("ds_write_b64 %0, %1 offset:%2" ::"v"(ebuf_wr), "v"(two), "n"(i * 32) : "memory");
        }
    };
    i32x4 Rd[4];  // the row segments read back from the buffer, on their way to memory
    auto turn_read = [&]() {  // ... and out of it, as rows (written and read by the same wave: LDS operations of one wave complete in order)
#pragma unroll
        for (int r = 0; r < 4; ++r) Rd[r] = *reinterpret_cast<const i32x4*>(ebuf + (r * 4 + rd_row) * EST + rd_chunk * 16);
    };
    auto turn_store = [&](int j, int r) {
        __builtin_amdgcn_raw_buffer_store_b128(u32x4{(u32)Rd[r][0], (u32)Rd[r][1], (u32)Rd[r][2], (u32)Rd[r][3]}, ro_p,
                                               ((keep_p >> (j * 4 + r)) & 1u) ? off_p : kDropped, (uint32_t)(j * 16 + r * 4) * ld_out_b, 0);
    };
    // A step's vector-memory operations are, in this order, its stores (first half) and its eight weight loads (second
    // half, behind the barrier); the stage a step's barrier needs was requested two steps earlier, so what may still be
    // in flight behind it is everything of the step in between and this step's own stores (xres_allowed).
    for (;;) {
        // the tile after this one: the next of the unit, or the first of the workgroup's next unit
        bool has_next = true, new_unit = false;
        int pid_n = pid, m0n = m0, expert_n = expert, tn_n = tn + 1, tn_end_n = tn_end;
        if (tn_n >= tn_end) {
            has_next = nu_pid < units;
            new_unit = has_next;
            if (has_next) {
                pid_n = nu_pid;
                m0n = nu_m0;
                expert_n = nu_expert;
                tn_n = nu_tn;
                tn_end_n = nu_tn_end;
            } else {
                tn_n = tn;  // past the end the stream fetches this tile's first steps once more; nobody reads them
            }
        }
        const __amdgpu_buffer_rsrc_t rwn = w_rsrc(expert_n, tn_n * 256);
        const int n0 = tn * 256;
        // the block scales of the wave's 128 weight rows, one per K step: they came into LDS under the previous tile
        // (read by instructions written out: in front of an LDS read it knows of the compiler would wait for every
        // direct-to-LDS load in flight); the next tile's are requested now, ahead of this tile's first weight loads,
        // so the barrier of its third step covers them
        float sn[KT];
        {
            const uint32_t sa_lds = (uint32_t) reinterpret_cast<uintptr_t>((lds_void*)(smem + NBASE + ((wave * 2 + snpar) * 64) * 4));
            u32x4 lo;
            u32x2 hi;
            asm volatile("ds_read_b128 %0, %2\n\tds_read_b64 %1, %2 offset:16\n\ts_waitcnt lgkmcnt(0)" : "=&v"(lo), "=&v"(hi) : "v"(sa_lds) : "memory");
            const u32 raw[6] = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1]};
#pragma unroll
            for (int k = 0; k < KT; ++k) sn[k] = __uint_as_float(raw[k]);
        }
        dma_sn(expert_n, tn_n * 256, snpar ^ 1);

        float scp[4] = {0.f, 0.f, 0.f, 0.f};
        auto step = [&](auto kc) {
            constexpr int k = decltype(kc)::value;
            float sc[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) sc[j] = sm[j][k] * sn[k];
            const int ws_n = (ws + 1) & 3, ws_d = (ws + 3) & 3;
            // the loads of stream step + 3: past this tile's end they fetch the next tile
            constexpr bool into_next = k + 3 >= KT;
            const __amdgpu_buffer_rsrc_t rd = into_next ? rwn : rw;
            constexpr int kd = into_next ? k + 3 - KT : k + 3;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                if (i == 4) {
                    // the next step's stage has landed (fp32: the 32 stores of the tile before are issued in a tile's
                    // first step ahead of its barrier and are younger than what its first two barriers need)
                    constexpr int allowed = OUT_F32 ? (k < 2 ? 40 : 8) : xres_allowed<KT>(k);
                    asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" ::"n"(allowed) : "memory");
                    CFP8_PHASE_END();
                }
                if (i + 3 < 8) Wf[(i + 3) & 3] = frag(ws, i + 3);
                else Wf[(i + 3) & 3] = frag(ws_n, i + 3 - 8);
                if (i >= 4) {
                    dma_w(rd, kd, ws_d, 2 * (i - 4));
                    dma_w(rd, kd, ws_d, 2 * (i - 4) + 1);
                }
                if constexpr (OUT_F32) {
                    // a tile's first step, first half: the tile before leaves the accumulators, a pair of w tiles per
                    // w tile of this step and always ahead of the first write to them (w tile i is written from i + 1 on)
                    if constexpr (k == 0) {
                        if (i < 4) store_pair(i);
                    }
                } else {
                    // x tile k - 1 of the tile before: read back at the step's start, stored two and three w tiles later
                    if constexpr (k >= 1 && k <= 4) {
                        if (i == 0) turn_read();
#pragma unroll
                        for (int r = 0; r < 4; ++r)
                            if (i == kXresStoreAt[r]) turn_store(k - 1, r);
                    }
                    // x tile k of the tile before goes to the buffer right behind the barrier
                    if constexpr (k <= 3) {
                        if (i == 4) turn_write(k);
                    }
                }
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    P[i & 1][j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(Wf[i & 3], X[k][j], f32x4{0.f, 0.f, 0.f, 0.f}, 0, 0, 0, 0, 0, 0);
                    // the products of the w tile before this one join the accumulators under this one's MFMAs
                    if (i > 0) {
                        if constexpr (k == 0) {
#pragma unroll
                            for (int e = 0; e < 4; ++e) acc[i - 1][j][e] = P[(i - 1) & 1][j][e] * sc[j];
                        } else {
#pragma unroll
                            for (int e = 0; e < 4; ++e) acc[i - 1][j][e] = __builtin_fmaf(P[(i - 1) & 1][j][e], sc[j], acc[i - 1][j][e]);
                        }
                        asm volatile("" : "+v"(acc[i - 1][j]));
                    } else if constexpr (k == 1) {
#pragma unroll
                        for (int e = 0; e < 4; ++e) acc[7][j][e] = P[1][j][e] * scp[j];
                        asm volatile("" : "+v"(acc[7][j]));
                    } else if constexpr (k > 1) {
#pragma unroll
                        for (int e = 0; e < 4; ++e) acc[7][j][e] = __builtin_fmaf(P[1][j][e], scp[j], acc[7][j][e]);
                        asm volatile("" : "+v"(acc[7][j]));
                    }
                    // (the order is pinned MFMA by MFMA: left to itself the compiler folds a w tile's products right
                    // behind its own MFMAs, with wait states in front, and the matrix pipe idles under the VALU work)
                    CFP8_PHASE_END();
                }
            }
#pragma unroll
            for (int j = 0; j < 4; ++j) scp[j] = sc[j];
            ws = ws_n;
        };
        step(std::integral_constant<int, 0>{});
        step(std::integral_constant<int, 1>{});
        step(std::integral_constant<int, 2>{});
        if constexpr (KT > 3) step(std::integral_constant<int, 3>{});
        if constexpr (KT > 4) step(std::integral_constant<int, 4>{});
        if constexpr (KT > 5) step(std::integral_constant<int, 5>{});
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int e = 0; e < 4; ++e) acc[7][j][e] = __builtin_fmaf(P[1][j][e], scp[j], acc[7][j][e]);

        // this tile now waits in the accumulators: where its rows go
        if (fresh) {  // (uniform) the unit's first tile: its row indices have long landed
            keep = row_flags(upar, expert);
            fresh = false;
        }
        ro_p = __builtin_amdgcn_make_buffer_rsrc(static_cast<uint8_t*>(p.out) + (int64_t)m0 * p.ld_out * (OUT_F32 ? 4 : 2), 0, 0x80000000u, 0x00020000);
        keep_p = keep;
        if constexpr (OUT_F32) {
            off_p = (uint32_t)(wm * 64 + lrow) * ld_out_b + (uint32_t)(n0 + wn * 128 + quarter * 4) * 4u;
        } else {
            off_p = (uint32_t)(wm * 64 + rd_row) * ld_out_b + (uint32_t)(n0 + wn * 128 + rd_chunk * 8) * 2u;
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    Pk[j][i][0] = pack_bf16x2(acc[i][j][0], acc[i][j][1]);
                    Pk[j][i][1] = pack_bf16x2(acc[i][j][2], acc[i][j][3]);
                }
        }
        if (!has_next) break;
        pid = pid_n;
        m0 = m0n;
        expert = expert_n;
        tn = tn_n;
        tn_end = tn_end_n;
        rw = rwn;
        snpar ^= 1;
        if (new_unit) {
            // The activation fragments are free now: those of the workgroup's next unit are requested, its successor is
            // looked up while they are on their way, and then they are awaited.  The wait is written as the builtin,
            // which the compiler takes into account: it then knows that nothing it has requested is in flight when the
            // K steps begin and puts no waits of its own in front of the first use of each fragment and scale - waits
            // that, placed in every tile's steps, would also wait for the weight loads of the next two steps.  (One
            // block: with the wait under a second test of the same flag the compiler sees a path around it.)
            load_unit(m0, upar ^ 1);
            upar ^= 1;
            fresh = true;
            find_next_unit(pid);
            __builtin_amdgcn_s_waitcnt(kWaitVm0);
        }
    }
    // the last tile leaves
    if constexpr (OUT_F32) {
#pragma unroll
        for (int m = 0; m < 4; ++m) store_pair(m);
    } else {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            turn_write(j);
            turn_read();
#pragma unroll
            for (int r = 0; r < 4; ++r) turn_store(j, r);
        }
    }
    // the loads past the last tile land before the workgroup gives up its LDS
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
}

// Worth it from about 60 % of the tile slots filled (8 experts, 131 tile rows of 8 tiles, 45 % filled: 68 us against
// 62 us on the one-tile-per-workgroup kernel; 286 tile rows, 81 %: 100 against 124 us).
bool grouped_xres_pays(const GemmArgs& p) { return unit_plan(p.M / 128, p.N / 256, cu_count(), 1).fill >= 0.6; }

template <int KT>
static int launch_grouped_xres_kt(GemmArgs& p, int out_dtype, hipStream_t st) {
    p.tiles_m = p.M / 128;
    p.tiles_n = p.N / 256;
    const UnitPlan plan = unit_plan(p.tiles_m, p.tiles_n, cu_count(), 1);
    const int parts = plan.parts;
    const int64_t blocks = plan.blocks;
    p.unit_parts = parts;
    // stages, scale slots, row indices, the buffers that turn rows into stores
    constexpr size_t lds = (size_t)4 * 256 * 128 + 4 * 2 * 64 * sizeof(float) + 2 * 128 * sizeof(int32_t) + 4 * 16 * 272;
    using Kern = void (*)(const GemmArgs);
    const int f32 = out_dtype == CFP8_OUT_F32;
    const Kern kern = f32 ? static_cast<Kern>(gemm_grouped_xres_kernel<KT, true>) : static_cast<Kern>(gemm_grouped_xres_kernel<KT, false>);
    static std::atomic<bool> done[65][2];  // zero-initialised
    const int slot = device_slot();
    if (slot == 64) done[64][f32].store(false, std::memory_order_relaxed);
    if (int rc = raise_lds_limit(reinterpret_cast<const void*>(kern), lds, done[slot][f32])) return rc;
    {
        char name[64];
        snprintf(name, sizeof(name), "gemm_grouped_xres<%d> parts=%d", KT, parts);
        if (!note_launch(name, (unsigned)blocks, 256, lds)) return CFP8_OK;
    }
    hipLaunchKernelGGL(kern, dim3((unsigned)blocks), dim3(256), lds, st, p);
    return check_launch("gemm");
}
int launch_grouped_xres(GemmArgs& p, int out_dtype, hipStream_t st) {
    return (p.K >> 7) == 5 ? launch_grouped_xres_kt<5>(p, out_dtype, st) : launch_grouped_xres_kt<6>(p, out_dtype, st);
}

}  // namespace cfp8
