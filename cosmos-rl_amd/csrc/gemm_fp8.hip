// FP8 (OCP e4m3) GEMMs on the gfx950 matrix cores: rowwise-scaled, 128-block
// scaled and grouped block-scaled.  One kernel template serves all three.
//
//   out[m, n] = sum_k x[m, k] * w[n, k]   (both operands K-major, "nt")
//
// MFMA: v_mfma_f32_16x16x128_f8f6f4 (A and B in e4m3).  The weight tile is fed as
// the MFMA "A" operand and the activation tile as "B", so that a lane's four
// accumulators are four consecutive n of one output row m: the epilogue stores
// 8 contiguous bytes of bf16 per lane.  Lane l of a 16x16x128 MFMA supplies row
// (l & 15) and the 32 K-bytes of quarter (l >> 4) for both operands; any
// permutation of K shared by both operands leaves the dot products unchanged.
//
// Tiles: BM x BN x 128 per workgroup, LDS double-buffered.  An LDS tile is a
// sequence of 16-row blocks of 2 KiB; inside a block the 16-byte chunk c (0..7)
// of row r (0..15) sits at  c * 256 + ((r ^ ((c & 1) << 3)) << 4).  An MFMA
// operand read (16 consecutive lanes = 16 rows, same chunk) then covers one
// contiguous 256-byte segment - all 64 banks once - and a staging store (16
// consecutive lanes = 8 rows x 2 adjacent chunks) does too; measured on gfx950 a
// row-major tile with an XOR swizzle reads at half the LDS rate.
//
// Scaling: fp32 scales cannot ride in the MFMA (its scale operands are E8M0), so
//   rowwise:  acc over all of K, epilogue acc * sa[m] * sb[n];
//   block:    every K step is one 128-block; its MFMA result is folded into the
//             running sum as acc += part * (sa[m, kb] * sb[n / 128, kb]).
#include <atomic>
#include <stdio.h>
#include <stdlib.h>
#include <type_traits>

#include "cfp8_common.h"
#include "gemm_internal.h"

namespace cfp8 {


__device__ __forceinline__ int lds_chunk_offset(int row, int c) {
    return ((row >> 4) << 11) + (c << 8) + ((((row & 15) ^ ((c & 1) << 3))) << 4);
}

__device__ __forceinline__ i32x8 lds_frag(const uint8_t* tile, int row, int quarter) {
    const i32x4 lo = *reinterpret_cast<const i32x4*>(tile + lds_chunk_offset(row, 2 * quarter));
    const i32x4 hi = *reinterpret_cast<const i32x4*>(tile + lds_chunk_offset(row, 2 * quarter + 1));
    i32x8 r;
    r[0] = lo[0]; r[1] = lo[1]; r[2] = lo[2]; r[3] = lo[3];
    r[4] = hi[0]; r[5] = hi[1]; r[6] = hi[2]; r[7] = hi[3];
    return r;
}

// Workgroup id -> (tile_m, tile_n).  Consecutive workgroup ids are dealt round
// robin to the 8 XCDs, each with its own L2: give every XCD one contiguous range
// of tiles, and walk a range in bands of GM tile-rows so that co-resident
// workgroups share activation rows and weight rows in that L2.
// GM: tile-rows per band.  8 for the dense problems; the grouped kernels take kGroupedBandRows = 4, about the
// tile-rows of one expert at the MoE shapes served here (an expert's weight tile is then shared by the
// workgroups of one band: FETCH_SIZE of the K = 768 down projection of 128 experts falls from 1.34 to 1.10
// times its operand bytes, run time unchanged).
constexpr int kGroupedBandRows = 4;
template <int GM = 8>
__device__ __forceinline__ void tile_of_block(int pid, int tiles_m, int tiles_n, int& tm, int& tn) {
    const int total = tiles_m * tiles_n;
    const int xcd = pid & 7, local = pid >> 3;
    const int base = total >> 3, rem = total & 7;
    const int lin = xcd * base + (xcd < rem ? xcd : rem) + local;
    const int band = GM * tiles_n;
    const int g = lin / band, first = g * GM;
    const int gsz = (tiles_m - first) < GM ? (tiles_m - first) : GM;
    const int in = lin - g * band;
    tm = first + in % gsz;
    tn = in / gsz;
}

// KTAIL (rowwise only): K is a multiple of 16 but not of 128.  The last K step then ends inside its 128 bytes: lanes
// whose 16-byte chunk lies past K fetch chunk 0 of their row instead (nothing is read outside a row) and store zeros
// to LDS, for both operands, so the step's products are those of the K that exists.
template <int BM, int BN, int WM, int WN, int MODE, bool OUT_F32, bool SCALE_VEC, bool KTAIL = false>
__global__ __launch_bounds__(WM * WN * 64) __attribute__((amdgpu_waves_per_eu(2))) void gemm_kernel(const GemmArgs p) {
    static_assert(!KTAIL || MODE == kRowwise, "a K tail has no block scale of its own");
    constexpr int NT = WM * WN * 64;
    constexpr int WTM = BM / WM, WTN = BN / WN;  // wave tile
    constexpr int TM = WTM / 16, TN = WTN / 16;  // MFMA tiles per wave
    static_assert(WTM % 16 == 0 && WTN % 16 == 0, "wave tile must be a multiple of the MFMA tile");
    static_assert(MODE == kRowwise || WTN <= 128, "a wave's n range must stay inside one 128-block");

    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    constexpr int STAGE = (BM + BN) * 128;
    auto As = [&](int s) { return smem + s * STAGE; };
    auto Bs = [&](int s) { return smem + s * STAGE + BM * 128; };

    int tm, tn;
    tile_of_block(blockIdx.x, p.tiles_m, p.tiles_n, tm, tn);
    const int m0 = tm * BM, n0 = tn * BN;

    const uint8_t* bptr = p.b;
    const float* sbp = p.sb;
    int expert = 0;
    if (MODE == kGrouped) {
        expert = p.m_indices[m0];  // groups start on multiples of 128 = BM rows
        if (expert < 0) return;    // a tile of padding (uniform for the workgroup)
        bptr += (int64_t)expert * p.N * p.ld_b;
        sbp += (int64_t)expert * p.sb_stride_e;
    }

    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const int wm = wave % WM, wn = wave / WM;
    const int lrow = lane & 15, quarter = lane >> 4;
    const int KT = KTAIL ? (p.K + 127) >> 7 : p.K >> 7;

    // global -> register staging of one K step.  One wave-wide load covers 8 rows x
    // 128 bytes (8 full cache lines): lane = pair * 16 + row8 * 2 + half reads chunk
    // 2 * pair + half of row row8.
    constexpr int A_BLK = BM / 8, B_BLK = BN / 8, NW = NT / 64;
    constexpr int A_IT = (A_BLK + NW - 1) / NW, B_IT = (B_BLK + NW - 1) / NW;
    const int st_row8 = (lane >> 1) & 7, st_c = ((lane >> 4) << 1) | (lane & 1);
    // Every load below is unconditional and the K loop has no branch, so that the compiler can
    // count outstanding loads exactly and wait only for the ones it needs: rows past the edge of
    // a matrix read the last valid row instead (their products land in outputs that are never
    // stored), and steps past the end of K re-read the last tile.
    // Addresses are a wave-uniform 64-bit base plus a 32-bit lane offset (a tile spans fewer
    // than 2^32 bytes for any leading dimension below 2^24).
    i32x4 ra[A_IT], rb[B_IT];
    uint32_t oa[A_IT], ob[B_IT];
    const bool chunk_in_k = !KTAIL || st_c * 16 < (p.K & 127);  // this lane's chunk of the last K step lies inside K
    const uint32_t tail_back = chunk_in_k ? 0u : (uint32_t)st_c * 16u;  // what takes the lane back to chunk 0 there
    const uint8_t* const abase = p.a + (int64_t)m0 * p.ld_a;
    const uint8_t* const bbase = bptr + (int64_t)n0 * p.ld_b;
#pragma unroll
    for (int i = 0; i < A_IT; ++i) {
        const int r = (wave + NW * i) * 8 + st_row8;
        const int rr = (m0 + r) < p.M ? r : (p.M - 1 - m0);
        oa[i] = (uint32_t)rr * (uint32_t)p.ld_a + st_c * 16;
    }
#pragma unroll
    for (int i = 0; i < B_IT; ++i) {
        const int r = (wave + NW * i) * 8 + st_row8;
        const int rr = (n0 + r) < p.N ? r : (p.N - 1 - n0);
        ob[i] = (uint32_t)rr * (uint32_t)p.ld_b + st_c * 16;
    }
    auto load_tile = [&](int kt) {
        const int64_t k = (int64_t)(kt < KT ? kt : KT - 1) << 7;
        const uint8_t* const ak = abase + k;
        const uint8_t* const bk = bbase + k;
        const uint32_t back = KTAIL && kt >= KT - 1 ? tail_back : 0u;
#pragma unroll
        for (int i = 0; i < A_IT; ++i) ra[i] = *reinterpret_cast<const i32x4*>(ak + (oa[i] - back));
#pragma unroll
        for (int i = 0; i < B_IT; ++i) rb[i] = *reinterpret_cast<const i32x4*>(bk + (ob[i] - back));
    };
    // LDS stores number `first` .. `last`-1 of the A_IT + B_IT that make up one staged tile, which is K step `kt`
    auto store_part = [&](int stage, int first, int last, int kt) {
        const int keep = KTAIL && kt >= KT - 1 && !chunk_in_k ? 0 : -1;
#pragma unroll
        for (int i = 0; i < A_IT; ++i) {
            const int r = (wave + NW * i) * 8 + st_row8;
            if (i >= first && i < last && (A_BLK % NW == 0 || r < BM))
                *reinterpret_cast<i32x4*>(As(stage) + lds_chunk_offset(r, st_c)) = KTAIL ? ra[i] & keep : ra[i];
        }
#pragma unroll
        for (int i = 0; i < B_IT; ++i) {
            const int r = (wave + NW * i) * 8 + st_row8;
            if (A_IT + i >= first && A_IT + i < last && (B_BLK % NW == 0 || r < BN))
                *reinterpret_cast<i32x4*>(Bs(stage) + lds_chunk_offset(r, st_c)) = KTAIL ? rb[i] & keep : rb[i];
        }
    };
    constexpr int ST_ALL = A_IT + B_IT;
    constexpr int HALF = TM > 1 ? TM / 2 : 1;  // m-tiles over which the LDS stores of the next tile are spread

    // Block scales.  Activation scales are [M, K/128] row-major, so the scales of one K step lie
    // K/128 floats apart: fetched per step and lane they cost as many cache-line requests as the
    // operand tile itself.  Instead the workgroup fetches the scales of its BM rows for 8 K steps
    // at a time, 4 consecutive floats per thread (row = t / 2, half = t % 2), and turns them in LDS
    // to [K step][row], double buffered by group of 8 steps.  The weight scale is one value per
    // wave and step, fetched one step ahead.
    float* const sg_buf = reinterpret_cast<float*>(smem + 2 * STAGE);  // [2][8][BM]
    const int sg_row = t >> 1, sg_half = t & 1;
    const float* sg_ptr = p.sa;
    const float* psb = sbp;
    if (MODE != kRowwise) {
        const int r = sg_row < BM ? sg_row : BM - 1;
        sg_ptr = p.sa + (int64_t)((m0 + r) < p.M ? (m0 + r) : (p.M - 1)) * KT;
        psb += (int64_t)((n0 + wn * WTN) >> 7) * p.sb_stride_n;
    }
    f32x4 sg = {0.f, 0.f, 0.f, 0.f};
    auto sg_load = [&](int g) {  // scales of K steps 8g + 4 half .. + 3 of this thread's row; steps past K/128 repeat valid ones
        if (MODE == kRowwise) return;
        const int k0 = 8 * g + 4 * sg_half;
        if (SCALE_VEC) {
            sg = *reinterpret_cast<const f32x4*>(sg_ptr + (k0 + 4 <= KT ? k0 : KT - 4));
        } else {
#pragma unroll
            for (int e = 0; e < 4; ++e) sg[e] = sg_ptr[(k0 + e) < KT ? (k0 + e) : (KT - 1)];
        }
    };
    auto sg_store = [&](int g) {
        if (MODE == kRowwise) return;
        if (NT / 2 <= BM || sg_row < BM) {
#pragma unroll
            for (int e = 0; e < 4; ++e) sg_buf[((g & 1) * 8 + 4 * sg_half + e) * BM + sg_row] = sg[e];
        }
    };
    auto load_sn = [&](int kt) -> float {
        if (MODE == kRowwise) return 0.f;
        return psb[(int64_t)(kt < KT ? kt : KT - 1) * p.sb_stride_k];
    };

    f32x4 acc[TN][TM];
#pragma unroll
    for (int i = 0; i < TN; ++i)
#pragma unroll
        for (int j = 0; j < TM; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};

    // Pipeline over K steps.  At the top of step kt, LDS stage kt & 1 holds tile kt and the
    // staging registers hold tile kt+1 (loaded in the second half of step kt-1).  Its LDS stores
    // into the other stage are spread over the first HALF m-tiles of this step; the global loads
    // of tile kt+2 are issued right after them, so they have the rest of this step and the
    // barrier to land.  The last step stores a tile that nobody reads.  The activation scales of
    // the next group of 8 steps are requested in step 8g+6, right after that step's tile loads,
    // and stored to LDS in step 8g+7.
    load_tile(0);
    sg_load(0);
    float s_n = load_sn(0);
    __builtin_amdgcn_sched_barrier(0);  // weight scale before tile kt+1, as in the loop: one wait count fits both
    store_part(0, 0, ST_ALL, 0);
    sg_store(0);
    load_tile(1);
    __syncthreads();

    for (int kt = 0; kt < KT; ++kt) {
        const int cur = kt & 1;
        float s_m[TM];
        const float s_n_cur = s_n;
        if (MODE != kRowwise) {
            const float* const sgk = sg_buf + (((kt >> 3) & 1) * 8 + (kt & 7)) * BM + wm * WTM + lrow;
#pragma unroll
            for (int j = 0; j < TM; ++j) s_m[j] = sgk[j * 16];
            __builtin_amdgcn_sched_barrier(0);
            s_n = load_sn(kt + 1);
        }

        // weight fragments stay live for the whole step; activation fragments are
        // read one 16-row tile ahead of the MFMAs that consume them
        i32x8 fa[TN];
#pragma unroll
        for (int i = 0; i < TN; ++i) fa[i] = lds_frag(Bs(cur), wn * WTN + i * 16 + lrow, quarter);
        i32x8 fb = lds_frag(As(cur), wm * WTM + lrow, quarter);
        // block scaling: the products of m-tile j go to `part`; their scaled accumulation runs
        // one m-tile later, while the matrix pipe works on the next m-tile
        f32x4 part[TN];
#pragma unroll
        for (int j = 0; j <= TM; ++j) {
            f32x4 prev[TN];
            if (MODE != kRowwise) {
#pragma unroll
                for (int i = 0; i < TN; ++i) prev[i] = part[i];
            }
            if (j < TM) {
                i32x8 fb_next = fb;
                if (j + 1 < TM) fb_next = lds_frag(As(cur), wm * WTM + (j + 1) * 16 + lrow, quarter);
                if (j < HALF) store_part(cur ^ 1, ST_ALL * j / HALF, ST_ALL * (j + 1) / HALF, kt + 1);
                if (MODE != kRowwise && j == HALF - 1 && (kt & 7) == 7) sg_store((kt >> 3) + 1);
#pragma unroll
                for (int i = 0; i < TN; ++i) {
                    if (MODE == kRowwise)
                        acc[i][j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(fa[i], fb, acc[i][j], 0, 0, 0, 0, 0, 0);
                    else
                        part[i] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(fa[i], fb, f32x4{0.f, 0.f, 0.f, 0.f}, 0, 0, 0, 0, 0, 0);
                }
                if (j == HALF - 1) {
                    __builtin_amdgcn_sched_barrier(0);
                    load_tile(kt + 2);
                    if (MODE != kRowwise && (kt & 7) == 6) sg_load((kt >> 3) + 1);
                    __builtin_amdgcn_sched_barrier(0);
                }
                fb = fb_next;
            }
            if (MODE != kRowwise && j > 0) {
                const float scj = s_m[j - 1] * s_n_cur;
#pragma unroll
                for (int i = 0; i < TN; ++i)
#pragma unroll
                    for (int e = 0; e < 4; ++e) acc[i][j - 1][e] = __builtin_fmaf(prev[i][e], scj, acc[i][j - 1][e]);
            }
        }
        __syncthreads();
    }

    // epilogue: lane holds out[m][n .. n+3] for every (i, j).  Everything the epilogue reads from global memory (row
    // and column scales, which rows belong to the group) is read before its first store: loads and stores share one
    // counter, so a load behind a store waits for the store's acknowledgement.
    float sam[TM];
    f32x4 sbn[TN];
#pragma unroll
    for (int j = 0; j < TM; ++j) {
        const int m = m0 + wm * WTM + j * 16 + lrow;
        sam[j] = (MODE == kRowwise && m < p.M) ? p.sa[m] : 1.f;
    }
#pragma unroll
    for (int i = 0; i < TN; ++i) {
        const int n = n0 + wn * WTN + i * 16 + quarter * 4;
        sbn[i] = (MODE == kRowwise && n < p.N) ? *reinterpret_cast<const f32x4*>(p.sb + n) : f32x4{0.f, 0.f, 0.f, 0.f};
    }
    if constexpr (!OUT_F32 && BM >= 128) {
        // bf16, large tiles: scale, convert and turn the wave's block through LDS so that global
        // stores are 16 bytes per lane, a full row segment of the wave's block at a time, and
        // non-temporal (the output must not evict operand tiles from L2)
        constexpr int EST = WTN * 2 + 16;             // LDS row stride in bytes
        constexpr int LPR = WTN / 8;                  // lanes (16-byte chunks) per row
        constexpr int RPI = 64 / LPR;                 // rows per wave-wide store
        constexpr int HR = WTM / 2;                   // the block goes through LDS in two halves of HR rows
        static_assert(HR % 16 == 0 && WM * WN * HR * EST <= 2 * (BM + BN) * 128, "epilogue buffer must fit the operand stages");
        uint8_t* const ebuf = smem + wave * (HR * EST);
        const int rd_row = lane / LPR, rd_chunk = lane % LPR;
        bool keep[2][HR / RPI];
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
            for (int r = 0; r < HR / RPI; ++r) {
                const int m = m0 + wm * WTM + h * HR + r * RPI + rd_row, n = n0 + wn * WTN + rd_chunk * 8;
                bool ok = m < p.M && n < p.N;         // N % 16 == 0: an 8-wide chunk is inside or outside as a whole
                if (MODE == kGrouped && ok) ok = p.m_indices[m] == expert;
                keep[h][r] = ok;
            }
        __syncthreads();                              // every wave is done reading the operand stages
#pragma unroll
        for (int h = 0; h < 2; ++h) {
#pragma unroll
            for (int jj = 0; jj < TM / 2; ++jj) {
                const int j = h * (TM / 2) + jj;
#pragma unroll
                for (int i = 0; i < TN; ++i) {
                    f32x4 v = acc[i][j];
                    if (MODE == kRowwise) {
#pragma unroll
                        for (int e = 0; e < 4; ++e) v[e] = v[e] * sam[j] * sbn[i][e];
                    }
                    *reinterpret_cast<uint2*>(ebuf + (jj * 16 + lrow) * EST + (i * 16 + quarter * 4) * 2) =
                        make_uint2(pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3]));
                }
            }
            // written and read by the same wave: LDS operations of one wave complete in order
#pragma unroll
            for (int r = 0; r < HR / RPI; ++r) {
                const int row = r * RPI + rd_row;
                const int m = m0 + wm * WTM + h * HR + row, n = n0 + wn * WTN + rd_chunk * 8;
                if (keep[h][r]) {
                    const i32x4 d = *reinterpret_cast<const i32x4*>(ebuf + row * EST + rd_chunk * 16);
                    __builtin_nontemporal_store(d, reinterpret_cast<i32x4*>(static_cast<uint16_t*>(p.out) + (int64_t)m * p.ld_out + n));
                }
            }
        }
        return;
    }
    bool keep[TM];
#pragma unroll
    for (int j = 0; j < TM; ++j) {
        const int m = m0 + wm * WTM + j * 16 + lrow;
        keep[j] = m < p.M;
        if (MODE == kGrouped && keep[j]) keep[j] = p.m_indices[m] == expert;
    }
#pragma unroll
    for (int j = 0; j < TM; ++j) {
        const int m = m0 + wm * WTM + j * 16 + lrow;
        if (!keep[j]) continue;
#pragma unroll
        for (int i = 0; i < TN; ++i) {
            const int n = n0 + wn * WTN + i * 16 + quarter * 4;
            if (n >= p.N) continue;  // N % 16 == 0: a group of four is inside or outside as a whole
            f32x4 v = acc[i][j];
            if (MODE == kRowwise) {
#pragma unroll
                for (int e = 0; e < 4; ++e) v[e] = v[e] * sam[j] * sbn[i][e];
            }
            if (OUT_F32) {
                *reinterpret_cast<f32x4*>(static_cast<float*>(p.out) + (int64_t)m * p.ld_out + n) = v;
            } else {
                *reinterpret_cast<uint2*>(static_cast<uint16_t*>(p.out) + (int64_t)m * p.ld_out + n) =
                    make_uint2(pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3]));
            }
        }
    }
}

// ---------------------------------------------------------------------------
// Rowwise GEMM, large full tiles: 256 x 256 x 128 per workgroup, four wavefronts
// (one per SIMD, 2 x 2), each owning a 128 x 128 block = 64 accumulators of
// 16 x 16 (all 256 AGPRs).  Operand tiles go from global memory straight into
// LDS (buffer_load_dwordx4 ... lds: no staging registers, no LDS store instructions;
// in the buffer form the wave-uniform part of an address is a scalar offset, so a
// load costs two scalar additions and no vector arithmetic).
// Such a load puts lane l's 16 bytes at byte l * 16 of its 1 KiB destination, so
// the LDS layout is dictated by which bytes each lane asks for: a stage is
// row-major, row r at r * 128, and lane l of a load of 8 rows fetches chunk
// (l & 7) ^ f(r) of row r = l >> 3, f(r) = bit 1 of r | bit 3 of r << 2.  Eight
// consecutive lanes then read one whole 128-byte line of global memory (a
// lane-to-address map that fetches 16 bytes from each of 16 rows, which a
// chunk-major LDS layout would dictate, makes the same pipeline 25 % slower).
// The fragment reads (ds_read_b128, one chunk of one row per lane: lane = quarter *
// 16 + row) are free of bank conflicts with this f: the LDS serves a 16-byte read
// sixteen lanes at a time, and the sixteen are lanes 0-3, 12-15, 20-23, 24-27 (then
// 4-7, 8-11, 16-19, 28-31, and the same in the upper half of the wave), found by
// giving two lanes the same banks and watching which pairs cost a cycle; f puts
// those sixteen on sixteen different 16-byte bank groups (215 B/clk/CU from four
// waves that do nothing else, against 128 with f(r) = (r >> 1) & 7, which spreads
// sixteen CONSECUTIVE lanes).  The kernels here gain nothing measurable from it:
// none of them is bound by the LDS read rate.
// With one wave per SIMD nothing hides a stall, so the K step is written as a
// software pipeline of 32 groups of two MFMAs, each group preceded by at most
// one direct-to-LDS load and one fragment read.  LDS holds two activation
// stages and three weight stages of 32 KiB (all 160 KiB); step kt computes from
// activation stage kt % 2 and weight stage kt % 3:
//
//   S0 (w0,x0): LDS reads x1
//   S1 (w0,x1): LDS reads w1
//   -- wait for all but the eight newest loads and for own LDS reads, barrier: tile kt+1 complete, both stages of tile kt free --
//   S2 (w1,x0): LDS reads next w0     + loads of activation tile kt+2
//   S3 (w1,x1): LDS reads next x0     + loads of weight tile kt+3 (the eight newest at the next barrier)
//
// so an activation load has one K step (~2048 MFMA cycles) to land and a weight
// load two (weights come from HBM, activations mostly from the caches), and
// every fragment is read at least 16 MFMAs before its first use.  The tile's
// row scales are fetched the same way into the activation stage that no tile
// needs any more, one and a half steps before the epilogue.
// The epilogue turns each wave's block through LDS so that every global store
// is 16 bytes per lane and 256 contiguous bytes per output row, non-temporal
// (the output must not evict operand tiles from L2).
// Requires M % 256 == 0 and N % 256 == 0 (every address is then a per-lane part
// plus a wave-uniform part).
// ---------------------------------------------------------------------------
#define CFP8_MMA2(wb, wh, xb, xh, g)                                                                   \
    {                                                                                                  \
        _Pragma("unroll") for (int e = 0; e < 2; ++e) {                                                \
            const int j = (g) >> 1, i = ((g)&1) * 2 + e;                                               \
            acc[(wh)*4 + i][(xh)*4 + j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(            \
                W[wb][i], X[xb][j], acc[(wh)*4 + i][(xh)*4 + j], 0, 0, 0, 0, 0, 0);                    \
        }                                                                                              \
    }

template <bool OUT_F32>
__global__ __launch_bounds__(256) void gemm_rowwise_256_kernel(const GemmArgs p) {
    constexpr int BM = 256, BN = 256;
    constexpr int XS = BM * 128, WS = BN * 128;  // one activation / weight stage: 32 KiB each
    constexpr int WBASE = 2 * XS;                // LDS: two activation stages, then three weight stages = 160 KiB
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    int tm, tn;
    tile_of_block(blockIdx.x, p.tiles_m, p.tiles_n, tm, tn);
    const int m0 = tm * BM, n0 = tn * BN;
    const int t = threadIdx.x, lane = t & 63;
    const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
    const int wm = wave & 1, wn = wave >> 1;
    const int lrow = lane & 15, quarter = lane >> 4;
    const int KT = p.K >> 7;
    const int last = KT - 1;

    // Direct-to-LDS load i (0..7) of one operand's K step covers rows (wave + 4 i) * 8 .. + 7 of the tile.
    // The wave-uniform bases and strides pass through an empty asm so that the compiler keeps them in SGPRs for
    // the whole K loop: left alone it re-reads the kernel arguments inside the loop, and every scalar load has to be
    // waited for with lgkmcnt(0), which drains the LDS queue of the fragment reads in flight.
    uint64_t a_wave = reinterpret_cast<uint64_t>(p.a) + ((uint64_t)m0 + (uint64_t)wave * 8) * (uint64_t)p.ld_a;
    uint64_t b_wave = reinterpret_cast<uint64_t>(p.b) + ((uint64_t)n0 + (uint64_t)wave * 8) * (uint64_t)p.ld_b;
    uint32_t a_step = 32u * (uint32_t)p.ld_a, b_step = 32u * (uint32_t)p.ld_b;  // leading dimensions are < 2^24
    asm volatile("" : "+s"(a_wave), "+s"(b_wave), "+s"(a_step), "+s"(b_step));
    // f(r) of row r = (wave + 4 i) * 8 + (lane >> 3) is (wave & 1) * 4 + ((lane >> 4) & 1)
    const uint32_t chunk = (uint32_t)(((lane & 7) ^ ((wave & 1) * 4 + ((lane >> 4) & 1))) << 4);
    const uint32_t va_lane = (uint32_t)(lane >> 3) * (uint32_t)p.ld_a + chunk;
    const uint32_t vb_lane = (uint32_t)(lane >> 3) * (uint32_t)p.ld_b + chunk;
    typedef __attribute__((address_space(1))) const void gbl_void;
    typedef __attribute__((address_space(3))) void lds_void;
    // buffer form of the load: descriptor in SGPRs (base = this wave's first row, no bounds), per-lane offset in one
    // VGPR, the wave-uniform part of the address as the scalar offset - no vector arithmetic per load
    const __amdgpu_buffer_rsrc_t ra = __builtin_amdgcn_make_buffer_rsrc(reinterpret_cast<void*>(a_wave), 0, 0xFFFFFFFF, 0x00020000);
    const __amdgpu_buffer_rsrc_t rb = __builtin_amdgcn_make_buffer_rsrc(reinterpret_cast<void*>(b_wave), 0, 0xFFFFFFFF, 0x00020000);
    auto dma_x = [&](int kt, int stage, int i) {
        __builtin_amdgcn_raw_ptr_buffer_load_lds(ra, (lds_void*)(smem + stage * XS + (wave + 4 * i) * 1024), 16, va_lane,
                                                 (uint32_t)i * a_step + ((uint32_t)kt << 7), 0, 0);
    };
    auto dma_w = [&](int kt, int stage, int i) {
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rb, (lds_void*)(smem + WBASE + stage * WS + (wave + 4 * i) * 1024), 16, vb_lane,
                                                 (uint32_t)i * b_step + ((uint32_t)kt << 7), 0, 0);
    };

    f32x4 acc[8][8];  // [n tile][m tile]
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int j = 0; j < 8; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};

    // fragment of 16 rows: lane (lrow, quarter) reads chunks 2 quarter and 2 quarter + 1 of its row
    const int fsw = ((lrow >> 1) & 1) | (((lrow >> 3) & 1) << 2);
    const int x_off = (wm * 128 + lrow) * 128 + (((2 * quarter) ^ fsw) << 4);
    const int x_off2 = (wm * 128 + lrow) * 128 + (((2 * quarter + 1) ^ fsw) << 4);
    const int w_off = WBASE + (wn * 128 + lrow) * 128 + (((2 * quarter) ^ fsw) << 4);
    const int w_off2 = WBASE + (wn * 128 + lrow) * 128 + (((2 * quarter + 1) ^ fsw) << 4);
    auto frag = [&](int stage_bytes, int off, int off2, int tile16) {
        const uint8_t* base = smem + stage_bytes + tile16 * 2048;
        const i32x4 lo = *reinterpret_cast<const i32x4*>(base + off);
        const i32x4 hi = *reinterpret_cast<const i32x4*>(base + off2);
        i32x8 r;
        r[0] = lo[0]; r[1] = lo[1]; r[2] = lo[2]; r[3] = lo[3];
        r[4] = hi[0]; r[5] = hi[1]; r[6] = hi[2]; r[7] = hi[3];
        return r;
    };
    i32x8 W[2][4], X[2][4];  // weight / activation fragments of the two halves of the wave's block

    // prologue: activation tiles 0, 1 and weight tiles 0, 1, 2 into their stages
#pragma unroll
    for (int i = 0; i < 8; ++i) dma_x(0, 0, i);
#pragma unroll
    for (int i = 0; i < 8; ++i) dma_w(0, 0, i);
#pragma unroll
    for (int i = 0; i < 8; ++i) dma_x(1 < last ? 1 : last, 1, i);
#pragma unroll
    for (int i = 0; i < 8; ++i) dma_w(1 < last ? 1 : last, 1, i);
#pragma unroll
    for (int i = 0; i < 8; ++i) dma_w(2 < last ? 2 : last, 2, i);
    asm volatile("s_waitcnt vmcnt(24)" ::: "memory");  // tile 0 has landed; the other three loads stay in flight
    __syncthreads();
#pragma unroll
    for (int g = 0; g < 4; ++g) {
        W[0][g] = frag(0, w_off, w_off2, g);
        X[0][g] = frag(0, x_off, x_off2, g);
    }
    CFP8_PHASE_END();

    // Step kt computes from activation stage kt % 2 and weight stage kt % 3.  After its barrier nobody reads either
    // any more: activation tile kt + 2 and then weight tile kt + 3 are requested into them.  The next barrier needs
    // activation tile kt + 2 and weight tile kt + 2 (requested a step earlier), i.e. everything but the eight newest
    // loads: an activation load has one K step to land, a weight load two.
    int ws_cur = 0;  // kt % 3
    const int scale_step = last > 0 ? last - 1 : 0;
    for (int kt = 0; kt < KT; ++kt) {
        const int xs_cur = (kt & 1) * XS, xs_nxt = xs_cur ^ XS;
        const int ws_nxt = ws_cur == 2 ? 0 : ws_cur + 1;
        const int kw = kt + 3 < last ? kt + 3 : last;  // past the end: the last tile again, never consumed
#pragma unroll
        for (int g = 0; g < 8; ++g) {
            if (g < 4) X[1][g] = frag(xs_cur, x_off, x_off2, 4 + g);
            CFP8_MMA2(0, 0, 0, 0, g);
            CFP8_PHASE_END();
        }
#pragma unroll
        for (int g = 0; g < 8; ++g) {
            if (g < 4) W[1][g] = frag(ws_cur * WS, w_off, w_off2, 4 + g);
            CFP8_MMA2(0, 0, 1, 1, g);
            CFP8_PHASE_END();
        }
        CFP8_WAIT_BARRIER(8);
        CFP8_PHASE_END();
        if (kt == scale_step) {
            // no activation tile goes into stage (last + 1) % 2 any more: it takes the tile's 256 activation scales and
            // 256 weight scales for the epilogue (64 of each per wave, 4 bytes per lane), a step and a half ahead
            uint8_t* dst = smem + ((last + 1) & 1) * XS + wave * 256;
            __builtin_amdgcn_global_load_lds((gbl_void*)(p.sa + m0 + wave * 64 + lane), (lds_void*)dst, 4, 0, 0);
            __builtin_amdgcn_global_load_lds((gbl_void*)(p.sb + n0 + wave * 64 + lane), (lds_void*)(dst + 1024), 4, 0, 0);
        }
#pragma unroll
        for (int g = 0; g < 8; ++g) {
            if (g < 4) W[0][g] = frag(ws_nxt * WS, w_off, w_off2, g);  // after the last step: stale data, unused
            if (kt + 2 <= last) dma_x(kt + 2, kt & 1, g);
            CFP8_MMA2(1, 1, 0, 0, g);
            CFP8_PHASE_END();
        }
#pragma unroll
        for (int g = 0; g < 8; ++g) {
            if (g < 4) X[0][g] = frag(xs_nxt, x_off, x_off2, g);
            dma_w(kw, ws_cur, g);
            CFP8_MMA2(1, 1, 1, 1, g);
            CFP8_PHASE_END();
        }
        ws_cur = ws_nxt;
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the scales have landed, and nothing may still land in the stages
    __syncthreads();
    const float* const scale_lds = reinterpret_cast<const float*>(smem + ((last + 1) & 1) * XS);  // [0, 256): sa, [256, 512): sb

    float sam[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) sam[j] = scale_lds[wm * 128 + j * 16 + lrow];
    if (OUT_F32) {
        // a lane already owns 16 contiguous bytes: store directly
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int n = n0 + wn * 128 + i * 16 + quarter * 4;
            const f32x4 sbn = *reinterpret_cast<const f32x4*>(scale_lds + 256 + wn * 128 + i * 16 + quarter * 4);
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const int m = m0 + wm * 128 + j * 16 + lrow;
                f32x4 v = acc[i][j];
#pragma unroll
                for (int e = 0; e < 4; ++e) v[e] = v[e] * sam[j] * sbn[e];
                __builtin_nontemporal_store(v, reinterpret_cast<f32x4*>(static_cast<float*>(p.out) + (int64_t)m * p.ld_out + n));
            }
        }
        return;
    }
    // bf16: scale, convert, turn the wave's 128 x 128 block through LDS in two halves of 64 rows
    // (row stride 272 B keeps the 8-byte stores of 16 rows on different banks)
    f32x4 sbn[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) sbn[i] = *reinterpret_cast<const f32x4*>(scale_lds + 256 + wn * 128 + i * 16 + quarter * 4);
    __syncthreads();  // all waves are done reading the operand stages
    constexpr int EST = 272;
    uint8_t* const ebuf = smem + WBASE + wave * (64 * EST);  // in the weight stages: the scales sit in an activation stage
    const int rd_row = lane >> 4, rd_chunk = lane & 15;
#pragma unroll
    for (int h = 0; h < 2; ++h) {
#pragma unroll
        for (int jj = 0; jj < 4; ++jj) {
            const int j = h * 4 + jj;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                f32x4 v = acc[i][j];
#pragma unroll
                for (int e = 0; e < 4; ++e) v[e] = v[e] * sam[j] * sbn[i][e];
                *reinterpret_cast<uint2*>(ebuf + (jj * 16 + lrow) * EST + (i * 16 + quarter * 4) * 2) =
                    make_uint2(pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3]));
            }
        }
        // written and read by the same wave: LDS operations of one wave complete in order
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int row = r * 4 + rd_row;  // 0..63 within the half
            const i32x4 d = *reinterpret_cast<const i32x4*>(ebuf + row * EST + rd_chunk * 16);
            const int m = m0 + wm * 128 + h * 64 + row;
            __builtin_nontemporal_store(
                d, reinterpret_cast<i32x4*>(static_cast<uint16_t*>(p.out) + (int64_t)m * p.ld_out + n0 + wn * 128 + rd_chunk * 8));
        }
    }
}

// ---------------------------------------------------------------------------
// Persistent form of the 256 x 256 kernel: one workgroup per CU walks tiles b, b + gridDim.x, ...  The K steps of
// consecutive tiles form one stream: the loads of a tile's last two steps already fetch the first steps of the next
// tile, so a tile does not start with a round trip to memory, and the epilogue of a tile runs while those loads
// are in flight.  The weight stage that the last step would have filled is left free instead and serves the
// epilogue (the tile's scales and the buffer that turns the wave's block into row-contiguous stores, 16 rows at a
// time); it is filled right after.  Requires K >= 384.
// ---------------------------------------------------------------------------
// A last round that is at most half full (p.tail_tiles tiles, the last ones in the workgroups' order) would cost every
// workgroup's wait for the few that have a tile in it.  Those tiles are cut into quarters of 128 x 128 instead, dealt
// to all workgroups behind their last full tile and computed by the strip kernel's ring pipeline (same products in
// the same order of K, same epilogue arithmetic: the same bits).
template <int BM, int TN, bool OUT_F32>
__device__ __forceinline__ void rowwise_strip_block(const GemmArgs& p, uint8_t* const smem, const int m0, const int n0, const int t);

template <bool OUT_F32>
__global__ __launch_bounds__(256) void gemm_rowwise_256p_kernel(const GemmArgs p) {
    constexpr int BM = 256, BN = 256;
    constexpr int XS = BM * 128, WS = BN * 128;
    constexpr int WBASE = 2 * XS;
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    const int ntiles = p.tiles_m * p.tiles_n - p.tail_tiles;  // tiles taken whole
    const int t = threadIdx.x, lane = t & 63;
    const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
    const int wm = wave & 1, wn = wave >> 1;
    const int lrow = lane & 15, quarter = lane >> 4;
    const int KT = p.K >> 7;
    const int last = KT - 1;
    __builtin_assume(KT >= 3);
    uint32_t a_step = 32u * (uint32_t)p.ld_a, b_step = 32u * (uint32_t)p.ld_b;
    asm volatile("" : "+s"(a_step), "+s"(b_step));
    const uint32_t chunk = (uint32_t)(((lane & 7) ^ ((wave & 1) * 4 + ((lane >> 4) & 1))) << 4);
    const uint32_t va_lane = (uint32_t)(lane >> 3) * (uint32_t)p.ld_a + chunk;
    const uint32_t vb_lane = (uint32_t)(lane >> 3) * (uint32_t)p.ld_b + chunk;
    typedef __attribute__((address_space(1))) const void gbl_void;
    typedef __attribute__((address_space(3))) void lds_void;
    auto tile_rsrc = [&](int pid, int& m0, int& n0, __amdgpu_buffer_rsrc_t& ra, __amdgpu_buffer_rsrc_t& rb) {
        int tm, tn;
        tile_of_block(pid, p.tiles_m, p.tiles_n, tm, tn);
        m0 = tm * BM;
        n0 = tn * BN;
        const uint64_t aw = reinterpret_cast<uint64_t>(p.a) + ((uint64_t)m0 + (uint64_t)wave * 8) * (uint64_t)p.ld_a;
        const uint64_t bw = reinterpret_cast<uint64_t>(p.b) + ((uint64_t)n0 + (uint64_t)wave * 8) * (uint64_t)p.ld_b;
        ra = __builtin_amdgcn_make_buffer_rsrc(reinterpret_cast<void*>(aw), 0, 0xFFFFFFFF, 0x00020000);
        rb = __builtin_amdgcn_make_buffer_rsrc(reinterpret_cast<void*>(bw), 0, 0xFFFFFFFF, 0x00020000);
    };
    auto dma_x = [&](__amdgpu_buffer_rsrc_t r, int kt, int stage, int i) {
        __builtin_amdgcn_raw_ptr_buffer_load_lds(r, (lds_void*)(smem + stage * XS + (wave + 4 * i) * 1024), 16, va_lane,
                                                 (uint32_t)i * a_step + ((uint32_t)kt << 7), 0, 0);
    };
    auto dma_w = [&](__amdgpu_buffer_rsrc_t r, int kt, int stage, int i) {
        __builtin_amdgcn_raw_ptr_buffer_load_lds(r, (lds_void*)(smem + WBASE + stage * WS + (wave + 4 * i) * 1024), 16, vb_lane,
                                                 (uint32_t)i * b_step + ((uint32_t)kt << 7), 0, 0);
    };
    const int fsw = ((lrow >> 1) & 1) | (((lrow >> 3) & 1) << 2);
    const int x_off = (wm * 128 + lrow) * 128 + (((2 * quarter) ^ fsw) << 4);
    const int x_off2 = (wm * 128 + lrow) * 128 + (((2 * quarter + 1) ^ fsw) << 4);
    const int w_off = WBASE + (wn * 128 + lrow) * 128 + (((2 * quarter) ^ fsw) << 4);
    const int w_off2 = WBASE + (wn * 128 + lrow) * 128 + (((2 * quarter + 1) ^ fsw) << 4);
    auto frag = [&](int stage_bytes, int off, int off2, int tile16) {
        const uint8_t* base = smem + stage_bytes + tile16 * 2048;
        const i32x4 lo = *reinterpret_cast<const i32x4*>(base + off);
        const i32x4 hi = *reinterpret_cast<const i32x4*>(base + off2);
        i32x8 r;
        r[0] = lo[0]; r[1] = lo[1]; r[2] = lo[2]; r[3] = lo[3];
        r[4] = hi[0]; r[5] = hi[1]; r[6] = hi[2]; r[7] = hi[3];
        return r;
    };

    int pid = blockIdx.x;
    int m0, n0;
    __amdgpu_buffer_rsrc_t ra, rb;
    tile_rsrc(pid, m0, n0, ra, rb);
    // stages of the stream's next step: activation stage xs (0 or XS), weight stage ws (0..2)
    int xs = 0, ws = 0;
#pragma unroll
    for (int i = 0; i < 8; ++i) dma_x(ra, 0, 0, i);
#pragma unroll
    for (int i = 0; i < 8; ++i) dma_w(rb, 0, 0, i);
#pragma unroll
    for (int i = 0; i < 8; ++i) dma_x(ra, 1, 1, i);
#pragma unroll
    for (int i = 0; i < 8; ++i) dma_w(rb, 1, 1, i);

    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    for (;;) {
        // the third weight step of this tile
        {
            const int w2 = ws == 0 ? 2 : ws - 1;  // (ws + 2) % 3
#pragma unroll
            for (int i = 0; i < 8; ++i) dma_w(rb, 2, w2, i);
        }
        CFP8_WAIT_BARRIER(40);  // the activations of the second step have landed: they are older than the stores of the epilogue
        const int pid_n = pid + (int)gridDim.x;
        const bool has_next = pid_n < ntiles;
        int m0n = m0, n0n = n0;
        __amdgpu_buffer_rsrc_t ran = ra, rbn = rb;
        if (has_next) tile_rsrc(pid_n, m0n, n0n, ran, rbn);

        f32x4 acc[8][8];  // [n tile][m tile]
#pragma unroll
        for (int i = 0; i < 8; ++i)
#pragma unroll
            for (int j = 0; j < 8; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};
        i32x8 W[2][4], X[2][4];
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            W[0][g] = frag(ws * WS, w_off, w_off2, g);
            X[0][g] = frag(xs, x_off, x_off2, g);
        }
        CFP8_PHASE_END();

        int ws_free = 0;
        auto step = [&](int kt, auto wait_count) {
            const int xs_nxt = xs ^ XS;
            const int ws_nxt = ws == 2 ? 0 : ws + 1;
            // loads of stream steps + 2 (activations) and + 3 (weights): past this tile's end they fetch the next tile
            const bool xn = kt + 2 >= KT, wnx = kt + 3 >= KT;
            const __amdgpu_buffer_rsrc_t rx = xn ? ran : ra, rw = wnx ? rbn : rb;
            const int kx = xn ? kt + 2 - KT : kt + 2, kw = wnx ? kt + 3 - KT : kt + 3;
#pragma unroll
            for (int g = 0; g < 8; ++g) {
                if (g < 4) X[1][g] = frag(xs, x_off, x_off2, 4 + g);
                CFP8_MMA2(0, 0, 0, 0, g);
                CFP8_PHASE_END();
            }
#pragma unroll
            for (int g = 0; g < 8; ++g) {
                if (g < 4) W[1][g] = frag(ws * WS, w_off, w_off2, 4 + g);
                CFP8_MMA2(0, 0, 1, 1, g);
                CFP8_PHASE_END();
            }
            if constexpr (decltype(wait_count)::value == 40) CFP8_WAIT_BARRIER(40);
            else CFP8_WAIT_BARRIER(8);
            CFP8_PHASE_END();
            if (kt == last) {
                // the weight stage of this step stays free for the epilogue; it takes the tile's scales now
                uint8_t* dst = smem + WBASE + ws * WS + 24576 + wave * 256;
                const __amdgpu_buffer_rsrc_t rsa = __builtin_amdgcn_make_buffer_rsrc(
                    const_cast<float*>(p.sa) + m0 + wave * 64, 0, 0xFFFFFFFF, 0x00020000);
                const __amdgpu_buffer_rsrc_t rsb = __builtin_amdgcn_make_buffer_rsrc(
                    const_cast<float*>(p.sb) + n0 + wave * 64, 0, 0xFFFFFFFF, 0x00020000);
                __builtin_amdgcn_raw_ptr_buffer_load_lds(rsa, (lds_void*)dst, 4, (uint32_t)lane * 4u, 0, 0, 0);
                __builtin_amdgcn_raw_ptr_buffer_load_lds(rsb, (lds_void*)(dst + 1024), 4, (uint32_t)lane * 4u, 0, 0, 0);
                ws_free = ws;
            }
#pragma unroll
            for (int g = 0; g < 8; ++g) {
                if (g < 4) W[0][g] = frag(ws_nxt * WS, w_off, w_off2, g);
                dma_x(rx, kx, xs == 0 ? 0 : 1, g);
                CFP8_MMA2(1, 1, 0, 0, g);
                CFP8_PHASE_END();
            }
#pragma unroll
            for (int g = 0; g < 8; ++g) {
                if (g < 4) X[0][g] = frag(xs_nxt, x_off, x_off2, g);
                if (kt != last) dma_w(rw, kw, ws, g);
                CFP8_MMA2(1, 1, 1, 1, g);
                CFP8_PHASE_END();
            }
            xs = xs_nxt;
            ws = ws_nxt;
        };
        // the first step of a tile only needs loads that are older than the stores of the previous tile's epilogue
        // (at most 32 of them, and the eight loads of the third weight step are younger still)
        step(0, std::integral_constant<int, 40>{});
        for (int kt = 1; kt < KT; ++kt) step(kt, std::integral_constant<int, 8>{});
        // the scales have landed (the eight loads behind them belong to the next tile); every wave is done with the
        // stage that serves the epilogue
        CFP8_WAIT_BARRIER(8);

        const float* const scale_lds = reinterpret_cast<const float*>(smem + WBASE + ws_free * WS + 24576);
        float sam[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) sam[j] = scale_lds[wm * 128 + j * 16 + lrow];
        f32x4 sbn[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) sbn[i] = *reinterpret_cast<const f32x4*>(scale_lds + 256 + wn * 128 + i * 16 + quarter * 4);
        if (OUT_F32) {
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const int n = n0 + wn * 128 + i * 16 + quarter * 4;
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    const int m = m0 + wm * 128 + j * 16 + lrow;
                    f32x4 v = acc[i][j];
#pragma unroll
                    for (int e = 0; e < 4; ++e) v[e] = v[e] * sam[j] * sbn[i][e];
                    __builtin_nontemporal_store(v, reinterpret_cast<f32x4*>(static_cast<float*>(p.out) + (int64_t)m * p.ld_out + n));
                }
            }
        } else {
            constexpr int EST = 272;
            uint8_t* const ebuf = smem + WBASE + ws_free * WS + wave * (16 * EST);
            const int rd_row = lane >> 4, rd_chunk = lane & 15;
            const uint32_t ebuf_wr =
                (uint32_t) reinterpret_cast<uintptr_t>((lds_void*)(ebuf + lrow * EST + quarter * 8));
#pragma unroll
            for (int j = 0; j < 8; ++j) {
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    f32x4 v = acc[i][j];
#pragma unroll
                    for (int e = 0; e < 4; ++e) v[e] = v[e] * sam[j] * sbn[i][e];
                    // written as an instruction: in front of an LDS store it knows of, the compiler waits for the loads
                    // of the next tile that are still on their way into other parts of LDS
                    const uint64_t two = (uint64_t)pack_bf16x2(v[0], v[1]) | ((uint64_t)pack_bf16x2(v[2], v[3]) << 32);
                    asm volatile("ds_write_b64 %0, %1 offset:%2" ::"v"(ebuf_wr), "v"(two), "n"(i * 32) : "memory");
                }
                // written and read by the same wave: LDS operations of one wave complete in order
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const int row = r * 4 + rd_row;
                    const i32x4 d = *reinterpret_cast<const i32x4*>(ebuf + row * EST + rd_chunk * 16);
                    const int m = m0 + wm * 128 + j * 16 + row;
                    __builtin_nontemporal_store(
                        d, reinterpret_cast<i32x4*>(static_cast<uint16_t*>(p.out) + (int64_t)m * p.ld_out + n0 + wn * 128 + rd_chunk * 8));
                }
            }
        }
        if (!has_next) break;
        pid = pid_n;
        m0 = m0n;
        n0 = n0n;
        ra = ran;
        rb = rbn;
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");  // every wave is done with its part of the epilogue buffer
    }
    // the loads past the last tile (they fetched its first steps once more) land before the workgroup gives up its LDS
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    // the quarters of the tiles of the last round.  (The thread's number is formed anew here, from the wave's number and
    // a count of the lanes below, and passes through an empty asm: everything the quarter tiles derive from it would
    // otherwise be computed at the kernel's start and kept in registers through the tiles' K loops, which have none to
    // spare.)
    int t_late = wave * 64 + (int)__builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
    asm volatile("" : "+v"(t_late));
    // (likewise the kernel's arguments: read again from the kernel-argument segment, through a pointer the compiler
    // cannot see through, instead of being held in scalar registers from the kernel's start)
    uint64_t args_at = reinterpret_cast<uint64_t>(__builtin_amdgcn_kernarg_segment_ptr());
    uint32_t args_lo = (uint32_t)args_at, args_hi = (uint32_t)(args_at >> 32);
    asm volatile("" : "+s"(args_lo), "+s"(args_hi));
    args_lo = __builtin_amdgcn_readfirstlane(args_lo);  // (wave-uniform, which the compiler does not assume of an asm's result)
    args_hi = __builtin_amdgcn_readfirstlane(args_hi);
    typedef __attribute__((address_space(4))) const uint32_t ConstWord;  // (the segment is constant memory: scalar loads)
    const ConstWord* const words = reinterpret_cast<const ConstWord*>(((uint64_t)args_hi << 32) | args_lo);
    static_assert(sizeof(GemmArgs) % 4 == 0, "copied word by word");
    uint32_t copy[sizeof(GemmArgs) / 4];
#pragma unroll
    for (unsigned i = 0; i < sizeof(GemmArgs) / 4; ++i) copy[i] = words[i];
    GemmArgs late;
    __builtin_memcpy(&late, copy, sizeof(late));
    for (int u = (int)blockIdx.x; u < 4 * late.tail_tiles; u += (int)gridDim.x) {
        __syncthreads();  // every wave is done with the stages (the last tile's epilogue buffer, the quarter before)
        int tm, tn;
        tile_of_block(late.tiles_m * late.tiles_n - late.tail_tiles + (u >> 2), late.tiles_m, late.tiles_n, tm, tn);
        rowwise_strip_block<128, 8, OUT_F32>(late, smem, tm * BM + (u & 1) * 128, tn * BN + ((u >> 1) & 1) * 128, t_late);
    }
}

// ---------------------------------------------------------------------------
// The same pipeline on 256 x 128 tiles (256 activation rows, 128 weight rows), for problems whose 256 x 256
// tiles would fill the 256 CUs badly (a few hundred to a thousand tokens): four waves as 2 x 2, each a
// 128 x 64 block = 32 accumulator tiles.  A step is two groups of 16 MFMAs:
//
//   S0 (w, x0): LDS reads x1              + loads of weight tile kt+2 into weight stage (kt+2) % 3
//   -- wait for all but those four loads and for own LDS reads, barrier: tile kt+1 complete --
//   S1 (w, x1): LDS reads next w, next x0 + loads of activation tile kt+2 into activation stage kt % 2
//
// LDS: two activation stages of 32 KiB, three weight stages of 16 KiB and the tile's scales (fetched in the
// prologue).
// Requires M % 256 == 0 and N % 128 == 0.
// ---------------------------------------------------------------------------
// (Budgeted for two waves per SIMD, i.e. 256 registers: with all 512 on offer the compiler spreads the 128
// accumulators over both register files and copies them to and fro around the MFMAs.)
template <bool OUT_F32>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2))) void gemm_rowwise_256x128_kernel(const GemmArgs p) {
    constexpr int BM = 256, BN = 128;
    constexpr int XS = BM * 128, WS = BN * 128;
    constexpr int WBASE = 2 * XS, SBASE = WBASE + 3 * WS;  // 112 KiB of stages, then 384 scales
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    int tm, tn;
    tile_of_block(blockIdx.x, p.tiles_m, p.tiles_n, tm, tn);
    const int m0 = tm * BM, n0 = tn * BN;
    const int t = threadIdx.x, lane = t & 63;
    const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
    const int wm = wave & 1, wn = wave >> 1;
    const int lrow = lane & 15, quarter = lane >> 4;
    const int KT = p.K >> 7;
    const int last = KT - 1;

    // direct-to-LDS loads as in gemm_rowwise_256_kernel: load i covers rows (wave + 4 i) * 8 .. + 7 of its operand's tile
    uint64_t a_wave = reinterpret_cast<uint64_t>(p.a) + ((uint64_t)m0 + (uint64_t)wave * 8) * (uint64_t)p.ld_a;
    uint64_t b_wave = reinterpret_cast<uint64_t>(p.b) + ((uint64_t)n0 + (uint64_t)wave * 8) * (uint64_t)p.ld_b;
    uint32_t a_step = 32u * (uint32_t)p.ld_a, b_step = 32u * (uint32_t)p.ld_b;  // leading dimensions are < 2^24
    asm volatile("" : "+s"(a_wave), "+s"(b_wave), "+s"(a_step), "+s"(b_step));
    const uint32_t chunk = (uint32_t)(((lane & 7) ^ ((wave & 1) * 4 + ((lane >> 4) & 1))) << 4);
    const uint32_t va_lane = (uint32_t)(lane >> 3) * (uint32_t)p.ld_a + chunk;
    const uint32_t vb_lane = (uint32_t)(lane >> 3) * (uint32_t)p.ld_b + chunk;
    typedef __attribute__((address_space(1))) const void gbl_void;
    typedef __attribute__((address_space(3))) void lds_void;
    const __amdgpu_buffer_rsrc_t ra = __builtin_amdgcn_make_buffer_rsrc(reinterpret_cast<void*>(a_wave), 0, 0xFFFFFFFF, 0x00020000);
    const __amdgpu_buffer_rsrc_t rb = __builtin_amdgcn_make_buffer_rsrc(reinterpret_cast<void*>(b_wave), 0, 0xFFFFFFFF, 0x00020000);
    auto dma_x = [&](int kt, int stage, int i) {  // i < 8
        __builtin_amdgcn_raw_ptr_buffer_load_lds(ra, (lds_void*)(smem + stage * XS + (wave + 4 * i) * 1024), 16, va_lane,
                                                 (uint32_t)i * a_step + ((uint32_t)kt << 7), 0, 0);
    };
    auto dma_w = [&](int kt, int stage, int i) {  // i < 4
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rb, (lds_void*)(smem + WBASE + stage * WS + (wave + 4 * i) * 1024), 16, vb_lane,
                                                 (uint32_t)i * b_step + ((uint32_t)kt << 7), 0, 0);
    };

    f32x4 acc[4][8];  // [n tile][m tile]
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 8; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};

    const int fsw = ((lrow >> 1) & 1) | (((lrow >> 3) & 1) << 2);
    const int x_off = (wm * 128 + lrow) * 128 + (((2 * quarter) ^ fsw) << 4);
    const int x_off2 = (wm * 128 + lrow) * 128 + (((2 * quarter + 1) ^ fsw) << 4);
    const int w_off = WBASE + (wn * 64 + lrow) * 128 + (((2 * quarter) ^ fsw) << 4);
    const int w_off2 = WBASE + (wn * 64 + lrow) * 128 + (((2 * quarter + 1) ^ fsw) << 4);
    auto frag = [&](int stage_bytes, int off, int off2, int tile16) {
        const uint8_t* base = smem + stage_bytes + tile16 * 2048;
        const i32x4 lo = *reinterpret_cast<const i32x4*>(base + off);
        const i32x4 hi = *reinterpret_cast<const i32x4*>(base + off2);
        i32x8 r;
        r[0] = lo[0]; r[1] = lo[1]; r[2] = lo[2]; r[3] = lo[3];
        r[4] = hi[0]; r[5] = hi[1]; r[6] = hi[2]; r[7] = hi[3];
        return r;
    };
    i32x8 W[4], X[2][4];  // the wave's four weight fragments; X[h]: the halves of its 128 rows
    float* const scale_lds = reinterpret_cast<float*>(smem + SBASE);  // [0, 256): sa, [256, 384): sb

    // prologue: tiles 0 and 1 and the scales (weight tile 2 follows in the first step)
#pragma unroll
    for (int i = 0; i < 8; ++i) dma_x(0, 0, i);
#pragma unroll
    for (int i = 0; i < 4; ++i) dma_w(0, 0, i);
#pragma unroll
    for (int i = 0; i < 8; ++i) dma_x(1 < last ? 1 : last, 1, i);
#pragma unroll
    for (int i = 0; i < 4; ++i) dma_w(1 < last ? 1 : last, 1, i);
    __builtin_amdgcn_global_load_lds((gbl_void*)(p.sa + m0 + wave * 64 + lane), (lds_void*)(scale_lds + wave * 64), 4, 0, 0);
    if (wave < 2) __builtin_amdgcn_global_load_lds((gbl_void*)(p.sb + n0 + wave * 64 + lane), (lds_void*)(scale_lds + 256 + wave * 64), 4, 0, 0);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
#pragma unroll
    for (int g = 0; g < 4; ++g) X[0][g] = frag(0, x_off, x_off2, g);
#pragma unroll
    for (int g = 0; g < 3; ++g) W[g] = frag(0, w_off, w_off2, g);
    CFP8_PHASE_END();

    // Both groups walk the weight fragments in order (MFMA pair g uses W[g >> 1]), so a fragment's registers can take
    // the next step's fragment as soon as its last pair has been issued; the last one is read at the start of S0.
#define CFP8_MMA2N(xh, g)                                                                              \
    {                                                                                                  \
        _Pragma("unroll") for (int e = 0; e < 2; ++e) {                                                \
            const int i = (g) >> 1, j = ((g)&1) * 2 + e;                                               \
            acc[i][(xh)*4 + j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(                     \
                W[i], X[xh][j], acc[i][(xh)*4 + j], 0, 0, 0, 0, 0, 0);                                 \
        }                                                                                              \
    }
    int ws_cur = 0;  // kt % 3
    for (int kt = 0; kt < KT; ++kt) {
        const int xs_cur = (kt & 1) * XS, xs_nxt = xs_cur ^ XS;
        const int ws_nxt = ws_cur == 2 ? 0 : ws_cur + 1;
        const int ws_prv = ws_cur == 0 ? 2 : ws_cur - 1;  // (kt + 2) % 3
        const int kx = kt + 2 < last ? kt + 2 : last;     // past the end: the last tile again, never consumed
#pragma unroll
        for (int g = 0; g < 8; ++g) {
            if (g == 0) W[3] = frag(ws_cur * WS, w_off, w_off2, 3);
            else if (g <= 4) X[1][g - 1] = frag(xs_cur, x_off, x_off2, 4 + g - 1);
            if (g < 4) dma_w(kx, ws_prv, g);
            CFP8_MMA2N(0, g);
            CFP8_PHASE_END();
        }
        CFP8_WAIT_BARRIER(4);
        CFP8_PHASE_END();
#pragma unroll
        for (int g = 0; g < 8; ++g) {
            // (after the last step: stale data, unused)
            if (g == 0) X[0][0] = frag(xs_nxt, x_off, x_off2, 0);
            if (g == 1) X[0][1] = frag(xs_nxt, x_off, x_off2, 1);
            if (g == 2) W[0] = frag(ws_nxt * WS, w_off, w_off2, 0);
            if (g == 3) X[0][2] = frag(xs_nxt, x_off, x_off2, 2);
            if (g == 4) W[1] = frag(ws_nxt * WS, w_off, w_off2, 1);
            if (g == 5) X[0][3] = frag(xs_nxt, x_off, x_off2, 3);
            if (g == 6) W[2] = frag(ws_nxt * WS, w_off, w_off2, 2);
            dma_x(kx, kt & 1, g);
            CFP8_MMA2N(1, g);
            CFP8_PHASE_END();
        }
        ws_cur = ws_nxt;
    }
#undef CFP8_MMA2N
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the epilogue reuses the stages: nothing may still land there

    float sam[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) sam[j] = scale_lds[wm * 128 + j * 16 + lrow];
    f32x4 sbn[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) sbn[i] = *reinterpret_cast<const f32x4*>(scale_lds + 256 + wn * 64 + i * 16 + quarter * 4);
    if (OUT_F32) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int n = n0 + wn * 64 + i * 16 + quarter * 4;
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const int m = m0 + wm * 128 + j * 16 + lrow;
                f32x4 v = acc[i][j];
#pragma unroll
                for (int e = 0; e < 4; ++e) v[e] = v[e] * sam[j] * sbn[i][e];
                __builtin_nontemporal_store(v, reinterpret_cast<f32x4*>(static_cast<float*>(p.out) + (int64_t)m * p.ld_out + n));
            }
        }
        return;
    }
    // bf16: the wave's 128 x 64 block goes through LDS in two halves of 64 rows (row stride 144 B), so that global
    // stores are 16 bytes per lane and 128 contiguous bytes per row, non-temporal
    __syncthreads();  // all waves are done reading the operand stages
    constexpr int EST = 144;
    uint8_t* const ebuf = smem + wave * (64 * EST);
    const int rd_row = lane >> 3, rd_chunk = lane & 7;
#pragma unroll
    for (int h = 0; h < 2; ++h) {
#pragma unroll
        for (int jj = 0; jj < 4; ++jj) {
            const int j = h * 4 + jj;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                f32x4 v = acc[i][j];
#pragma unroll
                for (int e = 0; e < 4; ++e) v[e] = v[e] * sam[j] * sbn[i][e];
                *reinterpret_cast<uint2*>(ebuf + (jj * 16 + lrow) * EST + (i * 16 + quarter * 4) * 2) =
                    make_uint2(pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3]));
            }
        }
        // written and read by the same wave: LDS operations of one wave complete in order
#pragma unroll
        for (int r = 0; r < 8; ++r) {
            const int row = r * 8 + rd_row;  // 0..63 within the half
            const i32x4 d = *reinterpret_cast<const i32x4*>(ebuf + row * EST + rd_chunk * 16);
            const int m = m0 + wm * 128 + h * 64 + row;
            __builtin_nontemporal_store(
                d, reinterpret_cast<i32x4*>(static_cast<uint16_t*>(p.out) + (int64_t)m * p.ld_out + n0 + wn * 64 + rd_chunk * 8));
        }
    }
}

// ---------------------------------------------------------------------------
// SwiGLU + 1x128 requantisation of a grouped gate_up tile, in registers.
// The interleaved weight puts gate and up rows side by side in units of 16 (one MFMA tile): of a wave's four weight
// tiles, 0 and 2 are gate rows and 1 and 3 the up rows of the same hidden columns, so a lane that holds gate[m][c .. c+3]
// in acc[2 pp][j] holds up[m][c .. c+3] in acc[2 pp + 1][j] and forms h = bf16(bf16(silu(gate)) * up) without moving
// anything - both rounded to bf16 first, as the GEMM would have written them, so the result is bit for bit that of the
// grouped GEMM followed by the SwiGLU quantiser.  A wave covers 32 of the 128 hidden columns of the tile's 1x128 group;
// the four waves that share token rows exchange their maxima through 2 KiB of LDS (`xch`: [128 rows][4] bf16 bit
// patterns; one barrier), every lane derives the scale of its rows and casts its own values.  Per wave: 8 byte stores
// (4 bytes per lane) and 4 scale stores, issued unconditionally: a row that does not belong to the tile's expert gets an
// offset past the end of the buffer descriptor and the hardware drops it (the walking kernel counts stores between two
// tiles).  LDS is touched by instructions written out: in front of an LDS access it knows of, the compiler waits for
// every direct-to-LDS load in flight.
// ---------------------------------------------------------------------------
__device__ __forceinline__ u32 quarters_max(u32 v) {  // max over the four lanes l, l + 16, l + 32, l + 48; all get it
    typedef u32 u32x2s __attribute__((ext_vector_type(2)));
    const u32x2s a = __builtin_amdgcn_permlane32_swap(v, v, false, false);
    v = umax(a[0], a[1]);
    const u32x2s b = __builtin_amdgcn_permlane16_swap(v, v, false, false);
    return umax(b[0], b[1]);
}
// four bf16 (two packed words, element order preserved) -> four fp8 bytes
__device__ __forceinline__ u32 cast4(u32 w0, u32 w1, const Divider& d) {
    if (d.finite) {
        const u32 lo = cvt2<false>(d.fast(bf16_lo(w0)), d.fast(bf16_hi(w0)), 0u);
        return cvt2<true>(d.fast(bf16_lo(w1)), d.fast(bf16_hi(w1)), lo);
    }
    return slow_byte(bf16_lo(w0), d.s) | (slow_byte(bf16_hi(w0), d.s) << 8) | (slow_byte(bf16_lo(w1), d.s) << 16) |
           (slow_byte(bf16_hi(w1), d.s) << 24);
}

// acc: [weight tile][token tile] of the wave's 64 x 64 block; row_keep[j]: the wave's token row j * 16 + lrow belongs to
// the tile's expert; rq / rh: buffer descriptors of the tile's first row of the fp8 output and of its scales
__device__ __forceinline__ void swiglu_quant_epilogue(const f32x4 (&acc)[4][4], uint8_t* xch, int wm, int wn, int lrow, int quarter,
                                                      const bool (&row_keep)[4], __amdgpu_buffer_rsrc_t rq, __amdgpu_buffer_rsrc_t rh,
                                                      int ld_out, int ld_hs, int tn) {
    typedef __attribute__((address_space(3))) void lds_void;
    u32 h[4][2][2];  // [token tile][pair][two packed bf16 words] of h
    u32 mx[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        u32 m = 0;
#pragma unroll
        for (int pp = 0; pp < 2; ++pp) {
            const f32x4 g = acc[2 * pp][j], u = acc[2 * pp + 1][j];
            swiglu_quad(pack_bf16x2(g[0], g[1]), pack_bf16x2(g[2], g[3]), pack_bf16x2(u[0], u[1]), pack_bf16x2(u[2], u[3]), h[j][pp][0], h[j][pp][1]);
            m = pk_absmax(pk_absmax(m, h[j][pp][0]), h[j][pp][1]);
        }
        mx[j] = quarters_max(pk_fold(m));
    }
    const uint32_t xw = (uint32_t) reinterpret_cast<uintptr_t>((lds_void*)(xch + ((wm * 64 + lrow) * 4 + wn) * 4));
    const uint32_t xr = (uint32_t) reinterpret_cast<uintptr_t>((lds_void*)(xch + (wm * 64 + lrow) * 16));
#pragma unroll
    for (int j = 0; j < 4; ++j) asm volatile("ds_write_b32 %0, %1 offset:%2" ::"v"(xw), "v"(mx[j]), "n"(j * 256) : "memory");
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    u32x4 all[4];
    asm volatile("ds_read_b128 %0, %4\n\tds_read_b128 %1, %4 offset:256\n\tds_read_b128 %2, %4 offset:512\n\t"
                 "ds_read_b128 %3, %4 offset:768\n\ts_waitcnt lgkmcnt(0)"
                 : "=&v"(all[0]), "=&v"(all[1]), "=&v"(all[2]), "=&v"(all[3])
                 : "v"(xr)
                 : "memory");
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const u32 amax_bits = umax(umax(all[j][0], all[j][1]), umax(all[j][2], all[j][3]));
        const float scale = scale_from_amax(amax_from_bits(amax_bits));
        const Divider d(scale);
        const int r = wm * 64 + j * 16 + lrow;  // row of the tile
#pragma unroll
        for (int pp = 0; pp < 2; ++pp) {
            const u32 bytes = cast4(h[j][pp][0], h[j][pp][1], d);
            __builtin_amdgcn_raw_buffer_store_b32(bytes, rq, row_keep[j] ? (uint32_t)(r * ld_out + tn * 128 + wn * 32 + pp * 16 + quarter * 4) : 0xFFFFFFF0u, 0, 0);
        }
        __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(scale), rh,
                                              row_keep[j] && wn == 0 && quarter == 0 ? (uint32_t)((r * ld_hs + tn) * 4) : 0xFFFFFFF0u, 0, 0);
    }
}

// ---------------------------------------------------------------------------
// Block-scaled and grouped GEMM, full tiles: 256 x 128 (block) or 128 x 256 (grouped, whose groups are
// 128 rows) x 128 per workgroup, eight wavefronts (two per SIMD), each a 64 x 64 block = 4 x tiles
// times 4 w tiles.  Operand tiles go straight from global memory into LDS as in gemm_rowwise_256_kernel
// (row-major stages with XOR-ed chunks; two activation stages and three weight stages).  One wave keeps
// only one LDS instruction in progress at a time, so the K step is laid out around its LDS queue:
//
//   group 0: read x2 | per w tile i: rescale of last step's (i, x2), MFMA (i, x0)
//   group 1: read x3 | per i: rescale of last step's (i, x3), MFMA (i, x1)
//   wait for all but the newest weight loads and for own LDS reads, barrier: tile kt+1 complete, tile kt's stages free
//   tail:    next step's x0 | loads of activation tile kt+2 | per i: rescale of (i, x0), (i, x1), MFMAs (i, x2), (i, x3),
//            then next step's w tile i into the registers those MFMAs just consumed and a load of weight tile kt+3;
//            next step's x1 and scales
//
// No MFMA after the barrier waits for LDS, every rescale (acc += products * s_m * s_n, VALU) reads MFMA
// results issued at least five MFMAs earlier, and the first MFMAs of a step find their fragments read
// during the previous tail.  Activation scales reach LDS eight K steps at a time (turned to [step][row]),
// the tile's weight scales once in the prologue.  Requires M % BM == 0, N % BN == 0 and
// K / 128 * (BN / 128) <= kMaxTileWeightScales.
// ---------------------------------------------------------------------------
constexpr int kMaxTileWeightScales = 2048;

template <int BM, int BN, int MODE, bool OUT_F32, bool SCALE_VEC, bool SWIGLU = false>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2))) void gemm_block_w8_kernel(const GemmArgs p) {
    static_assert((BM == 256 && BN == 128) || (BM == 128 && BN == 256), "eight 64 x 64 wave tiles");
    static_assert(!SWIGLU || (MODE == kGrouped && BN == 256 && !OUT_F32), "the SwiGLU epilogue belongs to the grouped 128 x 256 tile");
    static_assert(MODE == kBlock || MODE == kGrouped, "block-scaled modes only");
    constexpr int WM = BM / 64;
    constexpr int XS = BM * 128, WS = BN * 128;  // one activation / weight stage
    constexpr int WBASE = 2 * XS;                // LDS: two activation stages, three weight stages, then the scales
    constexpr int SBASE = WBASE + 3 * WS;
    constexpr int A_IT = BM / 64, B_IT = BN / 64;  // wave-wide loads (8 rows x 128 B) per wave and K step: 4 + 2 or 2 + 4
    constexpr int NB = BN / 128;
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    int tm, tn;
    tile_of_block<MODE == kGrouped ? kGroupedBandRows : 8>(blockIdx.x, p.tiles_m, p.tiles_n, tm, tn);
    const int m0 = tm * BM, n0 = tn * BN;
    const int t = threadIdx.x, lane = t & 63;
    const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
    const int wm = wave % WM, wn = wave / WM;
    const int lrow = lane & 15, quarter = lane >> 4;
    const int KT = p.K >> 7;
    const int last = KT - 1;

    // global -> LDS directly (as in gemm_rowwise_256_kernel: row-major stages, 16-byte chunks XOR-ed by f(row)):
    // load i of an operand's K step covers rows (wave + 8 i) * 8 .. + 7 of its tile
    uint64_t a_wave = reinterpret_cast<uint64_t>(p.a) + ((uint64_t)m0 + (uint64_t)wave * 8) * (uint64_t)p.ld_a;
    uint32_t a_step = 64u * (uint32_t)p.ld_a, b_step = 64u * (uint32_t)p.ld_b;  // leading dimensions are < 2^24
    asm volatile("" : "+s"(a_wave), "+s"(a_step), "+s"(b_step));  // keep them in SGPRs for the whole loop
    const uint32_t chunk = (uint32_t)(((lane & 7) ^ ((wave & 1) * 4 + ((lane >> 4) & 1))) << 4);
    const uint32_t va_lane = (uint32_t)(lane >> 3) * (uint32_t)p.ld_a + chunk;
    const uint32_t vb_lane = (uint32_t)(lane >> 3) * (uint32_t)p.ld_b + chunk;
    typedef __attribute__((address_space(1))) const void gbl_void;
    typedef __attribute__((address_space(3))) void lds_void;
    const __amdgpu_buffer_rsrc_t ra = __builtin_amdgcn_make_buffer_rsrc(reinterpret_cast<void*>(a_wave), 0, 0xFFFFFFFF, 0x00020000);
    auto dma_x = [&](int kt, int stage, int i) {
        __builtin_amdgcn_raw_ptr_buffer_load_lds(ra, (lds_void*)(smem + stage * XS + (wave + 8 * i) * 1024), 16, va_lane,
                                                 (uint32_t)i * a_step + ((uint32_t)kt << 7), 0, 0);
    };
    // The activation tiles do not depend on the group: in the grouped form they are requested before the group's
    // expert is known (one dependent scalar load less in front of the first tile).
#pragma unroll
    for (int i = 0; i < A_IT; ++i) dma_x(0, 0, i);
#pragma unroll
    for (int i = 0; i < A_IT; ++i) dma_x(1 < last ? 1 : last, 1, i);
    const uint8_t* bptr = p.b;
    const float* sbp = p.sb;
    int expert = 0;
    if (MODE == kGrouped) {
        expert = p.m_indices[m0];  // groups start on multiples of 128 = BM rows
        if (expert < 0) {          // a tile of padding (uniform for the workgroup)
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // nothing may land in LDS once the workgroup has gone
            return;
        }
        bptr += (int64_t)expert * p.N * p.ld_b;
        sbp += (int64_t)expert * p.sb_stride_e;
    }
    uint64_t b_wave = reinterpret_cast<uint64_t>(bptr) + ((uint64_t)n0 + (uint64_t)wave * 8) * (uint64_t)p.ld_b;
    asm volatile("" : "+s"(b_wave));
    const __amdgpu_buffer_rsrc_t rb = __builtin_amdgcn_make_buffer_rsrc(reinterpret_cast<void*>(b_wave), 0, 0xFFFFFFFF, 0x00020000);
    auto dma_w = [&](int kt, int stage, int i) {
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rb, (lds_void*)(smem + WBASE + stage * WS + (wave + 8 * i) * 1024), 16, vb_lane,
                                                 (uint32_t)i * b_step + ((uint32_t)kt << 7), 0, 0);
    };

    // activation scales: 8 K steps of this tile's rows per fetch, 4 consecutive floats per thread
    float* const sg_buf = reinterpret_cast<float*>(smem + SBASE);  // [2][8][BM]
    float* const sn_lds = sg_buf + 2 * 8 * BM;                         // [KT][NB]
    const int sg_row = t >> 1, sg_half = t & 1;
    const float* const sg_ptr = p.sa + (int64_t)(m0 + (sg_row < BM ? sg_row : BM - 1)) * KT;
    f32x4 sg = {0.f, 0.f, 0.f, 0.f};
    auto sg_load = [&](int g) {
        const int k0 = 8 * g + 4 * sg_half;
        if (SCALE_VEC) {
            sg = *reinterpret_cast<const f32x4*>(sg_ptr + (k0 + 4 <= KT ? k0 : KT - 4));
        } else {
#pragma unroll
            for (int e = 0; e < 4; ++e) sg[e] = sg_ptr[(k0 + e) < KT ? (k0 + e) : (KT - 1)];
        }
    };
    auto sg_store = [&](int g) {
        if (BM == 256 || sg_row < BM) {
#pragma unroll
            for (int e = 0; e < 4; ++e) sg_buf[((g & 1) * 8 + 4 * sg_half + e) * BM + sg_row] = sg[e];
        }
    };

    f32x4 acc[4][4], P[2][4];  // [w tile][x tile]; raw products of two x tiles
#pragma unroll
    for (int i = 0; i < 4; ++i) {
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};
        P[0][i] = f32x4{0.f, 0.f, 0.f, 0.f};
        P[1][i] = f32x4{0.f, 0.f, 0.f, 0.f};
    }

    const int fsw = ((lrow >> 1) & 1) | (((lrow >> 3) & 1) << 2);
    const int x_off = (wm * 64 + lrow) * 128 + (((2 * quarter) ^ fsw) << 4);
    const int x_off2 = (wm * 64 + lrow) * 128 + (((2 * quarter + 1) ^ fsw) << 4);
    const int w_off = WBASE + (wn * 64 + lrow) * 128 + (((2 * quarter) ^ fsw) << 4);
    const int w_off2 = WBASE + (wn * 64 + lrow) * 128 + (((2 * quarter + 1) ^ fsw) << 4);
    auto frag = [&](int stage_bytes, int off, int off2, int tile16) {
        const uint8_t* base = smem + stage_bytes + tile16 * 2048;
        const i32x4 lo = *reinterpret_cast<const i32x4*>(base + off);
        const i32x4 hi = *reinterpret_cast<const i32x4*>(base + off2);
        i32x8 r;
        r[0] = lo[0]; r[1] = lo[1]; r[2] = lo[2]; r[3] = lo[3];
        r[4] = hi[0]; r[5] = hi[1]; r[6] = hi[2]; r[7] = hi[3];
        return r;
    };
    i32x8 W[4], X[4];
    float sm[4], s_n, s_nu = 0.f;  // s_nu: with the SwiGLU epilogue, the scale of the wave's up rows (s_n: of its gate rows)
    auto read_scales = [&](int kt) {  // s_m of this wave's four x tiles and s_n of its weight block for K step kt
        const int k = kt < last ? kt : last;
        const float* const sgk = sg_buf + (((k >> 3) & 1) * 8 + (k & 7)) * BM + wm * 64 + lrow;
#pragma unroll
        for (int j = 0; j < 4; ++j) sm[j] = sgk[j * 16];
        if (SWIGLU) {
            s_n = sn_lds[k * NB];
            s_nu = sn_lds[k * NB + 1];
        } else {
            s_n = sn_lds[k * NB + (NB == 2 ? wn >> 1 : 0)];
        }
    };

    // prologue: (activation tiles 0 and 1 are under way) weight tiles 0, 1, 2 into their stages, and the scales.  (The compiler waits
    // for every direct-to-LDS load in flight before an LDS store, here those of the scales: it cannot tell that they
    // go elsewhere.  So everything is requested at once and awaited together.)
#pragma unroll
    for (int i = 0; i < B_IT; ++i) dma_w(0, 0, i);
#pragma unroll
    for (int i = 0; i < B_IT; ++i) dma_w(1 < last ? 1 : last, 1, i);
#pragma unroll
    for (int i = 0; i < B_IT; ++i) dma_w(2 < last ? 2 : last, 2, i);
    sg_load(0);
    for (int idx = t; idx < KT * NB; idx += 512) {
        const int k = idx / NB, nb = idx - k * NB;
        sn_lds[idx] = sbp[(int64_t)((n0 >> 7) + nb) * p.sb_stride_n + (int64_t)k * p.sb_stride_k];
    }
    sg_store(0);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    // (the same order as in the loop's tail: the compiler merges both when it counts outstanding reads at the loop head)
    X[0] = frag(0, x_off, x_off2, 0);
    CFP8_PHASE_END();
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        W[i] = frag(0, w_off, w_off2, i);
        CFP8_PHASE_END();
    }
    X[1] = frag(0, x_off, x_off2, 1);
    read_scales(0);
    CFP8_PHASE_END();
    float sc2p = 0.f, sc3p = 0.f;  // scales of the products still waiting in P from the previous step
    float sc2pu = 0.f, sc3pu = 0.f;  // SwiGLU: those of the up tiles (weight tiles 1 and 3)
// the scale of weight tile i: with the SwiGLU epilogue odd tiles are up rows, which have a block scale of their own
#define CFP8_SC(x, i) ((SWIGLU && ((i)&1)) ? x##u : x)

// (the empty statement pins the four FMAs to this place: their results are not needed before the next step, and the
// compiler would otherwise sink them past the branches of the tail, half of them to just behind the barrier)
#define CFP8_RESCALE(i, j, pj, sc)                                                                            \
    {                                                                                                         \
        _Pragma("unroll") for (int e = 0; e < 4; ++e) acc[i][j][e] = __builtin_fmaf(P[pj][i][e], sc, acc[i][j][e]); \
        asm volatile("" : "+v"(acc[i][j]));                                                                   \
    }
#define CFP8_PRODUCT(i, j, pj) \
    P[pj][i] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(W[i], X[j], f32x4{0.f, 0.f, 0.f, 0.f}, 0, 0, 0, 0, 0, 0)
    // Step kt computes from activation stage kt % 2 and weight stage kt % 3; behind its barrier activation tile kt + 2
    // and then weight tile kt + 3 are requested into them.  The next barrier needs everything but those B_IT newest
    // loads: an activation load has one K step to land, a weight load two.
    int ws_cur = 0;  // kt % 3
    for (int kt = 0; kt < KT; ++kt) {
        const int xs_cur = (kt & 1) * XS, xs_nxt = xs_cur ^ XS;
        const int ws_nxt = ws_cur == 2 ? 0 : ws_cur + 1;
        const int kx = kt + 2 < last ? kt + 2 : last;  // past the end: the last tile again, never consumed
        const int kw = kt + 3 < last ? kt + 3 : last;
        // group 0
        X[2] = frag(xs_cur, x_off, x_off2, 2);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            CFP8_RESCALE(i, 2, 0, CFP8_SC(sc2p, i));
            CFP8_PRODUCT(i, 0, 0);
        }
        CFP8_PHASE_END();
        // group 1
        X[3] = frag(xs_cur, x_off, x_off2, 3);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            CFP8_RESCALE(i, 3, 1, CFP8_SC(sc3p, i));
            CFP8_PRODUCT(i, 1, 1);
        }
        CFP8_PHASE_END();
        if (B_IT == 2) CFP8_WAIT_BARRIER(2);
        else CFP8_WAIT_BARRIER(4);
        CFP8_PHASE_END();
        // tail.  The next group's activation scales are stored here, before this step's loads are requested: the
        // compiler makes an LDS store wait for every direct-to-LDS load in flight (it cannot tell that they go
        // elsewhere), and at this point only the weight loads of the previous step are, a whole step old.  The scales
        // were fetched a step earlier and are first read two barriers later, at the end of step 8 g + 7.
        if ((kt & 7) == 6) sg_store((kt >> 3) + 1);
        const float sc0 = sm[0] * s_n, sc1 = sm[1] * s_n;
        const float sc0u = sm[0] * s_nu, sc1u = sm[1] * s_nu;
        sc2p = sm[2] * s_n;
        sc3p = sm[3] * s_n;
        sc2pu = sm[2] * s_nu;
        sc3pu = sm[3] * s_nu;
        X[0] = frag(xs_nxt, x_off, x_off2, 0);  // after the last step: stale data, unused
#pragma unroll
        for (int i = 0; i < A_IT; ++i) dma_x(kx, kt & 1, i);
        if ((kt & 7) == 5) sg_load((kt >> 3) + 1);
        CFP8_PHASE_END();
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            CFP8_RESCALE(i, 0, 0, CFP8_SC(sc0, i));
            CFP8_RESCALE(i, 1, 1, CFP8_SC(sc1, i));
            CFP8_PRODUCT(i, 2, 0);
            CFP8_PRODUCT(i, 3, 1);
            CFP8_PHASE_END();
            W[i] = frag(ws_nxt * WS, w_off, w_off2, i);
            if (i < B_IT) dma_w(kw, ws_cur, i);
            CFP8_PHASE_END();
        }
        X[1] = frag(xs_nxt, x_off, x_off2, 1);
        read_scales(kt + 1);
        CFP8_PHASE_END();
        ws_cur = ws_nxt;
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // nothing may still land in the stages: the epilogues reuse them
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        CFP8_RESCALE(i, 2, 0, CFP8_SC(sc2p, i));
        CFP8_RESCALE(i, 3, 1, CFP8_SC(sc3p, i));
    }
#undef CFP8_RESCALE
#undef CFP8_PRODUCT
#undef CFP8_SC

    // epilogue: lane holds out[m][n .. n+3] for every (i, j)
    if constexpr (SWIGLU) {
        bool row_keep[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) row_keep[j] = p.m_indices[m0 + wm * 64 + j * 16 + lrow] == expert;
        __syncthreads();  // all waves are done reading the operand stages: their first bytes serve the exchange of maxima
        const __amdgpu_buffer_rsrc_t rq = __builtin_amdgcn_make_buffer_rsrc(static_cast<uint8_t*>(p.out) + (int64_t)m0 * p.ld_out, 0, 0x80000000u, 0x00020000);
        const __amdgpu_buffer_rsrc_t rh = __builtin_amdgcn_make_buffer_rsrc(p.h_scales + (int64_t)m0 * p.ld_hs, 0, 0x80000000u, 0x00020000);
        swiglu_quant_epilogue(acc, smem, wm, wn, lrow, quarter, row_keep, rq, rh, (int)p.ld_out, (int)p.ld_hs, tn);
        return;
    }
    if (OUT_F32) {
        // (which rows belong to the group is read before the first store: a load behind a store would have to wait
        // for the store's acknowledgement, loads and stores share one counter)
        bool keep[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) keep[j] = MODE != kGrouped || p.m_indices[m0 + wm * 64 + j * 16 + lrow] == expert;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int m = m0 + wm * 64 + j * 16 + lrow;
            if (!keep[j]) continue;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int n = n0 + wn * 64 + i * 16 + quarter * 4;
                __builtin_nontemporal_store(acc[i][j], reinterpret_cast<f32x4*>(static_cast<float*>(p.out) + (int64_t)m * p.ld_out + n));
            }
        }
        return;
    }
    // bf16: turn the wave's 64 x 64 block through LDS in two halves of 32 rows (row stride 144 B), so that
    // global stores are 16 bytes per lane and 128 contiguous bytes per row, non-temporal
    constexpr int EST = 144;
    uint8_t* const ebuf = smem + wave * (32 * EST);
    const int rd_row = lane >> 3, rd_chunk = lane & 7;
    // Which of this lane's eight output rows belong to the group is read now, before the first store: loads and
    // stores share one counter, so a load behind a store waits for the store's acknowledgement - per row, that
    // was most of a short-K tile's epilogue.
    bool keep[2][4];
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int r = 0; r < 4; ++r)
            keep[h][r] = MODE != kGrouped || p.m_indices[m0 + wm * 64 + h * 32 + r * 8 + rd_row] == expert;
    __syncthreads();  // all waves are done reading the operand stages
#pragma unroll
    for (int h = 0; h < 2; ++h) {
#pragma unroll
        for (int jj = 0; jj < 2; ++jj) {
            const int j = h * 2 + jj;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const f32x4 v = acc[i][j];
                *reinterpret_cast<uint2*>(ebuf + (jj * 16 + lrow) * EST + (i * 16 + quarter * 4) * 2) =
                    make_uint2(pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3]));
            }
        }
        // written and read by the same wave: LDS operations of one wave complete in order
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int row = r * 8 + rd_row;  // 0..31 within the half
            const int m = m0 + wm * 64 + h * 32 + row;
            if (!keep[h][r]) continue;
            const i32x4 d = *reinterpret_cast<const i32x4*>(ebuf + row * EST + rd_chunk * 16);
            __builtin_nontemporal_store(
                d, reinterpret_cast<i32x4*>(static_cast<uint16_t*>(p.out) + (int64_t)m * p.ld_out + n0 + wn * 64 + rd_chunk * 8));
        }
    }
}

// ---------------------------------------------------------------------------
// Block-scaled GEMM on 256 x 256 tiles: eight wavefronts (two per SIMD), each a 128 x 64 block = 8 x tiles times 4 w
// tiles, so a K step moves two thirds of the operand bytes per flop through the load path and three quarters through
// the fragment reads of the 64 x 64 blocks of gemm_block_w8_kernel.  128 accumulator registers per wave leave no room
// to hold a step's products apart for the rescale, so the accumulator of a row is kept in the units of the running
// step's scale: before step k it is multiplied by s(k-1) / s(k) (s = activation scale of the row x weight scale of the
// block), the MFMAs of the step then accumulate straight into it, and the epilogue multiplies by the last s.  In exact
// arithmetic that is sum_k dot_k * s(k); in fp32 it adds one rounding per element and step to the rescale and the
// rounding of the quotient, which is why results differ from the other kernel forms in the last bits.
// Two activation and two weight stages (128 KiB), loads go straight to LDS; a step is six groups of 4 MFMAs (x tiles
// 0..5, each fragment read two groups ahead), the barrier, and a w-major tail on x tiles 6 and 7 whose MFMAs use
// fragments already in registers while the next step's w tiles, x tiles 0 and 1 and scales are read and the tiles after
// next requested.  Requires M % 256 == 0, N % 256 == 0, K / 128 <= 1024.
// ---------------------------------------------------------------------------
template <bool OUT_F32, bool SCALE_VEC>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2))) void gemm_block_256_kernel(const GemmArgs p) {
    constexpr int BM = 256, BN = 256, NB = 2;
    constexpr int XS = BM * 128, WS = BN * 128;
    constexpr int WBASE = 2 * XS;
    constexpr int SBASE = WBASE + 2 * WS;
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    int tm, tn;
    tile_of_block<8>(blockIdx.x, p.tiles_m, p.tiles_n, tm, tn);
    const int m0 = tm * BM, n0 = tn * BN;
    const int t = threadIdx.x, lane = t & 63;
    const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
    const int wm = wave & 1, wn = wave >> 1;  // rows wm * 128 .. + 127, columns wn * 64 .. + 63 of the tile
    const int lrow = lane & 15, quarter = lane >> 4;
    const int KT = p.K >> 7;
    const int last = KT - 1;

    // global -> LDS directly: load i of an operand's K step covers rows (wave + 8 i) * 8 .. + 7 of its tile
    uint64_t a_wave = reinterpret_cast<uint64_t>(p.a) + ((uint64_t)m0 + (uint64_t)wave * 8) * (uint64_t)p.ld_a;
    uint64_t b_wave = reinterpret_cast<uint64_t>(p.b) + ((uint64_t)n0 + (uint64_t)wave * 8) * (uint64_t)p.ld_b;
    uint32_t a_step = 64u * (uint32_t)p.ld_a, b_step = 64u * (uint32_t)p.ld_b;
    asm volatile("" : "+s"(a_wave), "+s"(b_wave), "+s"(a_step), "+s"(b_step));
    const uint32_t chunk = (uint32_t)(((lane & 7) ^ ((wave & 1) * 4 + ((lane >> 4) & 1))) << 4);
    const uint32_t va_lane = (uint32_t)(lane >> 3) * (uint32_t)p.ld_a + chunk;
    const uint32_t vb_lane = (uint32_t)(lane >> 3) * (uint32_t)p.ld_b + chunk;
    typedef __attribute__((address_space(3))) void lds_void;
    const __amdgpu_buffer_rsrc_t ra = __builtin_amdgcn_make_buffer_rsrc(reinterpret_cast<void*>(a_wave), 0, 0xFFFFFFFF, 0x00020000);
    const __amdgpu_buffer_rsrc_t rb = __builtin_amdgcn_make_buffer_rsrc(reinterpret_cast<void*>(b_wave), 0, 0xFFFFFFFF, 0x00020000);
    auto dma_x = [&](int kt, int stage, int i) {
        __builtin_amdgcn_raw_ptr_buffer_load_lds(ra, (lds_void*)(smem + stage * XS + (wave + 8 * i) * 1024), 16, va_lane,
                                                 (uint32_t)i * a_step + ((uint32_t)kt << 7), 0, 0);
    };
    auto dma_w = [&](int kt, int stage, int i) {
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rb, (lds_void*)(smem + WBASE + stage * WS + (wave + 8 * i) * 1024), 16, vb_lane,
                                                 (uint32_t)i * b_step + ((uint32_t)kt << 7), 0, 0);
    };
#pragma unroll
    for (int i = 0; i < 4; ++i) dma_x(0, 0, i);
#pragma unroll
    for (int i = 0; i < 4; ++i) dma_w(0, 0, i);
#pragma unroll
    for (int i = 0; i < 4; ++i) dma_x(1 < last ? 1 : last, 1, i);
#pragma unroll
    for (int i = 0; i < 4; ++i) dma_w(1 < last ? 1 : last, 1, i);

    // activation scales: 8 K steps of this tile's rows per fetch, 4 consecutive floats per thread
    float* const sg_buf = reinterpret_cast<float*>(smem + SBASE);  // [2][8][BM]
    float* const sn_lds = sg_buf + 2 * 8 * BM;                         // [KT][NB]
    const int sg_row = t >> 1, sg_half = t & 1;
    const float* const sg_ptr = p.sa + (int64_t)(m0 + sg_row) * KT;
    f32x4 sg = {0.f, 0.f, 0.f, 0.f};
    auto sg_load = [&](int g) {
        const int k0 = 8 * g + 4 * sg_half;
        if (SCALE_VEC) {
            sg = *reinterpret_cast<const f32x4*>(sg_ptr + (k0 + 4 <= KT ? k0 : KT - 4));
        } else {
#pragma unroll
            for (int e = 0; e < 4; ++e) sg[e] = sg_ptr[(k0 + e) < KT ? (k0 + e) : (KT - 1)];
        }
    };
    auto sg_store = [&](int g) {
#pragma unroll
        for (int e = 0; e < 4; ++e) sg_buf[((g & 1) * 8 + 4 * sg_half + e) * BM + sg_row] = sg[e];
    };

    f32x4 acc[4][8];  // [w tile][x tile], in units of the running step's scale of the row
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 8; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};

    const int fsw = ((lrow >> 1) & 1) | (((lrow >> 3) & 1) << 2);
    const int x_off = (wm * 128 + lrow) * 128 + (((2 * quarter) ^ fsw) << 4);
    const int x_off2 = (wm * 128 + lrow) * 128 + (((2 * quarter + 1) ^ fsw) << 4);
    const int w_off = WBASE + (wn * 64 + lrow) * 128 + (((2 * quarter) ^ fsw) << 4);
    const int w_off2 = WBASE + (wn * 64 + lrow) * 128 + (((2 * quarter + 1) ^ fsw) << 4);
    auto frag = [&](int stage_bytes, int off, int off2, int tile16) {
        const uint8_t* base = smem + stage_bytes + tile16 * 2048;
        const i32x4 lo = *reinterpret_cast<const i32x4*>(base + off);
        const i32x4 hi = *reinterpret_cast<const i32x4*>(base + off2);
        i32x8 r;
        r[0] = lo[0]; r[1] = lo[1]; r[2] = lo[2]; r[3] = lo[3];
        r[4] = hi[0]; r[5] = hi[1]; r[6] = hi[2]; r[7] = hi[3];
        return r;
    };
    i32x8 W[4], X[4];       // x tile j of a step lives in X[j & 3]
    float s_run[8];         // scale the accumulators of x tile j are expressed in
    float s_nxt[8];         // scales of the step whose fragments are being read
    auto read_scales = [&](int kt) {
        const int k = kt < last ? kt : last;
        const float* const sgk = sg_buf + (((k >> 3) & 1) * 8 + (k & 7)) * BM + wm * 128 + lrow;
        const float s_n = sn_lds[k * NB + (wn >> 1)];
#pragma unroll
        for (int j = 0; j < 8; ++j) s_nxt[j] = sgk[j * 16] * s_n;
    };

    sg_load(0);
    for (int idx = t; idx < KT * NB; idx += 512) {
        const int k = idx / NB, nb = idx - k * NB;
        sn_lds[idx] = p.sb[(int64_t)((n0 >> 7) + nb) * p.sb_stride_n + (int64_t)k * p.sb_stride_k];
    }
    sg_store(0);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    X[0] = frag(0, x_off, x_off2, 0);
    CFP8_PHASE_END();
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        W[i] = frag(0, w_off, w_off2, i);
        CFP8_PHASE_END();
    }
    X[1] = frag(0, x_off, x_off2, 1);
    read_scales(0);
    CFP8_PHASE_END();
#pragma unroll
    for (int j = 0; j < 8; ++j) s_run[j] = s_nxt[j];

// the accumulators of x tile j go from the previous step's units to this step's
#define CFP8_RESCALE256(j, rho)                                                                 \
    {                                                                                           \
        _Pragma("unroll") for (int i = 0; i < 4; ++i) {                                         \
            _Pragma("unroll") for (int e = 0; e < 4; ++e) acc[i][j][e] = acc[i][j][e] * (rho); \
            asm volatile("" : "+v"(acc[i][j]));                                                 \
        }                                                                                       \
    }
#define CFP8_MMA256(i, j) \
    acc[i][j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(W[i], X[(j)&3], acc[i][j], 0, 0, 0, 0, 0, 0)

    for (int kt = 0; kt < KT; ++kt) {
        const int xs_cur = (kt & 1) * XS, xs_nxt = xs_cur ^ XS;
        const int ws_nxt = ((kt & 1) ^ 1) * WS;
        const int kn = kt + 2 < last ? kt + 2 : last;  // past the end: the last tile again, never consumed
        // s_nxt holds this step's scales: the factors that take every x tile's accumulators to them
        float rho[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            rho[j] = s_run[j] * __builtin_amdgcn_rcpf(s_nxt[j]);
            s_run[j] = s_nxt[j];
        }
        CFP8_RESCALE256(0, rho[0]);
        // x tiles 0 .. 5: fragment of tile g + 2 read, MFMAs of tile g, rescale of tile g + 1
#pragma unroll
        for (int g = 0; g < 6; ++g) {
            X[(g + 2) & 3] = frag(xs_cur, x_off, x_off2, g + 2);
#pragma unroll
            for (int i = 0; i < 4; ++i) CFP8_MMA256(i, g);
            CFP8_RESCALE256(g + 1, rho[g + 1]);
            CFP8_PHASE_END();
        }
        CFP8_RESCALE256(7, rho[7]);
        CFP8_WAIT_BARRIER(0);  // the tiles of step kt + 1 have landed, everyone is done reading this step's stages
        CFP8_PHASE_END();
        // tail (the next group's activation scales are stored before this step's loads are requested: an LDS store the
        // compiler knows of waits for every direct-to-LDS load in flight)
        if ((kt & 7) == 6) sg_store((kt >> 3) + 1);
        X[0] = frag(xs_nxt, x_off, x_off2, 0);  // after the last step: stale data, unused
#pragma unroll
        for (int i = 0; i < 4; ++i) dma_x(kn, kt & 1, i);
        if ((kt & 7) == 5) sg_load((kt >> 3) + 1);
        CFP8_PHASE_END();
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            CFP8_MMA256(i, 6);
            CFP8_MMA256(i, 7);
            CFP8_PHASE_END();
            W[i] = frag(WBASE - WBASE + ws_nxt, w_off, w_off2, i);
            dma_w(kn, kt & 1, i);
            CFP8_PHASE_END();
        }
        X[1] = frag(xs_nxt, x_off, x_off2, 1);
        read_scales(kt + 1);
        CFP8_PHASE_END();
    }
#undef CFP8_RESCALE256
#undef CFP8_MMA256
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // nothing may still land in the stages: the epilogue reuses them
    // back to plain units: the last step's scale of each row
#pragma unroll
    for (int j = 0; j < 8; ++j)
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int e = 0; e < 4; ++e) acc[i][j][e] *= s_run[j];

    // epilogue: lane holds out[m][n .. n+3] for every (i, j)
    if (OUT_F32) {
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const int m = m0 + wm * 128 + j * 16 + lrow;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int n = n0 + wn * 64 + i * 16 + quarter * 4;
                __builtin_nontemporal_store(acc[i][j], reinterpret_cast<f32x4*>(static_cast<float*>(p.out) + (int64_t)m * p.ld_out + n));
            }
        }
        return;
    }
    // bf16: turn the wave's 128 x 64 block through LDS in four parts of 32 rows (row stride 144 B), so that global
    // stores are 16 bytes per lane and 128 contiguous bytes per row, non-temporal
    constexpr int EST = 144;
    uint8_t* const ebuf = smem + wave * (32 * EST);
    const int rd_row = lane >> 3, rd_chunk = lane & 7;
    __syncthreads();  // all waves are done reading the operand stages
#pragma unroll
    for (int h = 0; h < 4; ++h) {
#pragma unroll
        for (int jj = 0; jj < 2; ++jj) {
            const int j = h * 2 + jj;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const f32x4 v = acc[i][j];
                *reinterpret_cast<uint2*>(ebuf + (jj * 16 + lrow) * EST + (i * 16 + quarter * 4) * 2) =
                    make_uint2(pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3]));
            }
        }
        // written and read by the same wave: LDS operations of one wave complete in order
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int row = r * 8 + rd_row;  // 0..31 within the part
            const int m = m0 + wm * 128 + h * 32 + row;
            const i32x4 d = *reinterpret_cast<const i32x4*>(ebuf + row * EST + rd_chunk * 16);
            __builtin_nontemporal_store(
                d, reinterpret_cast<i32x4*>(static_cast<uint16_t*>(p.out) + (int64_t)m * p.ld_out + n0 + wn * 64 + rd_chunk * 8));
        }
    }
}

// ---------------------------------------------------------------------------
// Launch record.  cfp8_gemm_dispatch_info walks the very dispatch code below with launching switched off and
// gets back which kernels a problem would run, with grid, workgroup size and LDS bytes - so a test can pin, on
// a machine without a GPU, that a shape still takes the kernel form its parity tests cover.
// ---------------------------------------------------------------------------
struct LaunchRecord {
    bool dry = false;   // record only: no HIP call is made
    int cus = 256;      // compute units assumed while dry
    char text[768];
    size_t len = 0;
};
static thread_local LaunchRecord g_rec;
bool dry_run() { return g_rec.dry; }
// returns true when the kernel is to be launched for real
bool note_launch(const char* kernel, unsigned grid, unsigned block, size_t lds) {
    if (!g_rec.dry) return true;
    const int n = snprintf(g_rec.text + g_rec.len, sizeof(g_rec.text) - g_rec.len, "%s%s grid=%u block=%u lds=%zu", g_rec.len ? "; " : "",
                           kernel, grid, block, lds);
    if (n > 0) g_rec.len = g_rec.len + (size_t)n < sizeof(g_rec.text) ? g_rec.len + (size_t)n : sizeof(g_rec.text) - 1;
    return false;
}
static int launched(const char* what) { return dry_run() ? CFP8_OK : check_launch(what); }

// Kernels that use more than 64 KiB of LDS need the limit raised once per device and function.
// `flag` is that (device, function) pair's once-flag; a race on the first call raises it twice, harmlessly.
int raise_lds_limit(const void* fn, size_t lds, std::atomic<bool>& flag) {
    if (dry_run() || flag.load(std::memory_order_relaxed)) return CFP8_OK;
    hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return set_error(CFP8_ELAUNCH, "gemm: cannot raise the LDS limit: %s", hipGetErrorString(e));
    flag.store(true, std::memory_order_relaxed);
    return CFP8_OK;
}
int device_slot() {  // 0..63 for the first 64 ordinals, 64 (never cached) beyond
    if (dry_run()) return 64;
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) dev = 64;
    return dev >= 0 && dev < 64 ? dev : 64;
}

int cu_count() {  // compute units of the current device
    if (dry_run()) return g_rec.cus;
    static std::atomic<int> cached[64];  // zero-initialised
    const int slot = device_slot();
    if (slot < 64) {
        const int c = cached[slot].load(std::memory_order_relaxed);
        if (c > 0) return c;
    }
    int dev = 0, cus = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess ||
        cus <= 0)
        return 256;
    if (slot < 64) cached[slot].store(cus, std::memory_order_relaxed);
    return cus;
}

static int launch_rowwise_256p(GemmArgs& p, int out_dtype, hipStream_t st) {
    p.tiles_m = p.M / 256;
    p.tiles_n = p.N / 256;
    const int64_t tiles = (int64_t)p.tiles_m * p.tiles_n;
    const int cus = cu_count();
    const int64_t blocks = tiles < cus ? tiles : cus;
    // a last round that is at most half full is taken apart into quarter tiles (the strip kernel's ring needs K >= 128
    // only; its stores take any pitch)
    const int64_t rem = tiles % blocks;
    p.tail_tiles = (tiles > blocks && rem > 0 && rem * 2 <= blocks) ? (int)rem : 0;
    constexpr size_t lds = (size_t)(2 + 3) * 256 * 128;
    static std::atomic<bool> raised[65][2];  // zero-initialised
    const int v = out_dtype == CFP8_OUT_F32 ? 1 : 0;
    const void* fn = v ? reinterpret_cast<const void*>(gemm_rowwise_256p_kernel<true>)
                       : reinterpret_cast<const void*>(gemm_rowwise_256p_kernel<false>);
    const int slot = device_slot();
    if (slot == 64) raised[64][v].store(false, std::memory_order_relaxed);
    if (int rc = raise_lds_limit(fn, lds, raised[slot][v])) return rc;
    static_assert(lds == (size_t)5 * (128 + 128) * 128, "the ring of the quarter tiles takes the same LDS");
    {
        char name[64];
        if (p.tail_tiles) snprintf(name, sizeof(name), "gemm_rowwise_256p tail=%d", p.tail_tiles);
        else snprintf(name, sizeof(name), "gemm_rowwise_256p");
        if (!note_launch(name, (unsigned)blocks, 256, lds)) return CFP8_OK;
    }
    if (v) hipLaunchKernelGGL(gemm_rowwise_256p_kernel<true>, dim3((unsigned)blocks), dim3(256), lds, st, p);
    else hipLaunchKernelGGL(gemm_rowwise_256p_kernel<false>, dim3((unsigned)blocks), dim3(256), lds, st, p);
    return check_launch("gemm");
}

static int launch_rowwise_256x128(GemmArgs& p, int out_dtype, hipStream_t st) {
    p.tiles_m = p.M / 256;
    p.tiles_n = p.N / 128;
    const int64_t blocks = (int64_t)p.tiles_m * p.tiles_n;
    constexpr size_t lds = (size_t)(2 * 256 + 3 * 128) * 128 + 384 * sizeof(float);
    static std::atomic<bool> raised[65][2];  // zero-initialised
    const int v = out_dtype == CFP8_OUT_F32 ? 1 : 0;
    const void* fn = v ? reinterpret_cast<const void*>(gemm_rowwise_256x128_kernel<true>)
                       : reinterpret_cast<const void*>(gemm_rowwise_256x128_kernel<false>);
    const int slot = device_slot();
    if (slot == 64) raised[64][v].store(false, std::memory_order_relaxed);
    if (int rc = raise_lds_limit(fn, lds, raised[slot][v])) return rc;
    if (!note_launch("gemm_rowwise_256x128", (unsigned)blocks, 256, lds)) return CFP8_OK;
    if (v) hipLaunchKernelGGL(gemm_rowwise_256x128_kernel<true>, dim3((unsigned)blocks), dim3(256), lds, st, p);
    else hipLaunchKernelGGL(gemm_rowwise_256x128_kernel<false>, dim3((unsigned)blocks), dim3(256), lds, st, p);
    return check_launch("gemm");
}

static int launch_rowwise_256(GemmArgs& p, int out_dtype, hipStream_t st) {
    // more tiles than CUs: one workgroup per CU that walks its tiles and loads the next one under the current one
    // (8192 x 18944 x 3584: 427-439 against 470 us)
    if (p.K >= 384 && (int64_t)(p.M / 256) * (p.N / 256) > cu_count()) return launch_rowwise_256p(p, out_dtype, st);
    p.tiles_m = p.M / 256;
    p.tiles_n = p.N / 256;
    const int64_t blocks = (int64_t)p.tiles_m * p.tiles_n;
    constexpr size_t lds = (size_t)(2 + 3) * 256 * 128;  // two activation stages and three weight stages: all 160 KiB
    static std::atomic<bool> raised[65][2];  // zero-initialised
    const int v = out_dtype == CFP8_OUT_F32 ? 1 : 0;
    const void* fn = v ? reinterpret_cast<const void*>(gemm_rowwise_256_kernel<true>)
                       : reinterpret_cast<const void*>(gemm_rowwise_256_kernel<false>);
    const int slot = device_slot();
    if (slot == 64) raised[64][v].store(false, std::memory_order_relaxed);
    if (int rc = raise_lds_limit(fn, lds, raised[slot][v])) return rc;
    if (!note_launch("gemm_rowwise_256", (unsigned)blocks, 256, lds)) return CFP8_OK;
    if (v) hipLaunchKernelGGL(gemm_rowwise_256_kernel<true>, dim3((unsigned)blocks), dim3(256), lds, st, p);
    else hipLaunchKernelGGL(gemm_rowwise_256_kernel<false>, dim3((unsigned)blocks), dim3(256), lds, st, p);
    return check_launch("gemm");
}

// ---------------------------------------------------------------------------
// Rowwise GEMM for M <= 64 (decode-time batches): the 18944 x 3584 weight is read
// once and nothing else matters, so the kernel is a weight streamer bounded by
// HBM.  A workgroup of 2 NTL waves owns 16 NTL weight rows; wave (nt, kh) takes the 16
// rows of n-tile nt and the kh-th half of every chunk of KS K steps, reads its
// weight fragments straight from global memory into MFMA operand registers
// (streaming loads, one chunk ahead) and the activation fragments of the
// chunk from LDS, where the workgroup stages them once per chunk (activations of
// 64 tokens are as many bytes per chunk as the workgroup's weights, so they must
// not be re-read per wave).  The two K halves are summed through LDS at the end.
// ---------------------------------------------------------------------------
template <int TM, int NTL, int KS, bool OUT_F32>
__global__ __launch_bounds__(NTL * 128) void gemm_rowwise_skinny_kernel(const GemmArgs p) {
    constexpr int NW = NTL * 2;                   // waves: NTL n-tiles x 2 K halves
    constexpr int HS = KS / 2;                    // K steps per wave and chunk
    constexpr int XU = KS * TM * 2;               // wave-wide loads that stage one chunk of activations
    constexpr int XI = (XU + NW - 1) / NW;
    constexpr int XSTAGE = KS * TM * 2048;        // bytes of one activation stage
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    const int t = threadIdx.x, lane = t & 63;
    const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
    const int nt = wave % NTL, kh = wave / NTL;
    const int lrow = lane & 15, quarter = lane >> 4;
    // K slices of one n-block are neighbours in the grid; slice s covers K steps [kt0, KT)
    const int slice = p.k_slices > 1 ? (int)(blockIdx.x % (unsigned)p.k_slices) : 0;
    const int n0 = (p.k_slices > 1 ? (int)(blockIdx.x / (unsigned)p.k_slices) : (int)blockIdx.x) * (NTL * 16);
    const int kt0 = slice * p.slice_steps;
    const int KT = p.k_slices > 1 ? ((p.K >> 7) < kt0 + p.slice_steps ? (p.K >> 7) : kt0 + p.slice_steps) : (p.K >> 7);
    const int chunks = (KT - kt0 + KS - 1) / KS;

    // activation staging: one wave-wide load = 8 rows x 128 bytes of one K step
    const int st_row8 = (lane >> 1) & 7, st_c = ((lane >> 4) << 1) | (lane & 1);
    i32x4 xr[XI];
    auto xload = [&](int chunk) {
#pragma unroll
        for (int i = 0; i < XI; ++i) {
            const int unit = wave + NW * i, ks = unit % KS, row = (unit / KS) * 8 + st_row8;
            const int kt = kt0 + chunk * KS + ks;
            const bool ok = unit < XU && row < p.M && kt < KT;
            xr[i] = ok ? *reinterpret_cast<const i32x4*>(p.a + (int64_t)row * p.ld_a + ((int64_t)kt << 7) + st_c * 16)
                       : i32x4{0, 0, 0, 0};
        }
    };
    auto xstore = [&](int stage) {
#pragma unroll
        for (int i = 0; i < XI; ++i) {
            const int unit = wave + NW * i, ks = unit % KS, row = (unit / KS) * 8 + st_row8;
            if (XU % NW == 0 || unit < XU)
                *reinterpret_cast<i32x4*>(smem + stage * XSTAGE + (ks * TM + (row >> 4)) * 2048 + lds_chunk_offset(row & 15, st_c)) = xr[i];
        }
    };
    // weight fragments: this wave's two K steps of a chunk, 32 contiguous bytes per lane and step
    const int wrow = n0 + nt * 16 + lrow;
    const bool wok = wrow < p.N;
    const uint8_t* wptr = p.b + (int64_t)(wok ? wrow : 0) * p.ld_b + quarter * 32;
    i32x8 wf[HS];
    auto wload = [&](int chunk) {
#pragma unroll
        for (int h = 0; h < HS; ++h) {
            const int kt = kt0 + chunk * KS + kh * HS + h;
            if (wok && kt < KT) {
                const u32x4 lo = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(wptr + ((int64_t)kt << 7)));
                const u32x4 hi = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(wptr + ((int64_t)kt << 7) + 16));
                wf[h][0] = lo[0]; wf[h][1] = lo[1]; wf[h][2] = lo[2]; wf[h][3] = lo[3];
                wf[h][4] = hi[0]; wf[h][5] = hi[1]; wf[h][6] = hi[2]; wf[h][7] = hi[3];
            } else {
#pragma unroll
                for (int e = 0; e < 8; ++e) wf[h][e] = 0;
            }
        }
    };

    f32x4 acc[TM];
#pragma unroll
    for (int j = 0; j < TM; ++j) acc[j] = f32x4{0.f, 0.f, 0.f, 0.f};

    xload(0);
    wload(0);
    xstore(0);
    __syncthreads();
    for (int c = 0; c < chunks; ++c) {
        const int cur = c & 1;
        i32x8 wcur[HS];
#pragma unroll
        for (int h = 0; h < HS; ++h) wcur[h] = wf[h];
        if (c + 1 < chunks) {
            xload(c + 1);
            wload(c + 1);
        }
#pragma unroll
        for (int h = 0; h < HS; ++h) {
            const int ks = kh * HS + h;
#pragma unroll
            for (int j = 0; j < TM; ++j) {
                const i32x8 fx = lds_frag(smem + cur * XSTAGE + (ks * TM + j) * 2048, lrow, quarter);
                acc[j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(wcur[h], fx, acc[j], 0, 0, 0, 0, 0, 0);
            }
        }
        if (c + 1 < chunks) xstore(cur ^ 1);
        __syncthreads();
    }

    // sum the two K halves through LDS (the stages are free now), then scale and store
    float* red = reinterpret_cast<float*>(smem);
    if (kh == 1) {
#pragma unroll
        for (int j = 0; j < TM; ++j) *reinterpret_cast<f32x4*>(red + ((nt * TM + j) * 64 + lane) * 4) = acc[j];
    }
    __syncthreads();
    if (kh == 0) {
        const int n = n0 + nt * 16 + quarter * 4;
        if (n < p.N && p.k_slices > 1) {
            // a K slice: the unscaled sums go to this slice's plane of the partial buffer
            float* const plane = p.partial + (int64_t)slice * p.M * p.N;
#pragma unroll
            for (int j = 0; j < TM; ++j) {
                const int m = j * 16 + lrow;
                if (m >= p.M) continue;
                const f32x4 o = *reinterpret_cast<const f32x4*>(red + ((nt * TM + j) * 64 + lane) * 4);
                f32x4 v;
#pragma unroll
                for (int e = 0; e < 4; ++e) v[e] = acc[j][e] + o[e];
                *reinterpret_cast<f32x4*>(plane + (int64_t)m * p.N + n) = v;
            }
        } else if (n < p.N) {
            const f32x4 sbn = *reinterpret_cast<const f32x4*>(p.sb + n);
#pragma unroll
            for (int j = 0; j < TM; ++j) {
                const int m = j * 16 + lrow;
                if (m >= p.M) continue;
                const f32x4 o = *reinterpret_cast<const f32x4*>(red + ((nt * TM + j) * 64 + lane) * 4);
                const float sam = p.sa[m];
                f32x4 v;
#pragma unroll
                for (int e = 0; e < 4; ++e) v[e] = (acc[j][e] + o[e]) * sam * sbn[e];
                if (OUT_F32) *reinterpret_cast<f32x4*>(static_cast<float*>(p.out) + (int64_t)m * p.ld_out + n) = v;
                else *reinterpret_cast<uint2*>(static_cast<uint16_t*>(p.out) + (int64_t)m * p.ld_out + n) =
                        make_uint2(pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3]));
            }
        }
    }
}

// ---------------------------------------------------------------------------
// Rowwise GEMM for M <= 16 (single-token decode): no LDS staging and no barrier
// in the loop.  A workgroup owns 16 weight rows; its four waves split K (wave w
// takes K steps w, w + 4, ...), each issuing the loads of eight K steps (16 KiB
// of weights per wave) before the first MFMA.  The few activation rows come
// straight from global memory (they stay in L2), rows >= M are zero.
// ---------------------------------------------------------------------------
template <bool OUT_F32>
__global__ __launch_bounds__(256) void gemm_rowwise_gemv_kernel(const GemmArgs p) {
    __shared__ __attribute__((aligned(16))) float red[3 * 64 * 4];
    const int t = threadIdx.x, lane = t & 63;
    const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
    const int lrow = lane & 15, quarter = lane >> 4;
    const int n0 = blockIdx.x * 16;
    const int KT = p.K >> 7;
    const int wrow = n0 + lrow;
    const bool wok = wrow < p.N, xok = lrow < p.M;
    const uint8_t* wptr = p.b + (int64_t)(wok ? wrow : 0) * p.ld_b + quarter * 32;
    const uint8_t* xptr = p.a + (int64_t)(xok ? lrow : 0) * p.ld_a + quarter * 32;
    f32x4 acc = f32x4{0.f, 0.f, 0.f, 0.f};
    for (int base = wave; base < KT; base += 32) {
        u32x4 wl[8], wh[8], xl[8], xh[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int kt = base + 4 * i;
            const bool in = kt < KT;
            const int64_t off = (int64_t)(in ? kt : 0) << 7;
            wl[i] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(wptr + off));
            wh[i] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(wptr + off + 16));
            xl[i] = *reinterpret_cast<const u32x4*>(xptr + off);
            xh[i] = *reinterpret_cast<const u32x4*>(xptr + off + 16);
        }
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const bool in = base + 4 * i < KT;
            i32x8 fw, fx;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                fw[e] = (in && wok) ? (int)wl[i][e] : 0;
                fw[4 + e] = (in && wok) ? (int)wh[i][e] : 0;
                fx[e] = (in && xok) ? (int)xl[i][e] : 0;
                fx[4 + e] = (in && xok) ? (int)xh[i][e] : 0;
            }
            acc = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(fw, fx, acc, 0, 0, 0, 0, 0, 0);
        }
    }
    if (wave > 0) *reinterpret_cast<f32x4*>(red + ((wave - 1) * 64 + lane) * 4) = acc;
    __syncthreads();
    if (wave == 0) {
        const int n = n0 + quarter * 4, m = lrow;
        if (n < p.N && m < p.M) {
#pragma unroll
            for (int w = 0; w < 3; ++w) {
                const f32x4 o = *reinterpret_cast<const f32x4*>(red + (w * 64 + lane) * 4);
#pragma unroll
                for (int e = 0; e < 4; ++e) acc[e] += o[e];
            }
            const f32x4 sbn = *reinterpret_cast<const f32x4*>(p.sb + n);
            const float sam = p.sa[m];
            f32x4 v;
#pragma unroll
            for (int e = 0; e < 4; ++e) v[e] = acc[e] * sam * sbn[e];
            if (OUT_F32) *reinterpret_cast<f32x4*>(static_cast<float*>(p.out) + (int64_t)m * p.ld_out + n) = v;
            else *reinterpret_cast<uint2*>(static_cast<uint16_t*>(p.out) + (int64_t)m * p.ld_out + n) =
                    make_uint2(pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3]));
        }
    }
}

// ---------------------------------------------------------------------------
// FP8 linear for at most 4 tokens and K <= 4096 in ONE launch: the gemv kernel above with the per-token
// quantisation folded in.  Every workgroup first requests its weights (all of a wave's K steps are in
// flight before anything else happens), then its 256 threads quantise the tokens together - each
// thread holds at most two 16-byte vectors of a token between the amax and the cast, exactly the
// arithmetic of the rowwise quantiser - into LDS, from where the MFMA fragments are read.  The
// quantisation hides behind the weight loads, and the separate launch (5 us plus the gap between two
// launches, a quarter of a single-token call) is gone.  Results are bit-identical to the two-launch path.
// ---------------------------------------------------------------------------
template <int MR, bool OUT_F32>
__global__ __launch_bounds__(256) void linear_gemv_fused_kernel(const uint4* __restrict__ x, int64_t ldx, const GemmArgs p) {
    extern __shared__ __attribute__((aligned(16))) uint8_t xq[];  // [M][K] fp8
    __shared__ __attribute__((aligned(16))) float red[3 * 64 * 4];
    __shared__ u32 amax_red[4][MR];
    const int t = threadIdx.x, lane = t & 63;
    const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
    const int lrow = lane & 15, quarter = lane >> 4;
    const int n0 = blockIdx.x * 16;
    const int KT = p.K >> 7;  // <= 32: one batch of 8 K steps per wave
    const int wrow = n0 + lrow;
    const bool wok = wrow < p.N, xok = lrow < p.M;
    const uint8_t* wptr = p.b + (int64_t)(wok ? wrow : 0) * p.ld_b + quarter * 32;
    u32x4 wl[8], wh[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const int kt = wave + 4 * i;
        const int64_t off = (int64_t)(kt < KT ? kt : 0) << 7;
        wl[i] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(wptr + off));
        wh[i] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(wptr + off + 16));
    }
    // the tokens (MR >= M of them): amax, scale, cast - rows >= M read row 0 and are never used
    const int nvec = p.K >> 3;
    uint4 v[MR][2];
    float scale[MR];
#pragma unroll
    for (int r = 0; r < MR; ++r) {
        const uint4* xr = x + (int64_t)(r < p.M ? r : 0) * ldx;
        u32 m = 0;
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int idx = t + 256 * j;
            v[r][j] = idx < nvec ? xr[idx] : make_uint4(0, 0, 0, 0);
            m = absmax8(m, v[r][j]);
        }
        m = wave_max(pk_fold(m));
        if (lane == 0) amax_red[wave][r] = m;
    }
    __syncthreads();
#pragma unroll
    for (int r = 0; r < MR; ++r) {
        const u32 m = umax(umax(amax_red[0][r], amax_red[1][r]), umax(amax_red[2][r], amax_red[3][r]));
        scale[r] = scale_from_amax(amax_from_bits(m));
        const Divider d(scale[r]);
        if (r < p.M) {
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                const int idx = t + 256 * j;
                if (idx < nvec) *reinterpret_cast<uint2*>(xq + (int64_t)r * p.K + idx * 8) = cast8(v[r][j], d);
            }
        }
    }
    __syncthreads();
    f32x4 acc = f32x4{0.f, 0.f, 0.f, 0.f};
    const uint8_t* xrow = xq + (xok ? lrow : 0) * p.K + quarter * 32;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const int kt = wave + 4 * i;
        const bool in = kt < KT;
        const u32x4 xl = *reinterpret_cast<const u32x4*>(xrow + ((in ? kt : 0) << 7));
        const u32x4 xh = *reinterpret_cast<const u32x4*>(xrow + ((in ? kt : 0) << 7) + 16);
        i32x8 fw, fx;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            fw[e] = (in && wok) ? (int)wl[i][e] : 0;
            fw[4 + e] = (in && wok) ? (int)wh[i][e] : 0;
            fx[e] = (in && xok) ? (int)xl[e] : 0;
            fx[4 + e] = (in && xok) ? (int)xh[e] : 0;
        }
        acc = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(fw, fx, acc, 0, 0, 0, 0, 0, 0);
    }
    if (wave > 0) *reinterpret_cast<f32x4*>(red + ((wave - 1) * 64 + lane) * 4) = acc;
    __syncthreads();
    if (wave == 0) {
        const int n = n0 + quarter * 4, m = lrow;
        if (n < p.N && m < p.M) {
#pragma unroll
            for (int w = 0; w < 3; ++w) {
                const f32x4 o = *reinterpret_cast<const f32x4*>(red + (w * 64 + lane) * 4);
#pragma unroll
                for (int e = 0; e < 4; ++e) acc[e] += o[e];
            }
            const f32x4 sbn = *reinterpret_cast<const f32x4*>(p.sb + n);
            float sam = scale[0];
#pragma unroll
            for (int r = 1; r < MR; ++r) sam = m == r ? scale[r] : sam;
            f32x4 o;
#pragma unroll
            for (int e = 0; e < 4; ++e) o[e] = acc[e] * sam * sbn[e];
            if (OUT_F32) *reinterpret_cast<f32x4*>(static_cast<float*>(p.out) + (int64_t)m * p.ld_out + n) = o;
            else *reinterpret_cast<uint2*>(static_cast<uint16_t*>(p.out) + (int64_t)m * p.ld_out + n) =
                    make_uint2(pack_bf16x2(o[0], o[1]), pack_bf16x2(o[2], o[3]));
        }
    }
}

// whether the one-launch kernel above takes the call
static bool fused_gemv_applies(int64_t M, int64_t K, const void* x, int64_t ld_x) {
    return M >= 1 && M <= 4 && K <= 4096 && K % 128 == 0 && aligned16(x) && ld_x % 8 == 0;
}
template <int MR>
static int launch_linear_gemv_fused_mr(const void* x, int64_t ld_x, GemmArgs& p, int out_dtype, hipStream_t st) {
    const int64_t blocks = (p.N + 15) / 16;
    const size_t lds = (size_t)p.M * (size_t)p.K;  // <= 16 KiB
    if (!note_launch("linear_gemv_fused", (unsigned)blocks, 256, lds)) return CFP8_OK;
    if (out_dtype == CFP8_OUT_F32)
        hipLaunchKernelGGL((linear_gemv_fused_kernel<MR, true>), dim3((unsigned)blocks), dim3(256), lds, st, static_cast<const uint4*>(x), ld_x / 8, p);
    else
        hipLaunchKernelGGL((linear_gemv_fused_kernel<MR, false>), dim3((unsigned)blocks), dim3(256), lds, st, static_cast<const uint4*>(x), ld_x / 8, p);
    return check_launch("linear");
}
static int launch_linear_gemv_fused(const void* x, int64_t ld_x, GemmArgs& p, int out_dtype, hipStream_t st) {
    if (p.M == 1) return launch_linear_gemv_fused_mr<1>(x, ld_x, p, out_dtype, st);
    if (p.M == 2) return launch_linear_gemv_fused_mr<2>(x, ld_x, p, out_dtype, st);
    return launch_linear_gemv_fused_mr<4>(x, ld_x, p, out_dtype, st);
}

static int launch_rowwise_gemv(GemmArgs& p, int out_dtype, hipStream_t st) {
    const int64_t blocks = (p.N + 15) / 16;
    if (!note_launch("gemm_rowwise_gemv", (unsigned)blocks, 256, 0)) return CFP8_OK;
    if (out_dtype == CFP8_OUT_F32) hipLaunchKernelGGL(gemm_rowwise_gemv_kernel<true>, dim3((unsigned)blocks), dim3(256), 0, st, p);
    else hipLaunchKernelGGL(gemm_rowwise_gemv_kernel<false>, dim3((unsigned)blocks), dim3(256), 0, st, p);
    return check_launch("gemm");
}

// ---------------------------------------------------------------------------
// Rowwise GEMM for 17..128 tokens (batched decode): a strip kernel.  A workgroup of four waves owns all BM (64 or
// 128) token rows and BN = 16 TN weight rows (80, or 32 for a narrow weight) over the whole of K, so the weight is
// read once by ~N / 80 workgroups - one per CU for an 18944-row weight.  Both operand tiles of a K step go from
// global memory straight into LDS (buffer_load ... lds, the row-major XOR-swizzled layout of the 256 x 256 kernel) in
// a ring of S stages; step kt waits for tile kt, requests tile kt + S - 1 into the stage that step kt - 1 used, and
// computes: one barrier per step, kStripLoads = BM / 32 + ceil(BN / 32) loads per wave and step, the barrier lets the
// loads of the S - 2 tiles in between pass.  What is in flight is therefore S - 1 steps of both operands: the ring
// is as deep as the LDS allows (BM = 64: 8 stages, 70 KB of weights in flight per CU; BM = 128: 5 stages).
// Rows beyond M and N are not fetched: the descriptors end with the matrix and a direct-to-LDS load writes zero for a
// lane beyond its descriptor.  Wave w computes token rows w BM / 4 ... against all TN weight tiles.
// ---------------------------------------------------------------------------
template <int BM, int TN, bool OUT_F32>
__device__ __forceinline__ void rowwise_strip_block(const GemmArgs& p, uint8_t* const smem, const int m0, const int n0, const int t) {
    constexpr int BN = TN * 16;
    constexpr int WROWS = (BN + 31) / 32 * 32;          // weight rows requested per step: 8 per wave and load
    constexpr int LX = BM / 32, LW = WROWS / 32;        // loads per wave and step
    constexpr int XS = BM * 128, WS = WROWS * 128;
    constexpr int S = BM == 64 ? 8 : 5;                 // ring depth: what the LDS holds (160 / 140 KiB)
    constexpr int XT = BM / 64;                         // token tiles per wave
    constexpr uint32_t kEnd = 0xEFFFFFFFu;
    constexpr int WBASE = S * XS;  // smem: S activation stages, then S weight stages
    const int lane = t & 63;
    const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
    const int lrow = lane & 15, quarter = lane >> 4;
    const int KT = p.K >> 7;
    const int last = KT - 1;

    uint64_t a_wave = reinterpret_cast<uint64_t>(p.a) + ((uint64_t)m0 + (uint64_t)wave * 8) * (uint64_t)p.ld_a;
    uint64_t b_wave = reinterpret_cast<uint64_t>(p.b) + ((uint64_t)n0 + (uint64_t)wave * 8) * (uint64_t)p.ld_b;
    uint32_t a_step = 32u * (uint32_t)p.ld_a, b_step = 32u * (uint32_t)p.ld_b;  // leading dimensions are < 2^24
    const int64_t a_rows = (int64_t)p.M - m0 - wave * 8, b_rows = (int64_t)p.N - n0 - wave * 8;
    const int64_t a_left = a_rows > 0 ? a_rows * p.ld_a : 0, b_left = b_rows > 0 ? b_rows * p.ld_b : 0;
    uint32_t a_end = a_left < (int64_t)kEnd ? (uint32_t)a_left : kEnd, b_end = b_left < (int64_t)kEnd ? (uint32_t)b_left : kEnd;
    asm volatile("" : "+s"(a_wave), "+s"(b_wave), "+s"(a_step), "+s"(b_step), "+s"(a_end), "+s"(b_end));
    // load i covers rows (wave + 4 i) * 8 .. + 7; f(r) of row r = (wave + 4 i) * 8 + (lane >> 3) is (wave & 1) * 4 + ((lane >> 4) & 1)
    const uint32_t chunk = (uint32_t)(((lane & 7) ^ ((wave & 1) * 4 + ((lane >> 4) & 1))) << 4);
    const uint32_t va_lane = (uint32_t)(lane >> 3) * (uint32_t)p.ld_a + chunk;
    const uint32_t vb_lane = (uint32_t)(lane >> 3) * (uint32_t)p.ld_b + chunk;
    typedef __attribute__((address_space(3))) void lds_void;
    const __amdgpu_buffer_rsrc_t ra = __builtin_amdgcn_make_buffer_rsrc(reinterpret_cast<void*>(a_wave), 0, (int)a_end, 0x00020000);
    const __amdgpu_buffer_rsrc_t rb = __builtin_amdgcn_make_buffer_rsrc(reinterpret_cast<void*>(b_wave), 0, (int)b_end, 0x00020000);
    auto dma = [&](int kt, int stage) {
#pragma unroll
        for (int i = 0; i < LX; ++i)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(ra, (lds_void*)(smem + stage * XS + (wave + 4 * i) * 1024), 16, va_lane,
                                                     (uint32_t)i * a_step + ((uint32_t)kt << 7), 0, 0);
#pragma unroll
        for (int i = 0; i < LW; ++i)  // the rows of the last load that lie beyond BN are not fetched (zeros nobody reads)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rb, (lds_void*)(smem + WBASE + stage * WS + (wave + 4 * i) * 1024), 16,
                                                     (wave + 4 * i) * 8 < BN ? vb_lane : 0xF0000000u,
                                                     (uint32_t)i * b_step + ((uint32_t)kt << 7), 0, 2);
    };

    // (the argument block may be a copy read from memory, whose pointers the compiler takes for generic ones: said
    // here that they point to global memory)
    typedef __attribute__((address_space(1))) const float gbl_float;
    typedef __attribute__((address_space(1))) const f32x4 gbl_f32x4;
    const gbl_float* const sa_g = (const gbl_float*)p.sa;
    const gbl_float* const sb_g = (const gbl_float*)p.sb;
    // the scales of the epilogue first: they are the oldest loads, every later wait covers them
    float sam[XT];
    f32x4 sbn[TN];
#pragma unroll
    for (int j = 0; j < XT; ++j) {
        const int m = m0 + wave * (BM / 4) + j * 16 + lrow;
        sam[j] = sa_g[m < p.M ? m : p.M - 1];
    }
#pragma unroll
    for (int i = 0; i < TN; ++i) {
        const int n = n0 + i * 16 + quarter * 4;
        sbn[i] = *(const gbl_f32x4*)(sb_g + (n < p.N ? n : 0));
    }

    f32x4 acc[TN][XT];
#pragma unroll
    for (int i = 0; i < TN; ++i)
#pragma unroll
        for (int j = 0; j < XT; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};

    const int fsw = ((lrow >> 1) & 1) | (((lrow >> 3) & 1) << 2);
    const int x_off = (wave * (BM / 4) + lrow) * 128 + (((2 * quarter) ^ fsw) << 4);
    const int x_off2 = (wave * (BM / 4) + lrow) * 128 + (((2 * quarter + 1) ^ fsw) << 4);
    const int w_off = WBASE + lrow * 128 + (((2 * quarter) ^ fsw) << 4);
    const int w_off2 = WBASE + lrow * 128 + (((2 * quarter + 1) ^ fsw) << 4);
    auto frag = [&](int stage_bytes, int off, int off2, int tile16) {
        const uint8_t* base = smem + stage_bytes + tile16 * 2048;
        const i32x4 lo = *reinterpret_cast<const i32x4*>(base + off);
        const i32x4 hi = *reinterpret_cast<const i32x4*>(base + off2);
        return i32x8{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    };

#pragma unroll
    for (int d = 0; d < S - 1; ++d) dma(d < last ? d : last, d);
    int cur = 0;  // kt % S
    for (int kt = 0; kt < KT; ++kt) {
        // tile kt has landed when at most the loads of the S - 2 tiles behind it are outstanding; after the barrier
        // nobody reads the stage of step kt - 1 any more
        asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" ::"n"((S - 2) * (LX + LW)) : "memory");
        const int nxt = cur == 0 ? S - 1 : cur - 1;  // (kt + S - 1) % S
        dma(kt + S - 1 < last ? kt + S - 1 : last, nxt);
        __builtin_amdgcn_sched_barrier(0);
        i32x8 wf[TN];
#pragma unroll
        for (int i = 0; i < TN; ++i) wf[i] = frag(cur * WS, w_off, w_off2, i);
#pragma unroll
        for (int j = 0; j < XT; ++j) {
            const i32x8 xf = frag(cur * XS, x_off, x_off2, j);
#pragma unroll
            for (int i = 0; i < TN; ++i)
                acc[i][j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(wf[i], xf, acc[i][j], 0, 0, 0, 0, 0, 0);
        }
        // the MFMAs are pure functions of registers: pinned here, or the compiler may move them past the next barrier
#pragma unroll
        for (int i = 0; i < TN; ++i)
#pragma unroll
            for (int j = 0; j < XT; ++j) asm volatile("" : "+v"(acc[i][j]));
        cur = cur == S - 1 ? 0 : cur + 1;
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // nothing may land in LDS once the workgroup has gone

#pragma unroll
    for (int j = 0; j < XT; ++j) {
        const int m = m0 + wave * (BM / 4) + j * 16 + lrow;
        if (m >= p.M) continue;
#pragma unroll
        for (int i = 0; i < TN; ++i) {
            const int n = n0 + i * 16 + quarter * 4;
            if (n >= p.N) continue;  // N % 16 == 0: a group of four is inside or outside as a whole
            f32x4 v;
#pragma unroll
            for (int e = 0; e < 4; ++e) v[e] = acc[i][j][e] * sam[j] * sbn[i][e];
            typedef __attribute__((address_space(1))) f32x4 gbl_out4;
            typedef __attribute__((address_space(1))) u32x2 gbl_out2;
            typedef __attribute__((address_space(1))) float gbl_outf;
            typedef __attribute__((address_space(1))) uint16_t gbl_outh;
            if (OUT_F32) *(gbl_out4*)((gbl_outf*)p.out + (int64_t)m * p.ld_out + n) = v;
            else *(gbl_out2*)((gbl_outh*)p.out + (int64_t)m * p.ld_out + n) = u32x2{pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3])};
        }
    }
}

template <int BM, int TN, bool OUT_F32>
__global__ __launch_bounds__(256) void gemm_rowwise_strip_kernel(const GemmArgs p) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    // token blocks of one weight strip are neighbours in the grid: they run at the same time and the second reads the
    // strip from the caches
    rowwise_strip_block<BM, TN, OUT_F32>(p, smem, (int)(blockIdx.x % (unsigned)p.tiles_m) * BM, (int)(blockIdx.x / (unsigned)p.tiles_m) * TN * 16,
                                         (int)threadIdx.x);
}

template <int BM, int TN>
static int launch_rowwise_strip_cfg(GemmArgs& p, int out_dtype, hipStream_t st) {
    constexpr int BN = TN * 16, WROWS = (BN + 31) / 32 * 32, S = BM == 64 ? 8 : 5;
    constexpr size_t lds = (size_t)S * (BM + WROWS) * 128;
    static_assert(lds <= 160 * 1024, "strip kernel LDS");
    p.tiles_m = (p.M + BM - 1) / BM;
    const int64_t blocks = (p.N + BN - 1) / BN * p.tiles_m;
    static std::atomic<bool> raised[65][2];
    const int v = out_dtype == CFP8_OUT_F32 ? 1 : 0;
    const void* fn = v ? reinterpret_cast<const void*>(gemm_rowwise_strip_kernel<BM, TN, true>)
                       : reinterpret_cast<const void*>(gemm_rowwise_strip_kernel<BM, TN, false>);
    const int slot = device_slot();
    if (slot == 64) raised[64][v].store(false, std::memory_order_relaxed);
    if (int rc = raise_lds_limit(fn, lds, raised[slot][v])) return rc;
    {
        char name[64];
        snprintf(name, sizeof(name), "gemm_rowwise_strip<%d,%d>", BM, TN);
        if (!note_launch(name, (unsigned)blocks, 256, lds)) return CFP8_OK;
    }
    if (v) hipLaunchKernelGGL((gemm_rowwise_strip_kernel<BM, TN, true>), dim3((unsigned)blocks), dim3(256), lds, st, p);
    else hipLaunchKernelGGL((gemm_rowwise_strip_kernel<BM, TN, false>), dim3((unsigned)blocks), dim3(256), lds, st, p);
    return check_launch("gemm");
}
// 17..128 tokens; 80 weight rows per workgroup unless that leaves most CUs without one.  (129..256 tokens as two token
// blocks on strips of 160 rows, still one workgroup per CU for an 18944-row weight, measured 41 against 48 us for the
// 256 x 128 tiles at 256 tokens: four ring stages and as many LDS cycles as MFMA cycles per step; not kept.)
static int launch_rowwise_strip(GemmArgs& p, int out_dtype, hipStream_t st) {
    const bool narrow = (p.N + 79) / 80 < 128;
    if (p.M <= 64) return narrow ? launch_rowwise_strip_cfg<64, 2>(p, out_dtype, st) : launch_rowwise_strip_cfg<64, 5>(p, out_dtype, st);
    return narrow ? launch_rowwise_strip_cfg<128, 2>(p, out_dtype, st) : launch_rowwise_strip_cfg<128, 5>(p, out_dtype, st);
}

// Sum of the K slices in slice order, scales, conversion: out[m, n] = (sum_s partial[s, m, n]) * sa[m] * sb[n]
template <bool OUT_F32>
__global__ __launch_bounds__(256) void splitk_reduce_kernel(const float* __restrict__ partial, int slices, int M, int N,
                                                            const float* __restrict__ sa, const float* __restrict__ sb,
                                                            void* __restrict__ out, int64_t ld_out) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;  // one thread per 4 consecutive columns
    const int nq = N >> 2;
    if (i >= (int64_t)M * nq) return;
    const int m = (int)(i / nq), n = (int)(i - (int64_t)m * nq) * 4;
    f32x4 v = *reinterpret_cast<const f32x4*>(partial + (int64_t)m * N + n);
    for (int s = 1; s < slices; ++s) {
        const f32x4 o = *reinterpret_cast<const f32x4*>(partial + ((int64_t)s * M + m) * N + n);
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] += o[e];
    }
    const float sam = sa[m];
    const f32x4 sbn = *reinterpret_cast<const f32x4*>(sb + n);
#pragma unroll
    for (int e = 0; e < 4; ++e) v[e] = v[e] * sam * sbn[e];
    if (OUT_F32) *reinterpret_cast<f32x4*>(static_cast<float*>(out) + (int64_t)m * ld_out + n) = v;
    else *reinterpret_cast<uint2*>(static_cast<uint16_t*>(out) + (int64_t)m * ld_out + n) =
            make_uint2(pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3]));
}

template <int TM, int NTL>
static int launch_rowwise_skinny_cfg(GemmArgs& p, int out_dtype, hipStream_t st) {
    constexpr int KS = 8;
    const int64_t blocks = (p.N + NTL * 16 - 1) / (NTL * 16) * (p.k_slices > 1 ? p.k_slices : 1);
    constexpr size_t lds = (size_t)2 * KS * TM * 2048;   // >= the NTL * TM * 1 KiB of the final reduction
    static_assert(lds >= (size_t)NTL * TM * 1024 && lds <= 160 * 1024, "skinny kernel LDS");
    static std::atomic<bool> raised[65][2];
    const int v = out_dtype == CFP8_OUT_F32 ? 1 : 0;
    const void* fn = v ? reinterpret_cast<const void*>(gemm_rowwise_skinny_kernel<TM, NTL, KS, true>)
                       : reinterpret_cast<const void*>(gemm_rowwise_skinny_kernel<TM, NTL, KS, false>);
    const int slot = device_slot();
    if (slot == 64) raised[64][v].store(false, std::memory_order_relaxed);
    if (int rc = raise_lds_limit(fn, lds, raised[slot][v])) return rc;
    {
        char name[64];
        snprintf(name, sizeof(name), "gemm_rowwise_skinny<%d,%d> k_slices=%d", TM, NTL, p.k_slices > 1 ? p.k_slices : 1);
        const bool real = note_launch(name, (unsigned)blocks, NTL * 128, lds);
        if (p.k_slices > 1) note_launch("splitk_reduce", (unsigned)(((int64_t)p.M * (p.N >> 2) + 255) / 256), 256, 0);
        if (!real) return CFP8_OK;
    }
    if (v) hipLaunchKernelGGL((gemm_rowwise_skinny_kernel<TM, NTL, KS, true>), dim3((unsigned)blocks), dim3(NTL * 128), lds, st, p);
    else hipLaunchKernelGGL((gemm_rowwise_skinny_kernel<TM, NTL, KS, false>), dim3((unsigned)blocks), dim3(NTL * 128), lds, st, p);
    if (p.k_slices > 1) {
        const unsigned rb = (unsigned)(((int64_t)p.M * (p.N >> 2) + 255) / 256);
        if (v) hipLaunchKernelGGL(splitk_reduce_kernel<true>, dim3(rb), dim3(256), 0, st, p.partial, p.k_slices, p.M, p.N, p.sa, p.sb, p.out, p.ld_out);
        else hipLaunchKernelGGL(splitk_reduce_kernel<false>, dim3(rb), dim3(256), 0, st, p.partial, p.k_slices, p.M, p.N, p.sa, p.sb, p.out, p.ld_out);
    }
    return check_launch("gemm");
}

// K slices for a weight with few rows and a long K (e.g. a down projection): with at most 256 n-tiles there
// are too few workgroups to pull the weight at memory speed, so K is cut into up to kMaxSlices slices of at
// least 7 steps, each slice a workgroup, as many as fit one round of 256.  Needs room for the partial sums.
constexpr int kMaxSlices = 8;
static int pick_k_slices(const GemmArgs& p, int ntl) {
    const int64_t ntiles = (p.N + 15) / 16;
    if (!p.partial || ntiles > 256 || p.N % 4) return 1;
    const int64_t nb = (ntiles + ntl - 1) / ntl;
    const int kt = p.K >> 7;
    int64_t s = 256 / nb;
    if (s > kt / 7) s = kt / 7;
    if (s > kMaxSlices) s = kMaxSlices;
    if (s < 2 || (size_t)s * (size_t)p.M * (size_t)p.N * 4 > p.partial_bytes) return 1;
    return (int)s;
}

// Rows of the weight per workgroup.  The kernel is bound by memory latency: a workgroup has one chunk of
// 1 KiB per weight row in flight, so what counts is that all weight rows are resident at once - one
// workgroup per CU (its two activation stages take most of the LDS), as close to 256 workgroups as the
// row count allows.  Measured for 64 tokens on the 18944 x 3584 weight: 80 rows (237 workgroups) 24 us,
// 64 rows (296, a second round on 40 CUs) 36 us, 96 rows (198) 26 us; on 3584 x 3584: 32 rows 15.5 us,
// 80 rows 19.5 us.
template <int TM>
static int launch_rowwise_skinny(GemmArgs& p, int out_dtype, hipStream_t st) {
    const int64_t ntiles = (p.N + 15) / 16, per = (ntiles + 255) / 256;
    p.k_slices = pick_k_slices(p, 4);
    if (p.k_slices > 1) {
        const int kt = p.K >> 7;
        p.slice_steps = (kt + p.k_slices - 1) / p.k_slices;
        return launch_rowwise_skinny_cfg<TM, 4>(p, out_dtype, st);
    }
    if (per <= 2) return launch_rowwise_skinny_cfg<TM, 2>(p, out_dtype, st);
    if (per == 3) return launch_rowwise_skinny_cfg<TM, 3>(p, out_dtype, st);
    if (per == 4) return launch_rowwise_skinny_cfg<TM, 4>(p, out_dtype, st);
    if (per == 6) return launch_rowwise_skinny_cfg<TM, 6>(p, out_dtype, st);
    if (per == 7 || per == 8) return launch_rowwise_skinny_cfg<TM, 8>(p, out_dtype, st);
    return launch_rowwise_skinny_cfg<TM, 5>(p, out_dtype, st);  // 5, and everything that takes several rounds anyway
}

// rowwise, K a multiple of 16 that is not one of 128: the generic kernel's form with a masked last K step
template <int BM, int BN, int WM, int WN>
static int launch_cfg_ktail(GemmArgs& p, int out_dtype, hipStream_t st) {
    p.tiles_m = (p.M + BM - 1) / BM;
    p.tiles_n = (p.N + BN - 1) / BN;
    const int64_t blocks = (int64_t)p.tiles_m * p.tiles_n;
    if (blocks > 0x7FFFFFFFll) return set_error(CFP8_EINVAL, "gemm: too many tiles for one launch");
    constexpr int NT = WM * WN * 64;
    constexpr size_t lds = (size_t)2 * (BM + BN) * 128;
    static_assert(lds <= 64 * 1024, "the K-tail form stays within the default LDS limit");
    {
        char name[64];
        snprintf(name, sizeof(name), "gemm_kernel<%d,%d,%d,%d,rowwise,ktail>", BM, BN, WM, WN);
        if (!note_launch(name, (unsigned)blocks, NT, lds)) return CFP8_OK;
    }
    if (out_dtype == CFP8_OUT_F32)
        hipLaunchKernelGGL((gemm_kernel<BM, BN, WM, WN, kRowwise, true, false, true>), dim3((unsigned)blocks), dim3(NT), lds, st, p);
    else
        hipLaunchKernelGGL((gemm_kernel<BM, BN, WM, WN, kRowwise, false, false, true>), dim3((unsigned)blocks), dim3(NT), lds, st, p);
    return check_launch("gemm");
}

template <int BM, int BN, int WM, int WN, int MODE>
static int launch_cfg(GemmArgs& p, int out_dtype, hipStream_t st) {
    p.tiles_m = (p.M + BM - 1) / BM;
    p.tiles_n = (p.N + BN - 1) / BN;
    const int64_t blocks = (int64_t)p.tiles_m * p.tiles_n;
    if (blocks > 0x7FFFFFFFll) return set_error(CFP8_EINVAL, "gemm: too many tiles for one launch");
    constexpr int NT = WM * WN * 64;
    // two operand stages, plus the turned activation scales of two groups of 8 K steps
    constexpr size_t lds = (size_t)2 * (BM + BN) * 128 + (MODE == kRowwise ? 0 : 2 * 8 * BM * sizeof(float));
    // 16-byte scale loads need every row of the scale matrix 16-byte aligned
    const bool vec = MODE != kRowwise && (p.K >> 7) % 4 == 0 && (reinterpret_cast<uintptr_t>(p.sa) & 15u) == 0;
    using Kern = void (*)(const GemmArgs);
    const Kern table[2][2] = {{gemm_kernel<BM, BN, WM, WN, MODE, false, false>, gemm_kernel<BM, BN, WM, WN, MODE, true, false>},
                              {gemm_kernel<BM, BN, WM, WN, MODE, false, MODE != kRowwise>, gemm_kernel<BM, BN, WM, WN, MODE, true, MODE != kRowwise>}};
    const int f32 = out_dtype == CFP8_OUT_F32;
    const Kern kern = table[vec][f32];
    if (lds > 64 * 1024) {
        static std::atomic<bool> done[65][2][2];  // zero-initialised
        const int slot = device_slot();
        if (slot == 64) done[64][vec][f32].store(false, std::memory_order_relaxed);
        if (int rc = raise_lds_limit(reinterpret_cast<const void*>(kern), lds, done[slot][vec][f32])) return rc;
    }
    {
        char name[64];
        snprintf(name, sizeof(name), "gemm_kernel<%d,%d,%d,%d,%s>", BM, BN, WM, WN, MODE == kRowwise ? "rowwise" : MODE == kBlock ? "block" : "grouped");
        if (!note_launch(name, (unsigned)blocks, NT, lds)) return CFP8_OK;
    }
    hipLaunchKernelGGL(kern, dim3((unsigned)blocks), dim3(NT), lds, st, p);
    return check_launch("gemm");
}

// ---------------------------------------------------------------------------
// Persistent form of the eight-wave block-scaled (256 x 128) and grouped (128 x 256) kernel, as
// gemm_rowwise_256p_kernel is of the rowwise one: one workgroup per CU walks tiles b, b + gridDim.x, ... (grouped:
// those that are not padding); the K steps of consecutive tiles form one stream of loads, so a tile starts on
// operands, fragments and scales that arrived under the previous tile, and its epilogue runs with the next tile's
// loads in flight.  Beyond the stages LDS holds the epilogue buffers of the eight waves (16 rows each), the weight
// scales of two tiles and, grouped, the expert of every row of two tiles.  Requires K >= 384; plain epilogues only.
// ---------------------------------------------------------------------------
constexpr int kPersistentBlockSteps = 32;  // K steps up to which the dispatch sends a problem here (LDS would hold 384)


template <int BM, int BN, int MODE, bool OUT_F32, bool SWIGLU = false>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2))) void gemm_block_w8p_kernel(const GemmArgs p) {
    static_assert((BM == 256 && BN == 128 && MODE == kBlock) || (BM == 128 && BN == 256 && MODE == kGrouped), "eight 64 x 64 wave tiles");
    static_assert(!SWIGLU || (MODE == kGrouped && !OUT_F32), "the SwiGLU epilogue belongs to the grouped 128 x 256 tile");
    constexpr int WM = BM / 64;
    constexpr int XS = BM * 128, WS = BN * 128;
    constexpr int WBASE = 2 * XS;
    constexpr int SBASE = WBASE + 3 * WS;            // turned activation scales: [2][8][BM]
    constexpr int EST = 144;                         // row stride of an epilogue buffer (64 bf16 + 16 B)
    constexpr int EBASE = SBASE + 2 * 8 * BM * 4;    // epilogue buffers: 16 rows per wave
    constexpr int IBASE = EBASE + 8 * 16 * EST;      // grouped: the expert of each row of the current and the next tile, [2][128]
    constexpr int NBASE = IBASE + 2 * 128 * 4;       // weight scales of the current and the next tile
    constexpr int A_IT = BM / 64, B_IT = BN / 64;
    constexpr int NB = BN / 128;
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    const int ntiles = p.tiles_m * p.tiles_n;
    const int t = threadIdx.x, lane = t & 63;
    const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
    const int wm = wave % WM, wn = wave / WM;
    const int lrow = lane & 15, quarter = lane >> 4;
    const int KT = p.K >> 7;
    const int last = KT - 1;
    __builtin_assume(KT >= 3);
    const int KTP = (KT * NB + 63) & ~63;            // floats of one weight-scale buffer
    const int G = (KT + 7) >> 3;                     // groups of eight K steps per tile
    uint32_t a_step = 64u * (uint32_t)p.ld_a, b_step = 64u * (uint32_t)p.ld_b;
    asm volatile("" : "+s"(a_step), "+s"(b_step));
    const uint32_t chunk = (uint32_t)(((lane & 7) ^ ((wave & 1) * 4 + ((lane >> 4) & 1))) << 4);
    const uint32_t va_lane = (uint32_t)(lane >> 3) * (uint32_t)p.ld_a + chunk;
    const uint32_t vb_lane = (uint32_t)(lane >> 3) * (uint32_t)p.ld_b + chunk;
    typedef __attribute__((address_space(3))) void lds_void;
    auto tile_expert = [&](int pid) {  // grouped: the expert of the tile's rows, negative for a tile of padding
        int tm, tn;
        tile_of_block<MODE == kGrouped ? kGroupedBandRows : 8>(pid, p.tiles_m, p.tiles_n, tm, tn);
        return scalar_table_load(p.m_indices, tm * BM);  // groups start on multiples of 128 = BM rows
    };
    auto next_tile = [&](int pid) {  // the next tile of this workgroup that is not padding
        int q = pid + (int)gridDim.x;
        if (MODE == kGrouped)
            while (q < ntiles && tile_expert(q) < 0) q += (int)gridDim.x;
        return q;
    };
    auto tile_rsrc = [&](int pid, int& m0, int& n0, int& expert, __amdgpu_buffer_rsrc_t& ra, __amdgpu_buffer_rsrc_t& rb) {
        int tm, tn;
        tile_of_block<MODE == kGrouped ? kGroupedBandRows : 8>(pid, p.tiles_m, p.tiles_n, tm, tn);
        m0 = tm * BM;
        n0 = tn * BN;
        expert = MODE == kGrouped ? scalar_table_load(p.m_indices, m0) : 0;
        const uint64_t aw = reinterpret_cast<uint64_t>(p.a) + ((uint64_t)m0 + (uint64_t)wave * 8) * (uint64_t)p.ld_a;
        const uint64_t bw = reinterpret_cast<uint64_t>(p.b) + ((uint64_t)expert * (uint64_t)p.N + (uint64_t)n0 + (uint64_t)wave * 8) * (uint64_t)p.ld_b;
        ra = __builtin_amdgcn_make_buffer_rsrc(reinterpret_cast<void*>(aw), 0, 0xFFFFFFFF, 0x00020000);
        rb = __builtin_amdgcn_make_buffer_rsrc(reinterpret_cast<void*>(bw), 0, 0xFFFFFFFF, 0x00020000);
    };
    auto dma_x = [&](__amdgpu_buffer_rsrc_t r, int kt, int stage, int i) {
        __builtin_amdgcn_raw_ptr_buffer_load_lds(r, (lds_void*)(smem + stage * XS + (wave + 8 * i) * 1024), 16, va_lane,
                                                 (uint32_t)i * a_step + ((uint32_t)kt << 7), 0, 0);
    };
    auto dma_w = [&](__amdgpu_buffer_rsrc_t r, int kt, int stage, int i) {
        __builtin_amdgcn_raw_ptr_buffer_load_lds(r, (lds_void*)(smem + WBASE + stage * WS + (wave + 8 * i) * 1024), 16, vb_lane,
                                                 (uint32_t)i * b_step + ((uint32_t)kt << 7), 0, 0);
    };
    // the KT x NB weight scales of the tile at column n0 into buffer par, 64 per wave-wide load (4 bytes per lane);
    // grouped: also the expert of each of the tile's rows (the epilogue writes only the rows of the tile's expert)
    auto dma_sn = [&](int m0_, int n0_, int expert_, int par) {
        const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc(
            const_cast<float*>(p.sb) + (int64_t)expert_ * p.sb_stride_e + (int64_t)(n0_ >> 7) * p.sb_stride_n, 0, 0xFFFFFFFF, 0x00020000);
        for (int base = wave * 64; base < KT * NB; base += 512) {
            const int idx = base + lane < KT * NB ? base + lane : KT * NB - 1;
            const int kk = NB == 2 ? idx >> 1 : idx, nb = NB == 2 ? idx & 1 : 0;
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, (lds_void*)(smem + NBASE + (par * KTP + base) * 4), 4,
                                                     ((uint32_t)nb * (uint32_t)p.sb_stride_n + (uint32_t)kk * (uint32_t)p.sb_stride_k) * 4u, 0, 0, 0);
        }
        if (MODE == kGrouped && wave < 2) {
            const __amdgpu_buffer_rsrc_t ri = __builtin_amdgcn_make_buffer_rsrc(
                const_cast<int32_t*>(p.m_indices) + m0_ + wave * 64, 0, 0xFFFFFFFF, 0x00020000);
            __builtin_amdgcn_raw_ptr_buffer_load_lds(ri, (lds_void*)(smem + IBASE + (par * 128 + wave * 64) * 4), 4, (uint32_t)lane * 4u, 0, 0, 0);
        }
    };
    float* const sg_buf = reinterpret_cast<float*>(smem + SBASE);
    const float* const sn_lds = reinterpret_cast<const float*>(smem + NBASE);
    f32x4 sg = {0.f, 0.f, 0.f, 0.f};
    // (scalar base and one per-lane offset: no per-lane pointers to keep in registers across the loop)
    auto sg_load = [&](int m0_, int g) {  // four of the K / 128 scales of this thread's activation row of the tile at m0_
        // one 16-byte buffer load whatever K is: buffer loads need dword alignment only, what lies past a row's end is
        // the next row's (never used), and past the end of the array the descriptor's size makes the load return zeros
        const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc(
            const_cast<float*>(p.sa) + (int64_t)m0_ * KT, 0, (int)(((int64_t)(p.M - m0_) * KT < (1 << 29) ? (int64_t)(p.M - m0_) * KT : (1 << 29) - 1) * 4), 0x00020000);
        int te = t;  // (addresses rebuilt at every use: kept across the K loop they would cost registers it does not have)
        asm volatile("" : "+v"(te));
        if (BM < 256 && te >= 2 * BM) return;
        const u32x4 v = __builtin_amdgcn_raw_buffer_load_b128(rs, ((te >> 1) * KT + 8 * g + 4 * (te & 1)) * 4, 0, 0);
        sg = f32x4{__uint_as_float(v[0]), __uint_as_float(v[1]), __uint_as_float(v[2]), __uint_as_float(v[3])};
    };
    auto sg_store = [&](int par) {
        int te = t;
        asm volatile("" : "+v"(te));
        if (BM < 256 && te >= 2 * BM) return;
#pragma unroll
        for (int e = 0; e < 4; ++e) sg_buf[((par & 1) * 8 + 4 * (te & 1) + e) * BM + (te >> 1)] = sg[e];
    };

    const int fsw = ((lrow >> 1) & 1) | (((lrow >> 3) & 1) << 2);
    const int x_off = (wm * 64 + lrow) * 128 + (((2 * quarter) ^ fsw) << 4);
    const int x_off2 = (wm * 64 + lrow) * 128 + (((2 * quarter + 1) ^ fsw) << 4);
    const int w_off = WBASE + (wn * 64 + lrow) * 128 + (((2 * quarter) ^ fsw) << 4);
    const int w_off2 = WBASE + (wn * 64 + lrow) * 128 + (((2 * quarter + 1) ^ fsw) << 4);
    auto frag = [&](int stage_bytes, int off, int off2, int tile16) {
        const uint8_t* base = smem + stage_bytes + tile16 * 2048;
        const i32x4 lo = *reinterpret_cast<const i32x4*>(base + off);
        const i32x4 hi = *reinterpret_cast<const i32x4*>(base + off2);
        i32x8 r;
        r[0] = lo[0]; r[1] = lo[1]; r[2] = lo[2]; r[3] = lo[3];
        r[4] = hi[0]; r[5] = hi[1]; r[6] = hi[2]; r[7] = hi[3];
        return r;
    };
    i32x8 W[4], X[4];
    float sm[4], s_n, s_nu = 0.f;  // s_nu: with the SwiGLU epilogue, the scale of the wave's up rows (s_n: of its gate rows)
    auto read_scales = [&](int gpar_, int snpar_, int k) {  // s_m of the wave's four x tiles and s_n of its weight block for step k
        const float* const sgk = sg_buf + (((gpar_ + (k >> 3)) & 1) * 8 + (k & 7)) * BM + wm * 64 + lrow;
#pragma unroll
        for (int j = 0; j < 4; ++j) sm[j] = sgk[j * 16];
        if (SWIGLU) {
            s_n = sn_lds[snpar_ * KTP + k * NB];
            s_nu = sn_lds[snpar_ * KTP + k * NB + 1];
        } else {
            s_n = sn_lds[snpar_ * KTP + k * NB + (NB == 2 ? wn >> 1 : 0)];
        }
    };

    int pid = blockIdx.x;
    if (MODE == kGrouped) {
        while (pid < ntiles && tile_expert(pid) < 0) pid += (int)gridDim.x;
        if (pid >= ntiles) return;  // nothing but padding for this workgroup (uniform)
    }
    int m0, n0, expert;
    __amdgpu_buffer_rsrc_t ra, rb;
    tile_rsrc(pid, m0, n0, expert, ra, rb);
#pragma unroll
    for (int i = 0; i < A_IT; ++i) dma_x(ra, 0, 0, i);
#pragma unroll
    for (int i = 0; i < A_IT; ++i) dma_x(ra, 1, 1, i);
#pragma unroll
    for (int k = 0; k < 3; ++k)
#pragma unroll
        for (int i = 0; i < B_IT; ++i) dma_w(rb, k, k, i);
    dma_sn(m0, n0, expert, 0);
    sg_load(m0, 0);
    sg_store(0);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    X[0] = frag(0, x_off, x_off2, 0);
    CFP8_PHASE_END();
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        W[i] = frag(0, w_off, w_off2, i);
        CFP8_PHASE_END();
    }
    X[1] = frag(0, x_off, x_off2, 1);
    read_scales(0, 0, 0);
    CFP8_PHASE_END();

    f32x4 acc[4][4], P[2][4];  // [w tile][x tile]; raw products of two x tiles
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        P[0][i] = f32x4{0.f, 0.f, 0.f, 0.f};
        P[1][i] = f32x4{0.f, 0.f, 0.f, 0.f};
    }
    float sc2p = 0.f, sc3p = 0.f;  // scales of the products still waiting in P from the previous step
    float sc2pu = 0.f, sc3pu = 0.f;  // SwiGLU: those of the up tiles (weight tiles 1 and 3)
// the scale of weight tile i: with the SwiGLU epilogue odd tiles are up rows, which have a block scale of their own
#define CFP8_SC(x, i) ((SWIGLU && ((i)&1)) ? x##u : x)
    int xs = 0, ws = 0;            // stages of the stream's current step: activation stage (0 or XS bytes), weight stage 0..2
    int gpar = 0, snpar = 0;       // scale buffers of the current tile: first group of activation scales, weight scales

// (the empty statement pins the four FMAs to this place: their results are not needed before the next step, and the
// compiler would otherwise sink them past the branches below to the end of the step, out of the MFMAs' shadow)
#define CFP8_RESCALE(i, j, pj, sc)                                                                            \
    {                                                                                                         \
        _Pragma("unroll") for (int e = 0; e < 4; ++e) acc[i][j][e] = __builtin_fmaf(P[pj][i][e], sc, acc[i][j][e]); \
        asm volatile("" : "+v"(acc[i][j]));                                                                   \
    }
#define CFP8_PRODUCT(i, j, pj) \
    P[pj][i] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(W[i], X[j], f32x4{0.f, 0.f, 0.f, 0.f}, 0, 0, 0, 0, 0, 0)
    for (;;) {
        const int pid_n = next_tile(pid);
        const bool has_next = pid_n < ntiles;
        int m0n = m0, n0n = n0, expert_n = expert;
        __amdgpu_buffer_rsrc_t ran = ra, rbn = rb;
        if (has_next) tile_rsrc(pid_n, m0n, n0n, expert_n, ran, rbn);
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};

        auto step = [&](int kt, auto wait_count) {
            const int xs_nxt = xs ^ XS;
            const int ws_nxt = ws == 2 ? 0 : ws + 1;
            // loads of stream steps + 2 (activations) and + 3 (weights): past this tile's end they fetch the next tile
            const bool xn = kt + 2 >= KT, wnx = kt + 3 >= KT;
            const __amdgpu_buffer_rsrc_t rx = xn ? ran : ra, rw = wnx ? rbn : rb;
            const int kx = xn ? kt + 2 - KT : kt + 2, kw = wnx ? kt + 3 - KT : kt + 3;
            // group 0
            X[2] = frag(xs, x_off, x_off2, 2);
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                CFP8_RESCALE(i, 2, 0, CFP8_SC(sc2p, i));
                CFP8_PRODUCT(i, 0, 0);
            }
            CFP8_PHASE_END();
            // group 1
            X[3] = frag(xs, x_off, x_off2, 3);
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                CFP8_RESCALE(i, 3, 1, CFP8_SC(sc3p, i));
                CFP8_PRODUCT(i, 1, 1);
            }
            CFP8_PHASE_END();
            // all but the B_IT newest weight loads; in a tile's first step the 8 or 16 stores of the previous tile's
            // epilogue are younger than everything this barrier needs
            if constexpr (decltype(wait_count)::value == 0) {
                if constexpr (B_IT == 2) CFP8_WAIT_BARRIER(2);
                else CFP8_WAIT_BARRIER(4);
            } else if constexpr (B_IT == 2) {
                if constexpr (OUT_F32) CFP8_WAIT_BARRIER(18);
                else CFP8_WAIT_BARRIER(10);
            } else {
                if constexpr (SWIGLU) CFP8_WAIT_BARRIER(16);  // 8 byte stores + 4 scale stores per wave
                else if constexpr (OUT_F32) CFP8_WAIT_BARRIER(20);
                else CFP8_WAIT_BARRIER(12);
            }
            CFP8_PHASE_END();
            // tail.  Scales fetched a step earlier go to LDS first (an LDS store the compiler knows of waits for every
            // load in flight; here those are a whole step old): the next group of this tile, or the first group of
            // the next tile, which is read from the end of the tile's last step on, one barrier later.
            if ((kt & 7) == 6 && kt + 2 <= last) sg_store(gpar + (kt >> 3) + 1);
            if (kt == last - 1) sg_store(gpar + G);
            const float sc0 = sm[0] * s_n, sc1 = sm[1] * s_n;
            const float sc0u = sm[0] * s_nu, sc1u = sm[1] * s_nu;
            sc2p = sm[2] * s_n;
            sc3p = sm[3] * s_n;
            sc2pu = sm[2] * s_nu;
            sc3pu = sm[3] * s_nu;
            X[0] = frag(xs_nxt, x_off, x_off2, 0);
            if (kt == last - 1) dma_sn(m0n, n0n, expert_n, snpar ^ 1);  // older than this step's weight loads: landed at the next barrier
#pragma unroll
            for (int i = 0; i < A_IT; ++i) dma_x(rx, kx, xs == 0 ? 0 : 1, i);
            if ((kt & 7) == 5 && kt + 3 <= last) sg_load(m0, (kt >> 3) + 1);
            if (kt == last - 2) sg_load(m0n, 0);
            CFP8_PHASE_END();
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                CFP8_RESCALE(i, 0, 0, CFP8_SC(sc0, i));
                CFP8_RESCALE(i, 1, 1, CFP8_SC(sc1, i));
                CFP8_PRODUCT(i, 2, 0);
                CFP8_PRODUCT(i, 3, 1);
                CFP8_PHASE_END();
                W[i] = frag(ws_nxt * WS, w_off, w_off2, i);
                if (i < B_IT) dma_w(rw, kw, ws, i);
                CFP8_PHASE_END();
            }
            X[1] = frag(xs_nxt, x_off, x_off2, 1);
            if (kt == last) read_scales(gpar + G, snpar ^ 1, 0);
            else read_scales(gpar, snpar, kt + 1);
            CFP8_PHASE_END();
            xs = xs_nxt;
            ws = ws_nxt;
        };
        step(0, std::integral_constant<int, 1>{});
        for (int kt = 1; kt < KT; ++kt) step(kt, std::integral_constant<int, 0>{});
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            CFP8_RESCALE(i, 2, 0, CFP8_SC(sc2p, i));
            CFP8_RESCALE(i, 3, 1, CFP8_SC(sc3p, i));
        }
        sc2p = 0.f;  // the products left in P belong to this tile
        sc3p = 0.f;
        sc2pu = 0.f;
        sc3pu = 0.f;

        // epilogue: lane holds out[m][n .. n+3] for every (i, j).  Its per-lane addresses are derived here, from a
        // lane number the compiler cannot see through: hoisted out of the tile loop they would occupy registers
        // across the K loop, which has none to spare.
        int le = lane;
        asm volatile("" : "+v"(le));
        const int lrow_e = le & 15, quarter_e = le >> 4;
        // grouped: rows that do not belong to the tile's expert stay unwritten.  Their stores are issued all the same,
        // with an offset past the end of the buffer descriptor (the hardware drops them): the barrier of the next tile's
        // first step counts on a fixed number of stores in front of the loads it lets pass.
        if constexpr (SWIGLU) {
            // (which of the wave's rows belong to the tile's expert: read by an instruction of its own, see swiglu_quant_epilogue)
            const uint32_t ie = (uint32_t) reinterpret_cast<uintptr_t>((lds_void*)(smem + IBASE + (snpar * 128 + wm * 64 + lrow_e) * 4));
            int re[4];
            asm volatile("ds_read_b32 %0, %4\n\tds_read_b32 %1, %4 offset:64\n\tds_read_b32 %2, %4 offset:128\n\t"
                         "ds_read_b32 %3, %4 offset:192\n\ts_waitcnt lgkmcnt(0)"
                         : "=&v"(re[0]), "=&v"(re[1]), "=&v"(re[2]), "=&v"(re[3])
                         : "v"(ie)
                         : "memory");
            const bool row_keep[4] = {re[0] == expert, re[1] == expert, re[2] == expert, re[3] == expert};
            const __amdgpu_buffer_rsrc_t rq = __builtin_amdgcn_make_buffer_rsrc(
                static_cast<uint8_t*>(p.out) + (int64_t)m0 * p.ld_out, 0, 0x80000000u, 0x00020000);
            const __amdgpu_buffer_rsrc_t rh = __builtin_amdgcn_make_buffer_rsrc(
                p.h_scales + (int64_t)m0 * p.ld_hs, 0, 0x80000000u, 0x00020000);
            // the exchange buffer is the first 2 KiB of the epilogue buffers; the K loop of the next tile (many barriers)
            // lies between this tile's reads of it and the next tile's writes
            swiglu_quant_epilogue(acc, smem + EBASE, wm, wn, lrow_e, quarter_e, row_keep, rq, rh, (int)p.ld_out, (int)p.ld_hs, n0 >> 8);
        } else {
        const int32_t* const row_expert = reinterpret_cast<const int32_t*>(smem + IBASE) + snpar * 128 + wm * 64;
        const __amdgpu_buffer_rsrc_t ro = __builtin_amdgcn_make_buffer_rsrc(
            static_cast<uint8_t*>(p.out) + (int64_t)m0 * p.ld_out * (OUT_F32 ? 4 : 2), 0, 0x80000000u, 0x00020000);
        if (OUT_F32) {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int r = wm * 64 + j * 16 + lrow_e;
                const bool keep = MODE != kGrouped || row_expert[j * 16 + lrow_e] == expert;
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int n = n0 + wn * 64 + i * 16 + quarter_e * 4;
                    if (MODE == kGrouped) {
                        const f32x4 v = acc[i][j];
                        __builtin_amdgcn_raw_buffer_store_b128(u32x4{__float_as_uint(v[0]), __float_as_uint(v[1]), __float_as_uint(v[2]), __float_as_uint(v[3])}, ro,
                                                               keep ? (uint32_t)((r * (int)p.ld_out + n) * 4) : 0xFFFFFFF0u, 0, 0);
                    } else {
                        __builtin_nontemporal_store(acc[i][j], reinterpret_cast<f32x4*>(static_cast<float*>(p.out) + (int64_t)(m0 + r) * p.ld_out + n));
                    }
                }
            }
        } else {
            // bf16: 16 rows of the wave's 64 x 64 block at a time through the wave's own buffer, so that global stores
            // are 16 bytes per lane and 128 contiguous bytes per row
            uint8_t* const ebuf = smem + EBASE + wave * (16 * EST);
            const int rd_row = le >> 3, rd_chunk = le & 7;
            const uint32_t ebuf_wr = (uint32_t) reinterpret_cast<uintptr_t>((lds_void*)(ebuf + lrow_e * EST + quarter_e * 8));
#pragma unroll
            for (int j = 0; j < 4; ++j) {
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const f32x4 v = acc[i][j];
                    // written as an instruction: in front of an LDS store it knows of, the compiler waits for the
                    // loads of the next tile that are on their way into other parts of LDS
                    const uint64_t two = (uint64_t)pack_bf16x2(v[0], v[1]) | ((uint64_t)pack_bf16x2(v[2], v[3]) << 32);
                    asm volatile("ds_write_b64 %0, %1 offset:%2" ::"v"(ebuf_wr), "v"(two), "n"(i * 32) : "memory");
                }
                // written and read by the same wave: LDS operations of one wave complete in order
#pragma unroll
                for (int r = 0; r < 2; ++r) {
                    const int row = r * 8 + rd_row;
                    const i32x4 d = *reinterpret_cast<const i32x4*>(ebuf + row * EST + rd_chunk * 16);
                    const int rr = wm * 64 + j * 16 + row;
                    if (MODE == kGrouped) {
                        const bool keep = row_expert[j * 16 + row] == expert;
                        __builtin_amdgcn_raw_buffer_store_b128(u32x4{(u32)d[0], (u32)d[1], (u32)d[2], (u32)d[3]}, ro,
                                                               keep ? (uint32_t)((rr * (int)p.ld_out + n0 + wn * 64 + rd_chunk * 8) * 2) : 0xFFFFFFF0u, 0, 0);
                    } else {
                        __builtin_nontemporal_store(
                            d, reinterpret_cast<i32x4*>(static_cast<uint16_t*>(p.out) + (int64_t)(m0 + rr) * p.ld_out + n0 + wn * 64 + rd_chunk * 8));
                    }
                }
            }
        }
        }
        if (!has_next) break;
        pid = pid_n;
        m0 = m0n;
        n0 = n0n;
        ra = ran;
        rb = rbn;
        expert = expert_n;
        gpar = (gpar + G) & 1;
        snpar ^= 1;
    }
#undef CFP8_RESCALE
#undef CFP8_PRODUCT
#undef CFP8_SC
    // the loads past the last tile (they fetched its first steps once more) land before the workgroup gives up its LDS
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
}

// the walking kernels address a tile's weight scales with 32-bit byte offsets from the tile's first scale
static bool scale_offsets_fit_32_bits(const GemmArgs& p) {
    return p.sb_stride_n >= 0 && p.sb_stride_k >= 0 && (int64_t)(p.K >> 7) * p.sb_stride_k + 2 * p.sb_stride_n < (1ll << 29);
}

template <int BM, int BN, int MODE>
static int launch_block_w8p(GemmArgs& p, int out_dtype, hipStream_t st) {
    p.tiles_m = p.M / BM;
    p.tiles_n = p.N / BN;
    const int64_t tiles = (int64_t)p.tiles_m * p.tiles_n;
    if (tiles > 0x7FFFFFFFll) return set_error(CFP8_EINVAL, "gemm: too many tiles for one launch");
    const int cus = cu_count();
    const int64_t blocks = tiles < cus ? tiles : cus;
    const int KT = p.K >> 7;
    // stages, turned activation scales, epilogue buffers, weight scales of two tiles
    const size_t lds = (size_t)(2 * BM + 3 * BN) * 128 + 2 * 8 * BM * sizeof(float) + 8 * 16 * 144 + 2 * 128 * sizeof(int32_t) +
                       (size_t)2 * ((KT * (BN / 128) + 63) & ~63) * sizeof(float);
    using Kern = void (*)(const GemmArgs);
    const int f32 = out_dtype == CFP8_OUT_F32;
    const Kern kern = f32 ? static_cast<Kern>(gemm_block_w8p_kernel<BM, BN, MODE, true>) : static_cast<Kern>(gemm_block_w8p_kernel<BM, BN, MODE, false>);
    constexpr size_t lds_max = 160 * 1024;
    static std::atomic<bool> done[65][2];  // zero-initialised
    const int slot = device_slot();
    if (slot == 64) done[64][f32].store(false, std::memory_order_relaxed);
    if (int rc = raise_lds_limit(reinterpret_cast<const void*>(kern), lds_max, done[slot][f32])) return rc;
    if (!note_launch(MODE == kGrouped ? "gemm_block_w8p<128,256,grouped>" : "gemm_block_w8p<256,128,block>", (unsigned)blocks, 512, lds)) return CFP8_OK;
    hipLaunchKernelGGL(kern, dim3((unsigned)blocks), dim3(512), lds, st, p);
    return check_launch("gemm");
}

template <int BM, int BN, int MODE>
static int launch_block_w8(GemmArgs& p, int out_dtype, hipStream_t st) {
    p.tiles_m = p.M / BM;
    p.tiles_n = p.N / BN;
    const int64_t blocks = (int64_t)p.tiles_m * p.tiles_n;
    if (blocks > 0x7FFFFFFFll) return set_error(CFP8_EINVAL, "gemm: too many tiles for one launch");
    // two activation and three weight stages, the turned activation scales of two groups of 8 K steps, the tile's weight scales
    const size_t lds = (size_t)(2 * BM + 3 * BN) * 128 + 2 * 8 * BM * sizeof(float) + (size_t)(p.K >> 7) * (BN / 128) * sizeof(float);
    const bool vec = (p.K >> 7) % 4 == 0 && (reinterpret_cast<uintptr_t>(p.sa) & 15u) == 0;
    using Kern = void (*)(const GemmArgs);
    const Kern table[2][2] = {{gemm_block_w8_kernel<BM, BN, MODE, false, false>, gemm_block_w8_kernel<BM, BN, MODE, true, false>},
                              {gemm_block_w8_kernel<BM, BN, MODE, false, true>, gemm_block_w8_kernel<BM, BN, MODE, true, true>}};
    const int f32 = out_dtype == CFP8_OUT_F32;
    const Kern kern = table[vec][f32];
    // the limit is raised to the largest size this kernel can ask for, once per device and instantiation
    constexpr size_t lds_max = (size_t)(2 * BM + 3 * BN) * 128 + 2 * 8 * BM * sizeof(float) + kMaxTileWeightScales * sizeof(float);
    static std::atomic<bool> done[65][2][2];  // zero-initialised
    const int slot = device_slot();
    if (slot == 64) done[64][vec][f32].store(false, std::memory_order_relaxed);
    if (int rc = raise_lds_limit(reinterpret_cast<const void*>(kern), lds_max, done[slot][vec][f32])) return rc;
    if (!note_launch(MODE == kGrouped ? "gemm_block_w8<128,256,grouped>" : "gemm_block_w8<256,128,block>", (unsigned)blocks, 512, lds)) return CFP8_OK;
    hipLaunchKernelGGL(kern, dim3((unsigned)blocks), dim3(512), lds, st, p);
    return check_launch("gemm");
}

static int launch_block_256(GemmArgs& p, int out_dtype, hipStream_t st) {
    p.tiles_m = p.M / 256;
    p.tiles_n = p.N / 256;
    const int64_t blocks = (int64_t)p.tiles_m * p.tiles_n;
    if (blocks > 0x7FFFFFFFll) return set_error(CFP8_EINVAL, "gemm: too many tiles for one launch");
    // two activation and two weight stages, the turned activation scales of two groups of 8 K steps, the tile's weight scales
    const size_t lds = (size_t)4 * 256 * 128 + 2 * 8 * 256 * sizeof(float) + (size_t)(p.K >> 7) * 2 * sizeof(float);
    const bool vec = (p.K >> 7) % 4 == 0 && (reinterpret_cast<uintptr_t>(p.sa) & 15u) == 0;
    using Kern = void (*)(const GemmArgs);
    const Kern table[2][2] = {{gemm_block_256_kernel<false, false>, gemm_block_256_kernel<true, false>},
                              {gemm_block_256_kernel<false, true>, gemm_block_256_kernel<true, true>}};
    const int f32 = out_dtype == CFP8_OUT_F32;
    const Kern kern = table[vec][f32];
    constexpr size_t lds_max = (size_t)4 * 256 * 128 + 2 * 8 * 256 * sizeof(float) + 1024 * 2 * sizeof(float);
    static std::atomic<bool> done[65][2][2];  // zero-initialised
    const int slot = device_slot();
    if (slot == 64) done[64][vec][f32].store(false, std::memory_order_relaxed);
    if (int rc = raise_lds_limit(reinterpret_cast<const void*>(kern), lds_max, done[slot][vec][f32])) return rc;
    if (!note_launch("gemm_block_256", (unsigned)blocks, 512, lds)) return CFP8_OK;
    hipLaunchKernelGGL(kern, dim3((unsigned)blocks), dim3(512), lds, st, p);
    return check_launch("gemm");
}

// grouped GEMM over interleaved gate / up weights with the SwiGLU + 1x128 quantisation epilogue
static int launch_grouped_swiglu(GemmArgs& p, hipStream_t st) {
    constexpr int BM = 128, BN = 256;
    p.tiles_m = p.M / BM;
    p.tiles_n = p.N / BN;
    const int64_t blocks = (int64_t)p.tiles_m * p.tiles_n;
    if (blocks > 0x7FFFFFFFll) return set_error(CFP8_EINVAL, "gemm: too many tiles for one launch");
    if ((p.K >> 7) >= 7 && (p.K >> 7) <= kPersistentBlockSteps && blocks > cu_count() && p.ld_out < (1 << 21) && p.ld_hs < (1 << 20) &&
        scale_offsets_fit_32_bits(p)) {
        // 7 to 32 K steps: one workgroup per CU that walks its tiles
        const int cus = cu_count();
        const int KT = p.K >> 7;
        const size_t lds = (size_t)(2 * BM + 3 * BN) * 128 + 2 * 8 * BM * sizeof(float) + 8 * 16 * 144 + 2 * 128 * sizeof(int32_t) +
                           (size_t)2 * ((KT * 2 + 63) & ~63) * sizeof(float);
        using Kern = void (*)(const GemmArgs);
        const Kern kern = gemm_block_w8p_kernel<BM, BN, kGrouped, false, true>;
        static std::atomic<bool> done[65];  // zero-initialised
        const int slot = device_slot();
        if (slot == 64) done[64].store(false, std::memory_order_relaxed);
        if (int rc = raise_lds_limit(reinterpret_cast<const void*>(kern), 160 * 1024, done[slot])) return rc;
        if (!note_launch("gemm_block_w8p<128,256,grouped,swiglu>", (unsigned)(blocks < cus ? blocks : cus), 512, lds)) return CFP8_OK;
        hipLaunchKernelGGL(kern, dim3((unsigned)(blocks < cus ? blocks : cus)), dim3(512), lds, st, p);
        return check_launch("gemm");
    }
    const size_t lds = (size_t)(2 * BM + 3 * BN) * 128 + 2 * 8 * BM * sizeof(float) + (size_t)(p.K >> 7) * (BN / 128) * sizeof(float);
    const bool vec = (p.K >> 7) % 4 == 0 && (reinterpret_cast<uintptr_t>(p.sa) & 15u) == 0;
    using Kern = void (*)(const GemmArgs);
    const Kern kern = vec ? static_cast<Kern>(gemm_block_w8_kernel<BM, BN, kGrouped, false, true, true>)
                          : static_cast<Kern>(gemm_block_w8_kernel<BM, BN, kGrouped, false, false, true>);
    constexpr size_t lds_max = (size_t)(2 * BM + 3 * BN) * 128 + 2 * 8 * BM * sizeof(float) + kMaxTileWeightScales * sizeof(float);
    static std::atomic<bool> done[65][2];  // zero-initialised
    const int slot = device_slot();
    if (slot == 64) done[64][vec].store(false, std::memory_order_relaxed);
    if (int rc = raise_lds_limit(reinterpret_cast<const void*>(kern), lds_max, done[slot][vec])) return rc;
    if (!note_launch("gemm_block_w8<128,256,grouped,swiglu>", (unsigned)blocks, 512, lds)) return CFP8_OK;
    hipLaunchKernelGGL(kern, dim3((unsigned)blocks), dim3(512), lds, st, p);
    return check_launch("gemm");
}

// the kernels that store 16 bytes per lane need every output row 16-byte aligned
static bool out_dtype_pitch_ok(const GemmArgs& p, int out_dtype) {
    return (p.ld_out * (out_dtype == CFP8_OUT_F32 ? 4 : 2)) % 16 == 0;
}

template <int MODE>
static int launch_gemm(GemmArgs& p, int out_dtype, hipStream_t st) {
    if (MODE == kGrouped) {
        // groups are 128-row aligned, so a tile is 128 rows; 256 columns per workgroup (8 waves) read a
        // quarter fewer operand bytes per flop than 128
        // 5 or 6 K steps (a down projection) and at least a tile per CU: the kernel that keeps the activation
        // fragments of a tile row in registers (73472 rows, N = 2048, K = 768: 176 against 241 us on the kernel below)
        if (p.M % 128 == 0 && p.N % 256 == 0 && (p.K >> 7) >= 5 && (p.K >> 7) <= 6 && p.sb_stride_k == 1 && p.ld_out < (1 << 21) &&
            (int64_t)(p.M / 128) * (p.N / 256) >= cu_count() && out_dtype_pitch_ok(p, out_dtype) && grouped_xres_pays(p))
            return launch_grouped_xres(p, out_dtype, st);
        if (p.M % 128 == 0 && p.N % 256 == 0 && (int64_t)(p.M / 128) * (p.N / 256) >= 384 && (p.K >> 7) * 2 <= kMaxTileWeightScales) {
            // 7 to 32 K steps: one workgroup per CU that walks its tiles (73600 rows, N = 2048: K = 896 196 against 215 us,
            // K = 1024 206 against 233 us, K = 1408 271 against 300 us; K = 2048, N = 7168: 1258 against 1360 us; K = 768:
            // 177 against 172 us, and level from K = 4608 on, those stay on the kernel below).  The epilogue addresses a
            // tile's rows with 32-bit offsets.
            if ((p.K >> 7) >= 7 && (p.K >> 7) <= kPersistentBlockSteps && (int64_t)(p.M / 128) * (p.N / 256) > cu_count() &&
                p.ld_out < (1 << 21) && scale_offsets_fit_32_bits(p))
                return launch_block_w8p<128, 256, kGrouped>(p, out_dtype, st);
            return launch_block_w8<128, 256, kGrouped>(p, out_dtype, st);
        }
        if (p.N % 256 == 0 && (int64_t)((p.M + 127) / 128) * (p.N / 256) >= 384)
            return launch_cfg<128, 256, 2, 4, kGrouped>(p, out_dtype, st);
        return launch_cfg<128, 128, 2, 2, kGrouped>(p, out_dtype, st);
    }
    if (MODE == kRowwise && (p.K & 127)) {
        // K = 16 k with a last step shorter than 128: only the generic kernel masks it
        if (p.M <= 16) return launch_cfg_ktail<16, 64, 1, 4>(p, out_dtype, st);
        if (p.M <= 64) return launch_cfg_ktail<64, 64, 1, 4>(p, out_dtype, st);
        return launch_cfg_ktail<128, 128, 2, 2>(p, out_dtype, st);
    }
    if (MODE == kRowwise && p.M <= 16) return launch_rowwise_gemv(p, out_dtype, st);
    if (MODE == kRowwise && p.M <= 128) {
        // a narrow weight with a long K is cut into K slices (the skinny kernels, at most 64 tokens); everything else
        // of 17..128 tokens takes the strip kernel
        if (p.M <= 64 && pick_k_slices(p, 4) > 1) return p.M <= 32 ? launch_rowwise_skinny<2>(p, out_dtype, st) : launch_rowwise_skinny<4>(p, out_dtype, st);
        return launch_rowwise_strip(p, out_dtype, st);
    }
    if (p.M <= 16) return launch_cfg<16, 64, 1, 4, MODE>(p, out_dtype, st);
    if (p.M <= 64) return launch_cfg<64, 64, 1, 4, MODE>(p, out_dtype, st);
    // block scaling, large M: one 8-wave workgroup per CU on a 256 x 128 tile reads a quarter fewer operand
    // bytes than two 128 x 128 workgroups, as long as there are enough tiles to fill the 256 CUs
    // block scaling, any number of tokens above 512: the first M / 256 * 256 rows take the full-tile kernels below, the
    // last < 256 rows are a small problem of their own (rows are independent, so the split changes no row's result)
    // (from 768 rows on: a body of 512 rows would fall below the `M > 512` of the full-tile forms it is cut out for)
    if (MODE == kBlock && p.M >= 768 && p.M % 256 != 0 && p.N % 128 == 0 && (int64_t)(p.M / 256) * (p.N / 128) >= 384 &&
        (p.K >> 7) <= kMaxTileWeightScales) {
        GemmArgs body = p;
        body.M = p.M / 256 * 256;
        if (int rc = launch_gemm<MODE>(body, out_dtype, st)) return rc;
        GemmArgs rest = p;
        rest.M = p.M - body.M;
        rest.a = p.a + (int64_t)body.M * p.ld_a;
        rest.sa = p.sa + (int64_t)body.M * (p.K >> 7);
        rest.out = static_cast<uint8_t*>(p.out) + (int64_t)body.M * p.ld_out * (out_dtype == CFP8_OUT_F32 ? 4 : 2);
        return launch_gemm<MODE>(rest, out_dtype, st);
    }
    // block scaling from 16 K steps on, enough 256 x 256 tiles to fill the CUs in rounds that are at least 4/5 full:
    // the 256 x 256 kernel (4096 x 18432 x K behind a flush: K = 2048 171 against 180 us, 4096 300 against 333, 7168 503
    // against 534, 16384 x 7168 x 18432 2.01 against 2.41 ms; at 12 steps the two are level, below that the walking 256 x 128 form is ahead, 108
    // against 101 us at K = 1024, and 288 tiles on 256 CUs take two rounds, 208 against 186 us).  A last round that is at
    // most half full goes to the 256 x 128 kernel as a launch of its own, as in the rowwise dispatch below.
    if (MODE == kBlock && p.M % 256 == 0 && p.N % 256 == 0 && (p.K >> 7) >= 16 && (p.K >> 7) <= 1024 && out_dtype_pitch_ok(p, out_dtype)) {
        const int64_t tm = p.M / 256, tn = p.N / 256, cus = cu_count(), tiles = tm * tn, rem = tiles % cus;
        const int64_t cut = rem > 0 && rem * 2 <= cus ? (rem + tm - 1) / tm : 0;  // tile-columns that hold the partial round
        const int64_t head = tm * (tn - cut), rounds = (head + cus - 1) / cus;
        if (head >= cus && head * 5 >= rounds * cus * 4) {
            if (cut == 0) return launch_block_256(p, out_dtype, st);
            GemmArgs h = p;
            h.N = (int)((tn - cut) * 256);
            if (int rc = launch_block_256(h, out_dtype, st)) return rc;
            GemmArgs tail = p;
            tail.N = (int)(cut * 256);
            tail.b = p.b + (int64_t)h.N * p.ld_b;
            tail.sb = p.sb + (int64_t)(h.N >> 7) * p.sb_stride_n;
            tail.out = static_cast<uint8_t*>(p.out) + (int64_t)h.N * (out_dtype == CFP8_OUT_F32 ? 4 : 2);
            return launch_block_w8<256, 128, kBlock>(tail, out_dtype, st);  // at most cus tiles of 256 x 128: one round
        }
    }
    if (MODE == kBlock && p.M > 512 && p.M % 256 == 0 && p.N % 128 == 0 && (int64_t)(p.M / 256) * (p.N / 128) >= 384 &&
        (p.K >> 7) <= kMaxTileWeightScales)
    {
        // more tiles than CUs and a short K: one workgroup per CU that walks its tiles, so that a tile does not begin
        // and end on an idle CU (8192 x 4096 x 512: 35 against 42 us, 4096 x 7168 x 2048: 79 against 83 us; from
        // K = 7168 on both forms run level, the K loop is all there is)
        if ((p.K >> 7) >= 3 && (p.K >> 7) <= kPersistentBlockSteps && (int64_t)(p.M / 256) * (p.N / 128) > cu_count() &&
            scale_offsets_fit_32_bits(p))
            return launch_block_w8p<256, 128, kBlock>(p, out_dtype, st);
        return launch_block_w8<256, 128, kBlock>(p, out_dtype, st);
    }
    if (MODE == kBlock && p.M > 512 && (int64_t)((p.M + 255) / 256) * ((p.N + 127) / 128) >= 384)
        return launch_cfg<256, 128, 4, 2, kBlock>(p, out_dtype, st);
    // measured on config 3 (N = 18944, K = 3584): 129..256 rows run 10 % faster as one 256 x 128 tile-row,
    if (MODE == kRowwise && p.M % 256 == 0 && p.N % 128 == 0 && (p.ld_out * (out_dtype == CFP8_OUT_F32 ? 4 : 2)) % 16 == 0) {
        // 256 x 128 tiles of the direct-to-LDS pipeline (2.1 PFLOP/s in steady state against 2.4 for 256 x 256 tiles)
        // wherever 256 x 256 tiles would leave at least half of the CUs idle (2048 x 3584 x 3584: 38 against 52 us,
        // 1024 x 4608 x 3584: 37 against 50 us, 1024 x 3584 x 18944: 155 against 205 us), and for N that is not a
        // multiple of 256
        const int64_t t256 = (int64_t)(p.M / 256) * ((p.N + 255) / 256);
        if (p.N % 256 != 0 || t256 <= 128) return launch_rowwise_256x128(p, out_dtype, st);
        // 512 rows on a wide weight: 129 .. 256 tiles of 256 x 256, one round of the direct-to-LDS kernel (config 3's
        // weight: 58 against 67 us for the register-staged 256 x 256 configuration below)
        if (p.M == 512) return launch_rowwise_256(p, out_dtype, st);
    }
    // 257..512 rows 7 % faster on 256 x 256 tiles than on 128 x 128
    if (MODE == kRowwise && p.M > 128 && p.M <= 256) return launch_cfg<256, 128, 4, 2, kRowwise>(p, out_dtype, st);
    if (MODE == kRowwise && p.M > 256 && p.M <= 512) return launch_cfg<256, 256, 2, 4, kRowwise>(p, out_dtype, st);
    if (p.M <= 512 || MODE != kRowwise) return launch_cfg<128, 128, 2, 2, MODE>(p, out_dtype, st);
    const bool out16 = (p.ld_out * (out_dtype == CFP8_OUT_F32 ? 4 : 2)) % 16 == 0;
    if (p.M % 256 != 0 && p.N % 256 == 0 && out16) {
        // any number of tokens: the first M / 256 * 256 rows take the 256 x 256 kernel, the last < 256 rows are
        // a small problem of their own (rows are independent, so the split changes no result)
        GemmArgs body = p;
        body.M = p.M / 256 * 256;
        if (int rc = launch_gemm<MODE>(body, out_dtype, st)) return rc;
        GemmArgs rest = p;
        rest.M = p.M - body.M;
        rest.a = p.a + (int64_t)body.M * p.ld_a;
        rest.sa = p.sa + body.M;
        rest.out = static_cast<uint8_t*>(p.out) + (int64_t)body.M * p.ld_out * (out_dtype == CFP8_OUT_F32 ? 4 : 2);
        return launch_gemm<MODE>(rest, out_dtype, st);
    }
    if (p.M % 256 == 0 && p.N % 256 == 0 && out16) {
        // One workgroup per CU and equal tiles: the launch runs in rounds of 256 tiles, and a last round that is
        // at most half full costs a whole round.  Then the last tile-columns go to a second launch on smaller
        // tiles and the first launch ends on a full round.
        const int64_t tm = p.M / 256, tn = p.N / 256, rem = (tm * tn) % 256;
        const int64_t cut = (rem + tm - 1) / tm;  // tile-columns that hold the partial round
        if (tm * tn > 256 && rem > 0 && rem <= 128 && cut < tn) {
            // the walking kernel deals the partial round's tiles to all its workgroups as quarter tiles itself
            // (1024 x 18944 x 3584: 81.8 against 84.2 us with the last ten tile-columns as a launch of their own; 8192 tokens:
            // 410 against 411 us)
            if (p.K >= 384) return launch_rowwise_256(p, out_dtype, st);
            GemmArgs head = p;
            head.N = (int)((tn - cut) * 256);
            if (int rc = launch_rowwise_256(head, out_dtype, st)) return rc;
            GemmArgs tail = p;
            tail.N = (int)(cut * 256);
            tail.b = p.b + (int64_t)head.N * p.ld_b;
            tail.sb = p.sb + head.N;
            tail.out = static_cast<uint8_t*>(p.out) + (int64_t)head.N * (out_dtype == CFP8_OUT_F32 ? 4 : 2);
            // few tail tiles: 128 x 128 tiles (4 waves, two workgroups per CU) spread them over more CUs
            // (M = 1024: 40 tile-columns' worth as 160 workgroups 72 us in all, as 80 of 256 x 128 78 us;
            // M = 2048: 320 against 160 workgroups, 125 against 122 us)
            if (cut * tm * 4 <= 256) return launch_cfg<128, 128, 2, 2, kRowwise>(tail, out_dtype, st);
            return launch_cfg<256, 128, 4, 2, kRowwise>(tail, out_dtype, st);
        }
        return launch_rowwise_256(p, out_dtype, st);
    }
    return launch_cfg<256, 256, 2, 4, kRowwise>(p, out_dtype, st);
}

static int check_common(const char* who, const void* a, const void* b, const float* sa, const float* sb,
                        const void* out, int64_t ld_a, int64_t ld_b, int64_t ld_out, int out_dtype, int64_t M,
                        int64_t N, int64_t K, int k_unit = 128) {
    if (M < 0 || N < 0 || K < 0) return set_error(CFP8_EINVAL, "%s: negative shape", who);
    if (M == 0 || N == 0) return CFP8_OK;  // nothing to compute: pointers may be null
    if (!a || !b || !sa || !sb || !out) return set_error(CFP8_EINVAL, "%s: null pointer", who);
    // (block scales cover 128 columns of K; the rowwise forms take any multiple of 16, the last K step then masked)
    if (K == 0 || K % k_unit || N % 16)
        return set_error(CFP8_EINVAL, "%s: K=%lld must be a positive multiple of %d and N=%lld a multiple of 16", who, (long long)K, k_unit, (long long)N);
    // the kernels index rows with 32-bit integers and tile-local byte offsets with 32 bits
    if (M > 0x7FFFFFFFll || N > 0x7FFFFFFFll || K > 0x7FFFFFFFll || ld_a >= (1ll << 24) || ld_b >= (1ll << 24))
        return set_error(CFP8_EINVAL, "%s: shape beyond the supported range (M, N, K < 2^31, leading dimensions < 2^24)", who);
    if (ld_a % 16 || ld_b % 16 || ld_a < K || ld_b < K || ld_out < N || ld_out % 4)
        return set_error(CFP8_EINVAL, "%s: bad leading dimension (ld_a=%lld ld_b=%lld ld_out=%lld)", who, (long long)ld_a, (long long)ld_b, (long long)ld_out);
    if (!aligned16(a) || !aligned16(b) || !aligned16(out) || !aligned16(sb))
        return set_error(CFP8_EINVAL, "%s: operands must be 16-byte aligned", who);
    if (out_dtype != CFP8_OUT_BF16 && out_dtype != CFP8_OUT_F32) return set_error(CFP8_EINVAL, "%s: unknown out_dtype %d", who, out_dtype);
    if (M > 0x7FFFFFFFll || N > 0x7FFFFFFFll || K > 0x7FFFFFFFll) return set_error(CFP8_EINVAL, "%s: dimension exceeds int32", who);
    return CFP8_OK;
}

int launch_quant_rowwise(const void* x, int64_t rows, int64_t cols, int64_t ld_x, void* q, int64_t ld_q,
                         float* scales, bool streaming_out, hipStream_t st);

}  // namespace cfp8

extern "C" int cfp8_gemm_dispatch_info(int kind, int64_t M, int64_t N, int64_t K, int out_dtype, int cus, int with_split_workspace,
                                       char* buf, size_t buf_bytes) {
    using namespace cfp8;
    if (!buf || buf_bytes == 0) return set_error(CFP8_EINVAL, "gemm_dispatch_info: no buffer");
    buf[0] = 0;
    const bool rowwise_kind = kind == CFP8_DISPATCH_ROWWISE || kind == CFP8_DISPATCH_LINEAR;
    if (M <= 0 || N <= 0 || K <= 0 || K % (rowwise_kind ? 16 : 128) || N % 16 || M > 0x7FFFFFFFll || N > 0x7FFFFFFFll || K > 0x7FFFFFFFll || cus <= 0)
        return set_error(CFP8_EINVAL, "gemm_dispatch_info: bad shape or compute-unit count");
    if (out_dtype != CFP8_OUT_BF16 && out_dtype != CFP8_OUT_F32) return set_error(CFP8_EINVAL, "gemm_dispatch_info: unknown out_dtype %d", out_dtype);
    // operands that pass every alignment test; nothing dereferences them
    static const uintptr_t fake = 0x100000;
    GemmArgs p{};
    p.a = reinterpret_cast<const uint8_t*>(fake);
    p.b = reinterpret_cast<const uint8_t*>(fake);
    p.sa = reinterpret_cast<const float*>(fake);
    p.sb = reinterpret_cast<const float*>(fake);
    p.m_indices = reinterpret_cast<const int32_t*>(fake);
    p.out = reinterpret_cast<void*>(fake);
    p.h_scales = reinterpret_cast<float*>(fake);
    p.ld_a = K; p.ld_b = K; p.ld_out = N;
    p.M = (int)M; p.N = (int)N; p.K = (int)K;
    g_rec.dry = true;
    g_rec.cus = cus;
    g_rec.len = 0;
    g_rec.text[0] = 0;
    int rc = CFP8_OK;
    const int64_t kb = K / 128, nb = (N + 127) / 128;
    switch (kind) {
        case CFP8_DISPATCH_ROWWISE:
            rc = launch_gemm<kRowwise>(p, out_dtype, nullptr);
            break;
        case CFP8_DISPATCH_LINEAR:
            if (fused_gemv_applies(M, K, reinterpret_cast<const void*>(fake), K)) {
                rc = launch_linear_gemv_fused(reinterpret_cast<const void*>(fake), K, p, out_dtype, nullptr);
            } else {
                note_launch("quant_rowwise", 0, 256, 0);
                if (with_split_workspace) {
                    p.partial = reinterpret_cast<float*>(fake);
                    p.partial_bytes = cfp8_linear_workspace_bytes_split(M, N, K) - cfp8_linear_workspace_bytes(M, K);
                }
                rc = launch_gemm<kRowwise>(p, out_dtype, nullptr);
            }
            break;
        case CFP8_DISPATCH_BLOCK:
            p.sb_stride_n = kb; p.sb_stride_k = 1;
            rc = launch_gemm<kBlock>(p, out_dtype, nullptr);
            break;
        case CFP8_DISPATCH_GROUPED:
            p.sb_stride_n = kb; p.sb_stride_k = 1; p.sb_stride_e = nb * kb;
            rc = M % 128 ? set_error(CFP8_EINVAL, "gemm_dispatch_info: grouped M must be a multiple of 128") : launch_gemm<kGrouped>(p, out_dtype, nullptr);
            break;
        case CFP8_DISPATCH_GROUPED_SWIGLU:  // N = 2 I; the quantised product has N / 2 columns
            p.sb_stride_n = kb; p.sb_stride_k = 1; p.sb_stride_e = nb * kb;
            p.ld_out = N / 2; p.ld_hs = N / 256;
            rc = (M % 128 || N % 256 || out_dtype != CFP8_OUT_BF16)
                     ? set_error(CFP8_EINVAL, "gemm_dispatch_info: grouped SwiGLU needs M %% 128 == 0, N %% 256 == 0 and the bf16 form")
                     : launch_grouped_swiglu(p, nullptr);
            break;
        default:
            rc = set_error(CFP8_EINVAL, "gemm_dispatch_info: unknown kind %d", kind);
    }
    g_rec.dry = false;
    if (rc) return rc;
    snprintf(buf, buf_bytes, "%s", g_rec.text);
    return CFP8_OK;
}

extern "C" int cfp8_scaled_mm_rowwise(const void* a, int64_t ld_a, const float* sa, const void* b, int64_t ld_b,
                                      const float* sb, void* out, int64_t ld_out, int out_dtype, int64_t M,
                                      int64_t N, int64_t K, void* stream) {
    using namespace cfp8;
    if (int rc = check_common("scaled_mm_rowwise", a, b, sa, sb, out, ld_a, ld_b, ld_out, out_dtype, M, N, K, 16)) return rc;
    if (M == 0 || N == 0) return CFP8_OK;
    if (K == 0) return set_error(CFP8_EINVAL, "scaled_mm_rowwise: K must be positive");
    if (int rc = check_device()) return rc;
    GemmArgs p{};
    p.a = static_cast<const uint8_t*>(a);
    p.b = static_cast<const uint8_t*>(b);
    p.sa = sa;
    p.sb = sb;
    p.out = out;
    p.ld_a = ld_a; p.ld_b = ld_b; p.ld_out = ld_out;
    p.M = (int)M; p.N = (int)N; p.K = (int)K;
    return launch_gemm<kRowwise>(p, out_dtype, static_cast<hipStream_t>(stream));
}

extern "C" size_t cfp8_linear_workspace_bytes(int64_t M, int64_t K) {
    if (M <= 0 || K <= 0) return 0;
    const size_t q = ((size_t)M * (size_t)K + 255) & ~(size_t)255;
    return q + (((size_t)M * 4 + 255) & ~(size_t)255);
}

extern "C" size_t cfp8_linear_workspace_bytes_split(int64_t M, int64_t N, int64_t K) {
    const size_t base = cfp8_linear_workspace_bytes(M, K);
    if (base == 0 || N <= 0 || M <= 16 || M > 64 || (N + 15) / 16 > 256 || N % 4 || (K >> 7) < 14) return base;
    return base + (size_t)cfp8::kMaxSlices * (size_t)M * (size_t)N * 4;
}

extern "C" int cfp8_linear_rowwise(const void* x, int64_t ld_x, const void* w, int64_t ld_w, const float* w_scale,
                                   void* out, int64_t ld_out, int out_dtype, int64_t M, int64_t N, int64_t K,
                                   void* workspace, size_t workspace_bytes, void* stream) {
    using namespace cfp8;
    if (M < 0 || N < 0 || K <= 0) return set_error(CFP8_EINVAL, "linear_rowwise: bad shape");
    if (M == 0 || N == 0) return CFP8_OK;
    if (!workspace || workspace_bytes < cfp8_linear_workspace_bytes(M, K))
        return set_error(CFP8_EWORKSPACE, "linear_rowwise: workspace of %zu bytes needed, %zu given", cfp8_linear_workspace_bytes(M, K), workspace_bytes);
    if (reinterpret_cast<uintptr_t>(workspace) & 255u) return set_error(CFP8_EINVAL, "linear_rowwise: workspace must be 256-byte aligned");
    if (!x || !aligned16(x) || ld_x % 8 || ld_x < K) return set_error(CFP8_EINVAL, "linear_rowwise: bad activation pointer or leading dimension");
    uint8_t* qx = static_cast<uint8_t*>(workspace);
    float* sx = reinterpret_cast<float*>(qx + (((size_t)M * (size_t)K + 255) & ~(size_t)255));
    if (int rc = check_common("linear_rowwise", qx, w, sx, w_scale, out, K, ld_w, ld_out, out_dtype, M, N, K, 16)) return rc;
    if (int rc = check_device()) return rc;
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (fused_gemv_applies(M, K, x, ld_x)) {
        GemmArgs f{};
        f.b = static_cast<const uint8_t*>(w);
        f.sb = w_scale;
        f.out = out;
        f.ld_b = ld_w; f.ld_out = ld_out;
        f.M = (int)M; f.N = (int)N; f.K = (int)K;
        return launch_linear_gemv_fused(x, ld_x, f, out_dtype, st);
    }
    if (int rc = launch_quant_rowwise(x, M, K, ld_x, qx, K, sx, false, st)) return rc;
    GemmArgs p{};
    p.a = qx;
    p.b = static_cast<const uint8_t*>(w);
    p.sa = sx;
    p.sb = w_scale;
    p.out = out;
    p.ld_a = K; p.ld_b = ld_w; p.ld_out = ld_out;
    p.M = (int)M; p.N = (int)N; p.K = (int)K;
    // what the workspace holds beyond the quantised activation is room for split-K partial sums
    const size_t base = cfp8_linear_workspace_bytes(M, K);
    p.partial = reinterpret_cast<float*>(static_cast<uint8_t*>(workspace) + base);
    p.partial_bytes = workspace_bytes - base;
    return launch_gemm<kRowwise>(p, out_dtype, st);
}

extern "C" int cfp8_gemm_block128(const void* a, int64_t ld_a, const float* sa, const void* b, int64_t ld_b,
                                  const float* sb, int64_t sb_stride_n, int64_t sb_stride_k, void* out,
                                  int64_t ld_out, int out_dtype, int64_t M, int64_t N, int64_t K, void* stream) {
    using namespace cfp8;
    if (int rc = check_common("gemm_block128", a, b, sa, sb, out, ld_a, ld_b, ld_out, out_dtype, M, N, K)) return rc;
    if (M == 0 || N == 0) return CFP8_OK;
    if (K == 0) return set_error(CFP8_EINVAL, "gemm_block128: K must be positive");
    if (int rc = check_device()) return rc;
    GemmArgs p{};
    p.a = static_cast<const uint8_t*>(a);
    p.b = static_cast<const uint8_t*>(b);
    p.sa = sa;
    p.sb = sb;
    p.out = out;
    p.ld_a = ld_a; p.ld_b = ld_b; p.ld_out = ld_out;
    p.sb_stride_n = sb_stride_n; p.sb_stride_k = sb_stride_k;
    p.M = (int)M; p.N = (int)N; p.K = (int)K;
    return launch_gemm<kBlock>(p, out_dtype, static_cast<hipStream_t>(stream));
}

extern "C" int cfp8_gemm_grouped_block128(const void* a, int64_t ld_a, const float* sa, const void* b,
                                          const float* sb, const int32_t* m_indices, void* out, int64_t ld_out,
                                          int out_dtype, int64_t M, int64_t N, int64_t K, int64_t E, void* stream) {
    using namespace cfp8;
    if (int rc = check_common("gemm_grouped_block128", a, b, sa, sb, out, ld_a, K, ld_out, out_dtype, M, N, K)) return rc;
    if (M == 0 || N == 0) return CFP8_OK;
    if (!m_indices) return set_error(CFP8_EINVAL, "gemm_grouped_block128: null m_indices");
    if (E <= 0) return set_error(CFP8_EINVAL, "gemm_grouped_block128: E must be positive");
    if (M % 128) return set_error(CFP8_EINVAL, "gemm_grouped_block128: M=%lld must be a multiple of the 128-row group alignment", (long long)M);
    if (K == 0) return set_error(CFP8_EINVAL, "gemm_grouped_block128: K must be positive");
    if (int rc = check_device()) return rc;
    GemmArgs p{};
    p.a = static_cast<const uint8_t*>(a);
    p.b = static_cast<const uint8_t*>(b);
    p.sa = sa;
    p.sb = sb;
    p.m_indices = m_indices;
    p.out = out;
    p.ld_a = ld_a; p.ld_b = K; p.ld_out = ld_out;
    const int64_t nb = (N + 127) / 128, kb = K / 128;
    p.sb_stride_n = kb; p.sb_stride_k = 1; p.sb_stride_e = nb * kb;
    p.M = (int)M; p.N = (int)N; p.K = (int)K;
    return launch_gemm<kGrouped>(p, out_dtype, static_cast<hipStream_t>(stream));
}

extern "C" int cfp8_gemm_grouped_swiglu_quant(const void* a, int64_t ld_a, const float* sa, const void* b, const float* sb,
                                              const int32_t* m_indices, void* q, int64_t ld_q, float* scales,
                                              int64_t M, int64_t I, int64_t K, int64_t E, void* stream) {
    using namespace cfp8;
    if (M < 0 || I < 0 || K < 0) return set_error(CFP8_EINVAL, "gemm_grouped_swiglu_quant: negative shape");
    if (M == 0 || I == 0) return CFP8_OK;
    if (int rc = check_common("gemm_grouped_swiglu_quant", a, b, sa, sb, q, ld_a, K, 2 * I, CFP8_OUT_BF16, M, 2 * I, K)) return rc;
    if (!m_indices || !scales) return set_error(CFP8_EINVAL, "gemm_grouped_swiglu_quant: null m_indices or scales");
    if (E <= 0) return set_error(CFP8_EINVAL, "gemm_grouped_swiglu_quant: E must be positive");
    if (M % 128 || I % 128 || K == 0 || (K >> 7) * 2 > kMaxTileWeightScales)
        return set_error(CFP8_EINVAL, "gemm_grouped_swiglu_quant: needs M %% 128 == 0, I %% 128 == 0 and 0 < K <= %d (M=%lld I=%lld K=%lld)",
                         kMaxTileWeightScales * 64, (long long)M, (long long)I, (long long)K);
    if (ld_q < I || ld_q % 16 || (reinterpret_cast<uintptr_t>(q) & 15u))
        return set_error(CFP8_EINVAL, "gemm_grouped_swiglu_quant: q must be 16-byte aligned with a pitch that is a multiple of 16 and >= I");
    if (int rc = check_device()) return rc;
    GemmArgs p{};
    p.a = static_cast<const uint8_t*>(a);
    p.b = static_cast<const uint8_t*>(b);
    p.sa = sa;
    p.sb = sb;
    p.m_indices = m_indices;
    p.out = q;
    p.h_scales = scales;
    p.ld_hs = I / 128;
    p.ld_a = ld_a; p.ld_b = K; p.ld_out = ld_q;
    const int64_t nb = 2 * I / 128, kb = K / 128;
    p.sb_stride_n = kb; p.sb_stride_k = 1; p.sb_stride_e = nb * kb;
    p.M = (int)M; p.N = (int)(2 * I); p.K = (int)K;
    return launch_grouped_swiglu(p, static_cast<hipStream_t>(stream));
}
