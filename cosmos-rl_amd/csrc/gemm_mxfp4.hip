// GEMM of FP8 activations with MXFP4 weights on the gfx950 matrix cores.
//
//   out[m, n] = sa[m] * sum_k x[m, k] * (e2m1(w[n, k]) * 2^(ws[n, k / 32] - 127))
//
// x is e4m3 [M, K] with one fp32 scale per row (the rowwise activation quantiser), w holds two e2m1 codes per
// byte (even k in the low nibble) with one e8m0 scale byte per 32 consecutive k, the format cfp8_quant_mxfp4
// writes.  v_mfma_scale_f32_16x16x128_f8f6f4 takes the two operands in different formats and applies the
// power-of-two block scales itself: lane l of the "A" operand supplies row l & 15, the 32 k of quarter l >> 4
// (16 bytes of e2m1) and the scale byte of exactly that row and quarter, so an MXFP4 block is one lane's
// share of one instruction and no scale arithmetic is left for the vector ALU.  The activation side passes
// the scale byte 127 (2^0); its fp32 row scale multiplies the accumulator once in the epilogue.
// The two formats number k differently inside the 128 of one instruction (found with one-hot operands and
// pinned by the one-hot test): an e2m1 lane's 32 codes are k = 32 q .. 32 q + 31, an e4m3 lane's registers
// 0-3 are k = 16 q .. 16 q + 15 and its registers 4-7 are k = 64 + 16 q .. 64 + 16 q + 15 (q = l >> 4).
// As in the FP8 kernels the weight tile is the MFMA "A" operand, so a lane's four accumulators are four
// consecutive n of one output row.
//
// Tiles: BM x BN per workgroup, two LDS stages of KB K steps of 128 each, filled through registers.  An activation stage is the
// chunk-major layout of the FP8 kernels (16-row blocks of 2 KiB).  A weight stage holds 64 bytes per row:
// 16-row blocks of 1 KiB, the 16-byte chunk c (0..3) of row r at c * 256 + ((r ^ (c << 2)) & 15) * 16, so that
// a fragment read (16 lanes = 16 rows of one chunk) and a staging store (16 lanes = 4 rows x 4 chunks) each
// cover all 64 banks once.  The scale bytes of a stage are kept as one 32-bit word per (quarter, wave
// column, row of the MFMA tile) whose byte i belongs to the wave's i-th 16-row tile: one LDS read per lane
// and K step, the byte is picked by the instruction's op_sel.
// K need not be a multiple of 128: the chunks of the last step that lie beyond K are loaded as zero with the
// scale byte 127.
#include <atomic>

#include "cfp8_common.h"

namespace cfp8 {

constexpr uint32_t kBeyond = 0xF0000000u;  // a per-lane buffer offset no descriptor here covers (they end at or below 0xEFFFFFFF)

struct Mx4Args {
    const uint8_t* a;    // activations e4m3 [M, K]
    const uint8_t* w;    // weights, packed e2m1 [G, N, K / 2]
    const uint8_t* ws;   // weight scales e8m0 [G, N, K / 32]
    const float* sa;     // [M]
    const int32_t* m_indices;  // [M] or null
    void* out;
    int64_t ld_a, ld_w, ld_ws, ld_out;
    int M, N, K;
    int tiles_m, tiles_n;
};

__device__ __forceinline__ int x_chunk_offset(int row, int c) {
    return ((row >> 4) << 11) + (c << 8) + ((((row & 15) ^ ((c & 1) << 3))) << 4);
}
__device__ __forceinline__ int w_chunk_offset(int row, int c) {
    return ((row >> 4) << 10) + (c << 8) + ((((row & 15) ^ (c << 2)) & 15) << 4);
}

// workgroup id -> tile: every XCD (workgroup ids are dealt to the 8 XCDs round robin) takes a contiguous
// range of tiles, walked in bands of GM tile-rows, so that co-resident workgroups share operand rows in L2
template <int GM>
__device__ __forceinline__ void mx4_tile_of_block(int pid, int tiles_m, int tiles_n, int& tm, int& tn) {
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

template <int I>
__device__ __forceinline__ f32x4 mfma_w4a8(const i32x4& w, const i32x8& x, const f32x4& c, int wscale) {
    const i32x8 a = {w[0], w[1], w[2], w[3], 0, 0, 0, 0};  // e2m1: the first four registers count
    return __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a, x, c, 4 /* A: e2m1 */, 0 /* B: e4m3 */, I, wscale, 0,
                                                            0x7F7F7F7F);
}

template <int BM, int BN, int WM, int WN, int KB, bool OUT_F32>
__global__ __launch_bounds__(WM * WN * 64) void gemm_mxfp4_kernel(const Mx4Args p) {
    constexpr int NT = WM * WN * 64, NW = WM * WN;
    constexpr int WTM = BM / WM, WTN = BN / WN;
    constexpr int TJ = WTM / 16, TI = WTN / 16;  // MFMA tiles per wave: TJ along m, TI along n
    static_assert(WTM % 16 == 0 && WTN % 16 == 0 && TI >= 1 && TI <= 8, "a wave holds 1..8 weight tiles: one or two scale words");
    constexpr int SWN = (TI + 3) / 4;        // scale words per lane and K step
    constexpr int XS = BM * 128, WS = BN * 64, SS = WN * 256 * SWN;  // bytes of one K step (scales: 4 quarters x WN x 16 lanes x SWN words)
    constexpr int SUB = XS + WS + SS;        // one K step of 128
    constexpr int STAGE = KB * SUB;          // a stage holds KB consecutive K steps

    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    auto Xs = [&](int s, int u) { return smem + s * STAGE + u * SUB; };
    auto Ws = [&](int s, int u) { return smem + s * STAGE + u * SUB + XS; };
    auto Ss = [&](int s, int u) { return smem + s * STAGE + u * SUB + XS + WS; };

    int tm, tn;
    mx4_tile_of_block<8>(blockIdx.x, p.tiles_m, p.tiles_n, tm, tn);
    const int m0 = tm * BM, n0 = tn * BN;

    const uint8_t* wptr = p.w;
    const uint8_t* wsptr = p.ws;
    int expert = 0;
    if (p.m_indices) {
        expert = p.m_indices[m0];  // groups start on multiples of 128 rows, BM divides 128
        if (expert < 0) return;    // a tile of padding (uniform for the workgroup)
        wptr += (int64_t)expert * p.N * p.ld_w;
        wsptr += (int64_t)expert * p.N * p.ld_ws;
    }

    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const int wm = wave % WM, wn = wave / WM;
    const int lrow = lane & 15, quarter = lane >> 4;
    const int KT = (p.K + 127) >> 7;        // K steps of 128
    const int NS = (KT + KB - 1) / KB;      // stages

    // global -> registers -> LDS.  Activations: a wave-wide load covers 8 rows x 128 bytes; weights: 16 rows x
    // 64 bytes.  Rows past the edge of a matrix read the last valid row (their products are never stored);
    // chunks past K read the row's first chunk and are replaced by zero.
    constexpr int X_BLK = BM / 8, W_BLK = BN / 16;
    constexpr int X_IT = (X_BLK + NW - 1) / NW, W_IT = (W_BLK + NW - 1) / NW;
    constexpr int S_IT = (BN * 4 + NT - 1) / NT;
    const int x_row8 = (lane >> 1) & 7, x_c = ((lane >> 4) << 1) | (lane & 1);
    const int w_row16 = lane >> 2, w_c = lane & 3;
    uint32_t ox[X_IT], ow[W_IT], os[S_IT];
    i32x4 rx[KB][X_IT], rw[KB][W_IT];
    uint32_t rs[KB][S_IT];
    const uint8_t* const xbase = p.a + (int64_t)m0 * p.ld_a;
    const uint8_t* const wbase = wptr + (int64_t)n0 * p.ld_w;
    const uint8_t* const sbase = wsptr + (int64_t)n0 * p.ld_ws;
#pragma unroll
    for (int i = 0; i < X_IT; ++i) {
        const int r = (wave + NW * i) * 8 + x_row8;
        const int rr = (m0 + r) < p.M ? r : (p.M - 1 - m0);
        ox[i] = (uint32_t)rr * (uint32_t)p.ld_a;
    }
#pragma unroll
    for (int i = 0; i < W_IT; ++i) {
        const int r = (wave + NW * i) * 16 + w_row16;
        const int rr = (n0 + r) < p.N ? r : (p.N - 1 - n0);
        ow[i] = (uint32_t)rr * (uint32_t)p.ld_w;
    }
#pragma unroll
    for (int i = 0; i < S_IT; ++i) {
        const int idx = t + NT * i, r = idx >> 2;
        const int rr = (n0 + r) < p.N ? r : (p.N - 1 - n0);
        os[i] = (uint32_t)rr * (uint32_t)p.ld_ws;
    }
    auto load_tile = [&](int s_) {  // stage s_ of the K loop; stages past the end re-read the last one
        const int s0 = (s_ < NS ? s_ : NS - 1) * KB;
#pragma unroll
        for (int u = 0; u < KB; ++u) {
            const int kt = s0 + u;               // may lie past KT: then every chunk is "beyond K"
            const int k = kt << 7;
            const bool x_ok = k + x_c * 16 < p.K, w_ok = k + w_c * 32 < p.K;
            const uint32_t xk = x_ok ? (uint32_t)(k + x_c * 16) : 0u, wk = w_ok ? (uint32_t)((k >> 1) + w_c * 16) : 0u;
#pragma unroll
            for (int i = 0; i < X_IT; ++i) {
                const i32x4 v = *reinterpret_cast<const i32x4*>(xbase + ox[i] + xk);
                rx[u][i] = x_ok ? v : i32x4{0, 0, 0, 0};
            }
#pragma unroll
            for (int i = 0; i < W_IT; ++i) {
                const i32x4 v = *reinterpret_cast<const i32x4*>(wbase + ow[i] + wk);
                rw[u][i] = w_ok ? v : i32x4{0, 0, 0, 0};
            }
#pragma unroll
            for (int i = 0; i < S_IT; ++i) {
                const int kb = (kt << 2) + ((t + NT * i) & 3);
                const bool ok = kb * 32 < p.K;
                const uint32_t v = sbase[os[i] + (ok ? (uint32_t)kb : 0u)];
                rs[u][i] = ok ? v : 127u;
            }
        }
    };
    auto store_tile = [&](int stage) {
#pragma unroll
        for (int u = 0; u < KB; ++u) {
#pragma unroll
            for (int i = 0; i < X_IT; ++i) {
                const int r = (wave + NW * i) * 8 + x_row8;
                if (X_BLK % NW == 0 || r < BM) *reinterpret_cast<i32x4*>(Xs(stage, u) + x_chunk_offset(r, x_c)) = rx[u][i];
            }
#pragma unroll
            for (int i = 0; i < W_IT; ++i) {
                const int r = (wave + NW * i) * 16 + w_row16;
                if (W_BLK % NW == 0 || r < BN) *reinterpret_cast<i32x4*>(Ws(stage, u) + w_chunk_offset(r, w_c)) = rw[u][i];
            }
#pragma unroll
            for (int i = 0; i < S_IT; ++i) {
                const int idx = t + NT * i, r = idx >> 2, kb = idx & 3;
                // word of (quarter kb, wave column r / WTN, tile row r % 16), byte = tile index inside the wave's columns
                if ((BN * 4) % NT == 0 || r < BN)
                    Ss(stage, u)[((kb * WN + r / WTN) * 16 + (r & 15)) * (4 * SWN) + ((r % WTN) >> 4)] = (uint8_t)rs[u][i];
            }
        }
    };

    f32x4 acc[TI][TJ];
#pragma unroll
    for (int i = 0; i < TI; ++i)
#pragma unroll
        for (int j = 0; j < TJ; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};

    // At the top of stage s, LDS stage s & 1 holds the K steps of stage s and the staging registers hold stage s + 1.
    // They are stored to the other LDS stage (free since the barrier that ended stage s - 1) after the first
    // step's fragments have been read, and the loads of stage s + 2 follow at once.  The last iteration stores a
    // stage nobody reads.
    load_tile(0);
    store_tile(0);
    load_tile(1);
    __syncthreads();

    for (int s = 0; s < NS; ++s) {
        const int cur = s & 1;
#pragma unroll
        for (int u = 0; u < KB; ++u) {
            i32x4 fw[TI];
#pragma unroll
            for (int i = 0; i < TI; ++i)
                fw[i] = *reinterpret_cast<const i32x4*>(Ws(cur, u) + w_chunk_offset(wn * WTN + i * 16 + lrow, quarter));
            int sw[SWN];
#pragma unroll
            for (int w = 0; w < SWN; ++w)
                sw[w] = *reinterpret_cast<const int*>(Ss(cur, u) + ((quarter * WN + wn) * 16 + lrow) * (4 * SWN) + 4 * w);
            i32x8 fx[TJ];
#pragma unroll
            for (int j = 0; j < TJ; ++j) {
                const int row = wm * WTM + j * 16 + lrow;
                const i32x4 lo = *reinterpret_cast<const i32x4*>(Xs(cur, u) + x_chunk_offset(row, quarter));
                const i32x4 hi = *reinterpret_cast<const i32x4*>(Xs(cur, u) + x_chunk_offset(row, 4 + quarter));
                fx[j] = i32x8{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
            }
            if (u == 0) {
                store_tile(cur ^ 1);
                __builtin_amdgcn_sched_barrier(0);
                load_tile(s + 2);
                __builtin_amdgcn_sched_barrier(0);
            }
#pragma unroll
            for (int j = 0; j < TJ; ++j) {
                acc[0][j] = mfma_w4a8<0>(fw[0], fx[j], acc[0][j], sw[0]);
                if constexpr (TI > 1) acc[1][j] = mfma_w4a8<1>(fw[1], fx[j], acc[1][j], sw[0]);
                if constexpr (TI > 2) acc[2][j] = mfma_w4a8<2>(fw[2], fx[j], acc[2][j], sw[0]);
                if constexpr (TI > 3) acc[3][j] = mfma_w4a8<3>(fw[3], fx[j], acc[3][j], sw[0]);
                if constexpr (TI > 4) acc[4][j] = mfma_w4a8<0>(fw[4], fx[j], acc[4][j], sw[SWN - 1]);
                if constexpr (TI > 5) acc[5][j] = mfma_w4a8<1>(fw[5], fx[j], acc[5][j], sw[SWN - 1]);
                if constexpr (TI > 6) acc[6][j] = mfma_w4a8<2>(fw[6], fx[j], acc[6][j], sw[SWN - 1]);
                if constexpr (TI > 7) acc[7][j] = mfma_w4a8<3>(fw[7], fx[j], acc[7][j], sw[SWN - 1]);
            }
        }
        __syncthreads();
    }

    // epilogue: lane holds out[m][n .. n + 3] for every (i, j); everything read from global memory is read before
    // the first store (loads and stores share one counter)
    float sam[TJ];
    bool keep[TJ];
#pragma unroll
    for (int j = 0; j < TJ; ++j) {
        const int m = m0 + wm * WTM + j * 16 + lrow;
        keep[j] = m < p.M;
        sam[j] = keep[j] ? p.sa[m] : 0.f;
        if (p.m_indices && keep[j]) keep[j] = p.m_indices[m] == expert;
    }
#pragma unroll
    for (int j = 0; j < TJ; ++j) {
        const int m = m0 + wm * WTM + j * 16 + lrow;
        if (!keep[j]) continue;
#pragma unroll
        for (int i = 0; i < TI; ++i) {
            const int n = n0 + wn * WTN + i * 16 + quarter * 4;
            if (n >= p.N) continue;  // N % 16 == 0: a group of four is inside or outside as a whole
            f32x4 v = acc[i][j];
#pragma unroll
            for (int e = 0; e < 4; ++e) v[e] *= sam[j];
            if (OUT_F32) {
                *reinterpret_cast<f32x4*>(static_cast<float*>(p.out) + (int64_t)m * p.ld_out + n) = v;
            } else {
                *reinterpret_cast<uint2*>(static_cast<uint16_t*>(p.out) + (int64_t)m * p.ld_out + n) =
                    make_uint2(pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3]));
            }
        }
    }
}

// At most 16 tokens (decode): the weight is read once and nothing else matters.  A workgroup owns 16 weight rows,
// its four waves split K (wave w takes K steps w, w + 4, ...) and each requests the codes and scale bytes of
// kGemvDepth of its steps - 16 bytes and one byte per lane and step, straight into MFMA operand registers -
// before the first MFMA.  The few activation rows come from global memory (they stay in L2); rows >= M, and
// chunks beyond K, are zero.  The four partial sums meet in LDS.
constexpr int kGemvDepth = 8;
template <bool OUT_F32>
__global__ __launch_bounds__(256) void gemm_mxfp4_gemv_kernel(const Mx4Args p) {
    __shared__ __attribute__((aligned(16))) float red[3 * 64 * 4];
    const int t = threadIdx.x, lane = t & 63;
    const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
    const int lrow = lane & 15, quarter = lane >> 4;
    const int n0 = blockIdx.x * 16;
    const int KT = (p.K + 127) >> 7;
    const int wrow = n0 + lrow;
    const bool wok = wrow < p.N, xok = lrow < p.M;
    const uint8_t* const wptr = p.w + (int64_t)(wok ? wrow : 0) * p.ld_w + quarter * 16;
    const uint8_t* const sptr = p.ws + (int64_t)(wok ? wrow : 0) * p.ld_ws + quarter;
    const uint8_t* const xptr = p.a + (int64_t)(xok ? lrow : 0) * p.ld_a + quarter * 16;
    const float sam = xok ? p.sa[lrow] : 0.f;  // requested first: nothing at the end waits for memory
    f32x4 acc = f32x4{0.f, 0.f, 0.f, 0.f};
    for (int base = wave; base < KT; base += 4 * kGemvDepth) {
        u32x4 wv[kGemvDepth], xl[kGemvDepth], xh[kGemvDepth];
        uint32_t sc[kGemvDepth];
#pragma unroll
        for (int i = 0; i < kGemvDepth; ++i) {
            const int kt = base + 4 * i;
            const int k = (kt < KT ? kt : 0) << 7;
            // a block of 32 lies inside K as a whole or not at all (K % 32 == 0); what lies outside is read from the
            // start of the row and dropped below
            const bool in_w = kt < KT && k + quarter * 32 < p.K, in_lo = kt < KT && k + quarter * 16 < p.K,
                       in_hi = kt < KT && k + 64 + quarter * 16 < p.K;
            wv[i] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(wptr + (in_w ? (k >> 1) : 0)));
            sc[i] = __builtin_nontemporal_load(sptr + (in_w ? (k >> 5) : 0));
            xl[i] = *reinterpret_cast<const u32x4*>(xptr + (in_lo ? k : 0));
            xh[i] = *reinterpret_cast<const u32x4*>(xptr + (in_hi ? k + 64 : 0));
        }
        __builtin_amdgcn_sched_barrier(0);  // every load of the pass is requested before the first MFMA
#pragma unroll
        for (int i = 0; i < kGemvDepth; ++i) {
            const int kt = base + 4 * i;
            const int k = (kt < KT ? kt : 0) << 7;
            const bool in_w = kt < KT && k + quarter * 32 < p.K, in_lo = kt < KT && k + quarter * 16 < p.K,
                       in_hi = kt < KT && k + 64 + quarter * 16 < p.K;
            i32x4 fw;
            i32x8 fx;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                fw[e] = (int)wv[i][e];                             // any e2m1 code is finite: the zero on the other side suffices
                fx[e] = (in_lo && xok) ? (int)xl[i][e] : 0;
                fx[4 + e] = (in_hi && xok) ? (int)xh[i][e] : 0;
            }
            const int scale = (in_w && wok) ? (int)sc[i] : 127;    // 255 would be NaN
            acc = mfma_w4a8<0>(fw, fx, acc, scale);
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
            f32x4 v;
#pragma unroll
            for (int e = 0; e < 4; ++e) v[e] = acc[e] * sam;
            if (OUT_F32) *reinterpret_cast<f32x4*>(static_cast<float*>(p.out) + (int64_t)m * p.ld_out + n) = v;
            else *reinterpret_cast<uint2*>(static_cast<uint16_t*>(p.out) + (int64_t)m * p.ld_out + n) =
                    make_uint2(pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3]));
        }
    }
}

// The same for at most kGemvLdsRows tokens with the activations in LDS: a workgroup first requests the weights of its
// first pass, then copies the M activation rows (K bytes each, zero beyond K) into LDS, and reads its MFMA
// fragments from there.  Without 64 registers of activations in flight a wave needs half the registers, so that
// every workgroup of a 18944-row weight is resident at once and the whole weight is requested at the start.
constexpr int kGemvLdsRows = 8;
template <bool OUT_F32>
__global__ __launch_bounds__(256) void gemm_mxfp4_gemv_lds_kernel(const Mx4Args p) {
    extern __shared__ __attribute__((aligned(16))) uint8_t xs[];  // [M][KT * 128 + 16]
    __shared__ __attribute__((aligned(16))) float red[3 * 64 * 4];
    const int t = threadIdx.x, lane = t & 63;
    const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
    const int lrow = lane & 15, quarter = lane >> 4;
    const int n0 = blockIdx.x * 16;
    const int KT = (p.K + 127) >> 7;
    const int pitch = KT * 128 + 16;
    const int wrow = n0 + lrow;
    const bool wok = wrow < p.N, xok = lrow < p.M;
    const uint8_t* const wptr = p.w + (int64_t)(wok ? wrow : 0) * p.ld_w + quarter * 16;
    const uint8_t* const sptr = p.ws + (int64_t)(wok ? wrow : 0) * p.ld_ws + quarter;
    const uint8_t* const xrow = xs + (xok ? lrow : 0) * pitch + quarter * 16;
    u32x4 wv[kGemvDepth];
    uint32_t sc[kGemvDepth];
    auto load_pass = [&](int base) {
#pragma unroll
        for (int i = 0; i < kGemvDepth; ++i) {
            const int kt = base + 4 * i;
            const int k = (kt < KT ? kt : 0) << 7;
            const bool in_w = kt < KT && k + quarter * 32 < p.K;
            wv[i] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(wptr + (in_w ? (k >> 1) : 0)));
            sc[i] = __builtin_nontemporal_load(sptr + (in_w ? (k >> 5) : 0));
        }
    };
    load_pass(wave);
    const float sam = xok ? p.sa[lrow] : 0.f;  // requested early: nothing at the end waits for memory
    {
        const int chunks = KT * 8, total = p.M * chunks;
        for (int idx = t; idx < total; idx += 256) {
            const int row = idx / chunks, c = idx - row * chunks;
            u32x4 v = {0u, 0u, 0u, 0u};
            if (c * 16 < p.K) v = *reinterpret_cast<const u32x4*>(p.a + (int64_t)row * p.ld_a + c * 16);
            *reinterpret_cast<u32x4*>(xs + row * pitch + c * 16) = v;
        }
    }
    __syncthreads();
    f32x4 acc = f32x4{0.f, 0.f, 0.f, 0.f};
    for (int base = wave; base < KT; base += 4 * kGemvDepth) {
        if (base != wave) load_pass(base);
#pragma unroll
        for (int i = 0; i < kGemvDepth; ++i) {
            const int kt = base + 4 * i;
            const int k = (kt < KT ? kt : 0) << 7;
            const bool in = kt < KT, in_w = in && k + quarter * 32 < p.K;
            i32x4 fw;
            i32x8 fx;
            const u32x4 lo = *reinterpret_cast<const u32x4*>(xrow + k), hi = *reinterpret_cast<const u32x4*>(xrow + k + 64);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                fw[e] = (int)wv[i][e];
                fx[e] = (in && xok) ? (int)lo[e] : 0;
                fx[4 + e] = (in && xok) ? (int)hi[e] : 0;
            }
            const int scale = (in_w && wok) ? (int)sc[i] : 127;
            acc = mfma_w4a8<0>(fw, fx, acc, scale);
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
            f32x4 v;
#pragma unroll
            for (int e = 0; e < 4; ++e) v[e] = acc[e] * sam;
            if (OUT_F32) *reinterpret_cast<f32x4*>(static_cast<float*>(p.out) + (int64_t)m * p.ld_out + n) = v;
            else *reinterpret_cast<uint2*>(static_cast<uint16_t*>(p.out) + (int64_t)m * p.ld_out + n) =
                    make_uint2(pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3]));
        }
    }
}

// 17..64 tokens: still a weight streamer.  A workgroup of 2 NTL waves owns 16 NTL weight rows; wave (nt, kh) takes the
// 16 rows of n-tile nt and the kh-th half of every chunk of KS K steps.  K is walked in passes of PC
// chunks: at the start of a pass a wave requests all of its weight codes and scale bytes of the pass (16 bytes + 1
// byte per lane and step, straight into MFMA operand registers, 8 steps = 40 registers), then the
// workgroup stages the activations chunk by chunk through two LDS buffers (the activations of 64 tokens are four
// times the bytes of the workgroup's weights per chunk, so they must not be fetched per wave).  The two K halves
// are summed through LDS at the end.
template <int TM, int NTL, int KS, int PC, bool OUT_F32>
__global__ __launch_bounds__(NTL * 128) void gemm_mxfp4_skinny_kernel(const Mx4Args p) {
    constexpr int NW = NTL * 2;                   // waves: NTL n-tiles x 2 K halves
    constexpr int HS = KS / 2;                    // K steps per wave and chunk
    constexpr int XU = KS * TM * 2;               // wave-wide loads that stage one chunk of activations
    constexpr int XI = (XU + NW - 1) / NW;
    constexpr int XSTAGE = KS * TM * 2048;        // bytes of one activation buffer
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    const int t = threadIdx.x, lane = t & 63;
    const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
    const int nt = wave % NTL, kh = wave / NTL;
    const int lrow = lane & 15, quarter = lane >> 4;
    const int n0 = blockIdx.x * (NTL * 16);
    const int KT = (p.K + 127) >> 7;
    const int chunks = (KT + KS - 1) / KS;

    // activation staging: one wave-wide load = 8 rows x 128 bytes of one K step
    const int st_row8 = (lane >> 1) & 7, st_c = ((lane >> 4) << 1) | (lane & 1);
    // through a buffer descriptor that ends with the M-th row: rows beyond M read zero, and the per-lane part of
    // an address (row, K step inside the chunk, 16-byte piece) is computed once
    i32x4 xr[XI];
    uint32_t xoff[XI];
    const int64_t a_left = (int64_t)p.M * p.ld_a;
    const __amdgpu_buffer_rsrc_t rx = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint8_t*>(p.a), 0, a_left < (int64_t)kBeyond ? (int)a_left : (int)kBeyond, 0x00020000);
#pragma unroll
    for (int i = 0; i < XI; ++i) {
        const int unit = wave + NW * i, ks = unit % KS, row = (unit / KS) * 8 + st_row8;
        xoff[i] = (unit < XU && row < p.M) ? (uint32_t)row * (uint32_t)p.ld_a + (ks << 7) + st_c * 16 : kBeyond;
    }
    auto xload = [&](int chunk) {
        const int k0 = (chunk * KS) << 7;
#pragma unroll
        for (int i = 0; i < XI; ++i) {
            const int unit = wave + NW * i, ks = unit % KS;
            const bool ok = k0 + (ks << 7) + st_c * 16 < p.K;     // beyond K: not fetched, zero
            const u32x4 v = __builtin_amdgcn_raw_buffer_load_b128(rx, ok ? xoff[i] : kBeyond, k0, 0);
            xr[i] = i32x4{(int)v[0], (int)v[1], (int)v[2], (int)v[3]};
        }
    };
    auto xstore = [&](int buf) {
#pragma unroll
        for (int i = 0; i < XI; ++i) {
            const int unit = wave + NW * i, ks = unit % KS, row = (unit / KS) * 8 + st_row8;
            if (XU % NW == 0 || unit < XU)
                *reinterpret_cast<i32x4*>(smem + buf * XSTAGE + (ks * TM + (row >> 4)) * 2048 + x_chunk_offset(row & 15, st_c)) = xr[i];
        }
    };
    // Weight codes and scale bytes come through buffer descriptors that end with the matrix: a load costs one
    // scalar offset (the K step is uniform for the wave) on top of a per-lane row offset.  Rows beyond N and blocks
    // beyond K are not fetched at all: their lane offset is kBeyond, past the end of any descriptor here (a
    // workgroup's rows span less than 2^31 bytes and a scalar offset is below 2^24, so the sum neither wraps nor
    // comes back into range), and such a load returns zero.
    const int wrow = n0 + nt * 16 + lrow;
    const bool wok = wrow < p.N;  // rows beyond N lie past the descriptors' end by themselves
    const int64_t w_left = (int64_t)(p.N - n0) * p.ld_w, s_left = (int64_t)(p.N - n0) * p.ld_ws;
    const __amdgpu_buffer_rsrc_t rw = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint8_t*>(p.w) + (int64_t)n0 * p.ld_w, 0, w_left < (int64_t)kBeyond ? (int)w_left : (int)kBeyond, 0x00020000);
    const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint8_t*>(p.ws) + (int64_t)n0 * p.ld_ws, 0, s_left < (int64_t)kBeyond ? (int)s_left : (int)kBeyond, 0x00020000);
    const uint32_t w_lane = (uint32_t)(nt * 16 + lrow) * (uint32_t)p.ld_w + quarter * 16;
    const uint32_t s_lane = (uint32_t)(nt * 16 + lrow) * (uint32_t)p.ld_ws + quarter;

    f32x4 acc[TM];
#pragma unroll
    for (int j = 0; j < TM; ++j) acc[j] = f32x4{0.f, 0.f, 0.f, 0.f};

    xload(0);
    for (int c0 = 0; c0 < chunks; c0 += PC) {
        // this wave's weights of the pass: chunk c0 + cc, steps kh * HS + h
        u32x4 wv[PC][HS];
        uint32_t sc[PC][HS];
#pragma unroll
        for (int cc = 0; cc < PC; ++cc)
#pragma unroll
            for (int h = 0; h < HS; ++h) {
                const int k = ((c0 + cc) * KS + kh * HS + h) << 7;
                const bool in_w = k + quarter * 32 < p.K;
                wv[cc][h] = __builtin_amdgcn_raw_buffer_load_b128(rw, in_w ? w_lane : kBeyond, k >> 1, 2);
                sc[cc][h] = __builtin_amdgcn_raw_buffer_load_b8(rs, in_w ? s_lane : kBeyond, k >> 5, 2);
            }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int cc = 0; cc < PC; ++cc) {
            const int c = c0 + cc;
            // the buffer of chunk c was last read during chunk c - 2, two barriers ago
            xstore(c & 1);
            __builtin_amdgcn_sched_barrier(0);
            xload(c + 1);           // chunks past the end load zeros
            __builtin_amdgcn_sched_barrier(0);
            __syncthreads();
#pragma unroll
            for (int h = 0; h < HS; ++h) {
                const int ks = kh * HS + h;
                const int k = (c * KS + ks) << 7;
                const bool in_w = k + quarter * 32 < p.K;
                const int scale = (in_w && wok) ? (int)sc[cc][h] : 127;  // 255 would be NaN; beyond K the activations are zero
                i32x4 fw;
#pragma unroll
                for (int e = 0; e < 4; ++e) fw[e] = (int)wv[cc][h][e];
#pragma unroll
                for (int j = 0; j < TM; ++j) {
                    const uint8_t* const xt = smem + (c & 1) * XSTAGE + (ks * TM + j) * 2048;
                    const i32x4 lo = *reinterpret_cast<const i32x4*>(xt + x_chunk_offset(lrow, quarter));
                    const i32x4 hi = *reinterpret_cast<const i32x4*>(xt + x_chunk_offset(lrow, 4 + quarter));
                    const i32x8 fx = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
                    acc[j] = mfma_w4a8<0>(fw, fx, acc[j], scale);
                }
                __builtin_amdgcn_sched_barrier(0);  // fragments of one K step at a time; nothing of the next chunk moves up
            }
            // the MFMAs are pure functions of registers: without a use here the compiler sinks all of a pass behind its
            // last barrier and keeps every fragment of the pass alive until then
#pragma unroll
            for (int j = 0; j < TM; ++j) asm volatile("" : "+v"(acc[j]));
        }
    }

    // sum the two K halves through LDS (both buffers may still be read by a slower wave: barrier first)
    __syncthreads();
    float* red = reinterpret_cast<float*>(smem);
    if (kh == 1) {
#pragma unroll
        for (int j = 0; j < TM; ++j) *reinterpret_cast<f32x4*>(red + ((nt * TM + j) * 64 + lane) * 4) = acc[j];
    }
    __syncthreads();
    if (kh == 0) {
        const int n = n0 + nt * 16 + quarter * 4;
        if (n < p.N) {
#pragma unroll
            for (int j = 0; j < TM; ++j) {
                const int m = j * 16 + lrow;
                if (m >= p.M) continue;
                const f32x4 o = *reinterpret_cast<const f32x4*>(red + ((nt * TM + j) * 64 + lane) * 4);
                const float sam = p.sa[m];
                f32x4 v;
#pragma unroll
                for (int e = 0; e < 4; ++e) v[e] = (acc[j][e] + o[e]) * sam;
                if (OUT_F32) *reinterpret_cast<f32x4*>(static_cast<float*>(p.out) + (int64_t)m * p.ld_out + n) = v;
                else *reinterpret_cast<uint2*>(static_cast<uint16_t*>(p.out) + (int64_t)m * p.ld_out + n) =
                        make_uint2(pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3]));
            }
        }
    }
}

// ---------------------------------------------------------------------------
// Large full tiles: 256 x 256 x 128 per workgroup, four wavefronts (one per SIMD, 2 x 2), each owning a 128 x 128
// block = 64 accumulators of 16 x 16.  Operands go from global memory straight into LDS (buffer_load ... lds: no
// staging registers, no LDS store instructions; the LDS layout is dictated by which bytes each lane asks for):
//   activations  two stages of 32 KiB, row-major, the 16-byte chunk c of row r at position c ^ ((r >> 1) & 7);
//   weights      three stages of 16 KiB, row r at r * 64, chunk c (0..3) at position c ^ ((r >> 2) & 3): a fragment
//                read (16 rows, one chunk) covers all 64 banks once;
//   scale bytes  three stages of 1 KiB: the four scale bytes of a row and K step are one 32-bit word, stored so
//                that a lane finds the words of its eight 16-row tiles next to each other (word index
//                wn * 128 + lrow * 8 + tile) and picks its quarter's byte with a shift.
// The K step is a software pipeline of 32 groups of two MFMAs, each preceded by at most one direct-to-LDS load
// and one fragment read; step kt computes from activation stage kt % 2 and weight / scale stage kt % 3:
//   S0 (w0,x0): LDS reads x1            S1 (w0,x1): LDS reads w1
//   -- wait for all but the five newest loads and for own LDS reads, barrier --
//   S2 (w1,x0): LDS reads next w0 and its scales + loads of activation tile kt + 2
//   S3 (w1,x1): LDS reads next x0 + loads of weight and scale tile kt + 3 (the five newest at the next barrier)
// Requires M % 256 == 0, N % 256 == 0, K % 128 == 0 and 4-byte aligned scale rows.
// ---------------------------------------------------------------------------
#define MX4_PHASE_END() __builtin_amdgcn_sched_barrier(0)
// written out as instructions: in front of a barrier it knows of, the compiler waits for every load it has issued,
// including the direct-to-LDS loads that are meant to stay in flight across the barrier
#define MX4_WAIT_BARRIER(vm) asm volatile("s_waitcnt vmcnt(" #vm ") lgkmcnt(0)\n\ts_barrier" ::: "memory")
#define MX4_MMA2(wh, xb, xh, g)                                                                              \
    {                                                                                                        \
        _Pragma("unroll") for (int e = 0; e < 2; ++e) {                                                      \
            const int j = (g) >> 1, i = ((g)&1) * 2 + e;                                                     \
            acc[(wh)*4 + i][(xh)*4 + j] =                                                                    \
                mfma_w4a8<0>(W[wh][i], X[xb][j], acc[(wh)*4 + i][(xh)*4 + j], (int)S[(wh)*4 + i]);          \
        }                                                                                                    \
    }

template <bool OUT_F32>
__global__ __launch_bounds__(256) void gemm_mxfp4_256_kernel(const Mx4Args p) {
    constexpr int BM = 256, BN = 256;
    constexpr int XS = BM * 128, WS = BN * 64, SS = BN * 4;
    constexpr int WBASE = 2 * XS, SBASE = WBASE + 3 * WS, ABASE = SBASE + 3 * SS;  // + 1 KiB of activation scales
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    int tm, tn;
    mx4_tile_of_block<8>(blockIdx.x, p.tiles_m, p.tiles_n, tm, tn);
    const int m0 = tm * BM, n0 = tn * BN;
    const int t = threadIdx.x, lane = t & 63;
    const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
    const int wm = wave & 1, wn = wave >> 1;
    const int lrow = lane & 15, quarter = lane >> 4;
    const int KT = p.K >> 7;
    const int last = KT - 1;

    // Wave-uniform bases pass through an empty asm so that they stay in SGPRs for the whole K loop (a scalar load
    // inside the loop would have to be waited for with lgkmcnt(0), which drains the fragment reads in flight).
    uint64_t a_wave = reinterpret_cast<uint64_t>(p.a) + ((uint64_t)m0 + (uint64_t)wave * 8) * (uint64_t)p.ld_a;
    uint64_t w_wave = reinterpret_cast<uint64_t>(p.w) + ((uint64_t)n0 + (uint64_t)wave * 16) * (uint64_t)p.ld_w;
    uint64_t s_tile = reinterpret_cast<uint64_t>(p.ws) + (uint64_t)n0 * (uint64_t)p.ld_ws;
    uint32_t a_step = 32u * (uint32_t)p.ld_a, w_step = 64u * (uint32_t)p.ld_w;  // pitches are < 2^24
    asm volatile("" : "+s"(a_wave), "+s"(w_wave), "+s"(s_tile), "+s"(a_step), "+s"(w_step));
    // activations: load i covers rows (wave + 4 i) * 8 .. + 7; (r >> 1) & 7 of row r = (wave + 4 i) * 8 + (lane >> 3)
    // is (wave & 1) * 4 + (lane >> 4)
    const uint32_t va_lane = (uint32_t)(lane >> 3) * (uint32_t)p.ld_a + (uint32_t)(((lane & 7) ^ ((wave & 1) * 4 + (lane >> 4))) << 4);
    // weights: load i covers rows (wave + 4 i) * 16 .. + 15; lane (row16, position) fetches chunk position ^ (row16 >> 2)
    const uint32_t vw_lane = (uint32_t)(lane >> 2) * (uint32_t)p.ld_w + (uint32_t)(((lane & 3) ^ ((lane >> 4) & 3)) << 4);
    // scale words: word wave * 64 + lane = wn' * 128 + lrow' * 8 + tile' belongs to row wn' * 128 + tile' * 16 + lrow'
    const int sword = wave * 64 + lane;
    const uint32_t vs_lane = (uint32_t)((sword >> 7) * 128 + (sword & 7) * 16 + ((sword >> 3) & 15)) * (uint32_t)p.ld_ws;
    typedef __attribute__((address_space(1))) const void gbl_void;
    typedef __attribute__((address_space(3))) void lds_void;
    const __amdgpu_buffer_rsrc_t ra = __builtin_amdgcn_make_buffer_rsrc(reinterpret_cast<void*>(a_wave), 0, 0xFFFFFFFF, 0x00020000);
    const __amdgpu_buffer_rsrc_t rw = __builtin_amdgcn_make_buffer_rsrc(reinterpret_cast<void*>(w_wave), 0, 0xFFFFFFFF, 0x00020000);
    const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc(reinterpret_cast<void*>(s_tile), 0, 0xFFFFFFFF, 0x00020000);
    auto dma_x = [&](int kt, int stage, int i) {
        __builtin_amdgcn_raw_ptr_buffer_load_lds(ra, (lds_void*)(smem + stage * XS + (wave + 4 * i) * 1024), 16, va_lane,
                                                 (uint32_t)i * a_step + ((uint32_t)kt << 7), 0, 0);
    };
    auto dma_w = [&](int kt, int stage, int i) {
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rw, (lds_void*)(smem + WBASE + stage * WS + (wave + 4 * i) * 1024), 16, vw_lane,
                                                 (uint32_t)i * w_step + ((uint32_t)kt << 6), 0, 0);
    };
    auto dma_s = [&](int kt, int stage) {
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, (lds_void*)(smem + SBASE + stage * SS + wave * 256), 4, vs_lane,
                                                 (uint32_t)kt << 2, 0, 0);
    };

    f32x4 acc[8][8];  // [n tile][m tile]
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int j = 0; j < 8; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};

    // activation fragment: the e4m3 operand's registers 0-3 are k = 16 q .. + 15, registers 4-7 k = 64 + 16 q .. + 15
    const int fsw = (lrow >> 1) & 7;
    const int x_off = (wm * 128 + lrow) * 128 + ((quarter ^ fsw) << 4);
    const int x_off2 = (wm * 128 + lrow) * 128 + (((4 + quarter) ^ fsw) << 4);
    const int w_off = WBASE + (wn * 128 + lrow) * 64 + ((quarter ^ ((lrow >> 2) & 3)) << 4);
    const int s_off = SBASE + (wn * 128 + lrow * 8) * 4;
    const unsigned sshift = 8u * (unsigned)quarter;
    auto xfrag = [&](int stage_bytes, int tile16) {
        const uint8_t* base = smem + stage_bytes + tile16 * 2048;
        const i32x4 lo = *reinterpret_cast<const i32x4*>(base + x_off);
        const i32x4 hi = *reinterpret_cast<const i32x4*>(base + x_off2);
        return i32x8{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    };
    auto wfrag = [&](int stage, int tile16) { return *reinterpret_cast<const i32x4*>(smem + stage * WS + tile16 * 1024 + w_off); };
    auto sfrag = [&](int stage, int half) { return *reinterpret_cast<const u32x4*>(smem + stage * SS + s_off + half * 16); };
    i32x4 W[2][4];
    i32x8 X[2][4];
    uint32_t S[8];  // this lane's scale byte of the wave's eight weight tiles, in the low byte
    u32x4 sraw, sraw_hi;  // scale words of tiles 0-3 / 4-7 of the next K step

    // prologue: the tile's 256 activation scales for the epilogue (64 per wave, 4 bytes per lane, a region of their
    // own), then activation tiles 0, 1 and weight + scale tiles 0, 1, 2 into their stages
    __builtin_amdgcn_global_load_lds((gbl_void*)(p.sa + m0 + wave * 64 + lane), (lds_void*)(smem + ABASE + wave * 256), 4, 0, 0);
#pragma unroll
    for (int i = 0; i < 8; ++i) dma_x(0, 0, i);
#pragma unroll
    for (int i = 0; i < 4; ++i) dma_w(0, 0, i);
    dma_s(0, 0);
#pragma unroll
    for (int i = 0; i < 8; ++i) dma_x(1 < last ? 1 : last, 1, i);
#pragma unroll
    for (int i = 0; i < 4; ++i) dma_w(1 < last ? 1 : last, 1, i);
    dma_s(1 < last ? 1 : last, 1);
#pragma unroll
    for (int i = 0; i < 4; ++i) dma_w(2 < last ? 2 : last, 2, i);
    dma_s(2 < last ? 2 : last, 2);
    MX4_WAIT_BARRIER(18);  // the scales and tile 0 (14 loads) have landed; the other 18 stay in flight
#pragma unroll
    for (int g = 0; g < 4; ++g) {
        W[0][g] = wfrag(0, g);
        X[0][g] = xfrag(0, g);
    }
    sraw = sfrag(0, 0);
    sraw_hi = sfrag(0, 1);
    asm volatile("" : "+v"(sraw), "+v"(sraw_hi));  // two 16-byte reads, not eight of four bytes
#pragma unroll
    for (int g = 0; g < 4; ++g) S[g] = sraw[g] >> sshift;
    MX4_PHASE_END();

    int ws_cur = 0;  // kt % 3
    for (int kt = 0; kt < KT; ++kt) {
        const int xs_cur = (kt & 1) * XS, xs_nxt = xs_cur ^ XS;
        const int ws_nxt = ws_cur == 2 ? 0 : ws_cur + 1;
        // past the end: the last tile again, into a stage nobody reads any more (no branch in the K loop)
        const int kw = kt + 3 < last ? kt + 3 : last, kx = kt + 2 < last ? kt + 2 : last;
#pragma unroll
        for (int g = 0; g < 8; ++g) {
            if (g < 4) X[1][g] = xfrag(xs_cur, 4 + g);
            MX4_MMA2(0, 0, 0, g);
            MX4_PHASE_END();
        }
#pragma unroll
        for (int g = 0; g < 8; ++g) {
            if (g < 4) W[1][g] = wfrag(ws_cur, 4 + g);
            if (g >= 4) S[g] = sraw_hi[g - 4] >> sshift;
            MX4_MMA2(0, 1, 1, g);
            MX4_PHASE_END();
        }
        MX4_WAIT_BARRIER(5);
        MX4_PHASE_END();
#pragma unroll
        for (int g = 0; g < 8; ++g) {
            if (g < 4) W[0][g] = wfrag(ws_nxt, g);  // after the last step: stale data, unused
            if (g == 4) {
                sraw = sfrag(ws_nxt, 0);
                asm volatile("" : "+v"(sraw));
            }
            if (g == 5) {
                sraw_hi = sfrag(ws_nxt, 1);  // S[4..7] are still in use: shifted into place in S1 of the next step
                asm volatile("" : "+v"(sraw_hi));
            }
            dma_x(kx, kt & 1, g);
            MX4_MMA2(1, 0, 0, g);
            MX4_PHASE_END();
        }
#pragma unroll
        for (int g = 0; g < 8; ++g) {
            if (g < 4) X[0][g] = xfrag(xs_nxt, g);
            if (g < 4) dma_w(kw, ws_cur, g);
            if (g == 4) dma_s(kw, ws_cur);
            if (g >= 4) S[g - 4] = sraw[g - 4] >> sshift;
            MX4_MMA2(1, 1, 1, g);
            MX4_PHASE_END();
        }
        ws_cur = ws_nxt;
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the scales have landed, and nothing may still land in the stages
    __syncthreads();
    const float* const sa_lds = reinterpret_cast<const float*>(smem + ABASE);

    float sam[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) sam[j] = sa_lds[wm * 128 + j * 16 + lrow];
    if (OUT_F32) {
        // a lane already owns 16 contiguous bytes: store directly
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int n = n0 + wn * 128 + i * 16 + quarter * 4;
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const int m = m0 + wm * 128 + j * 16 + lrow;
                f32x4 v = acc[i][j];
#pragma unroll
                for (int e = 0; e < 4; ++e) v[e] = v[e] * sam[j];
                __builtin_nontemporal_store(v, reinterpret_cast<f32x4*>(static_cast<float*>(p.out) + (int64_t)m * p.ld_out + n));
            }
        }
        return;
    }
    // bf16: scale, convert, turn the wave's 128 x 128 block through LDS in two halves of 64 rows
    // (row stride 272 B keeps the 8-byte stores of 16 rows on different banks)
    __syncthreads();  // all waves are done reading the operand stages
    constexpr int EST = 272;
    static_assert(4 * 64 * EST <= ABASE, "the epilogue buffers must not reach the activation scales");
    uint8_t* const ebuf = smem + wave * (64 * EST);
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
                for (int e = 0; e < 4; ++e) v[e] = v[e] * sam[j];
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
// The same pipeline on 128 x 256 tiles for every shape the kernel above does not take - any M, N % 16 == 0,
// K % 32 == 0 - and for the grouped layout (an expert's rows start on multiples of 128): four waves, 2 x 2, each a
// 64 x 128 block = 32 accumulators; two activation stages of 16 KiB, three weight stages of 16 KiB, three scale
// stages of 1 KiB; a K step is four phases of four groups of two MFMAs.  Per wave and step 4 activation + 4 weight
// + 1 scale load; the barrier lets the five newest pass.
// Edges cost nothing in the K loop: a direct-to-LDS buffer load writes zero for a lane whose offset lies beyond its
// descriptor (the scalar offset counts), so the descriptors end with the last row of their matrix (rows beyond M
// and N arrive as zeros) and, in the last K step of a K that is not a multiple of 128, the lanes whose 16 bytes lie
// beyond K ask for an offset beyond every descriptor.  The scale word of that step is read so that it ends with
// the row (a word that straddles the end of the last row would be refused as a whole), its bytes shifted
// accordingly, and the quarters beyond K take the scale byte 127.
// ---------------------------------------------------------------------------
#define MX4_MMA2N(wh, xb, xh, g)                                                                             \
    {                                                                                                        \
        _Pragma("unroll") for (int e = 0; e < 2; ++e) {                                                      \
            const int j = (g) >> 1, i = ((g)&1) * 2 + e;                                                     \
            acc[(wh)*4 + i][(xh)*2 + j] =                                                                    \
                mfma_w4a8<0>(W[wh][i], X[xb][j], acc[(wh)*4 + i][(xh)*2 + j], (int)S[(wh)*4 + i]);          \
        }                                                                                                    \
    }

template <bool OUT_F32>
__global__ __launch_bounds__(256) void gemm_mxfp4_128_kernel(const Mx4Args p) {
    constexpr int BM = 128, BN = 256;
    constexpr int XS = BM * 128, WS = BN * 64, SS = BN * 4;
    constexpr int WBASE = 2 * XS, SBASE = WBASE + 3 * WS, ABASE = SBASE + 3 * SS;  // + 512 bytes of activation scales
    constexpr uint32_t kEnd = 0xEFFFFFFFu;  // the longest descriptor: kBeyond stays beyond it
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    int tm, tn;
    if (p.m_indices) mx4_tile_of_block<4>(blockIdx.x, p.tiles_m, p.tiles_n, tm, tn);
    else mx4_tile_of_block<8>(blockIdx.x, p.tiles_m, p.tiles_n, tm, tn);
    const int m0 = tm * BM, n0 = tn * BN;
    const uint8_t* wmat = p.w;
    const uint8_t* smat = p.ws;
    int expert = 0;
    if (p.m_indices) {
        expert = p.m_indices[m0];  // groups start on multiples of 128 rows
        if (expert < 0) return;    // a tile of padding (uniform for the workgroup)
        wmat += (int64_t)expert * p.N * p.ld_w;
        smat += (int64_t)expert * p.N * p.ld_ws;
    }
    const int t = threadIdx.x, lane = t & 63;
    const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
    const int wm = wave & 1, wn = wave >> 1;
    const int lrow = lane & 15, quarter = lane >> 4;
    const int KT = (p.K + 127) >> 7;
    const int last = KT - 1;
    const int k_tail = p.K - (last << 7);            // 32 .. 128 elements in the last step
    const int vq = k_tail >> 5;                      // its valid quarters, 1 .. 4

    uint64_t a_wave = reinterpret_cast<uint64_t>(p.a) + ((uint64_t)m0 + (uint64_t)wave * 8) * (uint64_t)p.ld_a;
    uint64_t w_wave = reinterpret_cast<uint64_t>(wmat) + ((uint64_t)n0 + (uint64_t)wave * 16) * (uint64_t)p.ld_w;
    uint64_t s_tile = reinterpret_cast<uint64_t>(smat) + (uint64_t)n0 * (uint64_t)p.ld_ws;
    uint32_t a_step = 32u * (uint32_t)p.ld_a, w_step = 64u * (uint32_t)p.ld_w;  // pitches are < 2^24
    // bytes from a descriptor's base to the end of its matrix (none if the wave's first row is already outside)
    const int64_t a_rows = (int64_t)p.M - m0 - wave * 8, w_rows = (int64_t)p.N - n0 - wave * 16, s_rows = (int64_t)p.N - n0;
    const int64_t a_left = a_rows > 0 ? a_rows * p.ld_a : 0, w_left = w_rows > 0 ? w_rows * p.ld_w : 0, s_left = s_rows > 0 ? s_rows * p.ld_ws : 0;
    uint32_t a_end = a_left < (int64_t)kEnd ? (uint32_t)a_left : kEnd, w_end = w_left < (int64_t)kEnd ? (uint32_t)w_left : kEnd,
             s_end = s_left < (int64_t)kEnd ? (uint32_t)s_left : kEnd;
    asm volatile("" : "+s"(a_wave), "+s"(w_wave), "+s"(s_tile), "+s"(a_step), "+s"(w_step), "+s"(a_end), "+s"(w_end), "+s"(s_end));
    // activations: load i covers rows (wave + 4 i) * 8 .. + 7; lane (row8, position) fetches chunk position ^ ((r >> 1) & 7)
    const int xc = (lane & 7) ^ ((wave & 1) * 4 + (lane >> 4));
    const uint32_t va_lane = (uint32_t)(lane >> 3) * (uint32_t)p.ld_a + (uint32_t)(xc << 4);
    const uint32_t va_tail = xc * 16 < k_tail ? va_lane : kBeyond;
    // weights: load i covers rows (wave + 4 i) * 16 .. + 15; lane (row16, position) fetches chunk position ^ (row16 >> 2)
    const int wc = (lane & 3) ^ ((lane >> 4) & 3);
    const uint32_t vw_lane = (uint32_t)(lane >> 2) * (uint32_t)p.ld_w + (uint32_t)(wc << 4);
    const uint32_t vw_tail = wc * 32 < k_tail ? vw_lane : kBeyond;
    // scale words: word wave * 64 + lane = wn' * 128 + lrow' * 8 + tile' belongs to row wn' * 128 + tile' * 16 + lrow'
    const int sword = wave * 64 + lane;
    const uint32_t vs_lane = (uint32_t)((sword >> 7) * 128 + (sword & 7) * 16 + ((sword >> 3) & 15)) * (uint32_t)p.ld_ws;
    const uint32_t s_last = (uint32_t)(last * 4 - (4 - vq));  // the last step's word ends with the row (K >= 128)
    const unsigned sshift = 8u * (unsigned)quarter, sshift_tail = 8u * (unsigned)(quarter + 4 - vq);
    const bool q_in_tail = quarter < vq;
    typedef __attribute__((address_space(1))) const void gbl_void;
    typedef __attribute__((address_space(3))) void lds_void;
    const __amdgpu_buffer_rsrc_t ra = __builtin_amdgcn_make_buffer_rsrc(reinterpret_cast<void*>(a_wave), 0, (int)a_end, 0x00020000);
    const __amdgpu_buffer_rsrc_t rw = __builtin_amdgcn_make_buffer_rsrc(reinterpret_cast<void*>(w_wave), 0, (int)w_end, 0x00020000);
    const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc(reinterpret_cast<void*>(s_tile), 0, (int)s_end, 0x00020000);
    auto dma_x = [&](int kt, int stage, int i) {
        __builtin_amdgcn_raw_ptr_buffer_load_lds(ra, (lds_void*)(smem + stage * XS + (wave + 4 * i) * 1024), 16, kt == last ? va_tail : va_lane,
                                                 (uint32_t)i * a_step + ((uint32_t)kt << 7), 0, 0);
    };
    auto dma_w = [&](int kt, int stage, int i) {
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rw, (lds_void*)(smem + WBASE + stage * WS + (wave + 4 * i) * 1024), 16, kt == last ? vw_tail : vw_lane,
                                                 (uint32_t)i * w_step + ((uint32_t)kt << 6), 0, 0);
    };
    auto dma_s = [&](int kt, int stage) {
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, (lds_void*)(smem + SBASE + stage * SS + wave * 256), 4, vs_lane,
                                                 kt == last ? s_last : (uint32_t)kt << 2, 0, 0);
    };

    f32x4 acc[8][4];  // [n tile][m tile]
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};

    const int fsw = (lrow >> 1) & 7;
    const int x_off = (wm * 64 + lrow) * 128 + ((quarter ^ fsw) << 4);
    const int x_off2 = (wm * 64 + lrow) * 128 + (((4 + quarter) ^ fsw) << 4);
    const int w_off = WBASE + (wn * 128 + lrow) * 64 + ((quarter ^ ((lrow >> 2) & 3)) << 4);
    const int s_off = SBASE + (wn * 128 + lrow * 8) * 4;
    auto xfrag = [&](int stage_bytes, int tile16) {
        const uint8_t* base = smem + stage_bytes + tile16 * 2048;
        const i32x4 lo = *reinterpret_cast<const i32x4*>(base + x_off);
        const i32x4 hi = *reinterpret_cast<const i32x4*>(base + x_off2);
        return i32x8{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    };
    auto wfrag = [&](int stage, int tile16) { return *reinterpret_cast<const i32x4*>(smem + stage * WS + tile16 * 1024 + w_off); };
    auto sfrag = [&](int stage, int half) { return *reinterpret_cast<const u32x4*>(smem + stage * SS + s_off + half * 16); };
    // this lane's scale byte of a word of K step kt
    auto sbyte = [&](uint32_t word, int kt) -> uint32_t {
        const bool tail = kt == last;
        const uint32_t b = word >> (tail ? sshift_tail : sshift);
        return (tail && !q_in_tail) ? 127u : b;
    };
    i32x4 W[2][4];
    i32x8 X[2][2];
    uint32_t S[8];
    u32x4 sraw, sraw_hi;

    // prologue: the tile's 128 activation scales (64 per wave of the first two; rows beyond M repeat the last one), then
    // activation tiles 0, 1 and weight + scale tiles 0, 1, 2
    {
        const int m = m0 + (wave & 1) * 64 + lane;
        __builtin_amdgcn_global_load_lds((gbl_void*)(p.sa + (m < p.M ? m : p.M - 1)), (lds_void*)(smem + ABASE + (wave & 1) * 256), 4, 0, 0);
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) dma_x(0, 0, i);
#pragma unroll
    for (int i = 0; i < 4; ++i) dma_w(0, 0, i);
    dma_s(0, 0);
#pragma unroll
    for (int i = 0; i < 4; ++i) dma_x(1 < last ? 1 : last, 1, i);
#pragma unroll
    for (int i = 0; i < 4; ++i) dma_w(1 < last ? 1 : last, 1, i);
    dma_s(1 < last ? 1 : last, 1);
#pragma unroll
    for (int i = 0; i < 4; ++i) dma_w(2 < last ? 2 : last, 2, i);
    dma_s(2 < last ? 2 : last, 2);
    MX4_WAIT_BARRIER(14);  // the scales and tile 0 (10 loads) have landed; the other 14 stay in flight
#pragma unroll
    for (int g = 0; g < 4; ++g) W[0][g] = wfrag(0, g);
#pragma unroll
    for (int g = 0; g < 2; ++g) X[0][g] = xfrag(0, g);
    sraw = sfrag(0, 0);
    sraw_hi = sfrag(0, 1);
    asm volatile("" : "+v"(sraw), "+v"(sraw_hi));  // two 16-byte reads, not eight of four bytes
#pragma unroll
    for (int g = 0; g < 4; ++g) S[g] = sbyte(sraw[g], 0);
    MX4_PHASE_END();

    int ws_cur = 0;  // kt % 3
    for (int kt = 0; kt < KT; ++kt) {
        const int xs_cur = (kt & 1) * XS, xs_nxt = xs_cur ^ XS;
        const int ws_nxt = ws_cur == 2 ? 0 : ws_cur + 1;
        // past the end: the last tile again, into a stage nobody reads any more (no branch in the K loop)
        const int kw = kt + 3 < last ? kt + 3 : last, kx = kt + 2 < last ? kt + 2 : last;
#pragma unroll
        for (int g = 0; g < 4; ++g) {  // S0 (w0, x0): reads x1
            if (g < 2) X[1][g] = xfrag(xs_cur, 2 + g);
            MX4_MMA2N(0, 0, 0, g);
            MX4_PHASE_END();
        }
#pragma unroll
        for (int g = 0; g < 4; ++g) {  // S1 (w0, x1): reads w1, scale bytes of w1
            W[1][g] = wfrag(ws_cur, 4 + g);
            S[4 + g] = sbyte(sraw_hi[g], kt);
            MX4_MMA2N(0, 1, 1, g);
            MX4_PHASE_END();
        }
        MX4_WAIT_BARRIER(5);
        MX4_PHASE_END();
#pragma unroll
        for (int g = 0; g < 4; ++g) {  // S2 (w1, x0): reads next w0 and both scale words; loads of activation tile kt + 2
            W[0][g] = wfrag(ws_nxt, g);  // after the last step: stale data, unused
            if (g == 2) {
                sraw = sfrag(ws_nxt, 0);
                asm volatile("" : "+v"(sraw));
            }
            if (g == 3) {
                sraw_hi = sfrag(ws_nxt, 1);  // S[4..7] are still in use: shifted into place in S1 of the next step
                asm volatile("" : "+v"(sraw_hi));
            }
            dma_x(kx, kt & 1, g);
            MX4_MMA2N(1, 0, 0, g);
            MX4_PHASE_END();
        }
#pragma unroll
        for (int g = 0; g < 4; ++g) {  // S3 (w1, x1): reads next x0; loads of weight and scale tile kt + 3
            if (g < 2) X[0][g] = xfrag(xs_nxt, g);
            dma_w(kw, ws_cur, g);
            if (g == 3) dma_s(kw, ws_cur);
            S[g] = sbyte(sraw[g], kt + 1);
            MX4_MMA2N(1, 1, 1, g);
            MX4_PHASE_END();
        }
        ws_cur = ws_nxt;
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the scales have landed, and nothing may still land in the stages
    __syncthreads();
    const float* const sa_lds = reinterpret_cast<const float*>(smem + ABASE);

    float sam[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) sam[j] = sa_lds[wm * 64 + j * 16 + lrow];
    if (OUT_F32) {
        // a lane already owns 16 contiguous bytes: store directly; everything read from memory is read first
        bool keep[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int m = m0 + wm * 64 + j * 16 + lrow;
            keep[j] = m < p.M;
            if (p.m_indices && keep[j]) keep[j] = p.m_indices[m] == expert;
        }
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int n = n0 + wn * 128 + i * 16 + quarter * 4;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int m = m0 + wm * 64 + j * 16 + lrow;
                f32x4 v = acc[i][j];
#pragma unroll
                for (int e = 0; e < 4; ++e) v[e] = v[e] * sam[j];
                if (keep[j] && n < p.N)
                    __builtin_nontemporal_store(v, reinterpret_cast<f32x4*>(static_cast<float*>(p.out) + (int64_t)m * p.ld_out + n));
            }
        }
        return;
    }
    // bf16: scale, convert, turn the wave's 64 x 128 block through LDS (row stride 272 B keeps the 8-byte stores of 16
    // rows on different banks) so that a global store is 16 bytes per lane and 256 contiguous bytes per output row
    constexpr int EST = 272;
    static_assert(4 * 64 * EST <= ABASE, "the epilogue buffers must not reach the activation scales");
    const int rd_row = lane >> 4, rd_chunk = lane & 15;
    bool keep[16];
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        const int m = m0 + wm * 64 + r * 4 + rd_row;
        keep[r] = m < p.M && n0 + wn * 128 + rd_chunk * 8 < p.N;  // N % 16 == 0: a chunk of 8 is inside or outside as a whole
        if (p.m_indices && keep[r]) keep[r] = p.m_indices[m] == expert;
    }
    __syncthreads();  // all waves are done reading the operand stages
    uint8_t* const ebuf = smem + wave * (64 * EST);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            f32x4 v = acc[i][j];
#pragma unroll
            for (int e = 0; e < 4; ++e) v[e] = v[e] * sam[j];
            *reinterpret_cast<uint2*>(ebuf + (j * 16 + lrow) * EST + (i * 16 + quarter * 4) * 2) =
                make_uint2(pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3]));
        }
    }
    // written and read by the same wave: LDS operations of one wave complete in order
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        const int row = r * 4 + rd_row;
        const i32x4 d = *reinterpret_cast<const i32x4*>(ebuf + row * EST + rd_chunk * 16);
        const int m = m0 + wm * 64 + row;
        if (keep[r])
            __builtin_nontemporal_store(
                d, reinterpret_cast<i32x4*>(static_cast<uint16_t*>(p.out) + (int64_t)m * p.ld_out + n0 + wn * 128 + rd_chunk * 8));
    }
}

// ---------------------------------------------------------------------------
// The kernel above with twice the weight rows: 128 x 512 tiles, four waves, 2 x 2, each a 64 x 256 block = 64
// accumulators (all 256 AGPRs), i.e. the operand traffic per MFMA of the 256 x 256 kernel on tiles that are only
// 128 rows high - what the grouped layout allows.  Two activation stages of 16 KiB, three weight stages of 32 KiB,
// three scale stages of 2 KiB; a K step is four phases of eight groups of two MFMAs (one weight tile against the
// two activation tiles of a half).  Per wave and step 4 activation + 8 weight + 2 scale loads; the barrier lets the
// ten newest pass.  Edges and the last K step as above.
// ---------------------------------------------------------------------------
#define MX4_MMA2W(wh, xb, xh, g)                                                                             \
    {                                                                                                        \
        _Pragma("unroll") for (int e = 0; e < 2; ++e) {                                                      \
            acc[(wh)*8 + (g)][(xh)*2 + e] =                                                                  \
                mfma_w4a8<0>(W[wh][g], X[xb][e], acc[(wh)*8 + (g)][(xh)*2 + e], (int)S[(wh)*8 + (g)]);      \
        }                                                                                                    \
    }

template <bool OUT_F32>
__global__ __launch_bounds__(256) void gemm_mxfp4_128x512_kernel(const Mx4Args p) {
    constexpr int BM = 128, BN = 512;
    constexpr int XS = BM * 128, WS = BN * 64, SS = BN * 4;
    constexpr int WBASE = 2 * XS, SBASE = WBASE + 3 * WS, ABASE = SBASE + 3 * SS;  // + 512 bytes of activation scales
    constexpr uint32_t kEnd = 0xEFFFFFFFu;  // the longest descriptor: kBeyond stays beyond it
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    int tm, tn;
    if (p.m_indices) mx4_tile_of_block<4>(blockIdx.x, p.tiles_m, p.tiles_n, tm, tn);
    else mx4_tile_of_block<8>(blockIdx.x, p.tiles_m, p.tiles_n, tm, tn);
    const int m0 = tm * BM, n0 = tn * BN;
    const uint8_t* wmat = p.w;
    const uint8_t* smat = p.ws;
    int expert = 0;
    if (p.m_indices) {
        expert = p.m_indices[m0];  // groups start on multiples of 128 rows
        if (expert < 0) return;    // a tile of padding (uniform for the workgroup)
        wmat += (int64_t)expert * p.N * p.ld_w;
        smat += (int64_t)expert * p.N * p.ld_ws;
    }
    const int t = threadIdx.x, lane = t & 63;
    const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
    const int wm = wave & 1, wn = wave >> 1;
    const int lrow = lane & 15, quarter = lane >> 4;
    const int KT = (p.K + 127) >> 7;
    const int last = KT - 1;
    const int k_tail = p.K - (last << 7);            // 32 .. 128 elements in the last step
    const int vq = k_tail >> 5;                      // its valid quarters, 1 .. 4

    uint64_t a_wave = reinterpret_cast<uint64_t>(p.a) + ((uint64_t)m0 + (uint64_t)wave * 8) * (uint64_t)p.ld_a;
    uint64_t w_wave = reinterpret_cast<uint64_t>(wmat) + ((uint64_t)n0 + (uint64_t)wave * 16) * (uint64_t)p.ld_w;
    uint64_t s_tile = reinterpret_cast<uint64_t>(smat) + (uint64_t)n0 * (uint64_t)p.ld_ws;
    uint32_t a_step = 32u * (uint32_t)p.ld_a, w_step = 64u * (uint32_t)p.ld_w;  // pitches are < 2^24
    const int64_t a_rows = (int64_t)p.M - m0 - wave * 8, w_rows = (int64_t)p.N - n0 - wave * 16, s_rows = (int64_t)p.N - n0;
    const int64_t a_left = a_rows > 0 ? a_rows * p.ld_a : 0, w_left = w_rows > 0 ? w_rows * p.ld_w : 0, s_left = s_rows > 0 ? s_rows * p.ld_ws : 0;
    uint32_t a_end = a_left < (int64_t)kEnd ? (uint32_t)a_left : kEnd, w_end = w_left < (int64_t)kEnd ? (uint32_t)w_left : kEnd,
             s_end = s_left < (int64_t)kEnd ? (uint32_t)s_left : kEnd;
    asm volatile("" : "+s"(a_wave), "+s"(w_wave), "+s"(s_tile), "+s"(a_step), "+s"(w_step), "+s"(a_end), "+s"(w_end), "+s"(s_end));
    const int xc = (lane & 7) ^ ((wave & 1) * 4 + (lane >> 4));
    const uint32_t va_lane = (uint32_t)(lane >> 3) * (uint32_t)p.ld_a + (uint32_t)(xc << 4);
    const uint32_t va_tail = xc * 16 < k_tail ? va_lane : kBeyond;
    const int wc = (lane & 3) ^ ((lane >> 4) & 3);
    const uint32_t vw_lane = (uint32_t)(lane >> 2) * (uint32_t)p.ld_w + (uint32_t)(wc << 4);
    const uint32_t vw_tail = wc * 32 < k_tail ? vw_lane : kBeyond;
    // scale words: word (2 wave + u) * 64 + lane = wn' * 256 + lrow' * 16 + tile' belongs to row wn' * 256 + tile' * 16 + lrow'
    uint32_t vs_lane[2];
#pragma unroll
    for (int u = 0; u < 2; ++u) {
        const int sword = (wave * 2 + u) * 64 + lane;
        vs_lane[u] = (uint32_t)((sword >> 8) * 256 + (sword & 15) * 16 + ((sword >> 4) & 15)) * (uint32_t)p.ld_ws;
    }
    const uint32_t s_last = (uint32_t)(last * 4 - (4 - vq));  // the last step's word ends with the row (K >= 128)
    const unsigned sshift = 8u * (unsigned)quarter, sshift_tail = 8u * (unsigned)(quarter + 4 - vq);
    const bool q_in_tail = quarter < vq;
    typedef __attribute__((address_space(1))) const void gbl_void;
    typedef __attribute__((address_space(3))) void lds_void;
    const __amdgpu_buffer_rsrc_t ra = __builtin_amdgcn_make_buffer_rsrc(reinterpret_cast<void*>(a_wave), 0, (int)a_end, 0x00020000);
    const __amdgpu_buffer_rsrc_t rw = __builtin_amdgcn_make_buffer_rsrc(reinterpret_cast<void*>(w_wave), 0, (int)w_end, 0x00020000);
    const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc(reinterpret_cast<void*>(s_tile), 0, (int)s_end, 0x00020000);
    auto dma_x = [&](int kt, int stage, int i) {
        __builtin_amdgcn_raw_ptr_buffer_load_lds(ra, (lds_void*)(smem + stage * XS + (wave + 4 * i) * 1024), 16, kt == last ? va_tail : va_lane,
                                                 (uint32_t)i * a_step + ((uint32_t)kt << 7), 0, 0);
    };
    auto dma_w = [&](int kt, int stage, int i) {
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rw, (lds_void*)(smem + WBASE + stage * WS + (wave + 4 * i) * 1024), 16, kt == last ? vw_tail : vw_lane,
                                                 (uint32_t)i * w_step + ((uint32_t)kt << 6), 0, 0);
    };
    auto dma_s = [&](int kt, int stage, int u) {
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, (lds_void*)(smem + SBASE + stage * SS + (wave * 2 + u) * 256), 4, vs_lane[u],
                                                 kt == last ? s_last : (uint32_t)kt << 2, 0, 0);
    };

    f32x4 acc[16][4];  // [n tile][m tile]
#pragma unroll
    for (int i = 0; i < 16; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};

    const int fsw = (lrow >> 1) & 7;
    const int x_off = (wm * 64 + lrow) * 128 + ((quarter ^ fsw) << 4);
    const int x_off2 = (wm * 64 + lrow) * 128 + (((4 + quarter) ^ fsw) << 4);
    const int w_off = WBASE + (wn * 256 + lrow) * 64 + ((quarter ^ ((lrow >> 2) & 3)) << 4);
    const int s_off = SBASE + (wn * 256 + lrow * 16) * 4;
    auto xfrag = [&](int stage_bytes, int tile16) {
        const uint8_t* base = smem + stage_bytes + tile16 * 2048;
        const i32x4 lo = *reinterpret_cast<const i32x4*>(base + x_off);
        const i32x4 hi = *reinterpret_cast<const i32x4*>(base + x_off2);
        return i32x8{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    };
    auto wfrag = [&](int stage, int tile16) { return *reinterpret_cast<const i32x4*>(smem + stage * WS + tile16 * 1024 + w_off); };
    auto sfrag = [&](int stage, int part) { return *reinterpret_cast<const u32x4*>(smem + stage * SS + s_off + part * 16); };
    auto sbyte = [&](uint32_t word, int kt) -> uint32_t {
        const bool tail = kt == last;
        const uint32_t b = word >> (tail ? sshift_tail : sshift);
        return (tail && !q_in_tail) ? 127u : b;
    };
    i32x4 W[2][8];
    i32x8 X[2][2];
    uint32_t S[16];
    u32x4 sraw[4];  // scale words of tiles 0-3, 4-7 (the next step's first weight half) and 8-11, 12-15 (its second)

    {
        const int m = m0 + (wave & 1) * 64 + lane;
        __builtin_amdgcn_global_load_lds((gbl_void*)(p.sa + (m < p.M ? m : p.M - 1)), (lds_void*)(smem + ABASE + (wave & 1) * 256), 4, 0, 0);
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) dma_x(0, 0, i);
#pragma unroll
    for (int i = 0; i < 8; ++i) dma_w(0, 0, i);
    dma_s(0, 0, 0);
    dma_s(0, 0, 1);
#pragma unroll
    for (int i = 0; i < 4; ++i) dma_x(1 < last ? 1 : last, 1, i);
#pragma unroll
    for (int i = 0; i < 8; ++i) dma_w(1 < last ? 1 : last, 1, i);
    dma_s(1 < last ? 1 : last, 1, 0);
    dma_s(1 < last ? 1 : last, 1, 1);
#pragma unroll
    for (int i = 0; i < 8; ++i) dma_w(2 < last ? 2 : last, 2, i);
    dma_s(2 < last ? 2 : last, 2, 0);
    dma_s(2 < last ? 2 : last, 2, 1);
    MX4_WAIT_BARRIER(24);  // the scales and tile 0 (15 loads) have landed; the other 24 stay in flight
#pragma unroll
    for (int g = 0; g < 8; ++g) W[0][g] = wfrag(0, g);
#pragma unroll
    for (int g = 0; g < 2; ++g) X[0][g] = xfrag(0, g);
#pragma unroll
    for (int q4 = 0; q4 < 4; ++q4) sraw[q4] = sfrag(0, q4);
    asm volatile("" : "+v"(sraw[0]), "+v"(sraw[1]), "+v"(sraw[2]), "+v"(sraw[3]));  // four 16-byte reads, not sixteen of four bytes
#pragma unroll
    for (int g = 0; g < 8; ++g) S[g] = sbyte(sraw[g >> 2][g & 3], 0);
    MX4_PHASE_END();

    int ws_cur = 0;  // kt % 3
    for (int kt = 0; kt < KT; ++kt) {
        const int xs_cur = (kt & 1) * XS, xs_nxt = xs_cur ^ XS;
        const int ws_nxt = ws_cur == 2 ? 0 : ws_cur + 1;
        const int kw = kt + 3 < last ? kt + 3 : last, kx = kt + 2 < last ? kt + 2 : last;
#pragma unroll
        for (int g = 0; g < 8; ++g) {  // S0 (w0, x0): reads x1
            if (g < 2) X[1][g] = xfrag(xs_cur, 2 + g);
            MX4_MMA2W(0, 0, 0, g);
            MX4_PHASE_END();
        }
#pragma unroll
        for (int g = 0; g < 8; ++g) {  // S1 (w0, x1): reads w1, scale bytes of w1
            W[1][g] = wfrag(ws_cur, 8 + g);
            S[8 + g] = sbyte(sraw[2 + (g >> 2)][g & 3], kt);
            MX4_MMA2W(0, 1, 1, g);
            MX4_PHASE_END();
        }
        MX4_WAIT_BARRIER(10);
        MX4_PHASE_END();
#pragma unroll
        for (int g = 0; g < 8; ++g) {  // S2 (w1, x0): reads next w0 and the next scale words; loads of activation tile kt + 2
            W[0][g] = wfrag(ws_nxt, g);  // after the last step: stale data, unused
            if (g >= 4) {
                // words 8-15 are shifted into place in S1 of the next step (S[8..15] are still in use)
                sraw[g - 4] = sfrag(ws_nxt, g - 4);
                asm volatile("" : "+v"(sraw[g - 4]));
            }
            if (g < 4) dma_x(kx, kt & 1, g);
            MX4_MMA2W(1, 0, 0, g);
            MX4_PHASE_END();
        }
#pragma unroll
        for (int g = 0; g < 8; ++g) {  // S3 (w1, x1): reads next x0; loads of weight and scale tile kt + 3
            if (g < 2) X[0][g] = xfrag(xs_nxt, g);
            dma_w(kw, ws_cur, g);
            if (g >= 6) dma_s(kw, ws_cur, g - 6);
            S[g] = sbyte(sraw[g >> 2][g & 3], kt + 1);
            MX4_MMA2W(1, 1, 1, g);
            MX4_PHASE_END();
        }
        ws_cur = ws_nxt;
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the scales have landed, and nothing may still land in the stages
    __syncthreads();
    const float* const sa_lds = reinterpret_cast<const float*>(smem + ABASE);

    float sam[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) sam[j] = sa_lds[wm * 64 + j * 16 + lrow];
    if (OUT_F32) {
        bool keep[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int m = m0 + wm * 64 + j * 16 + lrow;
            keep[j] = m < p.M;
            if (p.m_indices && keep[j]) keep[j] = p.m_indices[m] == expert;
        }
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const int n = n0 + wn * 256 + i * 16 + quarter * 4;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int m = m0 + wm * 64 + j * 16 + lrow;
                f32x4 v = acc[i][j];
#pragma unroll
                for (int e = 0; e < 4; ++e) v[e] = v[e] * sam[j];
                if (keep[j] && n < p.N)
                    __builtin_nontemporal_store(v, reinterpret_cast<f32x4*>(static_cast<float*>(p.out) + (int64_t)m * p.ld_out + n));
            }
        }
        return;
    }
    // bf16: the wave's 64 x 256 block goes through LDS in two halves of 128 columns
    constexpr int EST = 272;
    static_assert(4 * 64 * EST <= ABASE, "the epilogue buffers must not reach the activation scales");
    const int rd_row = lane >> 4, rd_chunk = lane & 15;
    bool keep[16];
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        const int m = m0 + wm * 64 + r * 4 + rd_row;
        keep[r] = m < p.M;
        if (p.m_indices && keep[r]) keep[r] = p.m_indices[m] == expert;
    }
    __syncthreads();  // all waves are done reading the operand stages
    uint8_t* const ebuf = smem + wave * (64 * EST);
#pragma unroll
    for (int h = 0; h < 2; ++h) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                f32x4 v = acc[h * 8 + i][j];
#pragma unroll
                for (int e = 0; e < 4; ++e) v[e] = v[e] * sam[j];
                *reinterpret_cast<uint2*>(ebuf + (j * 16 + lrow) * EST + (i * 16 + quarter * 4) * 2) =
                    make_uint2(pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3]));
            }
        }
        // written and read by the same wave: LDS operations of one wave complete in order
        const int n = n0 + wn * 256 + h * 128 + rd_chunk * 8;  // N % 16 == 0: a chunk of 8 is inside or outside as a whole
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int row = r * 4 + rd_row;
            const i32x4 d = *reinterpret_cast<const i32x4*>(ebuf + row * EST + rd_chunk * 16);
            const int m = m0 + wm * 64 + row;
            if (keep[r] && n < p.N)
                __builtin_nontemporal_store(d, reinterpret_cast<i32x4*>(static_cast<uint16_t*>(p.out) + (int64_t)m * p.ld_out + n));
        }
    }
}

// ---------------------------------------------------------------------------
// 17..128 tokens (batched decode) on one weight matrix: a strip kernel.  A workgroup of four waves owns all BM (64 or
// 128) token rows and 80 weight rows over the whole of K, so the weight is read once by N / 80 workgroups - one per CU
// for an 18944-row weight.  Activation tile, weight codes and scale words of a K step go straight into LDS in a ring
// of S stages (9 for 64 rows, 6 for 128: all the LDS holds); step kt waits for tile kt, requests tile kt + S - 1 into
// the stage that step kt - 1 used, and computes: one barrier per step, BM / 32 activation + 2 weight + 1 scale loads
// per wave and step, the barrier lets the loads of the S - 2 tiles in between pass.  Wave w computes token rows
// w BM / 4 ... against the five weight tiles.  Edges and the last K step as in the 128 x 256 kernel.
// ---------------------------------------------------------------------------
template <int BM, bool OUT_F32>
__global__ __launch_bounds__(256) void gemm_mxfp4_strip_kernel(const Mx4Args p) {
    constexpr int TN = 5, BN = TN * 16;
    constexpr int LX = BM / 32, L = LX + 3;             // loads per wave and step
    constexpr int XS = BM * 128, WS = 8 * 1024, SS = 1024;  // a weight stage holds 8 groups of 16 rows x 64 bytes, 5 are used
    constexpr int S = BM == 64 ? 9 : 6;
    constexpr int XT = BM / 64;
    constexpr int WBASE = S * XS, SBASE = WBASE + S * WS;
    constexpr uint32_t kEnd = 0xEFFFFFFFu;
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    const int m0 = (int)(blockIdx.x % (unsigned)p.tiles_m) * BM, n0 = (int)(blockIdx.x / (unsigned)p.tiles_m) * BN;
    const int t = threadIdx.x, lane = t & 63;
    const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
    const int lrow = lane & 15, quarter = lane >> 4;
    const int KT = (p.K + 127) >> 7;
    const int last = KT - 1;
    const int k_tail = p.K - (last << 7);
    const int vq = k_tail >> 5;

    uint64_t a_wave = reinterpret_cast<uint64_t>(p.a) + ((uint64_t)m0 + (uint64_t)wave * 8) * (uint64_t)p.ld_a;
    uint64_t w_wave = reinterpret_cast<uint64_t>(p.w) + ((uint64_t)n0 + (uint64_t)wave * 16) * (uint64_t)p.ld_w;
    uint64_t s_tile = reinterpret_cast<uint64_t>(p.ws) + (uint64_t)n0 * (uint64_t)p.ld_ws;
    uint32_t a_step = 32u * (uint32_t)p.ld_a, w_step = 64u * (uint32_t)p.ld_w;
    const int64_t a_rows = (int64_t)p.M - m0 - wave * 8, w_rows = (int64_t)p.N - n0 - wave * 16, s_rows = (int64_t)p.N - n0;
    const int64_t a_left = a_rows > 0 ? a_rows * p.ld_a : 0, w_left = w_rows > 0 ? w_rows * p.ld_w : 0, s_left = s_rows > 0 ? s_rows * p.ld_ws : 0;
    uint32_t a_end = a_left < (int64_t)kEnd ? (uint32_t)a_left : kEnd, w_end = w_left < (int64_t)kEnd ? (uint32_t)w_left : kEnd,
             s_end = s_left < (int64_t)kEnd ? (uint32_t)s_left : kEnd;
    asm volatile("" : "+s"(a_wave), "+s"(w_wave), "+s"(s_tile), "+s"(a_step), "+s"(w_step), "+s"(a_end), "+s"(w_end), "+s"(s_end));
    const int xc = (lane & 7) ^ ((wave & 1) * 4 + (lane >> 4));
    const uint32_t va_lane = (uint32_t)(lane >> 3) * (uint32_t)p.ld_a + (uint32_t)(xc << 4);
    const uint32_t va_tail = xc * 16 < k_tail ? va_lane : kBeyond;
    const int wc = (lane & 3) ^ ((lane >> 4) & 3);
    const uint32_t vw_lane = (uint32_t)(lane >> 2) * (uint32_t)p.ld_w + (uint32_t)(wc << 4);
    const uint32_t vw_tail = wc * 32 < k_tail ? vw_lane : kBeyond;
    // scale words: word wave * 64 + lane = lrow' * 8 + tile' belongs to row tile' * 16 + lrow'; tiles 5..7 and the words of
    // waves 2 and 3 do not exist
    const int sword = wave * 64 + lane;
    const uint32_t vs_lane = (sword < 128 && (sword & 7) < TN) ? (uint32_t)((sword & 7) * 16 + (sword >> 3)) * (uint32_t)p.ld_ws : kBeyond;
    const uint32_t s_last = (uint32_t)(last * 4 - (4 - vq));
    const unsigned sshift = 8u * (unsigned)quarter, sshift_tail = 8u * (unsigned)(quarter + 4 - vq);
    const bool q_in_tail = quarter < vq;
    typedef __attribute__((address_space(3))) void lds_void;
    const __amdgpu_buffer_rsrc_t ra = __builtin_amdgcn_make_buffer_rsrc(reinterpret_cast<void*>(a_wave), 0, (int)a_end, 0x00020000);
    const __amdgpu_buffer_rsrc_t rw = __builtin_amdgcn_make_buffer_rsrc(reinterpret_cast<void*>(w_wave), 0, (int)w_end, 0x00020000);
    const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc(reinterpret_cast<void*>(s_tile), 0, (int)s_end, 0x00020000);
    auto dma = [&](int kt, int stage) {
        const bool tail = kt == last;
#pragma unroll
        for (int i = 0; i < LX; ++i)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(ra, (lds_void*)(smem + stage * XS + (wave + 4 * i) * 1024), 16, tail ? va_tail : va_lane,
                                                     (uint32_t)i * a_step + ((uint32_t)kt << 7), 0, 0);
#pragma unroll
        for (int i = 0; i < 2; ++i)  // groups of 16 weight rows wave and wave + 4: only group 4 of the second set exists
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rw, (lds_void*)(smem + WBASE + stage * WS + (wave + 4 * i) * 1024), 16,
                                                     (wave + 4 * i) < TN ? (tail ? vw_tail : vw_lane) : kBeyond,
                                                     (uint32_t)i * w_step + ((uint32_t)kt << 6), 0, 2);
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, (lds_void*)(smem + SBASE + stage * SS + wave * 256), 4, vs_lane,
                                                 tail ? s_last : (uint32_t)kt << 2, 0, 0);
    };

    float sam[XT];
#pragma unroll
    for (int j = 0; j < XT; ++j) {
        const int m = m0 + wave * (BM / 4) + j * 16 + lrow;
        sam[j] = p.sa[m < p.M ? m : p.M - 1];  // the oldest load: every later wait covers it
    }
    f32x4 acc[TN][XT];
#pragma unroll
    for (int i = 0; i < TN; ++i)
#pragma unroll
        for (int j = 0; j < XT; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};

    const int fsw = (lrow >> 1) & 7;
    const int x_off = (wave * (BM / 4) + lrow) * 128 + ((quarter ^ fsw) << 4);
    const int x_off2 = (wave * (BM / 4) + lrow) * 128 + (((4 + quarter) ^ fsw) << 4);
    const int w_off = WBASE + lrow * 64 + ((quarter ^ ((lrow >> 2) & 3)) << 4);
    const int s_off = SBASE + lrow * 32;

#pragma unroll
    for (int d = 0; d < S - 1; ++d) dma(d < last ? d : last, d);
    int cur = 0;  // kt % S
    for (int kt = 0; kt < KT; ++kt) {
        asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" ::"n"((S - 2) * L) : "memory");
        const int nxt = cur == 0 ? S - 1 : cur - 1;  // (kt + S - 1) % S
        dma(kt + S - 1 < last ? kt + S - 1 : last, nxt);
        __builtin_amdgcn_sched_barrier(0);
        const bool tail = kt == last;
        u32x4 s03 = *reinterpret_cast<const u32x4*>(smem + cur * SS + s_off);
        uint32_t s4 = *reinterpret_cast<const uint32_t*>(smem + cur * SS + s_off + 16);
        asm volatile("" : "+v"(s03));
        i32x4 fw[TN];
        uint32_t sb_[TN];
#pragma unroll
        for (int i = 0; i < TN; ++i) {
            fw[i] = *reinterpret_cast<const i32x4*>(smem + cur * WS + i * 1024 + w_off);
            const uint32_t word = i < 4 ? s03[i] : s4;
            const uint32_t b = word >> (tail ? sshift_tail : sshift);
            sb_[i] = (tail && !q_in_tail) ? 127u : b;
        }
#pragma unroll
        for (int j = 0; j < XT; ++j) {
            const uint8_t* base = smem + cur * XS + j * 2048;
            const i32x4 lo = *reinterpret_cast<const i32x4*>(base + x_off);
            const i32x4 hi = *reinterpret_cast<const i32x4*>(base + x_off2);
            const i32x8 xf = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
#pragma unroll
            for (int i = 0; i < TN; ++i) acc[i][j] = mfma_w4a8<0>(fw[i], xf, acc[i][j], (int)sb_[i]);
        }
        // pinned, or the compiler may move the MFMAs (pure functions of registers) past the next barrier
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
            for (int e = 0; e < 4; ++e) v[e] = acc[i][j][e] * sam[j];
            if (OUT_F32) *reinterpret_cast<f32x4*>(static_cast<float*>(p.out) + (int64_t)m * p.ld_out + n) = v;
            else *reinterpret_cast<uint2*>(static_cast<uint16_t*>(p.out) + (int64_t)m * p.ld_out + n) =
                    make_uint2(pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3]));
        }
    }
}

// more dynamic LDS than the default 64 KiB: the limit is raised once per device and kernel
static int ensure_lds(const void* fn, size_t lds, std::atomic<bool> (&raised)[64]) {
    if (lds <= 64 * 1024) return CFP8_OK;
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return set_error(CFP8_ELAUNCH, "gemm_mxfp4: no current device");
    const bool cached = dev >= 0 && dev < 64;
    if (cached && raised[dev].load(std::memory_order_acquire)) return CFP8_OK;
    if (hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess) {
        (void)hipGetLastError();
        return set_error(CFP8_ELAUNCH, "gemm_mxfp4: cannot raise the dynamic LDS limit to %zu bytes", lds);
    }
    if (cached) raised[dev].store(true, std::memory_order_release);
    return CFP8_OK;
}

// compute units of the current device (256 if the query fails), cached per device ordinal
static int mx4_cu_count() {
    static std::atomic<int> cached[64];  // zero-initialised
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) {
        (void)hipGetLastError();
        return 256;
    }
    if (dev >= 0 && dev < 64) {
        const int c = cached[dev].load(std::memory_order_relaxed);
        if (c > 0) return c;
    }
    int cus = 0;
    if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0) {
        (void)hipGetLastError();
        return 256;
    }
    if (dev >= 0 && dev < 64) cached[dev].store(cus, std::memory_order_relaxed);
    return cus;
}

static int launch_mx4_256(Mx4Args p, int out_dtype, hipStream_t st) {
    p.tiles_m = p.M / 256;
    p.tiles_n = p.N / 256;
    constexpr size_t lds = 2 * 256 * 128 + 3 * 256 * 64 + 3 * 256 * 4 + 1024;
    const bool f32 = out_dtype == CFP8_OUT_F32;
    static std::atomic<bool> raised[2][64];
    const void* fn = f32 ? reinterpret_cast<const void*>(gemm_mxfp4_256_kernel<true>) : reinterpret_cast<const void*>(gemm_mxfp4_256_kernel<false>);
    if (int rc = ensure_lds(fn, lds, raised[f32])) return rc;
    const unsigned blocks = (unsigned)(p.tiles_m * p.tiles_n);
    if (f32) hipLaunchKernelGGL(gemm_mxfp4_256_kernel<true>, dim3(blocks), dim3(256), lds, st, p);
    else hipLaunchKernelGGL(gemm_mxfp4_256_kernel<false>, dim3(blocks), dim3(256), lds, st, p);
    return check_launch("gemm_mxfp4");
}

static int launch_mx4_128(Mx4Args p, int out_dtype, hipStream_t st) {
    p.tiles_m = (p.M + 127) / 128;
    p.tiles_n = (p.N + 255) / 256;
    const int64_t tiles = (int64_t)p.tiles_m * p.tiles_n;
    if (tiles > 0x7FFFFFFFll) return set_error(CFP8_EINVAL, "gemm_mxfp4: too many tiles");
    constexpr size_t lds = 2 * 128 * 128 + 3 * 256 * 64 + 3 * 256 * 4 + 512;
    const bool f32 = out_dtype == CFP8_OUT_F32;
    static std::atomic<bool> raised[2][64];
    const void* fn = f32 ? reinterpret_cast<const void*>(gemm_mxfp4_128_kernel<true>) : reinterpret_cast<const void*>(gemm_mxfp4_128_kernel<false>);
    if (int rc = ensure_lds(fn, lds, raised[f32])) return rc;
    if (f32) hipLaunchKernelGGL(gemm_mxfp4_128_kernel<true>, dim3((unsigned)tiles), dim3(256), lds, st, p);
    else hipLaunchKernelGGL(gemm_mxfp4_128_kernel<false>, dim3((unsigned)tiles), dim3(256), lds, st, p);
    return check_launch("gemm_mxfp4");
}

static int launch_mx4_128x512(Mx4Args p, int out_dtype, hipStream_t st) {
    p.tiles_m = (p.M + 127) / 128;
    p.tiles_n = (p.N + 511) / 512;
    const int64_t tiles = (int64_t)p.tiles_m * p.tiles_n;
    if (tiles > 0x7FFFFFFFll) return set_error(CFP8_EINVAL, "gemm_mxfp4: too many tiles");
    constexpr size_t lds = 2 * 128 * 128 + 3 * 512 * 64 + 3 * 512 * 4 + 512;
    const bool f32 = out_dtype == CFP8_OUT_F32;
    static std::atomic<bool> raised[2][64];
    const void* fn = f32 ? reinterpret_cast<const void*>(gemm_mxfp4_128x512_kernel<true>) : reinterpret_cast<const void*>(gemm_mxfp4_128x512_kernel<false>);
    if (int rc = ensure_lds(fn, lds, raised[f32])) return rc;
    if (f32) hipLaunchKernelGGL(gemm_mxfp4_128x512_kernel<true>, dim3((unsigned)tiles), dim3(256), lds, st, p);
    else hipLaunchKernelGGL(gemm_mxfp4_128x512_kernel<false>, dim3((unsigned)tiles), dim3(256), lds, st, p);
    return check_launch("gemm_mxfp4");
}

template <int BM>
static int launch_mx4_strip(Mx4Args p, int out_dtype, hipStream_t st) {
    constexpr int S = BM == 64 ? 9 : 6;
    constexpr size_t lds = (size_t)S * (BM * 128 + 8 * 1024 + 1024);
    static_assert(lds <= 160 * 1024, "strip kernel LDS");
    p.tiles_m = (p.M + BM - 1) / BM;
    const int64_t blocks = (p.N + 79) / 80 * p.tiles_m;
    const bool f32 = out_dtype == CFP8_OUT_F32;
    static std::atomic<bool> raised[2][64];
    const void* fn = f32 ? reinterpret_cast<const void*>(gemm_mxfp4_strip_kernel<BM, true>) : reinterpret_cast<const void*>(gemm_mxfp4_strip_kernel<BM, false>);
    if (int rc = ensure_lds(fn, lds, raised[f32])) return rc;
    if (f32) hipLaunchKernelGGL((gemm_mxfp4_strip_kernel<BM, true>), dim3((unsigned)blocks), dim3(256), lds, st, p);
    else hipLaunchKernelGGL((gemm_mxfp4_strip_kernel<BM, false>), dim3((unsigned)blocks), dim3(256), lds, st, p);
    return check_launch("gemm_mxfp4");
}

template <int TM, int NTL>
static int launch_mx4_skinny(const Mx4Args& p, int out_dtype, hipStream_t st) {
    // 64 KiB of activation buffers either way, eight K steps of weights per wave in flight
    constexpr int KS = TM > 2 ? 4 : 8, PC = TM > 2 ? 4 : 2;
    constexpr size_t lds = (size_t)2 * KS * TM * 2048;  // >= the NTL * TM * 1 KiB of the final reduction
    static_assert(lds >= (size_t)NTL * TM * 1024 && lds <= 160 * 1024, "skinny kernel LDS");
    const unsigned blocks = (unsigned)((p.N + NTL * 16 - 1) / (NTL * 16));
    const bool f32 = out_dtype == CFP8_OUT_F32;
    const void* fn = f32 ? reinterpret_cast<const void*>(gemm_mxfp4_skinny_kernel<TM, NTL, KS, PC, true>)
                         : reinterpret_cast<const void*>(gemm_mxfp4_skinny_kernel<TM, NTL, KS, PC, false>);
    static std::atomic<bool> raised[2][64];
    if (int rc = ensure_lds(fn, lds, raised[f32])) return rc;
    if (f32) hipLaunchKernelGGL((gemm_mxfp4_skinny_kernel<TM, NTL, KS, PC, true>), dim3(blocks), dim3(NTL * 128), lds, st, p);
    else hipLaunchKernelGGL((gemm_mxfp4_skinny_kernel<TM, NTL, KS, PC, false>), dim3(blocks), dim3(NTL * 128), lds, st, p);
    return check_launch("gemm_mxfp4");
}

// The linear layer for at most 4 tokens and K <= 4096 in ONE launch: gemm_mxfp4_gemv_lds_kernel with the per-token FP8
// quantisation of the bf16 activations folded in.  A workgroup first requests its weights (all of a wave's K steps
// are in flight before anything else happens), then its 256 threads quantise the tokens together - a thread holds at
// most two 16-byte vectors of a token between the amax and the cast, the arithmetic of the rowwise quantiser -
// into LDS, from where the MFMA fragments are read.  Bit-identical to quantising first and calling the kernel above.
template <int MR, bool OUT_F32>
__global__ __launch_bounds__(256) void linear_mxfp4_gemv_fused_kernel(const uint4* __restrict__ x, int64_t ldx, const Mx4Args p) {
    extern __shared__ __attribute__((aligned(16))) uint8_t xs[];  // [M][KT * 128 + 16] fp8
    __shared__ __attribute__((aligned(16))) float red[3 * 64 * 4];
    __shared__ u32 amax_red[4][MR];
    const int t = threadIdx.x, lane = t & 63;
    const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
    const int lrow = lane & 15, quarter = lane >> 4;
    const int n0 = blockIdx.x * 16;
    const int KT = (p.K + 127) >> 7;  // <= 32: one pass of kGemvDepth K steps per wave
    const int pitch = KT * 128 + 16;
    const int wrow = n0 + lrow;
    const bool wok = wrow < p.N, xok = lrow < p.M;
    const uint8_t* const wptr = p.w + (int64_t)(wok ? wrow : 0) * p.ld_w + quarter * 16;
    const uint8_t* const sptr = p.ws + (int64_t)(wok ? wrow : 0) * p.ld_ws + quarter;
    u32x4 wv[kGemvDepth];
    uint32_t sc[kGemvDepth];
#pragma unroll
    for (int i = 0; i < kGemvDepth; ++i) {
        const int kt = wave + 4 * i;
        const int k = (kt < KT ? kt : 0) << 7;
        const bool in_w = kt < KT && k + quarter * 32 < p.K;
        wv[i] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(wptr + (in_w ? (k >> 1) : 0)));
        sc[i] = __builtin_nontemporal_load(sptr + (in_w ? (k >> 5) : 0));
    }
    // the tokens (MR >= M of them): amax, scale, cast - rows >= M read row 0 and are never used
    const int nvec = p.K >> 3, nvec_pad = KT * 16;
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
                const int idx = t + 256 * j;  // vectors between K and the end of the last K step are zero
                if (idx < nvec_pad) *reinterpret_cast<uint2*>(xs + r * pitch + idx * 8) = idx < nvec ? cast8(v[r][j], d) : make_uint2(0u, 0u);
            }
        }
    }
    __syncthreads();
    f32x4 acc = f32x4{0.f, 0.f, 0.f, 0.f};
    const uint8_t* const xrow = xs + (xok ? lrow : 0) * pitch + quarter * 16;
#pragma unroll
    for (int i = 0; i < kGemvDepth; ++i) {
        const int kt = wave + 4 * i;
        const int k = (kt < KT ? kt : 0) << 7;
        const bool in = kt < KT, in_w = in && k + quarter * 32 < p.K;
        const u32x4 lo = *reinterpret_cast<const u32x4*>(xrow + k), hi = *reinterpret_cast<const u32x4*>(xrow + k + 64);
        i32x4 fw;
        i32x8 fx;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            fw[e] = (int)wv[i][e];
            fx[e] = (in && xok) ? (int)lo[e] : 0;
            fx[4 + e] = (in && xok) ? (int)hi[e] : 0;
        }
        const int scale_w = (in_w && wok) ? (int)sc[i] : 127;
        acc = mfma_w4a8<0>(fw, fx, acc, scale_w);
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
            float sam = scale[0];
#pragma unroll
            for (int r = 1; r < MR; ++r) sam = m == r ? scale[r] : sam;
            f32x4 o;
#pragma unroll
            for (int e = 0; e < 4; ++e) o[e] = acc[e] * sam;
            if (OUT_F32) *reinterpret_cast<f32x4*>(static_cast<float*>(p.out) + (int64_t)m * p.ld_out + n) = o;
            else *reinterpret_cast<uint2*>(static_cast<uint16_t*>(p.out) + (int64_t)m * p.ld_out + n) =
                    make_uint2(pack_bf16x2(o[0], o[1]), pack_bf16x2(o[2], o[3]));
        }
    }
}

template <int MR>
static int launch_linear_mx4_fused_mr(const void* x, int64_t ld_x, const Mx4Args& p, int out_dtype, hipStream_t st) {
    const unsigned blocks = (unsigned)((p.N + 15) / 16);
    const size_t lds = (size_t)p.M * ((size_t)((p.K + 127) / 128) * 128 + 16);  // <= 4 x 4112 bytes
    if (out_dtype == CFP8_OUT_F32)
        hipLaunchKernelGGL((linear_mxfp4_gemv_fused_kernel<MR, true>), dim3(blocks), dim3(256), lds, st, static_cast<const uint4*>(x), ld_x / 8, p);
    else
        hipLaunchKernelGGL((linear_mxfp4_gemv_fused_kernel<MR, false>), dim3(blocks), dim3(256), lds, st, static_cast<const uint4*>(x), ld_x / 8, p);
    return check_launch("linear_mxfp4");
}

static int launch_mx4_gemv(const Mx4Args& p, int out_dtype, hipStream_t st) {
    const unsigned blocks = (unsigned)((p.N + 15) / 16);
    const size_t x_lds = (size_t)p.M * ((size_t)((p.K + 127) / 128) * 128 + 16);
    if (p.M <= kGemvLdsRows && x_lds <= 32 * 1024) {
        if (out_dtype == CFP8_OUT_F32) hipLaunchKernelGGL(gemm_mxfp4_gemv_lds_kernel<true>, dim3(blocks), dim3(256), x_lds, st, p);
        else hipLaunchKernelGGL(gemm_mxfp4_gemv_lds_kernel<false>, dim3(blocks), dim3(256), x_lds, st, p);
        return check_launch("gemm_mxfp4");
    }
    if (out_dtype == CFP8_OUT_F32) hipLaunchKernelGGL(gemm_mxfp4_gemv_kernel<true>, dim3(blocks), dim3(256), 0, st, p);
    else hipLaunchKernelGGL(gemm_mxfp4_gemv_kernel<false>, dim3(blocks), dim3(256), 0, st, p);
    return check_launch("gemm_mxfp4");
}

template <int BM, int BN, int WM, int WN, int KB>
static int launch_mx4(Mx4Args p, int out_dtype, hipStream_t st) {
    p.tiles_m = (p.M + BM - 1) / BM;
    p.tiles_n = (p.N + BN - 1) / BN;
    const int64_t tiles = (int64_t)p.tiles_m * p.tiles_n;
    if (tiles > 0x7FFFFFFFll) return set_error(CFP8_EINVAL, "gemm_mxfp4: too many tiles");
    constexpr size_t lds = 2 * KB * (BM * 128 + BN * 64 + WN * 256 * ((BN / WN / 16 + 3) / 4));
    static_assert(lds <= 160 * 1024, "two stages must fit LDS");
    const bool f32 = out_dtype == CFP8_OUT_F32;
    static std::atomic<bool> raised[2][64];
    const void* fn = f32 ? reinterpret_cast<const void*>(gemm_mxfp4_kernel<BM, BN, WM, WN, KB, true>)
                         : reinterpret_cast<const void*>(gemm_mxfp4_kernel<BM, BN, WM, WN, KB, false>);
    if (int rc = ensure_lds(fn, lds, raised[f32])) return rc;
    if (out_dtype == CFP8_OUT_F32)
        hipLaunchKernelGGL((gemm_mxfp4_kernel<BM, BN, WM, WN, KB, true>), dim3((unsigned)tiles), dim3(WM * WN * 64), lds, st, p);
    else
        hipLaunchKernelGGL((gemm_mxfp4_kernel<BM, BN, WM, WN, KB, false>), dim3((unsigned)tiles), dim3(WM * WN * 64), lds, st, p);
    return check_launch("gemm_mxfp4");
}

}  // namespace cfp8

extern "C" int cfp8_gemm_mxfp4(const void* a, int64_t ld_a, const float* sa, const void* w, int64_t ld_w, const void* ws,
                               int64_t ld_ws, const int32_t* m_indices, int64_t num_groups, void* out, int64_t ld_out,
                               int out_dtype, int64_t M, int64_t N, int64_t K, void* stream) {
    using namespace cfp8;
    if (M < 0 || N < 0 || K < 0 || num_groups < 0) return set_error(CFP8_EINVAL, "gemm_mxfp4: negative shape");
    if (out_dtype != CFP8_OUT_BF16 && out_dtype != CFP8_OUT_F32) return set_error(CFP8_EINVAL, "gemm_mxfp4: out_dtype must be CFP8_OUT_BF16 or CFP8_OUT_F32");
    if (M == 0 || N == 0) return CFP8_OK;
    if (!a || !sa || !w || !ws || !out) return set_error(CFP8_EINVAL, "gemm_mxfp4: null pointer");
    if (K == 0 || K % 32 || N % 16)
        return set_error(CFP8_EINVAL, "gemm_mxfp4: K=%lld must be a positive multiple of 32 and N=%lld a multiple of 16", (long long)K, (long long)N);
    if (m_indices ? num_groups < 1 : num_groups > 1)
        return set_error(CFP8_EINVAL, "gemm_mxfp4: num_groups=%lld needs m_indices (and m_indices at least one group)", (long long)num_groups);
    if (m_indices && M % 128) return set_error(CFP8_EINVAL, "gemm_mxfp4: grouped rows M=%lld must be a multiple of 128", (long long)M);
    if (M > 0x7FFFFFFFll || N > 0x7FFFFFFFll || K > 0x7FFFFFFFll || ld_a >= (1ll << 24) || ld_w >= (1ll << 24) || ld_ws >= (1ll << 24))
        return set_error(CFP8_EINVAL, "gemm_mxfp4: shape beyond the supported range (M, N, K < 2^31, pitches < 2^24)");
    if (ld_a < K || ld_a % 16 || ld_w < K / 2 || ld_w % 16 || ld_ws < K / 32 || ld_out < N)
        return set_error(CFP8_EINVAL, "gemm_mxfp4: pitches: ld_a >= K and ld_w >= K / 2 in bytes, both multiples of 16; ld_ws >= K / 32; ld_out >= N");
    if (!aligned16(a) || !aligned16(w)) return set_error(CFP8_EINVAL, "gemm_mxfp4: a and w must be 16-byte aligned");
    const int64_t out_align = out_dtype == CFP8_OUT_F32 ? 16 : 8;
    if ((reinterpret_cast<uintptr_t>(out) % out_align) || (ld_out * (out_dtype == CFP8_OUT_F32 ? 4 : 2)) % out_align)
        return set_error(CFP8_EINVAL, "gemm_mxfp4: out must be aligned to four elements and ld_out a multiple of 4");
    if (int rc = check_device()) return rc;
    Mx4Args p{};
    p.a = static_cast<const uint8_t*>(a);
    p.w = static_cast<const uint8_t*>(w);
    p.ws = static_cast<const uint8_t*>(ws);
    p.sa = sa;
    p.m_indices = m_indices;
    p.out = out;
    p.ld_a = ld_a; p.ld_w = ld_w; p.ld_ws = ld_ws; p.ld_out = ld_out;
    p.M = (int)M; p.N = (int)N; p.K = (int)K;
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (M <= 16 && !m_indices) return launch_mx4_gemv(p, out_dtype, st);
    if (M <= 16) return launch_mx4<16, 64, 1, 4, 2>(p, out_dtype, st);
    // 17..128 tokens on a wide weight: the strip kernel (a narrow weight leaves most CUs without a strip)
    if (M <= 128 && !m_indices && K >= 128 && (N + 79) / 80 >= 128) return M <= 64 ? launch_mx4_strip<64>(p, out_dtype, st) : launch_mx4_strip<128>(p, out_dtype, st);
    if (M <= 64 && !m_indices) {
        // few weight rows: narrow workgroups, so that there are enough of them
        const bool narrow = (N + 15) / 16 <= 512;
        if (M <= 32) return narrow ? launch_mx4_skinny<2, 3>(p, out_dtype, st) : launch_mx4_skinny<2, 5>(p, out_dtype, st);
        return narrow ? launch_mx4_skinny<4, 3>(p, out_dtype, st) : launch_mx4_skinny<4, 5>(p, out_dtype, st);
    }
    if (M <= 32) return launch_mx4<32, 64, 1, 4, 2>(p, out_dtype, st);
    if (M <= 64) return launch_mx4<64, 64, 1, 4, 2>(p, out_dtype, st);
    // 256 x 256 tiles of the direct-to-LDS pipeline once they fill at least half of the GPU
    const bool out16 = (reinterpret_cast<uintptr_t>(out) & 15u) == 0 && (ld_out * (out_dtype == CFP8_OUT_F32 ? 4 : 2)) % 16 == 0;
    if (!m_indices && M % 256 == 0 && N % 256 == 0 && K % 128 == 0 && ld_ws % 4 == 0 && (reinterpret_cast<uintptr_t>(ws) & 3u) == 0 &&
        out16 && (M / 256) * (N / 256) >= 128 && (M / 256) * (N / 256) <= 0x7FFFFFFFll) {
        // One workgroup per CU and equal tiles: the launch runs in rounds of as many tiles as there are CUs, and a last
        // round that is at most half full costs a whole round.  Then the last tile-columns go to a second launch on
        // smaller tiles and the first launch ends on a full round.
        const int64_t tm = M / 256, tn = N / 256, cus = mx4_cu_count(), rem = (tm * tn) % cus;
        const int64_t cut = (rem + tm - 1) / tm;  // tile-columns that hold the partial round
        if (tm * tn > cus && rem > 0 && rem * 2 <= cus && cut < tn) {
            Mx4Args head = p;
            head.N = (int)((tn - cut) * 256);
            if (int rc = launch_mx4_256(head, out_dtype, st)) return rc;
            Mx4Args tail = p;
            tail.N = (int)(cut * 256);
            tail.w = p.w + (int64_t)head.N * ld_w;
            tail.ws = p.ws + (int64_t)head.N * ld_ws;
            tail.out = static_cast<uint8_t*>(out) + (int64_t)head.N * (out_dtype == CFP8_OUT_F32 ? 4 : 2);
            return launch_mx4_128(tail, out_dtype, st);
        }
        return launch_mx4_256(p, out_dtype, st);
    }
    // every other shape with enough 128 x 256 tiles, and the grouped layout: the same pipeline with edges
    // (128 x 512 tiles when that still gives every CU a tile and wastes under an eighth of the last tile-column)
    // (its byte offsets inside a tile reach 463 weight rows: the pitch must stay below 2^23 for 32 bits)
    if (out16 && K >= 128 && ld_w < (1ll << 23) && (M + 127) / 128 * ((N + 511) / 512) >= 256 && (N + 511) / 512 * 512 - N <= N / 8)
        return launch_mx4_128x512(p, out_dtype, st);
    if (out16 && K >= 128 && (M + 127) / 128 * ((N + 255) / 256) >= 64) return launch_mx4_128(p, out_dtype, st);
    return launch_mx4<128, 128, 2, 2, 1>(p, out_dtype, st);
}


namespace cfp8 {
// quant_rowwise.hip
int launch_quant_rowwise(const void* x, int64_t rows, int64_t cols, int64_t ld_x, void* q, int64_t ld_q, float* scales,
                         bool streaming_out, hipStream_t st);
}  // namespace cfp8

extern "C" int cfp8_linear_mxfp4(const void* x, int64_t ld_x, const void* w, int64_t ld_w, const void* ws, int64_t ld_ws,
                                 void* out, int64_t ld_out, int out_dtype, int64_t M, int64_t N, int64_t K, void* workspace,
                                 size_t workspace_bytes, void* stream) {
    using namespace cfp8;
    if (M < 0 || N < 0 || K <= 0) return set_error(CFP8_EINVAL, "linear_mxfp4: bad shape");
    if (M == 0 || N == 0) return CFP8_OK;
    if (!x || !aligned16(x) || ld_x % 8 || ld_x < K) return set_error(CFP8_EINVAL, "linear_mxfp4: bad activation pointer or leading dimension");
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (M <= 4 && K <= 4096) {
        // one launch; the checks of cfp8_gemm_mxfp4 that apply to it
        if (out_dtype != CFP8_OUT_BF16 && out_dtype != CFP8_OUT_F32) return set_error(CFP8_EINVAL, "linear_mxfp4: out_dtype must be CFP8_OUT_BF16 or CFP8_OUT_F32");
        if (!w || !ws || !out) return set_error(CFP8_EINVAL, "linear_mxfp4: null pointer");
        if (K % 32 || N % 16) return set_error(CFP8_EINVAL, "linear_mxfp4: K=%lld must be a multiple of 32 and N=%lld a multiple of 16", (long long)K, (long long)N);
        if (N > 0x7FFFFFFFll || ld_w >= (1ll << 24) || ld_ws >= (1ll << 24) || ld_w < K / 2 || ld_w % 16 || ld_ws < K / 32 || ld_out < N || !aligned16(w))
            return set_error(CFP8_EINVAL, "linear_mxfp4: pitches: ld_w >= K / 2 bytes and a multiple of 16, ld_ws >= K / 32, ld_out >= N; w 16-byte aligned");
        const int64_t out_align = out_dtype == CFP8_OUT_F32 ? 16 : 8;
        if ((reinterpret_cast<uintptr_t>(out) % out_align) || (ld_out * (out_dtype == CFP8_OUT_F32 ? 4 : 2)) % out_align)
            return set_error(CFP8_EINVAL, "linear_mxfp4: out must be aligned to four elements and ld_out a multiple of 4");
        if (int rc = check_device()) return rc;
        Mx4Args p{};
        p.w = static_cast<const uint8_t*>(w);
        p.ws = static_cast<const uint8_t*>(ws);
        p.out = out;
        p.ld_w = ld_w; p.ld_ws = ld_ws; p.ld_out = ld_out;
        p.M = (int)M; p.N = (int)N; p.K = (int)K;
        if (M == 1) return launch_linear_mx4_fused_mr<1>(x, ld_x, p, out_dtype, st);
        if (M == 2) return launch_linear_mx4_fused_mr<2>(x, ld_x, p, out_dtype, st);
        return launch_linear_mx4_fused_mr<4>(x, ld_x, p, out_dtype, st);
    }
    if (!workspace || workspace_bytes < cfp8_linear_workspace_bytes(M, K))
        return set_error(CFP8_EWORKSPACE, "linear_mxfp4: workspace of %zu bytes needed, %zu given", cfp8_linear_workspace_bytes(M, K), workspace_bytes);
    if (reinterpret_cast<uintptr_t>(workspace) & 255u) return set_error(CFP8_EINVAL, "linear_mxfp4: workspace must be 256-byte aligned");
    uint8_t* qx = static_cast<uint8_t*>(workspace);
    float* sx = reinterpret_cast<float*>(qx + (((size_t)M * (size_t)K + 255) & ~(size_t)255));
    if (int rc = check_device()) return rc;
    if (int rc = launch_quant_rowwise(x, M, K, ld_x, qx, K, sx, false, st)) return rc;
    return cfp8_gemm_mxfp4(qx, K, sx, w, ld_w, ws, ld_ws, nullptr, 0, out, ld_out, out_dtype, M, N, K, stream);
}
