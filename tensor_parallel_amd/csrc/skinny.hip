// Rank-shard Linear for decode-sized M (M <= 64): weight streaming, HBM-bound.
//
// Three kernels:
//   skinny_kernel (4 <= M <= 32, int8 weights up to 64): a block owns 16 output columns (16 rows of w; for the
//     SiLU-gated pair 16 gate rows + 16 up rows) and splits K over its wavefronts in chunks of 256 bytes of every
//     w row. v_mfma_f32_16x16x32 does both the multiply and the reduction over K, so no cross-lane shuffles are
//     needed. Partial sums of the wavefronts meet in LDS; the epilogue applies scale, outliers, bias, activation
//     and stores 16 consecutive columns per row.
//   skinny_resident_kernel (9 <= M <= 16, 16-bit weights, several weight tiles per CU): the same products, but a
//     block stays on its CU, keeps its x fragments in registers and walks a range of output columns.
//   gemv_kernel (M <= 3): one wavefront per output column, v_dot2 products, x in LDS.
//
// The weight is either the activation dtype (bf16/f16) or int8 (weight-only quantisation: converted to
// the activation dtype in registers, exact for |q| <= 128).
#include "common.h"

#include <stdlib.h>
#include <mutex>
#include <type_traits>

namespace tpamd {
namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;

enum { SK_LINEAR = 0, SK_SWIGLU = 1 };
constexpr int SK_WAVES = 8;
constexpr int SK_THREADS = SK_WAVES * 64;

struct SkinnyParams {
    const char *x;
    const char *w;
    const char *w2;
    const char *bias;
    const float *scale;        // int8 path: per output row
    const int *outlier_idx;    // int8 path
    const char *w_out;         // int8 path: [N, n_out] in activation dtype
    const char *addend;        // linear: added to the rounded result, or NULL
    char *y;
    int M, N, K;
    int n_out;
    int64_t ldx, ldw, ldy, ld_wout, ldadd;
    int act;
};

template <int DT>
__device__ __forceinline__ f32x4 mfma16(uint4 a, uint4 b, f32x4 c) {
    if constexpr (DT == TPAMD_BF16)
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
    else
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
}

// One output element from its fp32 sums (s1 = the up sum of a gated pair): the reference's op chain with its
// roundings to the tensor dtype (gate and up products, SiLU, product), or bias and activation.
template <int DT, int MODE>
__device__ __forceinline__ void skinny_store_output(const SkinnyParams &p, float s0, float s1, int m, int n) {
    uint16_t out;
    if constexpr (MODE == SK_SWIGLU) {
        const float gv = half_to_f32<DT>(f32_to_half<DT>(s0));
        const float u = half_to_f32<DT>(f32_to_half<DT>(s1));
        const float sl = half_to_f32<DT>(f32_to_half<DT>(silu_f32(gv)));
        out = f32_to_half<DT>(sl * u);
    } else {
        float v = s0;
        if (p.bias) v += half_to_f32<DT>(reinterpret_cast<const uint16_t *>(p.bias)[n]);
        if (p.act == TPAMD_ACT_GELU) v = gelu_erf(v);
        out = f32_to_half<DT>(v);
        if (p.addend != nullptr)  // one step of the sum over rank partials: both operands in the tensor dtype
            out = f32_to_half<DT>(half_to_f32<DT>(out) + half_to_f32<DT>(reinterpret_cast<const uint16_t *>(p.addend)[static_cast<int64_t>(m) * p.ldadd + n]));
    }
    reinterpret_cast<uint16_t *>(p.y)[static_cast<int64_t>(m) * p.ldy + n] = out;
}

// W8 = weight is int8. MT = number of 16-row tiles of x (M <= 16*MT). MODE = SK_LINEAR / SK_SWIGLU.
//
// Fetching. The MFMA row operand wants lane l to hold 16 bytes of row l%16 at K slot l/16; loading it that way
// makes every load instruction touch 16 rows x 64 bytes, and the pace of such a kernel is set by the number of
// half-line requests, not by bytes (measured: 1.5-2x slower). So a load instruction here fetches 8 rows x 128
// contiguous bytes (whole cache lines), and the loaded registers go through a wavefront-private LDS tile:
// written in fetch order, read back in MFMA operand order. x takes the same route when the weights are 16-bit.
//
// CG = groups of 16 output columns per block. With CG > 1 the x fragments of a chunk are reused for CG weight
// tiles, which divides the x bytes a block pulls from L2 per weight byte by CG (what limits this kernel once
// M * 2 bytes of x per K element outweigh the 16 * itemsize(w) bytes of w); the registers this costs are taken
// from the prefetch buffers, so CG > 1 loads a chunk, multiplies it and only then loads the next, and relies on
// the 8 wavefronts of the block being out of phase. CG > 1 needs N % (16 * CG) == 0.
//
// PAIR (gated pair, 16-bit weights, CG = 1): the 16-row weight tile is 8 gate rows followed by the 8 up rows of the
// same 8 output columns, so a block owns 8 columns instead of 16: one accumulator tile instead of two (95 instead of
// 160 registers, so several blocks share a CU) and twice the blocks (N = 5504: 688 instead of 344 for 256 CUs).
// NW = wavefronts per block.
template <int DT, bool W8, int MT, int MODE, int CG, int NW = SK_WAVES, bool PAIR = false>
__global__ __launch_bounds__(NW * 64) void skinny_kernel(SkinnyParams p) {
    static_assert(!PAIR || (MODE == SK_SWIGLU && CG == 1 && !W8), "PAIR is the gated pair with 16-bit weights");
    constexpr int NMAT = (MODE == SK_SWIGLU && !PAIR) ? 2 : 1;
    constexpr int NA = NMAT * CG;             // weight tiles per chunk: index a = cg * NMAT + matrix
    constexpr bool PRE = CG == 1;             // double-buffered loads
    constexpr int LANE_K = W8 ? 64 : 32;      // K elements per lane per chunk (64 bytes of w)
    constexpr int CHUNK_K = LANE_K * 4;       // K elements per chunk
    constexpr int WV = 4;                     // 16-byte loads of w per lane per chunk
    constexpr int XV = LANE_K / 8;            // 16-byte loads of x per lane per chunk per m-tile

    constexpr int TROW = 272;                 // staged row pitch: 256 bytes + 16 pad
    __shared__ float red[NW][NMAT][MT][4][64];
    __shared__ __align__(16) char stage_all[NW][16 * TROW];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int lr = lane & 15, lg = lane >> 4;
    const int n0 = blockIdx.x * (PAIR ? 8 : 16 * CG);
    const int64_t cg_stride = static_cast<int64_t>(16) * p.ldw * (W8 ? 1 : 2);  // bytes from one column group to the next

    int wrow = n0 + lr;
    wrow = wrow < p.N ? wrow : p.N - 1;
    const int wbytes = W8 ? 1 : 2;
    const char *wp[2];
    const char *wp2[2];
    (void)wp2;
    // fetch order: load i of a chunk covers rows (lane/8) + 8*(i&1), bytes (i/2)*128 + (lane%8)*16 of the chunk's 256
    const int crow = lane >> 3, cpiece = lane & 7;
    char *stage = stage_all[wave];
    const int st_wr = crow * TROW + cpiece * 16;   // + (i&1)*8*TROW + (i/2)*128
    const int st_rd = lr * TROW + lg * 16;         // + v*64
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        int r = n0 + crow + (PAIR ? 0 : 8 * h);  // PAIR: tile rows 0-7 are gate rows, 8-15 the up rows of the same columns
        r = r < p.N ? r : p.N - 1;
        wp[h] = (PAIR && h == 1 ? p.w2 : p.w) + static_cast<int64_t>(r) * p.ldw * wbytes + cpiece * 16;
        if constexpr (NMAT == 2) wp2[h] = p.w2 + static_cast<int64_t>(r) * p.ldw * wbytes + cpiece * 16;
    }
    bool xok[MT];
#pragma unroll
    for (int t = 0; t < MT; ++t) {
        const int m = t * 16 + lr;
        xok[t] = m < p.M;
    }
    const char *xpc[MT][2];
    bool xokc[MT][2];
#pragma unroll
    for (int t = 0; t < MT; ++t)
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const int m = t * 16 + crow + 8 * h;
            xokc[t][h] = m < p.M;
            xpc[t][h] = p.x + static_cast<int64_t>(xokc[t][h] ? m : 0) * p.ldx * 2 + cpiece * 16;
        }

    f32x4 acc[NA][MT];
#pragma unroll
    for (int a = 0; a < NA; ++a)
#pragma unroll
        for (int t = 0; t < MT; ++t) acc[a][t] = f32x4{0.f, 0.f, 0.f, 0.f};

    const int nchunks = (p.K + CHUNK_K - 1) / CHUNK_K;

    // Register double buffers for the weights (and for x when it is small enough). Buffer indices are
    // compile-time constants so that the arrays stay in registers.
    constexpr bool XPRE = PRE && MT * XV <= 8;
    uint4 wv[PRE ? 2 : 1][NA][WV];
    uint4 xv[XPRE ? 2 : 1][MT][XV];
    auto load_w = [&](auto bufc, int c) {
        constexpr int buf = decltype(bufc)::value;
        const int64_t off = static_cast<int64_t>(c) * CHUNK_K * wbytes;
#pragma unroll
        for (int a = 0; a < NA; ++a)
#pragma unroll
            for (int i = 0; i < WV; ++i) {
                const int byte = (i >> 1) * 128 + cpiece * 16;            // inside the chunk's 256 bytes of the row
                // Past the end of K the row's first bytes are fetched instead (always a load, never a branch, and nothing
                // is done to the value until it is multiplied): x is zero there, so the product is too.
                const bool ok = c * CHUNK_K + byte / wbytes < p.K;
                const char *base = (a % NMAT == 0 ? wp[i & 1] : wp2[i & 1]) + (a / NMAT) * cg_stride;
                wv[buf][a][i] = nt_load_u4(ok ? base + off + (i >> 1) * 128 : base - cpiece * 16);
            }
    };
    // registers in fetch order -> registers in MFMA operand order, through this wavefront's LDS tile
    auto transpose = [&](uint4 *r) {
#pragma unroll
        for (int i = 0; i < WV; ++i) *reinterpret_cast<uint4 *>(stage + st_wr + (i & 1) * 8 * TROW + (i >> 1) * 128) = r[i];
        __builtin_amdgcn_wave_barrier();
        asm volatile("" ::: "memory");
        if constexpr (W8) {
            // (only x takes this branch with int8 weights, see compute) operand order that meets the int8 tile:
            // lane slot lg holds k = v'*64 + lg*16 + h*8 .. +8 for register 2*v' + h of the 256-element chunk
#pragma unroll
            for (int v = 0; v < WV; ++v) r[v] = *reinterpret_cast<const uint4 *>(stage + lr * TROW + (v >> 1) * 128 + lg * 32 + (v & 1) * 16);
        } else {
#pragma unroll
            for (int v = 0; v < WV; ++v) r[v] = *reinterpret_cast<const uint4 *>(stage + st_rd + v * 64);
        }
        __builtin_amdgcn_wave_barrier();
        asm volatile("" ::: "memory");
    };
    auto transpose_w = [&](uint4 *r) {
#pragma unroll
        for (int i = 0; i < WV; ++i) *reinterpret_cast<uint4 *>(stage + st_wr + (i & 1) * 8 * TROW + (i >> 1) * 128) = r[i];
        __builtin_amdgcn_wave_barrier();
        asm volatile("" ::: "memory");
#pragma unroll
        for (int v = 0; v < WV; ++v) r[v] = *reinterpret_cast<const uint4 *>(stage + st_rd + v * 64);
        __builtin_amdgcn_wave_barrier();
        asm volatile("" ::: "memory");
    };
    // x in fetch order too: load i covers rows (lane/8) + 8*(i&1), bytes (i/2)*128 + (lane%8)*16 of the chunk's
    // 256 (16-bit weights) or 512 (int8 weights) bytes of the row
    auto load_x = [&](auto bufc, int c) {
        constexpr int buf = decltype(bufc)::value;
        const int64_t xoff = static_cast<int64_t>(c) * CHUNK_K * 2;
#pragma unroll
        for (int t = 0; t < MT; ++t)
#pragma unroll
            for (int i = 0; i < XV; ++i) {
                const int byte = (i >> 1) * 128 + cpiece * 16;
                const bool ok = xokc[t][i & 1] && c * CHUNK_K + byte / 2 < p.K;
                // requested unconditionally (the first bytes of x when out of range) and zeroed in compute(): a branch
                // around a load, or a use right behind it, makes every later wait drain all loads
                xv[buf][t][i] = *reinterpret_cast<const uint4 *>(ok ? xpc[t][i & 1] + xoff + (i >> 1) * 128 : p.x);
            }
    };
    auto compute = [&](auto bufc, int c) {
        constexpr int buf = decltype(bufc)::value;
        constexpr int xb = XPRE ? buf : 0;
#pragma unroll
        for (int a = 0; a < NA; ++a) transpose_w(wv[PRE ? buf : 0][a]);
#pragma unroll
        for (int t = 0; t < MT; ++t) {
#pragma unroll
            for (int i = 0; i < XV; ++i) {
                const int byte = (i >> 1) * 128 + cpiece * 16;
                const bool ok = xokc[t][i & 1] && c * CHUNK_K + byte / 2 < p.K;
                const uint4 v = xv[xb][t][i];
                xv[xb][t][i] = make_uint4(ok ? v.x : 0u, ok ? v.y : 0u, ok ? v.z : 0u, ok ? v.w : 0u);
            }
            transpose(&xv[xb][t][0]);
            if constexpr (W8) transpose(&xv[xb][t][4]);  // second 256 bytes of the row's chunk
        }
#pragma unroll
        for (int a = 0; a < NA; ++a) {
            if constexpr (W8) {
#pragma unroll
                for (int v = 0; v < WV; ++v) {  // 16 int8 -> two operands of 8
                    const uint4 q = wv[PRE ? buf : 0][a][v];
                    uint4 w0, w1;
                    cvt_i8x4<DT>(q.x, w0.x, w0.y);
                    cvt_i8x4<DT>(q.y, w0.z, w0.w);
                    cvt_i8x4<DT>(q.z, w1.x, w1.y);
                    cvt_i8x4<DT>(q.w, w1.z, w1.w);
#pragma unroll
                    for (int t = 0; t < MT; ++t) {
                        acc[a][t] = mfma16<DT>(w0, xv[xb][t][2 * v], acc[a][t]);
                        acc[a][t] = mfma16<DT>(w1, xv[xb][t][2 * v + 1], acc[a][t]);
                    }
                }
            } else {
#pragma unroll
                for (int v = 0; v < WV; ++v)
#pragma unroll
                    for (int t = 0; t < MT; ++t) acc[a][t] = mfma16<DT>(wv[PRE ? buf : 0][a][v], xv[xb][t][v], acc[a][t]);
            }
        }
    };
    static_assert(W8 ? (XV == 2 * WV) : (XV == WV), "operand chunking");
    using B0 = std::integral_constant<int, 0>;
    using B1 = std::integral_constant<int, 1>;

    // This wavefront's chunks are wave, wave + SK_WAVES, ... The next chunk's loads are issued before the
    // current one is multiplied. Loads return in order, so whatever the multiply waits for is issued
    // ahead of the prefetch.
    // A prefetch past the wavefront's last chunk is a chunk past the end of K (loads of the rows' first bytes): every
    // pass through the loop issues the same loads, so each wait counts exactly the loads behind the one it needs.
    auto in_k = [&](int c) { return c < nchunks ? c : nchunks; };
    if constexpr (PRE) {
        int c = wave;
        load_w(B0{}, in_k(c));
        if constexpr (XPRE) load_x(B0{}, in_k(c));
        while (c < nchunks) {
            int cn = c + NW;
            if constexpr (!XPRE) load_x(B0{}, c);
            load_w(B1{}, in_k(cn));
            if constexpr (XPRE) load_x(B1{}, in_k(cn));
            compute(B0{}, c);
            c = cn;
            if (c >= nchunks) break;
            cn = c + NW;
            if constexpr (!XPRE) load_x(B0{}, c);
            load_w(B0{}, in_k(cn));
            if constexpr (XPRE) load_x(B0{}, in_k(cn));
            compute(B1{}, c);
            c = cn;
        }
    } else {
        for (int c = wave; c < nchunks; c += NW) {
            load_w(B0{}, c);
            load_x(B0{}, c);
            compute(B0{}, c);
        }
    }

    // ---- int8 path: the outlier columns, spread over the wavefronts in groups of 32 ----------------
    if constexpr (W8) {
        f32x4 acc_o[CG][MT];
#pragma unroll
        for (int g = 0; g < CG; ++g)
#pragma unroll
            for (int t = 0; t < MT; ++t) acc_o[g][t] = f32x4{0.f, 0.f, 0.f, 0.f};
        const uint16_t *xo = reinterpret_cast<const uint16_t *>(p.x);
        const uint16_t *wo = reinterpret_cast<const uint16_t *>(p.w_out);
        for (int s = wave; s * 32 < p.n_out; s += NW) {
            uint32_t wq[CG][4];
            uint32_t xq[MT][4];
#pragma unroll
            for (int g = 0; g < CG; ++g) wq[g][0] = wq[g][1] = wq[g][2] = wq[g][3] = 0;
#pragma unroll
            for (int t = 0; t < MT; ++t) xq[t][0] = xq[t][1] = xq[t][2] = xq[t][3] = 0;
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const int o = s * 32 + lg * 8 + j;
                if (o < p.n_out) {
                    const int col = p.outlier_idx[o];
#pragma unroll
                    for (int g = 0; g < CG; ++g) {
                        const int wr = CG == 1 ? wrow : n0 + g * 16 + lr;  // CG > 1: every row of the block exists
                        const uint32_t wval = wo[static_cast<int64_t>(wr) * p.ld_wout + o];
                        wq[g][j >> 1] |= wval << ((j & 1) * 16);
                    }
#pragma unroll
                    for (int t = 0; t < MT; ++t)
                        if (xok[t]) {
                            const uint32_t xval = xo[static_cast<int64_t>(t * 16 + lr) * p.ldx + col];
                            xq[t][j >> 1] |= xval << ((j & 1) * 16);
                        }
                }
            }
#pragma unroll
            for (int g = 0; g < CG; ++g)
#pragma unroll
                for (int t = 0; t < MT; ++t)
                    acc_o[g][t] = mfma16<DT>(make_uint4(wq[g][0], wq[g][1], wq[g][2], wq[g][3]),
                                             make_uint4(xq[t][0], xq[t][1], xq[t][2], xq[t][3]), acc_o[g][t]);
        }
        // fold the per-row scale in before the partial sums meet, then add the outlier product.
        // D[n_local][m_local]: lane -> m_local = lr, register i -> n_local = 4*lg + i
#pragma unroll
        for (int g = 0; g < CG; ++g) {
            float sc[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                int n = n0 + g * 16 + lg * 4 + i;
                n = n < p.N ? n : p.N - 1;
                sc[i] = p.scale[n];
            }
#pragma unroll
            for (int t = 0; t < MT; ++t)
#pragma unroll
                for (int i = 0; i < 4; ++i) acc[g * NMAT][t][i] = acc[g * NMAT][t][i] * sc[i] + acc_o[g][t][i];
        }
    }

    // ---- cross-wave reduction, one column group at a time through the same LDS array ------------------
#pragma unroll
    for (int g = 0; g < CG; ++g) {
        if (g > 0) __syncthreads();
#pragma unroll
        for (int a = 0; a < NMAT; ++a)
#pragma unroll
            for (int t = 0; t < MT; ++t)
#pragma unroll
                for (int i = 0; i < 4; ++i) red[wave][a][t][i][lane] = acc[g * NMAT + a][t][i];
        __syncthreads();

        // thread e -> output (m = e / 16, n_local = e % 16): 16 consecutive threads store one 32-byte row piece
        for (int e = tid; e < MT * 256; e += NW * 64) {
            const int m = e >> 4, nl = e & 15;
            if (PAIR && nl >= 8) continue;  // tile rows 8-15 are the up sums of columns 0-7
            const int n = n0 + g * 16 + nl;
            if (m >= p.M || n >= p.N) continue;
            const int t = m >> 4, src_lane = (nl >> 2) * 16 + (m & 15), i = nl & 3;
            float s0 = 0.f, s1 = 0.f;
#pragma unroll
            for (int w = 0; w < NW; ++w) {
                s0 += red[w][0][t][i][src_lane];
                if constexpr (NMAT == 2) s1 += red[w][1][t][i][src_lane];
                if constexpr (PAIR) s1 += red[w][0][t][i][src_lane + 32];  // row nl + 8: two lane groups further on
            }
            skinny_store_output<DT, MODE>(p, s0, s1, m, n);
        }
    }
}

// f(integral_constant<int, 0>) ... f(integral_constant<int, N - 1>): loop indices that stay compile-time constants
template <int N, int J = 0, class F>
__device__ __forceinline__ void static_for(F &&f) {
    if constexpr (J < N) {
        f(std::integral_constant<int, J>{});
        static_for<N, J + 1>(f);
    }
}

// ---- x-resident form of the weight-streaming kernel ------------------------------------------------------
// When there are several 16-row weight tiles per CU, the block above re-reads its K slices of x for every tile, and
// from 8 rows on those bytes weigh as much as the weights in what a CU can take in. Here a block stays on its CU and
// walks a contiguous range of output columns (the N columns are split evenly over the blocks; the last tile of a
// range is partly masked): wavefront w keeps the x fragments of its chunks w, w + 8, ... in registers for the whole
// launch (NCH chunks: K <= NCH * NW * 128). Weights go through DEPTH register slots per wavefront: as soon as a chunk
// has been multiplied, the chunk DEPTH further on in the stream (of this or the next tile) is requested into its slot,
// so a wavefront always has about DEPTH * 4 KiB of weights in flight.
// Partial sums of the wavefronts meet in LDS once per tile (two buffers, one barrier per tile).
// MODE SK_SWIGLU: the tile is 8 gate rows + the 8 up rows of the same 8 columns (16-bit weights only).
template <int DT, int MODE, int NW, int NCH, int DEPTH>
__global__ __launch_bounds__(NW * 64) void skinny_resident_kernel(SkinnyParams p) {
    static_assert(NCH % DEPTH == 0, "a chunk's slot must not depend on the tile");
    constexpr bool PAIR = MODE == SK_SWIGLU;
    constexpr int COLS = PAIR ? 8 : 16;
    constexpr int CHUNK_K = 128;                // K elements per chunk: 256 bytes of every row
    constexpr int TROW = 272;                   // staged row pitch: 256 bytes + 16 pad
    __shared__ float red[2][NW][4][64];
    __shared__ __align__(16) char stage_all[NW][16 * TROW];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int lr = lane & 15, lg = lane >> 4;
    const int crow = lane >> 3, cpiece = lane & 7;
    char *stage = stage_all[wave];
    const int st_wr = crow * TROW + cpiece * 16;   // + (i&1)*8*TROW + (i/2)*128
    const int st_rd = lr * TROW + lg * 16;         // + v*64
    const int nchunks = (p.K + CHUNK_K - 1) / CHUNK_K;
    const int col_begin = static_cast<int>(static_cast<int64_t>(blockIdx.x) * p.N / gridDim.x);
    const int col_end = static_cast<int>(static_cast<int64_t>(blockIdx.x + 1) * p.N / gridDim.x);

    // registers in fetch order (load i: rows lane/8 + 8*(i&1), bytes (i/2)*128 + (lane%8)*16 of the chunk's 256)
    // -> registers in MFMA operand order, through this wavefront's LDS tile
    auto transpose = [&](uint4 *r) {
#pragma unroll
        for (int i = 0; i < 4; ++i) *reinterpret_cast<uint4 *>(stage + st_wr + (i & 1) * 8 * TROW + (i >> 1) * 128) = r[i];
        __builtin_amdgcn_wave_barrier();
        asm volatile("" ::: "memory");
#pragma unroll
        for (int v = 0; v < 4; ++v) r[v] = *reinterpret_cast<const uint4 *>(stage + st_rd + v * 64);
        __builtin_amdgcn_wave_barrier();
        asm volatile("" ::: "memory");
    };

    // x: this wavefront's chunks, resident
    uint4 xq[NCH][4];
#pragma unroll
    for (int j = 0; j < NCH; ++j) {
        const int c = wave + j * NW;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int m = crow + 8 * (i & 1);
            const int byte = (i >> 1) * 128 + cpiece * 16;
            const bool ok = c < nchunks && m < p.M && c * CHUNK_K + byte / 2 < p.K;
            // requested unconditionally (the first bytes of x when out of range) and zeroed where the value is used:
            // a branch around a load, or a use right behind it, makes every later wait drain all loads
            xq[j][i] = *reinterpret_cast<const uint4 *>(p.x + (ok ? static_cast<int64_t>(m) * p.ldx * 2 + static_cast<int64_t>(c) * (CHUNK_K * 2) + byte : 0));
        }
    }
    auto zero_x_out_of_range = [&](int j) __attribute__((always_inline)) {
        const int c = wave + j * NW;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int m = crow + 8 * (i & 1);
            const int byte = (i >> 1) * 128 + cpiece * 16;
            const bool ok = c < nchunks && m < p.M && c * CHUNK_K + byte / 2 < p.K;
            const uint4 v = xq[j][i];
            xq[j][i] = make_uint4(ok ? v.x : 0u, ok ? v.y : 0u, ok ? v.z : 0u, ok ? v.w : 0u);
        }
    };

    uint4 wv[DEPTH][4];
    // chunk j of the tile whose first column is n0 (columns from n_valid on do not belong to this block)
    auto load_w = [&](auto jc, int n0, int n_valid) {
        constexpr int j = decltype(jc)::value;
        const int c = wave + j * NW;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int h = i & 1;
            const int col = PAIR ? crow : crow + 8 * h;              // column of the tile this row belongs to
            // Out of range, a load all the same: a column of another block reads the tile's first row again and one past the
            // last tile the matrix's last row (cached; such sums are never stored), a chunk past K reads its own row's first
            // bytes (x is zero there, so what a column adds up never depends on another row's weights).
            int row = col < n_valid ? n0 + col : n0;
            row = row < p.N ? row : p.N - 1;
            const char *base = (PAIR && h == 1 ? p.w2 : p.w) + static_cast<int64_t>(row) * p.ldw * 2;
            const int byte = (i >> 1) * 128 + cpiece * 16;
            const bool in_k = c < nchunks && c * CHUNK_K + byte / 2 < p.K;
            wv[j % DEPTH][i] = nt_load_u4(in_k ? base + static_cast<int64_t>(c) * (CHUNK_K * 2) + byte : base);
        }
    };
    auto for_each_chunk = [&](auto &&f) { static_for<NCH>(f); };

    int n0 = col_begin;
    static_for<DEPTH>([&](auto jc) { load_w(jc, n0, col_end - n0); });
#pragma unroll
    for (int j = 0; j < NCH; ++j) {
        zero_x_out_of_range(j);
        transpose(xq[j]);
    }

    for (int t = 0; n0 < col_end; ++t, n0 += COLS) {
        const int n_valid = col_end - n0 < COLS ? col_end - n0 : COLS;
        const int n_next = n0 + COLS;
        f32x4 acc = f32x4{0.f, 0.f, 0.f, 0.f};
        for_each_chunk([&](auto jc) {
            constexpr int j = decltype(jc)::value;
            // (chunks past the end of K are zeros on both sides: multiplied anyway, so that every slot is refilled
            // at the same place in every wavefront)
            transpose(wv[j % DEPTH]);
#pragma unroll
            for (int v = 0; v < 4; ++v) acc = mfma16<DT>(wv[j % DEPTH][v], xq[j][v], acc);
            if constexpr (j + DEPTH < NCH) load_w(std::integral_constant<int, j + DEPTH>{}, n0, n_valid);
            else load_w(std::integral_constant<int, j + DEPTH - NCH>{}, n_next, col_end - n_next);  // no further tile: n_valid <= 0
        });
        float(*rd)[4][64] = red[t & 1];
#pragma unroll
        for (int i = 0; i < 4; ++i) rd[wave][i][lane] = acc[i];
        __syncthreads();
        // thread e -> output (m = e / 16, n_local = e % 16)
        if (tid < 256) {
            const int m = tid >> 4, nl = tid & 15;
            if (m < p.M && nl < n_valid) {  // pair: tile rows 8-15 are the up sums of columns 0-7, n_valid <= 8
                const int n = n0 + nl;
                const int src_lane = (nl >> 2) * 16 + m, i = nl & 3;
                float s0 = 0.f, s1 = 0.f;
#pragma unroll
                for (int w = 0; w < NW; ++w) {
                    s0 += rd[w][i][src_lane];
                    if constexpr (PAIR) s1 += rd[w][i][src_lane + 32];  // row nl + 8: two lane groups further on
                }
                skinny_store_output<DT, MODE>(p, s0, s1, m, n);
            }
        }
    }
}

// ---- int8 weights, 12 <= M <= 64: K split over blocks, x resident -----------------------------------------
// With int8 weights x weighs 2 * M bytes per K element against 16 for the 16 weight rows of a tile, and a block
// that covers all of K has to pull all of x through its CU for every tile: at M = 32 that is as many bytes as the
// weights themselves. Here the grid is (column ranges, K splits): wavefront w of a block owns NCH chunks of 256 K
// elements (a split is NCH * 2048 elements), keeps their x fragments in registers (NCH x MT tiles of 16 rows x 8
// registers: 128 registers for MT * NCH = 4) and walks the 16-row weight tiles of the block's column range, so per
// CU x is read once per split while the weights of 256 or more columns stream past. A chunk's registers are refilled
// with the same chunk of the next tile as soon as it has been handed to the MFMA operands. Partial sums of the 8
// wavefronts meet in LDS once per tile (two buffers, one barrier per tile), are scaled per output row, get the
// outlier product added (split 0 only) and go to a [split][M][N] fp32 array; skinny_w8_finish_kernel adds the
// splits, bias and activation. DIRECT (a single split): bias, activation and the store to y happen here.
template <int DT, int MT, int NCH, bool DIRECT>
__global__ __launch_bounds__(SK_THREADS) void skinny_w8_split_kernel(SkinnyParams p, float *part, int cols_per_block) {
    constexpr int NW = SK_WAVES;
    constexpr int CHUNK_K = 256;                // K elements per chunk: 256 bytes of a weight row, 512 of an x row
    constexpr int TROW = 272;
    __shared__ float red[2][NW][MT][4][64];
    __shared__ __align__(16) char stage_all[NW][16 * TROW];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int lr = lane & 15, lg = lane >> 4;
    const int crow = lane >> 3, cpiece = lane & 7;
    char *stage = stage_all[wave];
    const int st_wr = crow * TROW + cpiece * 16;   // + (i&1)*8*TROW + (i/2)*128
    const int st_rd = lr * TROW + lg * 16;         // + v*64
    const uint4 zero4 = make_uint4(0, 0, 0, 0);
    const int split = blockIdx.y;
    const int col_begin = blockIdx.x * cols_per_block;
    const int col_end = col_begin + cols_per_block < p.N ? col_begin + cols_per_block : p.N;
    // first K element of this wavefront's chunk j
    auto chunk_k0 = [&](int j) { return (static_cast<int64_t>(split * NCH + j) * NW + wave) * CHUNK_K; };

    auto stage_in = [&](const uint4 *r) {
#pragma unroll
        for (int i = 0; i < 4; ++i) *reinterpret_cast<uint4 *>(stage + st_wr + (i & 1) * 8 * TROW + (i >> 1) * 128) = r[i];
        __builtin_amdgcn_wave_barrier();
        asm volatile("" ::: "memory");
    };
    auto stage_done = [&]() {
        __builtin_amdgcn_wave_barrier();
        asm volatile("" ::: "memory");
    };

    // x fragments of this wavefront's chunks, in the operand order that meets the int8 tile: lane slot lg holds
    // k = v*64 + lg*16 + h*8 .. +8 in register 2*v + h
    uint4 xq[NCH][MT][8];
#pragma unroll
    for (int j = 0; j < NCH; ++j)
#pragma unroll
        for (int t = 0; t < MT; ++t)
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const int m = t * 16 + crow + 8 * (i & 1);
                const int byte = (i >> 1) * 128 + cpiece * 16;
                const int64_t k0 = chunk_k0(j);
                const bool ok = m < p.M && k0 + byte / 2 < p.K;
                // always a load (the first bytes of x when out of range), zeroed below where it is first used
                xq[j][t][i] = *reinterpret_cast<const uint4 *>(p.x + (ok ? static_cast<int64_t>(m) * p.ldx * 2 + k0 * 2 + byte : 0));
            }
#pragma unroll
    for (int j = 0; j < NCH; ++j)
#pragma unroll
        for (int t = 0; t < MT; ++t)
#pragma unroll
            for (int half = 0; half < 2; ++half) {
#pragma unroll
                for (int i = half * 4; i < half * 4 + 4; ++i) {
                    const int m = t * 16 + crow + 8 * (i & 1);
                    const int byte = (i >> 1) * 128 + cpiece * 16;
                    const bool ok = m < p.M && chunk_k0(j) + byte / 2 < p.K;
                    const uint4 v = xq[j][t][i];
                    xq[j][t][i] = make_uint4(ok ? v.x : 0u, ok ? v.y : 0u, ok ? v.z : 0u, ok ? v.w : 0u);
                }
                stage_in(&xq[j][t][half * 4]);
#pragma unroll
                for (int v = 0; v < 4; ++v)
                    xq[j][t][half * 4 + v] = *reinterpret_cast<const uint4 *>(stage + lr * TROW + (v >> 1) * 128 + lg * 32 + (v & 1) * 16);
                stage_done();
            }

    // outlier columns (split 0): wavefront w takes outliers 32w .. 32w + 31 (n_out <= 256); its x values once
    const bool outl = split == 0 && wave * 32 < p.n_out;
    uint4 xo[MT];
#pragma unroll
    for (int t = 0; t < MT; ++t) {
        uint32_t q[4] = {0, 0, 0, 0};
        if (outl) {
            const uint16_t *xs = reinterpret_cast<const uint16_t *>(p.x);
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const int o = wave * 32 + lg * 8 + j;
                if (o < p.n_out && t * 16 + lr < p.M) {
                    const uint32_t xval = xs[static_cast<int64_t>(t * 16 + lr) * p.ldx + p.outlier_idx[o]];
                    q[j >> 1] |= xval << ((j & 1) * 16);
                }
            }
        }
        xo[t] = make_uint4(q[0], q[1], q[2], q[3]);
    }

    uint4 wv[NCH][4];
    auto load_w = [&](auto jc, int n0) {
        constexpr int j = decltype(jc)::value;
        const int64_t k0 = chunk_k0(j);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int row = n0 + crow + 8 * (i & 1);
            const int byte = (i >> 1) * 128 + cpiece * 16;
            // rows of another block and bytes past K: the first bytes of the matrix (x is zero past K, such rows are not stored)
            const bool ok = row < col_end && k0 + byte < p.K;
            wv[j][i] = nt_load_u4(p.w + (ok ? static_cast<int64_t>(row) * p.ldw + k0 + byte : 0));
        }
    };
    static_for<NCH>([&](auto jc) { load_w(jc, col_begin); });

    int t_index = 0;
    for (int n0 = col_begin; n0 < col_end; n0 += 16, ++t_index) {
        f32x4 acc[MT];
#pragma unroll
        for (int t = 0; t < MT; ++t) acc[t] = f32x4{0.f, 0.f, 0.f, 0.f};
        static_for<NCH>([&](auto jc) {
            constexpr int j = decltype(jc)::value;
            stage_in(wv[j]);
            uint4 wt[4];
#pragma unroll
            for (int v = 0; v < 4; ++v) wt[v] = *reinterpret_cast<const uint4 *>(stage + st_rd + v * 64);
            stage_done();
            load_w(jc, n0 + 16);  // past the last tile: every row is out of range
#pragma unroll
            for (int v = 0; v < 4; ++v) {  // 16 int8 -> two operands of 8
                uint4 w0, w1;
                cvt_i8x4<DT>(wt[v].x, w0.x, w0.y);
                cvt_i8x4<DT>(wt[v].y, w0.z, w0.w);
                cvt_i8x4<DT>(wt[v].z, w1.x, w1.y);
                cvt_i8x4<DT>(wt[v].w, w1.z, w1.w);
#pragma unroll
                for (int t = 0; t < MT; ++t) {
                    acc[t] = mfma16<DT>(w0, xq[j][t][2 * v], acc[t]);
                    acc[t] = mfma16<DT>(w1, xq[j][t][2 * v + 1], acc[t]);
                }
            }
        });
        // per-row scale, then the outlier product. D[n_local][m_local]: lane -> m_local = lr, register i -> n_local = 4*lg + i
        float sc[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int n = n0 + lg * 4 + i;
            sc[i] = p.scale[n < p.N ? n : p.N - 1];
        }
        uint4 wo4 = zero4;
        if (outl) {
            const uint16_t *wo = reinterpret_cast<const uint16_t *>(p.w_out);
            const int wr = n0 + lr < p.N ? n0 + lr : p.N - 1;
            uint32_t q[4] = {0, 0, 0, 0};
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const int o = wave * 32 + lg * 8 + j;
                if (o < p.n_out) q[j >> 1] |= static_cast<uint32_t>(wo[static_cast<int64_t>(wr) * p.ld_wout + o]) << ((j & 1) * 16);
            }
            wo4 = make_uint4(q[0], q[1], q[2], q[3]);
        }
        float(*rd)[MT][4][64] = red[t_index & 1];
#pragma unroll
        for (int t = 0; t < MT; ++t) {
            f32x4 v = f32x4{acc[t][0] * sc[0], acc[t][1] * sc[1], acc[t][2] * sc[2], acc[t][3] * sc[3]};
            if (outl) v = mfma16<DT>(wo4, xo[t], v);
#pragma unroll
            for (int i = 0; i < 4; ++i) rd[wave][t][i][lane] = v[i];
        }
        __syncthreads();
        for (int e = tid; e < MT * 256; e += NW * 64) {
            const int m = e >> 4, nl = e & 15, n = n0 + nl;
            if (m >= p.M || n >= col_end) continue;
            const int t = m >> 4, src_lane = (nl >> 2) * 16 + (m & 15), i = nl & 3;
            float sum = 0.f;
#pragma unroll
            for (int w = 0; w < NW; ++w) sum += rd[w][t][i][src_lane];
            if constexpr (DIRECT) skinny_store_output<DT, SK_LINEAR>(p, sum, 0.f, m, n);
            else part[(static_cast<int64_t>(split) * p.M + m) * p.N + n] = sum;
        }
    }
}

// y[m][n] = act(sum over splits of part[split][m][n] + bias[n]); VEC: four consecutive n per thread (N a multiple of 4),
// the planes requested eight at a time and added in plane order
template <int DT, bool VEC>
__global__ __launch_bounds__(256) void skinny_w8_finish_kernel(SkinnyParams p, const float *part, int splits) {
    const int64_t plane = static_cast<int64_t>(p.M) * p.N;
    if constexpr (VEC) {
        const int64_t e = (static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x) * 4;
        if (e >= plane) return;
        const int m = static_cast<int>(e / p.N), n = static_cast<int>(e % p.N);
        f32x4 v = f32x4{0.f, 0.f, 0.f, 0.f};
        int sp = 0;
        for (; sp + 8 <= splits; sp += 8) {
            f32x4 t[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) t[j] = *reinterpret_cast<const f32x4 *>(part + (sp + j) * plane + e);
#pragma unroll
            for (int j = 0; j < 8; ++j) v += t[j];
        }
        for (; sp < splits; ++sp) v += *reinterpret_cast<const f32x4 *>(part + sp * plane + e);
#pragma unroll
        for (int i = 0; i < 4; ++i) skinny_store_output<DT, SK_LINEAR>(p, v[i], 0.f, m, n + i);
    } else {
        const int64_t e = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
        if (e >= plane) return;
        const int m = static_cast<int>(e / p.N), n = static_cast<int>(e % p.N);
        float v = 0.f;
        for (int sp = 0; sp < splits; ++sp) v += part[sp * plane + e];
        skinny_store_output<DT, SK_LINEAR>(p, v, 0.f, m, n);
    }
}

// Launches the finishing pass over [splits][M][N] partial sums.
template <int DT>
int launch_w8_finish(const SkinnyParams &p, const float *part, int splits, hipStream_t s) {
    const int64_t outputs = static_cast<int64_t>(p.M) * p.N;
    if (p.N % 4 == 0) hipLaunchKernelGGL((skinny_w8_finish_kernel<DT, true>), dim3(static_cast<unsigned>((outputs / 4 + 255) / 256)), dim3(256), 0, s, p, part, splits);
    else hipLaunchKernelGGL((skinny_w8_finish_kernel<DT, false>), dim3(static_cast<unsigned>((outputs + 255) / 256)), dim3(256), 0, s, p, part, splits);
    TPAMD_HIP(hipGetLastError());
    return TPAMD_OK;
}

// ---- int8 weights, up to 64 rows: K split over blocks, x of the split resident in LDS, wavefronts own columns ----------
// The grid is (column ranges, K splits of KU * 128 elements [+ blocks for the outlier columns]). A block first stages the
// M rows of x of its K split in LDS in MFMA operand order (slot ((unit * 4 + o) * MT + t) of 1 KiB: lane (m = lane % 16,
// g = lane / 16) holds the 8 elements x[16 t + m][unit * 128 + (o / 2) * 64 + g * 16 + (o % 2) * 8 ...], which is what
// meets the two halves of a 16-byte int8 fragment); that is the only block-wide barrier. After it a wavefront owns every
// NW-th tile of 16 weight rows of the block's column range over the whole split and walks them two at a time: a unit is 128
// bytes of the 32 rows of a pair (four loads of 8 rows x 128 bytes), D units are in flight in registers, a unit goes from
// fetch order to operand order through a wavefront-private LDS tile (rows of 128 bytes, pieces swizzled instead of padded),
// is converted to the activation dtype, and every x operand read from LDS meets both tiles of the pair. Nothing is
// exchanged between wavefronts: a tile's sums are scaled per weight row and stored to the [plane][M][N] fp32 array straight
// from the accumulators (DIRECT, a single plane: bias, activation and the store to y happen here). Every weight load is
// issued unconditionally (past the last tile: the first bytes of the matrix, which stay in cache), so that each wait counts
// exactly the loads issued behind the one it needs. Timed with the products removed the kernel is no faster: its pace is
// set by the weight stream, the staging of x before the first product, and the partial sums (M * N * 4 bytes per plane,
// written here and read again by skinny_w8_finish_kernel, which adds the planes). The outlier columns of x (gathered into
// LDS in operand order, groups of 32) meet w_out in blocks of their own, one tile per wavefront, which fill one more plane.
constexpr int WC_NW = 8, WC_UNIT_K = 128, WC_STAGE = 32 * 128;  // per wavefront: two tiles of 16 staged rows

template <int DT, int MT, int KU, bool DIRECT>
__global__ __launch_bounds__(WC_NW * 64, MT == 1 ? 4 : 1) void skinny_w8_cols_kernel(SkinnyParams p, float *part, int cols_per_block, int k_planes) {
    constexpr int NW = WC_NW;
    extern __shared__ __align__(16) char smem[];
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lr = lane & 15, lg = lane >> 4;
    const int crow = lane >> 3, cpiece = lane & 7;
    const int plane = blockIdx.y;
    const int col_begin = blockIdx.x * cols_per_block;
    const int col_end = col_begin + cols_per_block < p.N ? col_begin + cols_per_block : p.N;
    const int tiles = (col_end - col_begin + 15) / 16;
    const int my_tiles = tiles > wave ? (tiles - wave + NW - 1) / NW : 0;  // tiles wave, wave + NW, ...
    const int pairs = (my_tiles + 1) / 2;

    auto store_tile = [&](const f32x4 (&v)[MT], int n0, int to_plane) __attribute__((always_inline)) {
        // D[n_local][m_local]: lane -> m_local = lr, register i -> n_local = 4 * lg + i
        const int n = n0 + lg * 4;
#pragma unroll
        for (int t = 0; t < MT; ++t) {
            const int m = t * 16 + lr;
            if (m >= p.M) continue;
            if constexpr (DIRECT) {
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    if (n + i < col_end) skinny_store_output<DT, SK_LINEAR>(p, v[t][i], 0.f, m, n + i);
            } else {
                float *dst = part + (static_cast<int64_t>(to_plane) * p.M + m) * p.N + n;
                if (n + 3 < col_end && (p.N & 3) == 0) *reinterpret_cast<f32x4 *>(dst) = v[t];
                else
#pragma unroll
                    for (int i = 0; i < 4; ++i)
                        if (n + i < col_end) dst[i] = v[t][i];
            }
        }
    };

    if (plane >= k_planes) {
        // The outlier plane: x values of the outlier columns in LDS (slot g * MT + t: lane (m, q) holds outliers
        // 32 g + 8 q ... + 8 of row 16 t + m), then one MFMA per tile, group and 16 rows of x. Block (bx, k_planes + j)
        // takes tiles 8 j ... 8 j + 7 of the column range, one per wavefront. Every gather is issued unconditionally
        // from a clamped address, so that the eight of a group are in flight together.
        const int groups = (p.n_out + 31) / 32;
        const uint16_t *xs = reinterpret_cast<const uint16_t *>(p.x);
        for (int sl = wave; sl < groups * MT; sl += NW) {
            const int g = sl / MT, t = sl % MT;
            const int m = t * 16 + lr < p.M ? t * 16 + lr : p.M - 1;
            int idx[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const int o = g * 32 + lg * 8 + j;
                idx[j] = p.outlier_idx[o < p.n_out ? o : p.n_out - 1];
            }
            uint32_t val[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) val[j] = xs[static_cast<int64_t>(m) * p.ldx + idx[j]];
            uint32_t q[4] = {0, 0, 0, 0};
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const bool ok = g * 32 + lg * 8 + j < p.n_out && t * 16 + lr < p.M;
                q[j >> 1] |= (ok ? val[j] : 0u) << ((j & 1) * 16);
            }
            *reinterpret_cast<uint4 *>(smem + (sl * 64 + lane) * 16) = make_uint4(q[0], q[1], q[2], q[3]);
        }
        __syncthreads();
        const uint16_t *wo = reinterpret_cast<const uint16_t *>(p.w_out);
        const int tile = (plane - k_planes) * NW + wave;
        if (tile >= tiles) return;
        const int n0 = col_begin + tile * 16;
        const int wr = n0 + lr < p.N ? n0 + lr : p.N - 1;
        f32x4 acc[MT];
#pragma unroll
        for (int t = 0; t < MT; ++t) acc[t] = f32x4{0.f, 0.f, 0.f, 0.f};
        for (int g = 0; g < groups; ++g) {
            uint32_t val[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const int o = g * 32 + lg * 8 + j;
                val[j] = wo[static_cast<int64_t>(wr) * p.ld_wout + (o < p.n_out ? o : p.n_out - 1)];
            }
            uint32_t q[4] = {0, 0, 0, 0};
#pragma unroll
            for (int j = 0; j < 8; ++j) q[j >> 1] |= (g * 32 + lg * 8 + j < p.n_out ? val[j] : 0u) << ((j & 1) * 16);
            const uint4 a = make_uint4(q[0], q[1], q[2], q[3]);
#pragma unroll
            for (int t = 0; t < MT; ++t)
                acc[t] = mfma16<DT>(a, *reinterpret_cast<const uint4 *>(smem + ((g * MT + t) * 64 + lane) * 16), acc[t]);
        }
        store_tile(acc, n0, k_planes);
        return;
    }

    char *stage = smem + KU * 4 * MT * 1024 + wave * WC_STAGE;
    const int64_t k_begin = static_cast<int64_t>(plane) * (KU * WC_UNIT_K);

    // x of this split first (it comes from L2 and must not queue behind the weights: loads return in order)
    constexpr int XS = KU * 4 * MT / NW;
    uint4 xr[XS];
#pragma unroll
    for (int j = 0; j < XS; ++j) {
        const int sl = wave + j * NW;
        const int t = sl % MT, o = (sl / MT) & 3, u = sl / (4 * MT);
        const int64_t k = k_begin + u * WC_UNIT_K + (o >> 1) * 64 + lg * 16 + (o & 1) * 8;
        const int m = t * 16 + lr;
        const bool ok = m < p.M && k < p.K;
        xr[j] = *reinterpret_cast<const uint4 *>(p.x + (ok ? (static_cast<int64_t>(m) * p.ldx + k) * 2 : 0));
    }

    // weights: unit u of the pair of tiles (2 q, 2 q + 1) of this wavefront into ring slot S; for a tile past the last one the
    // first bytes of the matrix. A slot: [tile A rows 0-7, A rows 8-15, B rows 0-7, B rows 8-15], 128 bytes of each row.
    // The four row addresses of a pair are worked out once (set_pair); a unit is an immediate offset from them. In the last
    // plane of a K that does not fill it, units past the end of K read the first bytes of the matrix instead (x is 0 there).
    // Units in flight per wavefront. Up to 16 rows two of them keep the kernel within 128 registers, so that two blocks
    // fit a CU (64 KiB of LDS each): the blocks of the outlier plane then run beside the others instead of after them
    // (Falcon-40B MLP shard at 2 / 4 / 16 rows: 29.0 + 30.2 / 29.4 + 30.4 / 34.1 + 34.5 -> 26.7 + 28.7 / 27.5 + 29.2 / 32.2 + 33.9 us).
    constexpr int D = MT == 1 ? 2 : 4;
    static_assert(KU % D == 0, "the ring divides a tile");
    uint4 wv[D][4];
    const char *rowp[4];
    const bool k_ragged = k_begin + KU * WC_UNIT_K > p.K;  // uniform over the block
    auto set_pair = [&](int q) __attribute__((always_inline)) {
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const int i = 2 * q + h;
            const int n0 = col_begin + (wave + i * NW) * 16;
            const bool live = i < my_tiles;
            const int r0 = n0 + crow < p.N ? n0 + crow : p.N - 1;
            const int r1 = n0 + crow + 8 < p.N ? n0 + crow + 8 : p.N - 1;
            rowp[2 * h] = p.w + (live ? static_cast<int64_t>(r0) * p.ldw + k_begin : 0) + cpiece * 16;
            rowp[2 * h + 1] = p.w + (live ? static_cast<int64_t>(r1) * p.ldw + k_begin : 0) + cpiece * 16;
        }
    };
    auto issue = [&](auto sc_, auto uc) __attribute__((always_inline)) {
        constexpr int S = decltype(sc_)::value, u = decltype(uc)::value;
        if (k_ragged) {
            const bool in_k = k_begin + u * WC_UNIT_K + cpiece * 16 < p.K;
#pragma unroll
            for (int r = 0; r < 4; ++r) wv[S][r] = nt_load_u4(in_k ? rowp[r] + u * WC_UNIT_K : p.w + cpiece * 16);
        } else {
#pragma unroll
            for (int r = 0; r < 4; ++r) wv[S][r] = nt_load_u4(rowp[r] + u * WC_UNIT_K);
        }
    };
    set_pair(0);
    static_for<D>([&](auto sc_) { issue(sc_, sc_); });

#pragma unroll
    for (int j = 0; j < XS; ++j) {
        const int sl = wave + j * NW;
        const int t = sl % MT, o = (sl / MT) & 3, u = sl / (4 * MT);
        const int64_t k = k_begin + u * WC_UNIT_K + (o >> 1) * 64 + lg * 16 + (o & 1) * 8;
        const bool ok = t * 16 + lr < p.M && k < p.K;
        const uint4 v = xr[j];
        *reinterpret_cast<uint4 *>(smem + (sl * 64 + lane) * 16) = make_uint4(ok ? v.x : 0u, ok ? v.y : 0u, ok ? v.z : 0u, ok ? v.w : 0u);
    }
    __syncthreads();

    // staged rows are 128 bytes, piece c of row r at piece c ^ (r / 2 % 8): conflict-free for the writes (8 rows x 8 pieces)
    // and for the reads (16 rows x 1 piece per quarter wavefront) without padding
    const int wr_off = crow * 128 + ((cpiece ^ (crow >> 1)) * 16);           // rows crow and crow + 8 share r / 2 % 8 ^ 4
    const int wr_off8 = (crow + 8) * 128 + ((cpiece ^ ((crow >> 1) + 4)) * 16);
    int rd_off[2];
#pragma unroll
    for (int v = 0; v < 2; ++v) rd_off[v] = lr * 128 + (((v * 4 + lg) ^ ((lr >> 1) & 7)) * 16);

    for (int q = 0; q < pairs; ++q) {
        f32x4 acc[2][MT];
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
            for (int t = 0; t < MT; ++t) acc[h][t] = f32x4{0.f, 0.f, 0.f, 0.f};
        // the tiles' scales are requested before further weights
        float sc[2][4];
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int n = col_begin + (wave + (2 * q + h) * NW) * 16 + lg * 4 + e;
                sc[h][e] = p.scale[n < p.N ? n : p.N - 1];
            }
        static_for<KU>([&](auto uc) {
            constexpr int u = decltype(uc)::value;
            constexpr int S = u % D;
            *reinterpret_cast<uint4 *>(stage + wr_off) = wv[S][0];
            *reinterpret_cast<uint4 *>(stage + wr_off8) = wv[S][1];
            *reinterpret_cast<uint4 *>(stage + 2048 + wr_off) = wv[S][2];
            *reinterpret_cast<uint4 *>(stage + 2048 + wr_off8) = wv[S][3];
            __builtin_amdgcn_wave_barrier();
            uint4 wt[2][2];
#pragma unroll
            for (int h = 0; h < 2; ++h)
#pragma unroll
                for (int v = 0; v < 2; ++v) wt[h][v] = *reinterpret_cast<const uint4 *>(stage + h * 2048 + rd_off[v]);
            __builtin_amdgcn_wave_barrier();
            if constexpr (u + D == KU) set_pair(q + 1);  // the units requested from here on belong to the next pair
            issue(std::integral_constant<int, S>{}, std::integral_constant<int, (u + D) % KU>{});
#pragma unroll
            for (int v = 0; v < 2; ++v) {
                uint4 w0[2], w1[2];
#pragma unroll
                for (int h = 0; h < 2; ++h) {
                    cvt_i8x4<DT>(wt[h][v].x, w0[h].x, w0[h].y);
                    cvt_i8x4<DT>(wt[h][v].y, w0[h].z, w0[h].w);
                    cvt_i8x4<DT>(wt[h][v].z, w1[h].x, w1[h].y);
                    cvt_i8x4<DT>(wt[h][v].w, w1[h].z, w1[h].w);
                }
                const char *xs0 = smem + (((u * 4 + v * 2) * MT) * 64 + lane) * 16;
#pragma unroll
                for (int t = 0; t < MT; ++t) {
                    const uint4 x0 = *reinterpret_cast<const uint4 *>(xs0 + t * 1024);
                    const uint4 x1 = *reinterpret_cast<const uint4 *>(xs0 + (MT + t) * 1024);
                    acc[0][t] = mfma16<DT>(w0[0], x0, acc[0][t]);
                    acc[1][t] = mfma16<DT>(w0[1], x0, acc[1][t]);
                    acc[0][t] = mfma16<DT>(w1[0], x1, acc[0][t]);
                    acc[1][t] = mfma16<DT>(w1[1], x1, acc[1][t]);
                }
            }
        });
#pragma unroll
        for (int h = 0; h < 2; ++h) {
#pragma unroll
            for (int t = 0; t < MT; ++t)
#pragma unroll
                for (int e = 0; e < 4; ++e) acc[h][t][e] *= sc[h][e];
            store_tile(acc[h], col_begin + (wave + (2 * q + h) * NW) * 16, plane);  // past the last tile: nothing is inside the range
        }
    }
}

// ---- M <= 4: row-streaming kernel --------------------------------------------------------------------
// One wavefront owns one output column (linear: one row of w; gated pair: the gate row and the up row of that
// column) over the whole of K. A load instruction covers 1 KiB of consecutive bytes of a row, K_BATCH of them
// per row are in flight before anything is multiplied, x (at most 4 rows) sits in LDS, products go through
// v_dot2 with fp32 accumulation, and 64 lane sums meet in a butterfly at the end.
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(2))) _Float16 f16x2;

template <int DT>
__device__ __forceinline__ float dot2(uint32_t a, uint32_t b, float c) {
    if constexpr (DT == TPAMD_BF16)
        return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, a), __builtin_bit_cast(bf16x2, b), c, false);
    else
        return __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2, a), __builtin_bit_cast(f16x2, b), c, false);
}
template <int DT>
__device__ __forceinline__ float dot8(uint4 w, uint4 x, float c) {
    c = dot2<DT>(w.x, x.x, c);
    c = dot2<DT>(w.y, x.y, c);
    c = dot2<DT>(w.z, x.z, c);
    return dot2<DT>(w.w, x.w, c);
}
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off);
    return v;
}

// GV_WAVES wavefronts per block; K_BATCH = loads per row in flight before anything is multiplied.
template <int DT, bool W8, int MODE, int MR, int GV_WAVES, int K_BATCH>
__global__ __launch_bounds__(GV_WAVES * 64) void gemv_kernel(SkinnyParams p) {
    constexpr int GV_THREADS = GV_WAVES * 64;
    constexpr int NMAT = MODE == SK_SWIGLU ? 2 : 1;
    constexpr int STEP_K = W8 ? 1024 : 512;          // K elements per wavefront-wide 16-byte load of w
    constexpr int XPL = W8 ? 2 : 1;                  // 16-byte pieces of x per lane per step

    extern __shared__ __align__(16) char xs[];       // x[MR][K]
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int n = blockIdx.x * GV_WAVES + wave;
    const bool live = n < p.N;
    const int row = live ? n : p.N - 1;
    const int wbytes = W8 ? 1 : 2;
    const int row_bytes = p.K * 2;
    const int nsteps = (p.K + STEP_K - 1) / STEP_K;
    const uint4 zero4 = make_uint4(0, 0, 0, 0);

    const char *wp[NMAT];
    wp[0] = p.w + static_cast<int64_t>(row) * p.ldw * wbytes + lane * 16;
    if constexpr (NMAT == 2) wp[1] = p.w2 + static_cast<int64_t>(row) * p.ldw * wbytes + lane * 16;
    const int lane_k = lane * (W8 ? 16 : 8);          // first K element of this lane inside a step

    float acc[NMAT][MR];
#pragma unroll
    for (int a = 0; a < NMAT; ++a)
#pragma unroll
        for (int m = 0; m < MR; ++m) acc[a][m] = 0.f;

    uint4 wv[K_BATCH][NMAT];
    auto issue = [&](int s0) {
#pragma unroll
        for (int j = 0; j < K_BATCH; ++j) {
            const int s = s0 + j;
            const bool ok = s < nsteps && s * STEP_K + lane_k < p.K;
#pragma unroll
            for (int a = 0; a < NMAT; ++a) {
                // out-of-range pieces are fetched from the row's start (always valid) and zeroed: unconditional
                // loads keep the whole batch in flight together
                const uint4 raw = nt_load_u4(ok ? wp[a] + static_cast<int64_t>(s) * STEP_K * wbytes : wp[a] - lane * 16);
                wv[j][a] = ok ? raw : zero4;
            }
        }
    };

    issue(0);
    // stage x while the first batch is in flight
    for (int m = 0; m < MR; ++m)
        for (int i = tid; i * 8 < p.K; i += GV_THREADS)
            *reinterpret_cast<uint4 *>(xs + m * row_bytes + i * 16) =
                *reinterpret_cast<const uint4 *>(p.x + (static_cast<int64_t>(m) * p.ldx + i * 8) * 2);
    __syncthreads();

    for (int s0 = 0; s0 < nsteps; s0 += K_BATCH) {
        if (s0 > 0) issue(s0);
#pragma unroll
        for (int j = 0; j < K_BATCH; ++j) {
            const int k = (s0 + j) * STEP_K + lane_k;
            if (s0 + j < nsteps && k < p.K) {
#pragma unroll
                for (int m = 0; m < MR; ++m) {
                    uint4 xv[XPL];
#pragma unroll
                    for (int h = 0; h < XPL; ++h) xv[h] = *reinterpret_cast<const uint4 *>(xs + m * row_bytes + (k + h * 8) * 2);
#pragma unroll
                    for (int a = 0; a < NMAT; ++a) {
                        if constexpr (W8) {
                            uint4 w0, w1;
                            cvt_i8x4<DT>(wv[j][a].x, w0.x, w0.y);
                            cvt_i8x4<DT>(wv[j][a].y, w0.z, w0.w);
                            cvt_i8x4<DT>(wv[j][a].z, w1.x, w1.y);
                            cvt_i8x4<DT>(wv[j][a].w, w1.z, w1.w);
                            acc[a][m] = dot8<DT>(w0, xv[0], acc[a][m]);
                            acc[a][m] = dot8<DT>(w1, xv[XPL - 1], acc[a][m]);
                        } else {
                            acc[a][m] = dot8<DT>(wv[j][a], xv[0], acc[a][m]);
                        }
                    }
                }
            }
        }
    }

    float acc_o[MR];
    if constexpr (W8) {
        // outlier columns: lanes stride over them
        const uint16_t *xo = reinterpret_cast<const uint16_t *>(xs);
        const uint16_t *wo = reinterpret_cast<const uint16_t *>(p.w_out);
#pragma unroll
        for (int m = 0; m < MR; ++m) acc_o[m] = 0.f;
        for (int o = lane; o < p.n_out; o += 64) {
            const float wval = half_to_f32<DT>(wo[static_cast<int64_t>(row) * p.ld_wout + o]);
            const int col = p.outlier_idx[o];
#pragma unroll
            for (int m = 0; m < MR; ++m) acc_o[m] = fmaf(half_to_f32<DT>(xo[m * p.K + col]), wval, acc_o[m]);
        }
    }

#pragma unroll
    for (int m = 0; m < MR; ++m) {
        float s0 = wave_sum(acc[0][m]);
        float s1 = 0.f;
        if constexpr (NMAT == 2) s1 = wave_sum(acc[NMAT - 1][m]);
        if constexpr (W8) s0 = s0 * p.scale[row] + wave_sum(acc_o[m]);
        if (lane == 0 && live) skinny_store_output<DT, MODE>(p, s0, s1, m, n);
    }
}

constexpr int GEMV_MAX_M = 3;  // the row kernels take at most 3 rows (large matrices go to the MFMA kernels from 3 rows on, see skinny_dispatch)
constexpr int64_t GEMV_MAX_X_BYTES = 64 * 1024;  // x[M][K] lives in LDS

template <int DT, bool W8, int MODE>
int launch_gemv(const SkinnyParams &p, hipStream_t s) {
    // measured on the Llama-7B shard shapes: small blocks and short batches for the gated pair (two rows per
    // wavefront), whole rows in flight for a single matrix
    constexpr int GV_WAVES = MODE == SK_SWIGLU ? 4 : 8;
    constexpr int GV_THREADS = GV_WAVES * 64;
    constexpr int KB = MODE == SK_SWIGLU ? 4 : 12;
    const unsigned grid = static_cast<unsigned>((p.N + GV_WAVES - 1) / GV_WAVES);
    const size_t lds = static_cast<size_t>(p.M) * p.K * 2;
    switch (p.M) {
        case 1: hipLaunchKernelGGL((gemv_kernel<DT, W8, MODE, 1, GV_WAVES, KB>), dim3(grid), dim3(GV_THREADS), lds, s, p); break;
        case 2: hipLaunchKernelGGL((gemv_kernel<DT, W8, MODE, 2, GV_WAVES, KB>), dim3(grid), dim3(GV_THREADS), lds, s, p); break;
        default: hipLaunchKernelGGL((gemv_kernel<DT, W8, MODE, 3, GV_WAVES, KB>), dim3(grid), dim3(GV_THREADS), lds, s, p); break;
    }
    TPAMD_HIP(hipGetLastError());
    return TPAMD_OK;
}

// ---- M <= 3, K <= 8192: every piece of a column's weights in flight at once, all counts known at compile time --------
// Same mapping as gemv_kernel (a wavefront owns an output column, x in LDS) for the shapes decode meets: a row takes
// at most NP 1-KiB loads per matrix, issued back to back before x is staged, and multiplied as they arrive in a fully
// unrolled sequence; the 64 lane sums meet through DPP row operations and four lane reads instead of six LDS-crossbar
// shuffles. WAVES wavefronts per block share one copy of x.
template <int CTRL>
__device__ __forceinline__ float dpp_add(float v) {
    const int t = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true);
    return v + __builtin_bit_cast(float, t);
}
// Sum over the 64 lanes, in every lane: pairs, quads, eights and sixteens inside each row of 16 lanes (quad_perm
// [1,0,3,2], quad_perm [2,3,0,1], row_half_mirror, row_mirror), then the four row sums as (r0 + r1) + (r2 + r3).
__device__ __forceinline__ float wave_sum_dpp(float v) {
    v = dpp_add<0xb1>(v);
    v = dpp_add<0x4e>(v);
    v = dpp_add<0x141>(v);
    v = dpp_add<0x140>(v);
    const int r = __builtin_bit_cast(int, v);
    const float a = __builtin_bit_cast(float, __builtin_amdgcn_readlane(r, 0)), b = __builtin_bit_cast(float, __builtin_amdgcn_readlane(r, 16));
    const float c = __builtin_bit_cast(float, __builtin_amdgcn_readlane(r, 32)), d = __builtin_bit_cast(float, __builtin_amdgcn_readlane(r, 48));
    return (a + b) + (c + d);
}

// int8 weights (W8, plain linear): a piece is 1024 K elements; the outlier products' operands (at most 128 outlier
// columns) and the row's scale are requested ahead of everything else, so that no wavefront ends on a memory round trip.
template <int DT, bool W8, int MODE, int MR, int WAVES, int NP, bool WHOLE>
__global__ __launch_bounds__(WAVES * 64) void gemv_rows_kernel(SkinnyParams p) {
    static_assert(!W8 || MODE == SK_LINEAR, "int8 weights: plain linear only");
    constexpr int THREADS = WAVES * 64;
    constexpr int NMAT = MODE == SK_SWIGLU ? 2 : 1;
    constexpr int PIECE_K = W8 ? 1024 : 512;  // K elements in one wavefront-wide 16-byte load of w
    constexpr int OB = 2;                     // int8: outlier columns per lane
    extern __shared__ __align__(16) char xs[];  // x[MR][K]
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int n = blockIdx.x * WAVES + wave;
    const int row = n < p.N ? n : p.N - 1;
    const int K = WHOLE ? NP * PIECE_K : p.K;  // WHOLE: K is exactly NP pieces, nothing to mask
    const int w_row_bytes = W8 ? K : K * 2, x_row_bytes = K * 2;
    const int x_lds_row = W8 ? (x_row_bytes + 2047) & ~2047 : x_row_bytes;  // int8: rows of x are permuted within whole 2 KiB
    const char *w0 = p.w + static_cast<int64_t>(row) * p.ldw * (W8 ? 1 : 2) + lane * 16;
    const char *w1 = NMAT == 2 ? p.w2 + static_cast<int64_t>(row) * p.ldw * 2 + lane * 16 : nullptr;
    // int8: a lane's 16 weights of a piece meet 32 bytes of x. Stored as they come, the two 16-byte reads of the 64 lanes
    // would be 32 bytes apart and collide in the LDS banks two by two; so within every 2 KiB of x (one piece) the first
    // halves of all lanes' 32 bytes are stored together and the second halves behind them: both reads are contiguous.
    auto x_slot = [](int byte_at) -> int {
        if constexpr (!W8) return byte_at;
        else return (byte_at & ~2047) | ((byte_at & 16) << 6) | ((byte_at >> 1) & 1008) | (byte_at & 15);
    };
    uint16_t o_w[OB];
    int o_col[OB];
    float row_scale = 1.f;
    if constexpr (W8) {
        row_scale = p.scale[row];
#pragma unroll
        for (int i = 0; i < OB; ++i) {
            const int o = lane + i * 64;
            const bool in = o < p.n_out;
            o_w[i] = in ? reinterpret_cast<const uint16_t *>(p.w_out)[static_cast<int64_t>(row) * p.ld_wout + o] : static_cast<uint16_t>(0);
            o_col[i] = in ? p.outlier_idx[o] : 0;
        }
    }
    // x is requested first and the weights right behind it: loads return in order, so x can be staged (and the block
    // can meet) while the weights are still on their way, and every piece is multiplied as it arrives
    constexpr int XL = (NP * PIECE_K / 8 + THREADS - 1) / THREADS;  // 16-byte pieces of one row of x per thread
    uint4 xr[MR][XL];
#pragma unroll
    for (int m = 0; m < MR; ++m)
#pragma unroll
        for (int i = 0; i < XL; ++i) {
            const int at = (tid + i * THREADS) * 16;
            xr[m][i] = *reinterpret_cast<const uint4 *>(p.x + static_cast<int64_t>(m) * p.ldx * 2 + (at < x_row_bytes ? at : 0));
        }
    uint4 wv[NMAT][NP];
#pragma unroll
    for (int j = 0; j < NP; ++j) {
        // pieces past K are fetched from the row's start (always valid) and zeroed
        const bool ok = WHOLE || j * 1024 + lane * 16 < w_row_bytes;
        const uint4 a = nt_load_u4(ok ? w0 + j * 1024 : w0 - lane * 16);
        wv[0][j] = ok ? a : make_uint4(0, 0, 0, 0);
        if constexpr (NMAT == 2) {
            const uint4 b = nt_load_u4(ok ? w1 + j * 1024 : w1 - lane * 16);
            wv[NMAT - 1][j] = ok ? b : make_uint4(0, 0, 0, 0);
        }
    }
#pragma unroll
    for (int m = 0; m < MR; ++m)
#pragma unroll
        for (int i = 0; i < XL; ++i) {
            const int at = (tid + i * THREADS) * 16;
            if (at < x_row_bytes) *reinterpret_cast<uint4 *>(xs + m * x_lds_row + x_slot(at)) = xr[m][i];
        }
    __syncthreads();
    float acc[NMAT][MR], acc2[MR];  // int8: two sums per row of x, so that consecutive products do not wait for each other
#pragma unroll
    for (int m = 0; m < MR; ++m) {
        acc2[m] = 0.f;
#pragma unroll
        for (int a = 0; a < NMAT; ++a) acc[a][m] = 0.f;
    }
#pragma unroll
    for (int j = 0; j < NP; ++j) {
        const int k = WHOLE || j * 1024 + lane * 16 < w_row_bytes ? j * PIECE_K + lane * (PIECE_K / 64) : 0;
        if constexpr (W8) {
            uint4 lo, hi;
            cvt_i8x4<DT>(wv[0][j].x, lo.x, lo.y);
            cvt_i8x4<DT>(wv[0][j].y, lo.z, lo.w);
            cvt_i8x4<DT>(wv[0][j].z, hi.x, hi.y);
            cvt_i8x4<DT>(wv[0][j].w, hi.z, hi.w);
#pragma unroll
            for (int m = 0; m < MR; ++m) {
                const uint4 xv = *reinterpret_cast<const uint4 *>(xs + m * x_lds_row + x_slot(k * 2));
                const uint4 xv1 = *reinterpret_cast<const uint4 *>(xs + m * x_lds_row + x_slot(k * 2 + 16));
                acc[0][m] = dot8<DT>(lo, xv, acc[0][m]);
                acc2[m] = dot8<DT>(hi, xv1, acc2[m]);
            }
        } else {
#pragma unroll
            for (int m = 0; m < MR; ++m) {
                const uint4 xv = *reinterpret_cast<const uint4 *>(xs + m * x_lds_row + k * 2);
#pragma unroll
                for (int a = 0; a < NMAT; ++a) acc[a][m] = dot8<DT>(wv[a][j], xv, acc[a][m]);
            }
        }
    }
#pragma unroll
    for (int m = 0; m < MR; ++m) {
        float s0 = wave_sum_dpp(W8 ? acc[0][m] + acc2[m] : acc[0][m]);
        float s1 = 0.f;
        if constexpr (NMAT == 2) s1 = wave_sum_dpp(acc[NMAT - 1][m]);
        if constexpr (W8) {
            float ao = 0.f;
#pragma unroll
            for (int i = 0; i < OB; ++i)
                ao = fmaf(half_to_f32<DT>(*reinterpret_cast<const uint16_t *>(xs + m * x_lds_row + x_slot(o_col[i] * 2))), half_to_f32<DT>(o_w[i]), ao);
            s0 = s0 * row_scale + wave_sum_dpp(ao);
        }
        if (lane == 0 && n < p.N) skinny_store_output<DT, MODE>(p, s0, s1, m, n);
    }
}

template <int DT, bool W8, int MODE, int WAVES, int NP>
void launch_gemv_rows_m(const SkinnyParams &p, hipStream_t s) {
    const dim3 grid(static_cast<unsigned>((p.N + WAVES - 1) / WAVES)), block(WAVES * 64);
    const size_t lds = W8 ? static_cast<size_t>(p.M) * ((p.K * 2 + 2047) / 2048 * 2048) : static_cast<size_t>(p.M) * p.K * 2;
    const bool whole = p.K == NP * (W8 ? 1024 : 512);
#define TPAMD_ROWS_M(MRV) \
    if (whole) hipLaunchKernelGGL((gemv_rows_kernel<DT, W8, MODE, MRV, WAVES, NP, true>), grid, block, lds, s, p); \
    else hipLaunchKernelGGL((gemv_rows_kernel<DT, W8, MODE, MRV, WAVES, NP, false>), grid, block, lds, s, p)
    switch (p.M) {
        case 1: TPAMD_ROWS_M(1); break;
        case 2: TPAMD_ROWS_M(2); break;
        default: TPAMD_ROWS_M(3); break;
    }
#undef TPAMD_ROWS_M
}

// Which kernel takes M <= 3 rows of 16-bit weights. Fitted on a sweep of 342 shapes (single matrix and gated pair, M = 1..3,
// N = 1376..32000, K = 2048..8192; checked and adjusted on 525 more with other N and K, where it is 1 % off the best choice; each timed inside a HIP graph on weights that rotate through more memory than the
// caches hold): sum over the sweep 7197 us with the rules before, 6986 us with these, 6948 us with the best kernel per shape.
//  - a block of W wavefronts owns W output columns (W column pairs of a gated pair) and a CU's share of HBM bandwidth
//    is what bounds it, so what counts is the most columns any CU gets: ceil(ceil(N / W) / CUs) * W. 16 wavefronts
//    win when that is no worse than with 8 (N = 5504: 32 against 24 on 256 CUs, 13 % slower) and rows are long enough
//    to pay for the larger block; 4 wavefronts win on small N where they balance better (N = 2752: 12 against 16);
//  - 2 rows of long rows (K > 6144 single, K >= 7680 gated pair) on 4096 columns or more go to the MFMA kernels like 3
//    rows do (single 8192 x 8192: 24.2 us there, 26.3 us here; 12800 x 7168: 32.7 against 37.5-41.9 us; pair 5504 x 8192:
//    29.7 against 33.1 us); a lone row of a long-rowed wide pair goes to the general kernel (12800 x 7168: 55 against 58-66 us);
//  - gated pairs with 2 rows, 8192 columns or more and K around 4096 go to the general kernel (11008 x 4096: 28.1 against 29.0 us).
enum RowsPath { ROWS_W4, ROWS_W8, ROWS_W16, ROWS_GENERAL, ROWS_MFMA };
inline RowsPath pick_rows_path(bool pair, int64_t M, int64_t N, int64_t K, int cus) {
    auto most_cols = [&](int64_t w) { return ((N + w - 1) / w + cus - 1) / cus * w; };
    const bool bal16 = most_cols(16) <= most_cols(8) && N >= 2752;
    const bool bal4 = most_cols(4) < most_cols(8) && N < 4096;
    if (M == 3 && K >= 3072 && K <= 8192) {
        // 3 rows go to the MFMA kernels (Llama-7B MLP shard step: 36.4 us here, 28.3 us there), except a single matrix of at
        // most 2048 columns (1376 x 6144: 6.5 against 8.4 us, 1024 x 8192: 7.0 against 9.2 us) and, with K near 4096, of at
        // most 5504 (4096 x 4096: 7.6 against 8.2 us)
        if (!pair && N <= 2048) return N <= 1024 ? ROWS_W4 : ROWS_W8;
        if (!pair && K >= 3584 && K <= 4608 && N <= 5504) return bal16 ? ROWS_W16 : ROWS_W8;
        return ROWS_MFMA;
    }
    if (!pair) {
        if (M == 2 && K > 6144) return N >= 4096 ? ROWS_MFMA : bal4 ? ROWS_W4 : ROWS_W8;
        if (M == 3) return ROWS_W8;
        return bal16 && K >= (M == 2 ? 4096 : 3072) ? ROWS_W16 : ROWS_W8;
    }
    const bool near_4096 = K >= 3584 && K <= 4608;
    if (M == 1) {
        if (near_4096 && bal16) return ROWS_W16;
        if (K > 6144 && N > 11008) return ROWS_GENERAL;
        return bal4 || (K > 6144 && N >= 2752) ? ROWS_W4 : ROWS_W8;
    }
    if (M == 2) {
        if (K >= 5120 && N >= 4096) return K >= 7680 ? ROWS_MFMA : ROWS_GENERAL;  // 7168 x 5120: 24.9 us general, 27.8 us MFMA
        if (K >= 3584 && N >= 8192) return ROWS_GENERAL;
        if (near_4096 && bal16) return ROWS_W16;
        return bal4 ? ROWS_W4 : ROWS_W8;
    }
    return ROWS_W8;
}

// M <= 3 and at most 16 pieces per row: K <= 8192 for 16-bit weights, K <= 16384 (and at most 128 outlier columns) for
// int8. `path`: what pick_rows_path chose (int8: ROWS_W8). *done = false: not taken.
template <int DT, bool W8, int MODE>
int launch_gemv_rows(const SkinnyParams &p, hipStream_t s, RowsPath path, bool *done) {
    *done = false;
    const int knob = tuning().gemv_rows;  // wavefronts per block; 0 = the general kernel
    const int piece_k = W8 ? 1024 : 512;
    if (knob == 0 || (knob == TUNE_UNSET && path == ROWS_GENERAL)) return TPAMD_OK;
    if (p.K > 16 * piece_k || p.K % (W8 ? 16 : 8) != 0 || (W8 && p.n_out > 128)) return TPAMD_OK;
    // int8 with 2 or 3 rows of x: every further row costs as much again in LDS reads (32 bytes of x per 16 weights), and
    // the general kernel's staggered blocks hide that better (Falcon-40B MLP shard, 2 rows: 66 us against 83 us here)
    if (W8 && p.M > 1) return TPAMD_OK;
    // int8, M = 1, 16384 x 8192 + 8192 x 16384 with 16 / 8 / 4 wavefronts per block: 51.6 / 48.0 / 50.4 us (the general
    // kernel: 58.8 us)
    const int waves = knob != TUNE_UNSET ? knob : path == ROWS_W16 ? 16 : path == ROWS_W4 ? 4 : 8;
    const int np = (p.K + piece_k - 1) / piece_k;
#define TPAMD_ROWS_CASE(W) \
    if (np <= 4) launch_gemv_rows_m<DT, W8, MODE, W, 4>(p, s); else if (np <= 8) launch_gemv_rows_m<DT, W8, MODE, W, 8>(p, s); \
    else if (np <= 11) launch_gemv_rows_m<DT, W8, MODE, W, 11>(p, s); else if (np <= 12) launch_gemv_rows_m<DT, W8, MODE, W, 12>(p, s); \
    else launch_gemv_rows_m<DT, W8, MODE, W, 16>(p, s)
    if (waves == 4) { TPAMD_ROWS_CASE(4); }
    else if (waves == 16) { TPAMD_ROWS_CASE(16); }
    else { TPAMD_ROWS_CASE(8); }
#undef TPAMD_ROWS_CASE
    TPAMD_HIP(hipGetLastError());
    *done = true;
    return TPAMD_OK;
}

// Column groups per block: as many as keep at least one block per CU and divide N; they pay once x outweighs w.
inline int pick_cg(const SkinnyParams &p, bool w8, bool swiglu) {
    if (const int v = tuning().skinny_cg; v != TUNE_UNSET) return v == 4 ? 4 : v == 2 ? 2 : 1;
    if (p.M < (w8 ? 4 : 12)) return 1;  // measured: below this the prefetching single-group kernel is faster
    if (!swiglu && p.N % 64 == 0 && p.N / 64 >= 256) return 4;
    if (p.N % 32 == 0 && p.N / 32 >= 256) return 2;
    return 1;
}

// Gated pair with 16-bit weights and at most 32 rows: the 8-column form (measured 5-12 % faster than the
// 16-column forms at every M from 4 to 32 on the Llama-7B shard shapes).
inline bool pick_pair(const SkinnyParams &p) {
    if (tuning().skinny_pair != TUNE_UNSET) return tuning().skinny_pair != 0;
    return p.M <= 32;
}

// The x-resident kernel against the plain one (more blocks per CU, x re-read per tile) and, for the gated pair, the one
// that stages x in LDS. Measured inside a HIP graph at 4 / 8 / 12 / 16 rows (us; plain | resident | x in LDS):
//   pair 5504 x 4096:   18.9 19.7 20.5 20.5 | 17.9 17.9 18.0 17.8 | 19.1 19.5 20.2 20.2
//   pair 11008 x 5504:  45.6 46.3 48.9 51.6 | 42.1 40.9 41.0 41.6 | 48.4 47.4 48.2 49.0
//   pair 2752 x 4096:   12.5 13.0 13.5 14.3 | 11.6 11.7 11.7 11.8 | 13.1 13.3 13.8 14.3
//   pair 1376 x 8192:   11.8 12.7 13.7 14.6 | 11.9 11.9 12.1 12.1 | 15.1 15.6 16.6 17.9
//   pair 16384 x 8192:  85.1 84.9 88.2 93.2 | 93.1 92.4 94.8 95.4 | 86.7 86.6 86.8 87.8
//   pair 4096 x 2048:    9.2  9.3  9.7 10.0 | 10.5 10.5 10.4 10.6 |  9.5  9.6  9.9 10.2
// 16-bit weights, 4 to 16 rows, K from 3072 to 8192 (the x fragments have to fit the registers: 4 chunks per wavefront
// and 4 register slots for the weights up to K = 4096, 6 and 3 up to 6144, 8 and 2 up to 8192).
template <int MODE>
inline bool pick_resident(const SkinnyParams &p, int cus) {
    if (p.M > 16 || p.K > 8192) return false;
    if (tuning().skinny_resident != TUNE_UNSET) return tuning().skinny_resident != 0;
    const int64_t tiles = (p.N + (MODE == SK_SWIGLU ? 7 : 15)) / (MODE == SK_SWIGLU ? 8 : 16);
    if (p.M < (MODE == SK_SWIGLU ? 3 : 2) || p.K < 3072) return false;  // 2 rows of a gated pair: up to 26 % slower here (11008 x 6144)
    if (MODE == SK_SWIGLU) {
        // Refitted on a sweep of 220 pair shapes (N from 1376 to 14336, K from 2048 to 8192, 4 to 16 rows, in a HIP graph,
        // plain 8-column kernel | this one | x staged in LDS). Whole rounds of one tile per CU suit the plain kernel, whose
        // blocks then fill the CUs evenly (2048 x 3072 ... 8192: 4-36 %; 4096 and 8192 x 8192: 16-41 %); otherwise this
        // kernel is the fastest from K = 3072 on, except on few tiles at K = 3072 and, at K = 8192, few tiles below 8 rows
        // and more than four tiles per CU up to 8 rows.
        if (tiles == cus) return false;
        if (p.K <= 6144) return tiles * 2 >= cus && !(p.K < 4096 && tiles < cus);
        if ((tiles % cus == 0 && tiles <= 4ll * cus) || (tiles > 4ll * cus && tiles < 7ll * cus && p.M <= 8)) return false;
        return tiles > cus || p.M >= 8;
    }
    // Single matrix: refitted on a sweep of 900 shapes (N from 1024 to 20480 in steps of 512 and the model widths between,
    // K from 2048 to 8192, 4 to 16 rows, in a HIP graph, plain | this kernel): the sum over the sweep is 18.9 ms with the
    // rules before, 18.0 ms with these, 17.98 ms with the better kernel per shape. The persistent x-resident blocks take
    // the tiles in turn, so a ragged last round costs them nothing, while the plain kernel's blocks fill the CUs unevenly
    // whenever the tiles are not a whole number of rounds:
    //  - more tiles than CUs and K >= 4096: this kernel (9216 x 8192 at 4-8 rows 31.1-32.1 -> 27.9-28.5 us, 12544 x 8192 at
    //    12-16 rows 47.8 -> 37.8 us, 20480 x 5504 at 12-16 rows 56-57 -> 39 us), except, up to 8 rows, on two or four
    //    whole rounds (8192 and 16384 columns: the plain kernel by 3-9 %);
    //  - at most one tile per CU: the plain kernel, except long rows on few tiles from 12 rows on (K >= 5504 on at most
    //    0.7 of the CUs: 5-20 %) and 16 rows on at most half the CUs;
    //  - K = 3072: from 12 rows on above one tile per CU except between three and four (there the plain kernel wins by
    //    4-8 %), from 8 rows on above two tiles per CU.
    const bool even_whole = tiles % (2ll * cus) == 0 && tiles <= 4ll * cus;
    if (p.K >= 3584) {
        if (tiles <= cus) return (p.K >= 5504 && p.M >= 12 && tiles * 10 <= 7ll * cus) || (p.M >= 16 && tiles * 2 <= cus);
        return p.M >= 12 || !even_whole;
    }
    if (tiles <= cus) return false;
    if (p.M >= 12) return !(tiles >= 3ll * cus && tiles < 4ll * cus);
    return p.M >= 8 && tiles > 2ll * cus && !even_whole;
}

template <int DT, int MODE>
int launch_resident(const SkinnyParams &p, int cus, hipStream_t s) {
    const int64_t tiles = (p.N + (MODE == SK_SWIGLU ? 7 : 15)) / (MODE == SK_SWIGLU ? 8 : 16);
    const unsigned grid = static_cast<unsigned>(tiles < cus ? tiles : cus);
    // K <= 4096: 4 chunks per wavefront, a slot each; up to 6144: 6 chunks and 3 slots (6 slots do not fit the
    // registers); up to 8192: 8 chunks and 2 slots.
    // (Two blocks of 4 wavefronts per CU, 8 chunks each and 4 slots, were measured too: the registers do not fit and
    // the kernel takes twice as long.)
    if (p.K <= 4096) hipLaunchKernelGGL((skinny_resident_kernel<DT, MODE, 8, 4, 4>), dim3(grid), dim3(512), 0, s, p);
    else if (p.K <= 6144) hipLaunchKernelGGL((skinny_resident_kernel<DT, MODE, 8, 6, 3>), dim3(grid), dim3(512), 0, s, p);
    else hipLaunchKernelGGL((skinny_resident_kernel<DT, MODE, 8, 8, 2>), dim3(grid), dim3(512), 0, s, p);
    TPAMD_HIP(hipGetLastError());
    return TPAMD_OK;
}

// Which of the three int8 kernels takes 2 to 64 rows: the K-split kernel whose wavefronts own columns ("cols": x of the
// split in LDS, fp32 partial planes, a finishing pass), the older K-split kernel ("split": x in registers) or the unsplit
// one. Fitted on a sweep of 600 shapes (N 2048-28672, K 2048-16384, 2-64 rows, each kernel forced, inside a HIP graph on
// weights that rotate through more memory than the caches hold) and checked on 290 random ones: 0.8 % and 0.7 % off the
// best kernel per shape in the geometric mean (the thresholds on the matrix size that these rules replace: 6.3 % and 5.1 %,
// up to 80 % on wide matrices with short rows, 11008 x 3072 at 64 rows: 50 us unsplit, 28 us here).
//  - K >= 4096 and more than 4096 columns: cols, except on one, two or four whole rounds of 16-column tiles per CU
//    (4096, 8192, 16384 columns on 256 CUs), where the unsplit kernel's blocks fill the CUs evenly and win up to 32 rows
//    (16384 x 4096 at 16 rows: 18.5 against 21.3 us) unless rows are very long (K > 11008) or there are only 2 of x;
//    at K = 4096 and 24-32 rows the older split kernel is the faster one off those rounds (11008 x 4096: 5-10 %);
//  - up to 4096 columns: unsplit, except very long rows (K >= 16384, or K >= 11008 from 48 rows on);
//  - K < 4096: cols on 18000 columns or more, and from 11008 columns on for 2 rows and from 24 rows on.
enum W8Path { W8_PLAIN, W8_SPLIT, W8_COLS };
inline W8Path pick_w8_path(const SkinnyParams &p, int cus) {
    const int64_t tiles = (p.N + 15) / 16;
    const bool whole = tiles == cus || (tiles % (2ll * cus) == 0 && tiles <= 4ll * cus);
    if (p.M < 2) return W8_PLAIN;
    if (p.K >= 4096) {
        if (p.N > 4096) {
            if (!whole || p.M == 2 || p.K > 11008) return p.K < 5120 && p.M >= 24 && p.M <= 32 && !whole ? W8_SPLIT : W8_COLS;
            if (p.M >= 48) return p.K >= 5120 || p.N >= 16384 ? W8_COLS : W8_SPLIT;
            return W8_PLAIN;
        }
        return p.K >= 16384 || (p.K >= 11008 && p.M >= 48 && p.N >= 3072) ? W8_COLS : W8_PLAIN;
    }
    const bool wide = p.N >= 18000 || (p.N >= 11008 && (p.M == 2 || (p.M >= 24 && (!whole || (p.K >= 3072 && p.M >= 48)))));
    return wide ? W8_COLS : W8_PLAIN;
}

// int8 weights, K split over blocks: K at least 4096, at most 64 rows and 256 outlier columns.
// Needs the per-device scratch buffer for the partial sums; without it (first use under stream capture) the
// caller takes the unsplit kernel.
template <int DT>
int launch_w8_split(const SkinnyParams &p, hipStream_t s, bool *done) {
    *done = false;
    int dev = 0, cus = 256;
    TPAMD_HIP(hipGetDevice(&dev));
    if (int rc_cus = device_cus(dev, &cus); rc_cus != TPAMD_OK) return rc_cus;
    if (tuning().w8_split != TUNE_UNSET) {
        if (tuning().w8_split == 0) return TPAMD_OK;
    } else if (pick_w8_path(p, cus) != W8_SPLIT) {
        return TPAMD_OK;
    }
    if (p.K < 4096 || p.n_out > 256 || p.M > 64) return TPAMD_OK;
    // x fragments fill 128 registers: 4 chunks per wavefront (8192 K elements per split) for 16 rows, 2 for 32, 1 for 64
    const int nch = p.M <= 16 ? 4 : p.M <= 32 ? 2 : 1;
    const int splits = (p.K + nch * 2048 - 1) / (nch * 2048);
    if (splits > cus) return TPAMD_OK;  // K in the millions: not what this kernel is laid out for
    int col_blocks = cus / splits > 0 ? cus / splits : 1;
    int cols_per_block = (p.N + col_blocks - 1) / col_blocks;
    cols_per_block = (cols_per_block + 15) / 16 * 16;
    col_blocks = (p.N + cols_per_block - 1) / cols_per_block;
    const dim3 grid(static_cast<unsigned>(col_blocks), static_cast<unsigned>(splits));
    if (splits == 1) {  // nothing to add up: no scratch buffer, no second launch
        if (p.M <= 16) hipLaunchKernelGGL((skinny_w8_split_kernel<DT, 1, 4, true>), grid, dim3(SK_THREADS), 0, s, p, nullptr, cols_per_block);
        else if (p.M <= 32) hipLaunchKernelGGL((skinny_w8_split_kernel<DT, 2, 2, true>), grid, dim3(SK_THREADS), 0, s, p, nullptr, cols_per_block);
        else hipLaunchKernelGGL((skinny_w8_split_kernel<DT, 4, 1, true>), grid, dim3(SK_THREADS), 0, s, p, nullptr, cols_per_block);
        TPAMD_HIP(hipGetLastError());
        *done = true;
        return TPAMD_OK;
    }
    const size_t need = static_cast<size_t>(splits) * p.M * p.N * sizeof(float);
    std::lock_guard<std::mutex> hold(splitk_mutex(dev));
    void *ws = nullptr;
    const int rc = splitk_scratch(dev, s, need, static_cast<size_t>(4) * cus * 128 * 128 * sizeof(float), &ws);
    if (rc != TPAMD_OK) return rc;
    if (ws == nullptr) return TPAMD_OK;
    float *part = static_cast<float *>(ws);
    if (p.M <= 16) hipLaunchKernelGGL((skinny_w8_split_kernel<DT, 1, 4, false>), grid, dim3(SK_THREADS), 0, s, p, part, cols_per_block);
    else if (p.M <= 32) hipLaunchKernelGGL((skinny_w8_split_kernel<DT, 2, 2, false>), grid, dim3(SK_THREADS), 0, s, p, part, cols_per_block);
    else hipLaunchKernelGGL((skinny_w8_split_kernel<DT, 4, 1, false>), grid, dim3(SK_THREADS), 0, s, p, part, cols_per_block);
    TPAMD_HIP(hipGetLastError());
    if (int rc_f = launch_w8_finish<DT>(p, part, splits, s); rc_f != TPAMD_OK) return rc_f;
    *done = true;
    return TPAMD_OK;
}

// int8 weights, wavefronts own columns: K a multiple of 16, at most 64 rows and 256 outlier columns, and enough columns
// that every wavefront of a block gets a tile. *done = false: not taken.
template <int DT, int MT, bool DIRECT>
int configure_w8_cols(int dev, size_t lds) {
    static thread_local int configured_dev = -1;  // per instantiation and host thread
    if (configured_dev != dev) {
        TPAMD_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(skinny_w8_cols_kernel<DT, MT, 8, DIRECT>),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds)));
        configured_dev = dev;
    }
    return TPAMD_OK;
}

template <int DT, int MT>
int launch_w8_cols_mt(const SkinnyParams &p, int dev, int cus, hipStream_t s, bool *done) {
    constexpr int KU = 8;
    const int k_planes = (p.K + KU * WC_UNIT_K - 1) / (KU * WC_UNIT_K);
    const int planes = k_planes + (p.n_out > 0 ? 1 : 0);
    if (k_planes > cus) return TPAMD_OK;
    int col_blocks = cus / k_planes;
    int cols_per_block = (p.N + col_blocks - 1) / col_blocks;
    cols_per_block = (cols_per_block + 16 * WC_NW - 1) / (16 * WC_NW) * (16 * WC_NW);
    col_blocks = (p.N + cols_per_block - 1) / cols_per_block;
    const size_t lds = static_cast<size_t>(KU) * 4 * MT * 1024 + WC_NW * WC_STAGE;
    // the outlier plane is worked on by one block per 8 tiles of a column range (a tile per wavefront)
    const int outlier_blocks = p.n_out > 0 ? (cols_per_block / 16 + WC_NW - 1) / WC_NW : 0;
    const dim3 grid(static_cast<unsigned>(col_blocks), static_cast<unsigned>(k_planes + outlier_blocks));
    if (planes == 1) {
        if (int rc = configure_w8_cols<DT, MT, true>(dev, lds); rc != TPAMD_OK) return rc;
        hipLaunchKernelGGL((skinny_w8_cols_kernel<DT, MT, KU, true>), grid, dim3(WC_NW * 64), lds, s, p, nullptr, cols_per_block, k_planes);
        TPAMD_HIP(hipGetLastError());
        *done = true;
        return TPAMD_OK;
    }
    if (int rc = configure_w8_cols<DT, MT, false>(dev, lds); rc != TPAMD_OK) return rc;
    const size_t need = static_cast<size_t>(planes) * p.M * p.N * sizeof(float);
    std::lock_guard<std::mutex> hold(splitk_mutex(dev));
    void *ws = nullptr;
    const int rc = splitk_scratch(dev, s, need, static_cast<size_t>(4) * cus * 128 * 128 * sizeof(float), &ws);
    if (rc != TPAMD_OK) return rc;
    if (ws == nullptr) return TPAMD_OK;
    float *part = static_cast<float *>(ws);
    hipLaunchKernelGGL((skinny_w8_cols_kernel<DT, MT, KU, false>), grid, dim3(WC_NW * 64), lds, s, p, part, cols_per_block, k_planes);
    TPAMD_HIP(hipGetLastError());
    if (int rc_f = launch_w8_finish<DT>(p, part, planes, s); rc_f != TPAMD_OK) return rc_f;
    *done = true;
    return TPAMD_OK;
}

template <int DT>
int launch_w8_cols(const SkinnyParams &p, hipStream_t s, bool *done) {
    *done = false;
    if (tuning().w8_cols == 0) return TPAMD_OK;
    if (p.M > 64 || p.K % 16 != 0 || p.n_out > 256) return TPAMD_OK;
    int dev = 0, cus = 256;
    TPAMD_HIP(hipGetDevice(&dev));
    if (int rc_cus = device_cus(dev, &cus); rc_cus != TPAMD_OK) return rc_cus;
    if (tuning().w8_cols == TUNE_UNSET) {
        if (tuning().w8_split != TUNE_UNSET) return TPAMD_OK;  // an explicit choice between the two older kernels
        if (pick_w8_path(p, cus) != W8_COLS) return TPAMD_OK;
    }
    if (p.M <= 16) return launch_w8_cols_mt<DT, 1>(p, dev, cus, s, done);
    if (p.M <= 32) return launch_w8_cols_mt<DT, 2>(p, dev, cus, s, done);
    if (p.M <= 48) return launch_w8_cols_mt<DT, 3>(p, dev, cus, s, done);
    return launch_w8_cols_mt<DT, 4>(p, dev, cus, s, done);
}

// ---- gated pair, 4 <= M <= 16: x through LDS in MFMA operand order, chunk by chunk ------------------------------------
// One block of NW wavefronts per CU walks an even share of the 8-column tiles (8 gate rows + the 8 up rows of the same
// columns). K is cut into units of 64 elements (128 bytes of every weight row: two loads of 8 rows x 128 bytes per
// wavefront, two MFMAs); the units of a chunk of CH units are dealt to the wavefronts in turn. x is not kept in registers
// (which is what limits the loads in flight of the x-resident kernel) but staged in LDS in operand order: slot (unit, m) of
// 1 KiB holds for lane (q, j) the 8 elements x[j][unit * 64 + (q + 4 m) * 8 ...], so an operand read is one contiguous
// ds_read_b128 per lane. Two chunk buffers: while a chunk is multiplied every wavefront fetches its share of the next chunk
// into registers and stores it behind its last product of the chunk; one block-wide barrier per chunk. The weights go
// through D register slots per wavefront that are refilled as soon as a unit has been handed to the MFMAs; the list of
// units a wavefront walks (chunk by chunk, tile by tile) has the same length for every wavefront and entries past the end
// of K multiply a slot of zeros, so the loop body has no branch and every wait counts exactly the loads issued behind
// the one it needs. Rows past N and bytes past K are read from valid addresses of the same matrix (never stored; x is
// zero there). The tiles' partial sums meet in LDS once, at the end, in the then idle x buffers.
constexpr int XL_UNIT_K = 64;
constexpr int XL_SROW = 144;   // staged weight row pitch: 128 bytes + 16 pad
constexpr int XL_T_MAX = 8;    // tiles per block
constexpr int XL_NW = 8, XL_D = 2, XL_CH = 32;
constexpr size_t XL_LDS = 2 * XL_CH * 2048 + 2048 + XL_NW * 16 * XL_SROW;

template <int DT, int NW, int D, int CH>
__global__ __launch_bounds__(NW * 64) void skinny_pair_xlds_kernel(SkinnyParams p) {
    constexpr int COLS = 8;
    constexpr int XS = CH * 2 / NW;      // 1 KiB slots of a chunk of x per wavefront
    constexpr int PER_TILE = CH / NW;    // list entries per tile and chunk
    static_assert(CH % (NW * D) == 0, "every wavefront gets whole groups of D units of a chunk");
    static_assert(XL_T_MAX * NW * 4 * 64 * 4 <= 2 * CH * 2048, "the partial sums fit the x buffers");
    extern __shared__ __align__(16) char smem[];
    // layout: [x: 2 buffers of CH * 2 KiB][2 KiB of zeros][stage: NW * 16 * XL_SROW]
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    char *zeros = smem + 2 * CH * 2048;
    char *stage = zeros + 2048 + wave * (16 * XL_SROW);
    float *red = reinterpret_cast<float *>(smem);

    const int lr = lane & 15, lg = lane >> 4;
    const int crow = lane >> 3, cpiece = lane & 7;
    const int tiles_total = (p.N + COLS - 1) / COLS;
    const int tb = static_cast<int>(static_cast<int64_t>(tiles_total) * blockIdx.x / gridDim.x);
    const int te = static_cast<int>(static_cast<int64_t>(tiles_total) * (blockIdx.x + 1) / gridDim.x);
    const int T = te - tb;
    const int units_total = (p.K + XL_UNIT_K - 1) / XL_UNIT_K;
    const int chunks = (units_total + CH - 1) / CH;
    const uint4 zero4 = make_uint4(0, 0, 0, 0);

    int ic = 0, it = 0, ij = 0;  // issue cursor: chunk, tile, position in the tile's list
    uint4 wv[D][2];
    auto issue = [&](uint4 (&dst)[2]) __attribute__((always_inline)) {
        const bool live = ic < chunks;
        const int c = live ? ic : chunks - 1, t = live ? it : T - 1;
        int u = c * CH + wave + ij * NW;
        u = u < units_total ? u : units_total - 1;
        const int n0 = (tb + t) * COLS;
        const int64_t kbyte = static_cast<int64_t>(u) * (XL_UNIT_K * 2) + cpiece * 16;
        const int64_t kb = kbyte < static_cast<int64_t>(p.K) * 2 ? kbyte : 0;
        const int row = n0 + crow < p.N ? n0 + crow : p.N - 1;
        dst[0] = nt_load_u4(p.w + static_cast<int64_t>(row) * p.ldw * 2 + kb);
        dst[1] = nt_load_u4(p.w2 + static_cast<int64_t>(row) * p.ldw * 2 + kb);
        if (live && ++ij == PER_TILE) {
            ij = 0;
            if (++it == T) { it = 0; ++ic; }
        }
    };
    // this wavefront's slots of a chunk of x: wave, wave + NW, ...
    uint4 xr[XS];
    auto fetch_x = [&](int c) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < XS; ++i) {
            const int sl = wave + i * NW;
            const int k = (c * CH + (sl >> 1)) * XL_UNIT_K + (lg + 4 * (sl & 1)) * 8;
            const bool ok = lr < p.M && k < p.K;
            xr[i] = *reinterpret_cast<const uint4 *>(p.x + (ok ? (static_cast<int64_t>(lr) * p.ldx + k) * 2 : 0));
        }
    };
    auto store_x = [&](int c) __attribute__((always_inline)) {
        char *xb = smem + (c & 1) * (CH * 2048);
#pragma unroll
        for (int i = 0; i < XS; ++i) {
            const int sl = wave + i * NW;
            const int k = (c * CH + (sl >> 1)) * XL_UNIT_K + (lg + 4 * (sl & 1)) * 8;
            const bool ok = lr < p.M && k < p.K;
            const uint4 v = xr[i];
            *reinterpret_cast<uint4 *>(xb + (sl * 64 + lane) * 16) = make_uint4(ok ? v.x : 0u, ok ? v.y : 0u, ok ? v.z : 0u, ok ? v.w : 0u);
        }
    };

    fetch_x(0);
#pragma unroll
    for (int d = 0; d < D; ++d) issue(wv[d]);
    if (wave < 2) *reinterpret_cast<uint4 *>(zeros + (wave * 64 + lane) * 16) = zero4;
    store_x(0);
    __syncthreads();

    f32x4 acc[XL_T_MAX];
#pragma unroll
    for (int t = 0; t < XL_T_MAX; ++t) acc[t] = f32x4{0.f, 0.f, 0.f, 0.f};

    for (int c = 0; c < chunks; ++c) {
        const char *xb = smem + (c & 1) * (CH * 2048);
        if (c + 1 < chunks) fetch_x(c + 1);
        for (int t = 0; t < T; ++t) {
            f32x4 cur = f32x4{0.f, 0.f, 0.f, 0.f};
            for (int i0 = 0; i0 < PER_TILE; i0 += D) {
#pragma unroll
                for (int d = 0; d < D; ++d) {
                    const int ul = wave + (i0 + d) * NW;  // unit within the chunk
                    // fetch order (8 rows x 128 bytes per load) -> MFMA operand order through the wavefront's LDS tile
                    *reinterpret_cast<uint4 *>(stage + crow * XL_SROW + cpiece * 16) = wv[d][0];
                    *reinterpret_cast<uint4 *>(stage + (crow + 8) * XL_SROW + cpiece * 16) = wv[d][1];
                    __builtin_amdgcn_wave_barrier();
                    const uint4 a0 = *reinterpret_cast<const uint4 *>(stage + lr * XL_SROW + lg * 16);
                    const uint4 a1 = *reinterpret_cast<const uint4 *>(stage + lr * XL_SROW + (lg + 4) * 16);
                    const char *xsl = c * CH + ul < units_total ? xb + ul * 2048 : zeros;
                    const uint4 b0 = *reinterpret_cast<const uint4 *>(xsl + lane * 16);
                    const uint4 b1 = *reinterpret_cast<const uint4 *>(xsl + 1024 + lane * 16);
                    __builtin_amdgcn_wave_barrier();
                    issue(wv[d]);
                    cur = mfma16<DT>(a0, b0, cur);
                    cur = mfma16<DT>(a1, b1, cur);
                }
            }
#pragma unroll
            for (int tt = 0; tt < XL_T_MAX; ++tt)
                if (t == tt) acc[tt] += cur;
        }
        if (c + 1 < chunks) store_x(c + 1);
        __syncthreads();  // the next chunk is staged; after the last chunk: everybody is done with x
    }
    // the tiles' partial sums meet in the x buffers; element e -> output (tile e / 256, m = e / 16 % 16, column e % 16 < 8)
#pragma unroll
    for (int tt = 0; tt < XL_T_MAX; ++tt)
        if (tt < T) {
#pragma unroll
            for (int i = 0; i < 4; ++i) red[((tt * NW + wave) * 4 + i) * 64 + lane] = acc[tt][i];
        }
    __syncthreads();
    for (int e = tid; e < T * 256; e += NW * 64) {
        const int tt = e >> 8, m = (e >> 4) & 15, nl = e & 15;
        const int n = (tb + tt) * COLS + nl;
        if (m < p.M && nl < COLS && n < p.N) {
            const int src_lane = (nl >> 2) * 16 + m, i = nl & 3;
            float s0 = 0.f, s1 = 0.f;
#pragma unroll
            for (int w = 0; w < NW; ++w) {
                s0 += red[((tt * NW + w) * 4 + i) * 64 + src_lane];
                s1 += red[((tt * NW + w) * 4 + i) * 64 + src_lane + 32];  // row nl + 8 of the tile: the up sum
            }
            skinny_store_output<DT, SK_SWIGLU>(p, s0, s1, m, n);
        }
    }
}

// Gated pair with 16-bit weights, 4 <= M <= 16, at most XL_T_MAX tiles of 8 columns per CU. *done = false: not taken.
template <int DT>
int launch_pair_xlds(const SkinnyParams &p, int cus, hipStream_t s, bool *done) {
    *done = false;
    if (tuning().skinny_xlds == 0) return TPAMD_OK;
    const int64_t tiles = (p.N + 7) / 8;
    if (p.M < 4 || p.M > 16 || p.K % 8 != 0 || tiles > static_cast<int64_t>(XL_T_MAX) * cus) return TPAMD_OK;
    if (tuning().skinny_xlds == TUNE_UNSET) {
        // Measured against the older kernels (inside a HIP graph, rows 4 / 8 / 16): 5504 columns at K = 4096 19.6 / 21.1 /
        // 21.9 -> 18.5 / 18.9 / 20.3 us, 2752 columns 13.8 / 15.1 / 16.6 -> 13.6 / 13.7 / 15.1 us, 14336 columns 43.3 / 44.9 /
        // 41.1 -> 39.1 / 39.6 / 41.0 us. It loses where the last chunk of K is mostly padding (K = 5504: 86 units in chunks
        // of 32, 11008 columns 46.6 / 50.6 / 48.9 -> 48.1 / 48.8 / 50.1 us) and, below 12 rows, where there is less than one
        // tile per CU (1376 columns at K = 8192, 8 rows: 13.7 -> 15.8 us; 16 rows: 21.5 -> 17.6 us).
        const int units = (p.K + XL_UNIT_K - 1) / XL_UNIT_K, padded = (units + XL_CH - 1) / XL_CH * XL_CH;
        if (padded * 100 > units * 107) return TPAMD_OK;
        if (tiles < cus && p.M < 12) return TPAMD_OK;
        // The later sweep of 220 pair shapes: this kernel is the fastest of the three only for short rows (K below 3072)
        // on more than two tiles per CU (5504 ... 14336 x 2048: 2-8 %); where the x-resident kernel declines a longer K
        // the plain kernel is the better second choice (K = 8192: by 8-41 %).
        if (p.K >= 3072 || tiles <= 2ll * cus) return TPAMD_OK;
    }
    static thread_local int configured_dev = -1;  // per instantiation and host thread
    int dev = 0;
    TPAMD_HIP(hipGetDevice(&dev));
    if (configured_dev != dev) {
        TPAMD_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(skinny_pair_xlds_kernel<DT, XL_NW, XL_D, XL_CH>),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(XL_LDS)));
        configured_dev = dev;
    }
    const unsigned grid = static_cast<unsigned>(tiles < cus ? tiles : cus);
    hipLaunchKernelGGL((skinny_pair_xlds_kernel<DT, XL_NW, XL_D, XL_CH>), dim3(grid), dim3(XL_NW * 64), XL_LDS, s, p);
    TPAMD_HIP(hipGetLastError());
    *done = true;
    return TPAMD_OK;
}

template <int DT, bool W8, int MODE>
int launch_skinny(const SkinnyParams &p, hipStream_t s) {
    if constexpr (W8) {
        bool done = false;
        int rc = launch_w8_cols<DT>(p, s, &done);
        if (rc != TPAMD_OK || done) return rc;
        rc = launch_w8_split<DT>(p, s, &done);
        if (rc != TPAMD_OK || done) return rc;
    }
    if constexpr (!W8) {
        int dev = 0, cus = 256;
        TPAMD_HIP(hipGetDevice(&dev));
        if (int rc_cus = device_cus(dev, &cus); rc_cus != TPAMD_OK) return rc_cus;
        if constexpr (MODE == SK_SWIGLU) {
            if (tuning().skinny_xlds == 1) {  // asked for by name: before the x-resident kernel
                bool done = false;
                const int rc = launch_pair_xlds<DT>(p, cus, s, &done);
                if (rc != TPAMD_OK || done) return rc;
            }
        }
        if (pick_resident<MODE>(p, cus)) return launch_resident<DT, MODE>(p, cus, s);
        if constexpr (MODE == SK_SWIGLU) {
            bool done = false;
            const int rc = launch_pair_xlds<DT>(p, cus, s, &done);
            if (rc != TPAMD_OK || done) return rc;
        }
    }
    if constexpr (MODE == SK_SWIGLU && !W8) {
        if (p.M <= 32 && pick_pair(p)) {
            const unsigned grid8 = static_cast<unsigned>((p.N + 7) / 8);
            if (p.M <= 16) hipLaunchKernelGGL((skinny_kernel<DT, false, 1, MODE, 1, SK_WAVES, true>), dim3(grid8), dim3(SK_THREADS), 0, s, p);
            else hipLaunchKernelGGL((skinny_kernel<DT, false, 2, MODE, 1, SK_WAVES, true>), dim3(grid8), dim3(SK_THREADS), 0, s, p);
            TPAMD_HIP(hipGetLastError());
            return TPAMD_OK;
        }
    }
    int cg = pick_cg(p, W8, MODE == SK_SWIGLU);
    if (MODE == SK_SWIGLU && cg > 2) cg = 2;  // two matrices per group: registers for 2 groups
    const unsigned grid = static_cast<unsigned>((p.N + 16 * cg - 1) / (16 * cg));
    if (cg > 1 && p.M > 32) {
        // the column-group kernels take 32 rows of x at a time; the weights of the later slabs come from L2 / the
        // Infinity Cache rather than HBM when they fit
        for (int m0 = 0; m0 < p.M; m0 += 32) {
            SkinnyParams q = p;
            q.x = p.x + static_cast<int64_t>(m0) * p.ldx * 2;
            q.y = p.y + static_cast<int64_t>(m0) * p.ldy * 2;
            if (p.addend != nullptr) q.addend = p.addend + static_cast<int64_t>(m0) * p.ldadd * 2;
            q.M = p.M - m0 < 32 ? p.M - m0 : 32;
            const int rc = launch_skinny<DT, W8, MODE>(q, s);
            if (rc != TPAMD_OK) return rc;
        }
        return TPAMD_OK;
    }
    if (cg > 1) {
        TPAMD_REQUIRE(p.N % (16 * cg) == 0, "skinny: N %% %d != 0", 16 * cg);
        if constexpr (MODE == SK_SWIGLU) {
            if (p.M <= 16) hipLaunchKernelGGL((skinny_kernel<DT, W8, 1, MODE, 2>), dim3(grid), dim3(SK_THREADS), 0, s, p);
            else hipLaunchKernelGGL((skinny_kernel<DT, W8, 2, MODE, 2>), dim3(grid), dim3(SK_THREADS), 0, s, p);
        } else if (cg == 2) {
            if (p.M <= 16) hipLaunchKernelGGL((skinny_kernel<DT, W8, 1, MODE, 2>), dim3(grid), dim3(SK_THREADS), 0, s, p);
            else hipLaunchKernelGGL((skinny_kernel<DT, W8, 2, MODE, 2>), dim3(grid), dim3(SK_THREADS), 0, s, p);
        } else {
            if (p.M <= 16) hipLaunchKernelGGL((skinny_kernel<DT, W8, 1, MODE, 4>), dim3(grid), dim3(SK_THREADS), 0, s, p);
            else hipLaunchKernelGGL((skinny_kernel<DT, W8, 2, MODE, 4>), dim3(grid), dim3(SK_THREADS), 0, s, p);
        }
    } else {
        const unsigned grid1 = static_cast<unsigned>((p.N + 15) / 16);
        if (p.M <= 16) hipLaunchKernelGGL((skinny_kernel<DT, W8, 1, MODE, 1>), dim3(grid1), dim3(SK_THREADS), 0, s, p);
        else if (p.M <= 32) hipLaunchKernelGGL((skinny_kernel<DT, W8, 2, MODE, 1>), dim3(grid1), dim3(SK_THREADS), 0, s, p);
        else hipLaunchKernelGGL((skinny_kernel<DT, W8, 4, MODE, 1>), dim3(grid1), dim3(SK_THREADS), 0, s, p);
    }
    TPAMD_HIP(hipGetLastError());
    return TPAMD_OK;
}

}  // namespace

// M <= 64. dtype is BF16 or F16. `w8` selects the int8 weight path (linear only).
int skinny_dispatch(const void *x, const void *w, const void *w2, const void *bias, const void *addend, int64_t ldadd,
                    const void *scale, const void *outlier_idx, const void *w_out, int64_t n_out, void *y, int64_t M, int64_t N,
                    int64_t K, int64_t ldx, int64_t ldw, int64_t ldy, int64_t ld_wout, int dtype, int act, bool swiglu, bool w8,
                    hipStream_t s) {
    SkinnyParams p{};
    p.x = static_cast<const char *>(x);
    p.w = static_cast<const char *>(w);
    p.w2 = static_cast<const char *>(w2);
    p.bias = static_cast<const char *>(bias);
    p.scale = static_cast<const float *>(scale);
    p.outlier_idx = static_cast<const int *>(outlier_idx);
    p.w_out = static_cast<const char *>(w_out);
    p.addend = static_cast<const char *>(addend);
    p.ldadd = ldadd;
    p.y = static_cast<char *>(y);
    p.M = static_cast<int>(M); p.N = static_cast<int>(N); p.K = static_cast<int>(K);
    p.n_out = static_cast<int>(n_out);
    p.ldx = ldx; p.ldw = ldw; p.ldy = ldy; p.ld_wout = ld_wout;
    p.act = act;
    const bool bf = dtype == TPAMD_BF16;
    // 2 and 3 rows of int8 weights are faster through the K-split kernel where it applies
    if (w8 && M >= 2 && M <= GEMV_MAX_M) {
        bool done = false;
        const int rc = bf ? launch_w8_cols<TPAMD_BF16>(p, s, &done) : launch_w8_cols<TPAMD_F16>(p, s, &done);
        if (rc != TPAMD_OK || done) return rc;
    }
    if (M <= GEMV_MAX_M && M * K * 2 <= GEMV_MAX_X_BYTES) {
        RowsPath path = ROWS_W8;
        if (!w8) {
            int dev = 0, cus = 256;
            TPAMD_HIP(hipGetDevice(&dev));
            if (int rc_cus = device_cus(dev, &cus); rc_cus != TPAMD_OK) return rc_cus;
            const int knob = tuning().gemv_rows;  // -1: the MFMA kernels; other values: launch_gemv_rows
            path = knob == -1 ? ROWS_MFMA : knob != TUNE_UNSET ? ROWS_W8 : pick_rows_path(swiglu, M, N, K, cus);
        }
        if (path != ROWS_MFMA) {
            bool done = false;
            const int rc = w8 ? (bf ? launch_gemv_rows<TPAMD_BF16, true, SK_LINEAR>(p, s, path, &done) : launch_gemv_rows<TPAMD_F16, true, SK_LINEAR>(p, s, path, &done))
                         : swiglu ? (bf ? launch_gemv_rows<TPAMD_BF16, false, SK_SWIGLU>(p, s, path, &done) : launch_gemv_rows<TPAMD_F16, false, SK_SWIGLU>(p, s, path, &done))
                                  : (bf ? launch_gemv_rows<TPAMD_BF16, false, SK_LINEAR>(p, s, path, &done) : launch_gemv_rows<TPAMD_F16, false, SK_LINEAR>(p, s, path, &done));
            if (rc != TPAMD_OK || done) return rc;
            if (w8) return bf ? launch_gemv<TPAMD_BF16, true, SK_LINEAR>(p, s) : launch_gemv<TPAMD_F16, true, SK_LINEAR>(p, s);
            if (swiglu) return bf ? launch_gemv<TPAMD_BF16, false, SK_SWIGLU>(p, s) : launch_gemv<TPAMD_F16, false, SK_SWIGLU>(p, s);
            return bf ? launch_gemv<TPAMD_BF16, false, SK_LINEAR>(p, s) : launch_gemv<TPAMD_F16, false, SK_LINEAR>(p, s);
        }
    }
    if (w8) return bf ? launch_skinny<TPAMD_BF16, true, SK_LINEAR>(p, s) : launch_skinny<TPAMD_F16, true, SK_LINEAR>(p, s);
    if (swiglu) return bf ? launch_skinny<TPAMD_BF16, false, SK_SWIGLU>(p, s) : launch_skinny<TPAMD_F16, false, SK_SWIGLU>(p, s);
    return bf ? launch_skinny<TPAMD_BF16, false, SK_LINEAR>(p, s) : launch_skinny<TPAMD_F16, false, SK_LINEAR>(p, s);
}

}  // namespace tpamd
