// Rank-shard Linear for prefill-sized M: y[M,N] = act(x[M,K] . w[N,K]^T + bias) on MFMA (bf16/f16),
// and the fused SiLU-gated gate/up pair. Both operands are K-contiguous, so x rows and w rows are
// staged into LDS the same way and fed to the MFMA with w as the row operand: a lane then holds
// 4 consecutive output columns of one output row, which packs into one 8-byte store.
//
// Two kernels share the tiling (block tile BM x BN x 64, WAVES_M x WAVES_N wavefronts of 64 lanes, two LDS
// stages, one barrier per K tile):
//   gemm_direct4_kernel 256x256 tiles, K % 64 == 0, K >= 128, v_mfma_f32_16x16x32. Global loads go straight into LDS
//                       (no register staging); one block of 4 wavefronts (128x128 outputs each, accumulators in
//                       AGPRs) per CU walks through several output tiles; reads and loads of the next step are
//                       placed by hand between the MFMAs of the current one. The default for large problems.
//   gemm_direct_kernel  the same tile with 8 wavefronts (128x64 each): the two wavefronts of a SIMD alternate
//                       between a read phase and a multiply phase. Takes K == 64; within 1-8 % of the 4-wavefront
//                       kernel elsewhere (TPAMD_GEMM_W4=0 selects it).
//   gemm_kernel         any K (multiple of 8) and the 128x128 tiling for small problems, v_mfma_f32_32x32x16; next
//                       K tile prefetched into registers while the current one is multiplied.
#include "common.h"

#include <stdlib.h>
#include <mutex>
#include <type_traits>
#include <vector>

namespace tpamd {
namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8;
typedef __attribute__((ext_vector_type(16))) float f32x16;

enum { MODE_LINEAR = 0, MODE_SWIGLU = 1 };

struct GemmParams {
    const char *x;
    const char *w;   // linear: weight; swiglu: gate weight
    const char *w2;  // swiglu: up weight
    const char *bias;
    const char *addend;  // linear: added to the rounded result (another rank's partial sum), or NULL
    char *y;
    int M, N, K;
    int64_t ldx, ldw, ldy, ldadd;  // elements
    int act;
    int tiles_m, tiles_n;
    float *ws;          // split-K: partial tiles, [split][tile][128 x rows][128 w rows] fp32
    int kt_per_split;   // split-K: K tiles (of 64) per split
    int splits;         // split-K of the 256 x 256 kernel: work units = tiles x splits
};

constexpr int BK = 64;            // K elements per stage (128 bytes of a row)
constexpr int LDS_ROW = 144;      // bytes per staged row: 128 + 16 pad, conflict-free for b128 reads
constexpr int GROUP_M = 4;        // tile rows per L2 reuse group

template <int DT>
__device__ __forceinline__ f32x16 mfma32(uint4 a, uint4 b, f32x16 c) {
    if constexpr (DT == TPAMD_BF16)
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
    else
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
}

// Hardware spreads consecutive workgroup ids round-robin over the 8 XCDs (each with its own L2).
// Give every XCD one contiguous range of logical tile ids, then walk tiles in groups of GROUP_M tile
// rows so that the blocks resident on an XCD at one time share x and w tiles.
__device__ __forceinline__ void tile_of_block(int bid, int nblocks, int tiles_m, int tiles_n, int &tm, int &tn) {
    const int per = nblocks >> 3, rem = nblocks & 7;
    const int xcd = bid & 7, in_xcd = bid >> 3;
    const int logical = (xcd < rem ? xcd * (per + 1) : rem * (per + 1) + (xcd - rem) * per) + in_xcd;
    const int group_size = GROUP_M * tiles_n;
    const int g = logical / group_size;
    const int first_m = g * GROUP_M;
    const int gm = (tiles_m - first_m) < GROUP_M ? (tiles_m - first_m) : GROUP_M;
    const int in_group = logical - g * group_size;
    tm = first_m + in_group % gm;
    tn = in_group / gm;
}

// Epilogue shared by both kernels. D[n_local][m_local]: lane -> m_local = l32, register i -> n_local = 8*(i/4) + 4*lhi + i%4,
// so a lane owns 4 consecutive output columns of one row: one 8-byte store.
template <int DT, int MODE, int BM, int BN, int WAVES_M, int WAVES_N, int TM, int TN>
__device__ __forceinline__ void epilogue(const GemmParams &p, f32x16 (&acc)[TM][TN], int m0, int n0, int wm, int wn, int l32, int lhi) {
#pragma unroll
    for (int a = 0; a < TM; ++a) {
        const int m = m0 + wm * (BM / WAVES_M) + a * 32 + l32;
        if (m >= p.M) continue;
        char *yrow = p.y + static_cast<int64_t>(m) * p.ldy * 2;
        if constexpr (MODE == MODE_SWIGLU) {
#pragma unroll
            for (int b = 0; b < TN / 2; ++b) {
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const int n = n0 + wn * (BN / 2 / WAVES_N) + b * 32 + q * 8 + lhi * 4;
                    if (n >= p.N) continue;  // N is a multiple of 4: the group of 4 is all in or all out
                    uint16_t h[4];
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        const float g = half_to_f32<DT>(f32_to_half<DT>(acc[a][b][q * 4 + j]));
                        const float u = half_to_f32<DT>(f32_to_half<DT>(acc[a][b + TN / 2][q * 4 + j]));
                        const float s = half_to_f32<DT>(f32_to_half<DT>(silu_f32(g)));
                        h[j] = f32_to_half<DT>(s * u);
                    }
                    uint2 o;
                    o.x = h[0] | (static_cast<uint32_t>(h[1]) << 16);
                    o.y = h[2] | (static_cast<uint32_t>(h[3]) << 16);
                    *reinterpret_cast<uint2 *>(yrow + static_cast<int64_t>(n) * 2) = o;
                }
            }
        } else {
#pragma unroll
            for (int b = 0; b < TN; ++b) {
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const int n = n0 + wn * (BN / WAVES_N) + b * 32 + q * 8 + lhi * 4;
                    if (n >= p.N) continue;
                    float bv[4] = {0.f, 0.f, 0.f, 0.f};
                    if (p.bias) {
                        const uint2 braw = *reinterpret_cast<const uint2 *>(p.bias + static_cast<int64_t>(n) * 2);
                        bv[0] = half_to_f32<DT>(braw.x & 0xffffu); bv[1] = half_to_f32<DT>(braw.x >> 16);
                        bv[2] = half_to_f32<DT>(braw.y & 0xffffu); bv[3] = half_to_f32<DT>(braw.y >> 16);
                    }
                    uint16_t h[4];
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        float v = acc[a][b][q * 4 + j] + bv[j];
                        if (p.act == TPAMD_ACT_GELU) v = gelu_erf(v);
                        h[j] = f32_to_half<DT>(v);
                    }
                    uint2 o;
                    o.x = h[0] | (static_cast<uint32_t>(h[1]) << 16);
                    o.y = h[2] | (static_cast<uint32_t>(h[3]) << 16);
                    if (p.addend != nullptr) {
                        const uint2 araw = *reinterpret_cast<const uint2 *>(p.addend + (static_cast<int64_t>(m) * p.ldadd + n) * 2);
                        o.x = add_packed2<DT>(o.x, araw.x);
                        o.y = add_packed2<DT>(o.y, araw.y);
                    }
                    *reinterpret_cast<uint2 *>(yrow + static_cast<int64_t>(n) * 2) = o;
                }
            }
        }
    }
}

template <int DT, int MODE, int BM, int BN, int WAVES_M, int WAVES_N>
__global__ __launch_bounds__(WAVES_M *WAVES_N * 64) void gemm_kernel(GemmParams p) {
    constexpr int NT = WAVES_M * WAVES_N * 64;
    constexpr int TM = BM / WAVES_M / 32;   // 32-row MFMA tiles of x per wave
    constexpr int TN = BN / WAVES_N / 32;   // 32-row MFMA tiles of w per wave
    constexpr int XC = BM * 8 / NT;         // 16-byte chunks of the x tile per thread
    constexpr int WC = BN * 8 / NT;
    constexpr int STAGE = (BM + BN) * LDS_ROW;
    static_assert(BM * 8 % NT == 0 && BN * 8 % NT == 0, "tile/threads mismatch");
    static_assert(MODE == MODE_LINEAR || TN % 2 == 0, "swiglu needs an even number of w tiles per wave");

    extern __shared__ __align__(16) char smem[];

    int tile_m, tile_n;
    tile_of_block(blockIdx.x, gridDim.x, p.tiles_m, p.tiles_n, tile_m, tile_n);
    const int m0 = tile_m * BM;
    // swiglu: a block owns BN/2 columns of h and stages BN/2 gate rows followed by BN/2 up rows
    const int n0 = tile_n * (MODE == MODE_SWIGLU ? BN / 2 : BN);

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int wm = wave / WAVES_N, wn = wave % WAVES_N;
    const int l32 = lane & 31, lhi = lane >> 5;

    // ---- global -> register staging addresses (row clamped so that every load is in bounds) -------
    const int ld_chunk = tid & 7;      // which 16 bytes of the 128-byte row segment
    const int ld_row = tid >> 3;       // + i * (NT / 8)
    const char *xg[XC];
    const char *wg[WC];
#pragma unroll
    for (int i = 0; i < XC; ++i) {
        int r = m0 + ld_row + i * (NT / 8);
        r = r < p.M ? r : p.M - 1;
        xg[i] = p.x + (static_cast<int64_t>(r) * p.ldx + ld_chunk * 8) * 2;
    }
#pragma unroll
    for (int i = 0; i < WC; ++i) {
        const int tr = ld_row + i * (NT / 8);  // row inside the staged w tile
        const char *base = p.w;
        int r;
        if constexpr (MODE == MODE_SWIGLU) {
            base = tr < BN / 2 ? p.w : p.w2;
            r = n0 + (tr < BN / 2 ? tr : tr - BN / 2);
        } else {
            r = n0 + tr;
        }
        r = r < p.N ? r : p.N - 1;
        wg[i] = base + (static_cast<int64_t>(r) * p.ldw + ld_chunk * 8) * 2;
    }
    const int st_off = ld_row * LDS_ROW + ld_chunk * 16;  // + i * (NT/8) * LDS_ROW

    uint4 xr[XC], wr[WC];
    auto load_global = [&](int kt) {
        const int k = kt * BK + ld_chunk * 8;
        const bool ok = k < p.K;  // K is a multiple of 8: a chunk is entirely inside or outside
        // Past the end of K the row's first chunk is fetched instead: a load, not a branch around one (which would turn
        // into a branch per dword). store_lds() writes zeros for x there, so whatever w holds is multiplied by zero.
        const int64_t off = ok ? static_cast<int64_t>(kt) * BK * 2 : -static_cast<int64_t>(ld_chunk) * 16;
#pragma unroll
        for (int i = 0; i < XC; ++i) xr[i] = *reinterpret_cast<const uint4 *>(xg[i] + off);
#pragma unroll
        for (int i = 0; i < WC; ++i) wr[i] = *reinterpret_cast<const uint4 *>(wg[i] + off);
    };
    auto store_lds = [&](int stage, int kt) {
        char *xs = smem + stage * STAGE;
        char *ws = xs + BM * LDS_ROW;
        const bool ok = kt * BK + ld_chunk * 8 < p.K;
#pragma unroll
        for (int i = 0; i < XC; ++i)
            *reinterpret_cast<uint4 *>(xs + st_off + i * (NT / 8) * LDS_ROW) = make_uint4(ok ? xr[i].x : 0u, ok ? xr[i].y : 0u, ok ? xr[i].z : 0u, ok ? xr[i].w : 0u);
#pragma unroll
        for (int i = 0; i < WC; ++i) *reinterpret_cast<uint4 *>(ws + st_off + i * (NT / 8) * LDS_ROW) = wr[i];
    };

    // ---- LDS -> MFMA operand addresses -----------------------------------------------------------------
    int x_rd[TM], w_rd[TN];
#pragma unroll
    for (int t = 0; t < TM; ++t) x_rd[t] = (wm * (BM / WAVES_M) + t * 32 + l32) * LDS_ROW + lhi * 16;
#pragma unroll
    for (int t = 0; t < TN; ++t) {
        int row;
        if constexpr (MODE == MODE_SWIGLU)
            row = (t / (TN / 2)) * (BN / 2) + wn * (BN / 2 / WAVES_N) + (t % (TN / 2)) * 32;
        else
            row = wn * (BN / WAVES_N) + t * 32;
        w_rd[t] = BM * LDS_ROW + (row + l32) * LDS_ROW + lhi * 16;
    }

    f32x16 acc[TM][TN];
#pragma unroll
    for (int a = 0; a < TM; ++a)
#pragma unroll
        for (int b = 0; b < TN; ++b)
#pragma unroll
            for (int i = 0; i < 16; ++i) acc[a][b][i] = 0.0f;

    const int KT = (p.K + BK - 1) / BK;
    load_global(0);
    store_lds(0, 0);
    __syncthreads();

    for (int kt = 0; kt < KT; ++kt) {
        const bool more = kt + 1 < KT;
        if (more) load_global(kt + 1);
        const char *stage = smem + (kt & 1) * STAGE;
#pragma unroll
        for (int ks = 0; ks < BK / 16; ++ks) {
            uint4 xf[TM], wf[TN];
#pragma unroll
            for (int t = 0; t < TM; ++t) xf[t] = *reinterpret_cast<const uint4 *>(stage + x_rd[t] + ks * 32);
#pragma unroll
            for (int t = 0; t < TN; ++t) wf[t] = *reinterpret_cast<const uint4 *>(stage + w_rd[t] + ks * 32);
#pragma unroll
            for (int a = 0; a < TM; ++a)
#pragma unroll
                for (int b = 0; b < TN; ++b) acc[a][b] = mfma32<DT>(wf[b], xf[a], acc[a][b]);
        }
        if (more) store_lds((kt + 1) & 1, kt + 1);
        __syncthreads();
    }

    epilogue<DT, MODE, BM, BN, WAVES_M, WAVES_N>(p, acc, m0, n0, wm, wn, l32, lhi);
}

typedef __attribute__((address_space(3))) void lds_void;
// Global->LDS load through a buffer descriptor: each lane's 16 bytes land at lds_base + lane * 16 (lds_base must be
// the same for the whole wavefront); address = descriptor base + per-lane 32-bit offset + wavefront-uniform
// offset, range-checked by the hardware against the descriptor's extent (a load beyond it returns zeros).
// No per-lane 64-bit address arithmetic is needed to step through K.
__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void *base, uint32_t extent_bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, static_cast<int>(extent_bytes), 0x00020000);
}
__device__ __forceinline__ void buffer_load16_to_lds(__amdgpu_buffer_rsrc_t rsrc, uint32_t lane_off, uint32_t uniform_off, void *lds_base) {
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (lds_void *)lds_base, 16, static_cast<int>(lane_off), static_cast<int>(uniform_off), 0, 0);
}
// Fragment read that the compiler does not see as an LDS access. With ordinary loads it waits for every
// in-flight global->LDS load before each LDS read (it cannot tell that they go to the other stage), which
// serialises the pipeline; this way the waits are the counted ones written out in the main loop.
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
template <int OFFSET>
__device__ __forceinline__ u32x4 lds_read16(uint32_t lds_addr) {
    static_assert(OFFSET >= 0 && OFFSET < 65536, "ds offset field is 16 bits");
    u32x4 v;
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(v) : "v"(lds_addr), "n"(OFFSET));
    return v;
}
__device__ __forceinline__ uint32_t lds_addr_of(const void *p) {
    return static_cast<uint32_t>(reinterpret_cast<uintptr_t>((const __attribute__((address_space(3))) char *)p));
}
// All of this wavefront's loads and LDS accesses done, then the workgroup barrier. The memory clobber keeps
// the compiler from moving LDS accesses across it.
__device__ __forceinline__ void drain_and_barrier() {
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

typedef __attribute__((ext_vector_type(4))) float f32x4;
template <int DT>
__device__ __forceinline__ f32x4 mfma16(u32x4 a, u32x4 b, f32x4 c) {
    if constexpr (DT == TPAMD_BF16)
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
    else
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
}

// Four consecutive output columns n..n+3 of one row, from fp32 sums to the packed 16-bit store value.
// linear: v = bias/activation of g; swiglu: g = gate sums, u = up sums.
template <int DT, int MODE>
__device__ __forceinline__ uint2 finish4(const GemmParams &p, const float (&g)[4], const float (&u)[4], int n, const char *add_row = nullptr) {
    uint2 o;
    if constexpr (MODE == MODE_SWIGLU) {
        // gate and up products rounded to the tensor dtype, then silu and the product each rounded again
        uint32_t out[2];
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const uint32_t g2 = pack2_half<DT>(g[2 * j], g[2 * j + 1]);
            const uint32_t u2 = pack2_half<DT>(u[2 * j], u[2 * j + 1]);
            const uint32_t s2 = pack2_half<DT>(silu_f32(lo_half_to_f32<DT>(g2)), silu_f32(hi_half_to_f32<DT>(g2)));
            out[j] = pack2_half<DT>(lo_half_to_f32<DT>(s2) * lo_half_to_f32<DT>(u2), hi_half_to_f32<DT>(s2) * hi_half_to_f32<DT>(u2));
        }
        o.x = out[0];
        o.y = out[1];
    } else {
        float v[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) v[j] = g[j];
        if (p.bias) {
            const uint2 braw = *reinterpret_cast<const uint2 *>(p.bias + static_cast<int64_t>(n) * 2);
            v[0] += lo_half_to_f32<DT>(braw.x); v[1] += hi_half_to_f32<DT>(braw.x);
            v[2] += lo_half_to_f32<DT>(braw.y); v[3] += hi_half_to_f32<DT>(braw.y);
        }
        if (p.act == TPAMD_ACT_GELU) {
#pragma unroll
            for (int j = 0; j < 4; ++j) v[j] = gelu_erf(v[j]);
        }
        o.x = pack2_half<DT>(v[0], v[1]);
        o.y = pack2_half<DT>(v[2], v[3]);
        if (add_row != nullptr) {  // the row of p.addend this output row belongs to
            const uint2 araw = *reinterpret_cast<const uint2 *>(add_row + static_cast<int64_t>(n) * 2);
            o.x = add_packed2<DT>(o.x, araw.x);
            o.y = add_packed2<DT>(o.y, araw.y);
        }
    }
    return o;
}

// Epilogue of the direct kernels. With w as the first MFMA operand a lane holds D[n = 4*(lane/16) + i][m = lane%16],
// i = 0..3: four consecutive output columns of one output row, one 8-byte store.
// acc[a][b]: a = 16-row tile of x (TMX per wavefront), b = 16-row tile of w (4 per wavefront; swiglu: 2 gate + 2 up).
template <int DT, int MODE, int TMX>
__device__ __forceinline__ void epilogue16(const GemmParams &p, f32x4 (&acc)[TMX][4], int m_wave, int n_wave, int l16, int lq) {
#pragma unroll
    for (int a = 0; a < TMX; ++a) {
        const int m = m_wave + a * 16 + l16;
        if (m >= p.M) continue;
        char *yrow = p.y + static_cast<int64_t>(m) * p.ldy * 2;
#pragma unroll
        for (int b = 0; b < (MODE == MODE_SWIGLU ? 2 : 4); ++b) {
            const int n = n_wave + b * 16 + lq * 4;
            if (n >= p.N) continue;  // N is a multiple of 4: the group of 4 is all in or all out
            float g[4], u[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                g[j] = acc[a][b][j];
                u[j] = MODE == MODE_SWIGLU ? acc[a][(b + 2) & 3][j] : 0.f;
            }
            const char *add_row = MODE == MODE_LINEAR && p.addend != nullptr ? p.addend + static_cast<int64_t>(m) * p.ldadd * 2 : nullptr;
            *reinterpret_cast<uint2 *>(yrow + static_cast<int64_t>(n) * 2) = finish4<DT, MODE>(p, g, u, n, add_row);
        }
    }
}

// Epilogue of the 4-wavefront kernels. A lane holds 4 consecutive columns of one row per accumulator tile; stored like
// that, an instruction would write 32-byte pieces of 16 rows. Instead the packed results of 16 rows x (16 * GB)
// columns go through a wavefront-private LDS slab (16 rows, EP_PITCH bytes apart) and leave as 16 bytes per lane:
// whole 128-byte lines, 8 rows per store instruction, when GB = 4.
// acc[a][b]: a = 16-row tile of x, b = 16-row tile of w. The wavefront's columns are GROUPS runs of 16 * GB; gated pair:
// tile b holds gate sums and tile b + UP the up sums of the same columns. wide: 16-byte stores are aligned.
constexpr int EP_PITCH = 144;
// ADD: the addend (p.addend, not NULL) of the 16 rows after next is requested while the current 16 rows are converted and
// stored, one set of registers ahead: asked for at the point of use, every piece is a full memory round trip with
// nothing else to do on this SIMD (10 us on the 4096 x 4096 x 5504 down projection).
template <int DT, int MODE, bool GELU, int TMX, int NBT, int GROUPS, int GB, int UP, bool ADD = false>
__device__ __forceinline__ void staged_epilogue(const GemmParams &p, f32x4 (&acc)[TMX][NBT], char *slab, int m_wave, int n_wave,
                                                int lane, bool wide) {
    static_assert(GB == 4 || GB == 2, "64 or 32 columns per slab");
    const int l16 = lane & 15, lq = lane >> 4;
    uint2 braw[GROUPS * GB];
    if constexpr (MODE == MODE_LINEAR) {
#pragma unroll
        for (int b = 0; b < GROUPS * GB; ++b) {
            const int n = n_wave + b * 16 + lq * 4;
            braw[b] = p.bias != nullptr && n < p.N ? *reinterpret_cast<const uint2 *>(p.bias + static_cast<int64_t>(n) * 2) : make_uint2(0, 0);
        }
    }
    constexpr int LANES_PER_ROW = GB * 2;            // 16 bytes per lane
    constexpr int ROWS_PER_READ = 64 / LANES_PER_ROW;
    constexpr int READS = 16 / ROWS_PER_READ;
    const int rd_row = lane / LANES_PER_ROW, rd_col = lane % LANES_PER_ROW;
    uint2 addv[2][ADD ? GROUPS * READS : 1][2];
    auto request_addend = [&](int a) {
#pragma unroll
        for (int gq = 0; gq < GROUPS; ++gq)
#pragma unroll
            for (int h = 0; h < READS; ++h) {
                const int m = m_wave + a * 16 + h * ROWS_PER_READ + rd_row;
                const int n = n_wave + gq * (16 * GB) + rd_col * 8;
                const bool in = m < p.M && n < p.N;
                const char *ap = p.addend + (in ? (static_cast<int64_t>(m) * p.ldadd + n) * 2 : 0);
                addv[a & 1][gq * READS + h][0] = *reinterpret_cast<const uint2 *>(ap);
                addv[a & 1][gq * READS + h][1] = in && n + 8 <= p.N ? *reinterpret_cast<const uint2 *>(ap + 8) : make_uint2(0, 0);
            }
    };
    if constexpr (ADD) request_addend(0);
#pragma unroll
    for (int a = 0; a < TMX; ++a) {
        if constexpr (ADD) {
            if (a + 1 < TMX) request_addend(a + 1);
        }
#pragma unroll
        for (int gq = 0; gq < GROUPS; ++gq) {
#pragma unroll
            for (int bb = 0; bb < GB; ++bb) {
                const int b = gq * GB + bb;
                uint2 o;
                if constexpr (MODE == MODE_SWIGLU) {
                    float gsum[4], usum[4];
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        gsum[j] = acc[a][b][j];
                        usum[j] = acc[a][b + UP][j];
                    }
                    o = finish4<DT, MODE>(p, gsum, usum, 0);
                } else {
                    float v[4];
#pragma unroll
                    for (int j = 0; j < 4; ++j) v[j] = acc[a][b][j];
                    v[0] += lo_half_to_f32<DT>(braw[b].x); v[1] += hi_half_to_f32<DT>(braw[b].x);
                    v[2] += lo_half_to_f32<DT>(braw[b].y); v[3] += hi_half_to_f32<DT>(braw[b].y);
                    if constexpr (GELU) {
#pragma unroll
                        for (int j = 0; j < 4; ++j) v[j] = gelu_erf(v[j]);
                    }
                    o.x = pack2_half<DT>(v[0], v[1]);
                    o.y = pack2_half<DT>(v[2], v[3]);
                }
                *reinterpret_cast<uint2 *>(slab + l16 * EP_PITCH + bb * 32 + lq * 8) = o;
            }
            __builtin_amdgcn_wave_barrier();
            asm volatile("" ::: "memory");
#pragma unroll
            for (int h = 0; h < READS; ++h) {
                const int row = h * ROWS_PER_READ + rd_row;
                const uint4 vs = *reinterpret_cast<const uint4 *>(slab + row * EP_PITCH + rd_col * 16);
                const int m = m_wave + a * 16 + row;
                const int n = n_wave + gq * (16 * GB) + rd_col * 8;
                if (m >= p.M || n >= p.N) continue;
                char *dst = p.y + (static_cast<int64_t>(m) * p.ldy + n) * 2;
                uint4 v = vs;
                if constexpr (ADD) {
                    {  // the lane that stores 8 outputs adds the same 8 elements of the addend
                        const uint2 a0 = addv[a & 1][gq * READS + h][0], a1 = addv[a & 1][gq * READS + h][1];
                        v.x = add_packed2<DT>(v.x, a0.x); v.y = add_packed2<DT>(v.y, a0.y);
                        v.z = add_packed2<DT>(v.z, a1.x); v.w = add_packed2<DT>(v.w, a1.y);
                    }
                }
                if (n + 8 <= p.N) {
                    if (wide) *reinterpret_cast<uint4 *>(dst) = v;
                    else {
                        *reinterpret_cast<uint2 *>(dst) = make_uint2(v.x, v.y);
                        *reinterpret_cast<uint2 *>(dst + 8) = make_uint2(v.z, v.w);
                    }
                } else {
                    *reinterpret_cast<uint2 *>(dst) = make_uint2(v.x, v.y);  // N is a multiple of 4
                }
            }
            __builtin_amdgcn_wave_barrier();
            asm volatile("" ::: "memory");
        }
    }
}

// gemm_direct_kernel: 256 x 256 x 64 tiles, 8 wavefronts (2 x 4, 128 x-rows by 64 w-rows each), 2 LDS stages.
//
// MFMA shape: v_mfma_f32_16x16x32. Under the chip's power limit it sustains about 14% more flops than the
// 32x32x16 shape on random operands (it reads and writes a quarter of the accumulator bytes per instruction for
// half the flops), and the main loop is power-bound.
//
// LDS layout: staged rows are grouped in blocks of 8 (1 KiB, what one wavefront-wide 16-byte-per-lane load fills),
// blocks are 1152 bytes apart, and inside a block the 16-byte chunk c of row r sits in slot c ^ (r % 8). Reads of
// one chunk index over 16 consecutive rows are then bank-conflict free, and every group of 8 lanes of a load still
// fetches one whole 128-byte row segment.
//
// Global->LDS loads go through buffer descriptors (wavefront-uniform base and K offset, 32-bit per-lane offset
// computed once), fragment reads are inline ds_read_b128. The main loop runs in phases that end at workgroup
// barriers (described where it is written out): the two wavefronts of a SIMD alternate between reading fragments
// and multiplying. Measured against a loop that interleaved one read or load between MFMAs inside every wavefront:
// same speed on a single round of tiles, 3-7 % faster when a CU runs several tiles in a row.
template <int DT, int MODE>
__global__ __launch_bounds__(512) void gemm_direct_kernel(GemmParams p) {
    constexpr int BM = 256, BN = 256, WAVES_N = 4, NW = 8;
    constexpr int BN_OUT = MODE == MODE_SWIGLU ? BN / 2 : BN;
    constexpr int BLK = 1152;
    constexpr int XREG = (BM / 8) * BLK, WREG = (BN / 8) * BLK, STAGE = XREG + WREG;
    constexpr int XB = BM / 8 / NW, WB = BN / 8 / NW;  // 1 KiB blocks per wavefront per operand
    static_assert(XB == 4 && WB == 4, "8 loads per wavefront per tile");

    extern __shared__ __align__(16) char smem[];

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int wm = wave / WAVES_N, wn = wave % WAVES_N;
    const int l16 = lane & 15, lq = lane >> 4;

    // ---- output tiles of this block: the launch has at most one block per CU and a block walks through tile
    // ids blockIdx.x, blockIdx.x + gridDim.x, ... (gridDim.x is a multiple of 8 whenever there is more than one
    // round, so a block stays with one XCD's share of the tiles)
    const int total_tiles = p.tiles_m * p.tiles_n;
    const int KT = p.K / BK;
    const int last = KT - 1;

    // ---- global -> LDS: lane (rb, slot) of a load fetches chunk slot ^ rb of row rb of its block. The load
    // context (offsets and descriptors) belongs to the tile whose K tiles are being fetched, which is the next
    // output tile while the last K tile of the current one is multiplied.
    const int rb = lane >> 3, slot = lane & 7;
    const int lchunk = slot ^ rb;
    const int wave_s = __builtin_amdgcn_readfirstlane(wave);
    uint32_t x_off[XB], w_off[WB];
    __amdgpu_buffer_rsrc_t x_rsrc, w_rsrc, w2_rsrc;
    auto set_load_tile = [&](int tile_id) {
        int tile_m, tile_n;
        tile_of_block(tile_id, total_tiles, p.tiles_m, p.tiles_n, tile_m, tile_n);
        const int m0 = tile_m * BM, n0 = tile_n * BN_OUT;
        const char *x_base = p.x + static_cast<int64_t>(m0) * p.ldx * 2;
        const char *w_base = p.w + static_cast<int64_t>(n0) * p.ldw * 2;
        const char *w2_base = MODE == MODE_SWIGLU ? p.w2 + static_cast<int64_t>(n0) * p.ldw * 2 : w_base;
#pragma unroll
        for (int i = 0; i < XB; ++i) {
            int r = (wave_s + i * NW) * 8 + rb;
            r = m0 + r < p.M ? r : p.M - 1 - m0;  // clamp to the last valid row of x
            x_off[i] = static_cast<uint32_t>(r) * static_cast<uint32_t>(p.ldx * 2) + lchunk * 16;
        }
#pragma unroll
        for (int i = 0; i < WB; ++i) {
            int tr = (wave_s + i * NW) * 8 + rb;
            if constexpr (MODE == MODE_SWIGLU) tr = tr < BN / 2 ? tr : tr - BN / 2;  // gate rows, then up rows
            tr = n0 + tr < p.N ? tr : p.N - 1 - n0;
            w_off[i] = static_cast<uint32_t>(tr) * static_cast<uint32_t>(p.ldw * 2) + lchunk * 16;
        }
        // descriptor extents: up to the end of the last valid row below the tile origin
        const int x_rows = p.M - m0 < BM ? p.M - m0 : BM;
        const int w_rows = p.N - n0 < BN ? p.N - n0 : BN;
        const uint32_t x_extent = static_cast<uint32_t>(x_rows - 1) * static_cast<uint32_t>(p.ldx * 2) + static_cast<uint32_t>(p.K) * 2;
        const uint32_t w_extent = static_cast<uint32_t>(w_rows - 1) * static_cast<uint32_t>(p.ldw * 2) + static_cast<uint32_t>(p.K) * 2;
        x_rsrc = make_rsrc(x_base, x_extent);
        w_rsrc = make_rsrc(w_base, w_extent);
        w2_rsrc = make_rsrc(w2_base, w_extent);
    };
    auto gx = [&](int i, int kt, int stage) {
        buffer_load16_to_lds(x_rsrc, x_off[i], static_cast<uint32_t>(kt) * (BK * 2), smem + stage * STAGE + (wave_s + i * NW) * BLK);
    };
    auto gw = [&](int i, int kt, int stage) {
        const bool up = MODE == MODE_SWIGLU && (wave_s + i * NW) * 8 >= BN / 2;  // i >= 2: known at compile time
        buffer_load16_to_lds(up ? w2_rsrc : w_rsrc, w_off[i], static_cast<uint32_t>(kt) * (BK * 2),
                             smem + stage * STAGE + XREG + (wave_s + i * NW) * BLK);
    };

    // ---- LDS -> MFMA operands: one per-lane base for x and one for w; the 16-row tiles of a wavefront are a
    // compile-time number of blocks apart, which goes into the instruction's offset field
    constexpr int T16 = 2 * BLK;  // 16 rows
    constexpr int WT1 = T16;
    constexpr int WT2 = MODE == MODE_SWIGLU ? (BN / 2 / 8) * BLK : 2 * T16;  // swiglu: first up tile, 128 staged rows on
    constexpr int WT3 = WT2 + T16;
    int x_rd0, w_rd0;
    {
        const int r = wm * 128 + l16;
        x_rd0 = (r >> 3) * BLK + (r & 7) * 128;
        const int row = (MODE == MODE_SWIGLU ? wn * 32 : wn * 64) + l16;
        w_rd0 = XREG + (row >> 3) * BLK + (row & 7) * 128;
    }
    int kk_off[2];
#pragma unroll
    for (int kk = 0; kk < 2; ++kk) kk_off[kk] = ((kk * 4 + lq) ^ (l16 & 7)) * 16;

    f32x4 acc[8][4];
    const uint32_t smem_base = lds_addr_of(smem);

    // Phased schedule: a K step of 32 is a read phase (12 fragment reads; in the first step also the 8 loads of the
    // following K tile) and a multiply phase (32 MFMAs), every phase ends at a workgroup barrier, and wavefronts
    // 4-7 run one phase behind wavefronts 0-3. Wavefronts w and w + 4 share a SIMD, so on every SIMD one wavefront
    // multiplies while the other reads. g counts K tiles across the output tiles of the block, stage = g & 1:
    //   phase      4g         4g+1       4g+2       4g+3       4g+4
    //   waves 0-3  R(g,0)+L   M(g,0)     R(g,1)     M(g,1)+V   R(g+1,0)+L
    //   waves 4-7  M(g-1,1)   R(g,0)+L   M(g,0)     R(g,1)+V   M(g,1)
    // L = loads of K tile g+1 into the other stage (all of its readers finished before the barrier that starts
    // phase 4g), V = wait for those loads, before the barrier that starts phase 4g+4 where K tile g+1 is read.
    // K tile g+1 is the first K tile of the block's next output tile when g is the last of the current one, so a
    // new output tile starts without a pipeline fill; the epilogue of wavefronts 0-3 runs under the last multiply
    // phase of wavefronts 4-7.
    u32x4 xq[8], wq[4];
#define TPAMD_PP_BARRIER() asm volatile("s_barrier" ::: "memory")
#define TPAMD_PP_READ(stage_off, kk)                                                                                \
    {                                                                                                               \
        const uint32_t xa = smem_base + (stage_off) + x_rd0 + kk_off[kk];                                           \
        const uint32_t wa = smem_base + (stage_off) + w_rd0 + kk_off[kk];                                           \
        wq[0] = lds_read16<0>(wa); wq[1] = lds_read16<WT1>(wa); wq[2] = lds_read16<WT2>(wa); wq[3] = lds_read16<WT3>(wa); \
        xq[0] = lds_read16<0>(xa); xq[1] = lds_read16<1 * T16>(xa); xq[2] = lds_read16<2 * T16>(xa);                \
        xq[3] = lds_read16<3 * T16>(xa); xq[4] = lds_read16<4 * T16>(xa); xq[5] = lds_read16<5 * T16>(xa);          \
        xq[6] = lds_read16<6 * T16>(xa); xq[7] = lds_read16<7 * T16>(xa);                                           \
    }
#define TPAMD_PP_FRAGS                                                                                              \
    "+v"(xq[0]), "+v"(xq[1]), "+v"(xq[2]), "+v"(xq[3]), "+v"(xq[4]), "+v"(xq[5]), "+v"(xq[6]), "+v"(xq[7]),         \
        "+v"(wq[0]), "+v"(wq[1]), "+v"(wq[2]), "+v"(wq[3])
#define TPAMD_PP_LANDED(VM)                                                                                         \
    if (VM) asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" : TPAMD_PP_FRAGS::"memory");                               \
    else asm volatile("s_waitcnt lgkmcnt(0)" : TPAMD_PP_FRAGS::"memory")
#define TPAMD_PP_MMA()                                                                                              \
    _Pragma("unroll") for (int a = 0; a < 8; ++a) _Pragma("unroll") for (int b = 0; b < 4; ++b)                     \
        acc[a][b] = mfma16<DT>(wq[b], xq[a], acc[a][b]);
    // one K tile: reads from stage g & 1, loads K tile `kload` of the load context into the other stage
#define TPAMD_PP_KTILE(LATE, kload)                                                                                 \
    {                                                                                                               \
        const int cur = (g & 1) * STAGE, ns = (g + 1) & 1;                                                          \
        __builtin_amdgcn_sched_barrier(0);                                                                          \
        TPAMD_PP_READ(cur, 0);                                                                                      \
        gx(0, kload, ns); gx(1, kload, ns); gx(2, kload, ns); gx(3, kload, ns);                                     \
        gw(0, kload, ns); gw(1, kload, ns); gw(2, kload, ns); gw(3, kload, ns);                                     \
        TPAMD_PP_LANDED(false); TPAMD_PP_BARRIER();                                                                 \
        __builtin_amdgcn_sched_barrier(0);                                                                          \
        TPAMD_PP_MMA();                                                                                             \
        __builtin_amdgcn_sched_barrier(0);                                                                          \
        TPAMD_PP_BARRIER();                                                                                         \
        TPAMD_PP_READ(cur, 1);                                                                                      \
        TPAMD_PP_LANDED(LATE); TPAMD_PP_BARRIER();                                                                  \
        __builtin_amdgcn_sched_barrier(0);                                                                          \
        TPAMD_PP_MMA();                                                                                             \
        __builtin_amdgcn_sched_barrier(0);                                                                          \
        if (!LATE) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");                                                 \
        TPAMD_PP_BARRIER();                                                                                         \
        ++g;                                                                                                        \
    }
    // all output tiles of the block; LATE = this wavefront runs one phase behind
#define TPAMD_PP_RUN(LATE)                                                                                          \
    for (int tile = blockIdx.x; tile < total_tiles; tile += gridDim.x) {                                            \
        int tile_m, tile_n;                                                                                         \
        tile_of_block(tile, total_tiles, p.tiles_m, p.tiles_n, tile_m, tile_n);                                     \
        _Pragma("unroll") for (int a = 0; a < 8; ++a) _Pragma("unroll") for (int b = 0; b < 4; ++b)                 \
            acc[a][b] = f32x4{0.f, 0.f, 0.f, 0.f};                                                                  \
        for (int kt = 0; kt < last; ++kt) TPAMD_PP_KTILE(LATE, kt + 1);                                             \
        const bool more = tile + static_cast<int>(gridDim.x) < total_tiles;                                         \
        if (more) set_load_tile(tile + gridDim.x);                                                                  \
        /* without a next tile the last K tile is fetched again, into the stage nobody reads any more */            \
        const int kfirst = more ? 0 : last;                                                                         \
        TPAMD_PP_KTILE(LATE, kfirst);                                                                               \
        epilogue16<DT, MODE, 8>(p, acc, tile_m * BM + wm * 128, tile_n * BN_OUT + (MODE == MODE_SWIGLU ? wn * 32 : wn * 64), l16, lq); \
    }

    int g = 0;
    set_load_tile(blockIdx.x);
#pragma unroll
    for (int i = 0; i < XB; ++i) gx(i, 0, 0);
#pragma unroll
    for (int i = 0; i < WB; ++i) gw(i, 0, 0);
    drain_and_barrier();
    if (wave_s < 4) {
        TPAMD_PP_RUN(false);
        TPAMD_PP_BARRIER();
    } else {
        TPAMD_PP_BARRIER();
        TPAMD_PP_RUN(true);
    }
#undef TPAMD_PP_BARRIER
#undef TPAMD_PP_READ
#undef TPAMD_PP_FRAGS
#undef TPAMD_PP_LANDED
#undef TPAMD_PP_MMA
#undef TPAMD_PP_KTILE
#undef TPAMD_PP_RUN
}

// gemm_direct4_kernel: the same 256 x 256 x 64 tile with 4 wavefronts (2 x 2, 128 x-rows by 128 w-rows each), one
// per SIMD with its 64 accumulator tiles in the upper half of the register file. A 128 x 128 wavefront tile reads 16
// fragments per 64 MFMAs where the 128 x 64 tile of the 8-wavefront kernel reads 12 per 32: a third less LDS traffic
// per flop, and half the wavefronts to issue loads and waits for. With a single wavefront per SIMD the reads and
// loads of the next step have to be spread between the MFMAs of the current one by hand:
//   step (g,0)  64 MFMAs on buffer 0; the 16 fragment reads of (g,1) follow the first 32, one per pair
//   barrier     every wavefront has read stage g&1 for the last time; K tile g+1 has landed
//   step (g,1)  64 MFMAs on buffer 1; the 16 reads of (g+1,0) follow the first 32; the 16 loads of K tile g+2 (into
//               stage g&1) are spread evenly over the step: bunched up they queue in the load path and land late
// Loads run two K tiles ahead of the multiplies, across output tiles (persistent blocks, as in the 8-wavefront kernel).
// SPLIT: a block's unit of work is (tile, K range of p.kt_per_split K tiles, at least 2); unit u is tile u % tiles,
// split u / tiles. Each wavefront leaves its 128 x 128 fp32 sums as one partial tile of the 128 x 128 tiling in p.ws,
// in the layout splitk_finish_kernel reads.
template <int DT, int MODE, bool SPLIT>
__global__ __launch_bounds__(256) void gemm_direct4_kernel(GemmParams p) {
    constexpr int BM = 256, BN = 256, NW = 4;
    constexpr int BN_OUT = MODE == MODE_SWIGLU ? BN / 2 : BN;
    constexpr int BLK = 1152;
    constexpr int XREG = (BM / 8) * BLK, WREG = (BN / 8) * BLK, STAGE = XREG + WREG;
    constexpr int XB = BM / 8 / NW, WB = BN / 8 / NW;
    static_assert(XB == 8 && WB == 8, "16 loads per wavefront per tile");

    extern __shared__ __align__(16) char smem[];

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int l16 = lane & 15, lq = lane >> 4;
    const int total_tiles = p.tiles_m * p.tiles_n;
    const int total_units = SPLIT ? total_tiles * p.splits : total_tiles;
    const int KT_ALL = p.K / BK;  // at least 2

    const int rb = lane >> 3, slot = lane & 7;
    const int lchunk = slot ^ rb;
    const int wave_s = __builtin_amdgcn_readfirstlane(wave);
    uint32_t x_off[XB], w_off[WB];
    __amdgpu_buffer_rsrc_t x_rsrc, w_rsrc, w2_rsrc;
    int kbase = 0;  // first K tile of the unit the loads are fetching
    auto set_load_tile = [&](int unit) {
        int tile_m, tile_n;
        const int tile_id = SPLIT ? unit % total_tiles : unit;
        if constexpr (SPLIT) kbase = (unit / total_tiles) * p.kt_per_split;
        tile_of_block(tile_id, total_tiles, p.tiles_m, p.tiles_n, tile_m, tile_n);
        const int m0 = tile_m * BM, n0 = tile_n * BN_OUT;
        const char *x_base = p.x + static_cast<int64_t>(m0) * p.ldx * 2;
        const char *w_base = p.w + static_cast<int64_t>(n0) * p.ldw * 2;
        const char *w2_base = MODE == MODE_SWIGLU ? p.w2 + static_cast<int64_t>(n0) * p.ldw * 2 : w_base;
        // A wavefront fetches 8 consecutive 1 KiB blocks (64 rows) of each operand. Four consecutive blocks share one
        // LDS base (M0) and differ in the instruction's immediate offset, which the hardware also adds to the global
        // address: it is taken off the per-lane offset here. A valid row is at least 8 * (i % 4) rows into the tile,
        // i.e. at least (i % 4) * 2048 bytes (K >= 128), so the difference stays non-negative; rows past the end are
        // clamped to the last valid row first, and if the difference then wraps, the range check returns zeros for
        // them, which is as good as any other value for rows whose outputs are not stored.
#pragma unroll
        for (int i = 0; i < XB; ++i) {
            int r = (wave_s * XB + i) * 8 + rb;
            r = m0 + r < p.M ? r : p.M - 1 - m0;
            x_off[i] = static_cast<uint32_t>(r) * static_cast<uint32_t>(p.ldx * 2) + lchunk * 16 - (i & 3) * BLK;
        }
#pragma unroll
        for (int i = 0; i < WB; ++i) {
            int tr = (wave_s * WB + i) * 8 + rb;
            if constexpr (MODE == MODE_SWIGLU) tr = tr < BN / 2 ? tr : tr - BN / 2;
            tr = n0 + tr < p.N ? tr : p.N - 1 - n0;
            w_off[i] = static_cast<uint32_t>(tr) * static_cast<uint32_t>(p.ldw * 2) + lchunk * 16 - (i & 3) * BLK;
        }
        const int x_rows = p.M - m0 < BM ? p.M - m0 : BM;
        const int w_rows = p.N - n0 < BN ? p.N - n0 : BN;
        const uint32_t x_extent = static_cast<uint32_t>(x_rows - 1) * static_cast<uint32_t>(p.ldx * 2) + static_cast<uint32_t>(p.K) * 2;
        const uint32_t w_extent = static_cast<uint32_t>(w_rows - 1) * static_cast<uint32_t>(p.ldw * 2) + static_cast<uint32_t>(p.K) * 2;
        x_rsrc = make_rsrc(x_base, x_extent);
        w_rsrc = make_rsrc(w_base, w_extent);
        w2_rsrc = make_rsrc(w2_base, w_extent);
    };
    auto gx = [&](auto ic, int kt, int stage) {
        constexpr int i = decltype(ic)::value;
        __builtin_amdgcn_raw_ptr_buffer_load_lds(x_rsrc, (lds_void *)(smem + stage * STAGE + (wave_s * XB + (i & ~3)) * BLK), 16,
                                                 static_cast<int>(x_off[i]), (kbase + kt) * (BK * 2), (i & 3) * BLK, 0);
    };
    auto gw = [&](auto ic, int kt, int stage) {
        constexpr int i = decltype(ic)::value;
        const bool up = MODE == MODE_SWIGLU && wave_s >= NW / 2;  // wavefronts 2 and 3 fetch the up rows
        __builtin_amdgcn_raw_ptr_buffer_load_lds(up ? w2_rsrc : w_rsrc, (lds_void *)(smem + stage * STAGE + XREG + (wave_s * WB + (i & ~3)) * BLK), 16,
                                                 static_cast<int>(w_off[i]), (kbase + kt) * (BK * 2), (i & 3) * BLK, 0);
    };
#define IC(n) std::integral_constant<int, n>{}

    constexpr int T16 = 2 * BLK;  // 16 staged rows
    constexpr int WHI = MODE == MODE_SWIGLU ? (BN / 2 / 8) * BLK : 4 * T16;  // w tiles 4-7: the up rows / the next 64 rows
    int x_rd0, w_rd0;
    {
        const int r = wm * 128 + l16;
        x_rd0 = (r >> 3) * BLK + (r & 7) * 128;
        const int row = (MODE == MODE_SWIGLU ? wn * 64 : wn * 128) + l16;
        w_rd0 = XREG + (row >> 3) * BLK + (row & 7) * 128;
    }
    int kk_off[2];
#pragma unroll
    for (int kk = 0; kk < 2; ++kk) kk_off[kk] = ((kk * 4 + lq) ^ (l16 & 7)) * 16;

    f32x4 acc[8][8];
    u32x4 xq[2][8], wq[2][8];
    const uint32_t smem_base = lds_addr_of(smem);
    // epilogue staging behind the two stages: 16 rows x 64 packed outputs per wavefront
    char *ep_slab = smem + 2 * STAGE + wave * (16 * EP_PITCH);
    const bool wide_stores = (reinterpret_cast<uintptr_t>(p.y) & 15) == 0 && p.ldy % 8 == 0;

#define T4_SB __builtin_amdgcn_sched_barrier(0)
#define T4_MFMA(buf, a, b) acc[a][b] = mfma16<DT>(wq[buf][b], xq[buf][a], acc[a][b])
#define T4_PAIR(buf, a, b) T4_MFMA(buf, a, b); T4_MFMA(buf, a, (b) + 1); T4_SB
#define T4_LANDED(buf)                                                                                              \
    asm volatile("s_waitcnt lgkmcnt(0)"                                                                             \
                 : "+v"(xq[buf][0]), "+v"(xq[buf][1]), "+v"(xq[buf][2]), "+v"(xq[buf][3]), "+v"(xq[buf][4]),        \
                   "+v"(xq[buf][5]), "+v"(xq[buf][6]), "+v"(xq[buf][7]), "+v"(wq[buf][0]), "+v"(wq[buf][1]),        \
                   "+v"(wq[buf][2]), "+v"(wq[buf][3]), "+v"(wq[buf][4]), "+v"(wq[buf][5]), "+v"(wq[buf][6]),        \
                   "+v"(wq[buf][7])::"memory")
    // 64 MFMAs on fragment buffer CUR; reads the fragments of (rd_stage_off, rd_kk) into buffer NXT; L0..L15: loads
#define T4_STEP(CUR, NXT, rd_stage_off, rd_kk, L0, L1, L2, L3, L4, L5, L6, L7, L8, L9, L10, L11, L12, L13, L14, L15) \
    {                                                                                                               \
        const uint32_t xa = smem_base + (rd_stage_off) + x_rd0 + kk_off[rd_kk];                                     \
        const uint32_t wa = smem_base + (rd_stage_off) + w_rd0 + kk_off[rd_kk];                                     \
        T4_SB; T4_LANDED(CUR); T4_SB;                                                                               \
        T4_PAIR(CUR, 0, 0); wq[NXT][0] = lds_read16<0>(wa); T4_SB;                                                  \
        T4_PAIR(CUR, 0, 2); wq[NXT][1] = lds_read16<1 * T16>(wa); T4_SB; L0; T4_SB;                                 \
        T4_PAIR(CUR, 0, 4); wq[NXT][2] = lds_read16<2 * T16>(wa); T4_SB;                                            \
        T4_PAIR(CUR, 0, 6); wq[NXT][3] = lds_read16<3 * T16>(wa); T4_SB; L1; T4_SB;                                 \
        T4_PAIR(CUR, 1, 0); wq[NXT][4] = lds_read16<WHI>(wa); T4_SB;                                                \
        T4_PAIR(CUR, 1, 2); wq[NXT][5] = lds_read16<WHI + 1 * T16>(wa); T4_SB; L2; T4_SB;                           \
        T4_PAIR(CUR, 1, 4); wq[NXT][6] = lds_read16<WHI + 2 * T16>(wa); T4_SB;                                      \
        T4_PAIR(CUR, 1, 6); wq[NXT][7] = lds_read16<WHI + 3 * T16>(wa); T4_SB; L3; T4_SB;                           \
        T4_PAIR(CUR, 2, 0); xq[NXT][0] = lds_read16<0>(xa); T4_SB;                                                  \
        T4_PAIR(CUR, 2, 2); xq[NXT][1] = lds_read16<1 * T16>(xa); T4_SB; L4; T4_SB;                                 \
        T4_PAIR(CUR, 2, 4); xq[NXT][2] = lds_read16<2 * T16>(xa); T4_SB;                                            \
        T4_PAIR(CUR, 2, 6); xq[NXT][3] = lds_read16<3 * T16>(xa); T4_SB; L5; T4_SB;                                 \
        T4_PAIR(CUR, 3, 0); xq[NXT][4] = lds_read16<4 * T16>(xa); T4_SB;                                            \
        T4_PAIR(CUR, 3, 2); xq[NXT][5] = lds_read16<5 * T16>(xa); T4_SB; L6; T4_SB;                                 \
        T4_PAIR(CUR, 3, 4); xq[NXT][6] = lds_read16<6 * T16>(xa); T4_SB;                                            \
        T4_PAIR(CUR, 3, 6); xq[NXT][7] = lds_read16<7 * T16>(xa); T4_SB; L7; T4_SB;                                 \
        T4_PAIR(CUR, 4, 0); T4_PAIR(CUR, 4, 2); L8; T4_SB; T4_PAIR(CUR, 4, 4); T4_PAIR(CUR, 4, 6); L9; T4_SB;       \
        T4_PAIR(CUR, 5, 0); T4_PAIR(CUR, 5, 2); L10; T4_SB; T4_PAIR(CUR, 5, 4); T4_PAIR(CUR, 5, 6); L11; T4_SB;     \
        T4_PAIR(CUR, 6, 0); T4_PAIR(CUR, 6, 2); L12; T4_SB; T4_PAIR(CUR, 6, 4); T4_PAIR(CUR, 6, 6); L13; T4_SB;     \
        T4_PAIR(CUR, 7, 0); T4_PAIR(CUR, 7, 2); L14; T4_SB; T4_PAIR(CUR, 7, 4); T4_PAIR(CUR, 7, 6); L15; T4_SB;     \
    }
#define T4_NOP (void)0
#define T4_TILE_BARRIER() asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory")
    // one K tile; kload = K tile (of the load context) fetched into the stage this one leaves
#define T4_KTILE(kload)                                                                                             \
    {                                                                                                               \
        const int cur = (g & 1) * STAGE, nxt = ((g + 1) & 1) * STAGE, cs = g & 1;                                   \
        T4_STEP(0, 1, cur, 1, T4_NOP, T4_NOP, T4_NOP, T4_NOP, T4_NOP, T4_NOP, T4_NOP, T4_NOP, T4_NOP, T4_NOP, T4_NOP, T4_NOP, T4_NOP, \
                T4_NOP, T4_NOP, T4_NOP);                                                                            \
        T4_TILE_BARRIER();                                                                                          \
        T4_STEP(1, 0, nxt, 0, gx(IC(0), kload, cs), gx(IC(1), kload, cs), gx(IC(2), kload, cs), gx(IC(3), kload, cs), gx(IC(4), kload, cs), gx(IC(5), kload, cs), \
                gx(IC(6), kload, cs), gx(IC(7), kload, cs), gw(IC(0), kload, cs), gw(IC(1), kload, cs), gw(IC(2), kload, cs), gw(IC(3), kload, cs),    \
                gw(IC(4), kload, cs), gw(IC(5), kload, cs), gw(IC(6), kload, cs), gw(IC(7), kload, cs));                            \
        ++g;                                                                                                        \
    }

    int g = 0;
    set_load_tile(blockIdx.x);
#define T4_ALL_LOADS(kt, stage)                                                                                     \
    gx(IC(0), kt, stage); gx(IC(1), kt, stage); gx(IC(2), kt, stage); gx(IC(3), kt, stage); gx(IC(4), kt, stage);   \
    gx(IC(5), kt, stage); gx(IC(6), kt, stage); gx(IC(7), kt, stage); gw(IC(0), kt, stage); gw(IC(1), kt, stage);   \
    gw(IC(2), kt, stage); gw(IC(3), kt, stage); gw(IC(4), kt, stage); gw(IC(5), kt, stage); gw(IC(6), kt, stage);   \
    gw(IC(7), kt, stage)
    // both K tiles are requested at once; loads return in order, so the first 16 being back means K tile 0 is there
    T4_ALL_LOADS(0, 0);
    T4_ALL_LOADS(1, 1);
    asm volatile("s_waitcnt vmcnt(16)\n\ts_barrier" ::: "memory");
#undef T4_ALL_LOADS
    {
        const uint32_t xa = smem_base + x_rd0 + kk_off[0];
        const uint32_t wa = smem_base + w_rd0 + kk_off[0];
        wq[0][0] = lds_read16<0>(wa); wq[0][1] = lds_read16<1 * T16>(wa); wq[0][2] = lds_read16<2 * T16>(wa); wq[0][3] = lds_read16<3 * T16>(wa);
        wq[0][4] = lds_read16<WHI>(wa); wq[0][5] = lds_read16<WHI + 1 * T16>(wa); wq[0][6] = lds_read16<WHI + 2 * T16>(wa); wq[0][7] = lds_read16<WHI + 3 * T16>(wa);
        xq[0][0] = lds_read16<0>(xa); xq[0][1] = lds_read16<1 * T16>(xa); xq[0][2] = lds_read16<2 * T16>(xa); xq[0][3] = lds_read16<3 * T16>(xa);
        xq[0][4] = lds_read16<4 * T16>(xa); xq[0][5] = lds_read16<5 * T16>(xa); xq[0][6] = lds_read16<6 * T16>(xa); xq[0][7] = lds_read16<7 * T16>(xa);
    }
    for (int unit = blockIdx.x; unit < total_units; unit += SPLIT ? total_units : static_cast<int>(gridDim.x)) {
        int tile_m, tile_n;
        const int tile = SPLIT ? unit % total_tiles : unit;
        const int split = SPLIT ? unit / total_tiles : 0;
        const int KT = SPLIT ? min(p.kt_per_split, KT_ALL - split * p.kt_per_split) : KT_ALL;
        const int last = KT - 1;
        tile_of_block(tile, total_tiles, p.tiles_m, p.tiles_n, tile_m, tile_n);
#pragma unroll
        for (int a = 0; a < 8; ++a)
#pragma unroll
            for (int b = 0; b < 8; ++b) acc[a][b] = f32x4{0.f, 0.f, 0.f, 0.f};
        for (int kt = 0; kt + 2 < KT; ++kt) T4_KTILE(kt + 2);
        const bool more = !SPLIT && unit + static_cast<int>(gridDim.x) < total_units;  // split: one unit per block
        if (more) set_load_tile(unit + gridDim.x);
        // without a next tile the last K tile is fetched again, into stages nobody reads any more
        const int k0 = more ? 0 : last, k1 = more ? 1 : last;
        T4_KTILE(k0);
        T4_KTILE(k1);
        if constexpr (SPLIT) {
            // the wavefront's sums are tile (2 tile_m + wm, 2 tile_n + wn) of the 128 x 128 tiling; partial tile
            // [x row][w row]: a lane's 4 values are 4 consecutive w rows of one x row, one 16-byte store
            const int tm128 = (p.M + 127) / 128, tn128 = (p.N + BN_OUT / 2 - 1) / (BN_OUT / 2);
            int split_now = split;
            asm volatile("" : "+s"(split_now));  // keeps the address arithmetic below out of the K loop's registers
            const int m128 = tile_m * 2 + wm, n128 = tile_n * 2 + wn;
            if (m128 < tm128 && n128 < tn128) {
                float *ws = p.ws + (static_cast<int64_t>(split_now) * tm128 * tn128 + m128 * tn128 + n128) * (128 * 128) + l16 * 128 + lq * 4;
                // the stores below are asm statements: the compiler does not count the wait states a memory
                // instruction needs before it may read registers an MFMA has just written
                asm volatile("s_nop 7\n\ts_nop 7\n\ts_nop 3" ::: "memory");
#pragma unroll
                for (int a = 0; a < 8; ++a) {
                    typedef __attribute__((address_space(1))) float global_float;
                    global_float *wsa = (global_float *)(ws + a * 16 * 128);
                    asm volatile("" : "+v"(wsa));  // one address per x tile, the rest are store offsets
                    if (m128 * 128 + a * 16 + l16 >= p.M) continue;  // the finishing pass reads valid rows only
#pragma unroll
                    for (int b = 0; b < 8; ++b)
                        // Stored from accumulator registers. The no-ops are the wait states a store of more than 8
                        // bytes needs before its data registers may be written again: the compiler does not see
                        // into the asm statement and may reuse them in the very next instruction.
                        asm volatile("global_store_dwordx4 %0, %1, off offset:%2\n\ts_nop 2" ::"v"(wsa), "a"(acc[a][b]), "n"(b * 64) : "memory");
                }
            }
            continue;
        }
        // epilogue: acc[a][b], b = w tile; gated pair: tiles 0-3 gate, 4-7 up
        const int m_wave = tile_m * BM + wm * 128;
        const int n_wave = tile_n * BN_OUT + (MODE == MODE_SWIGLU ? wn * 64 : wn * 128);
        if constexpr (MODE == MODE_SWIGLU) {
            staged_epilogue<DT, MODE, false, 8, 8, 1, 4, 4>(p, acc, ep_slab, m_wave, n_wave, lane, wide_stores);
        } else {
            if (p.act == TPAMD_ACT_GELU) {
                if (p.addend != nullptr) staged_epilogue<DT, MODE, true, 8, 8, 2, 4, 0, true>(p, acc, ep_slab, m_wave, n_wave, lane, wide_stores);
                else staged_epilogue<DT, MODE, true, 8, 8, 2, 4, 0>(p, acc, ep_slab, m_wave, n_wave, lane, wide_stores);
            } else if (p.addend != nullptr) staged_epilogue<DT, MODE, false, 8, 8, 2, 4, 0, true>(p, acc, ep_slab, m_wave, n_wave, lane, wide_stores);
            else staged_epilogue<DT, MODE, false, 8, 8, 2, 4, 0>(p, acc, ep_slab, m_wave, n_wave, lane, wide_stores);
        }
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // no global->LDS load in flight when the wavefront leaves
#undef T4_SB
#undef T4_MFMA
#undef T4_PAIR
#undef T4_LANDED
#undef T4_STEP
#undef T4_NOP
#undef T4_KTILE
#undef IC
#undef T4_TILE_BARRIER
}

// gemm_direct128_kernel: 128 x 128 x 64 tiles for problems whose 256 x 256 tiling would leave CUs idle.
// 4 wavefronts (2 x 2, 64 x-rows by 64 w-rows each), NS LDS stages of 36 KiB: NS = 2 lets two blocks share a CU,
// NS = 4 gives one block three tiles of look-ahead. Same LDS layout, loads, fragment reads and hand-ordered loop
// body as the 256 kernel; a K tile is two sub-steps of 16 MFMAs with the tile's barrier between them:
//   S1 (k 0..31)   reads the fragments of k 32..63;           loads: second half of tile kt + NS - 1
//   barrier        tile kt+1 has landed (at most (NS-2)*8 younger loads in flight), tile kt is read out
//   S2 (k 32..63)  reads the fragments of k 0..31 of tile kt+1; loads: first half of tile kt + NS into the freed stage
// SPLIT: the block covers K tiles [blockIdx.y * kt_per_split, ...) and leaves its fp32 partial tile in p.ws for
// splitk_finish_kernel.
// XQ < 4 (SPLIT, single matrix, M <= 32 * XQ): only the first XQ quarters of the x tile exist. The loads of the others
// are left out, and the two wavefronts that own x rows 64-127 only load: they read no fragments and multiply nothing,
// so LDS serves the other two and the incoming tiles alone. Measured at 17-64 rows inside a HIP graph: 4096 x 5504
// 17.3-19.2 -> 15.5-17.8 us, 4096 x 4096 14.2-15.6 -> 12.8-14.5 us, 8192 x 8192 29.0-33.0 -> 27.8-32.0 us, no difference from
// 11008 columns on (whole tiles there); leaving out the loads alone gives 1-2 %. The gated pair is 1-5 % slower this way (its wavefronts
// have half as many columns each) and keeps whole tiles.
template <int DT, int MODE, int NS, bool SPLIT, int XQ = 4>
__global__ __launch_bounds__(256) void gemm_direct128_kernel(GemmParams p) {
    static_assert(XQ == 4 || (SPLIT && MODE == MODE_LINEAR && (XQ == 1 || XQ == 2)), "part tiles of x: split kernel, single matrix");
    constexpr int BM = 128, BN = 128, WAVES_N = 2, NW = 4;
    constexpr int BLK = 1152;
    constexpr int XREG = (BM / 8) * BLK, WREG = (BN / 8) * BLK, STAGE = XREG + WREG;
    constexpr int XB = BM / 8 / NW, WB = BN / 8 / NW;
    static_assert(XB == 4 && WB == 4, "8 loads per wavefront per tile");
    static_assert(NS == 2 || NS == 4, "stage index is taken with a mask");

    extern __shared__ __align__(16) char smem[];

    int tile_m, tile_n;
    tile_of_block(blockIdx.x, gridDim.x, p.tiles_m, p.tiles_n, tile_m, tile_n);
    const int m0 = tile_m * BM;
    const int n0 = tile_n * (MODE == MODE_SWIGLU ? BN / 2 : BN);

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int wm = wave / WAVES_N, wn = wave % WAVES_N;
    const int l16 = lane & 15, lq = lane >> 4;

    const int rb = lane >> 3, slot = lane & 7;
    const int lchunk = slot ^ rb;
    const int wave_s = __builtin_amdgcn_readfirstlane(wave);
    const char *x_base = p.x + static_cast<int64_t>(m0) * p.ldx * 2;
    const char *w_base = p.w + static_cast<int64_t>(n0) * p.ldw * 2;
    const char *w2_base = MODE == MODE_SWIGLU ? p.w2 + static_cast<int64_t>(n0) * p.ldw * 2 : w_base;
    uint32_t x_off[XB], w_off[WB];
#pragma unroll
    for (int i = 0; i < XB; ++i) {
        int r = (wave_s + i * NW) * 8 + rb;
        r = m0 + r < p.M ? r : p.M - 1 - m0;
        x_off[i] = static_cast<uint32_t>(r) * static_cast<uint32_t>(p.ldx * 2) + lchunk * 16;
    }
#pragma unroll
    for (int i = 0; i < WB; ++i) {
        int tr = (wave_s + i * NW) * 8 + rb;
        if constexpr (MODE == MODE_SWIGLU) tr = tr < BN / 2 ? tr : tr - BN / 2;  // gate rows, then up rows
        tr = n0 + tr < p.N ? tr : p.N - 1 - n0;
        w_off[i] = static_cast<uint32_t>(tr) * static_cast<uint32_t>(p.ldw * 2) + lchunk * 16;
    }
    const int x_rows = p.M - m0 < BM ? p.M - m0 : BM;
    const int w_rows = p.N - n0 < BN ? p.N - n0 : BN;
    const uint32_t x_extent = static_cast<uint32_t>(x_rows - 1) * static_cast<uint32_t>(p.ldx * 2) + static_cast<uint32_t>(p.K) * 2;
    const uint32_t w_extent = static_cast<uint32_t>(w_rows - 1) * static_cast<uint32_t>(p.ldw * 2) + static_cast<uint32_t>(p.K) * 2;
    const __amdgpu_buffer_rsrc_t x_rsrc = make_rsrc(x_base, x_extent);
    const __amdgpu_buffer_rsrc_t w_rsrc = make_rsrc(w_base, w_extent);
    const __amdgpu_buffer_rsrc_t w2_rsrc = make_rsrc(w2_base, w_extent);

    // this block's K tiles: [kt0, kt0 + nk)
    const int KT = p.K / BK;
    const int kt0 = SPLIT ? static_cast<int>(blockIdx.y) * p.kt_per_split : 0;
    const int nk = SPLIT ? (KT - kt0 < p.kt_per_split ? KT - kt0 : p.kt_per_split) : KT;
    const int last = nk - 1;
    // loads of local tile j (clamped to the last one: such loads refill a stage nobody reads any more and keep
    // the loop free of branches)
    auto gx = [&](int i, int j) {
        if (i >= XQ) return;  // i is a constant at every call
        const int jj = j < last ? j : last;
        buffer_load16_to_lds(x_rsrc, x_off[i], static_cast<uint32_t>(kt0 + jj) * (BK * 2), smem + (j & (NS - 1)) * STAGE + (wave_s + i * NW) * BLK);
    };
    auto gw = [&](int i, int j) {
        const int jj = j < last ? j : last;
        const bool up = MODE == MODE_SWIGLU && (wave_s + i * NW) * 8 >= BN / 2;  // i >= 2: known at compile time
        buffer_load16_to_lds(up ? w2_rsrc : w_rsrc, w_off[i], static_cast<uint32_t>(kt0 + jj) * (BK * 2),
                             smem + (j & (NS - 1)) * STAGE + XREG + (wave_s + i * NW) * BLK);
    };

    constexpr int T16 = 2 * BLK;
    constexpr int WT1 = T16;
    constexpr int WT2 = MODE == MODE_SWIGLU ? (BN / 2 / 8) * BLK : 2 * T16;  // swiglu: first up tile, 64 staged rows on
    constexpr int WT3 = WT2 + T16;
    int x_rd0, w_rd0;
    {
        const int r = wm * 64 + l16;
        x_rd0 = (r >> 3) * BLK + (r & 7) * 128;
        const int row = (MODE == MODE_SWIGLU ? wn * 32 : wn * 64) + l16;
        w_rd0 = XREG + (row >> 3) * BLK + (row & 7) * 128;
    }
    int kk_off[2];
#pragma unroll
    for (int kk = 0; kk < 2; ++kk) kk_off[kk] = ((kk * 4 + lq) ^ (l16 & 7)) * 16;

    f32x4 acc[4][4];
#pragma unroll
    for (int a = 0; a < 4; ++a)
#pragma unroll
        for (int b = 0; b < 4; ++b) acc[a][b] = f32x4{0.f, 0.f, 0.f, 0.f};

    u32x4 xf[2][4], wf[2][4];
    const uint32_t smem_base = lds_addr_of(smem);
#define TPAMD_SB __builtin_amdgcn_sched_barrier(0)
#define TPAMD_WAIT(N, reg) asm volatile("s_waitcnt lgkmcnt(" #N ")" : "+v"(reg))
#define TPAMD_MFMA(S, a, b) acc[a][b] = mfma16<DT>(wf[S][b], xf[S][a], acc[a][b])
#define TPAMD_ROW(S, a) TPAMD_MFMA(S, a, 0); TPAMD_MFMA(S, a, 1); TPAMD_MFMA(S, a, 2); TPAMD_MFMA(S, a, 3)
    // 16 MFMAs on fragment set MS (read in the order x0 w0 w1 w2 w3 x1 x2 x3); the same 8 reads of (stage_off, kk)
    // into set RS follow the first 8 MFMAs one by one; L0..L3: loads or nothing
#define TPAMD_SUB(MS, RS, stage_off, kk, L0, L1, L2, L3)                                                            \
    {                                                                                                               \
        const uint32_t xa = smem_base + (stage_off) + x_rd0 + kk_off[kk];                                           \
        const uint32_t wa = smem_base + (stage_off) + w_rd0 + kk_off[kk];                                           \
        TPAMD_SB;                                                                                                   \
        TPAMD_WAIT(6, xf[MS][0]); TPAMD_WAIT(6, wf[MS][0]); TPAMD_SB;                                               \
        TPAMD_MFMA(MS, 0, 0); TPAMD_SB; xf[RS][0] = lds_read16<0>(xa); TPAMD_SB;                                    \
        TPAMD_WAIT(6, wf[MS][1]); TPAMD_SB;                                                                         \
        TPAMD_MFMA(MS, 0, 1); TPAMD_SB; wf[RS][0] = lds_read16<0>(wa); TPAMD_SB;                                    \
        TPAMD_WAIT(6, wf[MS][2]); TPAMD_SB;                                                                         \
        TPAMD_MFMA(MS, 0, 2); TPAMD_SB; wf[RS][1] = lds_read16<WT1>(wa); TPAMD_SB;                                  \
        TPAMD_WAIT(6, wf[MS][3]); TPAMD_SB;                                                                         \
        TPAMD_MFMA(MS, 0, 3); TPAMD_SB; wf[RS][2] = lds_read16<WT2>(wa); TPAMD_SB;                                  \
        TPAMD_WAIT(6, xf[MS][1]); TPAMD_SB;                                                                         \
        TPAMD_MFMA(MS, 1, 0); TPAMD_SB; wf[RS][3] = lds_read16<WT3>(wa); TPAMD_SB;                                  \
        TPAMD_MFMA(MS, 1, 1); TPAMD_SB; xf[RS][1] = lds_read16<1 * T16>(xa); TPAMD_SB;                              \
        TPAMD_MFMA(MS, 1, 2); TPAMD_SB; xf[RS][2] = lds_read16<2 * T16>(xa); TPAMD_SB;                              \
        TPAMD_MFMA(MS, 1, 3); TPAMD_SB; xf[RS][3] = lds_read16<3 * T16>(xa); TPAMD_SB;                              \
        TPAMD_WAIT(9, xf[MS][2]); TPAMD_SB;                                                                         \
        TPAMD_MFMA(MS, 2, 0); TPAMD_MFMA(MS, 2, 1); TPAMD_SB; L0; TPAMD_SB;                                         \
        TPAMD_MFMA(MS, 2, 2); TPAMD_MFMA(MS, 2, 3); TPAMD_SB; L1; TPAMD_SB;                                         \
        TPAMD_WAIT(8, xf[MS][3]); TPAMD_SB;                                                                         \
        TPAMD_MFMA(MS, 3, 0); TPAMD_MFMA(MS, 3, 1); TPAMD_SB; L2; TPAMD_SB;                                         \
        TPAMD_MFMA(MS, 3, 2); TPAMD_MFMA(MS, 3, 3); TPAMD_SB; L3; TPAMD_SB;                                         \
    }
    // the tile's barrier: all fragment reads of this wavefront done, all but the loads of the NS-2 youngest tiles landed
#define TPAMD_TILE_BARRIER()                                                                                        \
    if constexpr (NS == 2) asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");                 \
    else if constexpr (XQ == 4) asm volatile("s_waitcnt vmcnt(16) lgkmcnt(0)\n\ts_barrier" ::: "memory");          \
    else if constexpr (XQ == 2) asm volatile("s_waitcnt vmcnt(12) lgkmcnt(0)\n\ts_barrier" ::: "memory");          \
    else asm volatile("s_waitcnt vmcnt(10) lgkmcnt(0)\n\ts_barrier" ::: "memory")

    // prologue: tiles 0 .. NS-2 in flight, tile 0 landed, its first fragments read, first half of tile NS-1 issued
#pragma unroll
    for (int j = 0; j < NS - 1; ++j) {
#pragma unroll
        for (int i = 0; i < 4; ++i) gx(i, j);
#pragma unroll
        for (int i = 0; i < 4; ++i) gw(i, j);
    }
    TPAMD_TILE_BARRIER();
    if (XQ < 4 && wave_s >= WAVES_N) {
        // x rows 64-127 do not exist: this wavefront keeps its share of the loads going, in the places the others have
        // them, and meets them at every barrier
        gx(0, NS - 1); gx(1, NS - 1);
        for (int j = 0; j < last; ++j) {
            gw(0, j + NS - 1); gw(1, j + NS - 1); gw(2, j + NS - 1); gw(3, j + NS - 1);
            TPAMD_TILE_BARRIER();
            gx(0, j + NS); gx(1, j + NS);
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // nothing on its way into LDS when the block ends
        return;
    }
    {
        const uint32_t xa = smem_base + x_rd0 + kk_off[0];
        const uint32_t wa = smem_base + w_rd0 + kk_off[0];
        xf[0][0] = lds_read16<0>(xa);
        wf[0][0] = lds_read16<0>(wa);
        wf[0][1] = lds_read16<WT1>(wa);
        wf[0][2] = lds_read16<WT2>(wa);
        wf[0][3] = lds_read16<WT3>(wa);
        xf[0][1] = lds_read16<1 * T16>(xa);
        xf[0][2] = lds_read16<2 * T16>(xa);
        xf[0][3] = lds_read16<3 * T16>(xa);
    }
    gx(0, NS - 1); gx(1, NS - 1); gx(2, NS - 1); gx(3, NS - 1);
    for (int j = 0; j < last; ++j) {
        const int cur = (j & (NS - 1)) * STAGE, nxt = ((j + 1) & (NS - 1)) * STAGE;
        TPAMD_SUB(0, 1, cur, 1, gw(0, j + NS - 1), gw(1, j + NS - 1), gw(2, j + NS - 1), gw(3, j + NS - 1));
        TPAMD_TILE_BARRIER();
        TPAMD_SUB(1, 0, nxt, 0, gx(0, j + NS), gx(1, j + NS), gx(2, j + NS), gx(3, j + NS));
    }
    {
        const int cur = (last & (NS - 1)) * STAGE;
        TPAMD_SUB(0, 1, cur, 1, (void)0, (void)0, (void)0, (void)0);
        // nothing may still be on its way into LDS when the block ends (the memory is handed to the next block)
        asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
        TPAMD_WAIT(0, xf[1][0]); TPAMD_WAIT(0, xf[1][1]); TPAMD_WAIT(0, xf[1][2]); TPAMD_WAIT(0, xf[1][3]);
        TPAMD_WAIT(0, wf[1][0]); TPAMD_WAIT(0, wf[1][1]); TPAMD_WAIT(0, wf[1][2]); TPAMD_WAIT(0, wf[1][3]);
        TPAMD_ROW(1, 0); TPAMD_ROW(1, 1); TPAMD_ROW(1, 2); TPAMD_ROW(1, 3);
    }
#undef TPAMD_SB
#undef TPAMD_WAIT
#undef TPAMD_MFMA
#undef TPAMD_ROW
#undef TPAMD_SUB
#undef TPAMD_TILE_BARRIER

    if constexpr (SPLIT) {
        // partial tile [x row][w row]: a lane's 4 values are 4 consecutive w rows of one x row, one 16-byte store
        const int tile = tile_m * p.tiles_n + tile_n;
        float *ws = p.ws + (static_cast<int64_t>(blockIdx.y) * p.tiles_m * p.tiles_n + tile) * (BM * BN);
#pragma unroll
        for (int a = 0; a < 4; ++a)
#pragma unroll
            for (int b = 0; b < 4; ++b) {
                const int wr = (MODE == MODE_SWIGLU ? (b >> 1) * 64 + wn * 32 + (b & 1) * 16 : wn * 64 + b * 16) + lq * 4;
                const int xr = wm * 64 + a * 16 + l16;
                if (m0 + xr < p.M) *reinterpret_cast<f32x4 *>(ws + xr * BN + wr) = acc[a][b];  // the finishing pass reads valid rows only
            }
    } else {
        // the stages are free once every wavefront has read its last fragments: a slab per wavefront at their start
        __syncthreads();
        char *slab = smem + wave * (16 * EP_PITCH);
        const bool wide = (reinterpret_cast<uintptr_t>(p.y) & 15) == 0 && p.ldy % 8 == 0;
        const int m_wave = m0 + wm * 64, n_wave = n0 + (MODE == MODE_SWIGLU ? wn * 32 : wn * 64);
        if constexpr (MODE == MODE_SWIGLU) {
            staged_epilogue<DT, MODE, false, 4, 4, 1, 2, 2>(p, acc, slab, m_wave, n_wave, lane, wide);
        } else {
            if (p.act == TPAMD_ACT_GELU) {
                if (p.addend != nullptr) staged_epilogue<DT, MODE, true, 4, 4, 1, 4, 0, true>(p, acc, slab, m_wave, n_wave, lane, wide);
                else staged_epilogue<DT, MODE, true, 4, 4, 1, 4, 0>(p, acc, slab, m_wave, n_wave, lane, wide);
            } else if (p.addend != nullptr) staged_epilogue<DT, MODE, false, 4, 4, 1, 4, 0, true>(p, acc, slab, m_wave, n_wave, lane, wide);
            else staged_epilogue<DT, MODE, false, 4, 4, 1, 4, 0>(p, acc, slab, m_wave, n_wave, lane, wide);
        }
    }
}

// Sums the split-K partial tiles of one tile of the 128 x 128 tiling in split order and applies the epilogue. A partial
// tile is [128 x rows][128 w rows] fp32 (gated pair: w rows 0-63 are gate rows, 64-127 the up rows of the same 64
// output columns): 32 (gated pair: 16) consecutive threads read one row as 16-byte pieces and write 8 bytes each of
// one output row. Grid: (16 or 8 blocks of 256 threads per tile, tiles).
template <int DT, int MODE>
__global__ __launch_bounds__(256) void splitk_finish_kernel(GemmParams p, int splits) {
    constexpr int PER_ROW = MODE == MODE_SWIGLU ? 16 : 32;
    const int tile = blockIdx.y;
    const int tile_m = tile / p.tiles_n, tile_n = tile % p.tiles_n;
    const int64_t split_stride = static_cast<int64_t>(p.tiles_m) * p.tiles_n * (128 * 128);
    const float *tile0 = p.ws + static_cast<int64_t>(tile) * (128 * 128);
    {
        const int idx = blockIdx.x * 256 + threadIdx.x;
        const int r = idx / PER_ROW, c4 = idx % PER_ROW;
        const int m = tile_m * 128 + r;
        const int n = tile_n * (MODE == MODE_SWIGLU ? 64 : 128) + c4 * 4;
        if (m >= p.M || n >= p.N) return;
        float g[4] = {0.f, 0.f, 0.f, 0.f}, u[4] = {0.f, 0.f, 0.f, 0.f};
        const float *src = tile0 + r * 128 + c4 * 4;
        for (int sp = 0; sp < splits; ++sp) {
            const f32x4 gv = *reinterpret_cast<const f32x4 *>(src + sp * split_stride);
#pragma unroll
            for (int i = 0; i < 4; ++i) g[i] += gv[i];
            if constexpr (MODE == MODE_SWIGLU) {
                const f32x4 uv = *reinterpret_cast<const f32x4 *>(src + sp * split_stride + 64);
#pragma unroll
                for (int i = 0; i < 4; ++i) u[i] += uv[i];
            }
        }
        const char *add_row = MODE == MODE_LINEAR && p.addend != nullptr ? p.addend + static_cast<int64_t>(m) * p.ldadd * 2 : nullptr;
        *reinterpret_cast<uint2 *>(p.y + (static_cast<int64_t>(m) * p.ldy + n) * 2) = finish4<DT, MODE>(p, g, u, n, add_row);
    }
}

// ---- any dtype, any alignment: LDS-tiled FMA kernel, 64x64 tile, 256 threads, 4x4 outputs per thread ---------
// The fp32 path, and the fallback for 16-bit shapes the MFMA kernels do not take (K not a multiple of 8, N not a
// multiple of 4, unaligned pointers). Scalar loads, fp32 accumulation; no tuning beyond coalesced loads.
template <int DT>
__device__ __forceinline__ float load_elem(const char *base, int64_t idx) {
    if constexpr (DT == TPAMD_F32) return reinterpret_cast<const float *>(base)[idx];
    else return half_to_f32<DT>(reinterpret_cast<const uint16_t *>(base)[idx]);
}
template <int DT>
__device__ __forceinline__ void store_elem(char *base, int64_t idx, float v) {
    if constexpr (DT == TPAMD_F32) reinterpret_cast<float *>(base)[idx] = v;
    else reinterpret_cast<uint16_t *>(base)[idx] = f32_to_half<DT>(v);
}

template <int DT, int MODE>
__global__ __launch_bounds__(256) void gemm_generic_kernel(GemmParams p) {
    constexpr int T = 64, KT = 16;
    constexpr int NW = MODE == MODE_SWIGLU ? 2 : 1;
    __shared__ float xs[KT][T + 4];
    __shared__ float ws[NW][KT][T + 4];
    const int tid = threadIdx.x;
    const int m0 = blockIdx.y * T, n0 = blockIdx.x * T;
    const int tx = tid & 15, ty = tid >> 4;  // outputs: rows ty*4.., cols tx*4..
    float acc[NW][4][4] = {};
    const int lr = tid >> 2, lk = (tid & 3) * 4;  // 64 rows x 16 k: each thread loads 4 consecutive k
    for (int k0 = 0; k0 < p.K; k0 += KT) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int k = k0 + lk + j;
            const int mr = m0 + lr, nr = n0 + lr;
            xs[lk + j][lr] = (mr < p.M && k < p.K) ? load_elem<DT>(p.x, static_cast<int64_t>(mr) * p.ldx + k) : 0.f;
            ws[0][lk + j][lr] = (nr < p.N && k < p.K) ? load_elem<DT>(p.w, static_cast<int64_t>(nr) * p.ldw + k) : 0.f;
            if constexpr (NW == 2)
                ws[1][lk + j][lr] = (nr < p.N && k < p.K) ? load_elem<DT>(p.w2, static_cast<int64_t>(nr) * p.ldw + k) : 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int k = 0; k < KT; ++k) {
            float a[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) a[i] = xs[k][ty * 4 + i];
#pragma unroll
            for (int w = 0; w < NW; ++w) {
                float b[4];
#pragma unroll
                for (int i = 0; i < 4; ++i) b[i] = ws[w][k][tx * 4 + i];
#pragma unroll
                for (int i = 0; i < 4; ++i)
#pragma unroll
                    for (int j = 0; j < 4; ++j) acc[w][i][j] = fmaf(a[i], b[j], acc[w][i][j]);
            }
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int m = m0 + ty * 4 + i;
        if (m >= p.M) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int n = n0 + tx * 4 + j;
            if (n >= p.N) continue;
            float v;
            if constexpr (MODE == MODE_SWIGLU) {
                if constexpr (DT == TPAMD_F32) {
                    v = silu_f32(acc[0][i][j]) * acc[1][i][j];
                } else {  // the roundings of separate gate, up, silu and product ops in the tensor dtype
                    const float g = half_to_f32<DT>(f32_to_half<DT>(acc[0][i][j]));
                    const float u = half_to_f32<DT>(f32_to_half<DT>(acc[NW - 1][i][j]));
                    v = half_to_f32<DT>(f32_to_half<DT>(silu_f32(g))) * u;
                }
            } else {
                v = acc[0][i][j] + (p.bias ? load_elem<DT>(p.bias, n) : 0.f);
                if (p.act == TPAMD_ACT_GELU) v = gelu_erf(v);
                if (p.addend != nullptr) {  // round to the tensor dtype first, as a separate sum of two tensors would
                    if constexpr (DT != TPAMD_F32) v = half_to_f32<DT>(f32_to_half<DT>(v));
                    v += load_elem<DT>(p.addend, static_cast<int64_t>(m) * p.ldadd + n);
                }
            }
            store_elem<DT>(p.y, static_cast<int64_t>(m) * p.ldy + n, v);
        }
    }
}

// ---- int8 weights at prefill sizes: dequantised on the way into LDS ---------------------------------------------------
// y = act(scale[n] * (x . wq^T) + x[:, outliers] . w_out^T + bias) for more rows than the weight-streaming kernels
// take. Same tiling, staging and MFMA as gemm_kernel; a K tile of the weight is 64 bytes of every row (four 16-byte
// chunks of 16 int8), converted to the activation dtype in registers (exact) and stored as the 128 bytes the MFMA
// fragments read. After the last K tile the sums are multiplied by the rows' scales, and the outlier columns follow
// as up to 4 further K tiles of 64 (x gathered through outlier_idx, w_out read as it lies, both element by element:
// a percent of the work) into the same accumulators.
struct W8Extra {
    const float *scale;
    const int *outlier_idx;
    const char *w_out;
    int n_out;
    int64_t ld_wout;
};

template <int DT, int BM, int BN, int WAVES_M, int WAVES_N>
__global__ __launch_bounds__(WAVES_M *WAVES_N * 64) void gemm_w8_kernel(GemmParams p, W8Extra q) {
    constexpr int NT = WAVES_M * WAVES_N * 64;
    constexpr int TM = BM / WAVES_M / 32, TN = BN / WAVES_N / 32;
    constexpr int XC = BM * 8 / NT;   // 16-byte chunks of the x tile per thread (8 elements each)
    constexpr int WC = BN * 4 / NT;   // 16-byte chunks of the int8 tile per thread (16 elements each)
    constexpr int WO = BN * 8 / NT;   // 8-element pieces of the w_out tile per thread
    constexpr int STAGE = (BM + BN) * LDS_ROW;
    static_assert(BM * 8 % NT == 0 && BN * 4 % NT == 0, "tile/threads mismatch");
    extern __shared__ __align__(16) char smem[];

    int tile_m, tile_n;
    tile_of_block(blockIdx.x, gridDim.x, p.tiles_m, p.tiles_n, tile_m, tile_n);
    const int m0 = tile_m * BM, n0 = tile_n * BN;
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int wm = wave / WAVES_N, wn = wave % WAVES_N;
    const int l32 = lane & 31, lhi = lane >> 5;

    const int ld_chunk = tid & 7, ld_row = tid >> 3;      // x: 8 chunks per row
    const int wq_chunk = tid & 3, wq_row = tid >> 2;      // wq: 4 chunks per row
    const char *xg[XC];
    const char *wg[WC];
#pragma unroll
    for (int i = 0; i < XC; ++i) {
        int r = m0 + ld_row + i * (NT / 8);
        r = r < p.M ? r : p.M - 1;
        xg[i] = p.x + (static_cast<int64_t>(r) * p.ldx + ld_chunk * 8) * 2;
    }
#pragma unroll
    for (int i = 0; i < WC; ++i) {
        int r = n0 + wq_row + i * (NT / 4);
        r = r < p.N ? r : p.N - 1;
        wg[i] = p.w + static_cast<int64_t>(r) * p.ldw + wq_chunk * 16;
    }
    const int st_x = ld_row * LDS_ROW + ld_chunk * 16;
    const int st_w = wq_row * LDS_ROW + wq_chunk * 32;

    uint4 xr[XC], wr[WC];
    auto load_global = [&](int kt) {
        // K is a multiple of 16: chunks are entirely inside or outside. Past the end the row's first chunk is fetched
        // (a load, not a branch around one) and zeros are stored for both operands.
        const bool okx = kt * BK + ld_chunk * 8 < p.K, okw = kt * BK + wq_chunk * 16 < p.K;
        const int64_t offx = okx ? static_cast<int64_t>(kt) * BK * 2 : -static_cast<int64_t>(ld_chunk) * 16;
        const int64_t offw = okw ? static_cast<int64_t>(kt) * BK : -static_cast<int64_t>(wq_chunk) * 16;
#pragma unroll
        for (int i = 0; i < XC; ++i) xr[i] = *reinterpret_cast<const uint4 *>(xg[i] + offx);
#pragma unroll
        for (int i = 0; i < WC; ++i) wr[i] = *reinterpret_cast<const uint4 *>(wg[i] + offw);
    };
    auto store_lds = [&](int stage, int kt) {
        char *xs = smem + stage * STAGE;
        char *ws = xs + BM * LDS_ROW;
        const bool okx = kt * BK + ld_chunk * 8 < p.K, okw = kt * BK + wq_chunk * 16 < p.K;
#pragma unroll
        for (int i = 0; i < XC; ++i)
            *reinterpret_cast<uint4 *>(xs + st_x + i * (NT / 8) * LDS_ROW) = make_uint4(okx ? xr[i].x : 0u, okx ? xr[i].y : 0u, okx ? xr[i].z : 0u, okx ? xr[i].w : 0u);
#pragma unroll
        for (int i = 0; i < WC; ++i) {
            uint4 lo, hi;
            cvt_i8x4<DT>(wr[i].x, lo.x, lo.y);
            cvt_i8x4<DT>(wr[i].y, lo.z, lo.w);
            cvt_i8x4<DT>(wr[i].z, hi.x, hi.y);
            cvt_i8x4<DT>(wr[i].w, hi.z, hi.w);
            char *dst = ws + st_w + i * (NT / 4) * LDS_ROW;
            *reinterpret_cast<uint4 *>(dst) = okw ? lo : make_uint4(0, 0, 0, 0);
            *reinterpret_cast<uint4 *>(dst + 16) = okw ? hi : make_uint4(0, 0, 0, 0);
        }
    };
    int x_rd[TM], w_rd[TN];
#pragma unroll
    for (int t = 0; t < TM; ++t) x_rd[t] = (wm * (BM / WAVES_M) + t * 32 + l32) * LDS_ROW + lhi * 16;
#pragma unroll
    for (int t = 0; t < TN; ++t) w_rd[t] = BM * LDS_ROW + (wn * (BN / WAVES_N) + t * 32 + l32) * LDS_ROW + lhi * 16;

    f32x16 acc[TM][TN];
#pragma unroll
    for (int a = 0; a < TM; ++a)
#pragma unroll
        for (int b = 0; b < TN; ++b)
#pragma unroll
            for (int i = 0; i < 16; ++i) acc[a][b][i] = 0.0f;
    auto multiply = [&](const char *stage) {
#pragma unroll
        for (int ks = 0; ks < BK / 16; ++ks) {
            uint4 xf[TM], wf[TN];
#pragma unroll
            for (int t = 0; t < TM; ++t) xf[t] = *reinterpret_cast<const uint4 *>(stage + x_rd[t] + ks * 32);
#pragma unroll
            for (int t = 0; t < TN; ++t) wf[t] = *reinterpret_cast<const uint4 *>(stage + w_rd[t] + ks * 32);
#pragma unroll
            for (int a = 0; a < TM; ++a)
#pragma unroll
                for (int b = 0; b < TN; ++b) acc[a][b] = mfma32<DT>(wf[b], xf[a], acc[a][b]);
        }
    };

    const int KT = (p.K + BK - 1) / BK;
    load_global(0);
    store_lds(0, 0);
    __syncthreads();
    for (int kt = 0; kt < KT; ++kt) {
        const bool more = kt + 1 < KT;
        if (more) load_global(kt + 1);
        multiply(smem + (kt & 1) * STAGE);
        if (more) store_lds((kt + 1) & 1, kt + 1);
        __syncthreads();
    }
    // the int8 sums become real ones: D[n_local][m_local], register i -> n_local = 8 * (i / 4) + 4 * lhi + i % 4
#pragma unroll
    for (int b = 0; b < TN; ++b)
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            int n = n0 + wn * (BN / WAVES_N) + b * 32 + 8 * (i >> 2) + 4 * lhi + (i & 3);
            n = n < p.N ? n : p.N - 1;
            const float sc = q.scale[n];
#pragma unroll
            for (int a = 0; a < TM; ++a) acc[a][b][i] *= sc;
        }
    // outlier columns, 64 at a time, staged element by element into stage 0 (nobody reads the stages any more)
    const uint16_t *xe = reinterpret_cast<const uint16_t *>(p.x);
    const uint16_t *we = reinterpret_cast<const uint16_t *>(q.w_out);
    for (int o0 = 0; o0 < q.n_out; o0 += BK) {
        char *xs = smem;
        char *ws = xs + BM * LDS_ROW;
        int col[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const int o = o0 + ld_chunk * 8 + e;
            col[e] = q.outlier_idx[o < q.n_out ? o : q.n_out - 1];
        }
#pragma unroll
        for (int i = 0; i < XC; ++i) {
            int r = m0 + ld_row + i * (NT / 8);
            r = r < p.M ? r : p.M - 1;
            uint32_t v[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) v[e] = xe[static_cast<int64_t>(r) * p.ldx + col[e]];
            uint32_t d[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const uint32_t lo = o0 + ld_chunk * 8 + 2 * e < q.n_out ? v[2 * e] : 0u;
                const uint32_t hi = o0 + ld_chunk * 8 + 2 * e + 1 < q.n_out ? v[2 * e + 1] : 0u;
                d[e] = lo | (hi << 16);
            }
            *reinterpret_cast<uint4 *>(xs + st_x + i * (NT / 8) * LDS_ROW) = make_uint4(d[0], d[1], d[2], d[3]);
        }
#pragma unroll
        for (int i = 0; i < WO; ++i) {
            int r = n0 + ld_row + i * (NT / 8);
            r = r < p.N ? r : p.N - 1;
            uint32_t v[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const int o = o0 + ld_chunk * 8 + e;
                v[e] = we[static_cast<int64_t>(r) * q.ld_wout + (o < q.n_out ? o : q.n_out - 1)];
            }
            uint32_t d[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const uint32_t lo = o0 + ld_chunk * 8 + 2 * e < q.n_out ? v[2 * e] : 0u;
                const uint32_t hi = o0 + ld_chunk * 8 + 2 * e + 1 < q.n_out ? v[2 * e + 1] : 0u;
                d[e] = lo | (hi << 16);
            }
            *reinterpret_cast<uint4 *>(ws + st_x + i * (NT / 8) * LDS_ROW) = make_uint4(d[0], d[1], d[2], d[3]);
        }
        __syncthreads();
        multiply(smem);
        __syncthreads();
    }
    epilogue<DT, MODE_LINEAR, BM, BN, WAVES_M, WAVES_N>(p, acc, m0, n0, wm, wn, l32, lhi);
}

template <int DT, int BM, int BN, int WAVES_M, int WAVES_N>
int launch_gemm_w8(GemmParams p, const W8Extra &q, hipStream_t s) {
    constexpr int NT = WAVES_M * WAVES_N * 64;
    constexpr int LDS = 2 * (BM + BN) * LDS_ROW;
    auto kern = gemm_w8_kernel<DT, BM, BN, WAVES_M, WAVES_N>;
    static thread_local int configured_dev = -1;  // per instantiation and host thread
    int dev = 0;
    TPAMD_HIP(hipGetDevice(&dev));
    if (configured_dev != dev) {
        TPAMD_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, LDS));
        configured_dev = dev;
    }
    p.tiles_m = (p.M + BM - 1) / BM;
    p.tiles_n = (p.N + BN - 1) / BN;
    const int64_t blocks = static_cast<int64_t>(p.tiles_m) * p.tiles_n;
    TPAMD_REQUIRE(blocks < (1ll << 31), "gemm: too many tiles");
    hipLaunchKernelGGL(kern, dim3(static_cast<unsigned>(blocks)), dim3(NT), LDS, s, p, q);
    TPAMD_HIP(hipGetLastError());
    return TPAMD_OK;
}

// ---- fp32 on the matrix pipe: v_mfma_f32_32x32x2_f32 -------------------------------------------------------------
// y = act(x . w^T + bias) (+ addend) for fp32 operands whose rows are 16-byte aligned (K, leading dimensions and N
// multiples of 4). Same staging as gemm_kernel: a K tile is 128 bytes of every row (32 floats here), 16-byte chunks
// prefetched into registers while the current tile is multiplied, two LDS stages, one barrier per tile. The
// instruction multiplies a 32 x 2 by a 2 x 32 panel; which two k a step pairs up is free as long as both operands
// agree, so lane (row r, half h) uses k = 16 h + s in step s: its 16 operands of a K tile are 64 contiguous bytes of
// the staged row (four 16-byte reads). w is the first operand, so a lane holds 4 consecutive output columns of one
// row per group of 4 accumulator registers: one 16-byte store. Products and sums are fp32 throughout.
// BKF = floats of K per stage and row: 32 (128 bytes, two blocks per CU) for problems with many tiles; 128 for few tiles,
// where a block has its CU to itself and a loop of many short stages would wait for memory once per stage.
template <int BM, int BN, int WAVES_M, int WAVES_N, int BKF>
__global__ __launch_bounds__(WAVES_M *WAVES_N * 64) void gemm_f32_kernel(GemmParams p) {
    constexpr int NT = WAVES_M * WAVES_N * 64;
    constexpr int TM = BM / WAVES_M / 32, TN = BN / WAVES_N / 32;
    constexpr int CPR = BKF / 4;             // 16-byte chunks per staged row
    constexpr int ROW = BKF * 4 + 16;        // staged row pitch in bytes: conflict-free 16-byte reads
    constexpr int XC = BM * CPR / NT, WC = BN * CPR / NT;
    constexpr int STAGE = (BM + BN) * ROW;
    static_assert(BM * CPR % NT == 0 && BN * CPR % NT == 0 && NT % CPR == 0, "tile/threads mismatch");
    extern __shared__ __align__(16) char smem[];

    int tile_m, tile_n;
    tile_of_block(blockIdx.x, gridDim.x, p.tiles_m, p.tiles_n, tile_m, tile_n);
    const int m0 = tile_m * BM, n0 = tile_n * BN;
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int wm = wave / WAVES_N, wn = wave % WAVES_N;
    const int l32 = lane & 31, lhi = lane >> 5;

    const int ld_chunk = tid % CPR, ld_row = tid / CPR;
    const char *xg[XC];
    const char *wg[WC];
#pragma unroll
    for (int i = 0; i < XC; ++i) {
        int r = m0 + ld_row + i * (NT / CPR);
        r = r < p.M ? r : p.M - 1;  // rows past the end repeat the last one; their outputs are not stored
        xg[i] = p.x + (static_cast<int64_t>(r) * p.ldx + ld_chunk * 4) * 4;
    }
#pragma unroll
    for (int i = 0; i < WC; ++i) {
        int r = n0 + ld_row + i * (NT / CPR);
        r = r < p.N ? r : p.N - 1;
        wg[i] = p.w + (static_cast<int64_t>(r) * p.ldw + ld_chunk * 4) * 4;
    }
    const int st_off = ld_row * ROW + ld_chunk * 16;
    uint4 xr[XC], wr[WC];
    auto load_global = [&](int kt) {
        const bool ok = kt * BKF + ld_chunk * 4 < p.K;  // K is a multiple of 4: a chunk is entirely inside or outside
        // past the end of K the row's first chunk is fetched instead (a load, not a branch); zeros are stored for it
        const int64_t off = ok ? static_cast<int64_t>(kt) * BKF * 4 : -static_cast<int64_t>(ld_chunk) * 16;
#pragma unroll
        for (int i = 0; i < XC; ++i) xr[i] = *reinterpret_cast<const uint4 *>(xg[i] + off);
#pragma unroll
        for (int i = 0; i < WC; ++i) wr[i] = *reinterpret_cast<const uint4 *>(wg[i] + off);
    };
    auto store_lds = [&](int stage, int kt) {
        char *xs = smem + stage * STAGE;
        char *ws = xs + BM * ROW;
        const bool ok = kt * BKF + ld_chunk * 4 < p.K;
#pragma unroll
        for (int i = 0; i < XC; ++i)
            *reinterpret_cast<uint4 *>(xs + st_off + i * (NT / CPR) * ROW) = make_uint4(ok ? xr[i].x : 0u, ok ? xr[i].y : 0u, ok ? xr[i].z : 0u, ok ? xr[i].w : 0u);
#pragma unroll
        for (int i = 0; i < WC; ++i)  // both operands are zeroed: whatever the other one holds there must not meet a NaN
            *reinterpret_cast<uint4 *>(ws + st_off + i * (NT / CPR) * ROW) = make_uint4(ok ? wr[i].x : 0u, ok ? wr[i].y : 0u, ok ? wr[i].z : 0u, ok ? wr[i].w : 0u);
    };
    int x_rd[TM], w_rd[TN];
#pragma unroll
    for (int t = 0; t < TM; ++t) x_rd[t] = (wm * (BM / WAVES_M) + t * 32 + l32) * ROW + lhi * (BKF * 2);
#pragma unroll
    for (int t = 0; t < TN; ++t) w_rd[t] = BM * ROW + (wn * (BN / WAVES_N) + t * 32 + l32) * ROW + lhi * (BKF * 2);

    f32x16 acc[TM][TN];
#pragma unroll
    for (int a = 0; a < TM; ++a)
#pragma unroll
        for (int b = 0; b < TN; ++b)
#pragma unroll
            for (int i = 0; i < 16; ++i) acc[a][b][i] = 0.0f;

    const int KT = (p.K + BKF - 1) / BKF;
    load_global(0);
    store_lds(0, 0);
    __syncthreads();
    for (int kt = 0; kt < KT; ++kt) {
        const bool more = kt + 1 < KT;
        if (more) load_global(kt + 1);
        const char *stage = smem + (kt & 1) * STAGE;
#pragma unroll
        for (int q = 0; q < BKF / 8; ++q) {  // 4 floats of the lane's BKF / 2 at a time
            f32x4 xf[TM], wf[TN];
#pragma unroll
            for (int t = 0; t < TM; ++t) xf[t] = *reinterpret_cast<const f32x4 *>(stage + x_rd[t] + q * 16);
#pragma unroll
            for (int t = 0; t < TN; ++t) wf[t] = *reinterpret_cast<const f32x4 *>(stage + w_rd[t] + q * 16);
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int a = 0; a < TM; ++a)
#pragma unroll
                    for (int b = 0; b < TN; ++b) acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x2f32(wf[b][j], xf[a][j], acc[a][b], 0, 0, 0);
        }
        if (more) store_lds((kt + 1) & 1, kt + 1);
        __syncthreads();
    }
    // D[n_local][m_local]: lane -> m_local = l32, register i -> n_local = 8 * (i / 4) + 4 * lhi + i % 4
#pragma unroll
    for (int a = 0; a < TM; ++a) {
        const int m = m0 + wm * (BM / WAVES_M) + a * 32 + l32;
        if (m >= p.M) continue;
        float *yrow = reinterpret_cast<float *>(p.y) + static_cast<int64_t>(m) * p.ldy;
#pragma unroll
        for (int b = 0; b < TN; ++b)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const int n = n0 + wn * (BN / WAVES_N) + b * 32 + q * 8 + lhi * 4;
                if (n >= p.N) continue;  // N is a multiple of 4: the group of 4 is all in or all out
                f32x4 v = {acc[a][b][q * 4], acc[a][b][q * 4 + 1], acc[a][b][q * 4 + 2], acc[a][b][q * 4 + 3]};
                if (p.bias) v += *reinterpret_cast<const f32x4 *>(reinterpret_cast<const float *>(p.bias) + n);
                if (p.act == TPAMD_ACT_GELU) {
#pragma unroll
                    for (int j = 0; j < 4; ++j) v[j] = gelu_erf(v[j]);
                }
                if (p.addend != nullptr) v += *reinterpret_cast<const f32x4 *>(reinterpret_cast<const float *>(p.addend) + static_cast<int64_t>(m) * p.ldadd + n);
                *reinterpret_cast<f32x4 *>(yrow + n) = v;
            }
    }
}

// Few output tiles (the Linears of a small model on a short sequence): 32 x 32 tiles, and the four wavefronts of a block
// share a tile's K instead of its outputs. Wavefront w multiplies floats [32 w, 32 w + 32) of every 128-float stage, so a
// tile's chain of dependent MFMAs is a quarter as long and four times as many blocks are in flight; the four partial
// tiles meet in LDS and wavefront w finishes output columns 8 w .. 8 w + 7 of the tile.
__global__ __launch_bounds__(256) void gemm_f32_small_kernel(GemmParams p) {
    constexpr int T = 32, BKF = 128, CPR = BKF / 4, ROW = BKF * 4 + 16, NT = 256;
    constexpr int XC = T * CPR / NT;  // 16-byte chunks per thread and operand
    constexpr int STAGE = 2 * T * ROW;
    extern __shared__ __align__(16) char smem[];
    const int tile_n = blockIdx.x % p.tiles_n, tile_m = blockIdx.x / p.tiles_n;
    const int m0 = tile_m * T, n0 = tile_n * T;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int l32 = lane & 31, lhi = lane >> 5;
    const int ld_chunk = tid % CPR, ld_row = tid / CPR;
    const char *xg[XC];
    const char *wg[XC];
#pragma unroll
    for (int i = 0; i < XC; ++i) {
        int r = m0 + ld_row + i * (NT / CPR);
        r = r < p.M ? r : p.M - 1;
        xg[i] = p.x + (static_cast<int64_t>(r) * p.ldx + ld_chunk * 4) * 4;
        r = n0 + ld_row + i * (NT / CPR);
        r = r < p.N ? r : p.N - 1;
        wg[i] = p.w + (static_cast<int64_t>(r) * p.ldw + ld_chunk * 4) * 4;
    }
    const int st_off = ld_row * ROW + ld_chunk * 16;
    uint4 xr[XC], wr[XC];
    auto load_global = [&](int kt) {
        const bool ok = kt * BKF + ld_chunk * 4 < p.K;
        const int64_t off = ok ? static_cast<int64_t>(kt) * BKF * 4 : -static_cast<int64_t>(ld_chunk) * 16;
#pragma unroll
        for (int i = 0; i < XC; ++i) {
            xr[i] = *reinterpret_cast<const uint4 *>(xg[i] + off);
            wr[i] = *reinterpret_cast<const uint4 *>(wg[i] + off);
        }
    };
    auto store_lds = [&](int stage, int kt) {
        char *xs = smem + stage * STAGE;
        char *ws = xs + T * ROW;
        const bool ok = kt * BKF + ld_chunk * 4 < p.K;
#pragma unroll
        for (int i = 0; i < XC; ++i) {
            *reinterpret_cast<uint4 *>(xs + st_off + i * (NT / CPR) * ROW) = make_uint4(ok ? xr[i].x : 0u, ok ? xr[i].y : 0u, ok ? xr[i].z : 0u, ok ? xr[i].w : 0u);
            *reinterpret_cast<uint4 *>(ws + st_off + i * (NT / CPR) * ROW) = make_uint4(ok ? wr[i].x : 0u, ok ? wr[i].y : 0u, ok ? wr[i].z : 0u, ok ? wr[i].w : 0u);
        }
    };
    // lane (row l32, half lhi) of wavefront w: floats 32 w + 16 lhi + s of the stage in step s
    const int x_rd = l32 * ROW + wave * 128 + lhi * 64;
    const int w_rd = T * ROW + x_rd;
    f32x16 acc;
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[i] = 0.0f;
    const int KT = (p.K + BKF - 1) / BKF;
    load_global(0);
    store_lds(0, 0);
    __syncthreads();
    for (int kt = 0; kt < KT; ++kt) {
        const bool more = kt + 1 < KT;
        if (more) load_global(kt + 1);
        const char *stage = smem + (kt & 1) * STAGE;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const f32x4 xf = *reinterpret_cast<const f32x4 *>(stage + x_rd + q * 16);
            const f32x4 wf = *reinterpret_cast<const f32x4 *>(stage + w_rd + q * 16);
#pragma unroll
            for (int j = 0; j < 4; ++j) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(wf[j], xf[j], acc, 0, 0, 0);
        }
        if (more) store_lds((kt + 1) & 1, kt + 1);
        __syncthreads();
    }
    // the four partial tiles meet: red[wave][register][lane]
    float *red = reinterpret_cast<float *>(smem);
#pragma unroll
    for (int i = 0; i < 16; ++i) red[(wave * 16 + i) * 64 + lane] = acc[i];
    __syncthreads();
    f32x4 v;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        const int i = wave * 4 + e;
        v[e] = (red[(0 * 16 + i) * 64 + lane] + red[(1 * 16 + i) * 64 + lane]) + (red[(2 * 16 + i) * 64 + lane] + red[(3 * 16 + i) * 64 + lane]);
    }
    // D[n_local][m_local]: lane -> m_local = l32, register i -> n_local = 8 * (i / 4) + 4 * lhi + i % 4; here i / 4 = wave
    const int m = m0 + l32, n = n0 + 8 * wave + 4 * lhi;
    if (m >= p.M || n >= p.N) return;  // N is a multiple of 4: the group of 4 is all in or all out
    if (p.bias) v += *reinterpret_cast<const f32x4 *>(reinterpret_cast<const float *>(p.bias) + n);
    if (p.act == TPAMD_ACT_GELU) {
#pragma unroll
        for (int j = 0; j < 4; ++j) v[j] = gelu_erf(v[j]);
    }
    if (p.addend != nullptr) v += *reinterpret_cast<const f32x4 *>(reinterpret_cast<const float *>(p.addend) + static_cast<int64_t>(m) * p.ldadd + n);
    *reinterpret_cast<f32x4 *>(reinterpret_cast<float *>(p.y) + static_cast<int64_t>(m) * p.ldy + n) = v;
}

int launch_gemm_f32_small(GemmParams p, hipStream_t s) {
    constexpr int LDS = 2 * 2 * 32 * (128 * 4 + 16);
    static thread_local int configured_dev = -1;
    int dev = 0;
    TPAMD_HIP(hipGetDevice(&dev));
    if (configured_dev != dev) {
        TPAMD_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(gemm_f32_small_kernel), hipFuncAttributeMaxDynamicSharedMemorySize, LDS));
        configured_dev = dev;
    }
    p.tiles_m = (p.M + 31) / 32;
    p.tiles_n = (p.N + 31) / 32;
    const int64_t blocks = static_cast<int64_t>(p.tiles_m) * p.tiles_n;
    TPAMD_REQUIRE(blocks < (1ll << 31), "gemm: too many tiles");
    hipLaunchKernelGGL(gemm_f32_small_kernel, dim3(static_cast<unsigned>(blocks)), dim3(256), LDS, s, p);
    TPAMD_HIP(hipGetLastError());
    return TPAMD_OK;
}

template <int BM, int BN, int WAVES_M, int WAVES_N, int BKF>
int launch_gemm_f32(GemmParams p, hipStream_t s) {
    constexpr int NT = WAVES_M * WAVES_N * 64;
    constexpr int LDS = 2 * (BM + BN) * (BKF * 4 + 16);
    auto kern = gemm_f32_kernel<BM, BN, WAVES_M, WAVES_N, BKF>;
    static thread_local int configured_dev = -1;  // per instantiation and host thread
    int dev = 0;
    TPAMD_HIP(hipGetDevice(&dev));
    if (configured_dev != dev) {
        TPAMD_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, LDS));
        configured_dev = dev;
    }
    p.tiles_m = (p.M + BM - 1) / BM;
    p.tiles_n = (p.N + BN - 1) / BN;
    const int64_t blocks = static_cast<int64_t>(p.tiles_m) * p.tiles_n;
    TPAMD_REQUIRE(blocks < (1ll << 31), "gemm: too many tiles");
    hipLaunchKernelGGL(kern, dim3(static_cast<unsigned>(blocks)), dim3(NT), LDS, s, p);
    TPAMD_HIP(hipGetLastError());
    return TPAMD_OK;
}

template <int DT, int MODE, int BM, int BN, int WAVES_M, int WAVES_N>
int launch_gemm(GemmParams p, hipStream_t s) {
    constexpr int NT = WAVES_M * WAVES_N * 64;
    constexpr int LDS = 2 * (BM + BN) * LDS_ROW;
    auto kern = gemm_kernel<DT, MODE, BM, BN, WAVES_M, WAVES_N>;
    static thread_local int configured_dev = -1;  // per instantiation and host thread
    int dev = 0;
    TPAMD_HIP(hipGetDevice(&dev));
    if (configured_dev != dev) {
        TPAMD_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, LDS));
        configured_dev = dev;
    }
    p.tiles_m = (p.M + BM - 1) / BM;
    constexpr int BN_OUT = MODE == MODE_SWIGLU ? BN / 2 : BN;
    p.tiles_n = (p.N + BN_OUT - 1) / BN_OUT;
    const int64_t blocks = static_cast<int64_t>(p.tiles_m) * p.tiles_n;
    TPAMD_REQUIRE(blocks < (1ll << 31), "gemm: too many tiles");
    hipLaunchKernelGGL(kern, dim3(static_cast<unsigned>(blocks)), dim3(NT), LDS, s, p);
    TPAMD_HIP(hipGetLastError());
    return TPAMD_OK;
}

}  // namespace

namespace {

template <int DT, int MODE>
int launch_direct(GemmParams p, int cus, int splits, hipStream_t s) {
    constexpr int LDS = 2 * 64 * 1152 + 4 * 16 * 144;  // two stages + the 4-wavefront kernel's epilogue slabs
    const bool four = tuning().gemm_w4 != 0 && p.K >= 128;  // unset: the 4-wavefront kernel
    auto kern = four ? gemm_direct4_kernel<DT, MODE, false> : gemm_direct_kernel<DT, MODE>;
    static thread_local int configured_dev = -1;
    int dev = 0;
    TPAMD_HIP(hipGetDevice(&dev));
    if (configured_dev != dev) {
        TPAMD_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(gemm_direct_kernel<DT, MODE>), hipFuncAttributeMaxDynamicSharedMemorySize, LDS));
        TPAMD_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(gemm_direct4_kernel<DT, MODE, false>), hipFuncAttributeMaxDynamicSharedMemorySize, LDS));
        TPAMD_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(gemm_direct4_kernel<DT, MODE, true>), hipFuncAttributeMaxDynamicSharedMemorySize, LDS));
        configured_dev = dev;
    }
    p.tiles_m = (p.M + 255) / 256;
    constexpr int BN_OUT = MODE == MODE_SWIGLU ? 128 : 256;
    p.tiles_n = (p.N + BN_OUT - 1) / BN_OUT;
    const int64_t tiles = static_cast<int64_t>(p.tiles_m) * p.tiles_n;
    TPAMD_REQUIRE(tiles < (1ll << 31), "gemm: too many tiles");
    // one block per CU at most (a block needs most of a CU's LDS anyway); a multiple of 8 when blocks take several
    // tiles, so that a block's tiles all belong to one XCD's share
    int64_t blocks = tiles;
    if (tiles > cus) blocks = cus >= 8 ? (cus / 8) * 8 : cus;
    // K split over `splits` units per tile (all units in one round): every split gets at least 2 K tiles
    const int KT = p.K / 64;
    if (four && splits > 1 && KT >= 4) {
        p.kt_per_split = (KT + splits - 1) / splits;
        if (p.kt_per_split < 2) p.kt_per_split = 2;
        while (KT % p.kt_per_split == 1) ++p.kt_per_split;  // the last split would be a single K tile
        p.splits = (KT + p.kt_per_split - 1) / p.kt_per_split;
        if (p.splits > 1 && tiles * p.splits <= cus) {
            GemmParams f = p;  // the finishing pass sees the 128 x 128 tiling
            f.tiles_m = (p.M + 127) / 128;
            f.tiles_n = (p.N + BN_OUT / 2 - 1) / (BN_OUT / 2);
            const int64_t tiles128 = static_cast<int64_t>(f.tiles_m) * f.tiles_n;
            const size_t ws_bytes = static_cast<size_t>(p.splits) * tiles128 * 128 * 128 * sizeof(float);
            std::lock_guard<std::mutex> hold(splitk_mutex(dev));
            void *ws = nullptr;
            const int rc = splitk_scratch(dev, s, ws_bytes, static_cast<size_t>(4) * cus * 128 * 128 * sizeof(float), &ws);
            if (rc != TPAMD_OK) return rc;
            if (ws != nullptr) {
                p.ws = f.ws = static_cast<float *>(ws);
                hipLaunchKernelGGL((gemm_direct4_kernel<DT, MODE, true>), dim3(static_cast<unsigned>(tiles * p.splits)), dim3(256), LDS, s, p);
                TPAMD_HIP(hipGetLastError());
                hipLaunchKernelGGL((splitk_finish_kernel<DT, MODE>), dim3(MODE == MODE_SWIGLU ? 8 : 16, static_cast<unsigned>(tiles128)), dim3(256), 0, s, f, p.splits);
                TPAMD_HIP(hipGetLastError());
                return TPAMD_OK;
            }
        }
    }
    hipLaunchKernelGGL(kern, dim3(static_cast<unsigned>(blocks)), dim3(four ? 256 : 512), LDS, s, p);
    TPAMD_HIP(hipGetLastError());
    return TPAMD_OK;
}

}  // namespace

template <int DT, int MODE, int NS, bool SPLIT, int XQ = 4>
int configure128(int dev) {
    static thread_local int configured_dev = -1;
    if (configured_dev != dev) {
        TPAMD_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(gemm_direct128_kernel<DT, MODE, NS, SPLIT, XQ>),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, NS * 32 * 1152));
        configured_dev = dev;
    }
    return TPAMD_OK;
}

// Predicted time (microseconds) of the 128 x 128 tiling, with the K split and the number of LDS stages that give it,
// from a small cost model fitted on this part (least squares over 290 timings of 48 mid-sized shapes, then two sweeps of
// 100 shapes at 64-2048 rows with every split count and both stage counts, 1500 timings).
//  - two stages (two blocks fit a CU): a block that has its CU to itself takes 0.82 per K tile, two blocks sharing a CU
//    0.98 each (the pace of the CU's global->LDS path), 0.92 when blocks queue for several rounds of two per CU;
//  - four stages (one block per CU, three K tiles of look-ahead), in rounds of one block per CU: split launches 0.55 per
//    K tile; unsplit ones 0.60 when there is one row tile (every block streams weights nobody shares, about 27 GB/s
//    per CU), 0.42 with at most half the CUs busy and 0.55 otherwise for a single matrix, 0.62 (two row tiles) / 0.44 and
//    0.64 for the gated pair;
//  - no launch streams its weights (tiles_n column tiles of 16 KiB per K tile) faster than 5 TB/s;
//  - the partial tiles cost 4.6 + 0.39 per MB (written, read back and finished by a second launch; valid_rows = the
//    fraction of the tiles' rows that lie inside M: the others are not stored).
// Over the second sweep the choices are within 1.8 % of the best (split, stages) per shape; with two stages only they
// were 4.7 % off the best split (a single matrix 4096 x 4096 at 1024 rows: 51.5 us unsplit on two stages, 33.7 us on four).
inline double estimate128(int64_t tiles, int64_t tiles_m, int64_t tiles_n, int KT, int cus, double valid_rows, bool swiglu, int *splits,
                          bool *deep) {
    double best = 1e30;
    *splits = 1;
    *deep = false;
    const double stream = static_cast<double>(tiles_n) * KT * 16384.0 / 5.0e6;
    for (int sp = 1; sp <= 8; ++sp) {
        const int kt = (KT + sp - 1) / sp;
        if (sp > 1 && (kt < 4 || tiles * sp > 4ll * cus)) break;  // too little K per split / more than the scratch buffer holds
        const int64_t units = tiles * sp;
        const double finish = sp > 1 ? 4.6 + units * 0.065536 * valid_rows * 0.39 : 0.0;
        const double per_deep = sp > 1 ? 0.55
                                : tiles_m == 1 ? 0.60
                                : units * 2 <= cus ? (swiglu ? (tiles_m == 2 ? 0.62 : 0.44) : 0.42)
                                : (swiglu ? 0.64 : 0.55);
        const double loop_deep = static_cast<double>((units + cus - 1) / cus) * kt * per_deep;
        const double t_deep = (loop_deep > stream ? loop_deep : stream) + finish;
        if ((sp == 1 || units <= cus) && t_deep < best) { best = t_deep; *splits = sp; *deep = true; }  // split launches: one round only (measured)
        const double rounds = units <= cus ? 1.0 : static_cast<double>((units + 2 * cus - 1) / (2 * cus));
        const double per_kt = units <= cus ? 0.82 : units <= 2ll * cus ? 0.98 : 0.92;
        const double loop = rounds * kt * per_kt;
        const double t = (loop > stream ? loop : stream) + finish;
        if (t < best) { best = t; *splits = sp; *deep = false; }
    }
    return best;
}

template <int DT, int MODE, int NS, int XQ>
int launch_split128(const GemmParams &p, dim3 grid, int dev, hipStream_t s) {
    if (int rc = configure128<DT, MODE, NS, true, XQ>(dev); rc != TPAMD_OK) return rc;
    hipLaunchKernelGGL((gemm_direct128_kernel<DT, MODE, NS, true, XQ>), grid, dim3(256), NS * 32 * 1152, s, p);
    TPAMD_HIP(hipGetLastError());
    return TPAMD_OK;
}

// 128 x 128 tiles; split over K (fp32 partial tiles in stream-ordered scratch memory, then one finishing pass)
// when the tiles alone would not give every CU two blocks.
template <int DT, int MODE>
int launch_direct128(GemmParams p, int cus, hipStream_t s) {
    int dev = 0;
    TPAMD_HIP(hipGetDevice(&dev));
    p.tiles_m = (p.M + 127) / 128;
    constexpr int BN_OUT = MODE == MODE_SWIGLU ? 64 : 128;
    p.tiles_n = (p.N + BN_OUT - 1) / BN_OUT;
    const int64_t tiles = static_cast<int64_t>(p.tiles_m) * p.tiles_n;
    TPAMD_REQUIRE(tiles < (1ll << 31), "gemm: too many tiles");
    const int KT = p.K / 64;
    int splits = 1;
    bool deep = false;
    estimate128(tiles, p.tiles_m, p.tiles_n, KT, cus, static_cast<double>(p.M) / (p.tiles_m * 128.0), MODE == MODE_SWIGLU, &splits, &deep);
    if (tuning().gemm_splitk != TUNE_UNSET) {
        splits = tuning().gemm_splitk;
        deep = tiles * splits <= cus;
    }
    if (tuning().gemm_stages != TUNE_UNSET) deep = tuning().gemm_stages == 4;
    if (splits > 8) splits = 8;
    if (splits > KT) splits = KT;
    if (splits < 1) splits = 1;
    p.kt_per_split = (KT + splits - 1) / splits;
    splits = (KT + p.kt_per_split - 1) / p.kt_per_split;   // no empty split
    constexpr int LDS2 = 2 * 32 * 1152;
    if (splits > 1) {
        const int xq = MODE != MODE_LINEAR || tuning().gemm_part_x == 0 || tiles > 64 ? 4 : p.M <= 32 ? 1 : p.M <= 64 ? 2 : 4;  // tiles > 64: measured, no gain
        const size_t ws_bytes = static_cast<size_t>(splits) * tiles * 128 * 128 * sizeof(float);
        // the scratch buffer is ours until both launches are enqueued
        std::lock_guard<std::mutex> hold(splitk_mutex(dev));
        void *ws = nullptr;
        if (int rc = splitk_scratch(dev, s, ws_bytes, static_cast<size_t>(4) * cus * 128 * 128 * sizeof(float), &ws); rc != TPAMD_OK) return rc;
        if (ws != nullptr) {
            p.ws = static_cast<float *>(ws);
            const dim3 grid(static_cast<unsigned>(tiles), static_cast<unsigned>(splits));
            int launched = -1;
            if constexpr (MODE == MODE_LINEAR) {
                if (xq == 1) launched = deep ? launch_split128<DT, MODE, 4, 1>(p, grid, dev, s) : launch_split128<DT, MODE, 2, 1>(p, grid, dev, s);
                else if (xq == 2) launched = deep ? launch_split128<DT, MODE, 4, 2>(p, grid, dev, s) : launch_split128<DT, MODE, 2, 2>(p, grid, dev, s);
            }
            if (launched < 0) launched = deep ? launch_split128<DT, MODE, 4, 4>(p, grid, dev, s) : launch_split128<DT, MODE, 2, 4>(p, grid, dev, s);
            if (launched != TPAMD_OK) return launched;
            hipLaunchKernelGGL((splitk_finish_kernel<DT, MODE>), dim3(MODE == MODE_SWIGLU ? 8 : 16, static_cast<unsigned>(tiles)), dim3(256), 0, s, p, splits);
            TPAMD_HIP(hipGetLastError());
            return TPAMD_OK;
        }
    }
    if (deep) {
        int rc4 = configure128<DT, MODE, 4, false>(dev);
        if (rc4 != TPAMD_OK) return rc4;
        hipLaunchKernelGGL((gemm_direct128_kernel<DT, MODE, 4, false>), dim3(static_cast<unsigned>(tiles)), dim3(256), 2 * LDS2, s, p);
        TPAMD_HIP(hipGetLastError());
        return TPAMD_OK;
    }
    int rc = configure128<DT, MODE, 2, false>(dev);
    if (rc != TPAMD_OK) return rc;
    hipLaunchKernelGGL((gemm_direct128_kernel<DT, MODE, 2, false>), dim3(static_cast<unsigned>(tiles)), dim3(256), LDS2, s, p);
    TPAMD_HIP(hipGetLastError());
    return TPAMD_OK;
}

// Prefill-sized dispatch; called by linear.hip once M is above the skinny range.
template <int DT>
int gemm_large(GemmParams p, bool swiglu, hipStream_t s) {
    int dev = 0, cus = 256;
    TPAMD_HIP(hipGetDevice(&dev));
    if (int rc_cus = device_cus(dev, &cus); rc_cus != TPAMD_OK) return rc_cus;
    // the direct kernels address a tile with 32-bit byte offsets from the tile origin and step K in tiles of 64
    const bool direct_ok = p.K % 64 == 0 && p.K >= 64 && p.ldx < (1ll << 22) && p.ldw < (1ll << 22);
    // 256 x 256 tiles or 128 x 128 tiles (with K split): whichever the cost models predict to be faster. The 256 tiles
    // run in rounds of one per CU; fitted on the same timings, a K tile takes 1.47 us in a full round (the part is
    // power-limited then), 1.2 us in a round that fills at most three quarters of the CUs and 1.3 us in between.
    const int64_t big_tiles = static_cast<int64_t>((p.M + 255) / 256) * ((p.N + (swiglu ? 127 : 255)) / (swiglu ? 128 : 256));
    const int64_t small_tiles = static_cast<int64_t>((p.M + 127) / 128) * ((p.N + (swiglu ? 63 : 127)) / (swiglu ? 64 : 128));
    const int KT = static_cast<int>(p.K / 64);
    auto rounds256 = [&](int64_t units, int kt) {
        const int64_t full = units / cus, last = units % cus;
        return kt * (full * 1.47 + (last == 0 ? 0.0 : last * 4 <= 3ll * cus ? 1.2 : 1.3));
    };
    // no launch streams the weights faster than 5 TB/s (what bounds a few rows of a wide matrix: the pair 8192 x 8192 at
    // 17 rows took 79.8 us on this tiling in four splits, predicted 57 without this term, and 63.8 us on the other)
    const double stream = static_cast<double>(p.N) * p.K * (swiglu ? 4.0 : 2.0) / 5.0e6;
    auto floor256 = [&](double loop) { return loop > stream ? loop : stream; };
    double t256 = floor256(rounds256(big_tiles, KT));
    // ... or split over K while all units still fit one round; the partial tiles cost 9 us + 0.33 us per MB (more than
    // with the small tiles: all blocks finish together, so nothing overlaps the writes and the finishing pass)
    int splits256 = 1;
    const double valid256 = static_cast<double>(p.M) / (((p.M + 255) / 256) * 256.0);
    for (int sp = 2; sp <= 8 && big_tiles * sp <= cus; ++sp) {
        const int kt = (KT + sp - 1) / sp;
        if (kt < 4) break;
        const int64_t units = big_tiles * sp;
        const double t = floor256(rounds256(units, kt)) + 9.0 + units * 0.262144 * valid256 * 0.33;
        if (t < t256) { t256 = t; splits256 = sp; }
    }
    if (tuning().gemm_splitk256 != TUNE_UNSET) splits256 = tuning().gemm_splitk256;
    int unused_splits = 1;
    bool unused_deep = false;
    const int64_t small_tiles_m = (p.M + 127) / 128;
    const double t128 = estimate128(small_tiles, small_tiles_m, small_tiles / small_tiles_m, KT, cus,
                                    static_cast<double>(p.M) / (small_tiles_m * 128.0), swiglu, &unused_splits, &unused_deep);
    const bool big = tuning().gemm_tile != TUNE_UNSET ? tuning().gemm_tile == 256 : t256 < t128;
    if (direct_ok) {
        if (big) return swiglu ? launch_direct<DT, MODE_SWIGLU>(p, cus, splits256, s) : launch_direct<DT, MODE_LINEAR>(p, cus, splits256, s);
        return swiglu ? launch_direct128<DT, MODE_SWIGLU>(p, cus, s) : launch_direct128<DT, MODE_LINEAR>(p, cus, s);
    }
    if (big) return swiglu ? launch_gemm<DT, MODE_SWIGLU, 256, 256, 2, 4>(p, s) : launch_gemm<DT, MODE_LINEAR, 256, 256, 2, 4>(p, s);
    return swiglu ? launch_gemm<DT, MODE_SWIGLU, 128, 128, 2, 2>(p, s) : launch_gemm<DT, MODE_LINEAR, 128, 128, 2, 2>(p, s);
}

template <int DT>
int launch_generic(const GemmParams &p, bool swiglu, hipStream_t s) {
    dim3 grid(static_cast<unsigned>((p.N + 63) / 64), static_cast<unsigned>((p.M + 63) / 64));
    TPAMD_REQUIRE(grid.y < 65536, "linear (generic kernel): M too large");
    if (swiglu) hipLaunchKernelGGL((gemm_generic_kernel<DT, MODE_SWIGLU>), grid, dim3(256), 0, s, p);
    else hipLaunchKernelGGL((gemm_generic_kernel<DT, MODE_LINEAR>), grid, dim3(256), 0, s, p);
    TPAMD_HIP(hipGetLastError());
    return TPAMD_OK;
}

int generic_dispatch(const GemmParams &p, int dtype, bool swiglu, hipStream_t s) {
    if (dtype == TPAMD_F32) return launch_generic<TPAMD_F32>(p, swiglu, s);
    return dtype == TPAMD_BF16 ? launch_generic<TPAMD_BF16>(p, swiglu, s) : launch_generic<TPAMD_F16>(p, swiglu, s);
}

int gemm_dispatch(const void *x, const void *w, const void *w2, const void *bias, const void *addend, int64_t ldadd, void *y,
                  int64_t M, int64_t N, int64_t K, int64_t ldx, int64_t ldw, int64_t ldy, int dtype, int act, bool swiglu,
                  bool generic, hipStream_t s) {
    GemmParams p{};
    p.x = static_cast<const char *>(x);
    p.w = static_cast<const char *>(w);
    p.w2 = static_cast<const char *>(w2);
    p.bias = static_cast<const char *>(bias);
    p.addend = static_cast<const char *>(addend);
    p.y = static_cast<char *>(y);
    p.M = static_cast<int>(M); p.N = static_cast<int>(N); p.K = static_cast<int>(K);
    p.ldx = ldx; p.ldw = ldw; p.ldy = ldy; p.ldadd = ldadd;
    p.act = act;
    if (dtype == TPAMD_F32 && !swiglu && K >= 4 && K % 4 == 0 && N % 4 == 0 && ldx % 4 == 0 && ldw % 4 == 0 && ldy % 4 == 0 &&
        aligned(x, 16) && aligned(w, 16) && aligned(y, 16) && (!bias || aligned(bias, 16)) &&
        (!addend || (aligned(addend, 16) && ldadd % 4 == 0))) {
        // fp32 rows that 16-byte accesses can take: the matrix pipe. 128 x 128 tiles once they fill the CUs, else 64 x 64.
        int dev = 0, cus = 256;
        TPAMD_HIP(hipGetDevice(&dev));
        if (int rc = device_cus(dev, &cus); rc != TPAMD_OK) return rc;
        const int64_t tiles128 = ((M + 127) / 128) * ((N + 127) / 128);
        if (tiles128 >= cus) return launch_gemm_f32<128, 128, 2, 2, 32>(p, s);
        const int64_t tiles64 = ((M + 63) / 64) * ((N + 63) / 64);
        if (tiles64 >= 2 * cus) return launch_gemm_f32<64, 64, 2, 2, 32>(p, s);
        if (tiles64 * 2 >= cus) return launch_gemm_f32<64, 64, 2, 2, 128>(p, s);  // few tiles: long stages, a block per CU
        return launch_gemm_f32_small(p, s);  // fewer still: 32 x 32 tiles whose K is shared by the block's wavefronts
    }
    if (dtype == TPAMD_F32 || generic) return generic_dispatch(p, dtype, swiglu, s);
    return dtype == TPAMD_BF16 ? gemm_large<TPAMD_BF16>(p, swiglu, s) : gemm_large<TPAMD_F16>(p, swiglu, s);
}

// int8 weights above the weight-streaming kernels' row count. x, wq 16-byte aligned, K and ldw multiples of 16, ldx of 8
// (checked by the caller); N and ldy multiples of 4 and y 8-byte aligned for the packed stores.
int gemm_w8_dispatch(const void *x, const void *wq, const void *scale, const void *outlier_idx, const void *w_out, int64_t n_out,
                     const void *bias, void *y, int64_t M, int64_t N, int64_t K, int64_t ldx, int64_t ldw, int64_t ld_wout,
                     int64_t ldy, int dtype, int act, hipStream_t s) {
    GemmParams p{};
    p.x = static_cast<const char *>(x);
    p.w = static_cast<const char *>(wq);
    p.bias = static_cast<const char *>(bias);
    p.y = static_cast<char *>(y);
    p.M = static_cast<int>(M); p.N = static_cast<int>(N); p.K = static_cast<int>(K);
    p.ldx = ldx; p.ldw = ldw; p.ldy = ldy;
    p.act = act;
    W8Extra q{static_cast<const float *>(scale), static_cast<const int *>(outlier_idx), static_cast<const char *>(w_out),
              static_cast<int>(n_out), ld_wout};
    int dev = 0, cus = 256;
    TPAMD_HIP(hipGetDevice(&dev));
    if (int rc = device_cus(dev, &cus); rc != TPAMD_OK) return rc;
    const int64_t tiles256 = ((M + 255) / 256) * ((N + 255) / 256);
    const bool big = tiles256 * 2 >= cus;
    if (dtype == TPAMD_BF16) return big ? launch_gemm_w8<TPAMD_BF16, 256, 256, 2, 4>(p, q, s) : launch_gemm_w8<TPAMD_BF16, 128, 128, 2, 2>(p, q, s);
    return big ? launch_gemm_w8<TPAMD_F16, 256, 256, 2, 4>(p, q, s) : launch_gemm_w8<TPAMD_F16, 128, 128, 2, 2>(p, q, s);
}

}  // namespace tpamd
