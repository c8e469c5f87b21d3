// Rank-shard Linear for prefill-sized M: y[M,N] = act(x[M,K] . w[N,K]^T + bias) on MFMA (bf16/f16),
// and the fused SiLU-gated gate/up pair. Both operands are K-contiguous, so x rows and w rows are
// staged into LDS the same way and fed to v_mfma_f32_32x32x16 with w as the row operand: a lane then
// holds 4 consecutive output columns of one output row, which packs into one 8-byte store.
//
// Two kernels share the tiling (block tile BM x BN x 64, WAVES_M x WAVES_N wavefronts of 64 lanes, two LDS
// stages, one barrier per K tile):
//   gemm_direct_kernel  256x256 tiles, K % 64 == 0. Global loads go straight into LDS (no register staging),
//                       operand fragments are read one K step ahead of the MFMAs that use them, and the MFMAs of
//                       the last K step of a tile overlap the barrier and the first fragment reads of the next.
//   gemm_kernel         any K (multiple of 8) and the 128x128 tiling for small problems; next K tile prefetched
//                       into registers while the current one is multiplied.
#include "common.h"

#include <type_traits>

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
    char *y;
    int M, N, K;
    int64_t ldx, ldw, ldy;  // elements
    int act;
    int tiles_m, tiles_n;
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
        const int64_t off = static_cast<int64_t>(kt) * BK * 2;
#pragma unroll
        for (int i = 0; i < XC; ++i) xr[i] = ok ? *reinterpret_cast<const uint4 *>(xg[i] + off) : make_uint4(0, 0, 0, 0);
#pragma unroll
        for (int i = 0; i < WC; ++i) wr[i] = ok ? *reinterpret_cast<const uint4 *>(wg[i] + off) : make_uint4(0, 0, 0, 0);
    };
    auto store_lds = [&](int stage) {
        char *xs = smem + stage * STAGE;
        char *ws = xs + BM * LDS_ROW;
#pragma unroll
        for (int i = 0; i < XC; ++i) *reinterpret_cast<uint4 *>(xs + st_off + i * (NT / 8) * LDS_ROW) = xr[i];
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
    store_lds(0);
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
        if (more) store_lds((kt + 1) & 1);
        __syncthreads();
    }

    epilogue<DT, MODE, BM, BN, WAVES_M, WAVES_N>(p, acc, m0, n0, wm, wn, l32, lhi);
}

typedef __attribute__((address_space(3))) void lds_void;
// Each lane's 16 bytes land at lds_base + lane * 16; lds_base must be the same for the whole wavefront.
__device__ __forceinline__ void load16_to_lds(const void *g, void *lds_base) {
    __builtin_amdgcn_global_load_lds(g, (lds_void *)lds_base, 16, 0, 0);
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

// LDS layout of the direct kernel: staged rows are grouped in blocks of 8 (1 KiB, what one wavefront-wide
// 16-byte-per-lane load fills), blocks are 1152 bytes apart, and inside a block the 16-byte chunk c of row r
// sits in slot c ^ (r % 8). Reads of one chunk index over 32 consecutive rows are then bank-conflict free,
// and every group of 8 lanes of a load still fetches one whole 128-byte row segment.
template <int DT, int MODE>
__global__ __launch_bounds__(512) void gemm_direct_kernel(GemmParams p) {
    constexpr int BM = 256, BN = 256, WAVES_M = 2, WAVES_N = 4, NW = 8;
    constexpr int TM = BM / WAVES_M / 32, TN = BN / WAVES_N / 32;
    constexpr int BLK = 1152;
    constexpr int XREG = (BM / 8) * BLK, WREG = (BN / 8) * BLK, STAGE = XREG + WREG;
    constexpr int XB = BM / 8 / NW, WB = BN / 8 / NW;  // 1 KiB blocks per wavefront per operand

    extern __shared__ __align__(16) char smem[];

    int tile_m, tile_n;
    tile_of_block(blockIdx.x, gridDim.x, p.tiles_m, p.tiles_n, tile_m, tile_n);
    const int m0 = tile_m * BM;
    const int n0 = tile_n * (MODE == MODE_SWIGLU ? BN / 2 : BN);

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int wm = wave / WAVES_N, wn = wave % WAVES_N;
    const int l32 = lane & 31, lhi = lane >> 5;

    // ---- global -> LDS: lane (rb, slot) of a load fetches chunk slot ^ rb of row rb of its block.
    // Addresses are a wavefront-uniform base (tile origin + K offset, advanced on the scalar unit) plus a 32-bit
    // per-lane offset computed once, so the loop spends no vector instructions on address arithmetic; the LDS
    // destination of each load is uniform too.
    const int rb = lane >> 3, slot = lane & 7;
    const int lchunk = slot ^ rb;
    const int wave_s = __builtin_amdgcn_readfirstlane(wave);
    const char *x_base = p.x + static_cast<int64_t>(m0) * p.ldx * 2;
    const char *w_base = p.w + static_cast<int64_t>(n0) * p.ldw * 2;
    const char *w2_base = MODE == MODE_SWIGLU ? p.w2 + static_cast<int64_t>(n0) * p.ldw * 2 : nullptr;
    uint32_t x_off[XB], w_off[WB];
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
    auto load_x = [&](int kt, int stage) {
        const char *base = x_base + static_cast<int64_t>(kt) * BK * 2;
        char *xs = smem + stage * STAGE;
#pragma unroll
        for (int i = 0; i < XB; ++i) load16_to_lds(base + x_off[i], xs + (wave_s + i * NW) * BLK);
    };
    auto load_w = [&](int kt, int stage) {
        char *ws = smem + stage * STAGE + XREG;
#pragma unroll
        for (int i = 0; i < WB; ++i) {
            const char *base = w_base;
            if constexpr (MODE == MODE_SWIGLU) base = (wave_s + i * NW) * 8 < BN / 2 ? w_base : w2_base;  // uniform per load
            load16_to_lds(base + static_cast<int64_t>(kt) * BK * 2 + w_off[i], ws + (wave_s + i * NW) * BLK);
        }
    };

    // ---- LDS -> MFMA operand addresses: one per-lane base for x and one for w; the MFMA tiles of a wavefront are a
    // compile-time number of 1152-byte blocks apart, which goes into the instruction's offset field
    constexpr int X_TILE_STEP = 4 * BLK;                                         // 32 rows
    constexpr int W_TILE_STEP = (MODE == MODE_SWIGLU ? (BN / 2) / 8 : 4) * BLK;  // swiglu: gate tile -> up tile
    static_assert(MODE == MODE_LINEAR || TN == 2, "swiglu operand addressing assumes one gate and one up tile per wavefront");
    int x_rd0, w_rd0;
    {
        const int r = wm * (BM / WAVES_M) + l32;
        x_rd0 = (r >> 3) * BLK + (r & 7) * 128;
        const int row = (MODE == MODE_SWIGLU ? wn * (BN / 2 / WAVES_N) : wn * (BN / WAVES_N)) + l32;
        w_rd0 = XREG + (row >> 3) * BLK + (row & 7) * 128;
    }
    int ks_off[BK / 16];
#pragma unroll
    for (int ks = 0; ks < BK / 16; ++ks) ks_off[ks] = ((ks * 2 + lhi) ^ (l32 & 7)) * 16;

    f32x16 acc[TM][TN];
#pragma unroll
    for (int a = 0; a < TM; ++a)
#pragma unroll
        for (int b = 0; b < TN; ++b)
#pragma unroll
            for (int i = 0; i < 16; ++i) acc[a][b][i] = 0.0f;

    static_assert(TM == 4 && TN == 2, "the counted waits below assume 6 fragment reads per K step");
    u32x4 xf[2][TM], wf[2][TN];
    const uint32_t smem_base = lds_addr_of(smem);
    auto read_frags = [&](auto bufc, int stage_off, int ks) {
        constexpr int buf = decltype(bufc)::value;
        const uint32_t xa = smem_base + stage_off + x_rd0 + ks_off[ks];
        const uint32_t wa = smem_base + stage_off + w_rd0 + ks_off[ks];
        xf[buf][0] = lds_read16<0>(xa);
        xf[buf][1] = lds_read16<X_TILE_STEP>(xa);
        xf[buf][2] = lds_read16<2 * X_TILE_STEP>(xa);
        xf[buf][3] = lds_read16<3 * X_TILE_STEP>(xa);
        wf[buf][0] = lds_read16<0>(wa);
        wf[buf][1] = lds_read16<W_TILE_STEP>(wa);
    };
    // LDS reads return in order: "at most N outstanding" means every read issued before the last N has landed.
    // Naming the fragments as operands keeps the MFMAs that consume them behind the wait.
#define TPAMD_WAIT_FRAGS(N, buf)                                                                                    \
    asm volatile("s_waitcnt lgkmcnt(" #N ")"                                                                        \
                 : "+v"(xf[buf][0]), "+v"(xf[buf][1]), "+v"(xf[buf][2]), "+v"(xf[buf][3]), "+v"(wf[buf][0]), "+v"(wf[buf][1]))
#define TPAMD_DRAIN_BARRIER(buf)                                                                                    \
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier"                                                       \
                 : "+v"(xf[buf][0]), "+v"(xf[buf][1]), "+v"(xf[buf][2]), "+v"(xf[buf][3]), "+v"(wf[buf][0]), "+v"(wf[buf][1]) \
                 :: "memory")
    auto mfmas = [&](auto bufc) {
        constexpr int buf = decltype(bufc)::value;
        __builtin_amdgcn_s_setprio(1);  // the matrix pipe is the scarce unit: do not let the peer's loads cut in
#pragma unroll
        for (int a = 0; a < TM; ++a)
#pragma unroll
            for (int b = 0; b < TN; ++b)
                acc[a][b] = mfma32<DT>(__builtin_bit_cast(uint4, wf[buf][b]), __builtin_bit_cast(uint4, xf[buf][a]), acc[a][b]);
        __builtin_amdgcn_s_setprio(0);
    };
    using B0 = std::integral_constant<int, 0>;
    using B1 = std::integral_constant<int, 1>;

    const int KT = p.K / BK;  // K is a multiple of 64 here
    load_x(0, 0);
    load_w(0, 0);
    drain_and_barrier();
    read_frags(B0{}, 0, 0);
    for (int kt = 0; kt < KT; ++kt) {
        const bool more = kt + 1 < KT;
        const int cur = (kt & 1) * STAGE, nxt = ((kt + 1) & 1) * STAGE;
        // K step 0: fragments of step 1 and half of the next tile's loads are issued, then step 0 multiplies
        read_frags(B1{}, cur, 1);
        if (more) load_x(kt + 1, (kt + 1) & 1);
        TPAMD_WAIT_FRAGS(6, 0);
        mfmas(B0{});
        read_frags(B0{}, cur, 2);
        if (more) load_w(kt + 1, (kt + 1) & 1);
        TPAMD_WAIT_FRAGS(6, 1);
        mfmas(B1{});
        read_frags(B1{}, cur, 3);
        TPAMD_WAIT_FRAGS(6, 0);
        mfmas(B0{});
        // every wavefront is done reading this tile and the next one has landed; the MFMAs of step 3 then run
        // under the first fragment reads of the next tile
        TPAMD_DRAIN_BARRIER(1);
        if (more) read_frags(B0{}, nxt, 0);
        mfmas(B1{});
    }
#undef TPAMD_WAIT_FRAGS
#undef TPAMD_DRAIN_BARRIER

    epilogue<DT, MODE, BM, BN, WAVES_M, WAVES_N>(p, acc, m0, n0, wm, wn, l32, lhi);
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
            }
            store_elem<DT>(p.y, static_cast<int64_t>(m) * p.ldy + n, v);
        }
    }
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

template <int DT, int MODE>
int launch_direct(GemmParams p, hipStream_t s) {
    constexpr int LDS = 2 * 64 * 1152;
    auto kern = gemm_direct_kernel<DT, MODE>;
    static thread_local int configured_dev = -1;
    int dev = 0;
    TPAMD_HIP(hipGetDevice(&dev));
    if (configured_dev != dev) {
        TPAMD_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, LDS));
        configured_dev = dev;
    }
    p.tiles_m = (p.M + 255) / 256;
    constexpr int BN_OUT = MODE == MODE_SWIGLU ? 128 : 256;
    p.tiles_n = (p.N + BN_OUT - 1) / BN_OUT;
    const int64_t blocks = static_cast<int64_t>(p.tiles_m) * p.tiles_n;
    TPAMD_REQUIRE(blocks < (1ll << 31), "gemm: too many tiles");
    hipLaunchKernelGGL(kern, dim3(static_cast<unsigned>(blocks)), dim3(512), LDS, s, p);
    TPAMD_HIP(hipGetLastError());
    return TPAMD_OK;
}

}  // namespace

// Prefill-sized dispatch; called by linear.hip once M is above the skinny range.
template <int DT>
int gemm_large(GemmParams p, bool swiglu, hipStream_t s) {
    // 256x256 tiles once they fill the chip at least about once, else 128x128 tiles.
    const int64_t big_tiles = static_cast<int64_t>((p.M + 255) / 256) * ((p.N + (swiglu ? 127 : 255)) / (swiglu ? 128 : 256));
    if (big_tiles >= 200) {
        if (p.K % 64 == 0 && p.K >= 64) return swiglu ? launch_direct<DT, MODE_SWIGLU>(p, s) : launch_direct<DT, MODE_LINEAR>(p, s);
        return swiglu ? launch_gemm<DT, MODE_SWIGLU, 256, 256, 2, 4>(p, s) : launch_gemm<DT, MODE_LINEAR, 256, 256, 2, 4>(p, s);
    }
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

int gemm_dispatch(const void *x, const void *w, const void *w2, const void *bias, void *y, int64_t M, int64_t N,
                  int64_t K, int64_t ldx, int64_t ldw, int64_t ldy, int dtype, int act, bool swiglu, bool generic, hipStream_t s) {
    GemmParams p{};
    p.x = static_cast<const char *>(x);
    p.w = static_cast<const char *>(w);
    p.w2 = static_cast<const char *>(w2);
    p.bias = static_cast<const char *>(bias);
    p.y = static_cast<char *>(y);
    p.M = static_cast<int>(M); p.N = static_cast<int>(N); p.K = static_cast<int>(K);
    p.ldx = ldx; p.ldw = ldw; p.ldy = ldy;
    p.act = act;
    if (dtype == TPAMD_F32 || generic) return generic_dispatch(p, dtype, swiglu, s);
    return dtype == TPAMD_BF16 ? gemm_large<TPAMD_BF16>(p, swiglu, s) : gemm_large<TPAMD_F16>(p, swiglu, s);
}

}  // namespace tpamd
