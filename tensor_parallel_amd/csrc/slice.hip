// Slicing engine: a batched 2-D byte-region mover. One launch moves every (tensor, rank) shard of a
// state dict. The host cuts each job into tiles of at most TILE_UNITS vector units (128 KiB when units are 16 bytes); a
// persistent grid of one 1024-thread block per CU walks the tile table. A block moves a tile in two bursts: every lane
// requests its up to 8 units, the block waits for all of them, then every lane stores its units. Measured on 13.5 GB: such
// bursts of 128 KiB per CU copy at 5.78 TB/s (read + write), against 5.1-5.2 TB/s for the same bytes moved 16 KiB at a time
// by sixteen 256-thread blocks per CU, whose loads and stores mix at every moment. HBM-bound: every byte is read once and
// written once.
#include "common.h"

#include <algorithm>
#include <new>
#include <vector>

namespace tpamd {

namespace {

constexpr int COPY_THREADS = 1024;
constexpr int COPY_UNITS_PER_LANE = 8;
constexpr uint32_t MAX_TILE_UNITS = COPY_THREADS * COPY_UNITS_PER_LANE;  // vector units per tile (128 KiB when units are 16 bytes)
constexpr int TR_THREADS = 256;  // the transposing mover's block
constexpr int COPY_NT_DEFAULT = 3;  // bit 0: non-temporal loads, bit 1: non-temporal stores (TPAMD_COPY_NT overrides)

struct alignas(16) Tile {
    const char *src;
    char *dst;
    uint64_t src_pitch;
    uint64_t dst_pitch;
    uint32_t rows;
    uint32_t units_per_row;  // row length in units of `vec` bytes
    uint32_t magic;          // ceil(2^32 / units_per_row), 0 when units_per_row == 1
    uint32_t vec;            // 16, 8, 4, 2 or 1
};
static_assert(sizeof(Tile) == 48, "Tile layout");

// NT bit 0: non-temporal loads, bit 1: non-temporal stores.
template <int NT, typename V>
__device__ __forceinline__ V ld_stream(const V *p) {
    if constexpr ((NT & 1) != 0) return __builtin_nontemporal_load(p);
    else return *p;
}
template <int NT, typename V>
__device__ __forceinline__ void st_stream(V *p, V v) {
    if constexpr ((NT & 2) != 0) __builtin_nontemporal_store(v, p);
    else *p = v;
}

// Moves one tile with units of type V: all loads, then all stores. idx -> (row, col) uses a multiply-high by a host-made
// reciprocal: exact because idx < 2^13 and units_per_row <= 2^13. A full contiguous tile (the bulk of a state dict) takes
// a path without any arithmetic or predicate between its accesses: measured on 13.5 GB, bounds checks on every access of
// the bursts cost 7-12 % of the bandwidth. On the other tiles a wavefront whose 64 units all lie inside the tile (decided
// on scalars) skips the per-lane checks too.
template <int NT, typename V>
__device__ __forceinline__ void move_tile(const Tile &t, int tid) {
    const uint32_t upr = t.units_per_row;
    const uint32_t total = t.rows * upr;
    V v[COPY_UNITS_PER_LANE];
    if (t.rows == 1 && total == MAX_TILE_UNITS) {
        const V *s = reinterpret_cast<const V *>(t.src) + tid;
        V *d = reinterpret_cast<V *>(t.dst) + tid;
#pragma unroll
        for (int i = 0; i < COPY_UNITS_PER_LANE; ++i) v[i] = ld_stream<NT>(s + i * COPY_THREADS);
        // the block's reads are one burst and its writes another: nothing is stored before the lane's last load has arrived
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#pragma unroll
        for (int i = 0; i < COPY_UNITS_PER_LANE; ++i) st_stream<NT>(d + i * COPY_THREADS, v[i]);
        return;
    }
    // rows of upr units: unit idx = tid + i * 1024 sits at (row, col) = (idx / upr, idx % upr). One multiply-high places the
    // lane's first unit, every further one is a step of (1024 / upr, 1024 % upr) with a carry
    // (a single row - the ragged end of a contiguous region, a piece of a long row - never carries: magic is 0 there and
    // so it is for rows of one unit)
    const uint32_t magic = t.magic;
    const bool one_row = t.rows == 1;
    const uint32_t step_row = one_row ? 0u : magic ? __umulhi(static_cast<uint32_t>(COPY_THREADS), magic) : static_cast<uint32_t>(COPY_THREADS);
    const uint32_t step_col = COPY_THREADS - step_row * upr;
    const uint32_t wave_first = __builtin_amdgcn_readfirstlane(tid & ~63);
    uint32_t row = one_row ? 0u : magic ? __umulhi(static_cast<uint32_t>(tid), magic) : static_cast<uint32_t>(tid);
    uint32_t col = tid - row * upr;
    const uint32_t sp = static_cast<uint32_t>(t.src_pitch), dp = static_cast<uint32_t>(t.dst_pitch);  // the host keeps the pitches of such tiles below 4 GiB
    uint64_t src_at[COPY_UNITS_PER_LANE], dst_at[COPY_UNITS_PER_LANE];
#pragma unroll
    for (int i = 0; i < COPY_UNITS_PER_LANE; ++i) {
        // lanes past the end of the tile read its first unit again (a tile has at least one) and store nothing
        const bool in = wave_first + i * COPY_THREADS + 63 < total || tid + i * COPY_THREADS < total;
        src_at[i] = in ? static_cast<uint64_t>(row) * sp + col * static_cast<uint32_t>(sizeof(V)) : 0;
        dst_at[i] = static_cast<uint64_t>(row) * dp + col * static_cast<uint32_t>(sizeof(V));
        row += step_row;
        col += step_col;
        if (!one_row && col >= upr) {
            col -= upr;
            ++row;
        }
    }
#pragma unroll
    for (int i = 0; i < COPY_UNITS_PER_LANE; ++i) v[i] = ld_stream<NT>(reinterpret_cast<const V *>(t.src + src_at[i]));
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#pragma unroll
    for (int i = 0; i < COPY_UNITS_PER_LANE; ++i) {
        if (wave_first + i * COPY_THREADS + 63 < total) st_stream<NT>(reinterpret_cast<V *>(t.dst + dst_at[i]), v[i]);
        else if (tid + i * COPY_THREADS < total) st_stream<NT>(reinterpret_cast<V *>(t.dst + dst_at[i]), v[i]);
    }
}

template <int NT>
__global__ __launch_bounds__(COPY_THREADS) void copy_tiles_kernel(const Tile *__restrict__ tiles, uint32_t n_tiles) {
    const int tid = threadIdx.x;
    for (uint32_t ti = blockIdx.x; ti < n_tiles; ti += gridDim.x) {
        const Tile t = tiles[ti];  // block-uniform: scalar loads
        switch (t.vec) {
            case 16: move_tile<NT, v4u>(t, tid); break;
            case 8: move_tile<NT, v2u>(t, tid); break;
            case 4: move_tile<NT, uint32_t>(t, tid); break;
            case 2: move_tile<NT, uint16_t>(t, tid); break;
            default: move_tile<NT, uint8_t>(t, tid); break;
        }
    }
}

// ---- small batches: up to SMALL_MAX_JOBS jobs travel in the kernel arguments, tiles are derived on the device ----
constexpr int SMALL_MAX_JOBS = 16;
struct SmallJob {
    const char *src;
    char *dst;
    uint64_t rows, src_pitch, dst_pitch;
    uint64_t upr_full;    // row length in units of `vec` bytes
    uint32_t vec;
    uint32_t kind;        // 0 contiguous, 1 long rows, 2 short rows
    uint32_t tiles_per_row_or_rows_per_tile;
    uint32_t tile_begin;  // first global tile index of this job
};
struct SmallBatch {
    SmallJob job[SMALL_MAX_JOBS];
    uint32_t n_jobs, n_tiles;
};

__global__ __launch_bounds__(COPY_THREADS) void copy_small_kernel(SmallBatch b) {
    const int tid = threadIdx.x;
    for (uint32_t ti = blockIdx.x; ti < b.n_tiles; ti += gridDim.x) {
        uint32_t ji = 0;
        while (ji + 1 < b.n_jobs && b.job[ji + 1].tile_begin <= ti) ++ji;  // block-uniform
        const SmallJob &j = b.job[ji];
        const uint64_t local = ti - j.tile_begin;
        Tile t{};
        t.vec = j.vec;
        if (j.kind == 0) {
            const uint64_t units = j.rows * j.upr_full, u = local * MAX_TILE_UNITS;
            t.src = j.src + u * j.vec;
            t.dst = j.dst + u * j.vec;
            t.rows = 1;
            t.units_per_row = static_cast<uint32_t>(units - u < MAX_TILE_UNITS ? units - u : MAX_TILE_UNITS);
        } else if (j.kind == 1) {
            const uint64_t r = local / j.tiles_per_row_or_rows_per_tile, u = (local % j.tiles_per_row_or_rows_per_tile) * MAX_TILE_UNITS;
            t.src = j.src + r * j.src_pitch + u * j.vec;
            t.dst = j.dst + r * j.dst_pitch + u * j.vec;
            t.rows = 1;
            t.units_per_row = static_cast<uint32_t>(j.upr_full - u < MAX_TILE_UNITS ? j.upr_full - u : MAX_TILE_UNITS);
        } else {
            const uint64_t rpt = j.tiles_per_row_or_rows_per_tile, r = local * rpt;
            const uint32_t upr = static_cast<uint32_t>(j.upr_full);
            t.src = j.src + r * j.src_pitch;
            t.dst = j.dst + r * j.dst_pitch;
            t.src_pitch = j.src_pitch;
            t.dst_pitch = j.dst_pitch;
            t.rows = static_cast<uint32_t>(j.rows - r < rpt ? j.rows - r : rpt);
            t.units_per_row = upr;
            t.magic = upr == 1 ? 0u : static_cast<uint32_t>(((1ull << 32) + upr - 1) / upr);
        }
        switch (t.vec) {
            case 16: move_tile<3, v4u>(t, tid); break;
            case 8: move_tile<3, v2u>(t, tid); break;
            case 4: move_tile<3, uint32_t>(t, tid); break;
            case 2: move_tile<3, uint16_t>(t, tid); break;
            default: move_tile<3, uint8_t>(t, tid); break;
        }
    }
}

// ---- transposing mover: dst[c][r] = src[r][c] over 2-D element regions, staged through LDS ---------------------------
// A tile is TS x TS elements with TS * sizeof(E) = 128 bytes, so both the source rows read and the destination rows
// written are whole 128-byte lines. The block stages the tile in LDS row by row (16-byte loads, 8 lanes per source
// row), then every lane gathers the 16 bytes of one destination row segment from a column of the staged tile and
// stores them (8 lanes per destination row). Rows of the LDS tile are padded by 4 bytes: a lane's column reads walk
// down 128 / TS-apart rows and would otherwise all meet in one bank. Regions whose base addresses or pitches are not
// multiples of 16 bytes, and tiles cut by the region's edge, move element by element through the same staging.
constexpr int TR_MAX_JOBS = 16;
struct TransposeJob {
    const char *src;
    char *dst;
    uint64_t rows, cols;  // extent of the source region in elements
    uint64_t src_pitch, dst_pitch;
    uint32_t tiles_c;     // tiles along the source columns
    uint32_t tile_begin;  // first global tile index of this job
    uint32_t vec_ok;      // both sides allow 16-byte accesses
};
struct TransposeBatch {
    TransposeJob job[TR_MAX_JOBS];
    uint32_t n_jobs, n_tiles;
};

template <typename E>
__global__ __launch_bounds__(TR_THREADS) void transpose_tiles_kernel(TransposeBatch b) {
    constexpr int ES = sizeof(E);
    constexpr int TS = 128 / ES;       // tile edge in elements
    constexpr int PER = 16 / ES;       // elements per 16-byte chunk
    constexpr int PITCH = TS + 4 / ES; // LDS row pitch in elements (128 bytes + 4)
    constexpr int PASSES = TS / 32;    // 256 lanes cover 32 rows of 8 chunks per pass
    __shared__ __attribute__((aligned(4))) E tile[TS * PITCH];
    const int tid = threadIdx.x;
    const int chunk = tid & 7, lrow = tid >> 3;
    for (uint32_t ti = blockIdx.x; ti < b.n_tiles; ti += gridDim.x) {
        uint32_t ji = 0;
        while (ji + 1 < b.n_jobs && b.job[ji + 1].tile_begin <= ti) ++ji;  // block-uniform
        const TransposeJob &j = b.job[ji];
        const uint32_t local = ti - j.tile_begin;
        const uint64_t r0 = static_cast<uint64_t>(local / j.tiles_c) * TS, c0 = static_cast<uint64_t>(local % j.tiles_c) * TS;
        const uint32_t nr = static_cast<uint32_t>(j.rows - r0 < TS ? j.rows - r0 : TS);
        const uint32_t nc = static_cast<uint32_t>(j.cols - c0 < TS ? j.cols - c0 : TS);
        const bool whole = j.vec_ok && nr == TS && nc == TS;
        // stage: lane (lrow, chunk) of a pass brings elements [chunk * PER, +PER) of source row lrow + 32 * pass
        if (whole) {
            v4u regs[PASSES];
#pragma unroll
            for (int p = 0; p < PASSES; ++p)
                regs[p] = __builtin_nontemporal_load(reinterpret_cast<const v4u *>(j.src + (r0 + lrow + 32 * p) * j.src_pitch + c0 * ES) + chunk);
#pragma unroll
            for (int p = 0; p < PASSES; ++p) {
                uint32_t *row = reinterpret_cast<uint32_t *>(tile + (lrow + 32 * p) * PITCH) + chunk * 4;
                row[0] = regs[p].x, row[1] = regs[p].y, row[2] = regs[p].z, row[3] = regs[p].w;
            }
        } else {
#pragma unroll
            for (int p = 0; p < PASSES; ++p) {
                const uint32_t r = lrow + 32 * p;
                if (r >= nr) continue;
                const E *s = reinterpret_cast<const E *>(j.src + (r0 + r) * j.src_pitch) + c0;
                for (uint32_t c = chunk * PER; c < static_cast<uint32_t>(chunk + 1) * PER && c < nc; ++c) tile[r * PITCH + c] = s[c];
            }
        }
        __syncthreads();
        // write: lane (lrow, chunk) of a pass stores elements [chunk * PER, +PER) of destination row lrow + 32 * pass,
        // which are source rows chunk * PER ... of source column lrow + 32 * pass
#pragma unroll
        for (int p = 0; p < PASSES; ++p) {
            const uint32_t c = lrow + 32 * p;  // source column = destination row
            if (whole) {
                E v[PER];
#pragma unroll
                for (int i = 0; i < PER; ++i) v[i] = tile[(chunk * PER + i) * PITCH + c];
                v4u out;
                __builtin_memcpy(&out, v, 16);
                __builtin_nontemporal_store(out, reinterpret_cast<v4u *>(j.dst + (c0 + c) * j.dst_pitch + r0 * ES) + chunk);
            } else if (c < nc) {
                E *d = reinterpret_cast<E *>(j.dst + (c0 + c) * j.dst_pitch) + r0;
                for (uint32_t r = chunk * PER; r < static_cast<uint32_t>(chunk + 1) * PER && r < nr; ++r) d[r] = tile[r * PITCH + c];
            }
        }
        __syncthreads();  // the tile is reused by the next iteration
    }
}

template <int DT>
__global__ __launch_bounds__(256) void scale_kernel(const void *__restrict__ in, void *__restrict__ out, uint64_t n,
                                                    float w, int mul) {
    uint64_t i = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    const uint64_t stride = static_cast<uint64_t>(gridDim.x) * blockDim.x;
    for (; i < n; i += stride) {
        if constexpr (DT == TPAMD_F32) {
            float v = static_cast<const float *>(in)[i];
            static_cast<float *>(out)[i] = mul ? v * w : v / w;
        } else {
            float v = half_to_f32<DT>(static_cast<const uint16_t *>(in)[i]);
            static_cast<uint16_t *>(out)[i] = f32_to_half<DT>(mul ? v * w : v / w);
        }
    }
}

uint32_t pick_vec(const tpamd_copy_job &j) {
    uint64_t bits = reinterpret_cast<uintptr_t>(j.src_dev) | reinterpret_cast<uintptr_t>(j.dst_dev) | j.row_bytes;
    if (j.rows > 1) bits |= j.src_pitch | j.dst_pitch;
    for (uint32_t v = 16; v > 1; v >>= 1)
        if ((bits & (v - 1)) == 0) return v;
    return 1;
}

}  // namespace

}  // namespace tpamd

struct tpamd_copy_plan {
    tpamd::Tile *tiles_dev = nullptr;
    uint32_t n_tiles = 0;
    uint64_t bytes = 0;
    int device = -1;
    int grid = 0;
};

using namespace tpamd;

extern "C" int tpamd_copy_plan_create(const tpamd_copy_job *jobs, size_t n_jobs, tpamd_copy_plan **plan_out) {
    TPAMD_REQUIRE(plan_out != nullptr, "tpamd_copy_plan_create: plan_out is NULL");
    TPAMD_REQUIRE(jobs != nullptr || n_jobs == 0, "tpamd_copy_plan_create: jobs is NULL with n_jobs=%zu", n_jobs);
    *plan_out = nullptr;
    std::vector<Tile> tiles;
    uint64_t bytes = 0;
    uint32_t TILE_UNITS = MAX_TILE_UNITS;
    {  // tuning knob
        const int v = tuning().copy_tile_units;
        if (v >= 256 && v <= static_cast<int>(MAX_TILE_UNITS)) TILE_UNITS = static_cast<uint32_t>(v);
    }
    try {
        for (size_t ji = 0; ji < n_jobs; ++ji) {
            const tpamd_copy_job &j = jobs[ji];
            if (j.rows == 0 || j.row_bytes == 0) continue;
            TPAMD_REQUIRE(j.src_dev != nullptr && j.dst_dev != nullptr, "copy job %zu: null pointer", ji);
            TPAMD_REQUIRE(j.rows == 1 || (j.src_pitch >= j.row_bytes && j.dst_pitch >= j.row_bytes),
                          "copy job %zu: pitch (%llu src, %llu dst) smaller than row_bytes %llu", ji,
                          (unsigned long long)j.src_pitch, (unsigned long long)j.dst_pitch,
                          (unsigned long long)j.row_bytes);
            bytes += j.rows * j.row_bytes;
            const uint32_t vec = pick_vec(j);
            const uint64_t upr_full = j.row_bytes / vec;
            const char *src = static_cast<const char *>(j.src_dev);
            char *dst = static_cast<char *>(j.dst_dev);
            const bool contiguous = (j.rows == 1) || (j.src_pitch == j.row_bytes && j.dst_pitch == j.row_bytes);
            if (contiguous) {
                const uint64_t units = j.rows * upr_full;
                for (uint64_t u = 0; u < units; u += TILE_UNITS) {
                    Tile t{};
                    t.src = src + u * vec;
                    t.dst = dst + u * vec;
                    t.rows = 1;
                    t.units_per_row = static_cast<uint32_t>(units - u < TILE_UNITS ? units - u : TILE_UNITS);
                    t.vec = vec;
                    tiles.push_back(t);
                }
            } else if (upr_full >= TILE_UNITS) {  // long rows: cut every row into column tiles
                for (uint64_t r = 0; r < j.rows; ++r)
                    for (uint64_t u = 0; u < upr_full; u += TILE_UNITS) {
                        Tile t{};
                        t.src = src + r * j.src_pitch + u * vec;
                        t.dst = dst + r * j.dst_pitch + u * vec;
                        t.rows = 1;
                        t.units_per_row = static_cast<uint32_t>(upr_full - u < TILE_UNITS ? upr_full - u : TILE_UNITS);
                        t.vec = vec;
                        tiles.push_back(t);
                    }
            } else {  // short rows: several whole rows per tile
                TPAMD_REQUIRE(j.src_pitch < (1ull << 32) && j.dst_pitch < (1ull << 32), "copy job %zu: a pitch of 4 GiB or more with rows shorter than a tile", ji);
                const uint32_t upr = static_cast<uint32_t>(upr_full);
                const uint64_t rpt = TILE_UNITS / upr;  // >= 1
                for (uint64_t r = 0; r < j.rows; r += rpt) {
                    Tile t{};
                    t.src = src + r * j.src_pitch;
                    t.dst = dst + r * j.dst_pitch;
                    t.src_pitch = j.src_pitch;
                    t.dst_pitch = j.dst_pitch;
                    t.rows = static_cast<uint32_t>(j.rows - r < rpt ? j.rows - r : rpt);
                    t.units_per_row = upr;
                    t.magic = upr == 1 ? 0u : static_cast<uint32_t>(((1ull << 32) + upr - 1) / upr);
                    t.vec = vec;
                    tiles.push_back(t);
                }
            }
            TPAMD_REQUIRE(tiles.size() < 0xffffff00ull, "copy plan too large (%zu tiles)", tiles.size());
        }
    } catch (const std::bad_alloc &) {
        set_error("tpamd_copy_plan_create: out of host memory building the tile table");
        return TPAMD_ERR_NOMEM;
    }

    // Tiles in order of their source addresses: the shards of one tensor that different ranks cut out of the same rows
    // (a split along the inner axis reads every other piece of each row) are then moved by neighbouring blocks at the same
    // time, and between them the blocks read whole rows.
    if (tuning().copy_sort != 0)
        std::stable_sort(tiles.begin(), tiles.end(), [](const Tile &a, const Tile &b) { return a.src < b.src; });

    tpamd_copy_plan *plan = new (std::nothrow) tpamd_copy_plan();
    if (!plan) {
        set_error("tpamd_copy_plan_create: out of host memory");
        return TPAMD_ERR_NOMEM;
    }
    plan->n_tiles = static_cast<uint32_t>(tiles.size());
    plan->bytes = bytes;
    hipError_t e = hipGetDevice(&plan->device);
    hipDeviceProp_t prop;
    if (e == hipSuccess) e = hipGetDeviceProperties(&prop, plan->device);
    if (e == hipSuccess && plan->n_tiles) {
        int per_cu = 1;  // one 1024-thread block per CU: two per CU measured 1-2 % slower on 13.5 GB
        {
            const int v = tuning().copy_blocks_per_cu;
            if (v >= 1 && v <= 64) per_cu = v;
        }
        const uint64_t cap = static_cast<uint64_t>(prop.multiProcessorCount) * per_cu;
        plan->grid = static_cast<int>(plan->n_tiles < cap ? plan->n_tiles : cap);
        e = hipMalloc(reinterpret_cast<void **>(&plan->tiles_dev), tiles.size() * sizeof(Tile));
        if (e == hipSuccess)
            e = hipMemcpy(plan->tiles_dev, tiles.data(), tiles.size() * sizeof(Tile), hipMemcpyHostToDevice);
    }
    if (e != hipSuccess) {
        set_error("tpamd_copy_plan_create: %s", hipGetErrorString(e));
        if (plan->tiles_dev) (void)hipFree(plan->tiles_dev);
        delete plan;
        return TPAMD_ERR_HIP;
    }
    *plan_out = plan;
    return TPAMD_OK;
}

extern "C" int tpamd_copy_plan_run(const tpamd_copy_plan *plan, void *stream) {
    TPAMD_REQUIRE(plan != nullptr, "tpamd_copy_plan_run: plan is NULL");
    if (plan->n_tiles == 0) return TPAMD_OK;
    int dev = -1;
    TPAMD_HIP(hipGetDevice(&dev));
    TPAMD_REQUIRE(dev == plan->device, "tpamd_copy_plan_run: plan was made on device %d, current is %d", plan->device,
                  dev);
    const dim3 grid(plan->grid), block(COPY_THREADS);
    hipStream_t s = static_cast<hipStream_t>(stream);
    switch (tuning().copy_nt == TUNE_UNSET ? COPY_NT_DEFAULT : tuning().copy_nt & 3) {
        case 0: hipLaunchKernelGGL(copy_tiles_kernel<0>, grid, block, 0, s, plan->tiles_dev, plan->n_tiles); break;
        case 1: hipLaunchKernelGGL(copy_tiles_kernel<1>, grid, block, 0, s, plan->tiles_dev, plan->n_tiles); break;
        case 2: hipLaunchKernelGGL(copy_tiles_kernel<2>, grid, block, 0, s, plan->tiles_dev, plan->n_tiles); break;
        default: hipLaunchKernelGGL(copy_tiles_kernel<3>, grid, block, 0, s, plan->tiles_dev, plan->n_tiles); break;
    }
    TPAMD_HIP(hipGetLastError());
    return TPAMD_OK;
}

extern "C" int tpamd_copy_jobs_run(const tpamd_copy_job *jobs, size_t n_jobs, void *stream) {
    TPAMD_REQUIRE(n_jobs <= static_cast<size_t>(SMALL_MAX_JOBS), "tpamd_copy_jobs_run: at most %d jobs (got %zu); use a copy plan",
                  SMALL_MAX_JOBS, n_jobs);
    TPAMD_REQUIRE(jobs != nullptr || n_jobs == 0, "tpamd_copy_jobs_run: jobs is NULL");
    SmallBatch b{};
    uint64_t tiles = 0;
    for (size_t ji = 0; ji < n_jobs; ++ji) {
        const tpamd_copy_job &j = jobs[ji];
        if (j.rows == 0 || j.row_bytes == 0) continue;
        TPAMD_REQUIRE(j.src_dev != nullptr && j.dst_dev != nullptr, "copy job %zu: null pointer", ji);
        TPAMD_REQUIRE(j.rows == 1 || (j.src_pitch >= j.row_bytes && j.dst_pitch >= j.row_bytes),
                      "copy job %zu: pitch smaller than row_bytes", ji);
        SmallJob &d = b.job[b.n_jobs++];
        d.src = static_cast<const char *>(j.src_dev);
        d.dst = static_cast<char *>(j.dst_dev);
        d.rows = j.rows;
        d.src_pitch = j.src_pitch;
        d.dst_pitch = j.dst_pitch;
        d.vec = pick_vec(j);
        d.upr_full = j.row_bytes / d.vec;
        d.tile_begin = static_cast<uint32_t>(tiles);
        const bool contiguous = (j.rows == 1) || (j.src_pitch == j.row_bytes && j.dst_pitch == j.row_bytes);
        uint64_t nt;
        if (contiguous) {
            d.kind = 0;
            nt = (j.rows * d.upr_full + MAX_TILE_UNITS - 1) / MAX_TILE_UNITS;
        } else if (d.upr_full >= MAX_TILE_UNITS) {
            d.kind = 1;
            d.tiles_per_row_or_rows_per_tile = static_cast<uint32_t>((d.upr_full + MAX_TILE_UNITS - 1) / MAX_TILE_UNITS);
            nt = j.rows * d.tiles_per_row_or_rows_per_tile;
        } else {
            TPAMD_REQUIRE(j.src_pitch < (1ull << 32) && j.dst_pitch < (1ull << 32), "copy job %zu: a pitch of 4 GiB or more with rows shorter than a tile", ji);
            d.kind = 2;
            d.tiles_per_row_or_rows_per_tile = static_cast<uint32_t>(MAX_TILE_UNITS / d.upr_full);
            nt = (j.rows + d.tiles_per_row_or_rows_per_tile - 1) / d.tiles_per_row_or_rows_per_tile;
        }
        tiles += nt;
        TPAMD_REQUIRE(tiles < 0xffffff00ull, "tpamd_copy_jobs_run: too many tiles");
    }
    if (tiles == 0) return TPAMD_OK;
    b.n_tiles = static_cast<uint32_t>(tiles);
    int dev = 0, cus = 256;
    TPAMD_HIP(hipGetDevice(&dev));
    if (int rc_cus = device_cus(dev, &cus); rc_cus != TPAMD_OK) return rc_cus;
    const uint64_t cap = static_cast<uint64_t>(cus);
    hipLaunchKernelGGL(copy_small_kernel, dim3(static_cast<unsigned>(tiles < cap ? tiles : cap)), dim3(COPY_THREADS), 0,
                       static_cast<hipStream_t>(stream), b);
    TPAMD_HIP(hipGetLastError());
    return TPAMD_OK;
}

extern "C" int tpamd_transpose_jobs_run(const tpamd_transpose_job *jobs, size_t n_jobs, int elem_bytes, void *stream) {
    TPAMD_REQUIRE(n_jobs <= static_cast<size_t>(TR_MAX_JOBS), "tpamd_transpose_jobs_run: at most %d jobs (got %zu)", TR_MAX_JOBS, n_jobs);
    TPAMD_REQUIRE(jobs != nullptr || n_jobs == 0, "tpamd_transpose_jobs_run: jobs is NULL");
    TPAMD_REQUIRE(elem_bytes == 1 || elem_bytes == 2 || elem_bytes == 4, "tpamd_transpose_jobs_run: elem_bytes %d (1, 2 or 4)", elem_bytes);
    const uint64_t es = static_cast<uint64_t>(elem_bytes), ts = 128 / es;
    TransposeBatch b{};
    uint64_t tiles = 0;
    for (size_t ji = 0; ji < n_jobs; ++ji) {
        const tpamd_transpose_job &j = jobs[ji];
        if (j.rows == 0 || j.cols == 0) continue;
        TPAMD_REQUIRE(j.src_dev != nullptr && j.dst_dev != nullptr, "transpose job %zu: null pointer", ji);
        TPAMD_REQUIRE(j.src_pitch >= j.cols * es && j.dst_pitch >= j.rows * es,
                      "transpose job %zu: pitch (%llu src, %llu dst) smaller than a row (%llu, %llu bytes)", ji,
                      (unsigned long long)j.src_pitch, (unsigned long long)j.dst_pitch, (unsigned long long)(j.cols * es),
                      (unsigned long long)(j.rows * es));
        TPAMD_REQUIRE(j.src_pitch % es == 0 && j.dst_pitch % es == 0 && aligned(j.src_dev, es) && aligned(j.dst_dev, es),
                      "transpose job %zu: pointers and pitches must be multiples of the element size %d", ji, elem_bytes);
        TransposeJob &d = b.job[b.n_jobs++];
        d.src = static_cast<const char *>(j.src_dev);
        d.dst = static_cast<char *>(j.dst_dev);
        d.rows = j.rows;
        d.cols = j.cols;
        d.src_pitch = j.src_pitch;
        d.dst_pitch = j.dst_pitch;
        d.vec_ok = aligned(j.src_dev, 16) && aligned(j.dst_dev, 16) && j.src_pitch % 16 == 0 && j.dst_pitch % 16 == 0;
        const uint64_t tr = (j.rows + ts - 1) / ts, tc = (j.cols + ts - 1) / ts;
        TPAMD_REQUIRE(tc < 0x7fffffffull && tr < 0x7fffffffull && tiles + tr * tc < 0xffffff00ull, "tpamd_transpose_jobs_run: too many tiles");
        d.tiles_c = static_cast<uint32_t>(tc);
        d.tile_begin = static_cast<uint32_t>(tiles);
        tiles += tr * tc;
    }
    if (tiles == 0) return TPAMD_OK;
    b.n_tiles = static_cast<uint32_t>(tiles);
    int dev = 0, cus = 256;
    TPAMD_HIP(hipGetDevice(&dev));
    if (int rc_cus = device_cus(dev, &cus); rc_cus != TPAMD_OK) return rc_cus;
    const uint64_t cap = static_cast<uint64_t>(cus) * 8;
    const dim3 grid(static_cast<unsigned>(tiles < cap ? tiles : cap)), block(TR_THREADS);
    hipStream_t s = static_cast<hipStream_t>(stream);
    switch (elem_bytes) {
        case 1: hipLaunchKernelGGL(transpose_tiles_kernel<uint8_t>, grid, block, 0, s, b); break;
        case 2: hipLaunchKernelGGL(transpose_tiles_kernel<uint16_t>, grid, block, 0, s, b); break;
        default: hipLaunchKernelGGL(transpose_tiles_kernel<uint32_t>, grid, block, 0, s, b); break;
    }
    TPAMD_HIP(hipGetLastError());
    return TPAMD_OK;
}

extern "C" uint64_t tpamd_copy_plan_bytes(const tpamd_copy_plan *plan) { return plan ? plan->bytes : 0; }

extern "C" int tpamd_copy_plan_destroy(tpamd_copy_plan *plan) {
    if (!plan) return TPAMD_OK;
    hipError_t e = plan->tiles_dev ? hipFree(plan->tiles_dev) : hipSuccess;
    delete plan;
    if (e != hipSuccess) {
        set_error("tpamd_copy_plan_destroy: %s", hipGetErrorString(e));
        return TPAMD_ERR_HIP;
    }
    return TPAMD_OK;
}

extern "C" int tpamd_scale(const void *in_dev, void *out_dev, uint64_t n_elems, int dtype, int world_size, int mul,
                           void *stream) {
    TPAMD_REQUIRE(world_size >= 1, "tpamd_scale: world_size %d", world_size);
    if (n_elems == 0) return TPAMD_OK;
    TPAMD_REQUIRE(in_dev && out_dev, "tpamd_scale: null pointer");
    const uint64_t want = (n_elems + 255) / 256;
    const int grid = static_cast<int>(want < 4096 ? want : 4096);
    hipStream_t s = static_cast<hipStream_t>(stream);
    const float w = static_cast<float>(world_size);
    switch (dtype) {
        case TPAMD_BF16: hipLaunchKernelGGL(scale_kernel<TPAMD_BF16>, dim3(grid), dim3(256), 0, s, in_dev, out_dev, n_elems, w, mul); break;
        case TPAMD_F16: hipLaunchKernelGGL(scale_kernel<TPAMD_F16>, dim3(grid), dim3(256), 0, s, in_dev, out_dev, n_elems, w, mul); break;
        case TPAMD_F32: hipLaunchKernelGGL(scale_kernel<TPAMD_F32>, dim3(grid), dim3(256), 0, s, in_dev, out_dev, n_elems, w, mul); break;
        default: set_error("tpamd_scale: unknown dtype %d", dtype); return TPAMD_ERR_INVALID;
    }
    TPAMD_HIP(hipGetLastError());
    return TPAMD_OK;
}
