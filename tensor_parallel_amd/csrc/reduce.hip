// Single-device partial-sum reduction: out = sum_r parts[r]. HBM-bound: (W + 1) * n * itemsize bytes.
#include "common.h"

namespace tpamd {
namespace {

constexpr int MAX_WORLD = 16;
constexpr int RED_THREADS = 256;

struct Parts {
    const void *p[MAX_WORLD];
};

template <int DT, int ACCUM>
__device__ __forceinline__ void add_half(float &acc, uint16_t next) {
    // acc holds the running sum. In STEPWISE mode it is re-rounded to the tensor dtype after every add.
    acc += half_to_f32<DT>(next);
    if constexpr (ACCUM == TPAMD_ACCUM_STEPWISE) acc = half_to_f32<DT>(f32_to_half<DT>(acc));
}

// 16 bytes per lane per partial: 8 half elements or 4 floats.
template <int DT, int ACCUM>
__global__ __launch_bounds__(RED_THREADS) void reduce_kernel(Parts parts, int world, void *out,
                                                             uint64_t n_vec, uint64_t n_elems) {
    constexpr int EPV = (DT == TPAMD_F32) ? 4 : 8;
    const uint64_t stride = static_cast<uint64_t>(gridDim.x) * RED_THREADS;
    for (uint64_t v = static_cast<uint64_t>(blockIdx.x) * RED_THREADS + threadIdx.x; v < n_vec; v += stride) {
        float acc[EPV];
        {
            uint4 raw = nt_load_u4(static_cast<const uint4 *>(parts.p[0]) + v);
            if constexpr (DT == TPAMD_F32) {
                acc[0] = __uint_as_float(raw.x); acc[1] = __uint_as_float(raw.y);
                acc[2] = __uint_as_float(raw.z); acc[3] = __uint_as_float(raw.w);
            } else {
                const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    acc[2 * i] = half_to_f32<DT>(static_cast<uint16_t>(w[i] & 0xffffu));
                    acc[2 * i + 1] = half_to_f32<DT>(static_cast<uint16_t>(w[i] >> 16));
                }
            }
        }
        for (int r = 1; r < world; ++r) {
            uint4 raw = nt_load_u4(static_cast<const uint4 *>(parts.p[r]) + v);
            if constexpr (DT == TPAMD_F32) {
                acc[0] += __uint_as_float(raw.x); acc[1] += __uint_as_float(raw.y);
                acc[2] += __uint_as_float(raw.z); acc[3] += __uint_as_float(raw.w);
            } else {
                const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    add_half<DT, ACCUM>(acc[2 * i], static_cast<uint16_t>(w[i] & 0xffffu));
                    add_half<DT, ACCUM>(acc[2 * i + 1], static_cast<uint16_t>(w[i] >> 16));
                }
            }
        }
        uint4 o;
        if constexpr (DT == TPAMD_F32) {
            o.x = __float_as_uint(acc[0]); o.y = __float_as_uint(acc[1]);
            o.z = __float_as_uint(acc[2]); o.w = __float_as_uint(acc[3]);
        } else {
            uint32_t w[4];
#pragma unroll
            for (int i = 0; i < 4; ++i)
                w[i] = static_cast<uint32_t>(f32_to_half<DT>(acc[2 * i])) |
                       (static_cast<uint32_t>(f32_to_half<DT>(acc[2 * i + 1])) << 16);
            o = make_uint4(w[0], w[1], w[2], w[3]);
        }
        nt_store_u4(static_cast<uint4 *>(out) + v, o);
    }
    // scalar tail (n_elems not a multiple of the vector width): one thread per leftover element
    const uint64_t done = n_vec * EPV;
    const uint64_t t = static_cast<uint64_t>(blockIdx.x) * RED_THREADS + threadIdx.x;
    if (t < n_elems - done) {
        const uint64_t i = done + t;
        if constexpr (DT == TPAMD_F32) {
            float a = static_cast<const float *>(parts.p[0])[i];
            for (int r = 1; r < world; ++r) a += static_cast<const float *>(parts.p[r])[i];
            static_cast<float *>(out)[i] = a;
        } else {
            float a = half_to_f32<DT>(static_cast<const uint16_t *>(parts.p[0])[i]);
            for (int r = 1; r < world; ++r) add_half<DT, ACCUM>(a, static_cast<const uint16_t *>(parts.p[r])[i]);
            static_cast<uint16_t *>(out)[i] = f32_to_half<DT>(a);
        }
    }
}

template <int DT, int ACCUM>
void launch(const Parts &parts, int world, void *out, uint64_t n, hipStream_t s, int cus) {
    constexpr int EPV = (DT == TPAMD_F32) ? 4 : 8;
    const uint64_t n_vec = n / EPV;
    uint64_t want = (n_vec + RED_THREADS - 1) / RED_THREADS;
    if (want == 0) want = 1;
    const uint64_t cap = static_cast<uint64_t>(cus) * 8;
    const int grid = static_cast<int>(want < cap ? want : cap);
    hipLaunchKernelGGL((reduce_kernel<DT, ACCUM>), dim3(grid), dim3(RED_THREADS), 0, s, parts, world, out, n_vec, n);
}

}  // namespace
}  // namespace tpamd

using namespace tpamd;

extern "C" int tpamd_reduce_partials(const void *const *parts_dev, int world_size, void *out_dev, uint64_t n_elems,
                                     int dtype, int accum, void *stream) {
    TPAMD_REQUIRE(world_size >= 1 && world_size <= MAX_WORLD, "tpamd_reduce_partials: world_size %d not in [1,%d]",
                  world_size, MAX_WORLD);
    TPAMD_REQUIRE(accum == TPAMD_ACCUM_STEPWISE || accum == TPAMD_ACCUM_F32, "tpamd_reduce_partials: accum %d", accum);
    TPAMD_REQUIRE(dtype == TPAMD_BF16 || dtype == TPAMD_F16 || dtype == TPAMD_F32, "tpamd_reduce_partials: dtype %d",
                  dtype);
    if (n_elems == 0) return TPAMD_OK;
    TPAMD_REQUIRE(parts_dev && out_dev, "tpamd_reduce_partials: null pointer");
    Parts parts{};
    for (int r = 0; r < world_size; ++r) {
        TPAMD_REQUIRE(parts_dev[r] != nullptr, "tpamd_reduce_partials: partial %d is NULL", r);
        TPAMD_REQUIRE(aligned(parts_dev[r], 16), "tpamd_reduce_partials: partial %d not 16-byte aligned", r);
        parts.p[r] = parts_dev[r];
    }
    TPAMD_REQUIRE(aligned(out_dev, 16), "tpamd_reduce_partials: out not 16-byte aligned");
    int dev = 0, cus = 256;
    TPAMD_HIP(hipGetDevice(&dev));
    if (int rc_cus = device_cus(dev, &cus); rc_cus != TPAMD_OK) return rc_cus;
    hipStream_t s = static_cast<hipStream_t>(stream);
    // the tail handler needs at least (EPV - 1) threads in the grid: always true (grid >= 1 block of 256)
    if (dtype == TPAMD_F32) launch<TPAMD_F32, TPAMD_ACCUM_F32>(parts, world_size, out_dev, n_elems, s, cus);
    else if (dtype == TPAMD_BF16 && accum == TPAMD_ACCUM_STEPWISE) launch<TPAMD_BF16, TPAMD_ACCUM_STEPWISE>(parts, world_size, out_dev, n_elems, s, cus);
    else if (dtype == TPAMD_BF16) launch<TPAMD_BF16, TPAMD_ACCUM_F32>(parts, world_size, out_dev, n_elems, s, cus);
    else if (accum == TPAMD_ACCUM_STEPWISE) launch<TPAMD_F16, TPAMD_ACCUM_STEPWISE>(parts, world_size, out_dev, n_elems, s, cus);
    else launch<TPAMD_F16, TPAMD_ACCUM_F32>(parts, world_size, out_dev, n_elems, s, cus);
    TPAMD_HIP(hipGetLastError());
    return TPAMD_OK;
}
