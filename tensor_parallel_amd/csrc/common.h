// Shared host/device helpers for the gfx950 kernels behind include/tpamd.h.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>

#include <mutex>

#include "../../include/tpamd.h"

namespace tpamd {

// ---- error plumbing -----------------------------------------------------------------------------
void set_error(const char *fmt, ...);

#define TPAMD_REQUIRE(cond, ...)                 \
    do {                                         \
        if (!(cond)) {                           \
            ::tpamd::set_error(__VA_ARGS__);     \
            return TPAMD_ERR_INVALID;            \
        }                                        \
    } while (0)

#define TPAMD_HIP(call)                                                                          \
    do {                                                                                         \
        hipError_t e_ = (call);                                                                  \
        if (e_ != hipSuccess) {                                                                  \
            ::tpamd::set_error("%s failed: %s (%s:%d)", #call, hipGetErrorString(e_), __FILE__,  \
                               __LINE__);                                                        \
            return TPAMD_ERR_HIP;                                                                \
        }                                                                                        \
    } while (0)

// ---- tuning knobs: environment variables, read once when the library is loaded (tpamd_tuning_reload() re-reads them).
// TUNE_UNSET = the variable is not set and the library's own choice applies.
constexpr int TUNE_UNSET = -2147483647 - 1;
struct Tuning {
    int gemm_w4;             // TPAMD_GEMM_W4: 0 = the 8-wavefront 256 x 256 kernel instead of the 4-wavefront one
    int gemm_splitk;         // TPAMD_GEMM_SPLITK: K splits of the 128 x 128 tiling
    int gemm_splitk256;      // TPAMD_GEMM_SPLITK256: K splits of the 256 x 256 tiling
    int gemm_tile;           // TPAMD_GEMM_TILE: 256 or 128
    int gemm_stages;         // TPAMD_GEMM_STAGES: 4 / 2 = the K-split 128 x 128 kernel with four / two LDS stages (unset: four when there is at most one block per CU)
    int gemm_part_x;         // TPAMD_GEMM_PART_X: 0 = the K-split 128 x 128 kernel loads whole x tiles also for M <= 64
    int skinny_cg;           // TPAMD_SKINNY_CG: column groups per block (1, 2, 4)
    int skinny_pair;         // TPAMD_SKINNY_PAIR: 8-column form of the gated pair
    int skinny_resident;     // TPAMD_SKINNY_RESIDENT: x-resident kernel on/off
    int w8_split;            // TPAMD_W8_SPLIT: int8 K-split kernel on/off
    int w8_cols;             // TPAMD_W8_COLS: int8 K-split kernel whose wavefronts own columns (x of the split in LDS): 0 = off, 1 = whenever the shape allows
    int skinny_max_m;        // TPAMD_SKINNY_MAX_M: most rows of a single 16-bit matrix that go to the weight-streaming kernels (16 to 64; unset: by shape)
    int skinny_xlds;         // TPAMD_SKINNY_XLDS: 0 = gated pair at 4-16 rows through the older kernels
    int gemv_rows;           // TPAMD_GEMV_ROWS: wavefronts per block of the unrolled M <= 3 kernel (4, 8, 16); 0 = the general kernel, -1 = the MFMA kernels
    int attn_splits;         // TPAMD_ATTN_SPLITS: key-range splits of the attention kernel
    int attn_ring;           // TPAMD_ATTN_RING: 1 / 0 = the few-row attention kernel with / without several K / V tiles in flight
    int copy_tile_units;     // TPAMD_COPY_TILE_UNITS: 16-byte units per copy tile
    int copy_blocks_per_cu;  // TPAMD_COPY_BLOCKS_PER_CU
    int copy_sort;           // TPAMD_COPY_SORT: 0 = tiles stay in the order of the jobs instead of the order of their source addresses
    int copy_nt;             // TPAMD_COPY_NT: bit 0 non-temporal loads, bit 1 non-temporal stores of the slicing kernel
};
const Tuning &tuning();

// Compute units of device `dev` (asked from the runtime once per device).
int device_cus(int dev, int *cus_out);

// fp32 scratch memory of the K-split kernels (split-K partial tiles, split-key attention partials): defined in
// runtime.hip. Callers hold splitk_mutex(dev), the lock of their device, from the lookup until their launches that use
// the buffer are enqueued (two host threads that share a stream must not interleave a K-split launch and its finishing
// pass), and pass reserve = 4 * CUs * 64 KiB, so that a stream's buffer is allocated with the size every shape can live with.
std::mutex &splitk_mutex(int dev);
int splitk_scratch(int dev, hipStream_t stream, size_t need, size_t reserve, void **out);
// While one of these lives on a host thread, splitk_scratch() on that thread hands out the library's fixed array and
// allocates nothing.
// 64 MiB: what a stream's buffer holds on a 256-CU part (4 * CUs * 64 KiB), so every K split the cost models pick there fits.
constexpr size_t TPAMD_NOALLOC_SCRATCH_BYTES = static_cast<size_t>(64) << 20;
bool static_scratch_active();
int static_scratch(int dev, size_t need, void **out);
struct StaticScratchScope {
    StaticScratchScope();
    ~StaticScratchScope();
    StaticScratchScope(const StaticScratchScope &) = delete;
    StaticScratchScope &operator=(const StaticScratchScope &) = delete;
};

// Body of tpamd_linear / tpamd_linear_add / tpamd_linear_noalloc (api.hip).
int linear_entry(const char *who, const void *x_dev, const void *w_dev, const void *bias_dev, const void *addend_dev,
                 int64_t ldadd, void *y_dev, int64_t M, int64_t N, int64_t K, int64_t ldx, int64_t ldw, int64_t ldy, int dtype,
                 int act, void *stream);

static inline bool aligned(const void *p, uintptr_t a) { return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0; }

// ---- streaming (non-temporal) 16-byte accesses: data that is touched once should not displace cache lines
typedef uint32_t v4u __attribute__((ext_vector_type(4)));
typedef uint32_t v2u __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint4 nt_load_u4(const void *p) {
    const v4u v = __builtin_nontemporal_load(static_cast<const v4u *>(p));
    return make_uint4(v.x, v.y, v.z, v.w);
}
__device__ __forceinline__ void nt_store_u4(void *p, uint4 u) {
    const v4u v = {u.x, u.y, u.z, u.w};
    __builtin_nontemporal_store(v, static_cast<v4u *>(p));
}

// ---- device-side scalar conversions ---------------------------------------------------------------
// bf16 is handled as raw uint16_t bits so that rounding is spelled out (round to nearest even, NaN
// kept quiet), identical to what torch does when it stores an fp32 result into a bf16 tensor.
__device__ __forceinline__ float bf16_to_f32(uint16_t h) { return __uint_as_float(static_cast<uint32_t>(h) << 16); }

__device__ __forceinline__ uint16_t f32_to_bf16(float f) {
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return static_cast<uint16_t>((u >> 16) | 0x0040u);  // NaN
    u += 0x7fffu + ((u >> 16) & 1u);
    return static_cast<uint16_t>(u >> 16);
}

__device__ __forceinline__ float f16_to_f32(uint16_t h) {
    _Float16 v = __builtin_bit_cast(_Float16, h);
    return static_cast<float>(v);
}

__device__ __forceinline__ uint16_t f32_to_f16(float f) {
    _Float16 v = static_cast<_Float16>(f);  // v_cvt_f16_f32: round to nearest even
    return __builtin_bit_cast(uint16_t, v);
}

template <int DT>
__device__ __forceinline__ float half_to_f32(uint16_t h) {
    if constexpr (DT == TPAMD_BF16) return bf16_to_f32(h);
    else return f16_to_f32(h);
}
template <int DT>
__device__ __forceinline__ uint16_t f32_to_half(float f) {
    if constexpr (DT == TPAMD_BF16) return f32_to_bf16(f);
    else return f32_to_f16(f);
}

// Two fp32 values rounded to nearest even and packed (a in the low half): v_cvt_pk_bf16_f32 for bf16.
typedef float tpamd_f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 tpamd_bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 tpamd_f16x2 __attribute__((ext_vector_type(2)));
template <int DT>
__device__ __forceinline__ uint32_t pack2_half(float a, float b) {
    const tpamd_f32x2 v = {a, b};
    if constexpr (DT == TPAMD_BF16) return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, tpamd_bf16x2));
    else return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, tpamd_f16x2));
}
template <int DT>
__device__ __forceinline__ float lo_half_to_f32(uint32_t p) {
    if constexpr (DT == TPAMD_BF16) return __uint_as_float(p << 16);
    else return half_to_f32<DT>(static_cast<uint16_t>(p & 0xffffu));
}
template <int DT>
__device__ __forceinline__ float hi_half_to_f32(uint32_t p) {
    if constexpr (DT == TPAMD_BF16) return __uint_as_float(p & 0xffff0000u);
    else return half_to_f32<DT>(static_cast<uint16_t>(p >> 16));
}

// out = round(out + addend) per 16-bit element: the sum of two same-dtype tensors as torch computes it (fp32 add of the
// widened values, one rounding), which is one step of the reference's `sum([...])` over rank partials
// (src/tensor_parallel/cross_device_ops.py:49).
template <int DT>
__device__ __forceinline__ uint32_t add_packed2(uint32_t a, uint32_t b) {
    return pack2_half<DT>(lo_half_to_f32<DT>(a) + lo_half_to_f32<DT>(b), hi_half_to_f32<DT>(a) + hi_half_to_f32<DT>(b));
}

// out = round(round(a * c) + round(b * s)) per 16-bit element: the three torch ops of
// `(x * cos) + (rotate_half(x) * sin)` on tensors of the 16-bit dtype, each an fp32 operation rounded once.
template <int DT>
__device__ __forceinline__ uint32_t rot2(uint32_t a, uint32_t c, uint32_t b, uint32_t s, float sign) {
    const float a0 = lo_half_to_f32<DT>(a), a1 = hi_half_to_f32<DT>(a);
    const float b0 = sign * lo_half_to_f32<DT>(b), b1 = sign * hi_half_to_f32<DT>(b);
    const uint32_t ac = pack2_half<DT>(a0 * lo_half_to_f32<DT>(c), a1 * hi_half_to_f32<DT>(c));
    const uint32_t bs = pack2_half<DT>(b0 * lo_half_to_f32<DT>(s), b1 * hi_half_to_f32<DT>(s));
    return add_packed2<DT>(ac, bs);
}

template <int DT>
__device__ __forceinline__ uint4 rot8(uint4 a, uint4 c, uint4 b, uint4 s, float sign) {
    return make_uint4(rot2<DT>(a.x, c.x, b.x, s.x, sign), rot2<DT>(a.y, c.y, b.y, s.y, sign), rot2<DT>(a.z, c.z, b.z, s.z, sign),
                      rot2<DT>(a.w, c.w, b.w, s.w, sign));
}

// Four int8 (one dword) -> four values of the activation dtype, packed as lo = elements 0,1 and
// hi = elements 2,3. Exact: |q| <= 128 fits both f16 and bf16 significands.
template <int DT>
__device__ __forceinline__ void cvt_i8x4(uint32_t q, uint32_t &lo, uint32_t &hi) {
    const uint32_t u = q ^ 0x80808080u;  // biased to 0..255
    if constexpr (DT == TPAMD_F16) {
        // f16 0x6400 | u == 1024 + u; subtracting 1152 gives q
        const uint32_t p0 = __builtin_amdgcn_perm(0x64646464u, u, 0x04010400u);
        const uint32_t p1 = __builtin_amdgcn_perm(0x64646464u, u, 0x04030402u);
        const tpamd_f16x2 bias = {static_cast<_Float16>(1152.0f), static_cast<_Float16>(1152.0f)};
        lo = __builtin_bit_cast(uint32_t, __builtin_bit_cast(tpamd_f16x2, p0) - bias);
        hi = __builtin_bit_cast(uint32_t, __builtin_bit_cast(tpamd_f16x2, p1) - bias);
    } else {
        // f32 0x4B000000 | u == 2^23 + u; subtracting 2^23 + 128 gives q; its high half is the bf16
        const float f0 = __uint_as_float(__builtin_amdgcn_perm(0x4B000000u, u, 0x07050400u)) - 8388736.0f;
        const float f1 = __uint_as_float(__builtin_amdgcn_perm(0x4B000000u, u, 0x07050401u)) - 8388736.0f;
        const float f2 = __uint_as_float(__builtin_amdgcn_perm(0x4B000000u, u, 0x07050402u)) - 8388736.0f;
        const float f3 = __uint_as_float(__builtin_amdgcn_perm(0x4B000000u, u, 0x07050403u)) - 8388736.0f;
        lo = __builtin_amdgcn_perm(__float_as_uint(f1), __float_as_uint(f0), 0x07060302u);
        hi = __builtin_amdgcn_perm(__float_as_uint(f3), __float_as_uint(f2), 0x07060302u);
    }
}

__device__ __forceinline__ float gelu_erf(float x) { return 0.5f * x * (1.0f + erff(x * 0.70710678118654752440f)); }
// v_exp_f32 and v_rcp_f32 (1 ulp each) instead of the 10-instruction IEEE division sequence. Every kernel uses this
// one definition, so a row's result does not depend on which kernel the batch size selects.
__device__ __forceinline__ float silu_f32(float x) { return x * __builtin_amdgcn_rcpf(1.0f + __expf(-x)); }

}  // namespace tpamd
