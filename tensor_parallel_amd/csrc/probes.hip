// Measurement probes, built into their own library (libtpamd_probes.so) and used only by `bench.py --ceilings`: what one
// MI355X sustains on the two resources the hot path is bound by, measured with nothing else in the way.
//   tpamd_probe_mfma    a loop of nothing but bf16 MFMAs (no loads, no LDS), operands constant or random
//   tpamd_probe_stream  a read-only / write-only / copy stream over a buffer, 16 bytes per lane, plain or non-temporal, in small
//                       steps of many 256-thread blocks or in 128 KiB bursts of one 1024-thread block per CU
// The product library does not link this file.
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef uint32_t v4u __attribute__((ext_vector_type(4)));

// One wavefront per SIMD (4 per block, one block per CU), 16 or 8 independent accumulator tiles in AGPRs that are
// accumulated in place: the issue pattern of the GEMM kernels' inner loop without its loads and LDS reads. The MFMAs are
// written as asm so that nothing but them (and the loop counter) is in the loop.
// SHAPE 16: v_mfma_f32_16x16x32_bf16 (16 tiles), 32: v_mfma_f32_32x32x16_bf16 (8 tiles).
template <int SHAPE>
__global__ __launch_bounds__(256) void mfma_loop_kernel(const uint4 *operands, float *sink, int iters) {
    const int tid = blockIdx.x * 256 + threadIdx.x;
    v4u a[4], b[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const uint4 av = operands[tid * 8 + i], bv = operands[tid * 8 + 4 + i];
        a[i] = v4u{av.x, av.y, av.z, av.w};
        b[i] = v4u{bv.x, bv.y, bv.z, bv.w};
    }
    float s = 0.f;
    if constexpr (SHAPE == 32) {
        f32x16 acc[8];
#pragma unroll
        for (int i = 0; i < 8; ++i)
#pragma unroll
            for (int j = 0; j < 16; ++j) acc[i][j] = 0.f;
        for (int it = 0; it < iters; ++it) {
#pragma unroll
            for (int i = 0; i < 8; ++i)
                asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+a"(acc[i]) : "v"(a[i & 3]), "v"(b[(i >> 1) & 3]));
        }
#pragma unroll
        for (int i = 0; i < 8; ++i) s += acc[i][0];
    } else {
        f32x4 acc[16];
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[i] = f32x4{0.f, 0.f, 0.f, 0.f};
        for (int it = 0; it < iters; ++it) {
#pragma unroll
            for (int i = 0; i < 16; ++i)
                asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(acc[i]) : "v"(a[i & 3]), "v"(b[(i >> 2) & 3]));
        }
#pragma unroll
        for (int i = 0; i < 16; ++i) s += acc[i][0];
    }
    if (s == 123.456f) sink[threadIdx.x] = s;  // keeps the loop alive; never true for these operands
}

// MODE 0: read src, 1: write dst, 2: copy src -> dst. A persistent grid; block b handles pieces b, b + grid, ... of
// PIECE bytes (256 threads x 16 bytes x PIECE / 4096 accesses in flight per thread). NT: non-temporal accesses.
template <int MODE, bool NT, int PIECE>
__global__ __launch_bounds__(256) void stream_kernel(const char *src, char *dst, uint64_t pieces, float *sink) {
    constexpr int U = PIECE / 4096;
    uint32_t keep = 0;
    for (uint64_t p = blockIdx.x; p < pieces; p += gridDim.x) {
        const uint64_t off = p * PIECE + threadIdx.x * 16;
        v4u v[U];
#pragma unroll
        for (int i = 0; i < U; ++i) {
            if constexpr (MODE == 1) v[i] = v4u{static_cast<uint32_t>(p), 1u, 2u, 3u};
            else if constexpr (NT) v[i] = __builtin_nontemporal_load(reinterpret_cast<const v4u *>(src + off + i * 4096));
            else v[i] = *reinterpret_cast<const v4u *>(src + off + i * 4096);
        }
#pragma unroll
        for (int i = 0; i < U; ++i) {
            if constexpr (MODE == 0) keep ^= v[i].x ^ v[i].y ^ v[i].z ^ v[i].w;
            else if constexpr (NT) __builtin_nontemporal_store(v[i], reinterpret_cast<v4u *>(dst + off + i * 4096));
            else *reinterpret_cast<v4u *>(dst + off + i * 4096) = v[i];
        }
    }
    if (MODE == 0 && keep == 0x12345679u) sink[threadIdx.x] = 1.f;
}

// The same stream in bursts: one 1024-thread block moves 128 KiB at a time, all of its loads first (8 per lane), then, once the
// last one has arrived, all of its stores. MODE and NT as above.
template <int MODE, bool NT>
__global__ __launch_bounds__(1024) void burst_kernel(const char *src, char *dst, uint64_t pieces, float *sink) {
    constexpr int U = 8;
    uint32_t keep = 0;
    for (uint64_t p = blockIdx.x; p < pieces; p += gridDim.x) {
        const uint64_t off = p * 131072 + threadIdx.x * 16;
        v4u v[U];
#pragma unroll
        for (int i = 0; i < U; ++i) {
            if constexpr (MODE == 1) v[i] = v4u{static_cast<uint32_t>(p), 1u, 2u, 3u};
            else if constexpr (NT) v[i] = __builtin_nontemporal_load(reinterpret_cast<const v4u *>(src + off + i * 16384));
            else v[i] = *reinterpret_cast<const v4u *>(src + off + i * 16384);
        }
        if constexpr (MODE == 2) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#pragma unroll
        for (int i = 0; i < U; ++i) {
            if constexpr (MODE == 0) keep ^= v[i].x ^ v[i].y ^ v[i].z ^ v[i].w;
            else if constexpr (NT) __builtin_nontemporal_store(v[i], reinterpret_cast<v4u *>(dst + off + i * 16384));
            else *reinterpret_cast<v4u *>(dst + off + i * 16384) = v[i];
        }
    }
    if (MODE == 0 && keep == 0x12345679u) sink[threadIdx.x] = 1.f;
}

template <int MODE>
void launch_stream(bool nt, int piece, int blocks, hipStream_t s, const char *src, char *dst, uint64_t bytes, float *sink) {
    const uint64_t pieces = bytes / piece;
    if (piece == 131072) {
        if (nt) hipLaunchKernelGGL((burst_kernel<MODE, true>), dim3(blocks), dim3(1024), 0, s, src, dst, pieces, sink);
        else hipLaunchKernelGGL((burst_kernel<MODE, false>), dim3(blocks), dim3(1024), 0, s, src, dst, pieces, sink);
        return;
    }
#define TPAMD_PROBE_CASE(NTV, P) \
    if (nt == NTV && piece == P) hipLaunchKernelGGL((stream_kernel<MODE, NTV, P>), dim3(blocks), dim3(256), 0, s, src, dst, pieces, sink)
    TPAMD_PROBE_CASE(true, 16384); TPAMD_PROBE_CASE(false, 16384);
    TPAMD_PROBE_CASE(true, 32768); TPAMD_PROBE_CASE(false, 32768);
    TPAMD_PROBE_CASE(true, 4096); TPAMD_PROBE_CASE(false, 4096);
#undef TPAMD_PROBE_CASE
}

}  // namespace

// operands_dev: blocks * 256 * 8 * 16 bytes of bf16 values; sink_dev: 256 floats. shape: 16 or 32.
extern "C" int tpamd_probe_mfma(int shape, const void *operands_dev, void *sink_dev, int blocks, int iters, void *stream) {
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (shape == 32) hipLaunchKernelGGL((mfma_loop_kernel<32>), dim3(blocks), dim3(256), 0, s, static_cast<const uint4 *>(operands_dev), static_cast<float *>(sink_dev), iters);
    else if (shape == 16) hipLaunchKernelGGL((mfma_loop_kernel<16>), dim3(blocks), dim3(256), 0, s, static_cast<const uint4 *>(operands_dev), static_cast<float *>(sink_dev), iters);
    else return -1;
    return hipGetLastError() == hipSuccess ? 0 : -3;
}

// Floating-point operations of one tpamd_probe_mfma launch (4 wavefronts per block; 2 * 16 * 16 * 32 = 2 * 32 * 32 * 16 / 2).
extern "C" double tpamd_probe_mfma_flops(int shape, int blocks, int iters) {
    const double per_wave_iter = shape == 32 ? 8 * 32768.0 : 16 * 16384.0;
    return per_wave_iter * 4.0 * blocks * iters;
}

// mode 0 read, 1 write, 2 copy; nt != 0: non-temporal accesses; piece: 4096, 16384 or 32768 bytes per step of a 256-thread
// block, or 131072: bursts of a 1024-thread block; bytes must be a multiple of 32768 (of 131072 for bursts).
extern "C" int tpamd_probe_stream(int mode, int nt, int piece, const void *src_dev, void *dst_dev, uint64_t bytes, int blocks,
                                  void *sink_dev, void *stream) {
    if (bytes % 32768 != 0 || blocks <= 0 || (piece != 4096 && piece != 16384 && piece != 32768 && piece != 131072)) return -1;
    if (piece == 131072 && bytes % 131072 != 0) return -1;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const char *src = static_cast<const char *>(src_dev);
    char *dst = static_cast<char *>(dst_dev);
    float *sink = static_cast<float *>(sink_dev);
    if (mode == 0) launch_stream<0>(nt != 0, piece, blocks, s, src, dst, bytes, sink);
    else if (mode == 1) launch_stream<1>(nt != 0, piece, blocks, s, src, dst, bytes, sink);
    else if (mode == 2) launch_stream<2>(nt != 0, piece, blocks, s, src, dst, bytes, sink);
    else return -1;
    return hipGetLastError() == hipSuccess ? 0 : -3;
}
