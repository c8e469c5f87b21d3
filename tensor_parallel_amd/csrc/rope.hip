// Rotary position embedding of the new query and key rows and their hand-over to the rank-local key/value cache,
// in one launch: what sits between the fused QKV projection of a rank shard and its attention core.
//
// Every (batch, position, head) row of D contiguous elements is handled by D / 16 lanes. A lane owns 8 elements of the
// first half of the row and the 8 elements of the second half that rotate with them, so one 16-byte load per half
// gives it both members of its 8 pairs, and both 16-byte stores are whole. A block takes 256 lanes of one (batch,
// position): its q rows first, then k, then v (v rows are copied); the launch is bound by its latency at decode and by HBM at prefill, where it moves
// every byte once.
#include "common.h"

namespace tpamd {
namespace {

struct RopeParams {
    const char *q, *k, *v, *cos, *sin;
    char *q_out, *k_cache, *v_cache;
    int B, S, Hq, Hkv, D;
    int64_t pos0;
    // element strides; D is contiguous everywhere
    int64_t q_b, q_s, q_h, q_g, k_b, k_s, k_h, v_b, v_s, v_h;  // q_g: between the first query heads of consecutive key/value heads
    int per;                       // query heads per key/value head
    int64_t cs_b, cs_s;            // cos / sin: [B or 1, S, D]
    int64_t qo_b, qo_h, qo_s;      // q_out [B, Hq, S, D]
    int64_t kc_b, kc_h, kc_s;      // key cache [B, Hkv, S_max, D]
    int64_t vc_b, vc_h, vc_s;
    int lanes_per_pos;             // (Hq + 2 Hkv) * (D / 16): lanes of one (batch, position)
};

template <int DT>
__global__ __launch_bounds__(256) void rope_append_kernel(RopeParams p) {
    // grid: x = (batch, position), y = blocks of 256 lanes over that position's heads; 32-bit index arithmetic throughout
    const int t = blockIdx.y * 256 + threadIdx.x;
    if (t >= p.lanes_per_pos) return;
    const int shift = p.D == 64 ? 2 : 3;  // D / 16 lanes per head row
    const int chunk = t & ((1 << shift) - 1);
    const int head = t >> shift;
    const int b = static_cast<int>(blockIdx.x) / p.S;
    const int s = static_cast<int>(blockIdx.x) - b * p.S;
    const int half_bytes = p.D;  // D / 2 elements of 2 bytes
    const int at = chunk * 16;   // byte offset of the lane's 8 elements inside a half

    if (head >= p.Hq + p.Hkv) {  // value row: copied into the cache
        const int h = head - p.Hq - p.Hkv;
        const char *src = p.v + (static_cast<int64_t>(b) * p.v_b + s * p.v_s + h * p.v_h) * 2 + at;
        char *dst = p.v_cache + (static_cast<int64_t>(b) * p.vc_b + h * p.vc_h + (p.pos0 + s) * p.vc_s) * 2 + at;
        const uint4 lo = *reinterpret_cast<const uint4 *>(src), hi = *reinterpret_cast<const uint4 *>(src + half_bytes);
        *reinterpret_cast<uint4 *>(dst) = lo;
        *reinterpret_cast<uint4 *>(dst + half_bytes) = hi;
        return;
    }
    const bool is_q = head < p.Hq;
    const int h = is_q ? head : head - p.Hq;
    const char *src = is_q ? p.q + (b * p.q_b + s * p.q_s + (h / p.per) * p.q_g + (h % p.per) * p.q_h) * 2 : p.k + (b * p.k_b + s * p.k_s + h * p.k_h) * 2;
    char *dst = is_q ? p.q_out + (b * p.qo_b + h * p.qo_h + s * p.qo_s) * 2
                     : p.k_cache + (b * p.kc_b + h * p.kc_h + (p.pos0 + s) * p.kc_s) * 2;
    const int64_t cs = (b * p.cs_b + s * p.cs_s) * 2 + at;
    const uint4 x1 = *reinterpret_cast<const uint4 *>(src + at), x2 = *reinterpret_cast<const uint4 *>(src + at + half_bytes);
    const uint4 c1 = *reinterpret_cast<const uint4 *>(p.cos + cs), c2 = *reinterpret_cast<const uint4 *>(p.cos + cs + half_bytes);
    const uint4 s1 = *reinterpret_cast<const uint4 *>(p.sin + cs), s2 = *reinterpret_cast<const uint4 *>(p.sin + cs + half_bytes);
    // rotate_half(x) = cat(-x2, x1): first half x1 * cos1 - x2 * sin1, second half x2 * cos2 + x1 * sin2
    *reinterpret_cast<uint4 *>(dst + at) = rot8<DT>(x1, c1, x2, s1, -1.0f);
    *reinterpret_cast<uint4 *>(dst + at + half_bytes) = rot8<DT>(x2, c2, x1, s2, 1.0f);
}

}  // namespace
}  // namespace tpamd

using namespace tpamd;

extern "C" int tpamd_rope_append(const void *q_dev, const void *k_dev, const void *v_dev, const void *cos_dev, const void *sin_dev,
                                 void *q_out_dev, void *k_cache_dev, void *v_cache_dev, int64_t B, int64_t S, int64_t Hq,
                                 int64_t Hkv, int64_t D, int64_t pos0, int64_t cache_len, const int64_t *strides, int dtype,
                                 void *stream) {
    const char *who = "tpamd_rope_append";
    TPAMD_REQUIRE(dtype == TPAMD_BF16 || dtype == TPAMD_F16, "%s: dtype must be BF16 or F16", who);
    TPAMD_REQUIRE(B >= 0 && S >= 0 && Hq > 0 && Hkv > 0, "%s: bad dimension", who);
    TPAMD_REQUIRE(Hq % Hkv == 0, "%s: %lld query heads are not a multiple of %lld key/value heads", who, (long long)Hq, (long long)Hkv);
    TPAMD_REQUIRE(pos0 >= 0 && pos0 + S <= cache_len, "%s: positions [%lld, %lld) do not fit a cache of %lld positions", who,
                  (long long)pos0, (long long)(pos0 + S), (long long)cache_len);
    TPAMD_REQUIRE(strides != nullptr, "%s: strides is NULL", who);
    if (B == 0 || S == 0) return TPAMD_OK;
    TPAMD_REQUIRE(q_dev && k_dev && v_dev && cos_dev && sin_dev && q_out_dev && k_cache_dev && v_cache_dev, "%s: null pointer", who);
    TPAMD_REQUIRE(B < (1ll << 24) && S < (1ll << 24) && Hq + 2 * Hkv < (1ll << 16), "%s: dimension too large", who);
    bool ok = (D == 64 || D == 128) && aligned(q_dev, 16) && aligned(k_dev, 16) && aligned(v_dev, 16) && aligned(cos_dev, 16) &&
              aligned(sin_dev, 16) && aligned(q_out_dev, 16) && aligned(k_cache_dev, 16) && aligned(v_cache_dev, 16);
    for (int i = 0; i < 21; ++i) ok = ok && strides[i] % 8 == 0;  // every row starts on a 16-byte boundary
    if (!ok) {
        set_error("%s: head_dim must be 64 or 128 and every row 16-byte aligned", who);
        return TPAMD_ERR_UNSUPPORTED;
    }
    RopeParams p;
    p.q = static_cast<const char *>(q_dev); p.k = static_cast<const char *>(k_dev); p.v = static_cast<const char *>(v_dev);
    p.cos = static_cast<const char *>(cos_dev); p.sin = static_cast<const char *>(sin_dev);
    p.q_out = static_cast<char *>(q_out_dev); p.k_cache = static_cast<char *>(k_cache_dev); p.v_cache = static_cast<char *>(v_cache_dev);
    p.B = static_cast<int>(B); p.S = static_cast<int>(S); p.Hq = static_cast<int>(Hq); p.Hkv = static_cast<int>(Hkv); p.D = static_cast<int>(D);
    p.pos0 = pos0;
    p.q_b = strides[0]; p.q_s = strides[1]; p.q_h = strides[2];
    p.k_b = strides[3]; p.k_s = strides[4]; p.k_h = strides[5];
    p.v_b = strides[6]; p.v_s = strides[7]; p.v_h = strides[8];
    p.cs_b = strides[9]; p.cs_s = strides[10];
    p.qo_b = strides[11]; p.qo_h = strides[12]; p.qo_s = strides[13];
    p.kc_b = strides[14]; p.kc_h = strides[15]; p.kc_s = strides[16];
    p.vc_b = strides[17]; p.vc_h = strides[18]; p.vc_s = strides[19];
    p.q_g = strides[20];
    p.per = static_cast<int>(Hq / Hkv);
    p.lanes_per_pos = static_cast<int>((Hq + 2 * Hkv) * (D / 16));
    TPAMD_REQUIRE(B * S < (1ll << 31), "%s: too many positions for one launch", who);
    const dim3 grid(static_cast<unsigned>(B * S), static_cast<unsigned>((p.lanes_per_pos + 255) / 256));
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (dtype == TPAMD_BF16) hipLaunchKernelGGL(rope_append_kernel<TPAMD_BF16>, grid, dim3(256), 0, s, p);
    else hipLaunchKernelGGL(rope_append_kernel<TPAMD_F16>, grid, dim3(256), 0, s, p);
    TPAMD_HIP(hipGetLastError());
    return TPAMD_OK;
}
