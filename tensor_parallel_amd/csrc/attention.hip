// Rank-local attention core: softmax(scale * Q K^T + causal mask) V for the heads one rank owns, grouped-query
// layout (Hq = G * Hkv query heads share Hkv key/value heads), bf16/f16, head_dim 64 or 128.
//
// One kernel serves prefill and decode. The query rows that share a key/value head are put on one axis,
// row = g * Sq + sq (g = query head inside the group): at decode (Sq = 1, G = 16) the 16 heads of a group fill
// one MFMA tile and K / V of that head are read once for all of them; at prefill a tile is 64 consecutive
// positions of one head. A block (4 wavefronts, 16 rows each) walks the keys in tiles of 64:
//   S^T = K Q^T   v_mfma_f32_16x16x32 with K rows as the first operand: a lane then holds, for ONE query row,
//                 4 keys per 16-key tile, so the row maximum / sum need two cross-lane steps only,
//   online softmax in exp2 domain (scale * log2 e folded in),
//   O^T += V^T P^T the lane's 8 probabilities of two key tiles are exactly the second operand of the next MFMA
//                 (the K index of an MFMA may be permuted freely as long as both operands agree), the first
//                 operand comes from the row-major V tile in LDS through the LDS transpose load.
// O^T leaves a lane with 4 consecutive head-dim elements of one query row: one 8-byte store into [B, Sq, Hq, D].
//
// Long key ranges with few rows (decode) are split over blockIdx.z; every split leaves (m, l, unnormalised O) in
// the stream's scratch buffer and attention_combine_kernel merges them. For one new position per sequence
// (tpamd_attention_decode_rope) the kernel also applies the rotary embedding to its Q fragments, and the merge
// (attention_combine_newkey_kernel) adds the new position's key and value and writes them into the cache.
#include "common.h"

#include <stdlib.h>

namespace tpamd {
namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;

template <int DT>
__device__ __forceinline__ f32x4 mfma16(uint4 a, uint4 b, f32x4 c) {
    if constexpr (DT == TPAMD_BF16)
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
    else
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
}

typedef __attribute__((ext_vector_type(4))) short i16x4;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;  // 16 bytes on their way from global memory to LDS

// A loop whose counter is a constant expression inside the body (f gets Const<0>, Const<1>, ...): arrays indexed with it
// are split into registers from the start, not only if a later pass unrolls the loop.
template <int I>
struct Const {
    static constexpr int value = I;
};
template <int N, int I = 0, class F>
__device__ __forceinline__ void static_for(F &&f) {
    if constexpr (I < N) {
        f(Const<I>{});
        static_for<N, I + 1>(f);
    }
}

// ds_read_b64_tr_b16: every lane gives the LDS address of four 16-bit elements; within each group of 16 lanes,
// lane i receives element i % 4 of lanes i / 4, 4 + i / 4, 8 + i / 4 and 12 + i / 4 (in that order).
__device__ __forceinline__ uint2 lds_transpose_b64(const char *lds_ptr) {
    auto *ptr = reinterpret_cast<__attribute__((address_space(3))) i16x4 *>(reinterpret_cast<uintptr_t>(lds_ptr));
    return __builtin_bit_cast(uint2, __builtin_amdgcn_ds_read_tr16_b64_v4i16(ptr));
}

struct AttnParams {
    const char *q, *k, *v;
    char *o;
    float *part;  // split partials: [split][B*Hkv][rows_pad][D + 4] fp32 (O, then m, l, 2 unused)
    int B, Hq, Hkv, Sq, Skv, G;
    int64_t q_sb, q_sh, q_ss, k_sb, k_sh, k_ss, v_sb, v_sh, v_ss, o_sb, o_ss, o_sh;  // elements; head_dim is contiguous
    float scale_log2;  // scale * log2(e)
    int causal;        // query position sq sees keys j <= sq + (Skv - Sq)
    int nsplit, keys_per_split, rows_pad;
    int64_t q_sg;  // elements between the first query heads of consecutive key/value heads (G * q_sh for a plain [B, Hq, Sq, D])
    // Decode with the rotary embedding folded in (Sq = 1; tpamd_attention_decode_rope): q, new_k, new_v are the raw rows of
    // the projection output, cos / sin [B or 1, D]; the kernel rotates its Q fragments, always leaves partials, and the merge
    // adds the new position's key and value and writes them to the caches (k, v above) at position Skv.
    const char *cos, *sin, *new_k, *new_v;
    char *k_cache_w, *v_cache_w;  // k and v above, writable
    int64_t cs_b, nk_sb, nk_sh, nv_sb, nv_sh;
    int force_partials;
    // The number of cached positions read on the device (tpamd_attention_decode_rope_devpos): Skv above is then the
    // capacity of the caches, which the launch geometry is made for, and the kernels take the key count from here.
    const int64_t *skv_dev;
};

constexpr int AT_KEYS = 64;   // keys per tile

// RT = 16-row tiles per wavefront: 1 for few rows (decode), 2 for prefill, where every K and V^T fragment read
// from LDS then feeds two MFMAs (with one tile the fragment reads alone would need the whole LDS bandwidth).
// A block owns 64 * RT consecutive rows.
// At least two wavefronts per SIMD are asked for: that caps a wavefront at 256 registers, and with no need for
// AGPRs the compiler keeps MFMA results in ordinary VGPRs, where the softmax can use them without copies.
// P = K / V tiles a thread keeps requested ahead of the one being multiplied (see the two loops below).
template <int DT, int D, int RT, int P>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 8))) void attention_kernel(AttnParams p) {
    constexpr int KP = D * 2 + 16;   // K tile row pitch (bytes): conflict-free 16-byte reads
    constexpr int VP = D * 2 + 32;   // V tile row pitch (bytes): 8 consecutive keys' 32-byte pieces cover all banks
    constexpr int DT16 = D / 16, DK = D / 32;
    constexpr int ROWS = 64 * RT;
    __shared__ __align__(16) char ks[2][AT_KEYS * KP];  // two tiles each: one is multiplied while the next is written
    __shared__ __align__(16) char vs[2][AT_KEYS * VP];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int l16 = lane & 15, lq = lane >> 4;
    const int nrows = p.G * p.Sq;
    // keys in the cache and keys per block of a split: launch arguments, or derived from a count that lives on the device
    int Skv = p.Skv, keys_per_split = p.keys_per_split;
    if (p.skv_dev != nullptr) {
        const int64_t have = *p.skv_dev;
        Skv = have < 0 ? 0 : have < p.Skv ? static_cast<int>(have) : p.Skv;
        keys_per_split = ((Skv + p.nsplit - 1) / p.nsplit + AT_KEYS - 1) / AT_KEYS * AT_KEYS;
    }
    // Causal: a block's key range grows with the positions of its rows, and blocks are handed to the 8 XCDs in turn, so
    // the order must not let block lengths repeat with a period that divides 8 (position tiles within a head do:
    // one XCD would get every longest block and the kernel would take as long as without the mask). The (batch, kv head)
    // index runs fastest, so equally long blocks are neighbours and spread over the XCDs; the row tiles follow with the
    // longest first: all heads' last position tile, then the one before, ... when heads are whole numbers of
    // tiles, else simply the row tiles from the last to the first.
    int bh = blockIdx.y, row_tile = blockIdx.x;
    if (p.causal) {
        const int lin = blockIdx.x + gridDim.x * blockIdx.y;
        bh = lin % gridDim.y;
        const int slow = lin / gridDim.y;  // 0 ... gridDim.x - 1
        const int pt_per_head = p.Sq / ROWS;
        if (pt_per_head > 0 && p.Sq % ROWS == 0) row_tile = (slow % p.G) * pt_per_head + pt_per_head - 1 - slow / p.G;
        else row_tile = gridDim.x - 1 - slow;
    }
    const int b = bh / p.Hkv, hkv = bh % p.Hkv;
    const int row0 = row_tile * ROWS;
    const int shift = Skv - p.Sq;  // causal: key j visible to position sq iff j <= sq + shift

    // Causal: the wavefronts that own a block's first rows stop early (below), and a wavefront's number fixes its SIMD, so
    // every other row tile hands the rows out in the opposite order.
    const int wave_rows = (p.causal && (row_tile & 1)) ? 3 - wave : wave;
    // ---- this lane's query rows and their Q fragments (second MFMA operand): 8 head-dim elements at 32*kk + 8*lq
    int row[RT], sq[RT], head[RT], my_lim[RT];
    bool row_ok[RT];
    uint4 qf[RT][DK];
#pragma unroll
    for (int r = 0; r < RT; ++r) {
        row[r] = row0 + (wave_rows * RT + r) * 16 + l16;
        row_ok[r] = row[r] < nrows;
        const int g = row_ok[r] ? row[r] / p.Sq : 0;
        sq[r] = row_ok[r] ? row[r] % p.Sq : 0;
        head[r] = hkv * p.G + g;
        my_lim[r] = p.causal ? sq[r] + shift : Skv - 1;  // last key this row may see
        const char *qrow = p.q + (static_cast<int64_t>(b) * p.q_sb + static_cast<int64_t>(hkv) * p.q_sg + static_cast<int64_t>(g) * p.q_sh + static_cast<int64_t>(sq[r]) * p.q_ss) * 2;
#pragma unroll
        for (int kk = 0; kk < DK; ++kk)
            qf[r][kk] = *reinterpret_cast<const uint4 *>(qrow + (32 * kk + 8 * lq) * 2);  // rows past the end: row 0 of the group, never stored
        if (p.cos != nullptr) {
            // rotary embedding of the row, as rope_append_kernel does it: element d of the first half pairs with d + D / 2,
            // which is fragment kk + DK / 2 of the same lane
            const char *cs = p.cos + static_cast<int64_t>(b) * p.cs_b * 2, *sn = p.sin + static_cast<int64_t>(b) * p.cs_b * 2;
#pragma unroll
            for (int kk = 0; kk < DK / 2; ++kk) {
                const int at = (32 * kk + 8 * lq) * 2;
                const uint4 x1 = qf[r][kk], x2 = qf[r][kk + DK / 2];
                const uint4 c1 = *reinterpret_cast<const uint4 *>(cs + at), c2 = *reinterpret_cast<const uint4 *>(cs + at + D);
                const uint4 s1 = *reinterpret_cast<const uint4 *>(sn + at), s2 = *reinterpret_cast<const uint4 *>(sn + at + D);
                qf[r][kk] = rot8<DT>(x1, c1, x2, s1, -1.0f);
                qf[r][kk + DK / 2] = rot8<DT>(x2, c2, x1, s2, 1.0f);
            }
        }
    }

    // ---- key range of this block
    int k_begin = blockIdx.z * keys_per_split;
    int k_end = k_begin + keys_per_split < Skv ? k_begin + keys_per_split : Skv;
    if (k_begin > k_end) k_begin = k_end;  // a split behind the last key (count read on the device): an empty range
    if (p.causal) {
        // the largest position among this block's rows (a block that straddles two heads contains position Sq - 1)
        const int last_row = row0 + ROWS - 1 < nrows - 1 ? row0 + ROWS - 1 : nrows - 1;
        const int max_sq = (row0 / p.Sq != last_row / p.Sq) ? p.Sq - 1 : last_row % p.Sq;
        const int lim = max_sq + shift + 1;
        k_end = k_end < lim ? k_end : lim;
    }

    float m_run[RT];
    f32x4 acc[RT][DT16], l_acc[RT];  // l_acc[r][i]: the row sum of this lane's row r, the same in all four elements
    const uint32_t one2 = DT == TPAMD_BF16 ? 0x3f803f80u : 0x3c003c00u;  // two 1.0 in the tensor dtype
    const uint4 ones = make_uint4(one2, one2, one2, one2);
#pragma unroll
    for (int r = 0; r < RT; ++r) {
        m_run[r] = -INFINITY;
        l_acc[r] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int dt = 0; dt < DT16; ++dt) acc[r][dt] = f32x4{0.f, 0.f, 0.f, 0.f};
    }

    const char *kbase = p.k + (static_cast<int64_t>(b) * p.k_sb + static_cast<int64_t>(hkv) * p.k_sh) * 2;
    const char *vbase = p.v + (static_cast<int64_t>(b) * p.v_sb + static_cast<int64_t>(hkv) * p.v_sh) * 2;

    // K / V tiles travel global -> registers -> LDS (row-major, both), and a tile costs one barrier. A full tile's
    // addresses are a loop-invariant per-thread pointer plus a uniform offset.
    constexpr int CH = D / 8;                    // 16-byte chunks per key
    constexpr int LPT = AT_KEYS * CH / 256;      // chunks per thread per tile (2 for head_dim 64, 4 for 128)
    constexpr int KSTEP = 256 / CH;              // keys between a thread's chunks
    u32x4 kreg[P][LPT], vreg[P][LPT];
    const int key_j0 = tid / CH, chunk = tid % CH;  // thread's key inside a tile for j = 0
    const int64_t k_pitch = p.k_ss * 2, v_pitch = p.v_ss * 2;
    const char *kthr = kbase + chunk * 16 + key_j0 * k_pitch, *vthr = vbase + chunk * 16 + key_j0 * v_pitch;
    auto fetch = [&](int k0) {
        if (k0 + AT_KEYS <= k_end) {  // uniform
#pragma unroll
            for (int j = 0; j < LPT; ++j) {
                kreg[0][j] = *reinterpret_cast<const u32x4 *>(kthr + static_cast<int64_t>(k0 + j * KSTEP) * k_pitch);
                vreg[0][j] = *reinterpret_cast<const u32x4 *>(vthr + static_cast<int64_t>(k0 + j * KSTEP) * v_pitch);
            }
        } else {
#pragma unroll
            for (int j = 0; j < LPT; ++j) {
                const int key = k0 + key_j0 + j * KSTEP;
                const bool ok = key < k_end;
                // unconditional loads (first key of the range when out of it) keep all of them in flight together;
                // keys past the end are zero (and masked below)
                const int64_t kr = ok ? key : k_begin;
                const u32x4 kv4 = *reinterpret_cast<const u32x4 *>(kbase + chunk * 16 + kr * k_pitch);
                const u32x4 vv4 = *reinterpret_cast<const u32x4 *>(vbase + chunk * 16 + kr * v_pitch);
                kreg[0][j] = ok ? kv4 : u32x4{0, 0, 0, 0};
                vreg[0][j] = ok ? vv4 : u32x4{0, 0, 0, 0};
            }
        }
    };
    auto stage = [&](int buf) {
#pragma unroll
        for (int j = 0; j < LPT; ++j) {
            const int key = key_j0 + j * KSTEP;
            *reinterpret_cast<u32x4 *>(ks[buf] + key * KP + chunk * 16) = kreg[0][j];
            *reinterpret_cast<u32x4 *>(vs[buf] + key * VP + chunk * 16) = vreg[0][j];
        }
    };
    // The same two steps for the ring of P register sets (slot = tile % P, a constant once the loops are unrolled). The
    // loads are unconditional and sit on no branch, so the compiler can count, per slot, how many younger loads may still
    // be in flight when a slot is written to LDS, instead of waiting for all of them. A key past the end of the range reads
    // the first key of the range instead: finite numbers, whose scores are masked and whose probabilities are 0.
    const int64_t k_safe = k_begin < Skv ? k_begin : 0;
    auto fetch_slot = [&](auto slot, int tile) {
        static_for<LPT>([&](auto jc) {
            constexpr int S = decltype(slot)::value, j = decltype(jc)::value;
            const int key = k_begin + tile * AT_KEYS + key_j0 + j * KSTEP;
            const int64_t kr = key < k_end ? key : k_safe;
            kreg[S][j] = *reinterpret_cast<const u32x4 *>(kbase + chunk * 16 + kr * k_pitch);
            vreg[S][j] = *reinterpret_cast<const u32x4 *>(vbase + chunk * 16 + kr * v_pitch);
        });
    };
    auto stage_slot = [&](auto slot, int buf) {
        static_for<LPT>([&](auto jc) {
            constexpr int S = decltype(slot)::value, j = decltype(jc)::value;
            const int key = key_j0 + j * KSTEP;
            *reinterpret_cast<u32x4 *>(ks[buf] + key * KP + chunk * 16) = kreg[S][j];
            *reinterpret_cast<u32x4 *>(vs[buf] + key * VP + chunk * 16) = vreg[S][j];
        });
    };
    // The transposed V fragments come from the LDS transpose load: the 16 lanes of a group point at 4 keys x 16 head-dim
    // elements (lane j: key j / 4, elements 4 (j % 4) ...) and lane i gets back, for head-dim element i, its 4 keys.
    // This lane's address inside a V tile: key 4 lq + l16 / 4, element 4 (l16 % 4); (u, half, dt) add (32 u + 16 half)
    // keys and 16 dt elements.
    const int v_lane = (4 * lq + (l16 >> 2)) * VP + (l16 & 3) * 8;
    // A wavefront multiplies only the tiles some row of its own can see (causal: the block's range ends with the last row
    // of the block); for the tiles behind them it only takes part in the staging and the barriers.
    int wave_lim = my_lim[0];
#pragma unroll
    for (int r = 1; r < RT; ++r) wave_lim = max(wave_lim, my_lim[r]);
#pragma unroll
    for (int d = 1; d < 16; d *= 2) wave_lim = max(wave_lim, __shfl_xor(wave_lim, d));
    wave_lim = __builtin_amdgcn_readfirstlane(wave_lim);
    // ... and none at all when all its rows lie past the end (decode: 16 rows in a block of 64)
    bool any_row = false;
#pragma unroll
    for (int r = 0; r < RT; ++r) any_row = any_row || row_ok[r];
    const int k_stop = __any(any_row) ? min(k_end, wave_lim + 1) : k_begin;
    // One tile of 64 keys starting at k0, read from the LDS tiles kt (K) and vtile (V).
    auto tile_math = [&](const int k0, const char *kt, const char *vtile) {
        // ---- S^T = K Q^T: s[r][t][i] = score of key k0 + 16 t + 4 lq + i against query row r of this lane
        f32x4 s[RT][4];
#pragma unroll
        for (int t = 0; t < 4; ++t) {
#pragma unroll
            for (int r = 0; r < RT; ++r) s[r][t] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int kk = 0; kk < DK; ++kk) {
                const uint4 kf = *reinterpret_cast<const uint4 *>(kt + (16 * t + l16) * KP + (32 * kk + 8 * lq) * 2);
#pragma unroll
                for (int r = 0; r < RT; ++r) s[r][t] = mfma16<DT>(kf, qf[r][kk], s[r][t]);
            }
        }
        // ---- online softmax per row (the 4 lanes l16 + 16 * {0..3} hold the same row).
        // Probabilities are taken relative to a reference maximum m_run (in units of scale * log2 e) that is only
        // raised when the running maximum outgrows it by more than 2^LAZY: then the accumulators are rescaled;
        // otherwise p = 2^(x - m_run) <= 2^LAZY, well inside what 16-bit p and fp32 sums hold. A tile fully visible to
        // every row of the wavefront skips the masking. The row sums come out of the MFMA pipe (a row of ones appended
        // to V^T) instead of 16 additions per row and tile. The loop is paced by the vector instructions around the
        // MFMAs as much as by the MFMAs (on a SIMD the two did not overlap in any arrangement that was timed), so the
        // fast path of a tile is one fma, one exp2, half a 3-input maximum and half a pack per score, nothing else.
        constexpr float LAZY = 6.0f;
        uint4 pf[RT][2];
        bool tile_free = k0 + AT_KEYS <= k_end;
#pragma unroll
        for (int r = 0; r < RT; ++r) tile_free = tile_free && (k0 + AT_KEYS - 1 <= my_lim[r]);
        const bool no_mask = __all(tile_free);
#pragma unroll
        for (int r = 0; r < RT; ++r) {
            if (!no_mask) {
                // keys of this tile visible to the row: the first `vis`; key (t, i) of this lane sits at 16 t + 4 lq + i
                const int last = my_lim[r] < k_end - 1 ? my_lim[r] : k_end - 1;
                const int vis = last - k0 + 1 - 4 * lq;
#pragma unroll
                for (int t = 0; t < 4; ++t)
#pragma unroll
                    for (int i = 0; i < 4; ++i) s[r][t][i] = (16 * t + i < vis) ? s[r][t][i] : -INFINITY;
            }
            // x = score * scale log2 e - reference; the products are canonical numbers, so their maximum is a plain chain
            // of 3-input maxima (the MFMA results themselves would each be canonicalised first)
            const float neg_ref = m_run[r] == -INFINITY ? 0.f : -m_run[r];
#pragma unroll
            for (int t = 0; t < 4; ++t)
#pragma unroll
                for (int i = 0; i < 4; ++i) s[r][t][i] = fmaf(s[r][t][i], p.scale_log2, neg_ref);
            float mx = fmaxf(s[r][0][0], s[r][0][1]);
#pragma unroll
            for (int t = 0; t < 4; ++t)
#pragma unroll
                for (int i = (t == 0 ? 2 : 0); i < 4; i += 2) mx = fmaxf(fmaxf(mx, s[r][t][i]), s[r][t][i + 1]);
            // every lane looks at its own 16 keys: only when one of them outgrew the reference (or the row has none yet)
            // do the 4 lanes of a row exchange their maxima
            if (__any(mx > LAZY || m_run[r] == -INFINITY)) {
                mx = fmaxf(mx, __shfl_xor(mx, 16));
                mx = fmaxf(mx, __shfl_xor(mx, 32));
                // in absolute units; a row that keeps its reference goes through the same arithmetic with factor 1
                const float m_abs = mx - neg_ref;
                const bool up = m_abs > m_run[r] + LAZY;  // false for -inf on either side
                const float m_new = up ? m_abs : m_run[r];
                const float m_use = m_new == -INFINITY ? 0.f : m_new;  // a row with nothing visible yet
                const float alpha = __builtin_amdgcn_exp2f(m_run[r] - m_use);
                const float move = -neg_ref - m_use;  // x was taken against the old reference
                m_run[r] = m_new;
#pragma unroll
                for (int i = 0; i < 4; ++i) l_acc[r][i] *= alpha;
#pragma unroll
                for (int dt = 0; dt < DT16; ++dt)
#pragma unroll
                    for (int i = 0; i < 4; ++i) acc[r][dt][i] *= alpha;
#pragma unroll
                for (int t = 0; t < 4; ++t)
#pragma unroll
                    for (int i = 0; i < 4; ++i) s[r][t][i] += move;
            }
#pragma unroll
            for (int t = 0; t < 4; ++t)
#pragma unroll
                for (int i = 0; i < 4; ++i) s[r][t][i] = __builtin_amdgcn_exp2f(s[r][t][i]);
            // the lane's probabilities as the second MFMA operand. K slot (lq, e): e < 4 -> key 32 u + 4 lq + e,
            // e >= 4 -> key 32 u + 16 + 4 lq + e - 4
#pragma unroll
            for (int u = 0; u < 2; ++u) {
                pf[r][u].x = pack2_half<DT>(s[r][2 * u][0], s[r][2 * u][1]);
                pf[r][u].y = pack2_half<DT>(s[r][2 * u][2], s[r][2 * u][3]);
                pf[r][u].z = pack2_half<DT>(s[r][2 * u + 1][0], s[r][2 * u + 1][1]);
                pf[r][u].w = pack2_half<DT>(s[r][2 * u + 1][2], s[r][2 * u + 1][3]);
            }
        }

        // ---- O^T += V^T P^T, and the row sums: ones . P^T (every row of that product is the same sum)
#pragma unroll
        for (int u = 0; u < 2; ++u) {
#pragma unroll
            for (int dt = 0; dt < DT16; ++dt) {
                const uint2 lo = lds_transpose_b64(vtile + v_lane + (32 * u) * VP + 32 * dt);
                const uint2 hi = lds_transpose_b64(vtile + v_lane + (32 * u + 16) * VP + 32 * dt);
                const uint4 vf = make_uint4(lo.x, lo.y, hi.x, hi.y);
#pragma unroll
                for (int r = 0; r < RT; ++r) acc[r][dt] = mfma16<DT>(vf, pf[r][u], acc[r][dt]);
            }
#pragma unroll
            for (int r = 0; r < RT; ++r) l_acc[r] = mfma16<DT>(ones, pf[r][u], l_acc[r]);
        }
    };

    if constexpr (P == 1) {
        // One register set: the loads of tile i+2 are requested right after tile i+1 went into LDS, and fly during one
        // tile's MFMAs and softmax. Enough where a CU holds several blocks with long tiles (prefill).
        if (k_begin < k_end) {
            fetch(k_begin);
            stage(0);
        }
        // Wait here, on every path into the loop, for all that was requested so far (the Q fragments among it): the
        // compiler then knows that the only loads in flight at the top of the loop are the tile requested ahead, which
        // nothing reads before the end of the tile's arithmetic. Without it the first MFMAs of every tile waited for
        // all loads (s_waitcnt vmcnt(0)), the tile requested one barrier earlier included.
        __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0), the other counters left alone
        if (k_begin + AT_KEYS < k_end) fetch(k_begin + AT_KEYS);
        __syncthreads();
        int buf = 0;
        int k0 = k_begin;
        for (; k0 < k_stop; k0 += AT_KEYS, buf ^= 1) {
            tile_math(k0, ks[buf], vs[buf]);
            // the next tile into the other buffer (last read one tile ago, before the previous barrier)
            if (k0 + AT_KEYS < k_end) {
                stage(buf ^ 1);
                if (k0 + 2 * AT_KEYS < k_end) fetch(k0 + 2 * AT_KEYS);
            }
            __syncthreads();
        }
        for (; k0 < k_end; k0 += AT_KEYS, buf ^= 1) {
            if (k0 + AT_KEYS < k_end) {
                stage(buf ^ 1);
                if (k0 + 2 * AT_KEYS < k_end) fetch(k0 + 2 * AT_KEYS);
            }
            __syncthreads();
        }
    } else {
        // Few rows (decode): a tile's arithmetic is short, and with one register set a block would wait out one memory
        // round trip per tile. P sets keep P tiles requested: tile t + 1 goes from its slot into LDS after tile t was
        // multiplied, and the slot is asked for tile t + 1 + P at once. The loop body is repeated P times so that slots are
        // compile-time registers; the iterations past the last tile only stage and load harmless repeats.
        const int n_tiles = k_begin < k_end ? (k_end - k_begin + AT_KEYS - 1) / AT_KEYS : 0;
        const int n_math = k_begin < k_stop ? (k_stop - k_begin + AT_KEYS - 1) / AT_KEYS : 0;
        // (also for an empty range, where they read the fallback key: one path into the loop lets the compiler know that
        // the Q fragments have arrived by then, instead of waiting for every load in flight at the top of each round)
        static_for<P>([&](auto sl) { fetch_slot(sl, decltype(sl)::value); });
        stage_slot(Const<0>{}, 0);
        fetch_slot(Const<0>{}, P);
        __syncthreads();
        for (int g = 0; g < n_tiles; g += P) {
            static_for<P>([&](auto jc) {
                constexpr int j = decltype(jc)::value;
                const int t = g + j;
                if (t < n_math) tile_math(k_begin + t * AT_KEYS, ks[t & 1], vs[t & 1]);
                stage_slot(Const<(j + 1) % P>{}, (t + 1) & 1);
                fetch_slot(Const<(j + 1) % P>{}, t + 1 + P);
                __syncthreads();
            });
        }
    }

    // ---- acc[r][dt][i] = O[row r of this lane][d = 16 dt + 4 lq + i]
#pragma unroll
    for (int r = 0; r < RT; ++r) {
        if (!row_ok[r]) continue;
        if (p.nsplit == 1 && !p.force_partials) {
            const float l_row = l_acc[r][0];
            const float inv = l_row > 0.f ? 1.0f / l_row : 0.f;
            char *orow = p.o + (static_cast<int64_t>(b) * p.o_sb + static_cast<int64_t>(sq[r]) * p.o_ss + static_cast<int64_t>(head[r]) * p.o_sh) * 2;
#pragma unroll
            for (int dt = 0; dt < DT16; ++dt) {
                uint2 o2;
                o2.x = pack2_half<DT>(acc[r][dt][0] * inv, acc[r][dt][1] * inv);
                o2.y = pack2_half<DT>(acc[r][dt][2] * inv, acc[r][dt][3] * inv);
                *reinterpret_cast<uint2 *>(orow + (16 * dt + 4 * lq) * 2) = o2;
            }
        } else {
            float *pr = p.part + ((static_cast<int64_t>(blockIdx.z) * gridDim.y + bh) * p.rows_pad + row[r]) * (D + 4);
#pragma unroll
            for (int dt = 0; dt < DT16; ++dt) *reinterpret_cast<f32x4 *>(pr + 16 * dt + 4 * lq) = acc[r][dt];
            if (lq == 0) {
                pr[D] = m_run[r];
                pr[D + 1] = l_acc[r][0];
            }
        }
    }
}

// out[row] = sum_s 2^(m_s - M) O_s / sum_s 2^(m_s - M) l_s over the key splits. One thread per (row, 4 head-dim elements).
template <int DT, int D>
__global__ __launch_bounds__(256) void attention_combine_kernel(AttnParams p) {
    const int nrows = p.G * p.Sq;
    const int per_row = D / 4;
    const int64_t e = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
    const int bh = blockIdx.y;
    if (e >= static_cast<int64_t>(nrows) * per_row) return;
    const int row = static_cast<int>(e / per_row), d4 = static_cast<int>(e % per_row) * 4;
    // the splits' partials are requested eight at a time (a loop that loads, waits and adds per split costs a memory
    // round trip per split: 16 splits took 5.9 us)
    const int64_t split_pitch = static_cast<int64_t>(gridDim.y) * p.rows_pad * (D + 4);
    const float *pr0 = p.part + (static_cast<int64_t>(bh) * p.rows_pad + row) * (D + 4);
    float M = -INFINITY;
    for (int s0 = 0; s0 < p.nsplit; s0 += 8) {
        float ms[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) ms[j] = pr0[(s0 + j < p.nsplit ? s0 + j : s0) * split_pitch + D];
#pragma unroll
        for (int j = 0; j < 8; ++j) M = fmaxf(M, ms[j]);
    }
    const float m_use = M == -INFINITY ? 0.f : M;
    float o[4] = {0.f, 0.f, 0.f, 0.f}, l = 0.f;
    for (int s0 = 0; s0 < p.nsplit; s0 += 8) {
        float2 ml[8];
        f32x4 ov[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const float *pr = pr0 + (s0 + j < p.nsplit ? s0 + j : s0) * split_pitch;
            ml[j] = *reinterpret_cast<const float2 *>(pr + D);
            ov[j] = *reinterpret_cast<const f32x4 *>(pr + d4);
        }
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const float w = s0 + j < p.nsplit ? exp2f(ml[j].x - m_use) : 0.f;
            l += w * ml[j].y;
#pragma unroll
            for (int i = 0; i < 4; ++i) o[i] += w * ov[j][i];
        }
    }
    const float inv = l > 0.f ? 1.0f / l : 0.f;
    const int b = bh / p.Hkv, hkv = bh % p.Hkv, g = row / p.Sq, sq = row % p.Sq;
    const int head = hkv * p.G + g;
    uint2 o2;
    o2.x = pack2_half<DT>(o[0] * inv, o[1] * inv);
    o2.y = pack2_half<DT>(o[2] * inv, o[3] * inv);
    *reinterpret_cast<uint2 *>(p.o + (static_cast<int64_t>(b) * p.o_sb + static_cast<int64_t>(sq) * p.o_ss + static_cast<int64_t>(head) * p.o_sh + d4) * 2) = o2;
}

// The merge for decode with the rotary embedding folded in (Sq = 1): the splits over the cached keys (none when the
// cache is empty), plus the new position. A row's D / 4 threads (consecutive lanes of one wavefront) rotate their 4
// elements of the raw query and key rows exactly as rope_append_kernel does, meet for the dot product, and merge
// (score, 1, v) as one more partial in fp32; the threads of a group's first head also write the rotated key and the
// value into the caches at position Skv.
template <int DT, int D>
__global__ __launch_bounds__(256) void attention_combine_newkey_kernel(AttnParams p) {
    constexpr int per_row = D / 4;
    const int nrows = p.G;  // Sq = 1: a row is a query head of the group
    const int e = blockIdx.x * 256 + threadIdx.x;
    const int bh = blockIdx.y;
    const int b = bh / p.Hkv, hkv = bh % p.Hkv;
    // threads past the last row work on row 0 (they take part in the shuffles) and store nothing
    const bool live = e < nrows * per_row;
    const int row = live ? e / per_row : 0, d4 = (e % per_row) * 4;
    const bool lower = d4 < D / 2;
    const int partner = lower ? d4 + D / 2 : d4 - D / 2;
    const char *qrow = p.q + (static_cast<int64_t>(b) * p.q_sb + static_cast<int64_t>(hkv) * p.q_sg + static_cast<int64_t>(row) * p.q_sh) * 2;
    const char *krow = p.new_k + (static_cast<int64_t>(b) * p.nk_sb + static_cast<int64_t>(hkv) * p.nk_sh) * 2;
    const char *vrow = p.new_v + (static_cast<int64_t>(b) * p.nv_sb + static_cast<int64_t>(hkv) * p.nv_sh) * 2;
    const char *cs = p.cos + static_cast<int64_t>(b) * p.cs_b * 2, *sn = p.sin + static_cast<int64_t>(b) * p.cs_b * 2;
    const uint2 c = *reinterpret_cast<const uint2 *>(cs + d4 * 2), sv = *reinterpret_cast<const uint2 *>(sn + d4 * 2);
    const float sign = lower ? -1.0f : 1.0f;  // rotate_half(x) = cat(-x[D/2:], x[:D/2])
    auto rotated = [&](const char *r) {
        const uint2 own = *reinterpret_cast<const uint2 *>(r + d4 * 2), oth = *reinterpret_cast<const uint2 *>(r + partner * 2);
        return make_uint2(rot2<DT>(own.x, c.x, oth.x, sv.x, sign), rot2<DT>(own.y, c.y, oth.y, sv.y, sign));
    };
    const uint2 qr = rotated(qrow), kr = rotated(krow);
    const uint2 vn = *reinterpret_cast<const uint2 *>(vrow + d4 * 2);
    float dot = lo_half_to_f32<DT>(qr.x) * lo_half_to_f32<DT>(kr.x) + hi_half_to_f32<DT>(qr.x) * hi_half_to_f32<DT>(kr.x) +
                lo_half_to_f32<DT>(qr.y) * lo_half_to_f32<DT>(kr.y) + hi_half_to_f32<DT>(qr.y) * hi_half_to_f32<DT>(kr.y);
#pragma unroll
    for (int d = 1; d < per_row; d *= 2) dot += __shfl_xor(dot, d);
    const float x_new = dot * p.scale_log2;
    // where the new position goes: a launch argument, or the count on the device (then p.Skv is the caches' capacity, and a
    // count that has reached it leaves the caches alone)
    int64_t pos = p.Skv;
    bool room = true;
    if (p.skv_dev != nullptr) {
        pos = *p.skv_dev;
        room = pos >= 0 && pos < p.Skv;
    }
    if (live && row == 0 && room) {  // the new position's cache rows
        *reinterpret_cast<uint2 *>(p.k_cache_w + (static_cast<int64_t>(b) * p.k_sb + static_cast<int64_t>(hkv) * p.k_sh + pos * p.k_ss + d4) * 2) = kr;
        *reinterpret_cast<uint2 *>(p.v_cache_w + (static_cast<int64_t>(b) * p.v_sb + static_cast<int64_t>(hkv) * p.v_sh + pos * p.v_ss + d4) * 2) = vn;
    }
    if (!live) return;

    const int64_t split_pitch = static_cast<int64_t>(gridDim.y) * p.rows_pad * (D + 4);
    const float *pr0 = p.part + (static_cast<int64_t>(bh) * p.rows_pad + row) * (D + 4);
    float M = x_new;
    for (int s0 = 0; s0 < p.nsplit; s0 += 8) {
        float ms[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) ms[j] = pr0[(s0 + j < p.nsplit ? s0 + j : s0) * split_pitch + D];
#pragma unroll
        for (int j = 0; j < 8; ++j) M = fmaxf(M, ms[j]);
    }
    const float w_new = exp2f(x_new - M);
    float o[4] = {w_new * lo_half_to_f32<DT>(vn.x), w_new * hi_half_to_f32<DT>(vn.x), w_new * lo_half_to_f32<DT>(vn.y), w_new * hi_half_to_f32<DT>(vn.y)};
    float l = w_new;
    for (int s0 = 0; s0 < p.nsplit; s0 += 8) {
        float2 ml[8];
        f32x4 ov[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const float *pr = pr0 + (s0 + j < p.nsplit ? s0 + j : s0) * split_pitch;
            ml[j] = *reinterpret_cast<const float2 *>(pr + D);
            ov[j] = *reinterpret_cast<const f32x4 *>(pr + d4);
        }
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const float w = s0 + j < p.nsplit ? exp2f(ml[j].x - M) : 0.f;
            l += w * ml[j].y;
#pragma unroll
            for (int i = 0; i < 4; ++i) o[i] += w * ov[j][i];
        }
    }
    const float inv = 1.0f / l;  // l >= the new position's weight, which is 1 when it holds the maximum
    uint2 o2;
    o2.x = pack2_half<DT>(o[0] * inv, o[1] * inv);
    o2.y = pack2_half<DT>(o[2] * inv, o[3] * inv);
    const int head = hkv * p.G + row;
    *reinterpret_cast<uint2 *>(p.o + (static_cast<int64_t>(b) * p.o_sb + static_cast<int64_t>(head) * p.o_sh + d4) * 2) = o2;
}

template <int DT, int D>
int launch(AttnParams p, int cus, hipStream_t s) {
    int dev = 0;
    TPAMD_HIP(hipGetDevice(&dev));
    const int nrows = p.G * p.Sq;
    constexpr int RING = D == 64 ? 4 : 2;  // tiles requested ahead by the ring kernel: 64 registers either way
    constexpr int RING_MIN_TILES = 8;      // shorter key ranges: the ring's extra loads and idle rounds cost more than it hides
    // 128 rows per block (two 16-row tiles per wavefront) once that still leaves every CU a few blocks
    const bool wide = nrows >= 128 && static_cast<int64_t>((nrows + 127) / 128) * p.B * p.Hkv >= 2 * cus;
    const int block_rows = wide ? 128 : 64;
    const int row_tiles = (nrows + block_rows - 1) / block_rows;
    const int64_t blocks = static_cast<int64_t>(row_tiles) * p.B * p.Hkv;
    // Split the keys when the rows alone leave CUs idle. Fitted on a sweep of 144 decode shapes (D = 64 / 128, 1-1024
    // blocks, 512-32768 keys) and 32 shapes with several positions per sequence (short causal prefills, 8-256 new
    // positions on 2048-8192 cached keys), each with 1-64 splits, with and without the ring kernel, inside a HIP graph
    // on caches that rotate through more memory than the chip caches: within 1 % of the best choice per decode shape
    // in the geometric mean (the rules before: 5 %, up to 31 % on 8192 keys with few heads).
    //  - as many splits as give every CU a block, or two where blocks are light (D = 64 from 32 blocks on) or full
    //    (64 rows: the MFMA work of one block no longer hides another's loads);
    //  - but every split costs a partial to write and merge, every key a fixed time: the sum is least near
    //    sqrt(keys / 8) splits (512 keys: 8, 8192: 32, 32768: 64), which caps the count where heads are few; blocks of
    //    64 rows write 4-64 times the partials of a decode block: half as many splits, and 256 keys or more in each
    //    (a causal prefill of 512 positions on 16 heads: 8.9 us unsplit, 13.3 us in four);
    //  - with a block for every other CU, 512 keys are not worth a second launch (D = 64, 128 blocks: 8.5 us against
    //    9.1 us), and with one for every CU splitting pays only on long caches (D = 64, 256 blocks, 32768 keys: 431 us
    //    unsplit, 366 us in two).
    // The ring kernel (several tiles in flight per block) never beat the best split count of the plain kernel by more
    // than 1 % in these sweeps and stays behind TPAMD_ATTN_RING.
    int nsplit = 1;
    bool ring = false;
    const bool full_rows = nrows >= 64;
    const int per_cu = (D <= 64 && blocks >= 32) || full_rows ? 2 : 1;
    const int64_t keys_seen = p.causal && p.Sq > 1 ? p.Skv - (p.Sq < p.Skv ? p.Sq : p.Skv) / 2 : p.Skv;  // what a row sees on average
    if (blocks < static_cast<int64_t>(per_cu) * cus && !(!full_rows && blocks >= cus && keys_seen < 8192) && !(blocks * 2 >= cus && keys_seen <= 512)) {
        nsplit = static_cast<int>((static_cast<int64_t>(per_cu) * cus + blocks - 1) / blocks);
        int by_keys = static_cast<int>(lroundf(sqrtf(static_cast<float>(keys_seen) / 8.f)));
        if (full_rows) {
            // with a block for every other CU already, a split has to bring 1024 keys or more (224 blocks of 64 rows on 572 keys:
            // 11.9 us unsplit, 17.6 us in two; 320 blocks on 5936 keys: 88 us unsplit, 68 us in two, 60 us in four)
            const int64_t min_keys = blocks * 2 >= cus ? 1024 : blocks * 8 < cus ? 128 : 256;  // a handful of blocks: 10 on 692 keys, 10.2 us in two, 8.5 us in four
            by_keys = by_keys / 2 < keys_seen / min_keys ? by_keys / 2 : static_cast<int>(keys_seen / min_keys);
        }
        if (nsplit > by_keys) nsplit = by_keys;
        if (nsplit > 64) nsplit = 64;
        if (nsplit < 1) nsplit = 1;
        if (!full_rows && nsplit > 1) {
            if (D <= 64 && keys_seen < 512) {
                nsplit = 1;  // under 8 tiles of 64-wide heads the second launch costs what the split saves (300 keys: 6.2-7.6 us unsplit, 6.6-8.8 us split)
            } else {
                // Between half and one and a half times that count, the one whose blocks fill whole rounds best (one block per
                // CU at a time for D = 128, two for D = 64): a last round with a few blocks costs as much as a full one
                // (96 blocks on 20000 keys: 3 splits, 288 blocks, 205 us; 2 splits 180 us; 40 blocks: 7 splits 89 us, 6 splits
                // 75 us). On 90 random decode shapes with every count measured this took the choices from 4.1 % to 2.1 % off
                // the best count per shape in the geometric mean.
                const int64_t per_round = static_cast<int64_t>(cus) * (D <= 64 ? 2 : 1);
                const int hi = nsplit * 3 / 2 < by_keys ? nsplit * 3 / 2 : by_keys;
                int64_t best_cost = -1;
                int best_n = nsplit;
                for (int n = nsplit / 2 > 2 ? nsplit / 2 : 2; n <= hi && n <= 64; ++n) {
                    const int64_t kps = ((keys_seen + n - 1) / n + AT_KEYS - 1) / AT_KEYS * AT_KEYS;
                    if ((keys_seen + kps - 1) / kps != n) continue;  // this count rounds to another one
                    const int64_t cost = ((blocks * n + per_round - 1) / per_round) * kps;
                    if (best_cost < 0 || cost < best_cost) { best_cost = cost; best_n = n; }
                }
                nsplit = best_n;
            }
        }
    }
    if (tuning().attn_splits != TUNE_UNSET) {
        nsplit = tuning().attn_splits > 0 ? tuning().attn_splits : 1;
        ring = !wide && p.Skv / nsplit >= RING_MIN_TILES * AT_KEYS;
    }
    if (tuning().attn_ring != TUNE_UNSET) ring = !wide && tuning().attn_ring > 0;
    const bool newkey = p.cos != nullptr;  // decode with the new position merged in by the second launch
    if (p.Skv > 0) {
        p.keys_per_split = ((p.Skv + nsplit - 1) / nsplit + AT_KEYS - 1) / AT_KEYS * AT_KEYS;
        nsplit = (p.Skv + p.keys_per_split - 1) / p.keys_per_split;
    } else {
        nsplit = 0;  // an empty cache (newkey only): no partials, the merge sees the new position alone
        p.keys_per_split = AT_KEYS;
    }
    p.nsplit = nsplit;
    p.rows_pad = row_tiles * block_rows;
    p.force_partials = newkey ? 1 : 0;
    TPAMD_REQUIRE(p.B * p.Hkv < 65536 && nsplit < 65536, "attention: batch * kv heads too large for one launch");
    const dim3 grid(row_tiles, p.B * p.Hkv, nsplit > 0 ? nsplit : 1);
    auto run = [&](const AttnParams &prm, dim3 g, bool with_ring) {
        if (wide) hipLaunchKernelGGL((attention_kernel<DT, D, 2, 1>), g, dim3(256), 0, s, prm);
        else if (with_ring) hipLaunchKernelGGL((attention_kernel<DT, D, 1, RING>), g, dim3(256), 0, s, prm);
        else hipLaunchKernelGGL((attention_kernel<DT, D, 1, 1>), g, dim3(256), 0, s, prm);
        return hipGetLastError();
    };
    if (nsplit == 1 && !newkey) {
        TPAMD_HIP(run(p, grid, ring));
        return TPAMD_OK;
    }
    if (nsplit > 0) {
        const size_t need = static_cast<size_t>(nsplit) * p.B * p.Hkv * p.rows_pad * (D + 4) * sizeof(float);
        std::lock_guard<std::mutex> hold(splitk_mutex(dev));
        void *ws = nullptr;
        int rc = splitk_scratch(dev, s, need, static_cast<size_t>(4) * cus * 128 * 128 * sizeof(float), &ws);
        if (rc != TPAMD_OK) return rc;
        if (ws == nullptr) {  // no scratch (first use under stream capture, or more than it holds)
            if (newkey) {
                set_error("%s", "tpamd_attention_decode_rope: no scratch buffer for the partial results of this stream (its first use "
                                "under stream capture, or a batch that needs more than the buffer holds): call tpamd_rope_append and "
                                "tpamd_attention instead");
                return TPAMD_ERR_UNSUPPORTED;
            }
            p.nsplit = 1;  // one split, no partials
            p.keys_per_split = (p.Skv + AT_KEYS - 1) / AT_KEYS * AT_KEYS;
            TPAMD_HIP(run(p, dim3(row_tiles, p.B * p.Hkv, 1), p.Skv >= RING_MIN_TILES * AT_KEYS));
            return TPAMD_OK;
        }
        p.part = static_cast<float *>(ws);
        TPAMD_HIP(run(p, grid, ring));
        // (the merge below is enqueued under the same lock: the buffer is this call's until then)
        const unsigned cblocks = static_cast<unsigned>((static_cast<int64_t>(nrows) * (D / 4) + 255) / 256);
        if (newkey) hipLaunchKernelGGL((attention_combine_newkey_kernel<DT, D>), dim3(cblocks, p.B * p.Hkv), dim3(256), 0, s, p);
        else hipLaunchKernelGGL((attention_combine_kernel<DT, D>), dim3(cblocks, p.B * p.Hkv), dim3(256), 0, s, p);
        TPAMD_HIP(hipGetLastError());
        return TPAMD_OK;
    }
    // newkey on an empty cache
    const unsigned cblocks = static_cast<unsigned>((static_cast<int64_t>(nrows) * (D / 4) + 255) / 256);
    hipLaunchKernelGGL((attention_combine_newkey_kernel<DT, D>), dim3(cblocks, p.B * p.Hkv), dim3(256), 0, s, p);
    TPAMD_HIP(hipGetLastError());
    return TPAMD_OK;
}

}  // namespace

int attention_dispatch(const void *q, const void *k, const void *v, void *o, int64_t B, int64_t Hq, int64_t Hkv, int64_t Sq,
                       int64_t Skv, int64_t D, const int64_t *strides, float scale, int causal, int dtype, hipStream_t s) {
    int dev = 0, cus = 256;
    TPAMD_HIP(hipGetDevice(&dev));
    if (int rc_cus = device_cus(dev, &cus); rc_cus != TPAMD_OK) return rc_cus;
    AttnParams p{};
    p.q = static_cast<const char *>(q);
    p.k = static_cast<const char *>(k);
    p.v = static_cast<const char *>(v);
    p.o = static_cast<char *>(o);
    p.B = static_cast<int>(B); p.Hq = static_cast<int>(Hq); p.Hkv = static_cast<int>(Hkv);
    p.Sq = static_cast<int>(Sq); p.Skv = static_cast<int>(Skv); p.G = static_cast<int>(Hq / Hkv);
    p.q_sb = strides[0]; p.q_sh = strides[1]; p.q_ss = strides[2];
    p.k_sb = strides[3]; p.k_sh = strides[4]; p.k_ss = strides[5];
    p.v_sb = strides[6]; p.v_sh = strides[7]; p.v_ss = strides[8];
    p.o_sb = strides[9]; p.o_ss = strides[10]; p.o_sh = strides[11];
    p.q_sg = p.G * p.q_sh;
    p.scale_log2 = scale * 1.4426950408889634f;
    p.causal = causal;
    const bool bf = dtype == TPAMD_BF16;
    if (D == 64) return bf ? launch<TPAMD_BF16, 64>(p, cus, s) : launch<TPAMD_F16, 64>(p, cus, s);
    return bf ? launch<TPAMD_BF16, 128>(p, cus, s) : launch<TPAMD_F16, 128>(p, cus, s);
}

// One new position per sequence on a cache of `pos0` positions. strides (elements): {q batch, q head, q group, k batch,
// k head, v batch, v head, cos/sin batch, k_cache batch, k_cache head, k_cache position, v_cache batch, v_cache head,
// v_cache position, out batch, out head}.
// pos_dev == NULL: `pos0` positions are cached. Otherwise the count is read from *pos_dev by the kernels and `pos0` is the
// capacity of the caches: the grid and the key splits are made for the capacity, the blocks share out the keys there are.
int attention_decode_rope_dispatch(const void *q, const void *k, const void *v, const void *cos, const void *sin, void *k_cache,
                                   void *v_cache, void *o, int64_t B, int64_t Hq, int64_t Hkv, int64_t D, int64_t pos0,
                                   const int64_t *pos_dev, const int64_t *strides, float scale, int dtype, hipStream_t s) {
    int dev = 0, cus = 256;
    TPAMD_HIP(hipGetDevice(&dev));
    if (int rc_cus = device_cus(dev, &cus); rc_cus != TPAMD_OK) return rc_cus;
    AttnParams p{};
    p.q = static_cast<const char *>(q);
    p.k = static_cast<const char *>(k_cache);
    p.v = static_cast<const char *>(v_cache);
    p.k_cache_w = static_cast<char *>(k_cache);
    p.v_cache_w = static_cast<char *>(v_cache);
    p.new_k = static_cast<const char *>(k);
    p.new_v = static_cast<const char *>(v);
    p.cos = static_cast<const char *>(cos);
    p.sin = static_cast<const char *>(sin);
    p.o = static_cast<char *>(o);
    p.B = static_cast<int>(B); p.Hq = static_cast<int>(Hq); p.Hkv = static_cast<int>(Hkv);
    p.Sq = 1; p.Skv = static_cast<int>(pos0); p.G = static_cast<int>(Hq / Hkv);
    p.skv_dev = pos_dev;
    p.q_sb = strides[0]; p.q_sh = strides[1]; p.q_sg = strides[2]; p.q_ss = 0;
    p.nk_sb = strides[3]; p.nk_sh = strides[4];
    p.nv_sb = strides[5]; p.nv_sh = strides[6];
    p.cs_b = strides[7];
    p.k_sb = strides[8]; p.k_sh = strides[9]; p.k_ss = strides[10];
    p.v_sb = strides[11]; p.v_sh = strides[12]; p.v_ss = strides[13];
    p.o_sb = strides[14]; p.o_sh = strides[15]; p.o_ss = 0;
    p.scale_log2 = scale * 1.4426950408889634f;
    p.causal = 0;  // the one new position sees every cached key
    const bool bf = dtype == TPAMD_BF16;
    if (D == 64) return bf ? launch<TPAMD_BF16, 64>(p, cus, s) : launch<TPAMD_F16, 64>(p, cus, s);
    return bf ? launch<TPAMD_BF16, 128>(p, cus, s) : launch<TPAMD_F16, 128>(p, cus, s);
}

}  // namespace tpamd
