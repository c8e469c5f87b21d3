// C ABI entry points for the shard Linears, plus the library's error plumbing.
#include "common.h"

#include <string.h>

namespace tpamd {

static thread_local char g_err[512] = "";

void set_error(const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
}

int gemm_dispatch(const void *x, const void *w, const void *w2, const void *bias, const void *addend, int64_t ldadd, void *y,
                  int64_t M, int64_t N, int64_t K, int64_t ldx, int64_t ldw, int64_t ldy, int dtype, int act, bool swiglu,
                  bool generic, hipStream_t s);
int skinny_dispatch(const void *x, const void *w, const void *w2, const void *bias, const void *addend, int64_t ldadd,
                    const void *scale, const void *outlier_idx, const void *w_out, int64_t n_out, void *y, int64_t M, int64_t N,
                    int64_t K, int64_t ldx, int64_t ldw, int64_t ldy, int64_t ld_wout, int dtype, int act, bool swiglu, bool w8,
                    hipStream_t s);

int gemm_w8_dispatch(const void *x, const void *wq, const void *scale, const void *outlier_idx, const void *w_out, int64_t n_out,
                     const void *bias, void *y, int64_t M, int64_t N, int64_t K, int64_t ldx, int64_t ldw, int64_t ld_wout,
                     int64_t ldy, int dtype, int act, hipStream_t s);

int attention_dispatch(const void *q, const void *k, const void *v, void *o, int64_t B, int64_t Hq, int64_t Hkv, int64_t Sq,
                       int64_t Skv, int64_t D, const int64_t *strides, float scale, int causal, int dtype, hipStream_t s);
int attention_decode_rope_dispatch(const void *q, const void *k, const void *v, const void *cos, const void *sin, void *k_cache,
                                   void *v_cache, void *o, int64_t B, int64_t Hq, int64_t Hkv, int64_t D, int64_t pos0, const int64_t *pos_dev,
                                   const int64_t *strides, float scale, int dtype, hipStream_t s);

namespace {

// Largest M served by the weight-streaming kernels; above it the tiled MFMA kernels take over.
constexpr int64_t SKINNY_MAX_M = 16;

// A single 16-bit matrix with at most one 16-column tile per CU stays with the weight-streaming kernel for more rows: the
// tiled kernels split K over blocks there and pay a second launch. How far depends on the row length. Measured inside a
// HIP graph (us, streaming / tiled) at 17 / 32 / 48 / 64 rows:
//   2048 x 2048   6.3  6.8  8.6  8.9 /  9.3  9.9 10.3 10.9     4096 x 2048   6.9  7.7 10.2 10.7 / 10.3 11.2 11.6 12.6
//   3072 x 3072   8.0  9.1 10.7 11.3 / 11.0 11.8 12.0 12.8     (K <= 3072: streaming up to 64 rows)
//   2048 x 4096   9.1 10.2 12.9 13.5 / 10.6 11.2 11.6 12.2     4096 x 4096  10.0 11.4 14.8 16.0 / 12.0 12.6 13.4 14.4
//   4096 x 5504  13.5 15.0 18.5 19.9 / 16.3 16.9 18.0 19.1     4096 x 8192  16.7 18.7 23.3 24.7 / 17.9 18.8 19.5 20.3
//                                                              (longer rows: streaming up to 32 rows)
//   2048 x 8192  14.4 16.4 21.0 22.9 / 13.2 13.9 15.1 16.0     1536 x 6144  11.8 13.6 17.1 18.5 / 11.7 12.2 12.6 13.1
//                                                              (K >= 6144 on at most half a tile per CU: tiled from 17 rows)
// With more tiles the tiled kernels win from 17 rows on (11008 x 4096: 26.5 29.0 36.2 39.0 / 24.6 25.4 25.3 26.5), and the
// gated pair is faster through them at all of these sizes.
int skinny_row_limit(int64_t N, int64_t K, int64_t *rows) {
    *rows = SKINNY_MAX_M;
    if (tuning().skinny_max_m != TUNE_UNSET) {
        *rows = tuning().skinny_max_m < 64 ? tuning().skinny_max_m : 64;
        return TPAMD_OK;
    }
    int dev = 0, cus = 256;
    TPAMD_HIP(hipGetDevice(&dev));
    if (int rc = device_cus(dev, &cus); rc != TPAMD_OK) return rc;
    const int64_t tiles = (N + 15) / 16;
    if (K < 2048 || K > 8192 || tiles > cus) return TPAMD_OK;
    if (K <= 3072) *rows = 64;
    else if (!(K >= 6144 && tiles * 2 <= cus)) *rows = 32;
    return TPAMD_OK;
}
// The gated pair with at most one 8-column tile per CU (2048 columns on 256 CUs) and rows of up to 6144 elements stays
// with the weight-streaming kernel up to 32 rows. Measured inside a HIP graph (us, streaming / tiled) at 17 / 24 / 32 rows:
//   1376 x 2048   6.6  6.9  7.2 / 10.7 11.5 12.3     2048 x 4096  10.8 10.9 11.6 / 12.2 12.3 12.8
//   1376 x 4096  10.3 10.3 11.0 / 12.0 12.3 13.1     2048 x 5504  13.7 14.3 15.3 / 14.6 14.9 15.4
// With more columns the tiled kernels win (2752 x 4096: 17.4 18.4 20.0 / 14.5 14.7 15.1), and on K = 8192 from 1024 columns on.
int pair_row_limit(int64_t N, int64_t K, int64_t *rows) {
    *rows = SKINNY_MAX_M;
    if (tuning().skinny_max_m != TUNE_UNSET) {
        *rows = tuning().skinny_max_m < 32 ? tuning().skinny_max_m : 32;
        return TPAMD_OK;
    }
    int dev = 0, cus = 256;
    TPAMD_HIP(hipGetDevice(&dev));
    if (int rc = device_cus(dev, &cus); rc != TPAMD_OK) return rc;
    if (K >= 2048 && K <= 6144 && (N + 7) / 8 <= cus) *rows = 32;
    return TPAMD_OK;
}
constexpr int64_t SKINNY_W8_SLAB = 64;
constexpr int64_t W8_TILED_ABOVE = 128;  // int8 weights: rows from which the tiled MFMA kernel takes over from the slabs

// What the MFMA kernels need from 16-bit operands: 16-byte aligned rows of x and w, 8-byte aligned groups of 4
// outputs. Anything else goes to the scalar-load kernel.
bool mfma_ok(const void *x, const void *w, const void *w2, const void *bias, const void *y, int64_t N, int64_t K,
             int64_t ldx, int64_t ldw, int64_t ldy) {
    return aligned(x, 16) && aligned(w, 16) && (!w2 || aligned(w2, 16)) && aligned(y, 8) && (!bias || aligned(bias, 8)) &&
           K % 8 == 0 && ldx % 8 == 0 && ldw % 8 == 0 && N % 4 == 0 && ldy % 4 == 0;
}

int check_common(const char *who, const void *x, const void *w, const void *y, int64_t M, int64_t N, int64_t K,
                 int64_t ldx, int64_t ldw, int64_t ldy, int dtype) {
    TPAMD_REQUIRE(M >= 0 && N >= 0 && K >= 0, "%s: negative dimension (M=%lld N=%lld K=%lld)", who, (long long)M,
                  (long long)N, (long long)K);
    TPAMD_REQUIRE(M < (1ll << 31) && N < (1ll << 31) && K < (1ll << 31), "%s: dimension over 2^31", who);
    TPAMD_REQUIRE(dtype == TPAMD_BF16 || dtype == TPAMD_F16 || dtype == TPAMD_F32, "%s: unknown dtype %d", who, dtype);
    if (M == 0 || N == 0) return TPAMD_OK;
    TPAMD_REQUIRE(x && w && y, "%s: null pointer", who);
    TPAMD_REQUIRE(ldx >= K && ldw >= K && ldy >= N, "%s: leading dimension smaller than the row (ldx=%lld ldw=%lld ldy=%lld)",
                  who, (long long)ldx, (long long)ldw, (long long)ldy);
    return TPAMD_OK;
}

}  // namespace
}  // namespace tpamd

using namespace tpamd;

extern "C" int tpamd_abi_version(void) { return TPAMD_ABI_VERSION; }
extern "C" const char *tpamd_last_error(void) { return g_err; }

// y = act(x . w^T + bias), then, with an addend, y = round(y + addend) in the tensor dtype.
int tpamd::linear_entry(const char *who, const void *x_dev, const void *w_dev, const void *bias_dev, const void *addend_dev,
                        int64_t ldadd, void *y_dev, int64_t M, int64_t N, int64_t K, int64_t ldx, int64_t ldw, int64_t ldy,
                        int dtype, int act, void *stream) {
    int rc = check_common(who, x_dev, w_dev, y_dev, M, N, K, ldx, ldw, ldy, dtype);
    if (rc != TPAMD_OK) return rc;
    TPAMD_REQUIRE(act == TPAMD_ACT_NONE || act == TPAMD_ACT_GELU, "%s: unknown activation %d", who, act);
    if (M == 0 || N == 0) return TPAMD_OK;
    TPAMD_REQUIRE(addend_dev == nullptr || ldadd >= N, "%s: ldadd=%lld is smaller than N=%lld", who, (long long)ldadd, (long long)N);
    hipStream_t s = static_cast<hipStream_t>(stream);
    const bool fast = dtype != TPAMD_F32 && mfma_ok(x_dev, w_dev, nullptr, bias_dev, y_dev, N, K, ldx, ldw, ldy) &&
                      (addend_dev == nullptr || (aligned(addend_dev, 8) && ldadd % 4 == 0));
    int64_t skinny_rows = SKINNY_MAX_M;
    if (fast && M > SKINNY_MAX_M && M <= 64) {
        rc = skinny_row_limit(N, K, &skinny_rows);
        if (rc != TPAMD_OK) return rc;
    }
    if (fast && M <= skinny_rows)
        return skinny_dispatch(x_dev, w_dev, nullptr, bias_dev, addend_dev, ldadd, nullptr, nullptr, nullptr, 0, y_dev, M, N, K,
                               ldx, ldw, ldy, 0, dtype, act, false, false, s);
    return gemm_dispatch(x_dev, w_dev, nullptr, bias_dev, addend_dev, ldadd, y_dev, M, N, K, ldx, ldw, ldy, dtype, act, false,
                         !fast, s);
}

extern "C" int tpamd_linear(const void *x_dev, const void *w_dev, const void *bias_dev, void *y_dev, int64_t M, int64_t N,
                            int64_t K, int64_t ldx, int64_t ldw, int64_t ldy, int dtype, int act, void *stream) {
    return linear_entry("tpamd_linear", x_dev, w_dev, bias_dev, nullptr, 0, y_dev, M, N, K, ldx, ldw, ldy, dtype, act, stream);
}

extern "C" int tpamd_linear_add(const void *x_dev, const void *w_dev, const void *bias_dev, const void *addend_dev, void *y_dev,
                                int64_t M, int64_t N, int64_t K, int64_t ldx, int64_t ldw, int64_t ldadd, int64_t ldy, int dtype,
                                int act, void *stream) {
    TPAMD_REQUIRE(addend_dev != nullptr || M == 0 || N == 0, "tpamd_linear_add: addend is NULL");
    return linear_entry("tpamd_linear_add", x_dev, w_dev, bias_dev, addend_dev, ldadd, y_dev, M, N, K, ldx, ldw, ldy, dtype, act,
                        stream);
}

extern "C" int tpamd_swiglu_up(const void *x_dev, const void *wg_dev, const void *wu_dev, void *h_dev, int64_t M, int64_t N,
                               int64_t K, int64_t ldx, int64_t ldw, int64_t ldh, int dtype, void *stream) {
    int rc = check_common("tpamd_swiglu_up", x_dev, wg_dev, h_dev, M, N, K, ldx, ldw, ldh, dtype);
    if (rc != TPAMD_OK) return rc;
    if (M == 0 || N == 0) return TPAMD_OK;
    TPAMD_REQUIRE(wu_dev != nullptr, "tpamd_swiglu_up: wu is NULL");
    hipStream_t s = static_cast<hipStream_t>(stream);
    const bool fast = dtype != TPAMD_F32 && mfma_ok(x_dev, wg_dev, wu_dev, nullptr, h_dev, N, K, ldx, ldw, ldh);
    int64_t pair_rows = SKINNY_MAX_M;
    if (fast && M > SKINNY_MAX_M && M <= 32) {
        rc = pair_row_limit(N, K, &pair_rows);
        if (rc != TPAMD_OK) return rc;
    }
    if (fast && M <= pair_rows)
        return skinny_dispatch(x_dev, wg_dev, wu_dev, nullptr, nullptr, 0, nullptr, nullptr, nullptr, 0, h_dev, M, N, K, ldx, ldw,
                               ldh, 0, dtype, TPAMD_ACT_NONE, true, false, s);
    return gemm_dispatch(x_dev, wg_dev, wu_dev, nullptr, nullptr, 0, h_dev, M, N, K, ldx, ldw, ldh, dtype, TPAMD_ACT_NONE, true,
                         !fast, s);
}

extern "C" int tpamd_attention(const void *q_dev, const void *k_dev, const void *v_dev, void *out_dev, int64_t B, int64_t Hq,
                               int64_t Hkv, int64_t Sq, int64_t Skv, int64_t D, const int64_t *strides, float scale, int causal,
                               int dtype, void *stream) {
    const char *who = "tpamd_attention";
    TPAMD_REQUIRE(dtype == TPAMD_BF16 || dtype == TPAMD_F16, "%s: dtype must be BF16 or F16", who);
    TPAMD_REQUIRE(B >= 0 && Hq > 0 && Hkv > 0 && Sq >= 0 && Skv >= 0, "%s: bad dimension", who);
    TPAMD_REQUIRE(Hq % Hkv == 0, "%s: %lld query heads are not a multiple of %lld key/value heads", who, (long long)Hq, (long long)Hkv);
    TPAMD_REQUIRE(strides != nullptr, "%s: strides is NULL", who);
    TPAMD_REQUIRE(!causal || Skv >= Sq, "%s: causal attention needs Skv >= Sq", who);
    if (B == 0 || Sq == 0) return TPAMD_OK;
    TPAMD_REQUIRE(Skv > 0, "%s: no keys", who);
    TPAMD_REQUIRE(q_dev && k_dev && v_dev && out_dev, "%s: null pointer", who);
    TPAMD_REQUIRE(Hq * Sq / Hkv < (1ll << 30) && Skv < (1ll << 30), "%s: sequence too long", who);
    bool ok = (D == 64 || D == 128) && aligned(q_dev, 16) && aligned(k_dev, 16) && aligned(v_dev, 16) && aligned(out_dev, 8);
    for (int i = 0; i < 9; ++i) ok = ok && strides[i] % 8 == 0;   // 16-byte loads of q, k, v rows
    for (int i = 9; i < 12; ++i) ok = ok && strides[i] % 4 == 0;  // 8-byte stores
    if (!ok) {
        set_error("%s: head_dim must be 64 or 128 and rows 16-byte aligned", who);
        return TPAMD_ERR_UNSUPPORTED;
    }
    return attention_dispatch(q_dev, k_dev, v_dev, out_dev, B, Hq, Hkv, Sq, Skv, D, strides, scale, causal, dtype,
                              static_cast<hipStream_t>(stream));
}

extern "C" int tpamd_attention_decode_rope(const void *q_dev, const void *k_dev, const void *v_dev, const void *cos_dev,
                                           const void *sin_dev, void *k_cache_dev, void *v_cache_dev, void *out_dev, int64_t B,
                                           int64_t Hq, int64_t Hkv, int64_t D, int64_t pos0, int64_t cache_len,
                                           const int64_t *strides, float scale, int dtype, void *stream) {
    const char *who = "tpamd_attention_decode_rope";
    TPAMD_REQUIRE(dtype == TPAMD_BF16 || dtype == TPAMD_F16, "%s: dtype must be BF16 or F16", who);
    TPAMD_REQUIRE(B >= 0 && Hq > 0 && Hkv > 0, "%s: bad dimension", who);
    TPAMD_REQUIRE(Hq % Hkv == 0, "%s: %lld query heads are not a multiple of %lld key/value heads", who, (long long)Hq, (long long)Hkv);
    TPAMD_REQUIRE(pos0 >= 0 && pos0 < cache_len, "%s: position %lld does not fit a cache of %lld positions", who, (long long)pos0,
                  (long long)cache_len);
    TPAMD_REQUIRE(strides != nullptr, "%s: strides is NULL", who);
    if (B == 0) return TPAMD_OK;
    TPAMD_REQUIRE(q_dev && k_dev && v_dev && cos_dev && sin_dev && k_cache_dev && v_cache_dev && out_dev, "%s: null pointer", who);
    TPAMD_REQUIRE(Hq / Hkv < (1ll << 20) && pos0 < (1ll << 30), "%s: sequence too long", who);
    bool ok = (D == 64 || D == 128) && aligned(q_dev, 16) && aligned(k_dev, 16) && aligned(v_dev, 16) && aligned(cos_dev, 16) &&
              aligned(sin_dev, 16) && aligned(k_cache_dev, 16) && aligned(v_cache_dev, 16) && aligned(out_dev, 8);
    for (int i = 0; i < 14; ++i) ok = ok && strides[i] % 8 == 0;   // 16-byte loads of every row
    for (int i = 14; i < 16; ++i) ok = ok && strides[i] % 4 == 0;  // 8-byte stores
    if (!ok) {
        set_error("%s: head_dim must be 64 or 128 and rows 16-byte aligned", who);
        return TPAMD_ERR_UNSUPPORTED;
    }
    return attention_decode_rope_dispatch(q_dev, k_dev, v_dev, cos_dev, sin_dev, k_cache_dev, v_cache_dev, out_dev, B, Hq, Hkv, D,
                                          pos0, nullptr, strides, scale, dtype, static_cast<hipStream_t>(stream));
}

extern "C" int tpamd_attention_decode_rope_devpos(const void *q_dev, const void *k_dev, const void *v_dev, const void *cos_dev,
                                                  const void *sin_dev, void *k_cache_dev, void *v_cache_dev, void *out_dev,
                                                  int64_t B, int64_t Hq, int64_t Hkv, int64_t D, const int64_t *pos_dev,
                                                  int64_t cache_len, const int64_t *strides, float scale, int dtype,
                                                  void *stream) {
    const char *who = "tpamd_attention_decode_rope_devpos";
    TPAMD_REQUIRE(dtype == TPAMD_BF16 || dtype == TPAMD_F16, "%s: dtype must be BF16 or F16", who);
    TPAMD_REQUIRE(B >= 0 && Hq > 0 && Hkv > 0, "%s: bad dimension", who);
    TPAMD_REQUIRE(Hq % Hkv == 0, "%s: %lld query heads are not a multiple of %lld key/value heads", who, (long long)Hq, (long long)Hkv);
    TPAMD_REQUIRE(cache_len > 0 && cache_len < (1ll << 30), "%s: the caches must hold between 1 and 2^30 positions", who);
    TPAMD_REQUIRE(strides != nullptr, "%s: strides is NULL", who);
    if (B == 0) return TPAMD_OK;
    TPAMD_REQUIRE(q_dev && k_dev && v_dev && cos_dev && sin_dev && k_cache_dev && v_cache_dev && out_dev && pos_dev, "%s: null pointer", who);
    TPAMD_REQUIRE(Hq / Hkv < (1ll << 20), "%s: too many query heads per key/value head", who);
    bool ok = (D == 64 || D == 128) && aligned(q_dev, 16) && aligned(k_dev, 16) && aligned(v_dev, 16) && aligned(cos_dev, 16) &&
              aligned(sin_dev, 16) && aligned(k_cache_dev, 16) && aligned(v_cache_dev, 16) && aligned(out_dev, 8) && aligned(pos_dev, 8);
    for (int i = 0; i < 14; ++i) ok = ok && strides[i] % 8 == 0;   // 16-byte loads of every row
    for (int i = 14; i < 16; ++i) ok = ok && strides[i] % 4 == 0;  // 8-byte stores
    if (!ok) {
        set_error("%s: head_dim must be 64 or 128 and rows 16-byte aligned", who);
        return TPAMD_ERR_UNSUPPORTED;
    }
    return attention_decode_rope_dispatch(q_dev, k_dev, v_dev, cos_dev, sin_dev, k_cache_dev, v_cache_dev, out_dev, B, Hq, Hkv, D,
                                          cache_len, pos_dev, strides, scale, dtype, static_cast<hipStream_t>(stream));
}

extern "C" int tpamd_linear_w8(const void *x_dev, const void *wq_dev, const void *scale_dev, const void *outlier_idx_dev,
                               const void *w_out_dev, int64_t n_out, const void *bias_dev, void *y_dev, int64_t M, int64_t N,
                               int64_t K, int64_t ldx, int64_t ldw, int64_t ld_wout, int64_t ldy, int dtype, int act,
                               void *stream) {
    const char *who = "tpamd_linear_w8";
    TPAMD_REQUIRE(dtype == TPAMD_BF16 || dtype == TPAMD_F16, "%s: dtype must be BF16 or F16", who);
    TPAMD_REQUIRE(M >= 0 && N >= 0 && K >= 0 && n_out >= 0, "%s: negative dimension", who);
    TPAMD_REQUIRE(M < (1ll << 31) && N < (1ll << 31) && K < (1ll << 31), "%s: dimension over 2^31", who);
    TPAMD_REQUIRE(act == TPAMD_ACT_NONE || act == TPAMD_ACT_GELU, "%s: unknown activation %d", who, act);
    if (M == 0 || N == 0) return TPAMD_OK;
    TPAMD_REQUIRE(x_dev && wq_dev && scale_dev && y_dev, "%s: null pointer", who);
    TPAMD_REQUIRE(n_out == 0 || (outlier_idx_dev && w_out_dev && ld_wout >= n_out), "%s: outlier arguments inconsistent", who);
    TPAMD_REQUIRE(n_out <= K, "%s: more outlier columns (%lld) than K", who, (long long)n_out);
    TPAMD_REQUIRE(aligned(x_dev, 16) && aligned(wq_dev, 16), "%s: x and wq must be 16-byte aligned", who);
    TPAMD_REQUIRE(K % 16 == 0 && ldw % 16 == 0 && ldx % 8 == 0, "%s: K, ldw multiples of 16 and ldx of 8 required", who);
    TPAMD_REQUIRE(ldx >= K && ldw >= K && ldy >= N, "%s: leading dimension smaller than the row", who);
    hipStream_t s = static_cast<hipStream_t>(stream);
    const int esz = 2;
    // Above two slabs of the weight-streaming kernels the weights go through the matrix pipe once, dequantised on their
    // way into LDS; the packed stores of that kernel want groups of 4 outputs on 8-byte boundaries.
    // (measured on 16384 x 8192 / 8192 x 16384: 129-256 rows 131-135 / 225-231 us tiled against 153-204 / 153-203 us in
    // slabs; 512 rows 263 / 237 against 407 / 406; 1024 rows 309 / 484 us, 0.57-0.89 PFLOP/s). With fewer 128 x 128
    // tiles than CUs the slabs stay ahead up to 256 rows.
    const int64_t tiles128 = ((M + 127) / 128) * ((N + 127) / 128);
    if (M > W8_TILED_ABOVE && (tiles128 >= 256 || M > 2 * W8_TILED_ABOVE) && N % 4 == 0 && ldy % 4 == 0 && aligned(y_dev, 8) && (!bias_dev || aligned(bias_dev, 8)) && n_out <= 256)
        return gemm_w8_dispatch(x_dev, wq_dev, scale_dev, outlier_idx_dev, w_out_dev, n_out, bias_dev, y_dev, M, N, K, ldx, ldw,
                                ld_wout, ldy, dtype, act, s);
    for (int64_t m0 = 0; m0 < M; m0 += SKINNY_W8_SLAB) {  // weights are re-streamed once per slab of 64 rows
        const int64_t mm = M - m0 < SKINNY_W8_SLAB ? M - m0 : SKINNY_W8_SLAB;
        int rc = skinny_dispatch(static_cast<const char *>(x_dev) + m0 * ldx * esz, wq_dev, nullptr, bias_dev, nullptr, 0, scale_dev,
                                 outlier_idx_dev, w_out_dev, n_out, static_cast<char *>(y_dev) + m0 * ldy * esz, mm, N, K, ldx,
                                 ldw, ldy, ld_wout, dtype, act, false, true, s);
        if (rc != TPAMD_OK) return rc;
    }
    return TPAMD_OK;
}
