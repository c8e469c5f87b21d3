// tpamd_linear_noalloc: the shard Linear for callers that cannot allocate device memory (code under HIP graph capture,
// tight serving loops, harnesses that forbid hipMalloc). Same kernels and same choices as tpamd_linear; what differs is
// where the fp32 partial tiles of a K split go: into the fixed array below instead of a buffer from hipMalloc.
#include "common.h"

namespace tpamd {

// One copy of this array lives on every GPU the library is loaded on, at an address of its own, until the process ends.
// Host code never hands this name to a kernel or a HIP call: the device address is looked up once per device with
// hipGetSymbolAddress and kept in g_static_ptr, and that pointer is what the kernels get.
static __device__ __align__(256) char scratch[TPAMD_NOALLOC_SCRATCH_BYTES];

namespace {
constexpr int MAX_DEV = 64;
void *g_static_ptr[MAX_DEV];  // entry d guarded by splitk_mutex(d)
thread_local bool g_static_mode = false;
}  // namespace

StaticScratchScope::StaticScratchScope() { g_static_mode = true; }
StaticScratchScope::~StaticScratchScope() { g_static_mode = false; }
bool static_scratch_active() { return g_static_mode; }

// Called by splitk_scratch() with splitk_mutex(dev) held and `dev` current.
int static_scratch(int dev, size_t need, void **out) {
    *out = nullptr;
    if (need > TPAMD_NOALLOC_SCRATCH_BYTES) {
        set_error("tpamd_linear_noalloc: this shape splits K and needs %zu bytes of scratch memory, the fixed array holds %zu",
                  need, static_cast<size_t>(TPAMD_NOALLOC_SCRATCH_BYTES));
        return TPAMD_ERR_UNSUPPORTED;
    }
    if (dev < 0 || dev >= MAX_DEV) {
        set_error("tpamd_linear_noalloc: device index %d out of range", dev);
        return TPAMD_ERR_UNSUPPORTED;
    }
    if (g_static_ptr[dev] == nullptr) {
        void *ptr = nullptr;
        TPAMD_HIP(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
        if (ptr == nullptr) {
            set_error("tpamd_linear_noalloc: the scratch array has no address on device %d", dev);
            return TPAMD_ERR_HIP;
        }
        g_static_ptr[dev] = ptr;
    }
    *out = g_static_ptr[dev];
    return TPAMD_OK;
}

}  // namespace tpamd

using namespace tpamd;

extern "C" uint64_t tpamd_noalloc_scratch_bytes(void) { return TPAMD_NOALLOC_SCRATCH_BYTES; }

extern "C" int tpamd_linear_noalloc(const void *x_dev, const void *w_dev, const void *bias_dev, void *y_dev, int64_t M,
                                    int64_t N, int64_t K, int64_t ldx, int64_t ldw, int64_t ldy, int dtype, int act,
                                    void *stream) {
    StaticScratchScope fixed_array;
    return linear_entry("tpamd_linear_noalloc", x_dev, w_dev, bias_dev, nullptr, 0, y_dev, M, N, K, ldx, ldw, ldy, dtype, act,
                        stream);
}
