// Host-side state of the library: tuning knobs (read from the environment once), the number of compute units per
// device, and the fp32 scratch memory that the K-split kernels (16-bit and int8 Linears, split-key attention) put their
// partial results in: one buffer per (device, stream).
#include "common.h"

#include <stdlib.h>
#include <string.h>

#include <vector>

namespace tpamd {

// ---- tuning knobs -----------------------------------------------------------------------------------
namespace {

int env_int(const char *name) {
    const char *e = getenv(name);
    return e != nullptr && *e != '\0' ? atoi(e) : TUNE_UNSET;
}

Tuning read_tuning() {
    Tuning t;
    t.gemm_w4 = env_int("TPAMD_GEMM_W4");
    t.gemm_splitk = env_int("TPAMD_GEMM_SPLITK");
    t.gemm_splitk256 = env_int("TPAMD_GEMM_SPLITK256");
    t.gemm_tile = env_int("TPAMD_GEMM_TILE");
    t.gemm_part_x = env_int("TPAMD_GEMM_PART_X");
    t.gemm_stages = env_int("TPAMD_GEMM_STAGES");
    t.skinny_cg = env_int("TPAMD_SKINNY_CG");
    t.skinny_pair = env_int("TPAMD_SKINNY_PAIR");
    t.skinny_resident = env_int("TPAMD_SKINNY_RESIDENT");
    t.w8_split = env_int("TPAMD_W8_SPLIT");
    t.w8_cols = env_int("TPAMD_W8_COLS");
    t.skinny_xlds = env_int("TPAMD_SKINNY_XLDS");
    t.skinny_max_m = env_int("TPAMD_SKINNY_MAX_M");
    t.gemv_rows = env_int("TPAMD_GEMV_ROWS");
    t.attn_splits = env_int("TPAMD_ATTN_SPLITS");
    t.attn_ring = env_int("TPAMD_ATTN_RING");
    t.copy_tile_units = env_int("TPAMD_COPY_TILE_UNITS");
    t.copy_blocks_per_cu = env_int("TPAMD_COPY_BLOCKS_PER_CU");
    t.copy_sort = env_int("TPAMD_COPY_SORT");
    t.copy_nt = env_int("TPAMD_COPY_NT");
    return t;
}

Tuning g_tuning = read_tuning();  // before any entry point can run: the library's load time

}  // namespace

const Tuning &tuning() { return g_tuning; }

// ---- compute units per device -------------------------------------------------------------------------
int device_cus(int dev, int *cus_out) {
    constexpr int MAX_DEV = 64;
    static int cached[MAX_DEV];  // 0 = not asked yet; written once per device with the same value by whoever asks first
    if (dev >= 0 && dev < MAX_DEV && cached[dev] > 0) {
        *cus_out = cached[dev];
        return TPAMD_OK;
    }
    int cus = 0;
    TPAMD_HIP(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
    if (cus <= 0) cus = 1;
    if (dev >= 0 && dev < MAX_DEV) cached[dev] = cus;
    *cus_out = cus;
    return TPAMD_OK;
}

// ---- scratch memory -------------------------------------------------------------------------------------
namespace {

struct Entry {
    int dev;
    hipStream_t stream;
    bool spare;  // set aside for the first capturing stream that needs one; `stream` means nothing until then
    void *ptr;
    size_t bytes;
};
constexpr int LOCKS = 64;  // one lock and one list per device (devices 64 apart would share them)
std::vector<Entry> g_caches[LOCKS];  // list d guarded by splitk_mutex(d)
constexpr int MAX_BUFFERS_PER_DEVICE = 33;  // 32 streams (a framework's stream pool) and the spare

int slot_of(int dev) { return dev >= 0 ? dev % LOCKS : 0; }

}  // namespace

std::mutex &splitk_mutex(int dev) {
    static std::mutex m[LOCKS];
    return m[slot_of(dev)];
}

// The caller holds splitk_mutex(dev) from this call until its launches that use the buffer are enqueued.
// *out = a buffer of at least `need` bytes for work on `stream` of device `dev` (the current device), or NULL: then the
// caller runs its unsplit form. A stream's buffer is allocated at its first use with max(need, reserve) bytes and kept
// until the process ends; streams of one device never share one, so K-split work on different streams cannot meet in
// it. Allocating is not allowed while a stream is being captured, so the first allocation on a device also sets one
// spare buffer aside, and the first capturing stream that has no buffer of its own takes it over (frameworks capture
// on a stream of their own that runs nothing else). NULL comes back when a capturing stream finds no spare, when `need`
// is larger than the stream's buffer, and when the device already has its 33 buffers (32 streams and the spare).
// Inside a StaticScratchScope (noalloc.hip) the library's fixed array is handed out instead.
static int allocate_entry(int dev, hipStream_t stream, bool spare, size_t bytes, void **out) {
    void *ptr = nullptr;
    const hipError_t e = hipMalloc(&ptr, bytes);
    if (e != hipSuccess) {
        (void)hipGetLastError();
        set_error("hipMalloc of %zu bytes of K-split scratch memory failed: %s", bytes, hipGetErrorString(e));
        return TPAMD_ERR_NOMEM;
    }
    g_caches[slot_of(dev)].push_back(Entry{dev, stream, spare, ptr, bytes});
    if (out != nullptr) *out = ptr;
    return TPAMD_OK;
}

int splitk_scratch(int dev, hipStream_t stream, size_t need, size_t reserve, void **out) {
    *out = nullptr;
    if (static_scratch_active()) return static_scratch(dev, need, out);
    int on_device = 0;
    Entry *spare = nullptr;
    for (Entry &e : g_caches[slot_of(dev)]) {
        if (e.dev != dev) continue;
        ++on_device;
        if (e.spare) {
            spare = &e;
            continue;
        }
        if (e.stream == stream) {
            if (e.bytes >= need) *out = e.ptr;
            return TPAMD_OK;
        }
    }
    hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
    TPAMD_HIP(hipStreamIsCapturing(stream, &capturing));
    if (capturing != hipStreamCaptureStatusNone) {
        if (spare != nullptr && spare->bytes >= need) {  // from now on this is the capturing stream's buffer
            spare->spare = false;
            spare->stream = stream;
            *out = spare->ptr;
        }
        return TPAMD_OK;
    }
    if (on_device >= MAX_BUFFERS_PER_DEVICE) return TPAMD_OK;
    const size_t bytes = need > reserve ? need : reserve;
    const int rc = allocate_entry(dev, stream, false, bytes, out);
    if (rc != TPAMD_OK) return rc;
    if (spare == nullptr && on_device + 1 < MAX_BUFFERS_PER_DEVICE) {
        if (allocate_entry(dev, nullptr, true, reserve, nullptr) != TPAMD_OK) set_error("%s", "");  // no spare: captures run unsplit
    }
    return TPAMD_OK;
}

}  // namespace tpamd

using namespace tpamd;

extern "C" void tpamd_tuning_reload(void) { g_tuning = read_tuning(); }

// Gives back the buffer of `stream` on the current device. The caller says that no work that uses it is in flight or
// captured: the stream is synchronised here, then the buffer is freed and its slot is free for another stream.
extern "C" int tpamd_scratch_release(void *stream) {
    int dev = 0;
    TPAMD_HIP(hipGetDevice(&dev));
    void *ptr = nullptr;
    {
        std::lock_guard<std::mutex> hold(splitk_mutex(dev));
        std::vector<Entry> &g_cache = g_caches[slot_of(dev)];
        for (size_t i = 0; i < g_cache.size(); ++i) {
            const Entry &e = g_cache[i];
            if (e.dev == dev && !e.spare && e.stream == static_cast<hipStream_t>(stream)) {
                ptr = e.ptr;
                g_cache.erase(g_cache.begin() + static_cast<long>(i));
                break;
            }
        }
    }
    if (ptr == nullptr) return TPAMD_OK;  // the stream had none
    TPAMD_HIP(hipStreamSynchronize(static_cast<hipStream_t>(stream)));
    TPAMD_HIP(hipFree(ptr));
    return TPAMD_OK;
}

extern "C" int tpamd_scratch_query(void *stream, void **ptr_out, uint64_t *bytes_out) {
    TPAMD_REQUIRE(ptr_out != nullptr && bytes_out != nullptr, "tpamd_scratch_query: null output pointer");
    int dev = 0;
    TPAMD_HIP(hipGetDevice(&dev));
    *ptr_out = nullptr;
    *bytes_out = 0;
    std::lock_guard<std::mutex> hold(splitk_mutex(dev));
    for (const Entry &e : g_caches[slot_of(dev)])
        if (e.dev == dev && !e.spare && e.stream == static_cast<hipStream_t>(stream)) {
            *ptr_out = e.ptr;
            *bytes_out = e.bytes;
        }
    return TPAMD_OK;
}
