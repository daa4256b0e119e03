/* device.hip — process-wide state of the library: the environment knobs (read once) and the table of
 * devices that have been set up. Host code only. */
#include <hip/hip_runtime.h>

#include <cstdlib>
#include <cstring>
#include <mutex>

#include "../../include/plow_moe.h"
#include "tuning.h"

const PlowMoeTuning& plow_moe_tuning() {
    static PlowMoeTuning t;
    static std::once_flag once;
    std::call_once(once, [] {
        auto is = [](const char* name, const char* value) {
            const char* e = getenv(name);
            return e && !strcmp(e, value);
        };
        t.w8a8_kernel = is("PLOW_MOE_W8A8_KERNEL", "stream") ? 0 : is("PLOW_MOE_W8A8_KERNEL", "tiled") ? 1 : -1;
        t.tile_waves4 = is("PLOW_MOE_W8A8_TILE_WAVES", "4");
        t.tiled_nt = is("PLOW_MOE_TILED_NT", "0") ? 0 : is("PLOW_MOE_TILED_NT", "1") ? 1 : -1;
        const char* d = getenv("PLOW_MOE_SK_DEPTH");
        t.sk_depth = d ? atoi(d) : 3;
        if (t.sk_depth < 2 || t.sk_depth > 4) t.sk_depth = 3;
        t.sk_glu_regs = is("PLOW_MOE_SK_GLU", "regs");
        t.sk_down_regs = is("PLOW_MOE_SK_DOWN", "regs");
        t.sk_narrow = getenv("PLOW_MOE_SK_NARROW") != nullptr;
        t.a16_regs = is("PLOW_MOE_A16_KERNEL", "regs");
        t.score_tile8 = is("PLOW_MOE_SCORE_KERNEL", "tile8");
        t.score_valu = is("PLOW_MOE_SCORE_KERNEL", "valu");
        t.a16_tiled = !is("PLOW_MOE_A16_TILED", "0");
        t.a16_gemv = !is("PLOW_MOE_A16_GEMV", "0");
        t.a16_tiled_mx = !is("PLOW_MOE_A16_TILED_MX", "0");
        t.a16_down_wide = !is("PLOW_MOE_A16_DOWN_WIDE", "0");
        t.a16_private_rows = !is("PLOW_MOE_A16_PRIVATE_ROWS", "0");
        t.a16_dense_split = !is("PLOW_MOE_A16_DENSE_SPLIT", "0");
        t.gemv_direct = !is("PLOW_MOE_GEMV_DIRECT", "0");
        t.dense_overlap = !is("PLOW_MOE_DENSE_OVERLAP", "0");
        t.form_on_device = !is("PLOW_MOE_FORM_ON_DEVICE", "0");
        t.score_row_narrow = is("PLOW_MOE_SCORE_ROW", "narrow");
    });
    return t;
}

/* Workspace of the entry point that allocates nothing (plow_moe_exec_noalloc). In host code this name
 * is only a handle for hipGetSymbolAddress, never a device address: each GPU holds its own copy, whose
 * address plow_moe_device_setup resolves once per device and keeps in g_scratch_ptr. */
static __device__ __align__(256) unsigned char scratch[PLOW_MOE_STATIC_BYTES];

#define MAX_DEVICES 64
static std::mutex g_dev_mutex;
static uint32_t g_n_cu[MAX_DEVICES]; /* 0 = not set up; written once under the mutex */
static void* g_scratch_ptr[MAX_DEVICES];

int plow_moe_device_setup(int device) {
    if (device < 0 || device >= MAX_DEVICES) return PLOW_MOE_EINVAL;
    std::lock_guard<std::mutex> lock(g_dev_mutex);
    if (g_n_cu[device]) return 0;
    hipDeviceProp_t prop;
    if (hipGetDeviceProperties(&prop, device) != hipSuccess) return PLOW_MOE_EDEVICE;
    if (strncmp(prop.gcnArchName, "gfx950", 6) != 0) return PLOW_MOE_EUNSUPPORTED; /* CDNA4 only */
    int prev = 0;
    if (hipGetDevice(&prev) != hipSuccess || hipSetDevice(device) != hipSuccess) return PLOW_MOE_EDEVICE;
    int rc = plow_moe_route_setup();
    if (!rc) rc = plow_moe_w8a8_setup();
    if (!rc) rc = plow_moe_w8a8_tiled_setup();
    if (!rc) rc = plow_moe_a16_setup();
    void* ptr = nullptr;
    if (!rc && (hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)) != hipSuccess || !ptr)) rc = PLOW_MOE_EDEVICE;
    (void)hipSetDevice(prev);
    if (rc) return rc;
    g_scratch_ptr[device] = ptr; /* this device's copy of the array */
    __atomic_store_n(&g_n_cu[device], (uint32_t)prop.multiProcessorCount, __ATOMIC_RELEASE);
    return 0;
}

void* plow_moe_static_scratch() {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= MAX_DEVICES) return nullptr;
    if (!__atomic_load_n(&g_n_cu[dev], __ATOMIC_ACQUIRE)) return nullptr; /* not set up */
    return g_scratch_ptr[dev];
}

uint32_t plow_moe_n_cu() {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= MAX_DEVICES) return 0u;
    return __atomic_load_n(&g_n_cu[dev], __ATOMIC_ACQUIRE);
}
