// Device facts the launchers size their grids and LDS budgets by.
#include "lk_common.h"

#include <atomic>
#include <cstdlib>
#include <mutex>

const LkDevice& lk_device() {
    // One entry per visible device would be the general form; every launcher here runs on the
    // current device and the library is used one process per GPU, so the first query is kept.
    static LkDevice dev{0, 0};
    static std::once_flag once;
    std::call_once(once, [] {
        int id = 0;
        (void)hipGetDevice(&id);
        int cus = 0, lds = 0;
        if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, id) != hipSuccess || cus <= 0) cus = 256;
        if (hipDeviceGetAttribute(&lds, hipDeviceAttributeMaxSharedMemoryPerBlock, id) != hipSuccess || lds <= 0) lds = 64 * 1024;
        (void)hipGetLastError();
        dev.cus = cus;
        dev.lds_bytes = lds;
    });
    return dev;
}

extern "C" int lk_device_info(int* abi_version, int* compute_units, int* lds_bytes, int* wave_size) {
    const LkDevice& d = lk_device();
    if (abi_version) *abi_version = 1;
    if (compute_units) *compute_units = d.cus;
    if (lds_bytes) *lds_bytes = d.lds_bytes;
    if (wave_size) *wave_size = LK_WAVE;
    return LK_OK;
}

// ---------------------------------------------------------------- environment knobs
namespace {
std::atomic<unsigned> g_tune_epoch{1};
}

unsigned lk_tune_epoch() { return g_tune_epoch.load(std::memory_order_relaxed); }

int lk_tune_read(LkTuneSite& site) {
    const unsigned now = g_tune_epoch.load(std::memory_order_acquire);
    const char* v = getenv(site.name);
    site.value = v ? atoi(v) : 0;
    site.epoch = now;   // two threads racing here write the same pair
    return site.value;
}

extern "C" void lk_tune_refresh(void) { g_tune_epoch.fetch_add(1, std::memory_order_acq_rel); }
