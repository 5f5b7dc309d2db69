// Facts about a device and host objects tied to it, set up once and then reused, so that the launch
// path of every entry point consists of kernel launches and event record / wait calls only (the
// calls a stream capture can record).
#include <mutex>

#include "internal.h"

namespace nnueft_dev {

namespace {

constexpr int kMaxDevices = 64;

struct Slot {
    bool ready = false;
    DeviceInfo info{};
};
Slot g_slots[kMaxDevices];
std::mutex g_mutex;

struct ThreadEvents {
    hipEvent_t ev[kMaxDevices][2] = {};
    // events live until the thread ends; a thread that ends while the runtime is already shutting
    // down must not call into it, so they are left to the runtime
};
thread_local ThreadEvents t_events;

}  // namespace

int device_info(int* device, const DeviceInfo** info) {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
    if (dev < 0 || dev >= kMaxDevices) return NNUEFT_E_UNSUPPORTED;
    Slot& s = g_slots[dev];
    {
        std::lock_guard<std::mutex> lock(g_mutex);
        if (!s.ready) {
            DeviceInfo d{};
            e = hipDeviceGetAttribute(&d.max_lds, hipDeviceAttributeMaxSharedMemoryPerBlock, dev);
            if (e != hipSuccess) return (int)e;
            // older runtimes do not know the attribute: then the count stays unknown (0)
            if (hipDeviceGetAttribute(&d.xcds, hipDeviceAttributeNumberOfXccs, dev) != hipSuccess) {
                d.xcds = 0;
                (void)hipGetLastError();
            }
            e = hipDeviceGetAttribute(&d.cus, hipDeviceAttributeMultiprocessorCount, dev);
            if (e != hipSuccess) return (int)e;
            s.info = d;
            s.ready = true;
        }
    }
    if (device) *device = dev;
    *info = &s.info;
    return 0;
}

int thread_events(int device, hipEvent_t* fork, hipEvent_t* join) {
    if (device < 0 || device >= kMaxDevices) return NNUEFT_E_UNSUPPORTED;
    hipEvent_t* ev = t_events.ev[device];
    for (int i = 0; i < 2; ++i) {
        if (!ev[i]) {
            const hipError_t e = hipEventCreateWithFlags(&ev[i], hipEventDisableTiming);
            if (e != hipSuccess) {
                ev[i] = nullptr;
                return (int)e;
            }
        }
    }
    *fork = ev[0];
    *join = ev[1];
    return 0;
}

}  // namespace nnueft_dev

extern "C" int nnueft_device_xcds(void) {
    const nnueft_dev::DeviceInfo* info = nullptr;
    const int rc = nnueft_dev::device_info(nullptr, &info);
    if (rc) return rc > 0 ? -rc - 1000 : rc;
    return info->xcds;
}
