// nnueft_double_fwd for callers that cannot allocate: the scratch memory of the L2-blocked gather
// lives in a fixed array inside the library instead of a workspace argument.
#include <mutex>

#include "internal.h"

namespace {

// Holds pair order, keys and per-workgroup histograms of the pair sort for 2 * 65536 index lists
// over a table of up to 63 blocks (a 24576-row table has 32).
constexpr size_t kScratchBytes = (size_t)2 << 20;

// One copy per GPU the library runs on, from the first use there until the process ends.  In host
// code this name only stands for the symbol; the memory is reached through the address
// hipGetSymbolAddress returns on each device.
static __device__ __align__(256) unsigned char scratch[kScratchBytes];

constexpr int kMaxDevices = 64;
void* g_scratch_ptr[kMaxDevices];
std::mutex g_scratch_mutex;

// Address of the current device's copy of `scratch`, looked up once per device with that device current.
int scratch_of_current_device(void** out) {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
    if (dev < 0 || dev >= kMaxDevices) return NNUEFT_E_UNSUPPORTED;
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void* p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return (int)e;
        if (!p) return NNUEFT_E_SCRATCH;
        g_scratch_ptr[dev] = p;
    }
    *out = g_scratch_ptr[dev];
    return 0;
}

}  // namespace

extern "C" int nnueft_double_fwd_noalloc(const float* us, const float* them, const int32_t* widx,
                                         const int32_t* bidx, const int64_t* psqt_idx, const float* W,
                                         const float* bias, float max_act, float* l0, float* wpsqt, float* bpsqt,
                                         float* saved, int B, int K, int R, int L1, int n_psqt, void* stream) {
    if (B < 0 || K <= 0 || R <= 0 || L1 <= 0 || (L1 & 1) || n_psqt < 0) return NNUEFT_E_ARG;
    if (B == 0) return 0;
    // the L2-blocked path's scratch is what has to fit (the LDS-tiled path is taken when its lists fit too)
    const size_t need = nnueft_blocked::pair_sort_workspace(B, R, 0);
    if (need == 0) return NNUEFT_E_ARG;
    if (need > kScratchBytes) return NNUEFT_E_SCRATCH;
    void* ptr = nullptr;
    const int rc = scratch_of_current_device(&ptr);
    if (rc) return rc;
    // every word of the scratch a call reads it has written before (keys, histograms, order are
    // each filled completely for the call's own sizes), so nothing has to start at zero
    return nnueft_double_fwd(us, them, widx, bidx, psqt_idx, W, bias, max_act, l0, wpsqt, bpsqt, saved, B, K, R, L1,
                             n_psqt, ptr, kScratchBytes, stream);
}
