// Scratch of rnb_hip_gemv_dev_noalloc: a fixed array in the code object, so every GPU that loads the library holds its
// own copy until the process ends and no call ever allocates it.  Host code never uses the array's name as an
// address: it asks the runtime for the device address, once per device, and hands that to the kernels as an argument.
#include "kernels.h"

namespace rnb {

namespace {
static __device__ __align__(256) __attribute__((used)) unsigned char scratch[kStaticScratchBytes];
constexpr int kMaxDevices = 64;
void *g_address[kMaxDevices] = {};
}  // namespace

hipError_t static_scratch_address(int device, void **out) {
    *out = nullptr;
    if (device < 0 || device >= kMaxDevices) return hipErrorInvalidDevice;
    if (g_address[device] == nullptr) {
        void *p = nullptr;
        const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));  // of the current device
        if (e != hipSuccess) return e;
        g_address[device] = p;
    }
    *out = g_address[device];
    return hipSuccess;
}

}  // namespace rnb
