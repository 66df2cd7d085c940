// The SiLU lookup table as a device constant, and the host accessor that hands kernels its device address.
#include <atomic>

#include "scmx_common.h"
#include "silu_table.h"

namespace scmx {

// Not declared const: a const object at namespace scope has internal linkage and, with no device code in this file
// referring to it, would be dropped from the device image (kernels only ever read it).
__device__ silu_ce::Table g_silu_table = silu_ce::make();

// Device address of the table on the current device (every device holds its own copy of the constant).
const uint16_t* silu_table_device() {
    static std::atomic<const uint16_t*> cached[64];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return nullptr;
    const uint16_t* p = cached[dev].load(std::memory_order_acquire);
    if (!p) {
        void* addr = nullptr;
        if (hipGetSymbolAddress(&addr, HIP_SYMBOL(g_silu_table)) != hipSuccess) return nullptr;
        p = reinterpret_cast<const uint16_t*>(addr);
        cached[dev].store(p, std::memory_order_release);
    }
    return p;
}

}  // namespace scmx
