// sfno_sht_forward_static: RealSHT.forward for callers that cannot allocate device memory (code under HIP graph
// capture, serving loops, harnesses that forbid hipMalloc).  The Fourier buffer and the spectral-layout buffer that
// sfno_sht_forward takes as a caller-provided workspace live here in one file-scope device array instead.
//
// Every GPU the library runs on holds its own copy of the array, at its own address, until the process ends.  The
// array's name is a host-side handle, not a device address: host code asks the runtime for the address once per device
// (static_scratch_prepare, called by sfno_sht_plan_create with the plan's device current) and from then on passes that
// address, never the name, to the kernels.
#include <mutex>

#include "sfno_internal.h"

namespace {

static __device__ __align__(256) unsigned char scratch[SFNO_STATIC_SCRATCH_BYTES];

constexpr int kMaxDevices = 64;
std::mutex g_mutex;
void* g_scratch[kMaxDevices] = {};      // device address of `scratch` on each device, null until prepared
int g_status[kMaxDevices] = {};         // 0 = not asked yet, 1 = address known, -1 = the runtime refused

}  // namespace

namespace sfno {

int static_scratch_prepare() {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return SFNO_EHIP;
    std::lock_guard<std::mutex> lock(g_mutex);
    if (g_status[dev] == 1) return SFNO_OK;
    void* ptr = nullptr;
    if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)) != hipSuccess || !ptr) {
        (void)hipGetLastError();
        g_status[dev] = -1;
        return SFNO_EHIP;
    }
    g_scratch[dev] = ptr;
    g_status[dev] = 1;
    return SFNO_OK;
}

}  // namespace sfno

extern "C" int sfno_sht_forward_static(const sfno_sht_plan* p, const float* x, void* coeffs, int64_t rows, void* stream) {
    if (!p || !x || !coeffs || rows < 1) return SFNO_EINVAL;
    if (p->device < 0 || p->device >= kMaxDevices) return SFNO_EINVAL;
    const size_t need = sfno_sht_workspace_bytes(p, rows);
    if (need == 0) return SFNO_EINVAL;
    if (need > (size_t)SFNO_STATIC_SCRATCH_BYTES) return SFNO_EWORKSPACE;     // this many rows of this grid do not fit the array
    void* ptr;
    {
        std::lock_guard<std::mutex> lock(g_mutex);
        ptr = g_status[p->device] == 1 ? g_scratch[p->device] : nullptr;
    }
    if (!ptr) return SFNO_EHIP;          // the address look-up at plan creation failed on this device
    // Nothing in the buffers has to start at zero: the longitude kernel writes every element of the Fourier buffer it
    // owns (padding columns included), the Legendre kernel every element of the spectral layout that the layout pass reads.
    return sfno_sht_forward(p, x, coeffs, rows, ptr, (size_t)SFNO_STATIC_SCRATCH_BYTES, stream);
}
