// d8_matmul_grad_y_static: Math::MatrixMultiplyGradYGPU for callers that cannot allocate.
//
// dY += Xᵀ·dZ over a long collapsed batch (Deep8's Y1 case, deep8/src/math/MatrixMultiply.cu:381-420)
// has an output of few tiles, so the reduction is cut into pieces whose fp32 partial sums pass through a
// workspace before they are added in a fixed order.  d8_matmul_grad_y takes that workspace from its
// caller.  This variant keeps it in a file-scope device array of D8_STATIC_SCRATCH_BYTES instead, so that
// code under stream capture, serving loops and harnesses that forbid hipMalloc have an entry point that
// neither allocates nor asks them to.
//
// The array's name is a host-side stand-in, not a device address: the address of the device's own copy
// comes from hipGetSymbolAddress, once per device, and only that pointer is handed to kernels.
// Every call on a device shares the device's array: calls that overlap on one device (two streams, two
// host threads) race on the partial sums.  Nothing in it has to start at zero: every partial sum a call
// reads was written by that call's own product kernel earlier on the same stream.
#include <mutex>

#include "common.h"

namespace d8 {

enum { MAX_DEVICES = 64 };

static __device__ __align__(256) unsigned char scratch[D8_STATIC_SCRATCH_BYTES];
static void *scratch_ptr[MAX_DEVICES];  // per device: the address of its copy of `scratch`

int static_scratch_setup() {
    int dev = 0;
    D8_HIP(hipGetDevice(&dev));
    D8_REQUIRE(dev >= 0 && dev < MAX_DEVICES, "static scratch: device %d beyond the %d this library tracks", dev, (int)MAX_DEVICES);
    // one look-up per device, whichever host thread gets here first (the others wait for it)
    static std::once_flag once[MAX_DEVICES];
    static int status[MAX_DEVICES];
    std::call_once(once[dev], [dev] {
        void *p = nullptr;
        const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess) {
            status[dev] = fail((int)e, "static scratch: hipGetSymbolAddress: %s", hipGetErrorString(e));
        } else if (!p || ((size_t)p & 255) != 0) {
            status[dev] = fail(D8_ERR_ARGUMENT, "static scratch: bad device address %p", p);
        } else {
            scratch_ptr[dev] = p;
        }
    });
    return status[dev];
}

}  // namespace d8

using namespace d8;

extern "C" {

int d8_matmul_grad_y_static(int dtype, const void *x, int xb, int xr, int xc, void *dy, int yb, int yr, int yc,
                            const void *dz, void *stream) {
    // (the shape checks are d8_matmul_grad_y's own; a shape it rejects makes the size query return 0)
    const size_t need = d8_matmul_scratch_bytes(dtype, 2, xb, xr, xc, yb, yr, yc);
    D8_REQUIRE(need <= (size_t)D8_STATIC_SCRATCH_BYTES,
               "d8_matmul_grad_y_static: this shape splits its reduction through %zu bytes of partial sums, "
               "the static scratch holds %zu; use d8_matmul_grad_y with a caller-owned scratch",
               need, (size_t)D8_STATIC_SCRATCH_BYTES);
    void *ws = nullptr;
    if (need) {
        if (int rc = static_scratch_setup()) return rc;  // no-op after d8_device_init on this device
        int dev = 0;
        D8_HIP(hipGetDevice(&dev));
        ws = scratch_ptr[dev];
    }
    return d8_matmul_grad_y(dtype, x, xb, xr, xc, dy, yb, yr, yc, dz, ws, need, stream);
}

}  // extern "C"
