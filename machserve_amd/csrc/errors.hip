// Error channel of the extern "C" entry points: a refused call returns non-zero and
// leaves its reason here; and the count of kernels launched.  Role of `check` in
// crates/mach-kernel-sys/src/hip.rs:370.  (Memory, streams and graph capture are torch's: the
// entry points take raw pointers and a stream.)
#include "common.cuh"
#include <cstdarg>
#include <cstdio>

namespace ms {

static thread_local char g_error[512] = "";
static long g_launches = 0;  // kernels this library has launched (asked for by the benchmark's launch count)

void set_error(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
}

int check_launch(const char* what) {
    ++g_launches;
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
        set_error("%s: launch failed: %s", what, hipGetErrorString(e));
        return 2;
    }
    return 0;
}

// Compute units of the current device, asked once (256 if the device will not say).  The products' planners fill
// the chip by this count: two 128x128 blocks a CU, sixteen waves a CU.
int compute_units() {
    static int cus = 0;
    if (cus == 0) {
        int dev = 0, n = 0;
        if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n < 1)
            n = 256;
        (void)hipGetLastError();
        cus = n;
    }
    return cus;
}

}  // namespace ms

extern "C" const char* ms_last_error() { return ms::g_error; }

// Kernels launched by this library so far (every launch goes through check_launch).
extern "C" long ms_launch_count() { return ms::g_launches; }

// Compute units of the current device, as the planners count them.
extern "C" int ms_compute_units() { return ms::compute_units(); }

// Bytes of an element of this build: 2 (bfloat16 or half precision) or 4.
extern "C" int ms_elem_bytes() { return (int)sizeof(ms::elem_t); }
