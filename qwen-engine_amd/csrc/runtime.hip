// Error text of the C entry points and a query of the build's target.
#include "common.h"
#include <stdarg.h>
#include <stdio.h>

static thread_local char g_error[512] = "";

void qe_set_error(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
}

extern "C" const char* qe_last_error() { return g_error; }

// Compute units of the current device (asked once per device; 256, an MI355X's, if the runtime does not say).
extern "C" int qe_compute_units() {
    static int units[64];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
    if (units[dev] == 0) {
        hipDeviceProp_t prop;
        units[dev] = (hipGetDeviceProperties(&prop, dev) == hipSuccess && prop.multiProcessorCount > 0)
                         ? prop.multiProcessorCount : 256;
    }
    return units[dev];
}

// The float32 mode's attention and matrix products run on the matrix units (attention_f32.hip,
// gemm_f32.hip) unless this is switched off: then on the vector units' kernels, which sum in another
// order (for comparing the two).
int g_qe_matrix_f32 = 1;
extern "C" void qe_use_matrix_f32(int on) { g_qe_matrix_f32 = on; }
