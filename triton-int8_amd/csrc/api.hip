// Version / error / set-up entry points of libti8.
#include <mutex>
#include "ti8_common.h"

namespace ti8 {
char* err_buf() {
    static thread_local char buf[512] = {0};
    return buf;
}

static thread_local int last_gemm_kernel = TI8_KERNEL_NONE;
void note_gemm_kernel(int kind, int bm, int bn, int epi) {
    last_gemm_kernel = kind | (epi << 8) | ((bm / 64) << 16) | ((bn / 64) << 20);
}

int device_cu_count() {
    constexpr int MAX_DEV = 64;
    static std::atomic<int> count[MAX_DEV];
    const int dev = current_device() & (MAX_DEV - 1);
    int n = count[dev].load(std::memory_order_relaxed);
    if (n == 0) {
        hipDeviceProp_t prop;
        n = (hipGetDeviceProperties(&prop, current_device()) == hipSuccess && prop.multiProcessorCount > 0) ? prop.multiProcessorCount : 256;
        count[dev].store(n, std::memory_order_relaxed);
    }
    return n;
}
}  // namespace ti8

extern "C" int ti8_version(void) { return 300; }
extern "C" const char* ti8_last_error(void) { return ti8::err_buf(); }
extern "C" const char* ti8_arch(void) { return "gfx950"; }
extern "C" int ti8_last_gemm_kernel(void) { return ti8::last_gemm_kernel; }

extern "C" int ti8_init(void) {
    using namespace ti8;
    (void)device_cu_count();
    if (int e = init_gemm_kernels()) return e;
    if (int e = init_skinny_kernels()) return e;
    if (int e = init_fwht_kernels()) return e;
    if (int e = init_quant_scratch()) return e;
    // last: a device that refuses the persistent kernel's 160 KiB of LDS is not an error (the one-tile kernel serves
    // its shapes), but the message says so
    return init_chain_kernel();
}
