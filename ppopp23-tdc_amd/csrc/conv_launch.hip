// Host side of the convolution kernels: KernelId -> compiled function, the static scratch of the entry point that
// allocates nothing, occupancy queries, and the launch itself.
#include <hip/hip_runtime.h>

#include <mutex>

#include "tdc_internal.hpp"

namespace tdc {

// The kernels live in three translation units (conv_staged.hip, conv_stream.hip, conv_wino_stream.hip); each maps the
// KernelIds of its families to its instantiations.
const void *kernel_function(const KernelId &k) {
    return k.family == KernelId::STAGED        ? staged_kernel_function(k)
           : k.family == KernelId::STREAM_WINO ? wino_stream_kernel_function(k)
                                               : stream_kernel_function(k);
}

// ---------------------------------------------------------------------------
// Static scratch for callers that cannot allocate (HIP graph capture, serving loops whose harness forbids
// hipMalloc): the partial tiles and ticket counters of a split across workgroups (tile.ks > 1) in a device array
// that exists from module load to process exit, one copy per GPU.  4 MiB of partial tiles (256 -> 256 @7x7 with four
// slices needs 0.2 MiB, 2048 -> 256 @7x7 with eight 0.4 MiB) and 64 KiB of counters.
// In host code the array's NAME is not a device address; its address on the current device comes from
// hipGetSymbolAddress and is kept per device.
// ---------------------------------------------------------------------------
constexpr size_t kScratchWsBytes = 4u << 20;
constexpr size_t kScratchCtrBytes = 64u << 10;
static __device__ __align__(256) unsigned char scratch[kScratchWsBytes + kScratchCtrBytes];

size_t static_scratch_ws_bytes() { return kScratchWsBytes; }
size_t static_scratch_ctr_bytes() { return kScratchCtrBytes; }

int static_scratch_address(void **ptr_out) {
    constexpr int kMaxDevices = 64;
    static void *per_device[kMaxDevices] = {};
    static std::mutex mtx;
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
    if (dev < 0 || dev >= kMaxDevices) return (int)hipErrorInvalidDevice;
    std::lock_guard<std::mutex> lock(mtx);
    if (!per_device[dev]) {
        void *p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));   // the address of this device's copy
        if (e != hipSuccess) return (int)e;
        if (!p) return (int)hipErrorInvalidSymbol;
        per_device[dev] = p;
    }
    *ptr_out = per_device[dev];
    return 0;
}

__global__ void __launch_bounds__(256) tdc_zero_words_kernel(unsigned *dst, int n) {
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i < n) dst[i] = 0u;
}

int launch_zero_words(unsigned *dst, int n, void *stream) {
    if (n <= 0) return 0;
    hipLaunchKernelGGL(tdc_zero_words_kernel, dim3((n + 255) / 256), dim3(256), 0, (hipStream_t)stream, dst, n);
    return (int)hipGetLastError();
}

// Launch-path probe (tdc_launch_floor_time): same argument block as the convolution kernels, no memory access; every
// wave waits until the constant 100 MHz clock has advanced by `ticks`.
__global__ void __launch_bounds__(1024) tdc_launch_probe_kernel(const ConvKParams p, int ticks) {
    if (ticks <= 0) return;
    const unsigned long long t0 = __builtin_amdgcn_s_memrealtime();
    // (bounded: the clock always advances, and the host refuses more than 100 us)
    while ((long long)(__builtin_amdgcn_s_memrealtime() - t0) < (long long)ticks) __builtin_amdgcn_s_sleep(1);
    if (p.out && threadIdx.x == 0x7fffffff) p.out[0] = 0.0f;   // (never true: keeps the argument block alive)
}

int launch_floor_probe(const ConvKParams &kp, int grid, int block, int spin_ticks, void *stream) {
    hipLaunchKernelGGL(tdc_launch_probe_kernel, dim3(grid), dim3(block), 0, (hipStream_t)stream, kp, spin_ticks);
    return (int)hipGetLastError();
}

int kernel_resources(const void *fn, int block_threads, int dynamic_lds_bytes, int *vgprs, int *static_lds, int *max_threads,
                     int *max_wg_per_cu) {
    hipFuncAttributes attr{};
    hipError_t e = hipFuncGetAttributes(&attr, fn);
    if (e != hipSuccess) return (int)e;
    int blocks = 0;
    e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&blocks, fn, block_threads, (size_t)dynamic_lds_bytes);
    if (e != hipSuccess) return (int)e;
    *vgprs = attr.numRegs;
    *static_lds = (int)attr.sharedSizeBytes;
    *max_threads = attr.maxThreadsPerBlock;
    *max_wg_per_cu = blocks;
    return 0;
}

int prepare_conv_kernel(const void *fn, const Geometry &g) {
    if (!fn) return (int)hipErrorInvalidValue;
    // Dynamic LDS above the 64 KiB default has to be opted into per kernel function.  The attribute belongs to
    // the function, not to the plan, and several plans share one instantiation: always raise it to the whole
    // LDS, so that a later plan with a smaller request cannot lower it under an earlier plan's feet.
    if (g.lds_bytes > 64 * 1024) {
        hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, machine().lds_bytes_per_cu);
        if (e != hipSuccess) return (int)e;
    }
    return 0;
}

int launch_conv(const void *fn, const Geometry &g, const ConvKParams &kp, void *stream) {
    typedef void (*kernel_fn)(const ConvKParams);
    if (!fn) return (int)hipErrorInvalidValue;
    dim3 grid(8 * kp.xcd_chunk), block(g.threads);
    hipLaunchKernelGGL(reinterpret_cast<kernel_fn>(const_cast<void *>(fn)), grid, block,
                       (size_t)g.lds_bytes, (hipStream_t)stream, kp);
    return (int)hipGetLastError();
}

}  // namespace tdc
