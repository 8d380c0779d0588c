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

// Kernels are launched through their module function handle with the argument block handed over as ONE buffer
// (hipModuleLaunchKernel + HIP_LAUNCH_PARAM_BUFFER_POINTER): the host side of a launch is what bounds back-to-back
// small kernels on a stream, and this form costs the host 0.15-0.2 us less per launch than the <<<>>> form, which
// marshals the arguments one by one.  The handle belongs to the device that was current when it was looked up.
static int launch_with_buffer(void *handle, unsigned grid, unsigned block, unsigned lds, void *stream, void *args, size_t bytes) {
    void *extra[] = {HIP_LAUNCH_PARAM_BUFFER_POINTER, args, HIP_LAUNCH_PARAM_BUFFER_SIZE, &bytes, HIP_LAUNCH_PARAM_END};
    return (int)hipModuleLaunchKernel((hipFunction_t)handle, grid, 1, 1, block, 1, 1, lds, (hipStream_t)stream, nullptr, extra);
}

int launch_floor_probe_handle(void **handle_out) {
    hipFunction_t f = nullptr;
    hipError_t e = hipGetFuncBySymbol(&f, reinterpret_cast<const void *>(tdc_launch_probe_kernel));
    *handle_out = (void *)f;
    return (int)e;
}

int launch_floor_probe(void *handle, const ConvKParams &kp, int grid, int block, int spin_ticks, void *stream) {
    struct {
        ConvKParams kp;
        int ticks;
    } args{kp, spin_ticks};
    static_assert(offsetof(decltype(args), ticks) == sizeof(ConvKParams), "argument layout of tdc_launch_probe_kernel");
    return launch_with_buffer(handle, (unsigned)grid, (unsigned)block, 0, stream, &args, offsetof(decltype(args), ticks) + sizeof(int));
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

int prepare_conv_kernel(const void *fn, const Geometry &g, void **handle_out) {
    if (!fn) return (int)hipErrorInvalidValue;
    *handle_out = nullptr;
    // Dynamic LDS above the 64 KiB default has to be opted into per kernel function.  The attribute belongs to
    // the function, not to the plan, and several plans share one instantiation: always raise it to the whole
    // LDS, so that a later plan with a smaller request cannot lower it under an earlier plan's feet.
    if (g.lds_bytes > 64 * 1024) {
        hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, machine().lds_bytes_per_cu);
        if (e != hipSuccess) return (int)e;
    }
    hipFunction_t f = nullptr;
    hipError_t e = hipGetFuncBySymbol(&f, fn);
    if (e != hipSuccess) return (int)e;
    *handle_out = (void *)f;
    return 0;
}

int launch_conv(void *handle, const Geometry &g, const ConvKParams &kp, void *stream) {
    if (!handle) return (int)hipErrorInvalidValue;
    return launch_with_buffer(handle, 8u * (unsigned)kp.xcd_chunk, (unsigned)g.threads, (unsigned)g.lds_bytes, stream,
                              const_cast<ConvKParams *>(&kp), sizeof(ConvKParams));
}

}  // namespace tdc
