// Device-side pieces shared by the convolution kernels: MFMA wrappers, the multiply-high division, the common
// epilogue of a lane that holds four channels of a pixel, the kernel-argument touch, and the time-stamp macros of
// the profiling build.  Included by conv_staged.hip and conv_stream.hip only.
#pragma once
#include <hip/hip_runtime.h>

#include "tdc_internal.hpp"

#ifndef TDC_TOUCH_KERNARGS
#define TDC_TOUCH_KERNARGS 1
#endif

// Profiling build only (make STAMPS=1): every wave records s_memrealtime (the 100 MHz constant clock, comparable
// across compute units and dies) at the boundaries of its phases and leaves the eight values in a plan-owned buffer,
// [workgroup][wave][8].  The product build compiles none of it.
#ifndef TDC_STAMPS
#define TDC_STAMPS 0
#endif
#if TDC_STAMPS
#define TDC_STAMP_DECL unsigned long long tdc_stamp_[8] = {0, 0, 0, 0, 0, 0, 0, 0}
#define TDC_STAMP(i) tdc_stamp_[i] = __builtin_amdgcn_s_memrealtime()
#define TDC_STAMP_FLUSH(p, wg, wave, lane)                                                             \
    do {                                                                                               \
        if ((p).stamps && (lane) == 0) {                                                               \
            unsigned long long *dst_ = (p).stamps + ((size_t)(wg) * 16 + (wave)) * 8;                   \
            for (int i_ = 0; i_ < 8; ++i_) dst_[i_] = tdc_stamp_[i_];                                   \
        }                                                                                              \
    } while (0)
#else
#define TDC_STAMP_DECL
#define TDC_STAMP(i)
#define TDC_STAMP_FLUSH(p, wg, wave, lane)
#endif

namespace tdc {

typedef float f4_t __attribute__((ext_vector_type(4)));
typedef float f16_t __attribute__((ext_vector_type(16)));
typedef __attribute__((address_space(3))) void *lds_ptr_t;

template <int MF>
struct Mfma;

// v_mfma_f32_32x32x2_f32: A lane l = A[l%32][l/32], B lane l = B[l/32][l%32],
// D vgpr v lane l = D[8*(v/4) + 4*(l/32) + v%4][l%32].
template <>
struct Mfma<32> {
    using acc_t = f16_t;
    static constexpr int NACC = 16;
    static constexpr int KC = 2;
    static __device__ __forceinline__ acc_t run(float a, float b, acc_t c) {
        return __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ int row(int v, int lane) {
        return 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3);
    }
    static __device__ __forceinline__ int col(int lane) { return lane & 31; }
    static __device__ __forceinline__ int ksub(int lane) { return lane >> 5; }
};

// v_mfma_f32_16x16x4_f32: A lane l = A[l%16][l/16], B lane l = B[l/16][l%16],
// D vgpr v lane l = D[4*(l/16) + v][l%16].
template <>
struct Mfma<16> {
    using acc_t = f4_t;
    static constexpr int NACC = 4;
    static constexpr int KC = 4;
    static __device__ __forceinline__ acc_t run(float a, float b, acc_t c) {
        return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ int row(int v, int lane) { return 4 * (lane >> 4) + v; }
    static __device__ __forceinline__ int col(int lane) { return lane & 15; }
    static __device__ __forceinline__ int ksub(int lane) { return lane >> 4; }
};

// TAPS_WINO: 3x3 / stride 1 as Winograd F(2x2,3x3).  A pixel lane holds one 2x2 output tile; per four input
// channels a wave reads the 4x4 input patch of its tile from the SAME zero-haloed LDS window the direct path
// uses, transforms it in registers (V = B^T d B, 32 additions), and feeds 16 MFMAs — one per position of the
// transformed domain, against weights U = G g G^T prepared on the host — where the direct path needs 36 for
// the same four pixels.  The 16 accumulators of a lane are combined at the end (Y = A^T M A, in registers:
// every lane holds all 16 positions of its tile) into the 2x2 outputs.
// TAPS_3x3G: the direct 3x3 loop with its weights read from global memory straight into registers (like the
// Winograd path) instead of being staged in LDS: the LDS then holds input only and a pass can take all input channels.
// (the TAPS_* values themselves are declared next to KernelId)

constexpr int OOB_OFFSET = 0x7ffffff0;  // beyond any buffer: the load returns zero

// Output stores (plain: the lines stay in the die's L2 until the kernel ends).
__device__ __forceinline__ void store_out(float *p, float v) { *p = v; }
__device__ __forceinline__ void store_out(float *p, f4_t v) { *reinterpret_cast<f4_t *>(p) = v; }
typedef float f2_store_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ void store_out(float *p, f2_store_t v) { *reinterpret_cast<f2_store_t *>(p) = v; }

__device__ __forceinline__ int fdiv(int n, const FastDiv &f) {
    return (int)(__umulhi((unsigned)n, f.m) + ((unsigned)n & f.pass));
}

// Epilogue of a lane that holds four consecutive output channels (from ch0) of one pixel: + bias, + residual, ReLU,
// store.  All eight loads are requested before the first value is needed — one memory round trip for the lane
// instead of one per load (written naively, every load sits behind the previous channel's store, which it might alias).
__device__ __forceinline__ void finish_four_channels(const f4_t &acc, int ch0, int N, long long P, long long pix,
                                                     const float *__restrict__ bias, const float *__restrict__ resid,
                                                     int relu, float *__restrict__ out) {
    float bv[4] = {0.0f, 0.0f, 0.0f, 0.0f}, rv[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    if (bias) {
#pragma unroll
        for (int i = 0; i < 4; ++i) bv[i] = bias[min(ch0 + i, N - 1)];
    }
    if (resid) {
#pragma unroll
        for (int i = 0; i < 4; ++i) rv[i] = resid[(long long)min(ch0 + i, N - 1) * P + pix];
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        if (ch0 + i >= N) continue;
        float val = acc[i] + bv[i];
        val += rv[i];
        if (relu) val = fmaxf(val, 0.0f);
        store_out(out + ((long long)(ch0 + i) * P + pix), val);
    }
}

// The kernel arguments (about 530 bytes) are read through the scalar cache.  Left alone, the compiler fetches them in
// several dependent batches, and every batch that touches a cache line for the first time costs a round trip to L2
// before the first request can go out.  Touch every line of the argument block at once: whatever order the compiler
// then loads the values in, it hits the scalar cache.
__device__ __forceinline__ void touch_kernel_arguments() {
    if constexpr (TDC_TOUCH_KERNARGS) {
        static_assert(sizeof(ConvKParams) > 8 * 64 && sizeof(ConvKParams) <= 9 * 64, "touch exactly the lines of the argument block");
        const auto kargs = __builtin_amdgcn_kernarg_segment_ptr();
        unsigned t0, t1, t2, t3, t4, t5, t6, t7, t8;
        asm volatile(
            "s_load_dword %0, %9, 0x0\n\ts_load_dword %1, %9, 0x40\n\ts_load_dword %2, %9, 0x80\n\t"
            "s_load_dword %3, %9, 0xc0\n\ts_load_dword %4, %9, 0x100\n\ts_load_dword %5, %9, 0x140\n\t"
            "s_load_dword %6, %9, 0x180\n\ts_load_dword %7, %9, 0x1c0\n\ts_load_dword %8, %9, 0x200\n\ts_waitcnt lgkmcnt(0)"
            : "=&s"(t0), "=&s"(t1), "=&s"(t2), "=&s"(t3), "=&s"(t4), "=&s"(t5), "=&s"(t6), "=&s"(t7), "=&s"(t8)
            : "s"(kargs)
            : "memory");
    }
}

// Where image `img` of the batch starts in the input, the output and the residual.  A compute unit has ONE scalar
// unit for all its waves, and in the streamed kernels every wave's scalar prologue sits on the path to its first
// memory request (16 waves x ~130 scalar instructions is most of a microsecond), so the 64-bit stride products — a
// quarter of that prologue — are skipped for the first image, which is the only one in a single-image launch.
struct ImageBase {
    const float *in;
    float *out;
    const float *resid;
};
__device__ __forceinline__ ImageBase image_base(const ConvKParams &p, int img) {
    ImageBase b{p.in, p.out, p.resid};
    if (__builtin_expect(img != 0, 0)) {   // (wave-uniform: a scalar branch)
        b.in += (long long)img * p.in_bstride;
        b.out += (long long)img * p.out_bstride;
        if (b.resid) b.resid += (long long)img * p.resid_bstride;
    }
    return b;
}

}  // namespace tdc
