// Pooling kernels for the whole-network graphs: the layers between Tucker
// convolutions in the reference's networks (max pool after the stem, average
// pools before the classifier and in DenseNet transitions;
// inference/resnet_inet_tt.py:323,334,384,391 and the cuDNN wrappers of
// 2080Ti-evaluation/EndToEnd/resnet18-tk/src/Pool.cu:8-49).  HBM-bound,
// one thread per output element, coalesced along the output row.
#include <hip/hip_runtime.h>

#include <cfloat>

#include "tdc_internal.hpp"

namespace tdc {

// mode 0 = max (padding never wins), 1 = average over the full k*k window
// including padding zeros (count_include_pad, which equals PyTorch's AvgPool2d
// default and is irrelevant when pad == 0).
__global__ void __launch_bounds__(256) pool2d_kernel(const float *__restrict__ in, float *__restrict__ out,
                                                     int planes, int H, int W, int Ho, int Wo, int k, int stride,
                                                     int pad, int mode) {
    const long long total = (long long)planes * Ho * Wo;
    const long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= total) return;
    const int ox = (int)(idx % Wo);
    const long long t = idx / Wo;
    const int oy = (int)(t % Ho);
    const long long pl = t / Ho;
    const float *src = in + pl * H * W;
    float acc = mode == 0 ? -FLT_MAX : 0.0f;
    for (int r = 0; r < k; ++r) {
        const int iy = oy * stride - pad + r;
        if (iy < 0 || iy >= H) continue;
        for (int s = 0; s < k; ++s) {
            const int ix = ox * stride - pad + s;
            if (ix < 0 || ix >= W) continue;
            const float v = src[iy * W + ix];
            acc = mode == 0 ? fmaxf(acc, v) : acc + v;
        }
    }
    if (mode == 1) acc *= 1.0f / (float)(k * k);
    out[idx] = acc;
}

// Global average pool: one wave per plane, lanes stride over the H*W pixels, DPP-free shuffle reduction.
__global__ void __launch_bounds__(256) global_avgpool_kernel(const float *__restrict__ in, float *__restrict__ out,
                                                             int planes, int HW) {
    const int wave = (blockIdx.x * blockDim.x + threadIdx.x) >> 6;
    const int lane = threadIdx.x & 63;
    if (wave >= planes) return;
    const float *src = in + (long long)wave * HW;
    float acc = 0.0f;
    for (int i = lane; i < HW; i += 64) acc += src[i];
    for (int off = 32; off > 0; off >>= 1) acc += __shfl_down(acc, off, 64);
    if (lane == 0) out[wave] = acc / (float)HW;
}

// Copy [B, C, HW] into channels [c0, c0+C) of a [B, Ctot, HW] buffer (DenseNet concatenation;
// the reference's concate kernel, 2080Ti-evaluation/EndToEnd/densenet121-tk/src/Conv.cu:126-155).
__global__ void __launch_bounds__(256) copy_channels_kernel(const float *__restrict__ in, float *__restrict__ out,
                                                            int B, int C, int HW, int Ctot, int c0) {
    const long long total = (long long)B * C * HW;
    const long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= total) return;
    const long long per = (long long)C * HW;
    const long long b = idx / per;
    const long long rem = idx - b * per;
    out[b * (long long)Ctot * HW + (long long)c0 * HW + rem] = in[idx];
}

int launch_pool2d(const float *in, float *out, int planes, int H, int W, int Ho, int Wo, int k, int stride, int pad,
                  int mode, void *stream) {
    const long long total = (long long)planes * Ho * Wo;
    const unsigned blocks = (unsigned)((total + 255) / 256);
    hipLaunchKernelGGL(pool2d_kernel, dim3(blocks), dim3(256), 0, (hipStream_t)stream, in, out, planes, H, W, Ho, Wo, k,
                       stride, pad, mode);
    return (int)hipGetLastError();
}

int launch_global_avgpool(const float *in, float *out, int planes, int HW, void *stream) {
    const unsigned blocks = (unsigned)((planes + 3) / 4);  // 4 waves per block
    hipLaunchKernelGGL(global_avgpool_kernel, dim3(blocks), dim3(256), 0, (hipStream_t)stream, in, out, planes, HW);
    return (int)hipGetLastError();
}

int launch_copy_channels(const float *in, float *out, int B, int C, int HW, int Ctot, int c0, void *stream) {
    const long long total = (long long)B * C * HW;
    const unsigned blocks = (unsigned)((total + 255) / 256);
    hipLaunchKernelGGL(copy_channels_kernel, dim3(blocks), dim3(256), 0, (hipStream_t)stream, in, out, B, C, HW, Ctot, c0);
    return (int)hipGetLastError();
}

}  // namespace tdc
