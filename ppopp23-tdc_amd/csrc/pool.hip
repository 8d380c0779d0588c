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

// Every kernel takes batch strides in floats, so a tensor may be a channel slice of a wider
// buffer (DenseNet's growing concatenation is written in place).

// mode 0 = max (padding never wins), 1 = average over the full k*k window
// including padding zeros (count_include_pad, which equals PyTorch's AvgPool2d
// default and is irrelevant when pad == 0).
__global__ void __launch_bounds__(256) pool2d_kernel(const float *__restrict__ in, long long in_bs,
                                                     float *__restrict__ out, long long out_bs, int C, int H, int W,
                                                     int Ho, int Wo, int k, int stride, int pad, int mode) {
    // grid = (pixel blocks, channels, batch): no 64-bit division, one 32-bit division per thread
    const int pix = blockIdx.x * blockDim.x + threadIdx.x;
    if (pix >= Ho * Wo) return;
    const int c = blockIdx.y, b = blockIdx.z;
    const int oy = pix / Wo, ox = pix - oy * Wo;
    const float *src = in + b * in_bs + (long long)c * H * W;
    float acc = mode == 0 ? -FLT_MAX : 0.0f;
    const int iy0 = oy * stride - pad, ix0 = ox * stride - pad;
    for (int r = 0; r < k; ++r) {
        const int iy = iy0 + r;
        if ((unsigned)iy >= (unsigned)H) continue;
        const float *row = src + iy * W;
        for (int s = 0; s < k; ++s) {
            const int ix = ix0 + s;
            if ((unsigned)ix >= (unsigned)W) continue;
            const float v = row[ix];
            acc = mode == 0 ? fmaxf(acc, v) : acc + v;
        }
    }
    if (mode == 1) acc *= 1.0f / (float)(k * k);
    out[b * out_bs + (long long)c * Ho * Wo + pix] = acc;
}

// The same for the window sizes the networks use (3x3 max pool after the stem, 2x2 average pools in DenseNet's transitions),
// without branches: every load of the window is issued at once.  An index outside the image is clamped into it; for a max pool
// the clamped element lies inside the same window (pad < K), so the duplicate changes nothing, and the average variant is only
// launched when every window lies inside the image.  Same visiting order, so the results equal the general kernel's bit for bit.
template <int K, int MODE>
__global__ void __launch_bounds__(256) pool2d_fixed_kernel(const float *__restrict__ in, long long in_bs,
                                                           float *__restrict__ out, long long out_bs, int H, int W, int Ho,
                                                           int Wo, int stride, int pad) {
    const int pix = blockIdx.x * blockDim.x + threadIdx.x;
    if (pix >= Ho * Wo) return;
    const int c = blockIdx.y, b = blockIdx.z;
    const int oy = pix / Wo, ox = pix - oy * Wo;
    const float *src = in + b * in_bs + (long long)c * H * W;
    const int iy0 = oy * stride - pad, ix0 = ox * stride - pad;
    float v[K][K];
#pragma unroll
    for (int r = 0; r < K; ++r) {
        const int iy = min(max(iy0 + r, 0), H - 1);
#pragma unroll
        for (int s = 0; s < K; ++s) v[r][s] = src[iy * W + min(max(ix0 + s, 0), W - 1)];
    }
    float acc = MODE == 0 ? -FLT_MAX : 0.0f;
#pragma unroll
    for (int r = 0; r < K; ++r)
#pragma unroll
        for (int s = 0; s < K; ++s) acc = MODE == 0 ? fmaxf(acc, v[r][s]) : acc + v[r][s];
    if (MODE == 1) acc *= 1.0f / (float)(K * K);
    out[b * out_bs + (long long)c * Ho * Wo + pix] = acc;
}

// Global average pool: one wave per plane, lanes stride over the H*W pixels, shuffle reduction.
__global__ void __launch_bounds__(256) global_avgpool_kernel(const float *__restrict__ in, long long in_bs,
                                                             float *__restrict__ out, long long out_bs, int B, int C,
                                                             int HW) {
    const int wave = (blockIdx.x * blockDim.x + threadIdx.x) >> 6;
    const int lane = threadIdx.x & 63;
    if (wave >= B * C) return;
    const int b = wave / C, c = wave - b * C;
    const float *src = in + b * in_bs + (long long)c * HW;
    float acc = 0.0f;
    for (int i = lane; i < HW; i += 64) acc += src[i];
    for (int off = 32; off > 0; off >>= 1) acc += __shfl_down(acc, off, 64);
    if (lane == 0) out[b * out_bs + c] = acc / (float)HW;
}

// Copy [B, C, HW] between (possibly strided) tensors — channel concatenation (the reference's concate
// kernel, 2080Ti-evaluation/EndToEnd/densenet121-tk/src/Conv.cu:126-155).
__global__ void __launch_bounds__(256) copy_channels_kernel(const float *__restrict__ in, long long in_bs,
                                                            float *__restrict__ out, long long out_bs, int B, int C,
                                                            int HW) {
    const long long per = (long long)C * HW;
    const long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= per * B) return;
    const long long b = idx / per;
    const long long rem = idx - b * per;
    out[b * out_bs + rem] = in[b * in_bs + rem];
}

// Inference-mode BatchNorm (+ReLU) in front of a convolution: out = max(in*scale[c] + shift[c], 0).
// DenseNet normalises the concatenated features separately for every consumer
// (inference/densenet_inet_tt.py:66-70), so it cannot be folded into the producer.
__global__ void __launch_bounds__(256) affine_kernel(const float *__restrict__ in, long long in_bs,
                                                     float *__restrict__ out, long long out_bs,
                                                     const float *__restrict__ scale, const float *__restrict__ shift,
                                                     int B, int C, int HW, int relu) {
    const long long per = (long long)C * HW;
    const long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= per * B) return;
    const long long b = idx / per;
    const long long rem = idx - b * per;
    const int c = (int)(rem / HW);
    float v = in[b * in_bs + rem] * scale[c] + shift[c];
    if (relu) v = fmaxf(v, 0.0f);
    out[b * out_bs + rem] = v;
}

static unsigned blocks_for(long long total) { return (unsigned)((total + 255) / 256); }

int launch_pool2d(const float *in, long long in_bs, float *out, long long out_bs, int B, int C, int H, int W, int Ho,
                  int Wo, int k, int stride, int pad, int mode, void *stream) {
    if (C > 65535 || B > 65535) return (int)hipErrorInvalidValue;
    const dim3 grid(blocks_for((long long)Ho * Wo), C, B);
    const bool inside = (long long)(Ho - 1) * stride - pad + k <= H && (long long)(Wo - 1) * stride - pad + k <= W;
    if (mode == 0 && k == 3 && pad < 3 && H >= 1 && W >= 1)
        hipLaunchKernelGGL((pool2d_fixed_kernel<3, 0>), grid, dim3(256), 0, (hipStream_t)stream, in, in_bs, out, out_bs, H, W,
                           Ho, Wo, stride, pad);
    else if (mode == 1 && k == 2 && pad == 0 && inside)
        hipLaunchKernelGGL((pool2d_fixed_kernel<2, 1>), grid, dim3(256), 0, (hipStream_t)stream, in, in_bs, out, out_bs, H, W,
                           Ho, Wo, stride, pad);
    else
        hipLaunchKernelGGL(pool2d_kernel, grid, dim3(256), 0, (hipStream_t)stream, in, in_bs, out, out_bs, C, H, W, Ho, Wo, k,
                           stride, pad, mode);
    return (int)hipGetLastError();
}

int launch_global_avgpool(const float *in, long long in_bs, float *out, long long out_bs, int B, int C, int HW,
                          void *stream) {
    hipLaunchKernelGGL(global_avgpool_kernel, dim3((unsigned)((B * C + 3) / 4)), dim3(256), 0, (hipStream_t)stream, in,
                       in_bs, out, out_bs, B, C, HW);
    return (int)hipGetLastError();
}

int launch_copy_channels(const float *in, long long in_bs, float *out, long long out_bs, int B, int C, int HW,
                         void *stream) {
    hipLaunchKernelGGL(copy_channels_kernel, dim3(blocks_for((long long)B * C * HW)), dim3(256), 0, (hipStream_t)stream,
                       in, in_bs, out, out_bs, B, C, HW);
    return (int)hipGetLastError();
}

int launch_affine(const float *in, long long in_bs, float *out, long long out_bs, const float *scale, const float *shift,
                  int B, int C, int HW, int relu, void *stream) {
    hipLaunchKernelGGL(affine_kernel, dim3(blocks_for((long long)B * C * HW)), dim3(256), 0, (hipStream_t)stream, in, in_bs,
                       out, out_bs, scale, shift, B, C, HW, relu);
    return (int)hipGetLastError();
}

}  // namespace tdc
