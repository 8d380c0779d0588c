// Direct convolution as an implicit GEMM on the gfx950 fp32 matrix cores.
//
//   out[n][p] = sum_{c,r,s} w[n][c][r][s] * in[c][iy(p,r)][ix(p,s)]
//
// is computed as  D[M = out channels][N = flat output pixels] += A[M][K] * B[K][N]
// with K running over (input channel, filter tap).  A (weights) is pre-packed on
// the host in exactly the per-lane order the MFMA instruction wants and is
// streamed from L2 with one coalesced 256-byte load per wave per K-step.  B
// (input) is staged once per workgroup into LDS as raw rows with a zero halo
// ([channel][row][col], the same slab-plus-halo idea as the reference's
// load_input_2_shared_memory, 2080Ti-evaluation/TDC-LAYERS-ORACLE/
// template_benchmark_cudnn.template:340-363,377-389), and each K-step reads it
// with one conflict-free ds_read_b32: the 32 (or 16) pixel lanes of an MFMA
// column block read consecutive words of one row, shifted by the tap.
//
// Differences from the reference kernel (template_benchmark_cudnn.template:365-402):
//   * lanes index PIXELS (coalesced stores, conflict-free LDS), output channels
//     live in the MFMA accumulator rows; the reference maps lane -> channel and
//     broadcasts one LDS word to the whole warp;
//   * the split over input-channel slabs (the reference's TC / atomicAdd into a
//     pre-zeroed output) happens across the wavefronts of ONE workgroup and is
//     reduced through LDS in a fixed order: no atomics, no pre-zeroing,
//     bit-reproducible;
//   * pixels are tiled as a flat index over Ho*Wo, so ragged edges cost at most
//     one partial MFMA block per layer instead of one per row;
//   * bias, residual add and ReLU are fused into the store.
#include <hip/hip_runtime.h>

#include "tdc_internal.hpp"

namespace tdc {

typedef float f4_t __attribute__((ext_vector_type(4)));
typedef float f16_t __attribute__((ext_vector_type(16)));

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

enum : int { TAPS_GENERIC = 0, TAPS_1x1 = 1, TAPS_3x3 = 9 };

// Copy input channels [c0, c0+CCH) x rows [iy0, iy0+nrows) into LDS as
// [channel][row][RS] with zeros for the halo and for channels >= C.  One wave
// handles one channel at a time; its lanes cover as many whole rows as fit in
// 64 lanes (narrow images) or 64-column pieces of one row (wide images).
__device__ __forceinline__ void stage_chunk(const ConvKParams &p, const float *__restrict__ in,
                                            float *__restrict__ lds, int c0, int iy0, int nrows,
                                            int wave, int nwaves, int lane) {
    int rpp, lrow, lcol, cpasses;
    bool lane_on;
    if (p.RS <= 64) {
        rpp = 64 / p.RS;
        lrow = lane / p.RS;
        lcol = lane - lrow * p.RS;
        cpasses = 1;
        lane_on = lane < rpp * p.RS;
    } else {
        rpp = 1;
        lrow = 0;
        lcol = lane;
        cpasses = (p.RS + 63) >> 6;
        lane_on = true;
    }
    const int HW = p.H * p.W;
    for (int cl = wave; cl < p.CCH; cl += nwaves) {
        const int c = c0 + cl;
        const bool cok = c < p.C;
        const float *src = in + (long long)(cok ? c : 0) * HW;
        float *dst = lds + cl * p.CS;
#pragma unroll 4
        for (int rbase = 0; rbase < nrows; rbase += rpp) {
            const int row = rbase + lrow;
            const int iy = iy0 + row;
            const bool rok = cok && iy >= 0 && iy < p.H;
            for (int cp = 0; cp < cpasses; ++cp) {
                const int col = lcol + (cp << 6);
                const int ix = col - p.PL;
                const bool active = lane_on && row < nrows && col < p.RS;
                float v = 0.0f;
                if (active && rok && ix >= 0 && ix < p.W) v = src[iy * p.W + ix];
                if (active) dst[row * p.RS + col] = v;
            }
        }
    }
}

template <int MF, int MB, int NB, int TAPS, int MAXW>
__global__ void __launch_bounds__(MAXW * 64) tdc_conv_mfma_kernel(const ConvKParams p) {
    using M = Mfma<MF>;
    using acc_t = typename M::acc_t;
    constexpr int KC = M::KC;
    constexpr int NACC = M::NACC;
    extern __shared__ float lds[];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int nwaves = blockDim.x >> 6;
    const int wk = wave % p.WK;
    const int wn = (wave / p.WK) % p.WN;
    const int wm = wave / (p.WK * p.WN);

    const int PT = MF * NB * p.WN;
    const int MT = MF * MB * p.WM;
    const int p0 = blockIdx.x * PT;
    const int m0 = blockIdx.y * MT;
    const float *__restrict__ in = p.in + (long long)blockIdx.z * p.in_bstride;
    float *__restrict__ out = p.out + (long long)blockIdx.z * p.out_bstride;
    const float *__restrict__ resid =
        p.resid ? p.resid + (long long)blockIdx.z * p.out_bstride : nullptr;

    const int plast = min(p0 + PT, p.P) - 1;
    const int oy0 = p0 / p.Wo;
    const int oy1 = plast / p.Wo;
    const int iy0 = oy0 * p.stride - p.pad;
    const int nrows = (oy1 - oy0) * p.stride + (p.KH - 1) * p.dil + 1;

    // Per-lane LDS offset (floats) of tap (0,0), channel sub-index included.
    int boff[NB];
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) {
        int pp = p0 + (wn * NB + nb) * MF + M::col(lane);
        pp = min(pp, p.P - 1);
        const int oy = pp / p.Wo;
        const int ox = pp - oy * p.Wo;
        boff[nb] = (oy - oy0) * p.stride * p.RS + ox * p.stride + (p.PL - p.pad) +
                   M::ksub(lane) * p.CS;
    }

    // Per-lane base of this wave's A-operand stream for each of its M blocks.
    const int taps = (TAPS == TAPS_GENERIC) ? p.KH * p.KW : TAPS;
    const float *__restrict__ wbase[MB];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
        const int mblk = m0 / MF + wm * MB + mb;
        wbase[mb] = p.wpk + ((long long)mblk * p.ncg_total) * taps * 64 + lane;
    }

    acc_t acc[MB][NB];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
        for (int nb = 0; nb < NB; ++nb)
#pragma unroll
            for (int v = 0; v < NACC; ++v) acc[mb][nb][v] = 0.0f;

    const int ncgw = p.CPW / KC;  // channel groups this wave consumes per LDS pass
    const float *lbase = lds + wk * p.CPW * p.CS;

    for (int chunk = 0; chunk < p.nchunks; ++chunk) {
        if (chunk > 0) __syncthreads();
        stage_chunk(p, in, lds, chunk * p.CCH, iy0, nrows, wave, nwaves, lane);
        __syncthreads();
        const int cg0 = (chunk * p.CCH + wk * p.CPW) / KC;

        if constexpr (TAPS == TAPS_3x3) {
            // One channel group (9 K-steps) per iteration; the next group's
            // weights are requested before this group's MFMAs are issued.
            float a_nxt[9][MB];
#pragma unroll
            for (int t = 0; t < 9; ++t)
#pragma unroll
                for (int mb = 0; mb < MB; ++mb) a_nxt[t][mb] = wbase[mb][((long long)cg0 * 9 + t) * 64];
            for (int cg = 0; cg < ncgw; ++cg) {
                float a_cur[9][MB];
#pragma unroll
                for (int t = 0; t < 9; ++t)
#pragma unroll
                    for (int mb = 0; mb < MB; ++mb) a_cur[t][mb] = a_nxt[t][mb];
                const int cgn = cg0 + min(cg + 1, ncgw - 1);
#pragma unroll
                for (int t = 0; t < 9; ++t)
#pragma unroll
                    for (int mb = 0; mb < MB; ++mb)
                        a_nxt[t][mb] = wbase[mb][((long long)cgn * 9 + t) * 64];
                const float *lrow = lbase + cg * KC * p.CS;
#pragma unroll
                for (int r = 0; r < 3; ++r) {
#pragma unroll
                    for (int s = 0; s < 3; ++s) {
                        float b[NB];
#pragma unroll
                        for (int nb = 0; nb < NB; ++nb)
                            b[nb] = lrow[boff[nb] + r * p.dil * p.RS + s * p.dil];
#pragma unroll
                        for (int mb = 0; mb < MB; ++mb)
#pragma unroll
                            for (int nb = 0; nb < NB; ++nb)
                                acc[mb][nb] = M::run(a_cur[r * 3 + s][mb], b[nb], acc[mb][nb]);
                    }
                }
            }
        } else if constexpr (TAPS == TAPS_1x1) {
            // Four channel groups per iteration (ncgw is a multiple of 4 by
            // construction of the tile), same one-iteration-ahead weight fetch.
            constexpr int G = 4;
            float a_nxt[G][MB];
#pragma unroll
            for (int t = 0; t < G; ++t)
#pragma unroll
                for (int mb = 0; mb < MB; ++mb) a_nxt[t][mb] = wbase[mb][((long long)cg0 + t) * 64];
            for (int cg = 0; cg < ncgw; cg += G) {
                float a_cur[G][MB];
#pragma unroll
                for (int t = 0; t < G; ++t)
#pragma unroll
                    for (int mb = 0; mb < MB; ++mb) a_cur[t][mb] = a_nxt[t][mb];
                const int cgn = cg0 + min(cg + G, ncgw - G);
#pragma unroll
                for (int t = 0; t < G; ++t)
#pragma unroll
                    for (int mb = 0; mb < MB; ++mb)
                        a_nxt[t][mb] = wbase[mb][((long long)cgn + t) * 64];
#pragma unroll
                for (int t = 0; t < G; ++t) {
                    const float *lrow = lbase + (cg + t) * KC * p.CS;
                    float b[NB];
#pragma unroll
                    for (int nb = 0; nb < NB; ++nb) b[nb] = lrow[boff[nb]];
#pragma unroll
                    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
                        for (int nb = 0; nb < NB; ++nb)
                            acc[mb][nb] = M::run(a_cur[t][mb], b[nb], acc[mb][nb]);
                }
            }
        } else {
            // Any filter size / dilation: taps walked at run time.
            for (int cg = 0; cg < ncgw; ++cg) {
                const float *lrow = lbase + cg * KC * p.CS;
                int t = 0;
                for (int r = 0; r < p.KH; ++r) {
                    for (int s = 0; s < p.KW; ++s, ++t) {
                        float a[MB], b[NB];
#pragma unroll
                        for (int mb = 0; mb < MB; ++mb)
                            a[mb] = wbase[mb][((long long)(cg0 + cg) * taps + t) * 64];
#pragma unroll
                        for (int nb = 0; nb < NB; ++nb)
                            b[nb] = lrow[boff[nb] + r * p.dil * p.RS + s * p.dil];
#pragma unroll
                        for (int mb = 0; mb < MB; ++mb)
#pragma unroll
                            for (int nb = 0; nb < NB; ++nb)
                                acc[mb][nb] = M::run(a[mb], b[nb], acc[mb][nb]);
                    }
                }
            }
        }
    }

    if (p.WK == 1) {
        // Straight from the accumulators: each store instruction writes runs of
        // MF consecutive pixels of one output channel.
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) {
#pragma unroll
            for (int nb = 0; nb < NB; ++nb) {
                const int pp = p0 + (wn * NB + nb) * MF + M::col(lane);
#pragma unroll
                for (int v = 0; v < NACC; ++v) {
                    const int n = m0 + (wm * MB + mb) * MF + M::row(v, lane);
                    if (n < p.N && pp < p.P) {
                        float val = acc[mb][nb][v];
                        if (p.bias) val += p.bias[n];
                        const long long o = (long long)n * p.P + pp;
                        if (resid) val += resid[o];
                        if (p.relu) val = fmaxf(val, 0.0f);
                        out[o] = val;
                    }
                }
            }
        }
    } else {
        // Split-K across waves: park every wave's partial tile in LDS
        // ([wk][channel][pixel]) and add the WK slices in index order.
        __syncthreads();
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) {
#pragma unroll
            for (int nb = 0; nb < NB; ++nb) {
                const int pl = (wn * NB + nb) * MF + M::col(lane);
#pragma unroll
                for (int v = 0; v < NACC; ++v) {
                    const int ml = (wm * MB + mb) * MF + M::row(v, lane);
                    lds[(wk * MT + ml) * PT + pl] = acc[mb][nb][v];
                }
            }
        }
        __syncthreads();
        const int total = MT * PT;
        for (int idx = tid; idx < total; idx += blockDim.x) {
            const int ml = idx / PT;
            const int pl = idx - ml * PT;
            const int n = m0 + ml;
            const int pp = p0 + pl;
            if (n < p.N && pp < p.P) {
                float val = lds[idx];
                for (int k = 1; k < p.WK; ++k) val += lds[k * total + idx];
                if (p.bias) val += p.bias[n];
                const long long o = (long long)n * p.P + pp;
                if (resid) val += resid[o];
                if (p.relu) val = fmaxf(val, 0.0f);
                out[o] = val;
            }
        }
    }
}

// ---------------------------------------------------------------------------
// Instantiation table.  Tiles with a 2x2 block grid per wave need up to 64
// accumulator registers plus two weight buffers, so they are built for at most
// 8 waves per workgroup (256 registers per lane); the others for 16 waves.
// ---------------------------------------------------------------------------
typedef void (*kernel_fn)(const ConvKParams);

template <int MF, int TAPS>
static kernel_fn pick_mbnb(int mb, int nb) {
    if (mb == 1 && nb == 1) return tdc_conv_mfma_kernel<MF, 1, 1, TAPS, 16>;
    if (mb == 1 && nb == 2) return tdc_conv_mfma_kernel<MF, 1, 2, TAPS, 16>;
    if (mb == 2 && nb == 1) return tdc_conv_mfma_kernel<MF, 2, 1, TAPS, 16>;
    if (mb == 2 && nb == 2) return tdc_conv_mfma_kernel<MF, 2, 2, TAPS, 8>;
    return nullptr;
}

template <int TAPS>
static kernel_fn pick_mf(int mf, int mb, int nb) {
    if (mf == 32) return pick_mbnb<32, TAPS>(mb, nb);
    if (mf == 16) return pick_mbnb<16, TAPS>(mb, nb);
    return nullptr;
}

static int taps_mode(const ConvKParams &kp) {
    if (kp.KH == 3 && kp.KW == 3) return TAPS_3x3;
    if (kp.KH == 1 && kp.KW == 1) return TAPS_1x1;
    return TAPS_GENERIC;
}

static kernel_fn pick_kernel(const tdc_tile &t, int mode) {
    switch (mode) {
        case TAPS_3x3: return pick_mf<TAPS_3x3>(t.mf, t.mb, t.nb);
        case TAPS_1x1: return pick_mf<TAPS_1x1>(t.mf, t.mb, t.nb);
        default: return pick_mf<TAPS_GENERIC>(t.mf, t.mb, t.nb);
    }
}

const void *conv_kernel_for(const tdc_tile &t, int KH, int KW) {
    ConvKParams kp{};
    kp.KH = KH;
    kp.KW = KW;
    return reinterpret_cast<const void *>(pick_kernel(t, taps_mode(kp)));
}

int prepare_conv_kernel(const void *fn, const Geometry &g) {
    if (!fn) return (int)hipErrorInvalidValue;
    // Dynamic LDS above the 64 KiB default has to be opted into per kernel.
    if (g.lds_bytes > 64 * 1024) {
        hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, g.lds_bytes);
        if (e != hipSuccess) return (int)e;
    }
    return 0;
}

int launch_conv(const void *fn, const Geometry &g, const ConvKParams &kp, void *stream) {
    if (!fn) return (int)hipErrorInvalidValue;
    dim3 grid(g.grid_x, g.grid_y, g.grid_z), block(g.threads);
    hipLaunchKernelGGL(reinterpret_cast<kernel_fn>(const_cast<void *>(fn)), grid, block,
                       (size_t)g.lds_bytes, (hipStream_t)stream, kp);
    return (int)hipGetLastError();
}

}  // namespace tdc
