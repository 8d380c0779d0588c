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

template <int VW>
struct VecOf;
template <>
struct VecOf<1> { using type = float; };
template <>
struct VecOf<2> { using type = float2; };
template <>
struct VecOf<4> { using type = float4; };

// Copy input channels [c0, c0+CCH) x rows [iy0, iy0+nrows) into LDS as
// [channel][row][RS] with zeros for the halo and for channels >= C.  The slab is
// walked as a flat list of VW-wide vectors (RS, PL, W and CS are multiples of
// VW, so a vector is either all image or all halo); every thread issues U
// unconditional, clamped loads before it writes anything, so a wave keeps U
// global loads in flight instead of one.
template <int VW>
__device__ __forceinline__ void stage_chunk(const ConvKParams &p, const float *__restrict__ in,
                                            float *__restrict__ lds, int c0, int iy0, int nrows,
                                            int tid, int nthreads) {
    using vec_t = typename VecOf<VW>::type;
    constexpr int U = 4;
    const int rsv = p.RS / VW;
    const int per_ch = nrows * rsv;
    const int total = p.CCH * per_ch;
    const int plv = p.PL / VW;
    const int wv = p.W / VW;
    const vec_t *__restrict__ src = reinterpret_cast<const vec_t *>(in);
    for (int base = tid; base < total; base += nthreads * U) {
        vec_t v[U];
        int dst[U];
        bool inb[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int e = base + u * nthreads;
            const int ee = e < total ? e : 0;
            const int cl = ee / per_ch;
            const int rem = ee - cl * per_ch;
            const int row = rem / rsv;
            const int xv = rem - row * rsv;
            const int c = c0 + cl;
            const int iy = iy0 + row;
            const int ixv = xv - plv;
            inb[u] = c < p.C && iy >= 0 && iy < p.H && ixv >= 0 && ixv < wv;
            const int sidx = inb[u] ? (c * p.H + iy) * wv + ixv : 0;
            v[u] = src[sidx];
            dst[u] = e < total ? cl * p.CS + row * p.RS + xv * VW : -1;
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            vec_t val = v[u];
            if (!inb[u]) val = vec_t{};
            if (dst[u] >= 0) *reinterpret_cast<vec_t *>(lds + dst[u]) = val;
        }
    }
}

template <int MF, int MB, int NB, int TAPS, int MAXW>
__global__ void __launch_bounds__(MAXW * 64) tdc_conv_mfma_kernel(const ConvKParams p) {
    using M = Mfma<MF>;
    using acc_t = typename M::acc_t;
    constexpr int KC = M::KC;
    constexpr int NACC = M::NACC;
    // K-steps fetched per weight prefetch: one channel group of a 3x3 filter,
    // four channel groups of a 1x1 filter, a single step otherwise.
    constexpr int G = (TAPS == TAPS_3x3) ? 9 : (TAPS == TAPS_1x1) ? 4 : 1;
    extern __shared__ __align__(16) float lds[];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int nthreads = blockDim.x;
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

    // Per-lane base of this wave's A-operand stream for each of its M blocks.
    const int taps = (TAPS == TAPS_GENERIC) ? p.KH * p.KW : TAPS;
    const float *__restrict__ wbase[MB];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
        const int mblk = m0 / MF + wm * MB + mb;
        wbase[mb] = p.wpk + ((long long)mblk * p.ncg_total) * taps * 64 + lane;
    }
    const int ncgw = p.CPW / KC;  // channel groups this wave consumes per LDS pass
    // The wave's K-steps of pass `chunk` start at packed K-step index kfirst(chunk);
    // a pass holds nkw of them, consumed G at a time.
    const int nkw = ncgw * taps;
    auto kfirst = [&](int chunk) { return ((chunk * p.CCH + wk * p.CPW) / KC) * taps; };

    // First weights are requested before the input slab, so both fetches overlap.
    float a_nxt[G][MB];
#pragma unroll
    for (int t = 0; t < G; ++t)
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) a_nxt[t][mb] = wbase[mb][(long long)(kfirst(0) + t) * 64];

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

    acc_t acc[MB][NB];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
        for (int nb = 0; nb < NB; ++nb)
#pragma unroll
            for (int v = 0; v < NACC; ++v) acc[mb][nb][v] = 0.0f;

    const float *lbase = lds + wk * p.CPW * p.CS;

    for (int chunk = 0; chunk < p.nchunks; ++chunk) {
        if (chunk > 0) __syncthreads();
        if (p.VW == 4) stage_chunk<4>(p, in, lds, chunk * p.CCH, iy0, nrows, tid, nthreads);
        else if (p.VW == 2) stage_chunk<2>(p, in, lds, chunk * p.CCH, iy0, nrows, tid, nthreads);
        else stage_chunk<1>(p, in, lds, chunk * p.CCH, iy0, nrows, tid, nthreads);
        __syncthreads();
        const int k0 = kfirst(chunk);
        const int knext_chunk = kfirst(min(chunk + 1, p.nchunks - 1));

        for (int k = 0; k < nkw; k += G) {
            float a_cur[G][MB];
#pragma unroll
            for (int t = 0; t < G; ++t)
#pragma unroll
                for (int mb = 0; mb < MB; ++mb) a_cur[t][mb] = a_nxt[t][mb];
            // Next group of this pass, else the first group of the next pass,
            // else (very last group) a harmless re-read of the current one.
            int kn = k0 + k + G;
            if (k + G >= nkw) kn = (chunk + 1 < p.nchunks) ? knext_chunk : k0 + k;
#pragma unroll
            for (int t = 0; t < G; ++t)
#pragma unroll
                for (int mb = 0; mb < MB; ++mb) a_nxt[t][mb] = wbase[mb][(long long)(kn + t) * 64];

            if constexpr (TAPS == TAPS_3x3) {
                const float *lrow = lbase + (k / 9) * KC * p.CS;
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
            } else if constexpr (TAPS == TAPS_1x1) {
#pragma unroll
                for (int t = 0; t < G; ++t) {
                    const float *lrow = lbase + (k + t) * KC * p.CS;
                    float b[NB];
#pragma unroll
                    for (int nb = 0; nb < NB; ++nb) b[nb] = lrow[boff[nb]];
#pragma unroll
                    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
                        for (int nb = 0; nb < NB; ++nb)
                            acc[mb][nb] = M::run(a_cur[t][mb], b[nb], acc[mb][nb]);
                }
            } else {
                // Any filter size / dilation: decode the tap of this K-step.
                const int cg = k / taps;
                const int tap = k - cg * taps;
                const int r = tap / p.KW;
                const int s = tap - r * p.KW;
                const float *lrow = lbase + cg * KC * p.CS;
                float b[NB];
#pragma unroll
                for (int nb = 0; nb < NB; ++nb) b[nb] = lrow[boff[nb] + r * p.dil * p.RS + s * p.dil];
#pragma unroll
                for (int mb = 0; mb < MB; ++mb)
#pragma unroll
                    for (int nb = 0; nb < NB; ++nb)
                        acc[mb][nb] = M::run(a_cur[0][mb], b[nb], acc[mb][nb]);
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
        for (int idx = tid; idx < total; idx += nthreads) {
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
