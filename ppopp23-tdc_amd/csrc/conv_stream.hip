// Streamed convolution kernels: both operands go from global memory straight into registers, nothing is staged in
// LDS, one memory round trip per wave.  1x1 (tdc_conv1x1_stream_kernel), 3x3 (tdc_conv3x3_stream_kernel, with the
// fused 1x1 tail and head of a Tucker convolution) and 3x3 with several 14-pixel row blocks per wave
// (tdc_conv3x3_stream_rownb_kernel); each is described at its definition.
#include "conv_device.hpp"

namespace tdc {

// ---------------------------------------------------------------------------
// Streamed kernels whose input channels are split over KS workgroups: the lanes that hold a finished partial block
// (`holder`: four consecutive channels from `ch0` of pixel `pp`) leave it in the workspace ws[image][slice][N][P]; the
// workgroup that draws the last ticket of its (image, channel tile, pixel tile) reads all KS partials back and adds
// them in slice order, so the result does not depend on which workgroup that is.  Same protocol as the staged
// kernel: every workspace access is a relaxed device-scope atomic (written through, read past the die-local L2).
// Returns false in the workgroups that are done; every thread of the workgroup must call it.
// ---------------------------------------------------------------------------
__device__ __forceinline__ bool stream_join_slices(const ConvKParams &p, float *lds, f4_t &acc, bool holder, int ch0,
                                                   int pp, int img, int slice, int by, int bx) {
    const long long NP = (long long)p.N * p.P;
    if (holder) {
        float *wsz = p.ws + ((long long)img * p.KS + slice) * NP;
#pragma unroll
        for (int i = 0; i < 4; ++i)
            if (ch0 + i < p.N)
                __hip_atomic_store(wsz + (long long)(ch0 + i) * p.P + pp, acc[i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();
    unsigned *ticket = p.ctr + ((unsigned)img * p.grid_y + by) * p.grid_x + bx;
    if (threadIdx.x == 0) {
        const unsigned d = __hip_atomic_fetch_add(ticket, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        reinterpret_cast<unsigned *>(lds)[0] = d;
    }
    __syncthreads();
    const unsigned drawn = reinterpret_cast<const unsigned *>(lds)[0];
    if (drawn != (unsigned)p.KS - 1u) return false;
    if (threadIdx.x == 0) __hip_atomic_store(ticket, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);  // for the next launch
    if (holder) {
        const float *ws0 = p.ws + (long long)img * p.KS * NP;
        float part[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) part[i] = 0.0f;
        // (these loads go past the L2 and take a microsecond: eight slices are requested at once, then added in order)
        for (int s0 = 0; s0 < p.KS; s0 += 8) {
            float v[8][4];
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                const float *src = ws0 + (long long)min(s0 + u, p.KS - 1) * NP + pp;
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    v[u][i] = __hip_atomic_load(src + (long long)min(ch0 + i, p.N - 1) * p.P, __ATOMIC_RELAXED,
                                                __HIP_MEMORY_SCOPE_AGENT);
            }
#pragma unroll
            for (int u = 0; u < 8; ++u)
                if (s0 + u < p.KS) {
#pragma unroll
                    for (int i = 0; i < 4; ++i) part[i] += v[u][i];
                }
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) acc[i] = part[i];
    }
    return true;
}

// The partial blocks of the WK waves that split the input channels lie in LDS as [wave][register 0-3][lane].  Sum of
// register `i` over the WK slices from `first` on, in slice order (the result does not depend on timing), eight reads in
// flight at a time: read one by one, every slice would cost this wave a whole LDS round trip.
__device__ __forceinline__ float sum_slices(const float *lds, int first, int WK, int i, int lane) {
    const float *src = lds + (first * 4 + i) * 64 + lane;
    float sum = 0.0f;
    for (int w0 = 0; w0 < WK; w0 += 8) {
        float part[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) part[u] = src[min(w0 + u, WK - 1) * 256];
#pragma unroll
        for (int u = 0; u < 8; ++u)
            if (w0 + u < WK) sum += part[u];
    }
    return sum;
}

// One output channel `ch` of pixel `pix` (a lane of a wave that finishes ONE accumulator register of the block):
// + bias, + residual, ReLU, store.
__device__ __forceinline__ void finish_one_channel(float val, int ch, int N, long long P, long long pix,
                                                   const float *__restrict__ bias, const float *__restrict__ resid, int relu,
                                                   float *__restrict__ out) {
    if (ch >= N) return;
    const float bv = bias ? bias[ch] : 0.0f;
    const float rv = resid ? resid[(long long)ch * P + pix] : 0.0f;
    val += bv;
    val += rv;
    if (relu) val = fmaxf(val, 0.0f);
    store_out(out + ((long long)ch * P + pix), val);
}

// ---------------------------------------------------------------------------
// 1x1 convolution with many input channels over few pixels (tile.alg = 3): no LDS stage, no passes, no barrier
// before the reduction.  One workgroup owns a 16-channel x 16-pixel block of the output; its WK waves split the
// input channels, NQ runs of 16 channels each.  A wave requests ALL its operands up front, straight into
// registers (per run: one 128-bit load of packed weights, four 32-bit loads of the input, and two 128-bit loads of
// the input affine if there is one), then issues its 4*NQ MFMAs as the data arrives and leaves its 16x16 partial
// in LDS for wave 0 to add up in a fixed order.  Within a run lane (k, n) takes channels 16q + 4k + s over the four
// K-steps s, so that its weights and its scale/shift pairs are contiguous.
// Channels past C read as zero (range-checked vector offsets) and meet zero weights; pixel lanes past the image
// re-read its last pixel and are never stored.
// ---------------------------------------------------------------------------
// (eight runs per wave: 72 registers of operands, 136 with the affine; that variant is built for at most 8 waves)
// MODE 1: the instantiation whose input channels are dealt to p.KS workgroups.  MODE 2: stride > 1 (ResNet's downsampling
// shortcuts): output pixel (oy, ox) reads input pixel (oy * stride, ox * stride).  The plain one pays for neither.
template <int NQ, bool AFF, int MODE>
__global__ void __launch_bounds__(NQ == 8 ? 512 : 1024) tdc_conv1x1_stream_kernel(const ConvKParams p) {
    constexpr bool SPLIT = MODE == 1, STRIDED = MODE == 2;
    extern __shared__ __align__(16) float lds[];
    TDC_STAMP_DECL;
    TDC_STAMP(0);   // entry
    touch_kernel_arguments();
    TDC_STAMP(7);   // every line of the kernel arguments is in the scalar cache
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // = this wave's slice of the input channels
    // same die-aware decoding of the one-dimensional launch as the staged kernel
    const int logical = (int)(blockIdx.x & 7u) * p.xcd_chunk + (int)(blockIdx.x >> 3);
    if (logical >= p.n_wg) return;
    const int q1 = fdiv(logical, p.fd_g1);
    const int r1 = logical - q1 * p.fd_g1.d;
    const int bz = fdiv(q1, p.fd_g2);          // image * KS + slice of the input channels
    const int r2 = q1 - bz * p.fd_g2.d;
    const int img = SPLIT ? fdiv(bz, p.fd_ks) : bz;
    const int slice = SPLIT ? bz - img * p.KS : 0;
    const int KS = SPLIT ? p.KS : 1;
    const int bx = p.channel_major ? r1 : r2;  // pixel block
    const int by = p.channel_major ? r2 : r1;  // channel block
    const ImageBase image = image_base(p, img);
    const float *__restrict__ in = image.in;
    float *__restrict__ out = image.out;
    const float *__restrict__ resid = image.resid;
    const __amdgpu_buffer_rsrc_t in_rsrc =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(in), (short)0, (int)p.in_image_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t w_rsrc =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(p.wpk), (short)0, (int)p.wpk_bytes, 0x00020000);

    const int k = lane >> 4, n = lane & 15;
    const int px = bx * 16 + n;
    const int pxr = min(px, p.P - 1);
    const int cl = wave * (16 * NQ) + 4 * k;   // this lane's first channel inside the workgroup's slice
    const int c0 = slice * p.CCH + cl;         // ... and in the image
    // bytes between channels (with stride 1 the host presents the image as one row of H*W pixels)
    const unsigned HW4 = STRIDED ? (unsigned)(p.H * p.W) * 4u : (unsigned)p.W * 4u;
    unsigned pix4 = (unsigned)pxr * 4u;        // this lane's input pixel, in bytes from the start of a channel
    if constexpr (STRIDED) {
        const int oy = fdiv(pxr, p.fd_wtw);    // (fd_wtw holds the output row length here)
        const int ox = pxr - oy * p.Wo;
        pix4 = (unsigned)((oy * p.W + ox) * p.stride) * 4u;
    }

    f4_t a[NQ], sc[NQ], sh[NQ];
    float b[NQ][4];
    const int a_soff = ((by * KS + slice) * (p.CCH >> 4) + wave * NQ) * 1024;
    const unsigned b_voff = (unsigned)c0 * HW4 + pix4;
#pragma unroll
    for (int q = 0; q < NQ; ++q) {
        a[q] = __builtin_bit_cast(f4_t, __builtin_amdgcn_raw_buffer_load_b128(w_rsrc, lane * 16, a_soff + q * 1024, 0));
#pragma unroll
        for (int s4 = 0; s4 < 4; ++s4)   // (the whole offset goes through the range-checked vector operand)
            b[q][s4] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(in_rsrc, (int)(b_voff + (unsigned)(16 * q + s4) * HW4), 0, 0));
        if constexpr (AFF) {
            const __amdgpu_buffer_rsrc_t aff_rsrc =
                __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(p.in_aff + slice * 2 * p.CCH), (short)0, p.CCH * 8, 0x00020000);
            sc[q] = __builtin_bit_cast(f4_t, __builtin_amdgcn_raw_buffer_load_b128(aff_rsrc, (cl + 16 * q) * 4, 0, 0));
            sh[q] = __builtin_bit_cast(f4_t, __builtin_amdgcn_raw_buffer_load_b128(aff_rsrc, (p.CCH + cl + 16 * q) * 4, 0, 0));
        }
        __builtin_amdgcn_sched_barrier(0);   // requests in the order the MFMAs consume them
    }
    // (every request is issued before the first MFMA: the scheduler must not sink loads into the MFMA sequence)
    __builtin_amdgcn_sched_barrier(0);
    TDC_STAMP(1);   // every request issued
    // two accumulator chains: consecutive MFMAs do not wait for each other's result
    f4_t acc0 = (f4_t){0.0f, 0.0f, 0.0f, 0.0f}, acc1 = (f4_t){0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int q = 0; q < NQ; ++q) {
#pragma unroll
        for (int s4 = 0; s4 < 4; ++s4) {
            float v = b[q][s4];
            if constexpr (AFF) {
                v = v * sc[q][s4] + sh[q][s4];
                if (p.in_relu) v = fmaxf(v, 0.0f);
            }
            if (s4 & 1) acc1 = __builtin_amdgcn_mfma_f32_16x16x4f32(a[q][s4], v, acc1, 0, 0, 0);
            else acc0 = __builtin_amdgcn_mfma_f32_16x16x4f32(a[q][s4], v, acc0, 0, 0, 0);
        }
        __builtin_amdgcn_sched_barrier(0);   // run by run, as the data arrives
    }
    f4_t acc = acc0 + acc1;
    TDC_STAMP(4);   // MFMAs issued (the last results may still be in the pipe)
    // lane l holds rows 4*(l/16) .. +3 (output channels) of column l%16 (pixel)
    if (p.WK > 1) {
#pragma unroll
        for (int i = 0; i < 4; ++i) lds[(wave * 4 + i) * 64 + lane] = acc[i];
        __syncthreads();
        TDC_STAMP(5);   // everybody's partial blocks are in LDS
        if constexpr (!SPLIT) {
            if (p.WK >= 4) {
                // the first four waves share the final sum and the store: wave w finishes accumulator register w
                // (output channel 4k + w of its lanes' pixels)
                if (wave < 4 && px < p.P)
                    finish_one_channel(sum_slices(lds, 0, p.WK, wave, lane), by * 16 + 4 * k + wave, p.N, p.P, px, p.bias,
                                       resid, p.relu, out);
                TDC_STAMP(6);   // stores issued
                TDC_STAMP_FLUSH(p, logical, wave, lane);
                return;
            }
        }
        if (wave == 0) {
#pragma unroll
            for (int i = 0; i < 4; ++i) acc[i] = sum_slices(lds, 0, p.WK, i, lane);
        }
    }
    if constexpr (SPLIT) {
        // the input channels are split over KS workgroups: whoever finishes last adds the partial blocks in slice order
        if (!stream_join_slices(p, lds, acc, wave == 0 && px < p.P, by * 16 + 4 * k, px, img, slice, by, bx)) return;
    }
    if (wave == 0 && px < p.P) finish_four_channels(acc, by * 16 + 4 * k, p.N, p.P, px, p.bias, resid, p.relu, out);
    TDC_STAMP(6);   // stores issued
    TDC_STAMP_FLUSH(p, logical, wave, lane);
}

// ---------------------------------------------------------------------------
// 3x3 convolution streamed the same way (tile.alg = 4): one workgroup owns 16 output channels of a TH x TW tile of 16
// pixels, its WK waves split the input channels, CG groups of four channels each.  Per group a lane requests its nine
// input values (one per tap, four channels across the lane quarters) and its nine weights (packed as for
// tile.alg = 2: two 128-bit loads and one 32-bit load); padding, channels past C and lanes past the tile present an
// out-of-range offset and read zero without a memory access.
// ---------------------------------------------------------------------------
// INP: how a wave gets its pixel operands.
//   0  nine 32-bit requests per group of channels, one per tap;
//   1  (stride 1 and a tile of one row of 14 pixels) the 16 lanes of a quarter load the 16 consecutive input pixels
//      that the row of outputs touches, once per filter row, and the three taps of a row are lane shifts of that value
//      (three requests per group of channels instead of nine);
//   2  (tile.alg = 6) the tile's input WINDOW — (TH-1)*stride+3 rows of up to 24 columns, from the 4-column boundary
//      at or left of its first column — is loaded with ONE or two 128-bit requests per group of four channels (lane n
//      of a quarter takes four consecutive columns of one window row), masked where it leaves the image, and left in a
//      wave-private piece of LDS, from which every lane reads its nine taps.  The compute unit's address path takes
//      about as long for a 32-bit request of a wave as for a 128-bit one (12 against 16-17 cycles, measured), so the
//      window costs it a ninth (a third, against INP = 1) of the time; LDS reads are several times cheaper.  No
//      workgroup barrier is involved: a wave only reads what it wrote itself.
// MODE: 0 = plain, 1 = input channels dealt to p.KS workgroups, 2 = with the fused 1x1 tail, 3 = with a fused 1x1 head in
// front as well (a whole Tucker convolution in one launch: the workgroup first computes the first factor on its window of
// (TH + 2) x (TW + 2) pixels into LDS, which the core loop then reads instead of global memory).  Separate instantiations:
// code a launch never runs still costs it (0.13 us per launch measured for the split's code inside the plain kernel).
template <int CG, int INP, int MODE>
__global__ void __launch_bounds__(1024) tdc_conv3x3_stream_kernel(const ConvKParams p) {
    constexpr bool SPLIT = MODE == 1, TAIL = MODE == 2 || MODE == 3, HEAD = MODE == 3, ROW = INP == 1, WINDOW = INP == 2;
    extern __shared__ __align__(16) float lds[];
    TDC_STAMP_DECL;
    TDC_STAMP(0);   // entry
    touch_kernel_arguments();
    TDC_STAMP(7);   // every line of the kernel arguments is in the scalar cache
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int logical = (int)(blockIdx.x & 7u) * p.xcd_chunk + (int)(blockIdx.x >> 3);
    if (logical >= p.n_wg) return;
    const int q1 = fdiv(logical, p.fd_g1);
    const int r1 = logical - q1 * p.fd_g1.d;
    const int bz = fdiv(q1, p.fd_g2);          // image * KS + slice of the input channels
    const int r2 = q1 - bz * p.fd_g2.d;
    const int img = SPLIT ? fdiv(bz, p.fd_ks) : bz;
    const int slice = SPLIT ? bz - img * p.KS : 0;
    const int KS = SPLIT ? p.KS : 1;
    const int bx = p.channel_major ? r1 : r2;  // pixel tile
    const int by = p.channel_major ? r2 : r1;  // channel block
    const int tile_y = fdiv(bx, p.fd_ntx);
    const int tile_x = bx - tile_y * p.ntx;
    const ImageBase image = image_base(p, img);
    const float *__restrict__ in = image.in;
    float *__restrict__ out = image.out;
    const float *__restrict__ resid = image.resid;
    const __amdgpu_buffer_rsrc_t in_rsrc =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(in), (short)0, (int)p.in_image_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t w_rsrc =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(p.wpk), (short)0, (int)p.wpk_bytes, 0x00020000);

    // wave = (channel block of the workgroup) * WK + (slice of the input channels)
    const int wmi = fdiv(wave, p.fd_wk);
    const int wki = wave - wmi * p.WK;
    const int mblk = by * p.WM + wmi;   // this wave's block of 16 output channels
    // The weights depend on nothing but the channel block and the wave: request them before any pixel arithmetic.
    // packed as [channel tile][slice][block of the workgroup][group]: nine taps x 64 lanes x 4 bytes per group
    const int a_soff = ((((by * KS + slice) * p.WM + wmi) * (p.CCH >> 2)) + wki * CG) * 2304;
    f4_t a0[CG], a1[CG];
    float a8[CG], b[CG][9];
#pragma unroll
    for (int g = 0; g < CG; ++g) {
        a0[g] = __builtin_bit_cast(f4_t, __builtin_amdgcn_raw_buffer_load_b128(w_rsrc, lane * 16, a_soff + g * 2304, 0));
        a1[g] = __builtin_bit_cast(f4_t, __builtin_amdgcn_raw_buffer_load_b128(w_rsrc, lane * 16, a_soff + g * 2304 + 1024, 0));
        a8[g] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(w_rsrc, lane * 4, a_soff + g * 2304 + 2048, 0));
    }
    __builtin_amdgcn_sched_barrier(0);

    const int k = lane >> 4, n = lane & 15;
    const int jy = fdiv(n, p.fd_tw);
    const int jx = n - jy * p.TW;
    const int oy = tile_y * p.TH + jy, ox = tile_x * p.TW + jx;
    const bool live = jy < p.TH && oy < p.Ho && ox < p.Wo;
    const int iy0 = oy * p.stride - p.pad, ix0 = ox * p.stride - p.pad;
    const unsigned rowb = (unsigned)p.W * 4u;
    const unsigned chan_bytes = (unsigned)(p.H * p.W) * 4u;
    const unsigned base = (unsigned)(slice * p.CCH + wki * (4 * CG) + k) * chan_bytes;   // this lane's first channel
    if constexpr (HEAD) {
        // First factor on the window: 16 x 16 blocks (channels x window pixels) dealt to the waves, both operands
        // streamed from global memory four runs of 16 input channels at a time; pixels outside the image read zero,
        // which is the core's zero padding (the factor has no bias).
        float *F = lds + p.head_f_off;
        const __amdgpu_buffer_rsrc_t hw_rsrc = __builtin_amdgcn_make_buffer_rsrc(
            const_cast<float *>(p.head_w), (short)0, p.head_mblk * p.head_runs * 1024, 0x00020000);
        const int nwaves = p.WM * p.WK;
        const int nblk = p.head_mblk * p.head_npb;
        for (int blk = wave; blk < nblk; blk += nwaves) {
            const int cb = fdiv(blk, p.fd_hnpb);
            const int pb = blk - cb * p.head_npb;
            const int wq = pb * 16 + n;
            const int wy = fdiv(wq, p.fd_hww);
            const int wx = wq - wy * p.head_ww;
            const int iy = tile_y * p.TH - p.pad + wy, ix = tile_x * p.TW - p.pad + wx;
            const bool ok = wq < p.head_wq && (unsigned)iy < (unsigned)p.H && (unsigned)ix < (unsigned)p.W;
            const unsigned pix = ok ? (unsigned)(iy * p.W + ix) * 4u + (unsigned)(4 * k) * chan_bytes : (unsigned)OOB_OFFSET;
            f4_t h0 = (f4_t){0.0f, 0.0f, 0.0f, 0.0f}, h1 = (f4_t){0.0f, 0.0f, 0.0f, 0.0f};
            // (four runs per round trip: eight at once measured slower, the workgroup is bound by its compute unit's fill rate)
            for (int q0 = 0; q0 < p.head_runs; q0 += 4) {
                f4_t ha[4];
                float hb[4][4];
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    ha[u] = __builtin_bit_cast(f4_t, __builtin_amdgcn_raw_buffer_load_b128(
                                                         hw_rsrc, lane * 16, (cb * p.head_runs + q0 + u) * 1024, 0));
#pragma unroll
                    for (int s4 = 0; s4 < 4; ++s4)
                        hb[u][s4] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(
                            in_rsrc, (int)(pix + (unsigned)(16 * (q0 + u) + s4) * chan_bytes), 0, 0));
                }
#pragma unroll
                for (int u = 0; u < 4; ++u)
#pragma unroll
                    for (int s4 = 0; s4 < 4; ++s4) {
                        if (s4 & 1) h1 = __builtin_amdgcn_mfma_f32_16x16x4f32(ha[u][s4], hb[u][s4], h1, 0, 0, 0);
                        else h0 = __builtin_amdgcn_mfma_f32_16x16x4f32(ha[u][s4], hb[u][s4], h0, 0, 0, 0);
                    }
            }
            const f4_t h = h0 + h1;
#pragma unroll
            for (int i = 0; i < 4; ++i) F[(cb * 16 + 4 * k + i) * p.head_ld + wq] = h[i];
        }
        __syncthreads();
        // the core's pixel operand comes from that window: output pixel (jy, jx), tap (r, c) = window pixel (jy + r, jx + c)
        const float *Fk = F + (wki * (4 * CG) + k) * p.head_ld;
        const int wmax = p.head_npb * 16 - 1;
#pragma unroll
        for (int g = 0; g < CG; ++g)
#pragma unroll
            for (int t = 0; t < 9; ++t)
                b[g][t] = Fk[4 * g * p.head_ld + min((jy + t / 3) * p.head_ww + jx + t % 3, wmax)];
    } else if constexpr (WINDOW) {
        // The window of this tile: rows iyw0 .. iyw0 + win_rows - 1, columns from ixa (a multiple of four, at or left of
        // the tile's first input column) in win_L segments of four.  Lane n of a quarter takes slot q * 16 + n of its
        // channel, slot = row * win_L + segment; slots past the window and segments left or right of the image row, or in
        // a row above or below the image, present the out-of-range offset and read zeros; a segment that straddles the
        // right edge is loaded whole and masked.
        const int L = p.win_L, NS = p.win_ns;
        const int ixw0 = tile_x * p.TW * p.stride - p.pad;
        const int ixa = (ixw0 >> 2) << 2;                 // (arithmetic shift: floors negative columns too)
        const int iyw0 = tile_y * p.TH * p.stride - p.pad;
        constexpr int NREQ = 2;
        float *win = lds + p.win_off + wave * (CG * 4 * NS) + k * NS;     // this lane's channel of group 0
        unsigned soff[NREQ];
        int wslot[NREQ], ncol[NREQ];
#pragma unroll
        for (int q = 0; q < NREQ; ++q) {
            const int slot = q * 16 + n;
            const int row = fdiv(slot, p.fd_winL);
            const int cs = ixa + 4 * (slot - row * L);
            const bool ok = row < p.win_rows && (unsigned)(iyw0 + row) < (unsigned)p.H && (unsigned)cs < (unsigned)p.W;
            const unsigned m = ok ? 0xffffffffu : 0u;
            soff[q] = ((unsigned)((iyw0 + row) * p.W + cs) * 4u & m) | ((unsigned)OOB_OFFSET & ~m);
            wslot[q] = row < p.win_rows ? slot * 4 : -1;          // where this lane's four columns go (floats), or nowhere
            ncol[q] = p.W - cs;                                   // columns of the segment inside the row
        }
        f4_t wv[CG][NREQ];
#pragma unroll
        for (int g = 0; g < CG; ++g) {
#pragma unroll
            for (int q = 0; q < NREQ; ++q)
                if (q == 0 || p.win_nreq > 1)
                    wv[g][q] = __builtin_bit_cast(f4_t, __builtin_amdgcn_raw_buffer_load_b128(
                        in_rsrc, (int)(soff[q] + base + (unsigned)(4 * g) * chan_bytes), 0, 0));
            __builtin_amdgcn_sched_barrier(0);
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int g = 0; g < CG; ++g)
#pragma unroll
            for (int q = 0; q < NREQ; ++q)
                if ((q == 0 || p.win_nreq > 1) && wslot[q] >= 0) {
                    f4_t v = wv[g][q];
#pragma unroll
                    for (int e = 1; e < 4; ++e) v[e] = e < ncol[q] ? v[e] : 0.0f;
                    *reinterpret_cast<f4_t *>(win + g * 4 * NS + wslot[q]) = v;
                }
        // (the lanes of a wave exchange data through LDS here: its LDS instructions complete in order, and nothing may be
        //  moved across this point by the compiler)
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        const int jyc = min(jy, p.TH - 1);   // (lanes past the tile re-read its last row; they are never stored)
        const float *rd = win + (jyc * p.stride) * (4 * L) + jx * p.stride + (ixw0 - ixa);
#pragma unroll
        for (int g = 0; g < CG; ++g)
#pragma unroll
            for (int r = 0; r < 3; ++r)
#pragma unroll
                for (int c = 0; c < 3; ++c) b[g][r * 3 + c] = rd[g * 4 * NS + r * (4 * L) + c];
    } else if constexpr (ROW) {
        // lane n of a quarter: input column (tile's first column - pad + n) of the three input rows
        const int iyr = tile_y - p.pad, ixr = tile_x * 14 - p.pad + n;
        unsigned roff[3];
#pragma unroll
        for (int r = 0; r < 3; ++r) {
            const bool ok = (unsigned)(iyr + r) < (unsigned)p.H && (unsigned)ixr < (unsigned)p.W;
            const unsigned m = ok ? 0xffffffffu : 0u;
            roff[r] = ((unsigned)((iyr + r) * p.W + ixr) * 4u & m) | ((unsigned)OOB_OFFSET & ~m);
        }
        float rowv[CG][3];
#pragma unroll
        for (int g = 0; g < CG; ++g) {
#pragma unroll
            for (int r = 0; r < 3; ++r)
                rowv[g][r] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(
                    in_rsrc, (int)(roff[r] + base + (unsigned)(4 * g) * chan_bytes), 0, 0));
            __builtin_amdgcn_sched_barrier(0);
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int g = 0; g < CG; ++g)
#pragma unroll
            for (int r = 0; r < 3; ++r) {
                const int v = __builtin_bit_cast(int, rowv[g][r]);
                b[g][r * 3 + 0] = rowv[g][r];
                // row_shl:1 / row_shl:2 within the 16 lanes of a quarter: lane n takes the value of lane n+1 / n+2
                b[g][r * 3 + 1] = __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, v, 0x101, 0xf, 0xf, true));
                b[g][r * 3 + 2] = __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, v, 0x102, 0xf, 0xf, true));
            }
    } else {
        // byte offset of every tap inside one channel, or the out-of-range offset (branch-free: row and column tests apart)
        const unsigned off0 = (unsigned)(iy0 * p.W + ix0) * 4u;
        unsigned rmask[3], cmask[3];
#pragma unroll
        for (int r = 0; r < 3; ++r) {
            rmask[r] = ((unsigned)(iy0 + r) < (unsigned)p.H && live) ? 0xffffffffu : 0u;
            cmask[r] = ((unsigned)(ix0 + r) < (unsigned)p.W) ? 0xffffffffu : 0u;
        }
        unsigned toff[9];
#pragma unroll
        for (int r = 0; r < 3; ++r)
#pragma unroll
            for (int c = 0; c < 3; ++c) {
                const unsigned m = rmask[r] & cmask[c];
                toff[r * 3 + c] = ((off0 + (unsigned)r * rowb + (unsigned)c * 4u) & m) | ((unsigned)OOB_OFFSET & ~m);
            }
#pragma unroll
        for (int g = 0; g < CG; ++g) {
#pragma unroll
            for (int t = 0; t < 9; ++t)   // (the whole offset goes through the range-checked vector operand)
                b[g][t] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(
                    in_rsrc, (int)(toff[t] + base + (unsigned)(4 * g) * chan_bytes), 0, 0));
            __builtin_amdgcn_sched_barrier(0);   // requests in the order the MFMAs consume them
        }
    }
    __builtin_amdgcn_sched_barrier(0);
    TDC_STAMP(1);   // every request issued (window form: the input has crossed the LDS)
    f4_t acc0 = (f4_t){0.0f, 0.0f, 0.0f, 0.0f}, acc1 = (f4_t){0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int g = 0; g < CG; ++g) {
#pragma unroll
        for (int t = 0; t < 9; ++t) {
            const float av = t < 4 ? a0[g][t] : t < 8 ? a1[g][t - 4] : a8[g];
            if (t & 1) acc1 = __builtin_amdgcn_mfma_f32_16x16x4f32(av, b[g][t], acc1, 0, 0, 0);
            else acc0 = __builtin_amdgcn_mfma_f32_16x16x4f32(av, b[g][t], acc0, 0, 0, 0);
        }
        __builtin_amdgcn_sched_barrier(0);   // group by group, as the data arrives
    }
    f4_t acc = acc0 + acc1;
    TDC_STAMP(4);   // MFMAs issued (the last results may still be in the pipe)
    // lane l holds rows 4*(l/16) .. +3 (output channels) of column l%16 (pixel); the slices of a channel block are
    // added by its first wave, in slice order
    const int pp = oy * p.Wo + ox;
    if (p.WK > 1) {
#pragma unroll
        for (int i = 0; i < 4; ++i) lds[(wave * 4 + i) * 64 + lane] = acc[i];
        __syncthreads();
        TDC_STAMP(5);   // everybody's partial blocks are in LDS
        if constexpr (MODE == 0) {
            if (p.WK >= 4) {
                // the first four waves of a channel block share the final sum and the store: wave w finishes
                // accumulator register w (output channel 4k + w of its lanes' pixels)
                if (wki < 4 && live)
                    finish_one_channel(sum_slices(lds, wave - wki, p.WK, wki, lane), mblk * 16 + 4 * k + wki, p.N, p.P, pp,
                                       p.bias, resid, p.relu, out);
                TDC_STAMP(6);   // stores issued
                TDC_STAMP_FLUSH(p, logical, wave, lane);
                return;
            }
        }
        if (wki == 0) {
#pragma unroll
            for (int i = 0; i < 4; ++i) acc[i] = sum_slices(lds, wave, p.WK, i, lane);
        }
    }
    if constexpr (TAIL) {
        // Fused 1x1 tail, out2 = W2 * act(conv + bias): the workgroup owns every output channel of the convolution
        // (the host guarantees it).  The finished 16-pixel columns are parked in LDS as f[channel][pixel] — the B operand
        // of a second small GEMM whose A operand, the tail's packed weights, comes from global memory — and its
        // 16x16 output blocks are dealt to all waves.
        float *f = lds + p.tail_f_off;
        const int LD = p.tail_ld;
        if (wki == 0) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int ml = wmi * 16 + 4 * k + i;
                const int ch = by * 16 * p.WM + ml;
                float val = acc[i];
                if (p.bias && ch < p.N) val += p.bias[ch];
                if (p.relu) val = fmaxf(val, 0.0f);
                f[ml * LD + n] = val;
            }
        }
        __syncthreads();
        const int nwaves = p.WM * p.WK;
        for (int blk = wave; blk < p.tail_mblk; blk += nwaves) {
            const float *wa = p.tail_w + (size_t)blk * p.tail_ng * 64 + lane;
            const float *fb = f + k * LD + n;
            // (bias and residual of this block are requested before the small GEMM and arrive under it)
            const int n20 = blk * 16 + 4 * k;
            const long long ppc = live ? pp : 0;
            float tbv[4] = {0.0f, 0.0f, 0.0f, 0.0f}, trv[4] = {0.0f, 0.0f, 0.0f, 0.0f};
            if (p.tail_bias) {
#pragma unroll
                for (int v = 0; v < 4; ++v) tbv[v] = p.tail_bias[min(n20 + v, p.tail_N - 1)];
            }
            if (resid) {
#pragma unroll
                for (int v = 0; v < 4; ++v) trv[v] = resid[(long long)min(n20 + v, p.tail_N - 1) * p.P + ppc];
            }
            f4_t acc2 = {0.0f, 0.0f, 0.0f, 0.0f};
            for (int g0 = 0; g0 < p.tail_ng; g0 += 4) {
                float ta[4], tb[4];
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    const int g = min(g0 + u, p.tail_ng - 1);
                    ta[u] = wa[g * 64];
                    tb[u] = fb[g * 4 * LD];
                }
#pragma unroll
                for (int u = 0; u < 4; ++u)
                    if (g0 + u < p.tail_ng) acc2 = __builtin_amdgcn_mfma_f32_16x16x4f32(ta[u], tb[u], acc2, 0, 0, 0);
            }
            if (live) {
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    const int n2 = n20 + v;
                    if (n2 < p.tail_N) {
                        float val = acc2[v] + tbv[v];
                        val += trv[v];
                        if (p.tail_relu) val = fmaxf(val, 0.0f);
                        store_out(out + ((long long)n2 * p.P + pp), val);
                    }
                }
            }
        }
        return;
    }
    if constexpr (SPLIT) {
        if (!stream_join_slices(p, lds, acc, wki == 0 && live, mblk * 16 + 4 * k, pp, img, slice, by, bx)) return;
    }
    if (wki == 0 && live) finish_four_channels(acc, mblk * 16 + 4 * k, p.N, p.P, pp, p.bias, resid, p.relu, out);
    TDC_STAMP(6);   // stores issued
    TDC_STAMP_FLUSH(p, logical, wave, lane);
}

// ---------------------------------------------------------------------------
// The streamed 3x3 kernel with NB pixel blocks per wave (tile.alg = 4, tile.nb = 2 or 4; stride 1, rows of 14 pixels).
// The 16 x 16 block of the plain kernel reads the weights of its 16 channels once per 16 pixels and moves 30 times the
// algorithmic bytes through the L2s on the mid-size layers (64 -> 64 @56x56: 54 MB for 1.75 MB), which is what bounds
// them.  Here a workgroup owns NB horizontally adjacent 14-pixel row tiles: a wave still takes CG groups of four input
// channels and requests everything up front, but every weight operand it holds feeds NB MFMAs, one per pixel block,
// so the weights cross the L2 -> CU path NB times less often.  Per group and block a lane requests three values (one
// per filter row; the three taps of a row are lane shifts, as in the plain kernel's row mode).  The partial blocks
// of the WK waves meet in LDS as [wave][block][register][lane] and ALL threads share the final sum (in wave order, so
// the result does not depend on timing) and the store.
// ---------------------------------------------------------------------------
// WIN (tile.alg = 6): the three input rows under all NB blocks — 14 NB + 2 columns, from the 4-column boundary at or left
// of the first — come as two (NB = 2) or three (NB = 4) 128-bit requests per group of channels instead of 3 NB 32-bit
// ones, through a wave-private piece of LDS, from which every lane reads the nine taps of each of its blocks.
template <int CG, int NB, bool WIN>
__global__ void __launch_bounds__(1024) tdc_conv3x3_stream_rownb_kernel(const ConvKParams p) {
    extern __shared__ __align__(16) float lds[];
    TDC_STAMP_DECL;
    TDC_STAMP(0);   // entry
    touch_kernel_arguments();
    TDC_STAMP(7);   // every line of the kernel arguments is in the scalar cache
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int logical = (int)(blockIdx.x & 7u) * p.xcd_chunk + (int)(blockIdx.x >> 3);
    if (logical >= p.n_wg) return;
    const int q1 = fdiv(logical, p.fd_g1);
    const int r1 = logical - q1 * p.fd_g1.d;
    const int img = fdiv(q1, p.fd_g2);
    const int r2 = q1 - img * p.fd_g2.d;
    const int bx = p.channel_major ? r1 : r2;  // pixel tile of the workgroup: NB blocks side by side
    const int by = p.channel_major ? r2 : r1;  // channel tile
    const int tile_y = fdiv(bx, p.fd_ntx);     // = output row (tiles are one row high)
    const int tile_x = bx - tile_y * p.ntx;
    const ImageBase image = image_base(p, img);
    const float *__restrict__ in = image.in;
    float *__restrict__ out = image.out;
    const float *__restrict__ resid = image.resid;
    const __amdgpu_buffer_rsrc_t in_rsrc =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(in), (short)0, (int)p.in_image_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t w_rsrc =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(p.wpk), (short)0, (int)p.wpk_bytes, 0x00020000);

    // wave = (channel block of the workgroup) * WK + (slice of the input channels)
    const int wmi = fdiv(wave, p.fd_wk);
    const int wki = wave - wmi * p.WK;
    // weights first: they depend on nothing but the channel block and the wave (packed as for the plain kernel)
    const int a_soff = (((by * p.WM + wmi) * (p.CCH >> 2)) + wki * CG) * 2304;
    f4_t a0[CG], a1[CG];
    float a8[CG];
#pragma unroll
    for (int g = 0; g < CG; ++g) {
        a0[g] = __builtin_bit_cast(f4_t, __builtin_amdgcn_raw_buffer_load_b128(w_rsrc, lane * 16, a_soff + g * 2304, 0));
        a1[g] = __builtin_bit_cast(f4_t, __builtin_amdgcn_raw_buffer_load_b128(w_rsrc, lane * 16, a_soff + g * 2304 + 1024, 0));
        a8[g] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(w_rsrc, lane * 4, a_soff + g * 2304 + 2048, 0));
    }
    __builtin_amdgcn_sched_barrier(0);

    const int k = lane >> 4, n = lane & 15;
    const unsigned chan_bytes = (unsigned)(p.H * p.W) * 4u;
    const unsigned base = (unsigned)(wki * (4 * CG) + k) * chan_bytes;   // this lane's first channel
    // lane n of a quarter: input column (block's first column - pad + n) of the three input rows under the output row
    const int iyr = tile_y - p.pad;
    float rowv[WIN ? 1 : CG][NB][3];
    float bwin[WIN ? CG : 1][NB][9];
    if constexpr (WIN) {
        // slot = row * win_L + segment of four columns from ixa on; lane n of a quarter takes slot q * 16 + n of its channel
        constexpr int NREQ = NB == 2 ? 2 : 3;
        const int L = p.win_L, NS = p.win_ns;
        const int ixw0 = tile_x * NB * 14 - p.pad;
        const int ixa = (ixw0 >> 2) << 2;                 // (arithmetic shift: floors negative columns too)
        float *win = lds + p.win_off + wave * (CG * 4 * NS) + k * NS;     // this lane's channel of group 0
        unsigned soff[NREQ];
        int wslot[NREQ], ncol[NREQ];
#pragma unroll
        for (int q = 0; q < NREQ; ++q) {
            const int slot = q * 16 + n;
            const int row = fdiv(slot, p.fd_winL);
            const int cs = ixa + 4 * (slot - row * L);
            const bool ok = row < 3 && (unsigned)(iyr + row) < (unsigned)p.H && (unsigned)cs < (unsigned)p.W;
            const unsigned m = ok ? 0xffffffffu : 0u;
            soff[q] = ((unsigned)((iyr + row) * p.W + cs) * 4u & m) | ((unsigned)OOB_OFFSET & ~m);
            wslot[q] = row < 3 ? slot * 4 : -1;
            ncol[q] = p.W - cs;
        }
        f4_t wv[CG][NREQ];
#pragma unroll
        for (int g = 0; g < CG; ++g) {
#pragma unroll
            for (int q = 0; q < NREQ; ++q)
                wv[g][q] = __builtin_bit_cast(f4_t, __builtin_amdgcn_raw_buffer_load_b128(
                    in_rsrc, (int)(soff[q] + base + (unsigned)(4 * g) * chan_bytes), 0, 0));
            __builtin_amdgcn_sched_barrier(0);   // requests in the order the MFMAs consume them
        }
        __builtin_amdgcn_sched_barrier(0);
        TDC_STAMP(1);   // every request issued
#pragma unroll
        for (int g = 0; g < CG; ++g)
#pragma unroll
            for (int q = 0; q < NREQ; ++q)
                if (wslot[q] >= 0) {
                    f4_t v = wv[g][q];
#pragma unroll
                    for (int e = 1; e < 4; ++e) v[e] = e < ncol[q] ? v[e] : 0.0f;
                    *reinterpret_cast<f4_t *>(win + g * 4 * NS + wslot[q]) = v;
                }
        // (the lanes of a wave exchange data through LDS here: its LDS instructions complete in order, and nothing may be
        //  moved across this point by the compiler)
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        const float *rd = win + min(n, 13) + (ixw0 - ixa);   // (lanes 14 and 15 of a block re-read pixel 13; never stored)
#pragma unroll
        for (int g = 0; g < CG; ++g)
#pragma unroll
            for (int blk = 0; blk < NB; ++blk)
#pragma unroll
                for (int r = 0; r < 3; ++r)
#pragma unroll
                    for (int c = 0; c < 3; ++c) bwin[g][blk][r * 3 + c] = rd[g * 4 * NS + r * (4 * L) + blk * 14 + c];
    } else {
        unsigned roff[NB][3];
#pragma unroll
        for (int blk = 0; blk < NB; ++blk) {
            const int ixr = (tile_x * NB + blk) * 14 - p.pad + n;
#pragma unroll
            for (int r = 0; r < 3; ++r) {
                const bool ok = (unsigned)(iyr + r) < (unsigned)p.H && (unsigned)ixr < (unsigned)p.W;
                const unsigned m = ok ? 0xffffffffu : 0u;
                roff[blk][r] = ((unsigned)((iyr + r) * p.W + ixr) * 4u & m) | ((unsigned)OOB_OFFSET & ~m);
            }
        }
#pragma unroll
        for (int g = 0; g < CG; ++g) {
#pragma unroll
            for (int blk = 0; blk < NB; ++blk)
#pragma unroll
                for (int r = 0; r < 3; ++r)
                    rowv[g][blk][r] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(
                        in_rsrc, (int)(roff[blk][r] + base + (unsigned)(4 * g) * chan_bytes), 0, 0));
            __builtin_amdgcn_sched_barrier(0);   // requests in the order the MFMAs consume them
        }
        __builtin_amdgcn_sched_barrier(0);
        TDC_STAMP(1);   // every request issued
    }
    f4_t acc[NB];
#pragma unroll
    for (int blk = 0; blk < NB; ++blk) acc[blk] = (f4_t){0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int g = 0; g < CG; ++g) {
#pragma unroll
        for (int r = 0; r < 3; ++r) {
#pragma unroll
            for (int c = 0; c < 3; ++c) {
                const int t = r * 3 + c;
                const float av = t < 4 ? a0[g][t] : t < 8 ? a1[g][t - 4] : a8[g];
#pragma unroll
                for (int blk = 0; blk < NB; ++blk) {
                    float bv;
                    if constexpr (WIN) {
                        bv = bwin[g][blk][t];
                    } else {
                        const int v = __builtin_bit_cast(int, rowv[g][blk][r]);
                        // row_shl:c within the 16 lanes of a quarter: lane n takes the value of lane n + c
                        bv = c == 0 ? rowv[g][blk][r]
                           : c == 1 ? __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, v, 0x101, 0xf, 0xf, true))
                                    : __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, v, 0x102, 0xf, 0xf, true));
                    }
                    acc[blk] = __builtin_amdgcn_mfma_f32_16x16x4f32(av, bv, acc[blk], 0, 0, 0);
                }
            }
        }
        __builtin_amdgcn_sched_barrier(0);   // group by group, as the data arrives
    }
    TDC_STAMP(4);   // MFMAs issued (the last results may still be in the pipe)
    // lane l of block blk holds rows 4*(l/16) .. +3 (output channels) of column l%16 (pixel)
#pragma unroll
    for (int blk = 0; blk < NB; ++blk)
#pragma unroll
        for (int i = 0; i < 4; ++i) lds[((wave * NB + blk) * 4 + i) * 64 + lane] = acc[blk][i];
    __syncthreads();
    TDC_STAMP(5);   // everybody's partial blocks are in LDS
    const int nthreads = blockDim.x;
    const int total = p.WM * NB * 256;
    for (int idx = tid; idx < total; idx += nthreads) {
        const int l = idx & 63, i = (idx >> 6) & 3;
        const int rest = idx >> 8;                     // = channel block of the workgroup * NB + pixel block
        const int cb = rest / NB, blk = rest - cb * NB;
        const float *src = lds + (((cb * p.WK) * NB + blk) * 4 + i) * 64 + l;
        const int wstride = NB * 256;
        const int ch = (by * p.WM + cb) * 16 + 4 * (l >> 4) + i;
        const int px = l & 15;
        const int ox = (tile_x * NB + blk) * 14 + px;
        const bool ok = ch < p.N && px < 14 && ox < p.Wo;
        const long long o = ok ? (long long)ch * p.P + tile_y * p.Wo + ox : 0;
        // (bias and residual are requested before the partial sums are read and arrive under those reads)
        const float bv = p.bias ? p.bias[min(ch, p.N - 1)] : 0.0f;
        const float rv = resid ? resid[o] : 0.0f;
        float val = 0.0f;
        // four reads in flight at a time; the additions stay in wave order
        for (int w0 = 0; w0 < p.WK; w0 += 4) {
            float part[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) part[u] = src[min(w0 + u, p.WK - 1) * wstride];
#pragma unroll
            for (int u = 0; u < 4; ++u)
                if (w0 + u < p.WK) val += part[u];
        }
        if (ok) {
            val += bv;
            val += rv;
            if (p.relu) val = fmaxf(val, 0.0f);
            store_out(out + o, val);
        }
    }
    TDC_STAMP(6);   // stores issued
    TDC_STAMP_FLUSH(p, logical, wave, lane);
}

// ---------------------------------------------------------------------------
// Instantiation table of the streamed kernels: KernelId -> function.
// ---------------------------------------------------------------------------
typedef void (*kernel_fn)(const ConvKParams);

template <bool AFF, int MODE>
static kernel_fn pick_stream(int nq) {
    switch (nq) {
        case 1: return tdc_conv1x1_stream_kernel<1, AFF, MODE>;
        case 2: return tdc_conv1x1_stream_kernel<2, AFF, MODE>;
        case 4: return tdc_conv1x1_stream_kernel<4, AFF, MODE>;
        case 8: return tdc_conv1x1_stream_kernel<8, AFF, MODE>;
        default: return nullptr;
    }
}

template <int INP, int MODE>
static kernel_fn pick_stream3(int groups) {
    switch (groups) {
        case 1: return tdc_conv3x3_stream_kernel<1, INP, MODE>;
        case 2: return tdc_conv3x3_stream_kernel<2, INP, MODE>;
        case 4: return tdc_conv3x3_stream_kernel<4, INP, MODE>;
        default: return nullptr;
    }
}

const void *stream_kernel_function(const KernelId &k) {
    kernel_fn fn = nullptr;
    if (k.family == KernelId::STREAM_1x1) {
        const int nq = k.p[0], mode = k.p[2];
        if (k.p[1]) fn = mode == 2 ? pick_stream<true, 2>(nq) : mode == 1 ? pick_stream<true, 1>(nq) : mode == 0 ? pick_stream<true, 0>(nq) : nullptr;
        else fn = mode == 2 ? pick_stream<false, 2>(nq) : mode == 1 ? pick_stream<false, 1>(nq) : mode == 0 ? pick_stream<false, 0>(nq) : nullptr;
    } else if (k.family == KernelId::STREAM_3x3 && k.p[3] > 1) {
        // NB pixel blocks per wave: rows of 14 pixels, plain mode only
        const int cg = k.p[0], nb = k.p[3];
        if (k.p[1] == 1 && k.p[2] == 0) {
            if (nb == 2) fn = cg == 1 ? static_cast<kernel_fn>(tdc_conv3x3_stream_rownb_kernel<1, 2, false>)
                            : cg == 2 ? static_cast<kernel_fn>(tdc_conv3x3_stream_rownb_kernel<2, 2, false>)
                            : cg == 4 ? static_cast<kernel_fn>(tdc_conv3x3_stream_rownb_kernel<4, 2, false>) : nullptr;
            if (nb == 4) fn = cg == 1 ? static_cast<kernel_fn>(tdc_conv3x3_stream_rownb_kernel<1, 4, false>)
                            : cg == 2 ? static_cast<kernel_fn>(tdc_conv3x3_stream_rownb_kernel<2, 4, false>)
                            : cg == 4 ? static_cast<kernel_fn>(tdc_conv3x3_stream_rownb_kernel<4, 4, false>) : nullptr;
        } else if (k.p[1] == 2 && k.p[2] == 0) {      // the rows of all blocks as one window through LDS
            if (nb == 2) fn = cg == 1 ? static_cast<kernel_fn>(tdc_conv3x3_stream_rownb_kernel<1, 2, true>)
                            : cg == 2 ? static_cast<kernel_fn>(tdc_conv3x3_stream_rownb_kernel<2, 2, true>)
                            : cg == 4 ? static_cast<kernel_fn>(tdc_conv3x3_stream_rownb_kernel<4, 2, true>) : nullptr;
            if (nb == 4) fn = cg == 1 ? static_cast<kernel_fn>(tdc_conv3x3_stream_rownb_kernel<1, 4, true>)
                            : cg == 2 ? static_cast<kernel_fn>(tdc_conv3x3_stream_rownb_kernel<2, 4, true>) : nullptr;
        }
    } else if (k.family == KernelId::STREAM_3x3) {
        const int cg = k.p[0], mode = k.p[2];
        if (k.p[1] == 2) fn = mode == 2 ? pick_stream3<2, 2>(cg) : mode == 1 ? pick_stream3<2, 1>(cg) : mode == 0 ? pick_stream3<2, 0>(cg) : nullptr;
        else if (k.p[1] == 1) fn = mode == 2 ? pick_stream3<1, 2>(cg) : mode == 1 ? pick_stream3<1, 1>(cg) : mode == 0 ? pick_stream3<1, 0>(cg) : nullptr;
        else fn = mode == 3 ? pick_stream3<0, 3>(cg) : mode == 2 ? pick_stream3<0, 2>(cg) : mode == 1 ? pick_stream3<0, 1>(cg)
                : mode == 0 ? pick_stream3<0, 0>(cg) : nullptr;
    }
    return reinterpret_cast<const void *>(fn);
}

}  // namespace tdc
