// Direct convolution as an implicit GEMM on the gfx950 fp32 matrix cores.
//
//   out[n][oy][ox] = sum_{c,r,s} w[n][c][r][s] * in[c][oy*stride-pad+r*dil][ox*stride-pad+s*dil]
//
// is computed as  D[M = out channels][N = output pixels] += A[M][K] * B[K][N]
// with K running over (input channel, filter tap).
//
// One workgroup owns a TH x TW tile of output pixels and MT output channels.
// Input channels are consumed CCH at a time.  For every such pass the
// workgroup needs (a) the input window of its tile, [CCH][rows][cols] with a
// zero halo — the slab-plus-halo idea of the reference's
// load_input_2_shared_memory (2080Ti-evaluation/TDC-LAYERS-ORACLE/
// template_benchmark_cudnn.template:340-363,377-389) — and (b) the weights of
// its MT output channels for those CCH channels, pre-packed on the host in the
// per-lane order the MFMA A operand wants.  Both are copied global -> LDS by
// the buffer unit itself (`buffer_load_dwordx4 ... lds`): no register is
// involved, every wave fires all its copies of a pass at once, and lanes that
// fall on halo or padding present an out-of-range offset, which the hardware
// answers with zeros.  Two LDS stages alternate: while the MFMAs of pass i run
// out of one stage, the copies of pass i+1 land in the other.
//
// Each K-step is then two conflict-free ds_read_b32 (A: 64 consecutive words,
// B: the pixel lanes of a tile row read consecutive words, shifted by the tap)
// and MB*NB MFMAs.
//
// Three inner loops share this frame (tile.alg):
//   0  direct convolution as described, for every filter size (3x3 and 1x1 loops are specialised);
//   1  Winograd F(2x2,3x3) for 3x3 / stride 1: a lane holds a 2x2 output tile, transforms its 4x4 input patch in
//      registers and feeds 16 MFMAs per four input channels instead of 36;
//   2  the direct 3x3 loop with its A operands read from global memory (L2) straight into registers.
// In 1 and 2 the weights never pass through the LDS, which then stages input only, in longer passes.
//
// Differences from the reference kernel (template_benchmark_cudnn.template:365-402):
//   * lanes index PIXELS, output channels live in the MFMA accumulator rows; the
//     reference maps lane -> channel and broadcasts one LDS word to the warp;
//   * the split over input-channel slabs (the reference's TC / atomicAdd into a
//     pre-zeroed output) happens across the wavefronts of ONE workgroup and is
//     reduced through LDS in a fixed order: no atomics, no pre-zeroing,
//     bit-reproducible;
//   * when a layer has too few tiles to occupy the chip, the slabs can also be
//     dealt to KS workgroups: each writes its partial tile to a workspace, takes
//     a ticket from a per-tile counter, and the workgroup that draws the last
//     ticket adds the KS partials in index order — still no atomics on data
//     and no dependence on arrival order;
//   * tiles are two-dimensional (TH x TW), so the halo is paid on a short
//     perimeter instead of on whole image rows;
//   * bias, residual add and ReLU are fused into the store.
#include "conv_device.hpp"

namespace tdc {

// Copy planning.  A pass moves the input window of CCH channels and the weight
// slab of those channels into one LDS stage.  The stage is cut into blocks of
// 64 elements (E = 16 or 4 bytes each); one `buffer_load ... lds` instruction
// fills one block, lane l supplying element l.  Blocks are dealt round-robin to
// the waves.  Which input element belongs at a given LDS position does not
// depend on the pass except for a constant byte offset (CCH channels further
// on), so each lane works out the offsets of its first MAXPRE blocks once and
// keeps them in registers; halo, padding and positions past the slab get an
// out-of-range offset, which the buffer unit answers with zeros (channels past
// C fall off the end of the image buffer the same way).
constexpr int MAXPRE = 6;

__device__ __forceinline__ int input_copy_offset(const ConvKParams &p, int e, int iy0, int ix0a) {
    const int rsv = p.fd_rsv.d;  // elements per LDS row
    const int csv = p.fd_csv.d;  // elements per LDS channel slot
    // (every factor below is under 2^24 — checked on the host — so the full-rate 24-bit multiplier serves)
    const int cl = fdiv(e, p.fd_csv);
    const int rem = e - (int)__umul24(cl, csv);
    const int row = fdiv(rem, p.fd_rsv);
    const int xv = rem - (int)__umul24(row, rsv);
    const int iy = iy0 + row;
    const int ix = ix0a + (p.VW == 4 ? xv << 2 : xv);
    // Branch-free: unsigned compares fold the lower bounds in.
    const bool inb = (cl < p.CCH) & (row < p.nrows) & ((unsigned)iy < (unsigned)p.H) & ((unsigned)ix < (unsigned)p.W);
    const int off = ((int)__umul24(__umul24(cl, p.H) + iy, p.W) + ix) << 2;
    return inb ? off : OOB_OFFSET;
}

// One `buffer_load ... lds`: 64 elements of `vw` floats each from rsrc[voff + soff] to dst.
__device__ __forceinline__ void copy_block(int vw, __amdgpu_buffer_rsrc_t rsrc, float *dst, int voff, int soff) {
    if (vw == 4)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (lds_ptr_t)dst, 16, voff, soff, 0, 0);
    else
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (lds_ptr_t)dst, 4, voff, soff, 0, 0);
}

// Start the copies of pass `chunk` into the LDS stage at `stage`.  Nothing is
// waited for here.  The blocks are dealt to `dn` waves, of which this one is
// number `dw`; `use_pre` says that pre[] was computed for this dealing.
// Everything that does not depend on the lane is kept in scalar registers:
// vector ALU instructions issued next to MFMAs are not free.
// Weights: a linear copy in 16-byte elements, 1 KiB per instruction; always inside the packed buffer
// (or past its end, which reads as zero into the slack), so the block offset can ride in the scalar operand.
template <bool EXT>
__device__ __forceinline__ void issue_weights(const ConvKParams &p, __amdgpu_buffer_rsrc_t w_rsrc,
                                              float *__restrict__ stage, int lane16, int w_byte0, int dw, int dn, int chunk) {
    float *wdst = stage + p.in_stage_floats;
    const int wnblk = (p.wslab_floats + 255) >> 8;
    for (int blk = dw; blk < wnblk; blk += dn) copy_block(4, w_rsrc, wdst + (blk << 8), lane16, w_byte0 + (blk << 10));
    // The per-channel scale and shift of an input affine ride behind the weights: [pass][scale(CCH) | shift(CCH)].
    if constexpr (EXT) if (p.in_aff) {
        const __amdgpu_buffer_rsrc_t a_rsrc = __builtin_amdgcn_make_buffer_rsrc(
            const_cast<float *>(p.in_aff), (short)0, (int)(p.nchunks * p.CCH * 8), 0x00020000);
        float *adst = wdst + (wnblk << 8);
        const int anblk = (2 * p.CCH + 255) >> 8;
        for (int blk = dw; blk < anblk; blk += dn)
            copy_block(4, a_rsrc, adst + (blk << 8), lane16, chunk * p.CCH * 8 + (blk << 10));
    }
}

__device__ __forceinline__ void issue_inputs(const ConvKParams &p, __amdgpu_buffer_rsrc_t in_rsrc,
                                             float *__restrict__ stage, const int (&pre)[MAXPRE], bool use_pre, int chunk,
                                             int iy0, int ix0a, int dw, int dn, int lane) {
    const int VW = p.VW;
    const int blk_floats = 64 * VW;
    const int nblk = p.in_nblk;
    // This pass starts chunk*CCH channels further on.  The shift goes through the vector offset on
    // purpose: only that one is range-checked, and channels past C must read as zero.
    const int pass_bytes = chunk * p.CCH * p.H * p.W * 4;
    int first_computed = dw;
    if (use_pre) {
#pragma unroll
        for (int i = 0; i < MAXPRE; ++i) {
            const int blk = dw + i * dn;
            if (blk < nblk) copy_block(VW, in_rsrc, stage + blk * blk_floats, pre[i] + pass_bytes, 0);
        }
        first_computed = dw + MAXPRE * dn;
    }
    for (int blk = first_computed; blk < nblk; blk += dn)
        copy_block(VW, in_rsrc, stage + blk * blk_floats, input_copy_offset(p, (blk << 6) + lane, iy0, ix0a) + pass_bytes, 0);
}

// EXT: the instantiation also carries the fused extras (input affine, 1x1 tail).  They are compiled out of the
// plain kernels: their registers and code cost every layer 0.2-0.5 us otherwise (measured).
template <int MF, int MB, int NB, int TAPS, int MAXW, bool EXT>
__global__ void __launch_bounds__(MAXW * 64) tdc_conv_mfma_kernel(const ConvKParams p) {
    using M = Mfma<MF>;
    using acc_t = typename M::acc_t;
    constexpr int KC = M::KC;
    constexpr int NACC = M::NACC;
    constexpr bool WINO = TAPS == TAPS_WINO;
    extern __shared__ __align__(16) float lds[];

    touch_kernel_arguments();
    TDC_STAMP_DECL;
    TDC_STAMP(0);   // entry
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int nthreads = blockDim.x;
    const int nwaves = nthreads >> 6;
    // The last WL waves of the workgroup are loaders: after the first pass they issue all copies and
    // take no part in the matrix work, so the computing waves never stall on copy issue (a wave can
    // start an LDS copy only about once per hundred cycles).  WL == 0: everybody copies and computes.
    const int ncomp = nwaves - p.WL;
    const bool loader = wave >= ncomp;
    const int dw = p.WL ? wave - ncomp : wave;  // this wave's place among the dn waves that copy
    const int dn = p.WL ? p.WL : nwaves;
    const int cwave = loader ? 0 : wave;
    const int wave_nk = fdiv(cwave, p.fd_wk);  // computing wave = (wm * WN + wn) * WK + wk
    const int wk = cwave - wave_nk * p.WK;
    const int wm = fdiv(wave_nk, p.fd_wn);
    const int wn = wave_nk - wm * p.WN;

    // pixel lanes of the workgroup (>= TH*TW); a Winograd lane stands for 2x2 pixels
    const int PT = (WINO ? 4 : 1) * MF * NB * p.WN;
    const int MT = MF * MB * p.WM;
    // Workgroups are handed to the eight compute dies (XCDs, each with its own L2) round-robin by launch
    // index.  The launch is one-dimensional and the index is re-read as (die, slot), so that each die
    // works on a contiguous run of the logical order; that order has either the channel tiles of one
    // pixel tile adjacent (a die then reads its own part of the input, and all the weights) or the
    // pixel tiles of one channel tile adjacent (a die reads few weights, and all the input) — whichever
    // the host found cheaper for this layer.
    const int logical = (int)(blockIdx.x & 7u) * p.xcd_chunk + (int)(blockIdx.x >> 3);
    if (logical >= p.n_wg) return;
    const int q1 = fdiv(logical, p.fd_g1);
    const int r1 = logical - q1 * p.fd_g1.d;
    const int bz = fdiv(q1, p.fd_g2);
    const int r2 = q1 - bz * p.fd_g2.d;
    const int bx = p.channel_major ? r1 : r2;  // pixel tile
    const int by = p.channel_major ? r2 : r1;  // channel tile
    const int tile_y = fdiv(bx, p.fd_ntx);
    const int tile_x = bx - tile_y * p.ntx;
    const int oy0 = tile_y * p.TH;
    const int ox0 = tile_x * p.TW;
    const int m0 = by * MT;
    // bz = image * KS + slice of the input-channel passes
    const int img = fdiv(bz, p.fd_ks);
    const int ks = bz - img * p.KS;
    const int chunk0 = ks * p.cps;
    const int chunk1 = min(chunk0 + p.cps, p.nchunks);
    const float *__restrict__ in = p.in + (long long)img * p.in_bstride;
    float *__restrict__ out = p.out + (long long)img * p.out_bstride;
    const float *__restrict__ resid = p.resid ? p.resid + (long long)img * p.resid_bstride : nullptr;
    // Raw buffers: byte offsets at or beyond num_records read as zero.
    const __amdgpu_buffer_rsrc_t in_rsrc =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(in), (short)0, (int)p.in_image_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t w_rsrc =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(p.wpk), (short)0, (int)p.wpk_bytes, 0x00020000);

    const int iy0 = oy0 * p.stride - p.pad;
    const int ix0 = ox0 * p.stride - p.pad;
    // With 16-byte elements the window starts on a 4-float boundary of the image row.
    const int ix0a = (p.VW == 4) ? ((ix0 >> 2) << 2) : ix0;
    // Packed weights: [channel tile][pass][...]; one pass of this channel tile is contiguous.
    const unsigned w_pass_bytes = (unsigned)p.wslab_floats * 4u;
    const unsigned w_byte_base = (unsigned)by * (unsigned)p.nchunks * w_pass_bytes;

    // The weight copies of the first pass need no per-lane arithmetic: start them before anything else.
    const int lane16 = lane * 16;
    if constexpr (!WINO && TAPS != TAPS_3x3G)   // (those paths read their weights from global memory into registers)
        issue_weights<EXT>(p, w_rsrc, lds, lane16, (int)(w_byte_base + (unsigned)chunk0 * w_pass_bytes), wave, nwaves, chunk0);

    // Offsets of this lane's elements in its wave's first MAXPRE input blocks (pass 0), for the steady dealing
    // (positions past the stage decode to a channel >= CCH and so to the out-of-range offset).  With loader
    // waves the first pass is dealt differently and computes its offsets on the fly, so the table is only
    // filled afterwards, by the loaders, while the first copies are in flight.
    int pre[MAXPRE];
    const int in_nblk = p.in_nblk;
    auto fill_pre = [&]() {
#pragma unroll
        for (int i = 0; i < MAXPRE; ++i) {
            pre[i] = OOB_OFFSET;
            if (dw >= 0 && dw + i * dn < in_nblk)  // wave-uniform: no arithmetic for blocks this wave does not copy
                pre[i] = input_copy_offset(p, ((dw + i * dn) << 6) + lane, iy0, ix0a);
        }
    };
    if (p.WL == 0) {
        // Every offset goes out as a copy as soon as it is known (the scheduling barrier keeps the compiler
        // from computing the whole table first); blocks beyond the table follow.
        const int pass_bytes0 = chunk0 * p.CCH * p.H * p.W * 4;
#pragma unroll
        for (int i = 0; i < MAXPRE; ++i) {
            pre[i] = OOB_OFFSET;
            if (dw + i * dn < in_nblk) {
                pre[i] = input_copy_offset(p, ((dw + i * dn) << 6) + lane, iy0, ix0a);
                copy_block(p.VW, in_rsrc, lds + (dw + i * dn) * 64 * p.VW, pre[i] + pass_bytes0, 0);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        for (int blk = dw + MAXPRE * dn; blk < in_nblk; blk += dn)
            copy_block(p.VW, in_rsrc, lds + blk * 64 * p.VW, input_copy_offset(p, (blk << 6) + lane, iy0, ix0a) + pass_bytes0, 0);
    } else {
        issue_inputs(p, in_rsrc, lds, pre, false, chunk0, iy0, ix0a, wave, nwaves, lane);
        fill_pre();
    }
    auto issue = [&](int chunk) {
        if (dw < 0) return;
        float *stage = lds + ((chunk - chunk0) & (p.nstage - 1)) * p.stage_floats;
        const int w_byte0 = (int)(w_byte_base + (unsigned)chunk * w_pass_bytes);
        // Copy issue competes for the SIMD with other waves' MFMA streams and loses by default (measured:
        // ~330 cycles per copy instruction instead of ~115); it is short, so let it go first.
        __builtin_amdgcn_s_setprio(3);
        if constexpr (!WINO && TAPS != TAPS_3x3G) issue_weights<EXT>(p, w_rsrc, stage, lane16, w_byte0, dw, dn, chunk);
        issue_inputs(p, in_rsrc, stage, pre, true, chunk, iy0, ix0a, dw, dn, lane);
        __builtin_amdgcn_s_setprio(0);
    };

    // Per-lane LDS offset (floats) of tap (0,0) for each pixel block, channel sub-index included.
    int boff[NB];
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) {
        const int j = (wn * NB + nb) * MF + M::col(lane);
        int jy = fdiv(j, p.fd_tw);
        const int jx = j - jy * p.TW;
        jy = min(jy, p.TH - 1);  // lanes past the tile re-read its last row; they are never stored
        boff[nb] = jy * p.stride * p.RS + jx * p.stride + (ix0 - ix0a) + M::ksub(lane) * p.CS;
    }

    // Winograd: LDS offset of the top-left element of this lane's 4x4 input patch, and whether the lane's tile
    // exists (lanes past the workgroup tile re-read its last row of tiles and are never stored).
    int wino_off = 0, wino_ty = 0, wino_tx = 0;
    bool wino_live = false;
    if constexpr (WINO) {
        const int j = wn * 16 + (lane & 15);
        const int tht = p.TH >> 1;
        int ty = fdiv(j, p.fd_wtw);
        wino_tx = j - ty * (p.TW >> 1);
        wino_live = ty < tht && !loader;
        ty = min(ty, tht - 1);
        wino_ty = ty;
        wino_off = 2 * ty * p.RS + 2 * wino_tx + (ix0 - ix0a) + (lane >> 4) * p.CS;
    }
    f4_t wacc[WINO ? 16 : 1];
    if constexpr (WINO) {
#pragma unroll
        for (int x = 0; x < 16; ++x) wacc[x] = (f4_t){0.0f, 0.0f, 0.0f, 0.0f};
    }

    acc_t acc[MB][NB];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
        for (int nb = 0; nb < NB; ++nb)
#pragma unroll
            for (int v = 0; v < NACC; ++v) acc[mb][nb][v] = 0.0f;

    const int taps = (TAPS == TAPS_GENERIC) ? p.KH * p.KW : (TAPS == TAPS_3x3G) ? 9 : WINO ? 16 : TAPS;
    const int ncg_pass = p.CCH / KC;  // channel groups per pass
    const int ncgw = p.CPW / KC;      // ... of which this wave takes [wk*ncgw, (wk+1)*ncgw)

    // Winograd: the A operands come from global memory and do not depend on the staged input, so the first group
    // of every pass is requested before the wait and the barrier of that pass and is in registers when they end.
    f4_t wu0[WINO ? 4 : 1];
    auto wino_load_a = [&](int chunk, int g, f4_t(&u)[4]) {
        const int soff = (int)(w_byte_base + (unsigned)chunk * w_pass_bytes) + ((wm * ncg_pass + wk * ncgw + g) * 16) * 256;
#pragma unroll
        for (int q = 0; q < 4; ++q)
            u[q] = __builtin_bit_cast(f4_t, __builtin_amdgcn_raw_buffer_load_b128(w_rsrc, lane16, soff + q * 1024, 0));
    };
    if constexpr (WINO) {
        if (!loader) wino_load_a(chunk0, 0, wu0);
    }
    // Direct 3x3 with weights from global memory: a group is a PAIR of channel groups (18 K-steps per block, long
    // enough to cover the L2 latency one group ahead); per channel group and 16/32-row block the packed weights hold
    // [taps 0-3][lane][4] [taps 4-7][lane][4] [tap 8][lane]: two 128-bit loads and one 32-bit load per lane.
    float ga0[TAPS == TAPS_3x3G ? 18 : 1][MB];
    auto g3_load_a = [&](int chunk, int pair, float(&a)[18][MB]) {
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const int soff = (int)(w_byte_base + (unsigned)chunk * w_pass_bytes) +
                                 (((wm * MB + mb) * ncg_pass + wk * ncgw + pair * 2 + h) * 9) * 256;
                const f4_t q0 = __builtin_bit_cast(f4_t, __builtin_amdgcn_raw_buffer_load_b128(w_rsrc, lane16, soff, 0));
                const f4_t q1 = __builtin_bit_cast(f4_t, __builtin_amdgcn_raw_buffer_load_b128(w_rsrc, lane16, soff + 1024, 0));
                const float t8 = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(w_rsrc, lane * 4, soff + 2048, 0));
#pragma unroll
                for (int t = 0; t < 4; ++t) {
                    a[h * 9 + t][mb] = q0[t];
                    a[h * 9 + 4 + t][mb] = q1[t];
                }
                a[h * 9 + 8][mb] = t8;
            }
    };
    if constexpr (TAPS == TAPS_3x3G) {
        if (!loader) g3_load_a(chunk0, 0, ga0);
    }

    TDC_STAMP(1);   // first copies issued, offsets and operand addresses worked out
    for (int chunk = chunk0; chunk < chunk1; ++chunk) {
        // My copies of this pass have landed; after the barrier everybody's have, and
        // everybody is done reading the stage the next pass is about to overwrite.
        __builtin_amdgcn_s_waitcnt(0);
        if (chunk == chunk0) TDC_STAMP(2);   // my first copies have landed
        __syncthreads();
        if (chunk == chunk0) TDC_STAMP(3);   // everybody's have
        if (chunk + 1 < chunk1) issue(chunk + 1);
        if constexpr (EXT && TAPS == TAPS_1x1) {
            // Optional per-input-channel affine (+ReLU) in front of the convolution (an inference BatchNorm that
            // cannot be folded into a producer): applied in place to the freshly landed input window.  A 1x1
            // convolution without padding has no zero halo that would have to stay zero; lanes past the image and
            // channels past C are multiplied by zero weights or never stored.
            if (p.in_aff) {
                float *win = lds + ((chunk - chunk0) & (p.nstage - 1)) * p.stage_floats;
                const float *aff = win + p.in_stage_floats + ((p.wslab_floats + 255) & ~255);  // [scale(CCH) | shift(CCH)]
                const int nel = p.CCH * p.fd_csv.d;
                // four elements per thread in flight: the LDS round trips overlap
                for (int e0 = tid; e0 < nel; e0 += 4 * nthreads) {
                    if (p.VW == 4) {
                        f4_t v[4];
                        float sc[4], sh[4];
#pragma unroll
                        for (int u = 0; u < 4; ++u) {
                            const int e = min(e0 + u * nthreads, nel - 1);
                            const int cl = fdiv(e, p.fd_csv);
                            v[u] = *reinterpret_cast<f4_t *>(win + e * 4);
                            sc[u] = aff[cl];
                            sh[u] = aff[p.CCH + cl];
                        }
#pragma unroll
                        for (int u = 0; u < 4; ++u) {
#pragma unroll
                            for (int i = 0; i < 4; ++i) {
                                v[u][i] = v[u][i] * sc[u] + sh[u];
                                if (p.in_relu) v[u][i] = fmaxf(v[u][i], 0.0f);
                            }
                            if (e0 + u * nthreads < nel) *reinterpret_cast<f4_t *>(win + (e0 + u * nthreads) * 4) = v[u];
                        }
                    } else {
                        float v[4], sc[4], sh[4];
#pragma unroll
                        for (int u = 0; u < 4; ++u) {
                            const int e = min(e0 + u * nthreads, nel - 1);
                            const int cl = fdiv(e, p.fd_csv);
                            v[u] = win[e];
                            sc[u] = aff[cl];
                            sh[u] = aff[p.CCH + cl];
                        }
#pragma unroll
                        for (int u = 0; u < 4; ++u) {
                            v[u] = v[u] * sc[u] + sh[u];
                            if (p.in_relu) v[u] = fmaxf(v[u], 0.0f);
                            if (e0 + u * nthreads < nel) win[e0 + u * nthreads] = v[u];
                        }
                    }
                }
                __syncthreads();
            }
        }
        if (loader) continue;

        const float *stage = lds + ((chunk - chunk0) & (p.nstage - 1)) * p.stage_floats;
        const float *sin = stage + wk * p.CPW * p.CS;
        const float *sw[MB];
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
            sw[mb] = stage + p.in_stage_floats + (((wm * MB + mb) * ncg_pass + wk * ncgw) * taps) * 64 + lane;

        if constexpr (WINO) {
            // One group = four input channels: 16 raw patch values per lane (8 two-word LDS reads), the 16 A
            // operands (four 128-bit reads), the register transform, 16 MFMAs.  Two register sets ping-pong as
            // in the direct loops: patch and weights of group g+1 are read, and the patch transformed, between the
            // MFMAs of group g.
            static_assert(!WINO || (MF == 16 && MB == 1 && NB == 1), "Winograd path: one 16x16 block per wave");
            const float *praw = sin + wino_off;
            // A operands: straight from the packed weights in global memory (L2), 16 bytes per lane and quarter,
            // one group ahead like the patch reads; the scalar operand carries everything but the lane.
            const int RS = p.RS;
            const int gstep = KC * p.CS;
            float v0[16], v1[16];
            f4_t u1[4];
            auto load_patch = [&](int g, float(&v)[16]) {
                const float *b = praw + g * gstep;
                float d[4][4];
#pragma unroll
                for (int r = 0; r < 4; ++r)
#pragma unroll
                    for (int c = 0; c < 4; ++c) d[r][c] = b[r * RS + c];
                float tr[4][4];   // B^T d: rows
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    tr[0][c] = d[0][c] - d[2][c];
                    tr[1][c] = d[1][c] + d[2][c];
                    tr[2][c] = d[2][c] - d[1][c];
                    tr[3][c] = d[1][c] - d[3][c];
                }
#pragma unroll
                for (int i = 0; i < 4; ++i) {   // (B^T d) B: columns
                    v[i * 4 + 0] = tr[i][0] - tr[i][2];
                    v[i * 4 + 1] = tr[i][1] + tr[i][2];
                    v[i * 4 + 2] = tr[i][2] - tr[i][1];
                    v[i * 4 + 3] = tr[i][1] - tr[i][3];
                }
            };
            auto mfma_group = [&](const float(&v)[16], const f4_t(&u)[4]) {
#pragma unroll
                for (int x = 0; x < 16; ++x)
                    wacc[x] = __builtin_amdgcn_mfma_f32_16x16x4f32(u[x >> 2][x & 3], v[x], wacc[x], 0, 0, 0);
            };
            auto interleave = [&]() {
#pragma unroll
                for (int x = 0; x < 4; ++x) {
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);  // MFMA
                    __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);  // weight load
                }
#pragma unroll
                for (int x = 0; x < 8; ++x) {
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);  // MFMA
                    __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);  // LDS read
                }
#pragma unroll
                for (int x = 0; x < 4; ++x) {
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                    __builtin_amdgcn_sched_group_barrier(0x002, 8, 0);  // the transform's vector ALU work
                }
            };
            load_patch(0, v0);   // (its A operands are already on their way, or here)
            for (int g = 0; g + 1 < ncgw; g += 2) {
                __builtin_amdgcn_sched_barrier(0);
                wino_load_a(chunk, g + 1, u1);
                load_patch(g + 1, v1);
                mfma_group(v0, wu0);
                interleave();
                __builtin_amdgcn_sched_barrier(0);
                wino_load_a(chunk, min(g + 2, ncgw - 1), wu0);
                load_patch(min(g + 2, ncgw - 1), v0);
                mfma_group(v1, u1);
                interleave();
                __builtin_amdgcn_sched_barrier(0);
            }
            if (ncgw & 1) mfma_group(v0, wu0);
            if (chunk + 1 < chunk1) wino_load_a(chunk + 1, 0, wu0);
        } else if constexpr (TAPS == TAPS_3x3G) {
            const int npairs = ncgw >> 1;   // (the host only offers this path for an even number of channel groups)
            float a1[18][MB], b0[18][NB], b1[18][NB];
            auto load_b = [&](int pair, float(&b)[18][NB]) {
#pragma unroll
                for (int h = 0; h < 2; ++h) {
                    const float *lgrp = sin + (pair * 2 + h) * KC * p.CS;
#pragma unroll
                    for (int r = 0; r < 3; ++r)
#pragma unroll
                        for (int nb = 0; nb < NB; ++nb) {
                            const float *lrow = lgrp + boff[nb] + r * p.RS;
#pragma unroll
                            for (int c = 0; c < 3; ++c) b[h * 9 + r * 3 + c][nb] = lrow[c];
                        }
                }
            };
            auto mfma_pair = [&](const float(&a)[18][MB], const float(&b)[18][NB]) {
#pragma unroll
                for (int t = 0; t < 18; ++t)
#pragma unroll
                    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
                        for (int nb = 0; nb < NB; ++nb) acc[mb][nb] = M::run(a[t][mb], b[t][nb], acc[mb][nb]);
            };
            auto interleave = [&]() {
#pragma unroll
                for (int t = 0; t < 6; ++t) {
                    __builtin_amdgcn_sched_group_barrier(0x008, MB * NB, 0);  // MFMA
                    __builtin_amdgcn_sched_group_barrier(0x020, MB, 0);       // weight loads
                    __builtin_amdgcn_sched_group_barrier(0x100, NB, 0);       // LDS reads
                }
#pragma unroll
                for (int t = 6; t < 18; ++t) {
                    __builtin_amdgcn_sched_group_barrier(0x008, MB * NB, 0);
                    __builtin_amdgcn_sched_group_barrier(0x100, NB, 0);
                }
            };
            load_b(0, b0);   // (the weights of the first pair are already on their way, or here)
            for (int pp = 0; pp + 1 < npairs; pp += 2) {
                __builtin_amdgcn_sched_barrier(0);
                g3_load_a(chunk, pp + 1, a1);
                load_b(pp + 1, b1);
                mfma_pair(ga0, b0);
                interleave();
                __builtin_amdgcn_sched_barrier(0);
                g3_load_a(chunk, min(pp + 2, npairs - 1), ga0);
                load_b(min(pp + 2, npairs - 1), b0);
                mfma_pair(a1, b1);
                interleave();
                __builtin_amdgcn_sched_barrier(0);
            }
            if (npairs & 1) mfma_pair(ga0, b0);
            if (chunk + 1 < chunk1) g3_load_a(chunk + 1, 0, ga0);
        } else if constexpr (TAPS == TAPS_3x3) {
            // dilation 1: the column tap is an immediate offset of the LDS read, the row tap one of
            // three per-lane row addresses.  Two register sets ping-pong: the operands of channel
            // group g+1 are read from LDS before the MFMAs of group g are issued, so the matrix pipe
            // does not wait for LDS latency (one group is 9*MB*NB MFMAs deep).  The scheduling
            // barriers keep the compiler from sinking the reads back to their first use.
            float a0[9][MB], b0[9][NB], a1[9][MB], b1[9][NB];
            auto load_group = [&](int g, float(&a)[9][MB], float(&b)[9][NB]) {
                const float *lgrp = sin + g * KC * p.CS;
#pragma unroll
                for (int r = 0; r < 3; ++r) {
#pragma unroll
                    for (int nb = 0; nb < NB; ++nb) {
                        const float *lrow = lgrp + boff[nb] + r * p.RS;
#pragma unroll
                        for (int s = 0; s < 3; ++s) b[r * 3 + s][nb] = lrow[s];
                    }
                }
#pragma unroll
                for (int t = 0; t < 9; ++t)
#pragma unroll
                    for (int mb = 0; mb < MB; ++mb) a[t][mb] = sw[mb][(g * 9 + t) * 64];
            };
            auto mfma_group = [&](const float(&a)[9][MB], const float(&b)[9][NB]) {
#pragma unroll
                for (int t = 0; t < 9; ++t)
#pragma unroll
                    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
                        for (int nb = 0; nb < NB; ++nb) acc[mb][nb] = M::run(a[t][mb], b[t][nb], acc[mb][nb]);
            };
            // One scheduling region = the MFMAs of one group next to the LDS reads of the following one,
            // interleaved: a wave issues in order, so reads issued in one batch would leave the matrix
            // pipe idle for as long as the batch takes to issue.
            auto interleave = [&]() {
#pragma unroll
                for (int t = 0; t < 9; ++t) {
                    __builtin_amdgcn_sched_group_barrier(0x008, MB * NB, 0);  // MFMA
                    __builtin_amdgcn_sched_group_barrier(0x100, MB + NB, 0);  // LDS reads
                }
            };
            load_group(0, a0, b0);
            for (int g = 0; g + 1 < ncgw; g += 2) {
                __builtin_amdgcn_sched_barrier(0);
                load_group(g + 1, a1, b1);
                mfma_group(a0, b0);
                interleave();
                __builtin_amdgcn_sched_barrier(0);
                load_group(min(g + 2, ncgw - 1), a0, b0);
                mfma_group(a1, b1);
                interleave();
                __builtin_amdgcn_sched_barrier(0);
            }
            if (ncgw & 1) mfma_group(a0, b0);
        } else if constexpr (TAPS == TAPS_1x1) {
            // Same ping-pong and interleave, a group being four K-steps (channel groups).  All operand
            // addresses are running pointers: one vector add per pointer and group, immediate offsets
            // inside the group (A) or one pointer per K-step of the group (B, whose stride is a run-time
            // value).  The pointers stop at the last whole group, so the look-ahead past it re-reads
            // that group; the K-steps that do not fill a group come afterwards, one by one.
            constexpr int G = 4;
            float a0[G][MB], b0[G][NB], a1[G][MB], b1[G][NB];
            const int ngrp = ncgw / G;
            const int kstride = KC * p.CS;  // floats between the B operands of consecutive K-steps
            const float *pa[MB];
            const float *pb[NB][G];
#pragma unroll
            for (int mb = 0; mb < MB; ++mb) pa[mb] = sw[mb];
#pragma unroll
            for (int nb = 0; nb < NB; ++nb)
#pragma unroll
                for (int t = 0; t < G; ++t) pb[nb][t] = sin + boff[nb] + t * kstride;
            int at_group = 0;
            auto load_group = [&](float(&a)[G][MB], float(&b)[G][NB]) {
#pragma unroll
                for (int t = 0; t < G; ++t) {
#pragma unroll
                    for (int mb = 0; mb < MB; ++mb) a[t][mb] = pa[mb][t * 64];
#pragma unroll
                    for (int nb = 0; nb < NB; ++nb) b[t][nb] = *pb[nb][t];
                }
                const int adv = (at_group + 1 < ngrp) ? 1 : 0;
                at_group += adv;
#pragma unroll
                for (int mb = 0; mb < MB; ++mb) pa[mb] += adv * (G * 64);
#pragma unroll
                for (int nb = 0; nb < NB; ++nb)
#pragma unroll
                    for (int t = 0; t < G; ++t) pb[nb][t] += adv * (G * kstride);
            };
            auto mfma_group = [&](const float(&a)[G][MB], const float(&b)[G][NB]) {
#pragma unroll
                for (int t = 0; t < G; ++t)
#pragma unroll
                    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
                        for (int nb = 0; nb < NB; ++nb) acc[mb][nb] = M::run(a[t][mb], b[t][nb], acc[mb][nb]);
            };
            auto interleave = [&]() {
#pragma unroll
                for (int t = 0; t < G; ++t) {
                    __builtin_amdgcn_sched_group_barrier(0x008, MB * NB, 0);  // MFMA
                    __builtin_amdgcn_sched_group_barrier(0x100, MB + NB, 0);  // LDS reads
                }
            };
            if (ngrp > 0) {
                load_group(a0, b0);
                for (int gi = 0; gi + 1 < ngrp; gi += 2) {
                    __builtin_amdgcn_sched_barrier(0);
                    load_group(a1, b1);
                    mfma_group(a0, b0);
                    interleave();
                    __builtin_amdgcn_sched_barrier(0);
                    load_group(a0, b0);
                    mfma_group(a1, b1);
                    interleave();
                    __builtin_amdgcn_sched_barrier(0);
                }
                if (ngrp & 1) mfma_group(a0, b0);
            }
            for (int g = ngrp * G; g < ncgw; ++g) {
                float a[MB], b[NB];
#pragma unroll
                for (int mb = 0; mb < MB; ++mb) a[mb] = sw[mb][g * 64];
#pragma unroll
                for (int nb = 0; nb < NB; ++nb) b[nb] = sin[g * kstride + boff[nb]];
#pragma unroll
                for (int mb = 0; mb < MB; ++mb)
#pragma unroll
                    for (int nb = 0; nb < NB; ++nb) acc[mb][nb] = M::run(a[mb], b[nb], acc[mb][nb]);
            }
        } else if constexpr (TAPS == TAPS_7x7) {
            // 7x7, dilation 1 (the stems of the networks): the 49 K-steps of a channel group fully unrolled, the
            // operands of filter row r+1 read while the MFMAs of row r run (two register sets of seven K-steps).
            for (int g = 0; g < ncgw; ++g) {
                const float *lgrp = sin + g * KC * p.CS;
                float a[2][7][MB], b[2][7][NB];
                auto load_row = [&](int r, float(&ar)[7][MB], float(&br)[7][NB]) {
#pragma unroll
                    for (int s7 = 0; s7 < 7; ++s7) {
#pragma unroll
                        for (int mb = 0; mb < MB; ++mb) ar[s7][mb] = sw[mb][(g * 49 + r * 7 + s7) * 64];
#pragma unroll
                        for (int nb = 0; nb < NB; ++nb) br[s7][nb] = lgrp[boff[nb] + r * p.RS + s7];
                    }
                };
                load_row(0, a[0], b[0]);
#pragma unroll
                for (int r = 0; r < 7; ++r) {
                    if (r + 1 < 7) load_row(r + 1, a[(r + 1) & 1], b[(r + 1) & 1]);
#pragma unroll
                    for (int s7 = 0; s7 < 7; ++s7)
#pragma unroll
                        for (int mb = 0; mb < MB; ++mb)
#pragma unroll
                            for (int nb = 0; nb < NB; ++nb)
                                acc[mb][nb] = M::run(a[r & 1][s7][mb], b[r & 1][s7][nb], acc[mb][nb]);
                    if (r + 1 < 7) {
#pragma unroll
                        for (int s7 = 0; s7 < 7; ++s7) {
                            __builtin_amdgcn_sched_group_barrier(0x008, MB * NB, 0);  // MFMA
                            __builtin_amdgcn_sched_group_barrier(0x100, MB + NB, 0);  // LDS reads of the next row
                        }
                    }
                }
            }
        } else {
            // Any filter size / dilation: taps walked at run time.
            for (int g = 0; g < ncgw; ++g) {
                const float *lgrp = sin + g * KC * p.CS;
                int t = 0;
                for (int r = 0; r < p.KH; ++r) {
                    for (int s = 0; s < p.KW; ++s, ++t) {
                        float a[MB], b[NB];
#pragma unroll
                        for (int mb = 0; mb < MB; ++mb) a[mb] = sw[mb][(g * taps + t) * 64];
#pragma unroll
                        for (int nb = 0; nb < NB; ++nb) b[nb] = lgrp[boff[nb] + r * p.dil * p.RS + s * p.dil];
#pragma unroll
                        for (int mb = 0; mb < MB; ++mb)
#pragma unroll
                            for (int nb = 0; nb < NB; ++nb) acc[mb][nb] = M::run(a[mb], b[nb], acc[mb][nb]);
                    }
                }
            }
        }
    }
    TDC_STAMP(4);   // all passes done
    // Epilogue.  `each_output(sink)` walks this thread's share of the workgroup's output tile and
    // hands (channel, pixel offset in the image, accumulated value) to the sink.
    if constexpr (WINO) {
        // Output transform Y = A^T M A, A^T = [1 1 1 0; 0 1 -1 -1], per accumulator register (= output channel):
        // all 16 positions of a tile sit in the same lane.  The 2x2 results are parked in LDS as
        // [wk][channel][pixel of the workgroup tile]; the walk below adds the WK slices in index order and stores
        // runs of consecutive pixels.
        __syncthreads();
        if (wino_live) {
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                float sr[4][2];   // M A: per row i of M
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    sr[i][0] = wacc[i * 4 + 0][v] + wacc[i * 4 + 1][v] + wacc[i * 4 + 2][v];
                    sr[i][1] = wacc[i * 4 + 1][v] - wacc[i * 4 + 2][v] - wacc[i * 4 + 3][v];
                }
                const int ml = wm * 16 + 4 * (lane >> 4) + v;
                float *dst = lds + (wk * MT + ml) * PT + (2 * wino_ty) * p.TW + 2 * wino_tx;
#pragma unroll
                for (int c = 0; c < 2; ++c) {
                    dst[c] = sr[0][c] + sr[1][c] + sr[2][c];
                    dst[p.TW + c] = sr[1][c] - sr[2][c] - sr[3][c];
                }
            }
        }
        __syncthreads();
        TDC_STAMP(5);   // output transform parked, everybody's
    } else if (p.WK > 1) {
        // Split-K across waves: park every wave's partial tile in LDS
        // ([wk][channel][pixel lane]); the walk below adds the WK slices in index order.
        __syncthreads();
        if (!loader) {
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
        }
        __syncthreads();
    }
    // With `want_addends` the bias and the residual value of every output are requested before its value is
    // assembled (all of a pixel block's at once, or ahead of the partial sums' LDS reads) and handed to the sink,
    // so that the lane pays one memory round trip and not one per load.
    auto each_output = [&](auto &&sink, bool want_value, bool want_addends) {
        const bool load_bias = want_addends && p.bias != nullptr;
        const bool load_resid = want_addends && resid != nullptr;
        if (p.WK == 1 && !WINO) {
            // Straight from the accumulators: each store instruction writes runs of
            // consecutive pixels of one output channel.
#pragma unroll
            for (int nb = 0; nb < NB; ++nb) {
                const int j = (wn * NB + nb) * MF + M::col(lane);
                const int jy = fdiv(j, p.fd_tw);
                const int jx = j - jy * p.TW;
                const int oy = oy0 + jy, ox = ox0 + jx;
                const bool pix_ok = jy < p.TH && oy < p.Ho && ox < p.Wo && !loader;
                const int pp = pix_ok ? oy * p.Wo + ox : 0;
#pragma unroll
                for (int mb = 0; mb < MB; ++mb) {
#pragma unroll
                    for (int v0 = 0; v0 < NACC; v0 += 4) {
                        float bv[4], rv[4];
#pragma unroll
                        for (int u = 0; u < 4; ++u) {
                            const int n = min(m0 + (wm * MB + mb) * MF + M::row(v0 + u, lane), p.N - 1);
                            bv[u] = load_bias ? p.bias[n] : 0.0f;
                            rv[u] = load_resid ? resid[(long long)n * p.P + pp] : 0.0f;
                        }
#pragma unroll
                        for (int u = 0; u < 4; ++u) {
                            const int n = m0 + (wm * MB + mb) * MF + M::row(v0 + u, lane);
                            if (n < p.N && pix_ok) sink(n, pp, acc[mb][nb][v0 + u], bv[u], rv[u]);
                        }
                    }
                }
            }
        } else {
            const int total = MT * PT;
            for (int idx = tid; idx < total; idx += nthreads) {
                const int ml = fdiv(idx, p.fd_pt);
                const int j = idx - ml * PT;
                const int jy = fdiv(j, p.fd_tw);
                const int jx = j - jy * p.TW;
                const int n = m0 + ml;
                const int oy = oy0 + jy, ox = ox0 + jx;
                if (n < p.N && jy < p.TH && oy < p.Ho && ox < p.Wo) {
                    const float bv = load_bias ? p.bias[n] : 0.0f;
                    const float rv = load_resid ? resid[(long long)n * p.P + oy * p.Wo + ox] : 0.0f;
                    float val = 0.0f;
                    if (want_value) {
                        // four reads in flight at a time; the additions stay in slice order
                        for (int k0 = 0; k0 < p.WK; k0 += 4) {
                            float part[4];
#pragma unroll
                            for (int u = 0; u < 4; ++u) part[u] = lds[min(k0 + u, p.WK - 1) * total + idx];
#pragma unroll
                            for (int u = 0; u < 4; ++u)
                                if (k0 + u < p.WK) val += part[u];
                        }
                    }
                    sink(n, oy * p.Wo + ox, val, bv, rv);
                }
            }
        }
    };
    auto finish = [&](int n, int pp, float val, float bv, float rv) {
        val += bv;
        val += rv;
        if (p.relu) val = fmaxf(val, 0.0f);
        store_out(out + ((long long)n * p.P + pp), val);
    };
    if constexpr (EXT) if (p.tail_w) {
        // Fused tail: a 1x1 convolution over the output channels of this one, out2 = W2 * act(conv + bias), in the
        // same kernel (the last factor of a Tucker convolution behind its core, or the first factor of the next one
        // behind a bottleneck convolution).  The workgroup owns ALL output channels of the convolution (the host
        // guarantees one channel tile and no split across workgroups).  Its tile is parked in LDS as
        // f[channel][pixel lane] — the B operand of a second, small MFMA GEMM whose A operand is the tail's packed
        // weights — and the 16x16 output blocks of that GEMM are dealt to all waves.
        float *f = lds + p.tail_f_off;
        const int LD = p.tail_ld;
        if (p.WK == 1) {
            __syncthreads();  // slower waves may still be reading the last stage
            if (!loader) {
#pragma unroll
                for (int mb = 0; mb < MB; ++mb) {
#pragma unroll
                    for (int v = 0; v < NACC; ++v) {
                        const int ml = (wm * MB + mb) * MF + M::row(v, lane);
                        const float b1 = (p.bias && ml < p.N) ? p.bias[ml] : 0.0f;
#pragma unroll
                        for (int nb = 0; nb < NB; ++nb) {
                            float val = acc[mb][nb][v] + b1;
                            if (p.relu) val = fmaxf(val, 0.0f);
                            f[ml * LD + (wn * NB + nb) * MF + M::col(lane)] = val;
                        }
                    }
                }
            }
        } else {
            const int total = MT * PT;
            for (int idx = tid; idx < total; idx += nthreads) {
                const int ml = fdiv(idx, p.fd_pt);
                const int pl = idx - ml * PT;
                const float b1 = (p.bias && ml < p.N) ? p.bias[ml] : 0.0f;
                float val = 0.0f;
                for (int k0 = 0; k0 < p.WK; k0 += 4) {
                    float part[4];
#pragma unroll
                    for (int u = 0; u < 4; ++u) part[u] = lds[min(k0 + u, p.WK - 1) * total + idx];
#pragma unroll
                    for (int u = 0; u < 4; ++u)
                        if (k0 + u < p.WK) val += part[u];
                }
                val += b1;
                if (p.relu) val = fmaxf(val, 0.0f);
                f[ml * LD + pl] = val;
            }
        }
        __syncthreads();
        const int npx = PT >> 4;                  // 16-pixel blocks of the tile
        const int nblk = p.tail_mblk * npx;       // 16x16 output blocks
        const int ksub16 = lane >> 4, px16 = lane & 15;
        for (int blk = wave; blk < nblk; blk += nwaves) {
            const int mblk = fdiv(blk, p.fd_npx);
            const int pxblk = blk - mblk * npx;
            const float *wa = p.tail_w + (size_t)mblk * p.tail_ng * 64 + lane;
            const float *fb = f + ksub16 * LD + pxblk * 16 + px16;
            const int j = pxblk * 16 + px16;
            const int jy = fdiv(j, p.fd_tw);
            const int jx = j - jy * p.TW;
            const int oy = oy0 + jy, ox = ox0 + jx;
            const bool pix_ok = jy < p.TH && oy < p.Ho && ox < p.Wo;
            const int pp = pix_ok ? oy * p.Wo + ox : 0;
            // (bias and residual of this block are requested before the small GEMM and arrive under it)
            const int n20 = mblk * 16 + 4 * ksub16;
            float tbv[4] = {0.0f, 0.0f, 0.0f, 0.0f}, trv[4] = {0.0f, 0.0f, 0.0f, 0.0f};
            if (p.tail_bias) {
#pragma unroll
                for (int v = 0; v < 4; ++v) tbv[v] = p.tail_bias[min(n20 + v, p.tail_N - 1)];
            }
            if (resid) {
#pragma unroll
                for (int v = 0; v < 4; ++v) trv[v] = resid[(long long)min(n20 + v, p.tail_N - 1) * p.P + pp];
            }
            f4_t acc2 = {0.0f, 0.0f, 0.0f, 0.0f};
            for (int g0 = 0; g0 < p.tail_ng; g0 += 4) {
                float a[4], b[4];
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    const int g = min(g0 + u, p.tail_ng - 1);
                    a[u] = wa[g * 64];
                    b[u] = fb[g * 4 * LD];
                }
#pragma unroll
                for (int u = 0; u < 4; ++u)
                    if (g0 + u < p.tail_ng) acc2 = __builtin_amdgcn_mfma_f32_16x16x4f32(a[u], b[u], acc2, 0, 0, 0);
            }
            if (pix_ok) {
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
    if (p.KS == 1) {
        if constexpr (WINO) {
            // The parked tile rows are runs of TW (even) consecutive pixels: where image width and the output
            // address allow it, every thread finishes four (or two) consecutive pixels of one channel with one wide
            // LDS read per slice and one wide store.
            const unsigned long long addr_bits =
                reinterpret_cast<unsigned long long>(p.out) | reinterpret_cast<unsigned long long>(p.resid);
            const long long stride_bits = p.out_bstride | p.resid_bstride;
            auto walk = [&](auto vec_tag) {
                using vec_t = decltype(vec_tag);
                constexpr int V = sizeof(vec_t) / sizeof(float);
                const int total_v = (MT * PT) / V;
                for (int q = tid; q < total_v; q += nthreads) {
                    const int idx = q * V;
                    const int ml = fdiv(idx, p.fd_pt);
                    const int j = idx - ml * PT;
                    const int jy = fdiv(j, p.fd_tw);
                    const int jx = j - jy * p.TW;
                    const int n = m0 + ml;
                    const int oy = oy0 + jy, ox = ox0 + jx;
                    if (n < p.N && jy < p.TH && oy < p.Ho && ox < p.Wo) {
                        // (bias and residual are requested first and arrive under the LDS reads)
                        const long long o = (long long)n * p.P + oy * p.Wo + ox;
                        const float bv = p.bias ? p.bias[n] : 0.0f;
                        vec_t rv = vec_tag;
                        if (resid) rv = *reinterpret_cast<const vec_t *>(resid + o);
                        vec_t val = *reinterpret_cast<const vec_t *>(lds + idx);
                        for (int k = 1; k < p.WK; ++k) val += *reinterpret_cast<const vec_t *>(lds + k * (MT * PT) + idx);
                        val += bv;
                        val += rv;
                        if (p.relu) {
#pragma unroll
                            for (int e = 0; e < V; ++e) val[e] = fmaxf(val[e], 0.0f);
                        }
                        store_out(out + o, val);
                    }
                }
            };
            typedef float f2_t __attribute__((ext_vector_type(2)));
            if (((p.TW | p.Wo) & 3) == 0 && (stride_bits & 3) == 0 && (addr_bits & 15ull) == 0) {
                walk(f4_t{});
                TDC_STAMP(6);   // stores issued
                TDC_STAMP_FLUSH(p, logical, wave, lane);
                return;
            }
            if ((p.Wo & 1) == 0 && (stride_bits & 1) == 0 && (addr_bits & 7ull) == 0) {
                walk(f2_t{});
                TDC_STAMP(6);
                TDC_STAMP_FLUSH(p, logical, wave, lane);
                return;
            }
        }
        each_output(finish, true, true);
        TDC_STAMP(6);
        TDC_STAMP_FLUSH(p, logical, wave, lane);
        return;
    }

    // Split-K across workgroups.  Partial tiles go to ws[image][slice][channel][pixel]; the counter of
    // this (image, channel tile, pixel tile) hands out tickets, and whoever draws the last one finds
    // all KS partials complete.  The compute dies do not share an L2, and a device-scope fence would
    // write back and invalidate a whole L2 per workgroup — tens of microseconds.  Instead every access
    // to the workspace is itself a device-scope (relaxed) atomic: the stores write through, the loads
    // bypass the die-local L2, and "my stores are done" is the plain wait below.
    const long long NP = (long long)p.N * p.P;
    float *wsz = p.ws + (long long)bz * NP;
    each_output(
        [&](int n, int pp, float val, float, float) {
            __hip_atomic_store(wsz + (long long)n * p.P + pp, val, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        },
        true, false);
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();
    unsigned *ticket = p.ctr + ((unsigned)img * p.grid_y + by) * p.grid_x + bx;
    if (tid == 0) {
        const unsigned drawn = __hip_atomic_fetch_add(ticket, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        reinterpret_cast<unsigned *>(lds)[0] = drawn;
    }
    __syncthreads();
    const unsigned drawn = reinterpret_cast<const unsigned *>(lds)[0];
    if (drawn != (unsigned)p.KS - 1u) return;
    if (tid == 0) __hip_atomic_store(ticket, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);  // for the next launch
    const float *ws0 = p.ws + (long long)img * p.KS * NP;
    each_output(
        [&](int n, int pp, float, float bv, float rv) {
            const long long o = (long long)n * p.P + pp;
            // Four loads in flight at a time; the additions stay in slice order.
            float val = 0.0f;
            for (int k0 = 0; k0 < p.KS; k0 += 4) {
                float part[4];
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    const int k = min(k0 + u, p.KS - 1);
                    part[u] = __hip_atomic_load(ws0 + k * NP + o, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                }
#pragma unroll
                for (int u = 0; u < 4; ++u)
                    if (k0 + u < p.KS) val += part[u];
            }
            finish(n, pp, val, bv, rv);
        },
        false, true);
}

// ---------------------------------------------------------------------------
// Instantiation table: KernelId (worked out on the host from tile and filter, see kernel_id_for) -> function.
// A 2x2 block grid of MFMAs per wave is built for at most 8 waves per workgroup (256 registers per lane), the
// Winograd loop for 12, everything else for 16.
// ---------------------------------------------------------------------------
typedef void (*kernel_fn)(const ConvKParams);

template <int MF, int TAPS, bool EXT>
static kernel_fn pick_mbnb(int mb, int nb) {
    if (mb == 1 && nb == 1) return tdc_conv_mfma_kernel<MF, 1, 1, TAPS, 16, EXT>;
    if (mb == 1 && nb == 2) return tdc_conv_mfma_kernel<MF, 1, 2, TAPS, 16, EXT>;
    if (mb == 2 && nb == 1) return tdc_conv_mfma_kernel<MF, 2, 1, TAPS, 16, EXT>;
    if (mb == 2 && nb == 2) return tdc_conv_mfma_kernel<MF, 2, 2, TAPS, 8, EXT>;
    return nullptr;
}

template <int TAPS, bool EXT>
static kernel_fn pick_mf(int mf, int mb, int nb) {
    if (mf == 32) return pick_mbnb<32, TAPS, EXT>(mb, nb);
    if (mf == 16) return pick_mbnb<16, TAPS, EXT>(mb, nb);
    return nullptr;
}

const void *staged_kernel_function(const KernelId &k) {
    kernel_fn fn = nullptr;
    if (k.family == KernelId::STAGED) {
        const bool ext = k.p[5] != 0;
        switch (k.p[3]) {
            case TAPS_WINO:
                if (k.p[0] == 16 && k.p[1] == 1 && k.p[2] == 1 && !ext) fn = tdc_conv_mfma_kernel<16, 1, 1, TAPS_WINO, 12, false>;
                break;
            case TAPS_3x3G:
                if (k.p[1] == 1 && k.p[2] == 1 && !ext)
                    fn = k.p[0] == 16 ? static_cast<kernel_fn>(tdc_conv_mfma_kernel<16, 1, 1, TAPS_3x3G, 16, false>)
                       : k.p[0] == 32 ? static_cast<kernel_fn>(tdc_conv_mfma_kernel<32, 1, 1, TAPS_3x3G, 16, false>) : nullptr;
                break;
            case TAPS_3x3: fn = ext ? pick_mf<TAPS_3x3, true>(k.p[0], k.p[1], k.p[2]) : pick_mf<TAPS_3x3, false>(k.p[0], k.p[1], k.p[2]); break;
            case TAPS_1x1: fn = ext ? pick_mf<TAPS_1x1, true>(k.p[0], k.p[1], k.p[2]) : pick_mf<TAPS_1x1, false>(k.p[0], k.p[1], k.p[2]); break;
            case TAPS_7x7: fn = ext ? nullptr : pick_mf<TAPS_7x7, false>(k.p[0], k.p[1], k.p[2]); break;
            case TAPS_GENERIC: fn = ext ? pick_mf<TAPS_GENERIC, true>(k.p[0], k.p[1], k.p[2]) : pick_mf<TAPS_GENERIC, false>(k.p[0], k.p[1], k.p[2]); break;
            default: break;
        }
    }
    return reinterpret_cast<const void *>(fn);
}

}  // namespace tdc
