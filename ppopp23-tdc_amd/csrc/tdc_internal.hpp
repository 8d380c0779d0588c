// Internal declarations shared by the tile model, the weight packer, the kernel
// launcher and the C ABI.  Nothing here is exported.
#pragma once

#include <cstddef>
#include <cstdint>
#include <string>
#include <vector>

#include "tdc.h"

namespace tdc {

// ---- gfx950 (MI355X) machine description used by the analytic model -------
struct Machine {
    int cus = 256;                // 8 XCDs x 32 CUs
    int xcds = 8;
    int simds_per_cu = 4;
    int max_waves_per_simd = 8;
    int vgprs_per_simd_lane = 512;   // unified arch+acc file per lane
    int lds_bytes_per_cu = 160 * 1024;
    int max_wg_threads = 1024;
    double clock_ghz = 2.4;
    double hbm_tbps = 8.0;
    double fp32_tflops = 157.3;      // MFMA fp32 dense peak
};
const Machine &machine();

// ---- launch geometry derived from (desc, tile) ----------------------------
struct Geometry {
    // The kernel's view of the input: a 1x1 / stride 1 / pad 0 convolution is
    // run on the image flattened to one row of H*W pixels.
    int He = 0, We = 0;
    int Ho = 0, Wo = 0, P = 0;       // output height/width (of the kernel's view), Ho*Wo
    int kc = 0;                      // input channels consumed per MFMA (2 or 4)
    int taps = 0;                    // KH*KW
    int ktaps = 0;                   // K-steps per channel group: taps, or 16 for Winograd F(2x2,3x3)
    int wino = 0;                    // Winograd: pixel lanes hold 2x2 output tiles
    int TWt = 0, THt = 0;            // Winograd: the workgroup tile in 2x2 tiles (TW = 2*TWt, TH = 2*THt)
    int PT = 0, MT = 0;              // pixel lanes / output channels per workgroup
    int TW = 0, TH = 0;              // output tile
    int ntx = 0, nty = 0;            // tiles across / down
    int grid_x = 0, grid_y = 0, grid_z = 0;
    int waves = 0, threads = 0;
    int cpw = 0;                     // channels per wave per LDS pass (cch / wk)
    int nchunks = 0;                 // LDS passes over all input channels
    int ks = 1;                      // workgroups sharing those passes (split-K across workgroups)
    int cps = 0;                     // passes per workgroup: ceil(nchunks / ks)
    int c_pad = 0;                   // nchunks * cch
    int VW = 1;                      // floats per element of the LDS fill (4 if We%4==0, else 1)
    int nrows = 0, ncols = 0;        // input window of one tile
    int RS = 0;                      // LDS row stride (floats)
    int CS = 0;                      // LDS channel stride (floats)
    int in_stage_floats = 0;         // cch * CS, rounded up to 4
    int wslab_floats = 0;            // weights of one pass of one channel tile
    int aff_floats = 0;              // room for the scale/shift of an input affine (1x1 convolutions without padding)
    int tail_N = 0, tail_ng = 0, tail_ld = 0, tail_f_off = 0;   // fused 1x1 tail (0 = none)
    // tile.alg = 6: the input window a wave leaves in its own piece of LDS — rows, 4-column segments per row, requests per
    // group of channels (1 or 2), floats per channel (padded so that the four channel quarters fall into different banks),
    // and where the pieces start (floats)
    int win_rows = 0, win_L = 0, win_nreq = 0, win_ns = 0, win_off = 0;
    int stage_floats = 0;
    int nstage = 1;
    int lds_bytes = 0;
    int max_waves_kernel = 0;        // launch bound of the instantiated kernel
    int channel_major = 0;           // which logical workgroup order costs fewer L2 fills (see conv_staged.hip)
    double b_ways = 1.0;             // serialisation of the B-operand LDS read by bank conflicts (1 = none)
};

// Returns false (and a reason) when the tile cannot be launched for this shape.
// tail_N > 0: a 1x1 convolution with tail_N outputs is fused behind this one (needs one channel tile, no split
// across workgroups).
bool make_geometry(const tdc_conv_desc &d, const tdc_tile &t, Geometry &g, std::string *why, int tail_N = 0);
bool check_desc(const tdc_conv_desc &d, std::string *why);

bool model_evaluate(const tdc_conv_desc &d, const tdc_tile &t, tdc_tile_info &info, std::string *why, int tail_N = 0);
std::vector<tdc_tile> model_enumerate(const tdc_conv_desc &d, int tail_N = 0);
bool model_select(const tdc_conv_desc &d, tdc_tile_info &info, std::string *why, int tail_N = 0);
int model_constants(double *out, int cap);            // returns the number of constants
bool model_set_constants(const double *in, int n);

// ---- weight packing --------------------------------------------------------
// OIHW [N,C,KH,KW] -> [channel tile][pass][M block in tile][channel group in pass][tap][64 lanes]
// in MFMA A-operand order: lane l of an entry holds
// w[tile*MT + mblk*mf + l%mf][pass*cch + cg*kc + l/mf][tap], zero outside N x C.
// tile.alg = 2 regroups the nine taps of a channel group as [taps 0-3][lane][4] [taps 4-7][lane][4] [tap 8][lane];
// tile.alg = 1 and 5 store the 16 Winograd-domain values U = G g G^T of every (n, c) as [quarter][lane][4].
size_t packed_weight_floats(const Geometry &g);
void pack_weights(const tdc_conv_desc &d, const tdc_tile &t, const Geometry &g, const float *w_oihw, float *packed);

// Division of a small non-negative integer by a run-time constant without a branch:
// q = ((n * m) >> 32) + (n & pass) with m = floor(2^32 / d) + 1, pass = 0 for d > 1 (exact whenever
// n * d < 2^32) and m = 0, pass = ~0 for d == 1.
struct FastDiv {
    unsigned m;
    int d;
    unsigned pass;
};
inline FastDiv make_fastdiv(int d) {
    FastDiv f;
    f.d = d;
    f.m = d > 1 ? (unsigned)((1ULL << 32) / (unsigned)d + 1ULL) : 0u;
    f.pass = d > 1 ? 0u : ~0u;
    return f;
}

// ---- kernel arguments ------------------------------------------------------
struct ConvKParams {
    const float *in;
    const float *wpk;
    const float *bias;
    const float *resid;
    const float *in_aff;       // optional per-input-channel affine in front of a 1x1 convolution: [pass][scale(CCH) | shift(CCH)]
    const float *tail_w;       // fused 1x1 tail: packed weights [16-row block][K-step][64 lanes], or null
    const float *tail_bias;
    const float *head_w;       // fused 1x1 head (first factor in front of a streamed 3x3 core): packed [16-row block][run of 16 channels][lane][4]
    float *out;
    float *ws;                 // partial tiles of a split across workgroups: [image][slice][N][P]
    unsigned *ctr;             // one ticket counter per (image, channel tile, pixel tile), zero between launches
    int C, H, W, N, Ho, Wo, P;
    int KH, KW, stride, pad, dil;
    int TW, TH, ntx;
    int WM, WN, WK;
    int CCH, nchunks, CPW;
    int KS, cps;               // slices across workgroups, passes per slice
    int WL;                    // loader waves (the last WL of the workgroup)
    int grid_x, grid_y;        // pixel tiles, channel tiles
    int n_wg;                  // grid_x * grid_y * batch * KS
    int xcd_chunk;             // ceil(n_wg / 8): logical workgroups per compute die
    int channel_major;         // logical order: 1 = pixel tile fastest, 0 = channel tile fastest
    FastDiv fd_g1, fd_g2;      // the fastest / second extent of the logical order
    int RS, CS, VW, nrows;
    int in_stage_floats, wslab_floats, stage_floats, nstage;
    int in_nblk;                     // in_stage_floats / (64 * VW): copy blocks of the input window per pass
    int relu;
    int in_relu;               // ReLU after the input affine
    int tail_N, tail_mblk, tail_ng, tail_relu;   // tail outputs, their 16-row blocks, K-steps (ceil(N/4)), ReLU after it
    int tail_ld, tail_f_off;   // row stride and offset (floats) of the parked tile in LDS
    int head_C, head_runs;     // fused head: its input channels, runs of 16 of them (rounded up to a multiple of 4)
    int head_mblk, head_npb;   // ... 16-row blocks of its output (the core's input channels), 16-pixel blocks of the window
    int head_ww, head_wq;      // ... window width (TW + 2) and pixels ((TH + 2) * (TW + 2))
    int head_ld, head_f_off;   // ... row stride and offset (floats) of its output in LDS
    int win_rows, win_L, win_nreq, win_ns, win_off;   // tile.alg = 6: the wave-private input window in LDS (see Geometry)
    FastDiv fd_winL;
    FastDiv fd_hww, fd_hnpb;
    FastDiv fd_npx;            // 16-pixel blocks per tile
    FastDiv fd_csv, fd_rsv;      // LDS channel slot / row, in copy elements
    FastDiv fd_tw, fd_ntx, fd_pt;
    FastDiv fd_wtw;            // Winograd: 2x2 tiles per row of the workgroup tile; streamed 1x1 with stride > 1: output row length
    FastDiv fd_wk, fd_wn, fd_ks;
    unsigned wpk_bytes;
    unsigned in_image_bytes;   // C*H*W*4: reads at or past it return zero
    long long in_bstride;      // floats between consecutive images of the input (C*H*W when dense)
    long long out_bstride;     // ... of the output (N*P when dense)
    long long resid_bstride;   // ... of the residual
#if defined(TDC_STAMPS) && TDC_STAMPS
    unsigned long long *stamps;   // profiling build: [workgroup][16 waves][8] time stamps, or null
#endif
};

// Inner loop of the staged kernel (its TAPS template argument).
enum : int { TAPS_GENERIC = 0, TAPS_1x1 = 1, TAPS_3x3 = 9, TAPS_3x3G = 10, TAPS_WINO = 16, TAPS_7x7 = 49 };

// Which kernel instantiation serves a tile: worked out on the host (no device needed), so that the tile model, the
// launcher and the occupancy probe all speak of the same function.
//   STAGED      tdc_conv_mfma_kernel<MF, MB, NB, TAPS, MAXW, EXT>     p = {MF, MB, NB, TAPS, MAXW, EXT}
//   STREAM_1x1  tdc_conv1x1_stream_kernel<NQ, AFF, MODE>              p = {NQ, AFF, MODE}
//   STREAM_3x3  tdc_conv3x3_stream_kernel<CG, INP, MODE>              p = {CG, INP, MODE, 1}   (INP: 0 taps, 1 row shifts, 2 window in LDS)
//               tdc_conv3x3_stream_rownb_kernel<CG, NB>               p = {CG, 1, 0, NB}   (NB = 2 or 4 pixel blocks per wave)
//   STREAM_WINO tdc_wino3x3_stream_kernel<CG, MAXW>                   p = {CG, MAXW}
struct KernelId {
    enum Family : int { NONE = 0, STAGED = 1, STREAM_1x1 = 2, STREAM_3x3 = 3, STREAM_WINO = 4 };
    int family = NONE;
    int p[6] = {0, 0, 0, 0, 0, 0};
};
// `extras`: the instantiation that also carries the input affine and the fused 1x1 tail.  family == NONE: no kernel.
KernelId kernel_id_for(const tdc_tile &t, int KH, int KW, int dilation, int stride, bool extras);
KernelId kernel_id_with_head(const tdc_tile &t);
// Streamed Winograd kernel (tile.alg = 5): waves per workgroup it is built for, by groups of four channels per wave (0 = none).
int wino_stream_max_waves(int groups);   // streamed 3x3 with fused 1x1 head and tail
// The kernel's name as the compiler's resource report and the profiler print it, e.g.
// "tdc_conv_mfma_kernel<16, 1, 1, 9, 16, false>".
std::string kernel_name(const KernelId &k);
// Registers per lane (arch + acc) of that instantiation as compiled, rounded up to the allocation granule of 8;
// 0 for an unknown one.  Kept in step with the compiler's report by tests/test_model.py.
int kernel_vgprs(const KernelId &k);
// Resident waves of that instantiation per SIMD, as limited by vector and scalar registers (at most 8).
int kernel_waves_per_simd(const KernelId &k);
// The function itself (nullptr if not instantiated).
const void *kernel_function(const KernelId &k);
// (its parts, one per translation unit that holds kernels: conv_staged.hip, conv_stream.hip, conv_wino_stream.hip)
const void *staged_kernel_function(const KernelId &k);
const void *stream_kernel_function(const KernelId &k);
const void *wino_stream_kernel_function(const KernelId &k);
inline const void *conv_kernel_for(const tdc_tile &t, int KH, int KW, int dilation, int stride, bool extras) {
    return kernel_function(kernel_id_for(t, KH, KW, dilation, stride, extras));
}
inline const void *conv_kernel_with_head(const tdc_tile &t) { return kernel_function(kernel_id_with_head(t)); }
// One-time per-plan set-up: the dynamic-LDS attribute (above 64 KiB) and the kernel's module function handle on the
// current device, which launch_conv launches.  hipError_t as int.
int prepare_conv_kernel(const void *fn, const Geometry &g, void **handle_out);
// Enqueue the kernel.  Returns a hipError_t as int.
int launch_conv(void *handle, const Geometry &g, const ConvKParams &kp, void *stream);

// Static scratch (a device array that lives from module load to process exit, one copy per GPU) for the partial
// tiles and ticket counters of a split across workgroups, for callers that cannot allocate.  The address is the
// CURRENT device's copy (hipGetSymbolAddress, once per device); hipError_t as int.
size_t static_scratch_ws_bytes();
size_t static_scratch_ctr_bytes();
int static_scratch_address(void **ptr_out);
// dst[0..n) = 0 with a small fill kernel (safe under stream capture, unlike hipMemsetAsync).
int launch_zero_words(unsigned *dst, int n, void *stream);
// Launch-path probe: a kernel with the convolution kernels' argument block whose waves spin for `spin_ticks` ticks of
// the 100 MHz constant clock and touch no memory.
int launch_floor_probe_handle(void **handle_out);
int launch_floor_probe(void *handle, const ConvKParams &kp, int grid, int block, int spin_ticks, void *stream);
// What the compiled kernel really uses: registers per lane, static LDS, its launch bound, and how many workgroups
// of `block_threads` threads with `dynamic_lds_bytes` of LDS the runtime places on one compute unit.
int kernel_resources(const void *fn, int block_threads, int dynamic_lds_bytes, int *vgprs, int *static_lds, int *max_threads,
                     int *max_wg_per_cu);

// Pooling / concatenation kernels of the whole-network graphs (hipError_t as int).
// Batch strides are in floats; a tensor may be a channel slice of a wider buffer.
int launch_pool2d(const float *in, long long in_bstride, float *out, long long out_bstride, int B, int C, int H, int W,
                  int Ho, int Wo, int k, int stride, int pad, int mode, void *stream);
int launch_global_avgpool(const float *in, long long in_bstride, float *out, long long out_bstride, int B, int C, int HW,
                          void *stream);
int launch_copy_channels(const float *in, long long in_bstride, float *out, long long out_bstride, int B, int C, int HW,
                         void *stream);
// out = max(in * scale[c] + shift[c], 0) (relu != 0) per channel.
int launch_affine(const float *in, long long in_bstride, float *out, long long out_bstride, const float *scale,
                  const float *shift, int B, int C, int HW, int relu, void *stream);

void set_error(const std::string &msg);
int api_fail(int status, const std::string &msg);   // records the message, returns status

}  // namespace tdc
