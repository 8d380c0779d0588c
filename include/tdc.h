/*
 * tdc.h — C ABI of the MI355X (gfx950) Tucker-convolution library.
 *
 * Plain C: pointers, ints and sizes only.  Every entry point returns a
 * tdc_status (0 = success) and never terminates the process; the text of the
 * last failure on the calling thread is available from tdc_last_error_string().
 *
 * Tensors are fp32, contiguous NCHW; weights are handed over in PyTorch's OIHW
 * order and re-packed once at set-weights time.  Activations are DEVICE
 * pointers owned by the caller; weight/bias arguments are HOST pointers.
 * `stream` is a hipStream_t passed as void* (NULL = the default stream).
 *
 * What each entry point replaces in the reference (paths relative to the
 * reference tree):
 *   tdc_conv_*      Conv::initialize / Conv::forward
 *                   (2080Ti-evaluation/EndToEnd/resnet18-tk/inc/common.h:38-69,
 *                    src/Conv.cu:2-125) and the raw generated kernel
 *                   conv2d(input, kernel, outputs)
 *                   (2080Ti-evaluation/TDC-LAYERS-ORACLE/template_benchmark_cudnn.template:365-402,490-492)
 *   tdc_tkconv_*    TkConv::initialize / TkConv::forward (common.h:158-166,
 *                   src/BasicBlock.cu:14-31) and TKConv2dC.forward /
 *                   forward_features (inference/TKConv.py:90-106)
 *   tdc_net_*       the E2E drivers and BasicBlock/Pool/Add/Concate layer objects
 *                   (2080Ti-evaluation/EndToEnd/resnet18-tk/src/main.cu:19-156, inc/common.h:70-197)
 *   tdc_model_*     compute_latency / compute_*_vol / modeling
 *                   (2080Ti-evaluation/TDC-LAYERS-MODELING/model.py:136-156,209-235)
 *                   and the occupancy probe (2080Ti-evaluation/Gen-occupancy/template.cu:277-284)
 */
#ifndef TDC_H
#define TDC_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum tdc_status {
    TDC_OK = 0,
    TDC_ERR_INVALID = 1,     /* bad argument / inconsistent descriptor          */
    TDC_ERR_UNSUPPORTED = 2, /* legal request the library has no kernel for     */
    TDC_ERR_HIP = 3,         /* a HIP runtime call failed (see error string)    */
    TDC_ERR_NOMEM = 4,       /* host or device allocation failed                */
    TDC_ERR_STATE = 5        /* call order violated (e.g. forward before weights) */
} tdc_status;

/* One convolution: out[b,n,oy,ox] = sum_{c,r,s} w[n,c,r,s] * in[b,c,oy*stride-pad+r*dil, ox*stride-pad+s*dil]
 * (cross-correlation, zero padding, groups = 1), then optionally + bias[n],
 * + residual[b,n,oy,ox], then optionally ReLU — in that order. */
typedef struct tdc_conv_desc {
    int32_t batch;
    int32_t C;          /* input channels                                      */
    int32_t N;          /* OUTPUT channels (the reference's naming; not batch) */
    int32_t H, W;       /* input height / width                                */
    int32_t KH, KW;     /* filter height / width                               */
    int32_t stride;
    int32_t pad;
    int32_t dilation;
    int32_t has_bias;
    int32_t relu;       /* fuse max(x,0) after bias/residual                   */
} tdc_conv_desc;

/* Tiling of one convolution on the gfx950 compute unit.  One workgroup computes
 * (mf*mb*wm) output channels of a th x tw tile of output pixels (th is derived:
 * as many rows as fit in the workgroup's mf*nb*wn pixel lanes); its wm*wn*wk
 * computing wavefronts split output channels, pixels and input channels; input channels
 * are staged through LDS `cch` at a time, double-buffered (alg 0-2), or requested from
 * global memory into registers all at once (alg 3-6). */
typedef struct tdc_tile {
    int32_t mf;   /* MFMA block edge: 32 (v_mfma_f32_32x32x2_f32) or 16 (16x16x4) */
    int32_t mb;   /* MFMA blocks per wave along output channels (1 or 2)        */
    int32_t nb;   /* MFMA blocks per wave along pixels (1 or 2; alg 4 and 6 also 4: the
                     workgroup's tile is nb 16-pixel blocks side by side along a row)  */
    int32_t wm;   /* waves along output channels                               */
    int32_t wn;   /* waves along pixels                                        */
    int32_t wk;   /* waves along input channels (in-workgroup split-K)          */
    int32_t cch;  /* input channels staged in LDS per pass                      */
    int32_t tw;   /* output tile width in pixels                               */
    int32_t ks;   /* workgroups sharing the LDS passes of one tile (split-K across
                     workgroups, >= 1); partials meet in a plan-owned workspace and are
                     added in index order by the last workgroup to arrive             */
    int32_t wl;   /* extra wavefronts that only issue the global->LDS copies of the
                     next pass while the wm*wn*wk others compute (0 = every wave does both) */
    int32_t alg;  /* 0 = direct convolution, weights staged in LDS next to the input.
                     1 = Winograd F(2x2,3x3) for 3x3 / stride 1 / dilation 1 convolutions: the pixel lanes hold
                         2x2-pixel output tiles (tw counts those tiles), 16 MFMAs per four input channels and 16
                         tiles instead of 36; weights read from global memory into registers; mf = 16, mb = nb = 1.
                     2 = direct 3x3 / dilation 1 convolution with the weights read from global memory straight
                         into registers (the LDS holds input only, so a pass can take more input channels);
                         mb = nb = 1, an even number of channel groups per wave and pass.
                     3 = 1x1 / pad 0 convolution (any stride; ks = 1 when the stride is above 1) with BOTH operands read from global memory straight into
                         registers: no LDS stage, one pass; a workgroup owns 16 channels x 16 pixels, its wk (<= 16)
                         waves split the input channels in runs of 16; cch = 16 * wk * {1, 2, 4, 8}
                         (eight runs per wave: wk <= 8) with ks * cch >= C and ceil(C / cch) = ks: ks > 1 deals slices
                         of cch channels to ks workgroups; mf = 16, mb = nb = wm = wn = 1, wl = 0,
                         tw = min(16, pixels).  Carries the input affine, not a fused tail.
                     4 = the same for 3x3 / dilation 1 convolutions (any stride): 16 * wm channels x a 16-pixel tile
                         of width tw per workgroup (one wave per block of 16 channels and channel slice, wm * wk <= 16),
                         the input channels in groups of four; cch = 4 * wk * {1, 2, 4}, ceil(C / cch) = ks.  With stride 1 and
                         tw = 14 the three taps of a filter row are lane shifts of one request.  Carries a fused 1x1
                         tail when wm covers every output channel (and ks = 1).
                     5 = Winograd F(2x2,3x3) with BOTH operands read from global memory straight into registers
                         (3x3 / stride 1 / pad 1 / dilation 1, even image width): a workgroup owns 16 * wm channels of
                         one tile-row block (2 output rows x 28 columns, tw = 28), its wk waves split the input
                         channels in groups of four, cch = 4 * wk * {1, 2, 3, 4} >= C (one pass; at most 16
                         waves per workgroup); the input rows are loaded as column pairs, once per lane, and the
                         patch columns a tile shares with its neighbours are lane shifts; mf = 16, mb = nb = wn = 1,
                         ks = 1, wl = 0.  No fused tail.  Offered for single images only (batch 1).
                     6 = alg 4 with the input taken as a WINDOW: every lane requests 128-bit pieces of the input rows
                         its workgroup's tile covers (two or three requests per channel instead of one per filter row
                         or tap), the pieces cross a wave-private LDS buffer, and each lane reads its nine taps back
                         from there.  3x3 / dilation 1, pad <= 1, stride <= 2; same shapes, cch / wk / ks rules and
                         fused tail as alg 4 (nb = 4: at most two channel groups per wave).  The input base address
                         and row pitch need not be 16-byte aligned: the requests are element-masked at the row ends.
                     The model offers 3 to 6 where launch and latency dominate (few channels or few pixels); the
                     staged paths keep the layers whose operands are worth sharing through the LDS. */
} tdc_tile;

typedef struct tdc_tile_info {
    tdc_tile tile;
    int32_t grid_x, grid_y, grid_z;  /* pixel tiles, channel tiles, batch * ks */
    int32_t block_threads;
    int32_t lds_bytes;
    int32_t vgpr_estimate;           /* per lane, arch+acc                     */
    int32_t waves_per_simd;          /* resident, limited by VGPR/LDS/slots    */
    int32_t wg_per_cu;
    int32_t nchunks;                 /* LDS passes over all input channels (each workgroup runs ceil(nchunks/ks)) */
    int32_t th;                      /* output tile height in pixels           */
    double flops;                    /* algorithmic 2*Ho*Wo*C*N*KH*KW*batch    */
    double bytes;                    /* algorithmic: in + out + weights once   */
    double roof_us;                  /* max(bytes/8TB/s, flops/157.3TF)        */
    double pred_us;                  /* analytic model's predicted device time */
    double pred_l2_bytes;            /* modelled L2->LDS copy traffic (halo and re-reads included) */
} tdc_tile_info;

typedef struct tdc_conv_plan tdc_conv_plan;
typedef struct tdc_tkconv tdc_tkconv;

const char *tdc_last_error_string(void);
const char *tdc_version(void);

/* ---- single convolution -------------------------------------------------- */

/* `forced_tile` NULL = let the analytic model choose.  Needs a HIP device. */
int tdc_conv_plan_create(const tdc_conv_desc *desc, const tdc_tile *forced_tile,
                         tdc_conv_plan **plan_out);
/* Host OIHW weights [N,C,KH,KW]; bias [N] or NULL (must match has_bias). */
int tdc_conv_plan_set_weights(tdc_conv_plan *plan, const float *w_oihw, const float *bias);
/* A convolution with a 1x1 convolution fused behind it in the same kernel:
 *     out = relu2?( W_tail * relu1?(conv(x) + bias) + bias_tail + residual ),   W_tail: [tail_N, desc->N]
 * where bias / relu1 are desc->has_bias / desc->relu.  The intermediate never leaves the compute unit.  This is the
 * core convolution of the reference's TKConv2dC with its last factor (inference/TKConv.py:92-94), or a bottleneck
 * convolution with the first factor of the Tucker convolution that follows it.  One workgroup must own every output
 * channel of the convolution, which limits desc->N to 256 and suits small N; out / residual are
 * [batch, tail_N, Ho, Wo].  tail_N == 0 is tdc_conv_plan_create. */
int tdc_conv_plan_create_with_tail(const tdc_conv_desc *desc, int32_t tail_N, int32_t tail_has_bias, int32_t tail_relu,
                                   const tdc_tile *forced_tile, tdc_conv_plan **plan_out);
/* Host [tail_N, desc->N] weights of the tail and its bias [tail_N] or NULL (must match tail_has_bias). */
int tdc_conv_plan_set_tail_weights(tdc_conv_plan *plan, const float *w_tail, const float *bias_tail);
/* Optional, 1x1 convolutions without padding only: y = conv(relu?(x * scale[c] + shift[c])) in one kernel —
 * the norm -> relu -> conv order of the reference's DenseNet layers (inference/densenet_inet_tt.py:36-69), where the
 * BatchNorm sits in front of the convolution and cannot be folded into its weights.  Host arrays of C floats. */
int tdc_conv_plan_set_input_affine(tdc_conv_plan *plan, const float *scale, const float *shift, int32_t relu);

/* Fuse a 1x1 convolution IN FRONT of a plan that already carries a fused tail and runs the streamed 3x3 kernel
   (tile.alg = 4, stride 1): out = tail(act(conv3x3(W_head * x))).  With the tail this is a whole TKConv
   (inference/TKConv.py:90-95: the three F.conv2d calls) in one launch; the first factor is recomputed per
   workgroup on its (TH + 2) x (TW + 2) window and never reaches memory.  The head has no bias (as the reference's
   first factor), so the core's zero padding is the head applied to zero.  w_head is host [C][head_C] (C = the plan's
   input channels); from then on the plan's input has head_C channels.  TDC_ERR_UNSUPPORTED for other plans. */
int tdc_conv_plan_set_head(tdc_conv_plan *plan, int32_t head_C, const float *w_head);
int tdc_conv_plan_query(const tdc_conv_plan *plan, tdc_tile_info *info_out);
/* Occupancy probe: what the COMPILED kernel of this plan uses and how many of its workgroups the runtime places on one
 * compute unit (hipFuncGetAttributes, hipOccupancyMaxActiveBlocksPerMultiprocessor), next to what the analytic model
 * assumed for the same tile.  The counterpart of the reference's per-candidate occupancy measurement
 * (2080Ti-evaluation/Gen-occupancy/template.cu:277-284: cudaOccupancyMaxActiveBlocksPerMultiprocessor for every
 * (TH, TW, TC) kernel).  Needs the device; launches nothing. */
typedef struct tdc_kernel_occupancy {
    int32_t kernel_vgprs;            /* registers per lane of the compiled kernel (arch + acc)          */
    int32_t kernel_static_lds_bytes;
    int32_t kernel_max_threads;      /* its launch bound                                                 */
    int32_t runtime_wg_per_cu;       /* resident workgroups per CU for this plan's block size and LDS    */
    int32_t block_threads;
    int32_t dynamic_lds_bytes;
    int32_t model_vgprs;             /* tdc_tile_info.vgpr_estimate of the plan                          */
    int32_t model_wg_per_cu;         /* tdc_tile_info.wg_per_cu of the plan                              */
} tdc_kernel_occupancy;
int tdc_conv_plan_occupancy(const tdc_conv_plan *plan, tdc_kernel_occupancy *out);
/* d_residual may be NULL.  Output need not be pre-zeroed.  Asynchronous. */
int tdc_conv_forward(tdc_conv_plan *plan, const float *d_in, const float *d_residual,
                     float *d_out, void *stream);
/* tdc_conv_forward for callers that cannot allocate device memory or hold on to plan-owned scratch: HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc.  (No counterpart in the reference, whose layer
 * objects cudaMalloc at will.)  A plan whose tile deals the input channels to several workgroups (tile.ks > 1)
 * normally keeps their partial tiles and ticket counters in buffers the plan allocated; this entry point places them
 * in a device array that is part of the library image instead (4 MiB of partial tiles, 64 KiB of counters, one copy
 * per GPU for the life of the process) and clears the counters with a fill kernel on `stream` before the launch.  It
 * calls no hipMalloc / hipFree.  TDC_ERR_UNSUPPORTED when batch * ks * N * Ho * Wo * 4 exceeds 4 MiB or the plan has
 * more than 16384 (image, channel tile, pixel tile) counters.  Results are bit-identical to tdc_conv_forward.
 * Every call on one GPU shares that GPU's array: calls that can overlap on the device (different streams, or graph
 * branches) race; serialise them.  Plans with ks = 1 use no scratch and behave exactly like tdc_conv_forward. */
int tdc_conv_forward_static_ws(tdc_conv_plan *plan, const float *d_in, const float *d_residual,
                               float *d_out, void *stream);
/* Same with explicit distances (in floats) between consecutive images of the batch, so that a tensor can be
 * a channel slice of a wider NCHW buffer; 0 = densely packed. */
int tdc_conv_forward_strided(tdc_conv_plan *plan, const float *d_in, int64_t in_batch_stride,
                             const float *d_residual, int64_t residual_batch_stride, float *d_out,
                             int64_t out_batch_stride, void *stream);
/* Measurement helper (the reference times its kernel with one cudaEvent pair
 * around a single cold launch, template_benchmark_cudnn.template:491-496): run
 * `iters` back-to-back forwards on a private stream between two hipEvents
 * recorded on that stream and return the elapsed device time of the whole batch
 * in milliseconds.  With use_graph != 0 the launches are captured into one HIP
 * graph and the timed region is a single replay of it, which removes host launch
 * cost from the figure.  Synchronises the device before and after. */
int tdc_conv_time(tdc_conv_plan *plan, const float *d_in, const float *d_residual, float *d_out,
                  int32_t iters, int32_t use_graph, float *total_ms_out);
/* The launch path by itself, timed the same way: `launches` dependent launches of a kernel that carries the
 * convolution kernels' argument block, starts `grid` workgroups of `block` threads (a multiple of 64, at most 1024)
 * and keeps every wave busy for spin_us microseconds (0 = an empty kernel) without touching memory; stream launches,
 * or one replay of a HIP graph of all of them when use_graph != 0.  The empty kernel gives the launch floor every
 * layer pays; the spinning ones show how much of a kernel's own duration hides under the launch path of its
 * successor (launch-to-launch time = max(floor, duration + overhead), not floor + duration).  The reference's harness
 * has no counterpart: it times one cold launch (template_benchmark_cudnn.template:491-496). */
int tdc_launch_floor_time(int32_t launches, int32_t use_graph, int32_t grid, int32_t block, float spin_us,
                          float *total_ms_out);
/* Same for a list of plans run one after the other: one pass over the `n`
 * plans is one step; the timed region holds `iters` steps (each step one replay of
 * a HIP graph of the n launches when use_graph != 0). */
int tdc_conv_time_many(tdc_conv_plan *const *plans, const float *const *d_ins, float *const *d_outs,
                       int32_t n, int32_t iters, int32_t use_graph, float *total_ms_out);
void tdc_conv_plan_destroy(tdc_conv_plan *plan);

/* ---- TKConv operator: 1x1 C->R1, KxK R1->R2 (stride/pad/dilation), 1x1 R2->N (+bias) */

typedef struct tdc_tkconv_desc {
    int32_t batch;
    int32_t C;        /* in_channels                      */
    int32_t R1;       /* in_rank  (hp_dict.ranks[name][1]) */
    int32_t R2;       /* out_rank (hp_dict.ranks[name][0]) */
    int32_t N;        /* out_channels                     */
    int32_t H, W;
    int32_t K;        /* core kernel size (square)        */
    int32_t stride, pad, dilation;   /* of the core conv  */
    int32_t has_bias; /* bias of the last 1x1             */
    int32_t relu;     /* fuse ReLU after the last 1x1     */
} tdc_tkconv_desc;

int tdc_tkconv_create(const tdc_tkconv_desc *desc, tdc_tkconv **op_out);
/* Host pointers: first [R1,C,1,1], core [R2,R1,K,K], last [N,R2,1,1], bias [N] or NULL. */
int tdc_tkconv_set_weights(tdc_tkconv *op, const float *first, const float *core,
                           const float *last, const float *bias);
/* Full operator; intermediates live in op-owned device buffers. */
int tdc_tkconv_forward(tdc_tkconv *op, const float *d_in, const float *d_residual,
                       float *d_out, void *stream);
int tdc_tkconv_forward_strided(tdc_tkconv *op, const float *d_in, int64_t in_batch_stride,
                               const float *d_residual, int64_t residual_batch_stride, float *d_out,
                               int64_t out_batch_stride, void *stream);
/* Same, also copying out the two intermediates (either may be NULL). */
int tdc_tkconv_forward_features(tdc_tkconv *op, const float *d_in, float *d_feat_first,
                                float *d_feat_core, float *d_out, void *stream);
/* Only the KxK core conv: d_in is [batch,R1,H,W], d_out [batch,R2,Ho,Wo]. */
int tdc_tkconv_core_forward(tdc_tkconv *op, const float *d_in, float *d_out, void *stream);
/* Launches per forward: 3; 2 when the last factor is fused behind the core convolution (done automatically
 * when the tile model predicts it faster; TDC_EXPERIMENT_NO_FUSED_TAIL in the environment turns it off); 1 when the
 * first factor is fused in front as well (small first factors on 3x3 / stride 1 cores, see tdc_conv_plan_set_head;
 * TDC_EXPERIMENT_NO_FUSED_HEAD turns it off). */
int tdc_tkconv_num_kernels(const tdc_tkconv *op);
/* which: 0 = first 1x1, 1 = core, 2 = last 1x1 */
int tdc_tkconv_query(const tdc_tkconv *op, int which, tdc_tile_info *info_out);
void tdc_tkconv_destroy(tdc_tkconv *op);

/* ---- weight files --------------------------------------------------------------------
 * Raw little-endian float32, no header: the format of the reference's load_input
 * (2080Ti-evaluation/EndToEnd/resnet18-tk/src/common.cpp:2-19).  Unlike the reference, a file whose
 * length is not exactly `count` floats is an error (TDC_ERR_INVALID), not a warning. */
int tdc_load_bin(const char *path, float *dst_host, uint64_t count);
int tdc_save_bin(const char *path, const float *src_host, uint64_t count);

/* ---- whole-network forward graphs ----------------------------------------------
 * A net is a list of operators over net-owned device tensors (tensor 0 is the
 * input), captured into one HIP graph by tdc_net_finalize and replayed by
 * tdc_net_forward.  Counterpart of the reference's native E2E drivers and layer
 * objects (2080Ti-evaluation/EndToEnd/resnet18-tk/src/main.cu:19-156,
 * src/BasicBlock.cu:14-50, inc/common.h:70-197): BatchNorm is expected folded into
 * the weights/bias handed over, ReLU and the residual add ride in the
 * convolution epilogues.  Weight pointers are HOST pointers; ids are tensor ids. */
typedef struct tdc_net tdc_net;

int tdc_net_create(int32_t batch, int32_t C, int32_t H, int32_t W, tdc_net **net_out);
/* An uninitialised tensor (e.g. a concatenation buffer that producers fill slice by slice), and a view of
 * channels [c0, c0+C) of an existing tensor that shares its memory.  Views are valid inputs, residuals and
 * destinations. */
int tdc_net_tensor(tdc_net *net, int32_t C, int32_t H, int32_t W, int32_t *out);
int tdc_net_view(tdc_net *net, int32_t id, int32_t c0, int32_t C, int32_t *out);
/* Operators.  `dst` = -1 allocates the result tensor, otherwise the result is written into that tensor/view
 * (its shape must match).  `residual` = -1 for none.  *out receives the id of the result. */
/* Dense convolution (also the classifier: a 1x1 convolution on a [C,1,1] tensor). */
int tdc_net_conv(tdc_net *net, int32_t in, int32_t N, int32_t KH, int32_t KW, int32_t stride, int32_t pad,
                 const float *w_oihw, const float *bias, int32_t residual, int32_t relu, int32_t dst, int32_t *out);
/* Tucker convolution 1x1 C->R1, KxK R1->R2 (stride, pad), 1x1 R2->N, then +bias, +residual, ReLU. */
int tdc_net_tkconv(tdc_net *net, int32_t in, int32_t R1, int32_t R2, int32_t N, int32_t K, int32_t stride,
                   int32_t pad, const float *first, const float *core, const float *last, const float *bias,
                   int32_t residual, int32_t relu, int32_t dst, int32_t *out);
/* mode 0 = max, 1 = average (window count includes padding). */
int tdc_net_pool(tdc_net *net, int32_t in, int32_t mode, int32_t k, int32_t stride, int32_t pad, int32_t dst,
                 int32_t *out);
int tdc_net_global_avgpool(tdc_net *net, int32_t in, int32_t *out);
/* Per-channel y = x*scale[c] + shift[c], then ReLU if relu != 0 (inference BatchNorm in front of a convolution). */
int tdc_net_affine(tdc_net *net, int32_t in, const float *scale, const float *shift, int32_t relu, int32_t dst,
                   int32_t *out);
/* A convolution with a 1x1 convolution (tail_N outputs) fused behind it, see tdc_conv_plan_create_with_tail:
 * out = relu2?(W_tail * relu?(conv(x) + bias) + bias_tail + residual); the result has tail_N channels. */
int tdc_net_conv_tail(tdc_net *net, int32_t in, int32_t N, int32_t KH, int32_t KW, int32_t stride, int32_t pad,
                      const float *w_oihw, const float *bias, int32_t relu, int32_t tail_N, const float *w_tail,
                      const float *bias_tail, int32_t residual, int32_t tail_relu, int32_t dst, int32_t *out);
/* Gives the convolution added last (tdc_net_conv or tdc_net_conv_tail; 1x1, no padding) a per-channel affine
 * (+ReLU) on its input, see tdc_conv_plan_set_input_affine. */
int tdc_net_set_input_affine(tdc_net *net, const float *scale, const float *shift, int32_t relu);
/* tdc_net_affine followed by a 1x1 convolution (stride 1, no padding), as ONE kernel: the affine (+ReLU when
 * affine_relu != 0) is applied to the input window inside the convolution. */
int tdc_net_affine_conv(tdc_net *net, int32_t in, const float *scale, const float *shift, int32_t affine_relu, int32_t N,
                        const float *w_oi11, const float *bias, int32_t residual, int32_t relu, int32_t dst, int32_t *out);
/* Channel concatenation of n tensors of equal height/width into a new tensor (by copy). */
int tdc_net_concat(tdc_net *net, const int32_t *ins, int32_t n, int32_t *out);
int tdc_net_tensor_shape(const tdc_net *net, int32_t id, int32_t *C, int32_t *H, int32_t *W);
int tdc_net_num_kernels(const tdc_net *net);
/* Runs the net once eagerly, then captures it; `output_id` is what tdc_net_forward returns. */
int tdc_net_finalize(tdc_net *net, int32_t output_id);
/* d_in / d_out: device buffers copied to / from the net's own input / output tensors on `stream`
 * (NULL = leave the net's tensors as they are).  Asynchronous. */
int tdc_net_forward(tdc_net *net, const float *d_in, float *d_out, void *stream);
/* hipEvents around `iters` forwards (graph replays, or eager launches when use_graph == 0); blocks. */
int tdc_net_time(tdc_net *net, int32_t iters, int32_t use_graph, float *total_ms_out);
/* Copy any tensor of the net to the host (synchronises the device). */
int tdc_net_read_tensor(tdc_net *net, int32_t id, float *host_out);
void tdc_net_destroy(tdc_net *net);

/* ---- analytic gfx950 tile model (host only; works without a GPU) ---------- */

/* Fill `info_out` (tile, launch geometry, predicted time) for a given tile;
 * returns TDC_ERR_INVALID if the tile is not launchable for this shape. */
int tdc_model_evaluate(const tdc_conv_desc *desc, const tdc_tile *tile, tdc_tile_info *info_out);
/* Enumerate every launchable tile (up to `cap`) in the model's search order;
 * *count_out receives the number written. */
int tdc_model_enumerate(const tdc_conv_desc *desc, tdc_tile *tiles_out, int32_t cap,
                        int32_t *count_out);
/* The model's pick = argmin pred_us over tdc_model_enumerate. */
int tdc_model_select(const tdc_conv_desc *desc, tdc_tile_info *info_out);
/* The pick for the convolution with a 1x1 convolution of tail_N outputs fused behind it (tiles that hold all
 * desc->N channels in one workgroup only); fails if there is none.  Compare pred_us with the sum of the two
 * separate convolutions to decide whether the fusion pays. */
int tdc_model_select_with_tail(const tdc_conv_desc *desc, int32_t tail_N, tdc_tile_info *info_out);
/* Which compiled kernel serves `tile` for this convolution (`extras` != 0: the instantiation that also carries the
 * input affine / fused 1x1 tail), by the name the compiler's resource report and the profiler print, e.g.
 * "tdc_conv_mfma_kernel<16, 1, 1, 9, 16, false>", and the registers per lane the model's occupancy term assumes for
 * it (the compiled count rounded up to the allocation granule of 8) and the waves of it that fit one SIMD (vector
 * and scalar register limits, at most 8).  Host only; any output pointer may be NULL.  With tdc_conv_plan_occupancy
 * this replaces the reference's occupancy probe (2080Ti-evaluation/Gen-occupancy/template.cu:277-284). */
int tdc_model_kernel_info(const tdc_conv_desc *desc, const tdc_tile *tile, int32_t extras, char *name_out, int32_t cap,
                          int32_t *vgprs_out, int32_t *waves_per_simd_out);
/* Calibration constants of the latency model (launch floor, copy latency and rate, barrier cost, ...;
 * the counterpart of num_sm / num_threads / a,b,c / ratio in the reference's model.py:265-266,278).
 * get: writes up to `cap` values, *count_out = how many there are.  set: all of them, all > 0; process-wide.
 * The constants only steer the CHOICE of a tile: they are read while a plan is created (or a tdc_model_* call
 * runs) and never afterwards, so existing plans keep their tile, their kernels and their results whatever is set
 * later.  set may be called while other threads create plans: evaluations in flight finish with the old values. */
int tdc_model_get_constants(double *values_out, int32_t cap, int32_t *count_out);
int tdc_model_set_constants(const double *values, int32_t count);
/* Measured tile selection, process-wide.  With classes > 0 every plan created WITHOUT a forced tile (single
 * convolutions, the plans inside a tdc_tkconv, the layers of a tdc_net) times, on the device and with synthetic
 * data, the model's favourite tile of each of the `classes` most promising tile classes (same wave split, register
 * blocking and tile width) and keeps the fastest; the answer is remembered per problem for the life of the process.
 * The counterpart of the reference's measured oracle pick (2080Ti-evaluation/TDC-LAYERS-ORACLE/
 * gen_from_occupancy.py:51-66: the fastest row of the occupancy sweep), restricted to what the model cannot tell
 * apart.  0 (the default) = the model's pick alone, no device work at plan creation.  The environment variable
 * TDC_AUTOTUNE=k sets the initial value when the library is loaded. */
int tdc_set_autotune(int32_t classes);
int tdc_get_autotune(void);

#ifdef __cplusplus
}
#endif
#endif /* TDC_H */
