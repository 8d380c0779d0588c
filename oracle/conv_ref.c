/*
 * TEST INFRASTRUCTURE — CPU restatement of the reference's Tucker-convolution
 * path.  Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg
 * may load this file's shared object; the product library never does.
 *
 * What is restated (paths relative to the reference tree):
 *   ref_conv2d        the convolution every stage of TKConv2dC.forward performs
 *                     (inference/TKConv.py:90-95: F.conv2d = cross-correlation,
 *                     zero padding, groups 1) and the cuDNN descriptor the native
 *                     harness checks against (2080Ti-evaluation/TDC-LAYERS-ORACLE/
 *                     template_benchmark_cudnn.template:70-96: NCHW, OIHW filter,
 *                     CUDNN_CROSS_CORRELATION).  Accumulates in double so that it
 *                     is an arbiter between fp32 implementations, not one of them.
 *   ref_tkconv        TKConv2dC.forward (inference/TKConv.py:90-95): 1x1 C->R1,
 *                     KxK R1->R2 with stride/padding/dilation and no bias, 1x1
 *                     R2->N with bias.
 *   ref_tdc_tiled     the reference's own core-conv kernel, executed
 *                     sequentially: grid of (channel slab tc, row tile th) blocks,
 *                     threads (column tile tw, output channel n), zero-filled
 *                     shared slab [TC][TH+2][WPAD] filled at +1 column / +h_offset
 *                     row, 3x3 taps, partial sums added into a pre-zeroed output
 *                     (template_benchmark_cudnn.template:340-402 with the generated
 *                     body of gen_from_occupancy.py:67-111).  fp32 accumulation,
 *                     weights in the reference's [C][3][3][N] order.  Used to show
 *                     that on the reference's known-answer inputs (integers 0..9,
 *                     all-ones weights, template:418-428) every legal tiling gives
 *                     exactly the direct result — the `diff = 0` column of the
 *                     reference's recorded sweeps.
 *
 * Pinning: see tests/test_oracle.py (closed forms, shift/delta kernels,
 * stride-2 subsampling identity, brute-force numpy on tiny shapes, committed
 * golden vectors, and torch.nn.functional.conv2d itself).
 */
#include <stddef.h>
#include <stdlib.h>
#include <string.h>

static int out_dim(int in, int k, int stride, int pad, int dil) {
    return (in + 2 * pad - dil * (k - 1) - 1) / stride + 1;
}

/* in [B,C,H,W], w [N,C,KH,KW], bias [N] or NULL, resid [B,N,Ho,Wo] or NULL, out [B,N,Ho,Wo] */
int ref_conv2d(const float *in, const float *w, const float *bias, const float *resid, float *out,
               int B, int C, int N, int H, int W, int KH, int KW, int stride, int pad, int dil,
               int relu) {
    if (B < 1 || C < 1 || N < 1 || H < 1 || W < 1 || KH < 1 || KW < 1 || stride < 1 || pad < 0 || dil < 1)
        return 1;
    const int Ho = out_dim(H, KH, stride, pad, dil), Wo = out_dim(W, KW, stride, pad, dil);
    if (Ho < 1 || Wo < 1) return 1;
    for (int b = 0; b < B; ++b)
        for (int n = 0; n < N; ++n)
            for (int oy = 0; oy < Ho; ++oy)
                for (int ox = 0; ox < Wo; ++ox) {
                    double acc = 0.0;
                    for (int c = 0; c < C; ++c)
                        for (int r = 0; r < KH; ++r) {
                            const int iy = oy * stride - pad + r * dil;
                            if (iy < 0 || iy >= H) continue;
                            for (int s = 0; s < KW; ++s) {
                                const int ix = ox * stride - pad + s * dil;
                                if (ix < 0 || ix >= W) continue;
                                acc += (double)w[(((size_t)n * C + c) * KH + r) * KW + s] *
                                       (double)in[(((size_t)b * C + c) * H + iy) * W + ix];
                            }
                        }
                    const size_t o = (((size_t)b * N + n) * Ho + oy) * Wo + ox;
                    if (bias) acc += (double)bias[n];
                    if (resid) acc += (double)resid[o];
                    if (relu && acc < 0.0) acc = 0.0;
                    out[o] = (float)acc;
                }
    return 0;
}

/* x [B,C,H,W]; first [R1,C,1,1]; core [R2,R1,K,K]; last [N,R2,1,1]; bias [N] or NULL.
 * f1 [B,R1,H,W] and f2 [B,R2,Ho,Wo] receive the intermediates (forward_features,
 * inference/TKConv.py:97-106); out [B,N,Ho,Wo]. */
int ref_tkconv(const float *x, const float *first, const float *core, const float *last,
               const float *bias, float *f1, float *f2, float *out, int B, int C, int R1, int R2,
               int N, int H, int W, int K, int stride, int pad, int dil) {
    int rc = ref_conv2d(x, first, NULL, NULL, f1, B, C, R1, H, W, 1, 1, 1, 0, 1, 0);
    if (rc) return rc;
    rc = ref_conv2d(f1, core, NULL, NULL, f2, B, R1, R2, H, W, K, K, stride, pad, dil, 0);
    if (rc) return rc;
    const int Ho = out_dim(H, K, stride, pad, dil), Wo = out_dim(W, K, stride, pad, dil);
    return ref_conv2d(f2, last, bias, NULL, out, B, R2, N, Ho, Wo, 1, 1, 1, 0, 1, 0);
}

/* The reference kernel, block by block and thread by thread.  in [C][H][W],
 * w_oihw [N][C][3][3] (re-ordered here to the kernel's [C][3][3][N]), out
 * [N][H][W].  Requires TC | C like the reference (its loader has no channel
 * bound check).  Returns 0 on success. */
int ref_tdc_tiled(const float *in, const float *w_oihw, float *out, int C, int N, int H, int W,
                  int TH, int TW, int TC) {
    if (TH < 1 || TW < 1 || TC < 1 || C % TC != 0) return 1;
    const int THS = (H + TH - 1) / TH, TWS = (W + TW - 1) / TW, TCS = C / TC;
    const int WPAD = TWS * TW + 2;
    float *kern = (float *)malloc(sizeof(float) * (size_t)C * 9 * N);
    float *smem = (float *)malloc(sizeof(float) * (size_t)TC * (TH + 2) * WPAD);
    float *tmp = (float *)malloc(sizeof(float) * (size_t)TH * TW);
    if (!kern || !smem || !tmp) { free(kern); free(smem); free(tmp); return 2; }
    for (int c = 0; c < C; ++c)
        for (int r = 0; r < 3; ++r)
            for (int s = 0; s < 3; ++s)
                for (int n = 0; n < N; ++n)
                    kern[(size_t)c * N * 9 + r * 3 * N + s * N + n] = w_oihw[(((size_t)n * C + c) * 3 + r) * 3 + s];
    memset(out, 0, sizeof(float) * (size_t)N * H * W); /* cudaMemset before the launch */
    for (int tile = 0; tile < TCS * THS; ++tile) {
        const int tc_id = tile / THS, th_id = tile % THS;
        const int h_out_start = th_id * TH;
        const int c_offset = tc_id * TC;
        memset(smem, 0, sizeof(float) * (size_t)TC * (TH + 2) * WPAD);
        const int h_offset = (h_out_start == 0) ? 1 : 0;
        int h_padded_end = h_out_start + TH + 2;
        if (h_padded_end > H + 2) h_padded_end = H + 2;
        const int h_start = (h_out_start - 1 > 0) ? h_out_start - 1 : 0;
        const int h_end = (H < h_padded_end - 1) ? H : h_padded_end - 1;
        for (int c = 0; c < TC; ++c)
            for (int i = 0; i < (h_end - h_start) * W; ++i) {
                const int r = i / W, s = i % W;
                smem[(size_t)c * (TH + 2) * WPAD + (size_t)(h_offset + r) * WPAD + s + 1] =
                    in[(size_t)(c_offset + c) * H * W + (size_t)h_start * W + i];
            }
        for (int tw_id = 0; tw_id < TWS; ++tw_id)
            for (int n = 0; n < N; ++n) {
                const int w_out_start = tw_id * TW;
                for (int i = 0; i < TH * TW; ++i) tmp[i] = 0.0f;
                for (int c = 0; c < TC; ++c) {
                    const float *k9 = kern + (size_t)(c + c_offset) * N * 9 + n;
                    /* every smem element of the (TH+2)x(TW+2) window feeds each output it overlaps */
                    for (int h = 0; h < TH + 2; ++h)
                        for (int ww = 0; ww < TW + 2; ++ww) {
                            const float v = smem[(size_t)c * (TH + 2) * WPAD + (size_t)h * WPAD + w_out_start + ww];
                            for (int r = 0; r < 3; ++r)
                                for (int s = 0; s < 3; ++s) {
                                    const int oh = h - r, ow = ww - s;
                                    if (oh < 0 || oh >= TH || ow < 0 || ow >= TW) continue;
                                    tmp[oh * TW + ow] += v * k9[(r * 3 + s) * N];
                                }
                        }
                }
                const int wh = (TH < H - h_out_start) ? TH : H - h_out_start;
                const int wwid = (TW < W - w_out_start) ? TW : W - w_out_start;
                for (int th = 0; th < wh; ++th)
                    for (int tw = 0; tw < wwid; ++tw) /* atomicAdd in the reference */
                        out[(size_t)n * H * W + (size_t)(h_out_start + th) * W + w_out_start + tw] += tmp[th * TW + tw];
            }
    }
    free(kern); free(smem); free(tmp);
    return 0;
}
