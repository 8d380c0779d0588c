// Whole-network forward graphs: a list of Tucker / dense convolutions, pools,
// per-channel affine(+ReLU) layers and concatenations over net-owned device
// tensors, captured once into a HIP graph and replayed per inference.  This is
// what the reference's native E2E drivers do layer object by layer object on the
// default stream (2080Ti-evaluation/EndToEnd/resnet18-tk/src/main.cu:19-156,
// src/BasicBlock.cu:43-50, densenet121-tk/src/main.cu:6-84) — here with the
// topology supplied by the caller, BatchNorm/ReLU/residual work fused into the
// convolution epilogues where the network allows it, concatenation done in place
// (producers write into channel slices of one buffer), and one graph launch
// instead of one launch per layer.
#include <hip/hip_runtime_api.h>

#include <memory>
#include <new>
#include <string>
#include <vector>

#include "tdc_internal.hpp"

using namespace tdc;

namespace {

struct NetTensor {
    int C = 0, H = 0, W = 0;
    float *d = nullptr;       // first element (of image 0)
    long long bstride = 0;    // floats between images
    bool owner = false;
    size_t floats = 0;        // allocation size (owners only)
};

struct NetOp {
    enum Kind { CONV, TKCONV, POOL, GAP, COPY, AFFINE } kind = CONV;
    tdc_conv_plan *conv = nullptr;
    tdc_tkconv *tk = nullptr;
    float *d_scale = nullptr, *d_shift = nullptr;
    int in = -1, out = -1, resid = -1;
    int k = 0, stride = 0, pad = 0, mode = 0, relu = 0;
};

}  // namespace

struct tdc_net {
    int batch = 1;
    std::vector<NetTensor> tensors;
    std::vector<NetOp> ops;
    hipStream_t stream = nullptr;
    hipGraph_t graph = nullptr;
    hipGraphExec_t exec = nullptr;
    bool finalized = false;
    int out_id = -1;
    int kernels = 0;
};

namespace {

int hipf(const char *what, hipError_t e) {
    return api_fail(TDC_ERR_HIP, std::string(what) + ": " + hipGetErrorString(e));
}

int new_tensor(tdc_net *net, int C, int H, int W, int *id) {
    NetTensor t;
    t.C = C; t.H = H; t.W = W;
    t.bstride = (long long)C * H * W;
    t.floats = (size_t)net->batch * C * H * W;
    t.owner = true;
    hipError_t e = hipMalloc((void **)&t.d, t.floats * sizeof(float));
    if (e != hipSuccess) return hipf("hipMalloc(net tensor)", e);
    net->tensors.push_back(t);
    *id = (int)net->tensors.size() - 1;
    return TDC_OK;
}

bool valid_id(const tdc_net *net, int id) { return id >= 0 && id < (int)net->tensors.size(); }

int check_open(const tdc_net *net) {
    if (!net) return api_fail(TDC_ERR_INVALID, "null net");
    if (net->finalized) return api_fail(TDC_ERR_STATE, "net is already finalized");
    return TDC_OK;
}

// Destination of an operator: an existing tensor/view of exactly the produced shape, or a new tensor.
int resolve_dst(tdc_net *net, int dst, int C, int H, int W, int *id) {
    if (dst < 0) return new_tensor(net, C, H, W, id);
    if (!valid_id(net, dst)) return api_fail(TDC_ERR_INVALID, "bad destination tensor id");
    const NetTensor &t = net->tensors[dst];
    if (t.C != C || t.H != H || t.W != W) return api_fail(TDC_ERR_INVALID, "destination tensor shape does not match the result");
    *id = dst;
    return TDC_OK;
}

int run_ops(tdc_net *net, hipStream_t s) {
    for (const NetOp &op : net->ops) {
        const NetTensor &ti = net->tensors[op.in];
        const NetTensor &to = net->tensors[op.out];
        const float *resid = op.resid >= 0 ? net->tensors[op.resid].d : nullptr;
        const long long rbs = op.resid >= 0 ? net->tensors[op.resid].bstride : 0;
        int st = TDC_OK, he = 0;
        switch (op.kind) {
            case NetOp::CONV: st = tdc_conv_forward_strided(op.conv, ti.d, ti.bstride, resid, rbs, to.d, to.bstride, s); break;
            case NetOp::TKCONV: st = tdc_tkconv_forward_strided(op.tk, ti.d, ti.bstride, resid, rbs, to.d, to.bstride, s); break;
            case NetOp::POOL:
                he = launch_pool2d(ti.d, ti.bstride, to.d, to.bstride, net->batch, ti.C, ti.H, ti.W, to.H, to.W, op.k, op.stride,
                                   op.pad, op.mode, s);
                break;
            case NetOp::GAP: he = launch_global_avgpool(ti.d, ti.bstride, to.d, to.bstride, net->batch, ti.C, ti.H * ti.W, s); break;
            case NetOp::COPY: he = launch_copy_channels(ti.d, ti.bstride, to.d, to.bstride, net->batch, ti.C, ti.H * ti.W, s); break;
            case NetOp::AFFINE:
                he = launch_affine(ti.d, ti.bstride, to.d, to.bstride, op.d_scale, op.d_shift, net->batch, ti.C, ti.H * ti.W,
                                   op.relu, s);
                break;
        }
        if (st != TDC_OK) return st;
        if (he) return hipf("net kernel launch", (hipError_t)he);
    }
    return TDC_OK;
}

}  // namespace

extern "C" {

int tdc_net_create(int32_t batch, int32_t C, int32_t H, int32_t W, tdc_net **net_out) {
    if (!net_out || batch < 1 || C < 1 || H < 1 || W < 1) return api_fail(TDC_ERR_INVALID, "bad argument");
    *net_out = nullptr;
    std::unique_ptr<tdc_net> net(new (std::nothrow) tdc_net());
    if (!net) return api_fail(TDC_ERR_NOMEM, "out of host memory");
    net->batch = batch;
    hipError_t e = hipStreamCreate(&net->stream);
    if (e != hipSuccess) return hipf("hipStreamCreate", e);
    int id;
    int st = new_tensor(net.get(), C, H, W, &id);
    if (st != TDC_OK) {
        (void)hipStreamDestroy(net->stream);
        return st;
    }
    *net_out = net.release();
    return TDC_OK;
}

int tdc_net_tensor(tdc_net *net, int32_t C, int32_t H, int32_t W, int32_t *out) {
    int st = check_open(net);
    if (st != TDC_OK) return st;
    if (!out || C < 1 || H < 1 || W < 1) return api_fail(TDC_ERR_INVALID, "bad argument");
    int id;
    if ((st = new_tensor(net, C, H, W, &id)) != TDC_OK) return st;
    *out = id;
    return TDC_OK;
}

int tdc_net_view(tdc_net *net, int32_t id, int32_t c0, int32_t C, int32_t *out) {
    int st = check_open(net);
    if (st != TDC_OK) return st;
    if (!out || !valid_id(net, id)) return api_fail(TDC_ERR_INVALID, "bad tensor id");
    const NetTensor base = net->tensors[id];
    if (c0 < 0 || C < 1 || c0 + C > base.C) return api_fail(TDC_ERR_INVALID, "channel range outside the tensor");
    NetTensor v;
    v.C = C; v.H = base.H; v.W = base.W;
    v.d = base.d + (long long)c0 * base.H * base.W;
    v.bstride = base.bstride;
    v.owner = false;
    net->tensors.push_back(v);
    *out = (int)net->tensors.size() - 1;
    return TDC_OK;
}

// Shared by the plain and the tail-fused convolution operators.
static int net_add_conv(tdc_net *net, int32_t in, int32_t N, int32_t KH, int32_t KW, int32_t stride, int32_t pad,
                        const float *w, const float *bias, int32_t relu, int32_t tail_N, const float *w_tail,
                        const float *bias_tail, int32_t tail_relu, int32_t residual, int32_t dst, int32_t *out) {
    int st = check_open(net);
    if (st != TDC_OK) return st;
    if (!out || !w || !valid_id(net, in) || (residual >= 0 && !valid_id(net, residual)) || (tail_N > 0 && !w_tail))
        return api_fail(TDC_ERR_INVALID, "bad tensor id or null argument");
    const NetTensor ti = net->tensors[in];
    // without a tail the residual and the ReLU belong to the convolution's own epilogue
    tdc_conv_desc d{net->batch, ti.C, N, ti.H, ti.W, KH, KW, stride, pad, 1, bias != nullptr, relu != 0};
    std::string why;
    if (!check_desc(d, &why)) return api_fail(TDC_ERR_INVALID, why);
    const int Ho = (ti.H + 2 * pad - (KH - 1) - 1) / stride + 1, Wo = (ti.W + 2 * pad - (KW - 1) - 1) / stride + 1;
    const int Nout = tail_N > 0 ? tail_N : N;
    if (residual >= 0) {
        const NetTensor &tr = net->tensors[residual];
        if (tr.C != Nout || tr.H != Ho || tr.W != Wo)
            return api_fail(TDC_ERR_INVALID, "residual tensor shape does not match the convolution output");
    }
    int id;
    if ((st = resolve_dst(net, dst, Nout, Ho, Wo, &id)) != TDC_OK) return st;
    tdc_conv_plan *plan = nullptr;
    if ((st = tdc_conv_plan_create_with_tail(&d, tail_N, bias_tail != nullptr, tail_relu, nullptr, &plan)) != TDC_OK) return st;
    st = tdc_conv_plan_set_weights(plan, w, bias);
    if (st == TDC_OK && tail_N > 0) st = tdc_conv_plan_set_tail_weights(plan, w_tail, bias_tail);
    if (st != TDC_OK) {
        tdc_conv_plan_destroy(plan);
        return st;
    }
    NetOp op;
    op.kind = NetOp::CONV; op.conv = plan; op.in = in; op.out = id; op.resid = residual;
    net->ops.push_back(op);
    net->kernels += 1;
    *out = id;
    return TDC_OK;
}

int tdc_net_conv(tdc_net *net, int32_t in, int32_t N, int32_t KH, int32_t KW, int32_t stride, int32_t pad, const float *w,
                 const float *bias, int32_t residual, int32_t relu, int32_t dst, int32_t *out) {
    return net_add_conv(net, in, N, KH, KW, stride, pad, w, bias, relu, 0, nullptr, nullptr, 0, residual, dst, out);
}

int tdc_net_conv_tail(tdc_net *net, int32_t in, int32_t N, int32_t KH, int32_t KW, int32_t stride, int32_t pad,
                      const float *w, const float *bias, int32_t relu, int32_t tail_N, const float *w_tail,
                      const float *bias_tail, int32_t residual, int32_t tail_relu, int32_t dst, int32_t *out) {
    if (tail_N < 1) return api_fail(TDC_ERR_INVALID, "tail_N must be >= 1");
    return net_add_conv(net, in, N, KH, KW, stride, pad, w, bias, relu, tail_N, w_tail, bias_tail, tail_relu, residual, dst,
                        out);
}

int tdc_net_set_input_affine(tdc_net *net, const float *scale, const float *shift, int32_t relu) {
    int st = check_open(net);
    if (st != TDC_OK) return st;
    if (net->ops.empty() || net->ops.back().kind != NetOp::CONV)
        return api_fail(TDC_ERR_STATE, "the last operator added is not a convolution");
    return tdc_conv_plan_set_input_affine(net->ops.back().conv, scale, shift, relu);
}

int tdc_net_affine_conv(tdc_net *net, int32_t in, const float *scale, const float *shift, int32_t affine_relu, int32_t N,
                        const float *w, const float *bias, int32_t residual, int32_t relu, int32_t dst, int32_t *out) {
    if (!scale || !shift) return api_fail(TDC_ERR_INVALID, "null argument");
    int st = tdc_net_conv(net, in, N, 1, 1, 1, 0, w, bias, residual, relu, dst, out);
    if (st != TDC_OK) return st;
    // the convolution just appended is the last op
    return tdc_conv_plan_set_input_affine(net->ops.back().conv, scale, shift, affine_relu);
}

int tdc_net_tkconv(tdc_net *net, int32_t in, int32_t R1, int32_t R2, int32_t N, int32_t K, int32_t stride, int32_t pad,
                   const float *first, const float *core, const float *last, const float *bias, int32_t residual,
                   int32_t relu, int32_t dst, int32_t *out) {
    int st = check_open(net);
    if (st != TDC_OK) return st;
    if (!out || !first || !core || !last || !valid_id(net, in) || (residual >= 0 && !valid_id(net, residual)))
        return api_fail(TDC_ERR_INVALID, "bad tensor id or null argument");
    if (K < 1 || stride < 1 || pad < 0) return api_fail(TDC_ERR_INVALID, "bad core convolution geometry");
    const NetTensor ti = net->tensors[in];
    if (ti.H + 2 * pad < K || ti.W + 2 * pad < K) return api_fail(TDC_ERR_INVALID, "core filter larger than the padded input");
    const int Ho = (ti.H + 2 * pad - (K - 1) - 1) / stride + 1, Wo = (ti.W + 2 * pad - (K - 1) - 1) / stride + 1;
    if (residual >= 0) {
        const NetTensor &tr = net->tensors[residual];
        if (tr.C != N || tr.H != Ho || tr.W != Wo)
            return api_fail(TDC_ERR_INVALID, "residual tensor shape does not match the operator output");
    }
    int id;
    if ((st = resolve_dst(net, dst, N, Ho, Wo, &id)) != TDC_OK) return st;
    tdc_tkconv_desc d{net->batch, ti.C, R1, R2, N, ti.H, ti.W, K, stride, pad, 1, bias != nullptr, relu != 0};
    tdc_tkconv *tk = nullptr;
    if ((st = tdc_tkconv_create(&d, &tk)) != TDC_OK) return st;
    if ((st = tdc_tkconv_set_weights(tk, first, core, last, bias)) != TDC_OK) {
        tdc_tkconv_destroy(tk);
        return st;
    }
    NetOp op;
    op.kind = NetOp::TKCONV; op.tk = tk; op.in = in; op.out = id; op.resid = residual;
    net->ops.push_back(op);
    net->kernels += tdc_tkconv_num_kernels(tk);
    *out = id;
    return TDC_OK;
}

int tdc_net_pool(tdc_net *net, int32_t in, int32_t mode, int32_t k, int32_t stride, int32_t pad, int32_t dst, int32_t *out) {
    int st = check_open(net);
    if (st != TDC_OK) return st;
    if (!out || !valid_id(net, in) || k < 1 || stride < 1 || pad < 0 || 2 * pad > k || (mode != 0 && mode != 1))
        return api_fail(TDC_ERR_INVALID, "bad pooling argument");
    const NetTensor ti = net->tensors[in];
    if (ti.H + 2 * pad < k || ti.W + 2 * pad < k) return api_fail(TDC_ERR_INVALID, "pooling window larger than the input");
    const int Ho = (ti.H + 2 * pad - k) / stride + 1, Wo = (ti.W + 2 * pad - k) / stride + 1;
    int id;
    if ((st = resolve_dst(net, dst, ti.C, Ho, Wo, &id)) != TDC_OK) return st;
    NetOp op;
    op.kind = NetOp::POOL; op.in = in; op.out = id; op.k = k; op.stride = stride; op.pad = pad; op.mode = mode;
    net->ops.push_back(op);
    net->kernels += 1;
    *out = id;
    return TDC_OK;
}

int tdc_net_global_avgpool(tdc_net *net, int32_t in, int32_t *out) {
    int st = check_open(net);
    if (st != TDC_OK) return st;
    if (!out || !valid_id(net, in)) return api_fail(TDC_ERR_INVALID, "bad tensor id");
    const NetTensor ti = net->tensors[in];
    int id;
    if ((st = new_tensor(net, ti.C, 1, 1, &id)) != TDC_OK) return st;
    NetOp op;
    op.kind = NetOp::GAP; op.in = in; op.out = id;
    net->ops.push_back(op);
    net->kernels += 1;
    *out = id;
    return TDC_OK;
}

int tdc_net_affine(tdc_net *net, int32_t in, const float *scale, const float *shift, int32_t relu, int32_t dst,
                   int32_t *out) {
    int st = check_open(net);
    if (st != TDC_OK) return st;
    if (!out || !scale || !shift || !valid_id(net, in)) return api_fail(TDC_ERR_INVALID, "bad tensor id or null argument");
    const NetTensor ti = net->tensors[in];
    int id;
    if ((st = resolve_dst(net, dst, ti.C, ti.H, ti.W, &id)) != TDC_OK) return st;
    NetOp op;
    op.kind = NetOp::AFFINE; op.in = in; op.out = id; op.relu = relu != 0;
    hipError_t e = hipMalloc((void **)&op.d_scale, 2 * (size_t)ti.C * sizeof(float));
    if (e != hipSuccess) return hipf("hipMalloc(affine)", e);
    op.d_shift = op.d_scale + ti.C;
    e = hipMemcpy(op.d_scale, scale, (size_t)ti.C * sizeof(float), hipMemcpyHostToDevice);
    if (e == hipSuccess) e = hipMemcpy(op.d_shift, shift, (size_t)ti.C * sizeof(float), hipMemcpyHostToDevice);
    if (e != hipSuccess) {
        (void)hipFree(op.d_scale);
        return hipf("hipMemcpy(affine)", e);
    }
    net->ops.push_back(op);
    net->kernels += 1;
    *out = id;
    return TDC_OK;
}

int tdc_net_concat(tdc_net *net, const int32_t *ins, int32_t n, int32_t *out) {
    int st = check_open(net);
    if (st != TDC_OK) return st;
    if (!out || !ins || n < 1) return api_fail(TDC_ERR_INVALID, "bad argument");
    int Ctot = 0;
    for (int i = 0; i < n; ++i) {
        if (!valid_id(net, ins[i])) return api_fail(TDC_ERR_INVALID, "bad tensor id");
        const NetTensor &t = net->tensors[ins[i]];
        if (t.H != net->tensors[ins[0]].H || t.W != net->tensors[ins[0]].W)
            return api_fail(TDC_ERR_INVALID, "concatenated tensors differ in height/width");
        Ctot += t.C;
    }
    int id;
    if ((st = new_tensor(net, Ctot, net->tensors[ins[0]].H, net->tensors[ins[0]].W, &id)) != TDC_OK) return st;
    int c0 = 0;
    for (int i = 0; i < n; ++i) {
        int view;
        if ((st = tdc_net_view(net, id, c0, net->tensors[ins[i]].C, &view)) != TDC_OK) return st;
        NetOp op;
        op.kind = NetOp::COPY; op.in = ins[i]; op.out = view;
        net->ops.push_back(op);
        net->kernels += 1;
        c0 += net->tensors[ins[i]].C;
    }
    *out = id;
    return TDC_OK;
}

int tdc_net_tensor_shape(const tdc_net *net, int32_t id, int32_t *C, int32_t *H, int32_t *W) {
    if (!net || !valid_id(net, id) || !C || !H || !W) return api_fail(TDC_ERR_INVALID, "bad argument");
    *C = net->tensors[id].C; *H = net->tensors[id].H; *W = net->tensors[id].W;
    return TDC_OK;
}

int tdc_net_num_kernels(const tdc_net *net) { return net ? net->kernels : 0; }

int tdc_net_finalize(tdc_net *net, int32_t output_id) {
    int st = check_open(net);
    if (st != TDC_OK) return st;
    if (!valid_id(net, output_id) || net->ops.empty()) return api_fail(TDC_ERR_INVALID, "bad output id or empty net");
    // One eager pass first (warms every kernel outside capture), then capture.
    if ((st = run_ops(net, net->stream)) != TDC_OK) return st;
    hipError_t e = hipStreamSynchronize(net->stream);
    if (e != hipSuccess) return hipf("eager pass", e);
    e = hipStreamBeginCapture(net->stream, hipStreamCaptureModeThreadLocal);
    if (e != hipSuccess) return hipf("hipStreamBeginCapture", e);
    st = run_ops(net, net->stream);
    e = hipStreamEndCapture(net->stream, &net->graph);
    if (st != TDC_OK) return st;
    if (e != hipSuccess) return hipf("hipStreamEndCapture", e);
    e = hipGraphInstantiate(&net->exec, net->graph, nullptr, nullptr, 0);
    if (e != hipSuccess) return hipf("hipGraphInstantiate", e);
    net->out_id = output_id;
    net->finalized = true;
    return TDC_OK;
}

int tdc_net_forward(tdc_net *net, const float *d_in, float *d_out, void *stream) {
    if (!net) return api_fail(TDC_ERR_INVALID, "null net");
    if (!net->finalized) return api_fail(TDC_ERR_STATE, "tdc_net_forward before tdc_net_finalize");
    hipStream_t s = (hipStream_t)stream;
    const NetTensor &ti = net->tensors[0];
    const NetTensor &to = net->tensors[net->out_id];
    if (d_out && to.bstride != (long long)to.C * to.H * to.W)
        return api_fail(TDC_ERR_UNSUPPORTED, "the output tensor is a channel slice; read it with tdc_net_read_tensor");
    hipError_t e = hipSuccess;
    if (d_in && d_in != ti.d) e = hipMemcpyAsync(ti.d, d_in, ti.floats * sizeof(float), hipMemcpyDeviceToDevice, s);
    if (e == hipSuccess) e = hipGraphLaunch(net->exec, s);
    if (e == hipSuccess && d_out && d_out != to.d)
        e = hipMemcpyAsync(d_out, to.d, (size_t)net->batch * to.C * to.H * to.W * sizeof(float), hipMemcpyDeviceToDevice, s);
    if (e != hipSuccess) return hipf("tdc_net_forward", e);
    return TDC_OK;
}

int tdc_net_time(tdc_net *net, int32_t iters, int32_t use_graph, float *total_ms_out) {
    if (!net || iters < 1 || !total_ms_out) return api_fail(TDC_ERR_INVALID, "bad argument");
    if (!net->finalized) return api_fail(TDC_ERR_STATE, "tdc_net_time before tdc_net_finalize");
    hipEvent_t e0 = nullptr, e1 = nullptr;
    hipError_t e = hipDeviceSynchronize();
    if (e == hipSuccess) e = hipEventCreate(&e0);
    if (e == hipSuccess) e = hipEventCreate(&e1);
    int st = TDC_OK;
    if (e == hipSuccess) e = hipEventRecord(e0, net->stream);
    for (int i = 0; i < iters && e == hipSuccess && st == TDC_OK; ++i) {
        if (use_graph) e = hipGraphLaunch(net->exec, net->stream);
        else st = run_ops(net, net->stream);
    }
    if (e == hipSuccess) e = hipEventRecord(e1, net->stream);
    if (e == hipSuccess) e = hipEventSynchronize(e1);
    if (e == hipSuccess) e = hipEventElapsedTime(total_ms_out, e0, e1);
    if (e0) (void)hipEventDestroy(e0);
    if (e1) (void)hipEventDestroy(e1);
    if (st != TDC_OK) return st;
    if (e != hipSuccess) return hipf("tdc_net_time", e);
    return TDC_OK;
}

int tdc_net_read_tensor(tdc_net *net, int32_t id, float *host_out) {
    if (!net || !valid_id(net, id) || !host_out) return api_fail(TDC_ERR_INVALID, "bad argument");
    const NetTensor &t = net->tensors[id];
    const size_t image = (size_t)t.C * t.H * t.W;
    hipError_t e = hipDeviceSynchronize();
    for (int b = 0; b < net->batch && e == hipSuccess; ++b)
        e = hipMemcpy(host_out + b * image, t.d + b * t.bstride, image * sizeof(float), hipMemcpyDeviceToHost);
    if (e != hipSuccess) return hipf("tdc_net_read_tensor", e);
    return TDC_OK;
}

void tdc_net_destroy(tdc_net *net) {
    if (!net) return;
    if (net->exec) (void)hipGraphExecDestroy(net->exec);
    if (net->graph) (void)hipGraphDestroy(net->graph);
    for (NetOp &op : net->ops) {
        if (op.conv) tdc_conv_plan_destroy(op.conv);
        if (op.tk) tdc_tkconv_destroy(op.tk);
        if (op.d_scale) (void)hipFree(op.d_scale);
    }
    for (NetTensor &t : net->tensors)
        if (t.owner && t.d) (void)hipFree(t.d);
    if (net->stream) (void)hipStreamDestroy(net->stream);
    delete net;
}

}  // extern "C"
