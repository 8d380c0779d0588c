// C ABI: plans, weight upload, forward calls.  See include/tdc.h for the
// reference interfaces each entry point stands in for.
#include <hip/hip_runtime_api.h>

#include <algorithm>
#include <array>
#include <atomic>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <map>
#include <memory>
#include <mutex>
#include <new>
#include <string>
#include <vector>

#include "tdc_internal.hpp"

namespace tdc {

static thread_local std::string g_last_error;

void set_error(const std::string &msg) { g_last_error = msg; }

static int fail(tdc_status st, const std::string &msg) {
    set_error(msg);
    return (int)st;
}

int api_fail(int status, const std::string &msg) {
    set_error(msg);
    return status;
}

static int hip_fail(const char *what, int err) {
    return fail(TDC_ERR_HIP, std::string(what) + ": " + hipGetErrorString((hipError_t)err));
}

}  // namespace tdc

using namespace tdc;

struct tdc_conv_plan {
    tdc_conv_desc desc{};
    tdc_tile tile{};
    tdc_tile_info info{};
    Geometry geo{};
    const void *kernel = nullptr;
    void *kernel_handle = nullptr;   // the kernel's module function on the plan's device: what a forward launches
    float *d_wpk = nullptr;
    float *d_bias = nullptr;
    float *d_ws = nullptr;        // tile.ks > 1: partial tiles [batch][ks][N][P]
    unsigned *d_ctr = nullptr;    // tile.ks > 1: ticket counters, zero between launches
    float *d_in_aff = nullptr;    // optional input affine: [pass][scale(cch) | shift(cch)]
    int tail_N = 0;               // fused 1x1 tail (0 = none): outputs, epilogue flags, packed weights
    int tail_has_bias = 0, tail_relu = 0;
    float *d_tail_w = nullptr, *d_tail_bias = nullptr;
    int head_C = 0;               // fused 1x1 head (0 = none): its input channels, packed weights, LDS layout
    float *d_head_w = nullptr;
    int head_runs = 0, head_mblk = 0, head_npb = 0, head_ww = 0, head_wq = 0, head_ld = 0, head_f_off = 0;
    bool have_tail_weights = false;
    int in_relu = 0;
    bool have_weights = false;
    // The kernel arguments of a launch, but for what a call brings (buffers, batch strides, copy width): built when the
    // plan is created and again whenever a setter changes what they depend on, so that a forward copies and patches
    // them instead of recomputing two dozen divisions — host time per launch is what bounds small back-to-back kernels.
    ConvKParams kp{};
    FastDiv fd_csv1{}, fd_rsv1{};   // the two arguments that differ when the input is copied with 4-byte elements
#if defined(TDC_STAMPS) && TDC_STAMPS
    unsigned long long *d_stamps = nullptr;   // profiling build: per-wave time stamps of the last launch
    size_t stamp_words = 0;
#endif
};

#if defined(TDC_STAMPS) && TDC_STAMPS
// Profiling build only: copy the time stamps of the plan's last launch to the host, [workgroup][16 waves][8]
// values of the 100 MHz constant clock (0 = that wave wrote nothing); *words_out = how many were written.
extern "C" int tdc_debug_read_stamps(tdc_conv_plan *plan, unsigned long long *host_out, uint64_t cap, uint64_t *words_out) {
    if (!plan || !host_out || !words_out) return (int)TDC_ERR_INVALID;
    const size_t n = std::min<size_t>(plan->stamp_words, (size_t)cap);
    if (hipMemcpy(host_out, plan->d_stamps, n * 8, hipMemcpyDeviceToHost) != hipSuccess) return (int)TDC_ERR_HIP;
    *words_out = n;
    return TDC_OK;
}
#endif

static void free_plan_buffers(tdc_conv_plan *p) {
#if defined(TDC_STAMPS) && TDC_STAMPS
    if (p->d_stamps) (void)hipFree(p->d_stamps);
    p->d_stamps = nullptr;
#endif
    if (p->d_wpk) (void)hipFree(p->d_wpk);
    if (p->d_bias) (void)hipFree(p->d_bias);
    if (p->d_ws) (void)hipFree(p->d_ws);
    if (p->d_ctr) (void)hipFree(p->d_ctr);
    if (p->d_in_aff) (void)hipFree(p->d_in_aff);
    if (p->d_tail_w) (void)hipFree(p->d_tail_w);
    if (p->d_tail_bias) (void)hipFree(p->d_tail_bias);
    if (p->d_head_w) (void)hipFree(p->d_head_w);
    p->d_head_w = nullptr;
    p->d_in_aff = p->d_tail_w = p->d_tail_bias = nullptr;
    p->d_wpk = p->d_bias = p->d_ws = nullptr;
    p->d_ctr = nullptr;
}

struct tdc_tkconv {
    tdc_tkconv_desc desc{};
    tdc_conv_plan *first = nullptr;
    tdc_conv_plan *core = nullptr;
    tdc_conv_plan *last = nullptr;
    tdc_conv_plan *core_last = nullptr;   // core convolution with the last factor fused behind it, when that is faster
    tdc_conv_plan *whole = nullptr;       // first factor + core + last factor in one launch, when that is faster still
    float *d_f1 = nullptr;  // [batch, R1, H, W]
    float *d_f2 = nullptr;  // [batch, R2, Ho, Wo]
    size_t f1_floats = 0, f2_floats = 0;
};

static int time_plans(tdc_conv_plan *const *plans, const float *const *d_ins, float *const *d_outs, int n, int passes,
                      int iters, int use_graph, float *total_ms_out);

extern "C" {

const char *tdc_last_error_string(void) { return g_last_error.c_str(); }

const char *tdc_version(void) { return "tdc-amd 0.1 (gfx950)"; }

int tdc_model_evaluate(const tdc_conv_desc *desc, const tdc_tile *tile, tdc_tile_info *info_out) {
    if (!desc || !tile || !info_out) return fail(TDC_ERR_INVALID, "null argument");
    std::string why;
    if (!model_evaluate(*desc, *tile, *info_out, &why)) return fail(TDC_ERR_INVALID, why);
    return TDC_OK;
}

int tdc_model_enumerate(const tdc_conv_desc *desc, tdc_tile *tiles_out, int32_t cap, int32_t *count_out) {
    if (!desc || !count_out || cap < 0 || (cap > 0 && !tiles_out)) return fail(TDC_ERR_INVALID, "null argument");
    std::string why;
    if (!check_desc(*desc, &why)) return fail(TDC_ERR_INVALID, why);
    std::vector<tdc_tile> v = model_enumerate(*desc);
    int32_t n = 0;
    for (const tdc_tile &t : v) {
        if (n >= cap) break;
        tiles_out[n++] = t;
    }
    *count_out = n;
    return TDC_OK;
}

int tdc_model_select(const tdc_conv_desc *desc, tdc_tile_info *info_out) {
    if (!desc || !info_out) return fail(TDC_ERR_INVALID, "null argument");
    std::string why;
    if (!model_select(*desc, *info_out, &why)) return fail(TDC_ERR_INVALID, why);
    return TDC_OK;
}

int tdc_model_select_with_tail(const tdc_conv_desc *desc, int32_t tail_N, tdc_tile_info *info_out) {
    if (!desc || !info_out || tail_N < 0) return fail(TDC_ERR_INVALID, "null argument");
    std::string why;
    if (!model_select(*desc, *info_out, &why, tail_N)) return fail(TDC_ERR_INVALID, why);
    return TDC_OK;
}

int tdc_model_kernel_info(const tdc_conv_desc *desc, const tdc_tile *tile, int32_t extras, char *name_out, int32_t cap,
                          int32_t *vgprs_out, int32_t *waves_per_simd_out) {
    if (!desc || !tile || (cap > 0 && !name_out)) return fail(TDC_ERR_INVALID, "null argument");
    const KernelId k = kernel_id_for(*tile, desc->KH, desc->KW, desc->dilation, desc->stride, extras != 0);
    if (k.family == KernelId::NONE) return fail(TDC_ERR_UNSUPPORTED, "no kernel instantiated for this tile");
    const std::string name = kernel_name(k);
    if (cap > 0) {
        std::strncpy(name_out, name.c_str(), (size_t)cap - 1);
        name_out[cap - 1] = '\0';
    }
    if (vgprs_out) *vgprs_out = kernel_vgprs(k);
    if (waves_per_simd_out) *waves_per_simd_out = kernel_waves_per_simd(k);
    return TDC_OK;
}

int tdc_load_bin(const char *path, float *dst, uint64_t count) {
    if (!path || (!dst && count)) return fail(TDC_ERR_INVALID, "null argument");
    FILE *f = std::fopen(path, "rb");
    if (!f) return fail(TDC_ERR_INVALID, std::string("cannot open weight file ") + path);
    const size_t got = std::fread(dst, sizeof(float), (size_t)count, f);
    // exactly `count` floats: neither fewer nor a longer file
    char extra;
    const bool longer = std::fread(&extra, 1, 1, f) == 1;
    std::fclose(f);
    if (got != count || longer)
        return fail(TDC_ERR_INVALID, std::string("weight file ") + path + " does not hold exactly " + std::to_string(count) +
                                         " float32 values");
    return TDC_OK;
}

int tdc_save_bin(const char *path, const float *src, uint64_t count) {
    if (!path || (!src && count)) return fail(TDC_ERR_INVALID, "null argument");
    FILE *f = std::fopen(path, "wb");
    if (!f) return fail(TDC_ERR_INVALID, std::string("cannot create weight file ") + path);
    const size_t put = std::fwrite(src, sizeof(float), (size_t)count, f);
    const int rc = std::fclose(f);
    if (put != count || rc != 0) return fail(TDC_ERR_INVALID, std::string("short write to ") + path);
    return TDC_OK;
}

int tdc_model_get_constants(double *out, int32_t cap, int32_t *count_out) {
    if (!count_out || (cap > 0 && !out)) return fail(TDC_ERR_INVALID, "null argument");
    *count_out = model_constants(out, cap);
    return TDC_OK;
}

int tdc_model_set_constants(const double *values, int32_t count) {
    if (!values) return fail(TDC_ERR_INVALID, "null argument");
    if (!model_set_constants(values, count)) return fail(TDC_ERR_INVALID, "wrong number of constants, or a non-positive one");
    return TDC_OK;
}

// ---- Measured tile selection ------------------------------------------------
// The model ranks tens of thousands of candidates in milliseconds and is within a few per cent of the measured
// best on most shapes; where it is not, the better tile is usually the model's favourite of ANOTHER tile class
// (a different split of the workgroup into waves, or another tile width).  With tuning switched on, a plan
// created without a forced tile times the model's favourite of each of the `g_autotune` most promising classes
// on the device (synthetic data; the timing does not depend on values) and keeps the fastest.  This is the
// reference's measure-every-tile oracle (2080Ti-evaluation/TDC-LAYERS-ORACLE/gen_from_occupancy.py:51-66) cut
// down to the candidates the model cannot tell apart.  Results are remembered per problem for the life of the
// process.
static int autotune_from_env() {
    const char *e = std::getenv("TDC_AUTOTUNE");
    const int v = e ? std::atoi(e) : 0;
    return v < 0 ? 0 : (v > 256 ? 256 : v);
}
static std::atomic<int> g_autotune{autotune_from_env()};   // TDC_AUTOTUNE=k in the environment = tdc_set_autotune(k) at load
static std::mutex g_tune_mutex;
static std::map<std::array<int, 16>, tdc_tile> g_tuned;

// Timing runs need weights in place but not their values: fill the packed buffers with a constant (every float
// 0.0115) and mark the plan ready; `ready = false` afterwards makes the plan ask for real weights again.
static int synthetic_weights(tdc_conv_plan *plan, bool ready) {
    if (ready) {
        hipError_t e = hipMemset(plan->d_wpk, 0x3c, packed_weight_floats(plan->geo) * sizeof(float));
        if (e == hipSuccess && plan->d_bias) e = hipMemset(plan->d_bias, 0, (size_t)plan->desc.N * sizeof(float));
        if (e == hipSuccess && plan->d_tail_w)
            e = hipMemset(plan->d_tail_w, 0x3c, (size_t)((plan->tail_N + 15) / 16) * plan->geo.tail_ng * 64 * sizeof(float));
        if (e == hipSuccess && plan->d_tail_bias) e = hipMemset(plan->d_tail_bias, 0, (size_t)plan->tail_N * sizeof(float));
        if (e != hipSuccess) return hip_fail("hipMemset(synthetic weights)", e);
    }
    plan->have_weights = ready;
    plan->have_tail_weights = ready && plan->tail_N > 0;
    return TDC_OK;
}

static bool log_tuning() {
    static const bool on = std::getenv("TDC_LOG_TUNING") != nullptr;
    return on;
}

static int tune_tile(const tdc_conv_desc &d, int tail_N, int tail_has_bias, int tail_relu, int classes, tdc_tile &best_out) {
    const std::array<int, 16> key{d.batch, d.C, d.N, d.H, d.W, d.KH, d.KW, d.stride, d.pad, d.dilation,
                                  d.has_bias, d.relu, tail_N, tail_has_bias, tail_relu, classes};
    {
        std::lock_guard<std::mutex> lock(g_tune_mutex);
        auto hit = g_tuned.find(key);
        if (hit != g_tuned.end()) {
            best_out = hit->second;
            return TDC_OK;
        }
    }
    // the model's favourite per class (waves and register blocks, tile width), classes in order of promise
    std::map<std::array<int, 8>, tdc_tile_info> per_class;
    for (const tdc_tile &t : model_enumerate(d, tail_N)) {
        tdc_tile_info info;
        if (!model_evaluate(d, t, info, nullptr, tail_N)) continue;
        const std::array<int, 8> cls{t.mf, t.mb, t.nb, t.wm, t.wn, t.wk, t.tw, t.alg};
        auto it = per_class.find(cls);
        if (it == per_class.end() || info.pred_us < it->second.pred_us) per_class[cls] = info;
    }
    if (per_class.empty()) return fail(TDC_ERR_UNSUPPORTED, "no launchable tile for this shape");
    std::vector<tdc_tile_info> cands;
    for (const auto &kv : per_class) cands.push_back(kv.second);
    std::sort(cands.begin(), cands.end(), [](const tdc_tile_info &a, const tdc_tile_info &b) { return a.pred_us < b.pred_us; });
    if ((int)cands.size() > classes) cands.resize(classes);
    while (cands.size() > 1 && cands.back().pred_us > 1.3 * cands.front().pred_us) cands.pop_back();

    const long long Ho = (d.H + 2LL * d.pad - (long long)d.dilation * (d.KH - 1) - 1) / d.stride + 1;
    const long long Wo = (d.W + 2LL * d.pad - (long long)d.dilation * (d.KW - 1) - 1) / d.stride + 1;
    const size_t in_bytes = (size_t)d.batch * d.C * d.H * d.W * sizeof(float);
    const size_t out_bytes = (size_t)d.batch * (tail_N > 0 ? tail_N : d.N) * Ho * Wo * sizeof(float);
    float *d_in = nullptr, *d_out = nullptr;
    hipError_t e = hipMalloc((void **)&d_in, in_bytes);
    if (e == hipSuccess) e = hipMalloc((void **)&d_out, out_bytes);
    if (e == hipSuccess) e = hipMemset(d_in, 0x3c, in_bytes);   // every float = 0.0115
    int st = e == hipSuccess ? TDC_OK : hip_fail("hipMalloc(tuning buffers)", e);
    double best_us = 1e30;
    for (size_t i = 0; i < cands.size() && st == TDC_OK; ++i) {
        tdc_conv_plan *plan = nullptr;
        st = tdc_conv_plan_create_with_tail(&d, tail_N, tail_has_bias, tail_relu, &cands[i].tile, &plan);
        if (st != TDC_OK) break;
        st = synthetic_weights(plan, true);
        double us = 1e30;
        for (int rep = 0; rep < 4 && st == TDC_OK; ++rep) {   // the first repetition warms up
            float ms = 0.0f;
            st = tdc_conv_time(plan, d_in, nullptr, d_out, 20, 1, &ms);
            if (rep > 0) us = std::min(us, (double)ms * 1e3 / 20);
        }
        tdc_conv_plan_destroy(plan);
        // the model's own favourite (first in the list) is only given up for a clear win: timings repeat to about 1 %
        if (st == TDC_OK && (i == 0 || us < 0.985 * best_us)) {
            best_us = us;
            best_out = cands[i].tile;
        }
    }
    if (d_in) (void)hipFree(d_in);
    if (d_out) (void)hipFree(d_out);
    if (st != TDC_OK) return st;
    if (log_tuning())
        std::fprintf(stderr, "tdc tune: conv %dx%d B%d C%d N%d %dx%d s%d tail %d: %zu classes timed, best %.2f us, alg %d wm %d wk %d tw %d "
                     "(model's pick %s, alg %d)\n",
                     d.KH, d.KW, d.batch, d.C, d.N, d.H, d.W, d.stride, tail_N, cands.size(), best_us, best_out.alg, best_out.wm,
                     best_out.wk, best_out.tw, std::memcmp(&best_out, &cands[0].tile, sizeof(tdc_tile)) == 0 ? "kept" : "replaced",
                     cands[0].tile.alg);
    std::lock_guard<std::mutex> lock(g_tune_mutex);
    g_tuned[key] = best_out;
    return TDC_OK;
}

int tdc_set_autotune(int32_t classes) {
    if (classes < 0 || classes > 256) return fail(TDC_ERR_INVALID, "autotune classes must be in [0, 256]");
    g_autotune.store(classes);
    return TDC_OK;
}

int tdc_get_autotune(void) { return g_autotune.load(); }

// Everything in the kernel arguments that the plan fixes (see tdc_conv_plan::kp).
static void refresh_launch_params(tdc_conv_plan *plan) {
    const tdc_conv_desc &d = plan->desc;
    const Geometry &g = plan->geo;
    ConvKParams kp{};
    kp.wpk = plan->d_wpk;
    kp.bias = plan->d_bias;
    kp.in_aff = plan->d_in_aff;
    kp.tail_w = plan->tail_N > 0 ? plan->d_tail_w : nullptr;
    kp.tail_bias = plan->d_tail_bias;
    kp.tail_N = plan->tail_N; kp.tail_mblk = (plan->tail_N + 15) / 16; kp.tail_ng = g.tail_ng; kp.tail_relu = plan->tail_relu;
    kp.tail_ld = g.tail_ld; kp.tail_f_off = g.tail_f_off;
    kp.head_w = plan->d_head_w;
    kp.head_C = plan->head_C; kp.head_runs = plan->head_runs; kp.head_mblk = plan->head_mblk; kp.head_npb = plan->head_npb;
    kp.head_ww = plan->head_ww; kp.head_wq = plan->head_wq; kp.head_ld = plan->head_ld; kp.head_f_off = plan->head_f_off;
    kp.win_rows = g.win_rows; kp.win_L = g.win_L; kp.win_nreq = g.win_nreq; kp.win_ns = g.win_ns; kp.win_off = g.win_off;
    kp.fd_winL = make_fastdiv(std::max(g.win_L, 1));
    kp.fd_hww = make_fastdiv(std::max(plan->head_ww, 1));
    kp.fd_hnpb = make_fastdiv(std::max(plan->head_npb, 1));
    kp.fd_npx = make_fastdiv(g.PT / 16);
    kp.in_relu = plan->in_relu;
    const long long in_image = (long long)(plan->head_C > 0 ? plan->head_C : d.C) * d.H * d.W;
    kp.in_image_bytes = (unsigned)(in_image * 4);
    kp.C = d.C; kp.H = g.He; kp.W = g.We; kp.N = d.N;
    kp.Ho = g.Ho; kp.Wo = g.Wo; kp.P = g.P;
    kp.KH = d.KH; kp.KW = d.KW; kp.stride = d.stride; kp.pad = d.pad; kp.dil = d.dilation;
    kp.TW = g.TW; kp.TH = g.TH; kp.ntx = g.ntx;
    kp.WM = plan->tile.wm; kp.WN = plan->tile.wn; kp.WK = plan->tile.wk;
    kp.CCH = plan->tile.cch; kp.nchunks = g.nchunks; kp.CPW = g.cpw;
    kp.KS = g.ks; kp.cps = g.cps; kp.WL = plan->tile.wl;
    kp.RS = g.RS; kp.CS = g.CS; kp.nrows = g.nrows;
    kp.VW = g.VW;   // (a forward falls back to 4-byte copy elements when its input is not 16-byte aligned)
    kp.in_stage_floats = g.in_stage_floats; kp.wslab_floats = g.wslab_floats;
    kp.in_nblk = g.in_stage_floats / (64 * g.VW);
    kp.stage_floats = g.stage_floats; kp.nstage = g.nstage;
    kp.relu = d.relu;
    kp.fd_csv = make_fastdiv(g.CS / g.VW);
    kp.fd_rsv = make_fastdiv(g.RS / g.VW);
    plan->fd_csv1 = make_fastdiv(g.CS);
    plan->fd_rsv1 = make_fastdiv(g.RS);
    kp.fd_tw = make_fastdiv(g.TW);
    kp.fd_ntx = make_fastdiv(g.ntx);
    kp.fd_pt = make_fastdiv(g.PT);
    kp.fd_wtw = make_fastdiv(g.wino ? g.TWt : (plan->tile.alg == 3 && d.stride > 1) ? g.Wo : 1);
    kp.fd_wk = make_fastdiv(plan->tile.wk);
    kp.fd_wn = make_fastdiv(plan->tile.wn);
    kp.fd_ks = make_fastdiv(g.ks);
    kp.grid_x = g.grid_x; kp.grid_y = g.grid_y;
    kp.n_wg = g.grid_x * g.grid_y * g.grid_z;
    kp.xcd_chunk = (kp.n_wg + 7) / 8;
    kp.channel_major = g.channel_major;
    kp.fd_g1 = make_fastdiv(g.channel_major ? g.grid_x : g.grid_y);
    kp.fd_g2 = make_fastdiv(g.channel_major ? g.grid_y : g.grid_x);
    kp.wpk_bytes = (unsigned)(packed_weight_floats(g) * sizeof(float));
#if defined(TDC_STAMPS) && TDC_STAMPS
    kp.stamps = plan->d_stamps;
#endif
    plan->kp = kp;
}

int tdc_conv_plan_create(const tdc_conv_desc *desc, const tdc_tile *forced_tile, tdc_conv_plan **plan_out) {
    return tdc_conv_plan_create_with_tail(desc, 0, 0, 0, forced_tile, plan_out);
}

int tdc_conv_plan_create_with_tail(const tdc_conv_desc *desc, int32_t tail_N, int32_t tail_has_bias, int32_t tail_relu,
                                   const tdc_tile *forced_tile, tdc_conv_plan **plan_out) {
    if (!desc || !plan_out) return fail(TDC_ERR_INVALID, "null argument");
    if (tail_N < 0) return fail(TDC_ERR_INVALID, "tail_N must be >= 0");
    *plan_out = nullptr;
    std::string why;
    if (!check_desc(*desc, &why)) return fail(TDC_ERR_INVALID, why);
    int ndev = 0;
    hipError_t e = hipGetDeviceCount(&ndev);
    if (e != hipSuccess || ndev < 1)
        return fail(TDC_ERR_HIP, "no HIP device available: the convolution kernels only run on a gfx950 GPU");
    std::unique_ptr<tdc_conv_plan> p(new (std::nothrow) tdc_conv_plan());
    if (!p) return fail(TDC_ERR_NOMEM, "out of host memory");
    p->desc = *desc;
    p->tail_N = tail_N;
    p->tail_has_bias = tail_N > 0 && tail_has_bias;
    p->tail_relu = tail_N > 0 && tail_relu;
    if (forced_tile) {
        if (!model_evaluate(*desc, *forced_tile, p->info, &why, tail_N)) return fail(TDC_ERR_INVALID, "forced tile: " + why);
    } else if (g_autotune.load() > 0) {
        tdc_tile tuned{};
        const int st = tune_tile(*desc, tail_N, p->tail_has_bias, p->tail_relu, g_autotune.load(), tuned);
        if (st != TDC_OK) return st;
        if (!model_evaluate(*desc, tuned, p->info, &why, tail_N)) return fail(TDC_ERR_INVALID, "tuned tile: " + why);
    } else {
        if (!model_select(*desc, p->info, &why, tail_N)) return fail(TDC_ERR_UNSUPPORTED, why);
    }
    p->tile = p->info.tile;
    if (!make_geometry(*desc, p->tile, p->geo, &why, tail_N)) return fail(TDC_ERR_INVALID, why);
    p->kernel = conv_kernel_for(p->tile, desc->KH, desc->KW, desc->dilation, desc->stride, tail_N > 0);
    if (!p->kernel) return fail(TDC_ERR_UNSUPPORTED, "no kernel instantiated for this tile");
    int he = prepare_conv_kernel(p->kernel, p->geo, &p->kernel_handle);
    if (he) return hip_fail("kernel set-up (hipFuncSetAttribute / hipGetFuncBySymbol)", he);
    const size_t wfloats = packed_weight_floats(p->geo);
    e = hipMalloc((void **)&p->d_wpk, wfloats * sizeof(float));
    if (e != hipSuccess) return hip_fail("hipMalloc(packed weights)", e);
    if (desc->has_bias) {
        e = hipMalloc((void **)&p->d_bias, (size_t)desc->N * sizeof(float));
        if (e != hipSuccess) {
            free_plan_buffers(p.get());
            return hip_fail("hipMalloc(bias)", e);
        }
    }
    if (tail_N > 0) {
        const size_t tw = (size_t)((tail_N + 15) / 16) * p->geo.tail_ng * 64;
        e = hipMalloc((void **)&p->d_tail_w, tw * sizeof(float));
        if (e == hipSuccess && p->tail_has_bias) e = hipMalloc((void **)&p->d_tail_bias, (size_t)tail_N * sizeof(float));
        if (e != hipSuccess) {
            free_plan_buffers(p.get());
            return hip_fail("hipMalloc(tail weights)", e);
        }
    }
    if (p->tile.ks > 1) {
        const size_t ws_floats = (size_t)p->geo.grid_z * desc->N * p->geo.P;
        const size_t nctr = (size_t)desc->batch * p->geo.grid_y * p->geo.grid_x;
        e = hipMalloc((void **)&p->d_ws, ws_floats * sizeof(float));
        if (e == hipSuccess) e = hipMalloc((void **)&p->d_ctr, nctr * sizeof(unsigned));
        if (e == hipSuccess) e = hipMemset(p->d_ctr, 0, nctr * sizeof(unsigned));
        if (e != hipSuccess) {
            free_plan_buffers(p.get());
            return hip_fail("hipMalloc(split-K workspace)", e);
        }
    }
#if defined(TDC_STAMPS) && TDC_STAMPS
    p->stamp_words = (size_t)p->geo.grid_x * p->geo.grid_y * p->geo.grid_z * 16 * 8;
    e = hipMalloc((void **)&p->d_stamps, p->stamp_words * 8);
    if (e == hipSuccess) e = hipMemset(p->d_stamps, 0, p->stamp_words * 8);
    if (e != hipSuccess) {
        free_plan_buffers(p.get());
        return hip_fail("hipMalloc(time stamps)", e);
    }
#endif
    refresh_launch_params(p.get());
    *plan_out = p.release();
    return TDC_OK;
}

int tdc_conv_plan_set_weights(tdc_conv_plan *plan, const float *w_oihw, const float *bias) {
    if (!plan || !w_oihw) return fail(TDC_ERR_INVALID, "null argument");
    if ((plan->desc.has_bias != 0) != (bias != nullptr))
        return fail(TDC_ERR_INVALID, "bias pointer does not match desc.has_bias");
    const size_t wfloats = packed_weight_floats(plan->geo);
    std::vector<float> packed;
    try {
        packed.resize(wfloats);
    } catch (const std::bad_alloc &) {
        return fail(TDC_ERR_NOMEM, "out of host memory packing weights");
    }
    pack_weights(plan->desc, plan->tile, plan->geo, w_oihw, packed.data());
    hipError_t e = hipMemcpy(plan->d_wpk, packed.data(), wfloats * sizeof(float), hipMemcpyHostToDevice);
    if (e != hipSuccess) return hip_fail("hipMemcpy(packed weights)", e);
    if (bias) {
        e = hipMemcpy(plan->d_bias, bias, (size_t)plan->desc.N * sizeof(float), hipMemcpyHostToDevice);
        if (e != hipSuccess) return hip_fail("hipMemcpy(bias)", e);
    }
    plan->have_weights = true;
    return TDC_OK;
}

int tdc_conv_plan_set_tail_weights(tdc_conv_plan *plan, const float *w_tail, const float *bias_tail) {
    if (!plan || !w_tail) return fail(TDC_ERR_INVALID, "null argument");
    if (plan->tail_N <= 0) return fail(TDC_ERR_STATE, "this plan was created without a fused tail");
    if ((plan->tail_has_bias != 0) != (bias_tail != nullptr))
        return fail(TDC_ERR_INVALID, "tail bias pointer does not match the plan");
    // [16-row block][K-step][64 lanes] in MFMA A order: lane l of an entry holds w_tail[block*16 + l%16][4*kstep + l/16].
    const int N = plan->desc.N, N2 = plan->tail_N, ng = plan->geo.tail_ng, mblk = (N2 + 15) / 16;
    std::vector<float> packed((size_t)mblk * ng * 64, 0.0f);
    for (int mb = 0; mb < mblk; ++mb)
        for (int g = 0; g < ng; ++g)
            for (int l = 0; l < 64; ++l) {
                const int n2 = mb * 16 + l % 16, c = 4 * g + l / 16;
                if (n2 < N2 && c < N) packed[((size_t)mb * ng + g) * 64 + l] = w_tail[(size_t)n2 * N + c];
            }
    hipError_t e = hipMemcpy(plan->d_tail_w, packed.data(), packed.size() * sizeof(float), hipMemcpyHostToDevice);
    if (e == hipSuccess && bias_tail)
        e = hipMemcpy(plan->d_tail_bias, bias_tail, (size_t)N2 * sizeof(float), hipMemcpyHostToDevice);
    if (e != hipSuccess) return hip_fail("hipMemcpy(tail weights)", e);
    plan->have_tail_weights = true;
    return TDC_OK;
}

int tdc_conv_plan_set_input_affine(tdc_conv_plan *plan, const float *scale, const float *shift, int32_t relu) {
    if (!plan || !scale || !shift) return fail(TDC_ERR_INVALID, "null argument");
    const tdc_conv_desc &d = plan->desc;
    if (d.KH != 1 || d.KW != 1 || d.pad != 0)
        return fail(TDC_ERR_UNSUPPORTED, "an input affine can only be fused into a 1x1 convolution without padding");
    const int cch = plan->tile.cch, nchunks = plan->geo.nchunks;
    const size_t n = (size_t)nchunks * 2 * cch;
    std::vector<float> packed(n, 0.0f);   // channels past C: 0*x + 0
    for (int c = 0; c < d.C; ++c) {
        packed[(size_t)(c / cch) * 2 * cch + c % cch] = scale[c];
        packed[(size_t)(c / cch) * 2 * cch + cch + c % cch] = shift[c];
    }
    hipError_t e = hipSuccess;
    if (!plan->d_in_aff) e = hipMalloc((void **)&plan->d_in_aff, n * sizeof(float));
    if (e == hipSuccess) e = hipMemcpy(plan->d_in_aff, packed.data(), n * sizeof(float), hipMemcpyHostToDevice);
    if (e != hipSuccess) return hip_fail("input affine upload", e);
    // from now on this plan needs the kernel instantiation that carries the extras
    plan->kernel = conv_kernel_for(plan->tile, d.KH, d.KW, d.dilation, d.stride, true);
    if (!plan->kernel) return fail(TDC_ERR_UNSUPPORTED, "no kernel instantiated for this tile");
    if (int he = prepare_conv_kernel(plan->kernel, plan->geo, &plan->kernel_handle)) return hip_fail("kernel set-up (hipFuncSetAttribute / hipGetFuncBySymbol)", he);
    plan->in_relu = relu != 0;
    refresh_launch_params(plan);
    return TDC_OK;
}

int tdc_conv_plan_set_head(tdc_conv_plan *plan, int32_t head_C, const float *w_head) {
    if (!plan || !w_head) return fail(TDC_ERR_INVALID, "null argument");
    if (head_C < 1) return fail(TDC_ERR_INVALID, "head_C must be >= 1");
    const tdc_conv_desc &d = plan->desc;
    const tdc_tile &t = plan->tile;
    Geometry &g = plan->geo;
    if (t.alg != 4 || plan->tail_N <= 0 || d.KH != 3 || d.KW != 3 || d.stride != 1 || d.dilation != 1)
        return fail(TDC_ERR_UNSUPPORTED, "a fused head needs a streamed 3x3 / stride 1 plan (tile.alg = 4) with a fused tail");
    if (plan->d_in_aff) return fail(TDC_ERR_UNSUPPORTED, "a fused head cannot be combined with an input affine");
    if ((long long)head_C * d.H * d.W * 4 >= (1LL << 31)) return fail(TDC_ERR_UNSUPPORTED, "image too large for a fused head");
    const void *kernel = conv_kernel_with_head(t);
    if (!kernel) return fail(TDC_ERR_UNSUPPORTED, "no kernel instantiated for this tile");
    const int runs = ((head_C + 15) / 16 + 3) / 4 * 4;   // the kernel requests four runs at a time
    const int mblk = (t.cch + 15) / 16;                   // every input channel row of the core, padding included
    const int ww = g.TW + 2, wq = (g.TH + 2) * ww, npb = (wq + 15) / 16;
    int ld = npb * 16;
    if (ld % 32 == 0) ld += 16;                           // the four channel quarters of a K-step in different banks
    const int f_off = g.tail_f_off + g.MT * g.tail_ld;
    const long long lds = ((long long)f_off + (long long)mblk * 16 * ld) * 4;
    if (lds > machine().lds_bytes_per_cu) return fail(TDC_ERR_UNSUPPORTED, "the window of the fused head does not fit the LDS");
    // [16-row block][run][lane][4]: lane l (row l % 16, quarter l / 16) holds w_head[block*16 + l%16][16*run + 4*(l/16) + e]
    std::vector<float> packed((size_t)mblk * runs * 256, 0.0f);
    for (int cb = 0; cb < mblk; ++cb)
        for (int r = 0; r < runs; ++r)
            for (int l = 0; l < 64; ++l)
                for (int e = 0; e < 4; ++e) {
                    const int n = cb * 16 + l % 16, c = 16 * r + 4 * (l / 16) + e;
                    if (n < d.C && c < head_C) packed[(((size_t)cb * runs + r) * 64 + l) * 4 + e] = w_head[(size_t)n * head_C + c];
                }
    if (plan->d_head_w) (void)hipFree(plan->d_head_w);
    plan->d_head_w = nullptr;
    hipError_t e = hipMalloc((void **)&plan->d_head_w, packed.size() * sizeof(float));
    if (e == hipSuccess) e = hipMemcpy(plan->d_head_w, packed.data(), packed.size() * sizeof(float), hipMemcpyHostToDevice);
    if (e != hipSuccess) return hip_fail("fused head upload", e);
    g.lds_bytes = std::max(g.lds_bytes, (int)lds);
    plan->info.lds_bytes = g.lds_bytes;
    plan->kernel = kernel;
    if (int he = prepare_conv_kernel(plan->kernel, g, &plan->kernel_handle)) return hip_fail("kernel set-up (hipFuncSetAttribute / hipGetFuncBySymbol)", he);
    plan->head_C = head_C; plan->head_runs = runs; plan->head_mblk = mblk; plan->head_npb = npb;
    plan->head_ww = ww; plan->head_wq = wq; plan->head_ld = ld; plan->head_f_off = f_off;
    refresh_launch_params(plan);
    return TDC_OK;
}

int tdc_conv_plan_occupancy(const tdc_conv_plan *plan, tdc_kernel_occupancy *out) {
    if (!plan || !out) return fail(TDC_ERR_INVALID, "null argument");
    std::memset(out, 0, sizeof(*out));
    int vgprs = 0, static_lds = 0, max_threads = 0, wg = 0;
    if (int he = kernel_resources(plan->kernel, plan->geo.threads, plan->geo.lds_bytes, &vgprs, &static_lds, &max_threads, &wg))
        return hip_fail("hipFuncGetAttributes / hipOccupancyMaxActiveBlocksPerMultiprocessor", he);
    out->kernel_vgprs = vgprs;
    out->kernel_static_lds_bytes = static_lds;
    out->kernel_max_threads = max_threads;
    out->runtime_wg_per_cu = wg;
    out->block_threads = plan->geo.threads;
    out->dynamic_lds_bytes = plan->geo.lds_bytes;
    out->model_vgprs = plan->info.vgpr_estimate;
    out->model_wg_per_cu = plan->info.wg_per_cu;
    return TDC_OK;
}

int tdc_conv_plan_query(const tdc_conv_plan *plan, tdc_tile_info *info_out) {
    if (!plan || !info_out) return fail(TDC_ERR_INVALID, "null argument");
    *info_out = plan->info;
    return TDC_OK;
}

int tdc_conv_forward(tdc_conv_plan *plan, const float *d_in, const float *d_residual, float *d_out, void *stream) {
    return tdc_conv_forward_strided(plan, d_in, 0, d_residual, 0, d_out, 0, stream);
}

// The launch behind every forward entry point.  `ws` / `ctr`: where a plan whose tile splits the input channels over
// several workgroups keeps its partial tiles and ticket counters (the plan's own buffers, or the static scratch).
static int forward_impl(tdc_conv_plan *plan, const float *d_in, int64_t in_batch_stride, const float *d_residual,
                        int64_t residual_batch_stride, float *d_out, int64_t out_batch_stride, float *ws, unsigned *ctr,
                        void *stream);

int tdc_conv_forward_strided(tdc_conv_plan *plan, const float *d_in, int64_t in_batch_stride, const float *d_residual,
                             int64_t residual_batch_stride, float *d_out, int64_t out_batch_stride, void *stream) {
    if (!plan) return fail(TDC_ERR_INVALID, "null argument");
    return forward_impl(plan, d_in, in_batch_stride, d_residual, residual_batch_stride, d_out, out_batch_stride, plan->d_ws,
                        plan->d_ctr, stream);
}

int tdc_conv_forward_static_ws(tdc_conv_plan *plan, const float *d_in, const float *d_residual, float *d_out, void *stream) {
    if (!plan) return fail(TDC_ERR_INVALID, "null argument");
    if (plan->tile.ks <= 1)   // no partial tiles, no counters: nothing to place
        return forward_impl(plan, d_in, 0, d_residual, 0, d_out, 0, nullptr, nullptr, stream);
    const size_t ws_bytes = (size_t)plan->geo.grid_z * plan->desc.N * plan->geo.P * sizeof(float);
    const size_t ctr_bytes = (size_t)plan->desc.batch * plan->geo.grid_y * plan->geo.grid_x * sizeof(unsigned);
    if (ws_bytes > static_scratch_ws_bytes() || ctr_bytes > static_scratch_ctr_bytes())
        return fail(TDC_ERR_UNSUPPORTED,
                    "tdc_conv_forward_static_ws: this plan needs " + std::to_string(ws_bytes) + " bytes of partial tiles and " +
                        std::to_string(ctr_bytes) + " bytes of counters; the static scratch holds " +
                        std::to_string(static_scratch_ws_bytes()) + " and " + std::to_string(static_scratch_ctr_bytes()));
    void *base = nullptr;
    if (int he = static_scratch_address(&base)) return hip_fail("hipGetSymbolAddress(static scratch)", he);
    float *ws = reinterpret_cast<float *>(base);
    unsigned *ctr = reinterpret_cast<unsigned *>(reinterpret_cast<char *>(base) + static_scratch_ws_bytes());
    // The array keeps whatever the last call (of any plan) left in it: the counters this launch uses must start at
    // zero.  A fill kernel, not hipMemsetAsync: this call may sit inside a stream capture.
    if (int he = launch_zero_words(ctr, (int)(ctr_bytes / sizeof(unsigned)), stream)) return hip_fail("counter fill launch", he);
    return forward_impl(plan, d_in, 0, d_residual, 0, d_out, 0, ws, ctr, stream);
}

static int forward_impl(tdc_conv_plan *plan, const float *d_in, int64_t in_batch_stride, const float *d_residual,
                        int64_t residual_batch_stride, float *d_out, int64_t out_batch_stride, float *ws, unsigned *ctr,
                        void *stream) {
    if (!plan || !d_in || !d_out) return fail(TDC_ERR_INVALID, "null argument");
    if (in_batch_stride < 0 || out_batch_stride < 0 || residual_batch_stride < 0)
        return fail(TDC_ERR_INVALID, "negative batch stride");
    if (!plan->have_weights) return fail(TDC_ERR_STATE, "tdc_conv_forward before tdc_conv_plan_set_weights");
    if (plan->tail_N > 0 && !plan->have_tail_weights)
        return fail(TDC_ERR_STATE, "tdc_conv_forward before tdc_conv_plan_set_tail_weights");
    const tdc_conv_desc &d = plan->desc;
    const Geometry &g = plan->geo;
    const long long in_image = (long long)(plan->head_C > 0 ? plan->head_C : d.C) * d.H * d.W;
    const long long out_image = (long long)(plan->tail_N > 0 ? plan->tail_N : d.N) * g.P;
    if ((in_batch_stride && in_batch_stride < in_image) || (out_batch_stride && out_batch_stride < out_image) ||
        (residual_batch_stride && residual_batch_stride < out_image))
        return fail(TDC_ERR_INVALID, "batch stride smaller than one image");
    ConvKParams kp = plan->kp;
    kp.in = d_in;
    kp.resid = d_residual;
    kp.out = d_out;
    kp.ws = ws;
    kp.ctr = ctr;
    kp.in_bstride = in_batch_stride ? in_batch_stride : in_image;
    kp.out_bstride = out_batch_stride ? out_batch_stride : out_image;
    kp.resid_bstride = residual_batch_stride ? residual_batch_stride : out_image;
    // 16-byte copy elements need every image of the batch 16-byte aligned; otherwise 4-byte elements.
    if (g.VW == 4 && !(reinterpret_cast<uintptr_t>(d_in) % 16 == 0 && kp.in_bstride % 4 == 0)) {
        kp.VW = 1;
        kp.in_nblk = g.in_stage_floats / 64;   // (copy blocks of the element width this launch really copies with)
        kp.fd_csv = plan->fd_csv1;
        kp.fd_rsv = plan->fd_rsv1;
    }
    int he = launch_conv(plan->kernel_handle, g, kp, stream);
    if (he) return hip_fail("kernel launch", he);
    return TDC_OK;
}

int tdc_conv_time_many(tdc_conv_plan *const *plans, const float *const *d_ins, float *const *d_outs, int32_t n,
                       int32_t iters, int32_t use_graph, float *total_ms_out) {
    return time_plans(plans, d_ins, d_outs, n, 1, iters, use_graph, total_ms_out);
}

}  // extern "C"

// hipEvents around `iters` repetitions of `passes` passes over the list; with `use_graph` the `passes` passes are
// one HIP graph that is replayed `iters` times.
static int time_plans(tdc_conv_plan *const *plans, const float *const *d_ins, float *const *d_outs, int n, int passes,
                      int iters, int use_graph, float *total_ms_out) {
    if (!plans || !d_ins || !d_outs || !total_ms_out || n < 1 || iters < 1 || passes < 1)
        return fail(TDC_ERR_INVALID, "bad argument");
    for (int i = 0; i < n; ++i)
        if (!plans[i] || !d_ins[i] || !d_outs[i]) return fail(TDC_ERR_INVALID, "null plan or buffer in list");
    hipStream_t s = nullptr;
    hipEvent_t e0 = nullptr, e1 = nullptr;
    hipGraph_t graph = nullptr;
    hipGraphExec_t exec = nullptr;
    int st = TDC_OK;
    auto one_pass = [&]() {
        for (int k = 0; k < passes; ++k)
            for (int i = 0; i < n && st == TDC_OK; ++i) st = tdc_conv_forward(plans[i], d_ins[i], nullptr, d_outs[i], s);
    };
    const char *what = "hipStreamCreate";
    hipError_t e = hipDeviceSynchronize();
    if (e == hipSuccess) e = hipStreamCreate(&s);
    if (e == hipSuccess) { what = "hipEventCreate"; e = hipEventCreate(&e0); }
    if (e == hipSuccess) e = hipEventCreate(&e1);
    if (e == hipSuccess && use_graph) {
        // One pass over the list is one graph; the timed region replays it `iters` times.
        what = "graph capture";
        e = hipStreamBeginCapture(s, hipStreamCaptureModeThreadLocal);
        if (e == hipSuccess) {
            one_pass();
            e = hipStreamEndCapture(s, &graph);
        }
        if (e == hipSuccess && st == TDC_OK) e = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
        if (e == hipSuccess && st == TDC_OK) e = hipGraphLaunch(exec, s);  // untimed: upload
        if (e == hipSuccess && st == TDC_OK) e = hipStreamSynchronize(s);
    }
    if (e == hipSuccess && st == TDC_OK) {
        what = "timed region";
        e = hipEventRecord(e0, s);
        for (int it = 0; it < iters && st == TDC_OK && e == hipSuccess; ++it) {
            if (use_graph) e = hipGraphLaunch(exec, s);
            else one_pass();
        }
        if (e == hipSuccess) e = hipEventRecord(e1, s);
        if (e == hipSuccess) e = hipEventSynchronize(e1);
        if (e == hipSuccess) e = hipEventElapsedTime(total_ms_out, e0, e1);
    }
    if (exec) (void)hipGraphExecDestroy(exec);
    if (graph) (void)hipGraphDestroy(graph);
    if (e0) (void)hipEventDestroy(e0);
    if (e1) (void)hipEventDestroy(e1);
    if (s) (void)hipStreamDestroy(s);
    if (st != TDC_OK) return st;
    if (e != hipSuccess) return hip_fail(what, e);
    return TDC_OK;
}

extern "C" {

int tdc_conv_time(tdc_conv_plan *plan, const float *d_in, const float *d_residual, float *d_out, int32_t iters,
                  int32_t use_graph, float *total_ms_out) {
    if (!plan || !total_ms_out || iters < 1) return fail(TDC_ERR_INVALID, "bad argument");
    hipStream_t s = nullptr;
    hipEvent_t e0 = nullptr, e1 = nullptr;
    hipGraph_t graph = nullptr;
    hipGraphExec_t exec = nullptr;
    int st = TDC_OK;
    const char *what = "hipStreamCreate";
    hipError_t e = hipDeviceSynchronize();
    if (e == hipSuccess) e = hipStreamCreate(&s);
    if (e == hipSuccess) { what = "hipEventCreate"; e = hipEventCreate(&e0); }
    if (e == hipSuccess) e = hipEventCreate(&e1);
    if (e == hipSuccess && use_graph) {
        what = "graph capture";
        e = hipStreamBeginCapture(s, hipStreamCaptureModeThreadLocal);
        if (e == hipSuccess) {
            for (int i = 0; i < iters && st == TDC_OK; ++i) st = tdc_conv_forward(plan, d_in, d_residual, d_out, s);
            e = hipStreamEndCapture(s, &graph);
        }
        if (e == hipSuccess && st == TDC_OK) e = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
        // One untimed replay so that the timed one does not pay for the upload.
        if (e == hipSuccess && st == TDC_OK) e = hipGraphLaunch(exec, s);
        if (e == hipSuccess && st == TDC_OK) e = hipStreamSynchronize(s);
    }
    if (e == hipSuccess && st == TDC_OK) {
        what = "timed region";
        e = hipEventRecord(e0, s);
        if (use_graph) {
            if (e == hipSuccess) e = hipGraphLaunch(exec, s);
        } else {
            for (int i = 0; i < iters && st == TDC_OK; ++i) st = tdc_conv_forward(plan, d_in, d_residual, d_out, s);
        }
        if (e == hipSuccess) e = hipEventRecord(e1, s);
        if (e == hipSuccess) e = hipEventSynchronize(e1);
        if (e == hipSuccess) e = hipEventElapsedTime(total_ms_out, e0, e1);
    }
    if (exec) (void)hipGraphExecDestroy(exec);
    if (graph) (void)hipGraphDestroy(graph);
    if (e0) (void)hipEventDestroy(e0);
    if (e1) (void)hipEventDestroy(e1);
    if (s) (void)hipStreamDestroy(s);
    if (st != TDC_OK) return st;
    if (e != hipSuccess) return hip_fail(what, e);
    return TDC_OK;
}

int tdc_launch_floor_time(int32_t launches, int32_t use_graph, int32_t grid, int32_t block, float spin_us, float *total_ms_out) {
    if (!total_ms_out || launches < 1 || launches > 100000 || grid < 1 || grid > 65535 || block < 64 || block > 1024 ||
        block % 64 != 0 || !(spin_us >= 0.0f) || spin_us > 100.0f)
        return fail(TDC_ERR_INVALID, "bad argument");
    const int ticks = (int)(spin_us * 100.0f + 0.5f);
    ConvKParams kp{};
    hipStream_t s = nullptr;
    hipEvent_t e0 = nullptr, e1 = nullptr;
    hipGraph_t graph = nullptr;
    hipGraphExec_t exec = nullptr;
    int he = 0;
    void *probe = nullptr;
    if (int pe = launch_floor_probe_handle(&probe)) return hip_fail("hipGetFuncBySymbol(launch probe)", pe);
    const char *what = "hipStreamCreate";
    hipError_t e = hipDeviceSynchronize();
    if (e == hipSuccess) e = hipStreamCreate(&s);
    if (e == hipSuccess) { what = "hipEventCreate"; e = hipEventCreate(&e0); }
    if (e == hipSuccess) e = hipEventCreate(&e1);
    if (e == hipSuccess && use_graph) {
        what = "graph capture";
        e = hipStreamBeginCapture(s, hipStreamCaptureModeThreadLocal);
        if (e == hipSuccess) {
            for (int i = 0; i < launches && !he; ++i) he = launch_floor_probe(probe, kp, grid, block, ticks, s);
            e = hipStreamEndCapture(s, &graph);
        }
        if (e == hipSuccess && !he) e = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
        if (e == hipSuccess && !he) e = hipGraphLaunch(exec, s);   // untimed: upload
        if (e == hipSuccess && !he) e = hipStreamSynchronize(s);
    } else if (e == hipSuccess) {
        for (int i = 0; i < 20 && !he; ++i) he = launch_floor_probe(probe, kp, grid, block, ticks, s);   // untimed: warm-up
        e = hipStreamSynchronize(s);
    }
    if (e == hipSuccess && !he) {
        what = "timed region";
        e = hipEventRecord(e0, s);
        if (use_graph) {
            if (e == hipSuccess) e = hipGraphLaunch(exec, s);
        } else {
            for (int i = 0; i < launches && !he; ++i) he = launch_floor_probe(probe, kp, grid, block, ticks, s);
        }
        if (e == hipSuccess) e = hipEventRecord(e1, s);
        if (e == hipSuccess) e = hipEventSynchronize(e1);
        if (e == hipSuccess) e = hipEventElapsedTime(total_ms_out, e0, e1);
    }
    if (exec) (void)hipGraphExecDestroy(exec);
    if (graph) (void)hipGraphDestroy(graph);
    if (e0) (void)hipEventDestroy(e0);
    if (e1) (void)hipEventDestroy(e1);
    if (s) (void)hipStreamDestroy(s);
    if (he) return hip_fail("probe launch", he);
    if (e != hipSuccess) return hip_fail(what, e);
    return TDC_OK;
}

void tdc_conv_plan_destroy(tdc_conv_plan *plan) {
    if (!plan) return;
    free_plan_buffers(plan);
    delete plan;
}

// ---- TKConv ---------------------------------------------------------------

// Core + last factor: one fused launch or two?  Times both on the operator's own intermediates (synthetic
// weights) and drops the fused plan when the two launches are not slower.  Remembered per problem.
static std::map<std::array<int, 13>, bool> g_fusion_pays;

static int tkconv_measure_fusion(tdc_tkconv *op) {
    const tdc_tkconv_desc &d = op->desc;
    const std::array<int, 13> key{d.batch, d.C, d.R1, d.R2, d.N, d.H, d.W, d.K, d.stride, d.pad, d.dilation, d.has_bias, d.relu};
    bool known = false, pays = false;
    {
        std::lock_guard<std::mutex> lock(g_tune_mutex);
        auto hit = g_fusion_pays.find(key);
        if (hit != g_fusion_pays.end()) {
            known = true;
            pays = hit->second;
        }
    }
    if (!known) {
        // Both alternatives are timed BEHIND the first factor, so that the core reads an intermediate another kernel has
        // just written, as it does inside a network (timed on an intermediate that never changes, the two launches look up
        // to 20 % better than they are there).
        const size_t in_floats = (size_t)d.batch * d.C * d.H * d.W;
        const size_t out_floats = (size_t)d.batch * d.N * (op->f2_floats / ((size_t)d.batch * d.R2));
        float *d_in = nullptr, *d_out = nullptr;
        hipError_t e = hipMalloc((void **)&d_in, in_floats * sizeof(float));
        if (e == hipSuccess) e = hipMalloc((void **)&d_out, out_floats * sizeof(float));
        if (e == hipSuccess) e = hipMemset(d_in, 0x3c, in_floats * sizeof(float));
        if (e != hipSuccess) {
            if (d_in) (void)hipFree(d_in);
            if (d_out) (void)hipFree(d_out);
            return hip_fail("hipMalloc(fusion timing)", e);
        }
        int st = synthetic_weights(op->first, true);
        if (st == TDC_OK) st = synthetic_weights(op->core, true);
        if (st == TDC_OK) st = synthetic_weights(op->last, true);
        if (st == TDC_OK) st = synthetic_weights(op->core_last, true);
        tdc_conv_plan *two[3] = {op->first, op->core, op->last};
        const float *ins2[3] = {d_in, op->d_f1, op->d_f2};
        float *outs2[3] = {op->d_f1, op->d_f2, d_out};
        tdc_conv_plan *one[2] = {op->first, op->core_last};
        const float *ins1[2] = {d_in, op->d_f1};
        float *outs1[2] = {op->d_f1, d_out};
        double us_two = 1e30, us_one = 1e30;
        for (int rep = 0; rep < 4 && st == TDC_OK; ++rep) {   // the first repetition warms up
            float ms = 0.0f;
            // ten passes per graph: a graph launch costs more than one of these kernels
            st = time_plans(two, ins2, outs2, 3, 10, 2, 1, &ms);
            if (st == TDC_OK && rep > 0) us_two = std::min(us_two, (double)ms * 1e3 / 20);
            if (st == TDC_OK) st = time_plans(one, ins1, outs1, 2, 10, 2, 1, &ms);
            if (st == TDC_OK && rep > 0) us_one = std::min(us_one, (double)ms * 1e3 / 20);
        }
        (void)hipFree(d_in);
        (void)hipFree(d_out);
        synthetic_weights(op->first, false);
        synthetic_weights(op->core, false);
        synthetic_weights(op->last, false);
        synthetic_weights(op->core_last, false);
        if (st != TDC_OK) return st;
        pays = us_one < 1.05 * us_two;
        if (log_tuning())
            std::fprintf(stderr, "tdc tune: tkconv C%d R%d,%d N%d %dx%d K%d s%d: first + core+last fused %.2f us, three launches %.2f us\n",
                         d.C, d.R1, d.R2, d.N, d.H, d.W, d.K, d.stride, us_one, us_two);
        std::lock_guard<std::mutex> lock(g_tune_mutex);
        g_fusion_pays[key] = pays;
    }
    if (!pays) {
        tdc_conv_plan_destroy(op->core_last);
        op->core_last = nullptr;
    }
    return TDC_OK;
}

// One launch for the whole operator, or the first factor on its own in front of core + last?  Timed as dependent
// chains on the operator's own intermediates (synthetic weights); remembered per problem.
static std::map<std::array<int, 13>, bool> g_whole_pays;

static int tkconv_measure_whole(tdc_tkconv *op) {
    const tdc_tkconv_desc &d = op->desc;
    const std::array<int, 13> key{d.batch, d.C, d.R1, d.R2, d.N, d.H, d.W, d.K, d.stride, d.pad, d.dilation, d.has_bias, d.relu};
    bool known = false, pays = false;
    {
        std::lock_guard<std::mutex> lock(g_tune_mutex);
        auto hit = g_whole_pays.find(key);
        if (hit != g_whole_pays.end()) {
            known = true;
            pays = hit->second;
        }
    }
    if (!known) {
        const size_t in_floats = (size_t)d.batch * d.C * d.H * d.W;
        const size_t out_floats = (size_t)d.batch * d.N * (op->f2_floats / ((size_t)d.batch * d.R2));
        float *d_in = nullptr, *d_out = nullptr;
        hipError_t e = hipMalloc((void **)&d_in, in_floats * sizeof(float));
        if (e == hipSuccess) e = hipMalloc((void **)&d_out, out_floats * sizeof(float));
        if (e == hipSuccess) e = hipMemset(d_in, 0x3c, in_floats * sizeof(float));
        if (e != hipSuccess) {
            if (d_in) (void)hipFree(d_in);
            if (d_out) (void)hipFree(d_out);
            return hip_fail("hipMalloc(fusion timing)", e);
        }
        int st = synthetic_weights(op->first, true);
        if (st == TDC_OK) st = synthetic_weights(op->core_last, true);
        if (st == TDC_OK) st = synthetic_weights(op->whole, true);
        tdc_conv_plan *two[2] = {op->first, op->core_last};
        const float *ins[2] = {d_in, op->d_f1};
        float *outs[2] = {op->d_f1, d_out};
        tdc_conv_plan *one[1] = {op->whole};
        double us_two = 1e30, us_one = 1e30;
        for (int rep = 0; rep < 4 && st == TDC_OK; ++rep) {   // the first repetition warms up
            float ms = 0.0f;
            st = time_plans(two, ins, outs, 2, 10, 2, 1, &ms);
            if (st == TDC_OK && rep > 0) us_two = std::min(us_two, (double)ms * 1e3 / 20);
            if (st == TDC_OK) st = time_plans(one, ins, outs + 1, 1, 10, 2, 1, &ms);
            if (st == TDC_OK && rep > 0) us_one = std::min(us_one, (double)ms * 1e3 / 20);
        }
        (void)hipFree(d_in);
        (void)hipFree(d_out);
        synthetic_weights(op->first, false);
        synthetic_weights(op->core_last, false);
        synthetic_weights(op->whole, false);
        if (st != TDC_OK) return st;
        pays = us_one < 0.97 * us_two;
        if (log_tuning())
            std::fprintf(stderr, "tdc tune: tkconv C%d R%d,%d N%d %dx%d K%d s%d: one launch %.2f us, first + core+last %.2f us\n",
                         d.C, d.R1, d.R2, d.N, d.H, d.W, d.K, d.stride, us_one, us_two);
        std::lock_guard<std::mutex> lock(g_tune_mutex);
        g_whole_pays[key] = pays;
    }
    if (!pays) {
        tdc_conv_plan_destroy(op->whole);
        op->whole = nullptr;
    }
    return TDC_OK;
}

int tdc_tkconv_create(const tdc_tkconv_desc *desc, tdc_tkconv **op_out) {
    if (!desc || !op_out) return fail(TDC_ERR_INVALID, "null argument");
    *op_out = nullptr;
    if (desc->R1 < 1 || desc->R2 < 1 || desc->K < 1) return fail(TDC_ERR_INVALID, "R1, R2, K must be >= 1");
    std::unique_ptr<tdc_tkconv> op(new (std::nothrow) tdc_tkconv());
    if (!op) return fail(TDC_ERR_NOMEM, "out of host memory");
    op->desc = *desc;
    tdc_conv_desc d1{desc->batch, desc->C, desc->R1, desc->H, desc->W, 1, 1, 1, 0, 1, 0, 0};
    tdc_conv_desc d2{desc->batch, desc->R1, desc->R2, desc->H, desc->W, desc->K, desc->K,
                     desc->stride, desc->pad, desc->dilation, 0, 0};
    std::string why;
    if (!check_desc(d1, &why)) return fail(TDC_ERR_INVALID, "first 1x1: " + why);
    if (!check_desc(d2, &why)) return fail(TDC_ERR_INVALID, "core conv: " + why);
    const int Ho = (desc->H + 2 * desc->pad - desc->dilation * (desc->K - 1) - 1) / desc->stride + 1;
    const int Wo = (desc->W + 2 * desc->pad - desc->dilation * (desc->K - 1) - 1) / desc->stride + 1;
    tdc_conv_desc d3{desc->batch, desc->R2, desc->N, Ho, Wo, 1, 1, 1, 0, 1, desc->has_bias, desc->relu};
    if (!check_desc(d3, &why)) return fail(TDC_ERR_INVALID, "last 1x1: " + why);
    int st;
    auto cleanup = [&]() {
        tdc_conv_plan_destroy(op->first);
        tdc_conv_plan_destroy(op->core);
        tdc_conv_plan_destroy(op->last);
        tdc_conv_plan_destroy(op->core_last);
        tdc_conv_plan_destroy(op->whole);
        if (op->d_f1) (void)hipFree(op->d_f1);
        if (op->d_f2) (void)hipFree(op->d_f2);
    };
    if ((st = tdc_conv_plan_create(&d1, nullptr, &op->first)) != TDC_OK) { cleanup(); return st; }
    if ((st = tdc_conv_plan_create(&d2, nullptr, &op->core)) != TDC_OK) { cleanup(); return st; }
    if ((st = tdc_conv_plan_create(&d3, nullptr, &op->last)) != TDC_OK) { cleanup(); return st; }
    op->f1_floats = (size_t)desc->batch * desc->R1 * desc->H * desc->W;
    op->f2_floats = (size_t)desc->batch * desc->R2 * Ho * Wo;
    hipError_t e = hipMalloc((void **)&op->d_f1, op->f1_floats * sizeof(float));
    if (e != hipSuccess) { cleanup(); return hip_fail("hipMalloc(first intermediate)", e); }
    e = hipMalloc((void **)&op->d_f2, op->f2_floats * sizeof(float));
    if (e != hipSuccess) { cleanup(); return hip_fail("hipMalloc(core intermediate)", e); }
    // Core + last factor as one kernel, if the model predicts it faster than the two launches (it needs all R2
    // channels in one workgroup, so it only pays for small R2).  The three plain plans stay: they serve
    // forward_features and core_forward.
    if (!std::getenv("TDC_EXPERIMENT_NO_FUSED_TAIL")) {
        tdc_tile_info fused{};
        const double separate_us = op->core->info.pred_us + op->last->info.pred_us;
        const bool measure = g_autotune.load() > 0;
        // With measured selection on, a fused kernel predicted within 30 % of the two launches is built and the
        // two alternatives are timed; otherwise the prediction decides.
        if (model_select(d2, fused, nullptr, desc->N) && fused.pred_us < (measure ? 1.3 : 1.0) * separate_us) {
            st = tdc_conv_plan_create_with_tail(&d2, desc->N, desc->has_bias, desc->relu, nullptr, &op->core_last);
            if (st != TDC_OK) { cleanup(); return st; }
            if (measure && (st = tkconv_measure_fusion(op.get())) != TDC_OK) { cleanup(); return st; }
        }
        // The first factor too, recomputed per workgroup on its window (streamed 3x3 kernel, stride 1).  Every
        // workgroup then pulls the whole first factor through its compute unit, so this only pays while that factor is
        // small: without measurement, up to 16 KiB of its weights and 64 input channels.
        if (op->core_last && (op->core_last->tile.alg == 4 || op->core_last->tile.alg == 6) && desc->K == 3 && desc->stride == 1 && desc->dilation == 1 &&
            !std::getenv("TDC_EXPERIMENT_NO_FUSED_HEAD") &&
            (measure ? (long long)desc->C * desc->R1 <= 32768 : ((long long)desc->C * desc->R1 <= 4096 && desc->C <= 64))) {
            // (the same tile; the head's output is read from LDS, so a tile that passes its input window through LDS
            //  becomes the plain streamed one)
            tdc_tile head_tile = op->core_last->tile;
            head_tile.alg = 4;
            st = tdc_conv_plan_create_with_tail(&d2, desc->N, desc->has_bias, desc->relu, &head_tile, &op->whole);
            if (st == TDC_OK) {
                const std::vector<float> zeros((size_t)desc->R1 * desc->C, 0.0f);
                st = tdc_conv_plan_set_head(op->whole, desc->C, zeros.data());
                if (st == TDC_ERR_UNSUPPORTED) {
                    tdc_conv_plan_destroy(op->whole);
                    op->whole = nullptr;
                    st = TDC_OK;
                }
            }
            if (st != TDC_OK) { cleanup(); return st; }
            if (op->whole && measure && (st = tkconv_measure_whole(op.get())) != TDC_OK) { cleanup(); return st; }
        }
    }
    *op_out = op.release();
    return TDC_OK;
}

int tdc_tkconv_set_weights(tdc_tkconv *op, const float *first, const float *core, const float *last,
                           const float *bias) {
    if (!op || !first || !core || !last) return fail(TDC_ERR_INVALID, "null argument");
    int st;
    if ((st = tdc_conv_plan_set_weights(op->first, first, nullptr)) != TDC_OK) return st;
    if ((st = tdc_conv_plan_set_weights(op->core, core, nullptr)) != TDC_OK) return st;
    if ((st = tdc_conv_plan_set_weights(op->last, last, bias)) != TDC_OK) return st;
    if (op->core_last) {
        if ((st = tdc_conv_plan_set_weights(op->core_last, core, nullptr)) != TDC_OK) return st;
        if ((st = tdc_conv_plan_set_tail_weights(op->core_last, last, bias)) != TDC_OK) return st;
    }
    if (op->whole) {
        if ((st = tdc_conv_plan_set_weights(op->whole, core, nullptr)) != TDC_OK) return st;
        if ((st = tdc_conv_plan_set_tail_weights(op->whole, last, bias)) != TDC_OK) return st;
        if ((st = tdc_conv_plan_set_head(op->whole, op->desc.C, first)) != TDC_OK) return st;
    }
    return TDC_OK;
}

static int tkconv_forward_unfused(tdc_tkconv *op, const float *d_in, int64_t in_batch_stride, const float *d_residual,
                                  int64_t residual_batch_stride, float *d_out, int64_t out_batch_stride, void *stream) {
    int st;
    if ((st = tdc_conv_forward_strided(op->first, d_in, in_batch_stride, nullptr, 0, op->d_f1, 0, stream)) != TDC_OK) return st;
    if ((st = tdc_conv_forward(op->core, op->d_f1, nullptr, op->d_f2, stream)) != TDC_OK) return st;
    return tdc_conv_forward_strided(op->last, op->d_f2, 0, d_residual, residual_batch_stride, d_out, out_batch_stride, stream);
}

int tdc_tkconv_num_kernels(const tdc_tkconv *op) { return op ? (op->whole ? 1 : op->core_last ? 2 : 3) : 0; }

int tdc_tkconv_forward(tdc_tkconv *op, const float *d_in, const float *d_residual, float *d_out, void *stream) {
    return tdc_tkconv_forward_strided(op, d_in, 0, d_residual, 0, d_out, 0, stream);
}

int tdc_tkconv_forward_strided(tdc_tkconv *op, const float *d_in, int64_t in_batch_stride, const float *d_residual,
                               int64_t residual_batch_stride, float *d_out, int64_t out_batch_stride, void *stream) {
    if (!op || !d_in || !d_out) return fail(TDC_ERR_INVALID, "null argument");
    if (!op->core_last)
        return tkconv_forward_unfused(op, d_in, in_batch_stride, d_residual, residual_batch_stride, d_out, out_batch_stride,
                                      stream);
    if (op->whole)
        return tdc_conv_forward_strided(op->whole, d_in, in_batch_stride, d_residual, residual_batch_stride, d_out,
                                        out_batch_stride, stream);
    int st;
    if ((st = tdc_conv_forward_strided(op->first, d_in, in_batch_stride, nullptr, 0, op->d_f1, 0, stream)) != TDC_OK) return st;
    return tdc_conv_forward_strided(op->core_last, op->d_f1, 0, d_residual, residual_batch_stride, d_out, out_batch_stride,
                                    stream);
}

int tdc_tkconv_forward_features(tdc_tkconv *op, const float *d_in, float *d_feat_first, float *d_feat_core,
                                float *d_out, void *stream) {
    if (!op || !d_in || !d_out) return fail(TDC_ERR_INVALID, "null argument");
    int st = tkconv_forward_unfused(op, d_in, 0, nullptr, 0, d_out, 0, stream);   // the core's output is wanted
    if (st != TDC_OK) return st;
    hipError_t e;
    if (d_feat_first) {
        e = hipMemcpyAsync(d_feat_first, op->d_f1, op->f1_floats * sizeof(float), hipMemcpyDeviceToDevice,
                           (hipStream_t)stream);
        if (e != hipSuccess) return hip_fail("hipMemcpyAsync(first feature)", e);
    }
    if (d_feat_core) {
        e = hipMemcpyAsync(d_feat_core, op->d_f2, op->f2_floats * sizeof(float), hipMemcpyDeviceToDevice,
                           (hipStream_t)stream);
        if (e != hipSuccess) return hip_fail("hipMemcpyAsync(core feature)", e);
    }
    return TDC_OK;
}

int tdc_tkconv_core_forward(tdc_tkconv *op, const float *d_in, float *d_out, void *stream) {
    if (!op) return fail(TDC_ERR_INVALID, "null argument");
    return tdc_conv_forward(op->core, d_in, nullptr, d_out, stream);
}

int tdc_tkconv_query(const tdc_tkconv *op, int which, tdc_tile_info *info_out) {
    if (!op || !info_out) return fail(TDC_ERR_INVALID, "null argument");
    const tdc_conv_plan *p = which == 0 ? op->first : which == 1 ? op->core : which == 2 ? op->last : nullptr;
    if (!p) return fail(TDC_ERR_INVALID, "which must be 0, 1 or 2");
    return tdc_conv_plan_query(p, info_out);
}

void tdc_tkconv_destroy(tdc_tkconv *op) {
    if (!op) return;
    tdc_conv_plan_destroy(op->first);
    tdc_conv_plan_destroy(op->core);
    tdc_conv_plan_destroy(op->last);
    tdc_conv_plan_destroy(op->core_last);
    tdc_conv_plan_destroy(op->whole);
    if (op->d_f1) (void)hipFree(op->d_f1);
    if (op->d_f2) (void)hipFree(op->d_f2);
    delete op;
}

}  // extern "C"
