// Launch geometry, weight packing and the closed-form gfx950 tile model.
//
// The reference chooses (TH, TW, TC) per layer either from a measured sweep
// (2080Ti-evaluation/TDC-LAYERS-ORACLE/gen_from_occupancy.py:51-66) or from an
// analytic score that still needs a table of measured CUDA occupancies
// (2080Ti-evaluation/TDC-LAYERS-MODELING/model.py:136-156,209-235;
// 2080Ti-evaluation/Gen-occupancy/template.cu:277-284).  This file is the
// self-contained counterpart for one MI355X: occupancy comes from the register
// and LDS footprint of the tile, latency from MFMA issue cycles per SIMD, the
// copy volume of the staged input window and weights, and wave quantisation over
// 256 compute units.  Host-only code: it runs without a GPU.
#include <algorithm>
#include <array>
#include <map>
#include <mutex>
#include <shared_mutex>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>

#include "tdc_internal.hpp"

namespace tdc {

const Machine &machine() {
    static const Machine m;
    return m;
}

static inline int ceil_div(int a, int b) { return (a + b - 1) / b; }
static inline int round_up(int a, int b) { return ceil_div(a, b) * b; }

bool check_desc(const tdc_conv_desc &d, std::string *why) {
    auto fail = [&](const char *m) {
        if (why) *why = m;
        return false;
    };
    if (d.batch < 1 || d.C < 1 || d.N < 1 || d.H < 1 || d.W < 1) return fail("batch, C, N, H, W must be >= 1");
    if (d.KH < 1 || d.KW < 1) return fail("KH, KW must be >= 1");
    if (d.stride < 1) return fail("stride must be >= 1");
    if (d.pad < 0) return fail("pad must be >= 0");
    if (d.dilation < 1) return fail("dilation must be >= 1");
    const long long eh = (long long)d.H + 2LL * d.pad - (long long)d.dilation * (d.KH - 1) - 1;
    const long long ew = (long long)d.W + 2LL * d.pad - (long long)d.dilation * (d.KW - 1) - 1;
    if (eh < 0 || ew < 0) return fail("filter (with dilation) larger than padded input");
    // One image is addressed through a 32-bit buffer descriptor (byte offsets below 2^31).
    if ((long long)d.C * d.H * d.W >= (1LL << 29) || (long long)d.N * d.H * d.W >= (1LL << 29))
        return fail("per-image tensor exceeds 2^29 elements");
    if ((long long)d.N * d.C * d.KH * d.KW >= (1LL << 28)) return fail("weight tensor exceeds 2^28 elements");
    return true;
}

// LDS bank conflicts of the B-operand read.  The 64 lanes of a wave read one word each: lane l holds pixel
// l % mf of its block and input channel l / mf of the K-step, i.e. word jy*stride*RS + jx*stride + (l/mf)*CS
// (+ the same tap offset for everybody).  The LDS has 64 four-byte banks; lanes that hit one bank with
// different words are served one after the other.  Returned: that serialisation factor (1 = conflict-free),
// averaged over the pixel blocks of a workgroup tile.
static double b_read_conflict_ways(int mf, int PT, int TW, int TH, int RS, int CS, int stride) {
    double sum = 0.0;
    int blocks = 0;
    for (int j0 = 0; j0 < PT; j0 += mf, ++blocks) {
        int words[64][8], cnt[64];
        for (int b = 0; b < 64; ++b) cnt[b] = 0;
        int ways = 1;
        for (int l = 0; l < 64; ++l) {
            const int j = j0 + l % mf;
            const int jy = std::min(j / TW, TH - 1), jx = j % TW;
            const int w = jy * stride * RS + jx * stride + (l / mf) * CS;
            const int b = w & 63;
            bool seen = false;
            for (int i = 0; i < cnt[b]; ++i) seen |= (words[b][i] == w);
            if (!seen && cnt[b] < 8) words[b][cnt[b]++] = w;
            ways = std::max(ways, cnt[b]);
        }
        sum += ways;
    }
    return blocks ? sum / blocks : 1.0;
}

// LDS channel stride: the smallest stride from the raw window size upwards (inflating small windows by at
// most a quarter, larger ones by at most 64 words) that gives the B-operand read the fewest bank conflicts.
// For tiles whose pixel blocks lie in one row this is the classic rule — stride = 16 (mod 32) for the four
// channel quarters of a 16x16x4 step, 32 (mod 64) for the halves of a 32x32x2 step; narrow tiles whose
// blocks wrap over several rows cannot be made conflict-free and get the best stride there is.
static int pad_channel_stride(int raw, int mf, int vw, int PT, int TW, int TH, int RS, int stride, double *ways_out) {
    // Thousands of candidate tiles share a handful of window shapes: remember the answers (per thread).
    static thread_local std::map<std::array<int, 8>, std::pair<int, double>> memo;
    const std::array<int, 8> key{raw, mf, vw, PT, TW, TH, RS, stride};
    auto hit = memo.find(key);
    if (hit == memo.end()) {
        const int first = round_up(raw, vw);
        const int budget = std::max(raw / 4, std::min(64, raw));
        int best = first;
        double best_ways = 1e9;
        for (int cs = first; cs - raw <= budget; cs += vw) {
            const double ways = b_read_conflict_ways(mf, PT, TW, TH, RS, cs, stride);
            if (ways < best_ways - 1e-9) {
                best_ways = ways;
                best = cs;
            }
        }
        if (memo.size() > 100000) memo.clear();
        hit = memo.emplace(key, std::make_pair(best, best_ways)).first;
    }
    *ways_out = hit->second.second;
    return hit->second.first;
}

bool make_geometry(const tdc_conv_desc &d, const tdc_tile &t, Geometry &g, std::string *why, int tail_N) {
    auto fail = [&](const std::string &m) {
        if (why) *why = m;
        return false;
    };
    if (!check_desc(d, why)) return false;
    if (t.mf != 32 && t.mf != 16) return fail("tile.mf must be 16 or 32");
    if (t.mb < 1 || t.mb > 2 || t.nb < 1 || (t.nb > 2 && !((t.alg == 4 || t.alg == 6) && t.nb == 4)))
        return fail("tile.mb / tile.nb must be 1 or 2 (tile.nb may be 4 for tile.alg = 4)");
    if (t.wm < 1 || t.wn < 1 || t.wk < 1) return fail("tile.wm / wn / wk must be >= 1");
    g = Geometry();
    // (256 registers per lane for the 2x2 block grid, 168 for the Winograd path)
    g.max_waves_kernel = (t.mb == 2 && t.nb == 2) ? 8 : t.alg == 1 ? 12 : 16;
    if (t.alg == 5) {
        // streamed Winograd: the launch bound follows the groups of four channels a wave keeps in registers
        const int groups = (t.wk >= 1 && t.cch % (4 * t.wk) == 0) ? t.cch / (4 * t.wk) : 0;
        g.max_waves_kernel = wino_stream_max_waves(groups);
        if (!g.max_waves_kernel) return fail("tile.alg = 5 needs cch = 4 * wk * {1, 2, 3, 4}");
    }
    if (t.wl < 0 || t.wl > 8) return fail("tile.wl must be in [0, 8]");
    if ((long long)t.wm * t.wn * t.wk + t.wl > g.max_waves_kernel) return fail("too many waves per workgroup for this tile");
    g.waves = t.wm * t.wn * t.wk + t.wl;
    g.threads = g.waves * 64;
    const bool flat = (d.KH == 1 && d.KW == 1 && d.stride == 1 && d.pad == 0);
    g.He = flat ? 1 : d.H;
    g.We = flat ? d.H * d.W : d.W;
    // (the copy-offset arithmetic of the kernel uses 24-bit multiplies)
    if ((long long)(d.C + 1) * g.He >= (1LL << 24) || g.We >= (1 << 24)) return fail("image too large");
    g.Ho = (g.He + 2 * d.pad - d.dilation * (d.KH - 1) - 1) / d.stride + 1;
    g.Wo = (g.We + 2 * d.pad - d.dilation * (d.KW - 1) - 1) / d.stride + 1;
    g.P = g.Ho * g.Wo;
    g.kc = (t.mf == 32) ? 2 : 4;
    g.taps = d.KH * d.KW;
    g.ktaps = g.taps;
    g.MT = t.mf * t.mb * t.wm;
    if (t.alg < 0 || t.alg > 6) return fail("tile.alg must be in [0, 6]");
    if (t.alg == 5) {
        // Winograd F(2x2,3x3) streamed from global memory: 16*wm channels of one tile row block (2 rows x 28 columns) per
        // workgroup, the input channels split over wk waves in groups of four, everything in one pass
        if (d.KH != 3 || d.KW != 3 || d.stride != 1 || d.dilation != 1 || d.pad != 1)
            return fail("tile.alg = 5 needs a 3x3 / stride 1 / pad 1 / dilation 1 convolution");
        if (d.W % 2 != 0) return fail("tile.alg = 5 needs an even image width");
        if (t.mf != 16 || t.mb != 1 || t.nb != 1 || t.wn != 1) return fail("tile.alg = 5 needs mf = 16, mb = nb = wn = 1");
        if (t.wl != 0 || t.ks != 1) return fail("tile.alg = 5 has no loader waves and no split across workgroups");
        if (tail_N > 0) return fail("tile.alg = 5 cannot carry a fused tail");
        if (t.tw != 28) return fail("tile.alg = 5 needs tw = 28");
        if (t.cch < d.C || t.cch - d.C >= t.cch / t.wk) return fail("tile.alg = 5 takes all input channels in one pass without an idle wave");
        if ((long long)t.cch * d.H * d.W * 4 >= (1LL << 31)) return fail("image too large for tile.alg = 5");
    }
    if (t.alg == 6 && (d.pad > 1 || d.stride > 2)) return fail("tile.alg = 6 needs pad <= 1 and stride <= 2");
    if (t.alg == 6 && t.nb == 4 && t.cch / std::max(t.wk, 1) > 8) return fail("tile.alg = 6 with nb = 4 takes at most two groups per wave");
    if (t.alg == 4 || t.alg == 6) {
        // 3x3 convolution streamed from global memory: 16 channels x 16 pixels per workgroup, the input channels
        // split over wk waves in groups of four, everything in one pass (alg 6: the tile's input window through LDS)
        if (d.KH != 3 || d.KW != 3 || d.dilation != 1) return fail("tile.alg = 4 needs a 3x3 / dilation 1 convolution");
        if (t.mf != 16 || t.mb != 1 || t.wn != 1) return fail("tile.alg = 4 needs mf = 16, mb = 1, wn = 1");
        if (t.nb != 1) {
            // nb pixel blocks per wave (the weights a wave holds feed nb MFMAs each): rows of 14 pixels, stride 1
            if (d.stride != 1 || t.tw != 14) return fail("tile.alg = 4 with nb > 1 needs stride 1 and tw = 14");
            if (t.nb > ceil_div(g.Wo, 14)) return fail("tile.alg = 4: more pixel blocks per wave than an image row has 14-pixel tiles");
            if (tail_N > 0 || t.ks != 1) return fail("tile.alg = 4 with nb > 1 has no fused tail and no split across workgroups");
        }
        if (t.wm * t.wk > 16) return fail("tile.alg = 4: at most 16 waves (wm channel blocks x wk channel slices)");
        if (t.wl != 0) return fail("tile.alg = 4 has no loader waves");
        const int groups = (t.cch % (4 * t.wk) == 0) ? t.cch / (4 * t.wk) : 0;
        if (groups != 1 && groups != 2 && groups != 4) return fail("tile.alg = 4 needs cch = 4 * wk * {1, 2, 4}");
        if (ceil_div(d.C, t.cch) != t.ks) return fail("tile.alg = 4 takes its input channels in one pass: ks slices of cch channels must cover them exactly");
        if ((long long)t.cch * d.H * d.W * 4 >= (1LL << 31)) return fail("image too large for tile.alg = 4");
    }
    g.wino = t.alg == 1;
    if (t.alg == 3) {
        // 1x1 convolution streamed from global memory: a 16x16 output block per workgroup, the input channels split
        // over wk waves in runs of 16, everything in one pass
        if (d.KH != 1 || d.KW != 1 || d.pad != 0) return fail("tile.alg = 3 needs a 1x1 / pad 0 convolution");
        if (!flat && t.ks != 1) return fail("tile.alg = 3 with stride > 1 has no split across workgroups");
        if (t.mf != 16 || t.mb != 1 || t.nb != 1 || t.wm != 1 || t.wn != 1) return fail("tile.alg = 3 needs mf = 16 and one block per workgroup");
        if (t.wl != 0) return fail("tile.alg = 3 has no loader waves");
        if (tail_N > 0) return fail("tile.alg = 3 cannot carry a fused tail");
        const int runs = (t.cch % (16 * t.wk) == 0) ? t.cch / (16 * t.wk) : 0;
        if (runs != 1 && runs != 2 && runs != 4 && runs != 8) return fail("tile.alg = 3 needs cch = 16 * wk * {1, 2, 4, 8}");
        if (runs == 8 && t.wk > 8) return fail("tile.alg = 3 with eight runs per wave is built for at most 8 waves");
        if (ceil_div(d.C, t.cch) != t.ks) return fail("tile.alg = 3 takes its input channels in one pass: ks slices of cch channels must cover them exactly");
        if (t.tw != std::min(16, g.P)) return fail("tile.alg = 3 needs tw = min(16, pixels)");
        if ((long long)t.cch * g.We * 4 >= (1LL << 31)) return fail("image too large for tile.alg = 3");
    }
    if (t.alg == 2) {
        // direct 3x3 convolution with the weights read from global memory into registers, a pair of channel groups at a time
        if (d.KH != 3 || d.KW != 3 || d.dilation != 1) return fail("tile.alg = 2 needs a 3x3 / dilation 1 convolution");
        if (t.mb != 1 || t.nb != 1) return fail("tile.alg = 2 needs mb = nb = 1");
        if (tail_N > 0) return fail("tile.alg = 2 cannot carry a fused tail");
        if (t.cch % (2 * g.kc * t.wk) != 0) return fail("tile.alg = 2 needs an even number of channel groups per wave and pass");
    }
    if (t.alg == 1) {
        // Winograd F(2x2,3x3): a pixel lane holds one 2x2 output tile; the workgroup tile is THt x TWt such tiles.
        if (d.KH != 3 || d.KW != 3 || d.stride != 1 || d.dilation != 1) return fail("tile.alg needs a 3x3 / stride 1 / dilation 1 convolution");
        if (t.mf != 16 || t.mb != 1 || t.nb != 1) return fail("tile.alg needs mf = 16, mb = nb = 1");
        if (tail_N > 0) return fail("tile.alg cannot carry a fused tail");
        const int lanes = 16 * t.wn;
        const int Wt = ceil_div(g.Wo, 2), Ht = ceil_div(g.Ho, 2);
        if (t.tw < 1 || t.tw > lanes || t.tw > Wt) return fail("tile.tw must be in [1, min(ceil(Wo/2), tile lanes)]");
        g.ktaps = 16;
        g.TWt = t.tw;
        g.THt = std::min(lanes / t.tw, Ht);
        g.TW = 2 * g.TWt;
        g.TH = 2 * g.THt;
        g.PT = 4 * lanes;   // pixels the workgroup's lanes stand for
    } else if (t.alg == 5) {
        g.ktaps = 16;
        g.TW = 28;
        g.TH = 2;
        g.PT = 64;          // two rows of 32 columns in the parked tile (28 of them real)
    } else {
        g.PT = t.mf * t.nb * t.wn;
        // (the streamed 1x1 kernel walks the output in runs of 16 consecutive pixels, whatever the image's rows are)
        const bool runs = t.alg == 3 && !flat;
        if (t.tw < 1 || t.tw > g.PT || (!runs && t.tw > g.Wo)) return fail("tile.tw must be in [1, min(Wo, pixel lanes)]");
        g.TW = t.tw;
        g.TH = runs ? 1 : std::min(g.PT / t.tw, g.Ho);
        if (t.alg == 4 || t.alg == 6) g.TH = std::min(16 / t.tw, g.Ho);   // (a block is 16 pixel lanes, whatever nb is)
    }
    g.ntx = ceil_div(g.Wo, g.TW);
    if ((t.alg == 4 || t.alg == 6) && t.nb > 1) g.ntx = ceil_div(g.ntx, t.nb);   // a workgroup takes nb neighbouring tiles of a row
    g.nty = ceil_div(g.Ho, g.TH);
    if (t.alg == 3 && !flat) {
        g.ntx = ceil_div(g.P, 16);
        g.nty = 1;
    }
    // (the kernel divides the tile index by ntx with a 32-bit multiply-high)
    if ((long long)g.ntx * g.nty > 65535 * 16) return fail("grid too large");
    if ((long long)g.ntx * g.nty * g.ntx >= (1LL << 32)) return fail("grid too large");
    g.grid_x = g.ntx * g.nty;
    g.grid_y = ceil_div(d.N, g.MT);
    if (t.ks < 1 || t.ks > 64) return fail("tile.ks must be in [1, 64]");
    g.ks = t.ks;
    if ((long long)d.batch * t.ks > 65535) return fail("grid too large");
    g.grid_z = d.batch * t.ks;
    if (g.grid_y > 65535) return fail("grid too large");
    const int granule = g.kc * t.wk;
    if (t.cch < granule || t.cch % granule != 0) return fail("tile.cch must be a positive multiple of kc*wk");
    if (t.alg < 3 && t.cch > round_up(d.C, granule)) return fail("tile.cch exceeds the (padded) channel count");
    g.cpw = t.cch / t.wk;
    g.nchunks = ceil_div(d.C, t.cch);
    g.c_pad = g.nchunks * t.cch;
    g.cps = ceil_div(g.nchunks, t.ks);
    if ((t.ks - 1) * g.cps >= g.nchunks) return fail("tile.ks leaves a workgroup without input channels");
    g.nrows = (g.TH - 1) * d.stride + (d.KH - 1) * d.dilation + 1;
    g.ncols = (g.TW - 1) * d.stride + (d.KW - 1) * d.dilation + 1;
    // LDS rows are filled with 16-byte elements when image rows are a multiple of
    // 4 floats: the window then starts at the 4-float boundary at or left of its
    // first column, which can cost up to 3 extra columns.
    g.VW = (g.We % 4 == 0) ? 4 : 1;
    if (g.VW == 4) {
        int shift = 0;
        for (int tx = 0; tx < std::min(g.ntx, 4); ++tx) {
            const int ix0 = tx * g.TW * d.stride - d.pad;
            shift = std::max(shift, ((ix0 % 4) + 4) % 4);
        }
        g.RS = round_up(g.ncols + shift, 4);
    } else {
        g.RS = g.ncols;
    }
    // (Winograd: lane l reads the 4x4 input patch of tile l, two floats to the right and two rows down per tile)
    g.CS = t.alg == 1 ? pad_channel_stride(g.nrows * g.RS, 16, g.VW, 16 * t.wn, g.TWt, g.THt, g.RS, 2, &g.b_ways)
                  : pad_channel_stride(g.nrows * g.RS, t.mf, g.VW, g.PT, g.TW, g.TH, g.RS, d.stride, &g.b_ways);
    // Copies are issued in whole blocks of 64 elements (1 KiB with 16-byte elements): both parts of
    // a stage are rounded up to that, the slack receiving zeros.
    g.in_stage_floats = round_up(t.cch * g.CS, 256);
    g.wslab_floats = (t.wm * t.mb) * (t.cch / g.kc) * g.ktaps * 64;
    g.aff_floats = (d.KH == 1 && d.KW == 1 && d.pad == 0) ? round_up(2 * t.cch, 256) : 0;
    // (the Winograd path reads its weights straight from global memory into registers: the LDS holds input only)
    g.stage_floats = g.in_stage_floats + (t.alg ? 0 : round_up(g.wslab_floats, 256)) + g.aff_floats;   // (wino = 2 likewise)
    if (t.alg >= 3) g.in_stage_floats = g.aff_floats = g.stage_floats = 0;   // nothing is staged
    g.nstage = g.cps > 1 ? 2 : 1;
    const long long stage_bytes = (long long)g.nstage * g.stage_floats * 4;
    // (the Winograd path always parks its output tiles in LDS, also without a split over waves)
    // (... and so does the streamed 3x3 kernel with several pixel blocks per wave: all its threads share the final store)
    const long long red_bytes = (t.wk > 1 || t.alg == 1 || t.alg == 5 || ((t.alg == 4 || t.alg == 6) && t.nb > 1)) ? (long long)t.wk * g.MT * g.PT * 4 : 0;
    long long lds = std::max(stage_bytes, red_bytes);
    if (tail_N > 0) {
        // A fused 1x1 tail needs every output channel of the convolution in one workgroup; its tile is parked
        // in LDS behind the split-K partials with a row stride that keeps the four channel quarters of a
        // K-step in different banks.
        if (tail_N > 4096) return fail("fused tail too wide");
        if (g.grid_y != 1) return fail("a fused tail needs all output channels in one workgroup tile");
        if (t.ks != 1) return fail("a fused tail cannot be combined with a split across workgroups");
        g.tail_N = tail_N;
        g.tail_ng = ceil_div(d.N, 4);
        g.tail_ld = (g.PT % 32 == 0) ? g.PT + 16 : g.PT;
        g.tail_f_off = t.wk > 1 ? t.wk * g.MT * g.PT : 0;
        lds = std::max(lds, ((long long)g.tail_f_off + (long long)g.MT * g.tail_ld) * 4);
    }
    if (t.alg >= 3 && t.ks > 1) lds = std::max<long long>(lds, 16);   // the drawn ticket is passed through LDS
    if (t.alg == 6) {
        // The input window of a tile: (TH-1)*stride+3 rows; columns from the multiple of four at or left of the tile's first
        // input column (up to three more than the (TW-1)*stride+3 the taps touch), in segments of four.  One slot per lane
        // of a channel quarter and request.
        g.win_rows = (g.TH - 1) * d.stride + 3;
        g.win_L = ceil_div((g.TW * t.nb - 1) * d.stride + 3 + 3, 4);   // (nb > 1: the blocks lie side by side in one window)
        g.win_nreq = ceil_div(g.win_rows * g.win_L, 16);
        if (g.win_nreq > (t.nb == 4 ? 3 : 2)) return fail("tile.alg = 6: the input window of this tile needs too many requests per group");
        if (d.W < 4) return fail("tile.alg = 6 needs an image at least four columns wide");
        g.win_ns = g.win_rows * g.win_L * 4;
        while (g.win_ns % 32 != 16) g.win_ns += 4;
        g.win_off = (int)((lds + 15) / 16 * 4);
        lds = (long long)g.win_off * 4 + (long long)g.waves * (t.cch / t.wk) * g.win_ns * 4;
    }
    if (lds > machine().lds_bytes_per_cu) return fail("tile needs more than 160 KiB of LDS");
    g.lds_bytes = (int)lds;
    if (const char *e = std::getenv("TDC_EXPERIMENT_MIN_LDS")) g.lds_bytes = std::max(g.lds_bytes, std::atoi(e));
    if ((long long)g.grid_y * g.nchunks * g.wslab_floats * 4 >= (1LL << 31)) return fail("packed weights exceed 2 GiB");
    // (the kernel decodes a one-dimensional launch index with 32-bit multiply-high divisions)
    const long long n_wg = (long long)g.grid_x * g.grid_y * g.grid_z;
    if (n_wg + 8 >= (1LL << 28) || n_wg * std::max(g.grid_x, g.grid_y) >= (1LL << 32)) return fail("grid too large");
    // Bytes the eight die-private L2s fill in total, for the two logical workgroup orders: with the channel
    // tiles of a pixel tile adjacent a die reads its share of the input and every weight; with the pixel tiles
    // of a channel tile adjacent it reads every input pixel of min(channel tiles, 8) ... and its own weights.
    const double in_bytes = 4.0 * d.C * d.H * d.W, w_bytes = 4.0 * d.N * d.C * g.taps;
    const double dies = (double)std::min<long long>(8, n_wg);
    const double pixel_major = in_bytes + dies * w_bytes;
    const double channel_major = std::min<double>(g.grid_y, dies) * in_bytes + std::max(1.0, dies / g.grid_y) * w_bytes;
    g.channel_major = channel_major < pixel_major ? 1 : 0;
    if (const char *e = std::getenv("TDC_EXPERIMENT_XCD_ORDER")) g.channel_major = std::atoi(e) != 0;
    return true;
}

size_t packed_weight_floats(const Geometry &g) {
    return (size_t)g.grid_y * (size_t)g.nchunks * (size_t)g.wslab_floats;
}

void pack_weights(const tdc_conv_desc &d, const tdc_tile &t, const Geometry &g, const float *w, float *packed) {
    const int mbw = t.wm * t.mb;
    const int ncg = t.cch / g.kc;
    const int taps = g.taps;
    float *dst = packed;
    if (t.alg == 2 || t.alg == 4 || t.alg == 6) {
        // per (channel tile, pass, M block, channel group): [taps 0-3][lane][4] [taps 4-7][lane][4] [tap 8][lane]
        for (int by = 0; by < g.grid_y; ++by)
            for (int chunk = 0; chunk < g.nchunks; ++chunk)
                for (int mbl = 0; mbl < mbw; ++mbl)
                    for (int cg = 0; cg < ncg; ++cg, dst += 9 * 64)
                        for (int tap = 0; tap < 9; ++tap)
                            for (int l = 0; l < 64; ++l) {
                                const int n = by * g.MT + mbl * t.mf + l % t.mf;
                                const int c = chunk * t.cch + cg * g.kc + l / t.mf;
                                const float v = (n < d.N && c < d.C) ? w[((size_t)n * d.C + c) * 9 + tap] : 0.0f;
                                dst[tap < 8 ? (tap / 4) * 256 + l * 4 + tap % 4 : 512 + l] = v;
                            }
        return;
    }
    if (t.alg == 3) {
        // per (channel block, run of 16 input channels): [lane][s], lane (n = l % 16, k = l / 16) holding
        // w[block*16 + n][16*run + 4*k + s]; the runs of all slices of a split across workgroups follow each other
        const int runs = g.nchunks * (t.cch / 16);
        for (int by = 0; by < g.grid_y; ++by)
            for (int r = 0; r < runs; ++r)
                for (int l = 0; l < 64; ++l)
                    for (int e = 0; e < 4; ++e) {
                        const int n = by * 16 + l % 16, c = 16 * r + 4 * (l / 16) + e;
                        *dst++ = (n < d.N && c < d.C) ? w[(size_t)n * d.C + c] : 0.0f;
                    }
        return;
    }
    if (g.wino || t.alg == 5) {
        // Winograd F(2x2,3x3): U = G g G^T per (output channel, input channel), G = [1 0 0; .5 .5 .5; .5 -.5 .5; 0 0 1].
        // Per (channel tile, pass, M block, channel group): [q = 0..3][64 lanes][e = 0..3] holding U[q][e] of
        // (n = l % 16, c = l / 16), so that one 128-bit LDS read fetches the A operands of four of the 16 MFMAs.
        static const double G[4][3] = {{1, 0, 0}, {0.5, 0.5, 0.5}, {0.5, -0.5, 0.5}, {0, 0, 1}};
        for (int by = 0; by < g.grid_y; ++by)
            for (int chunk = 0; chunk < g.nchunks; ++chunk)
                for (int mbl = 0; mbl < mbw; ++mbl)
                    for (int cg = 0; cg < ncg; ++cg)
                        for (int q = 0; q < 4; ++q)
                            for (int l = 0; l < 64; ++l) {
                                const int n = by * g.MT + mbl * 16 + l % 16;
                                const int c = chunk * t.cch + cg * 4 + l / 16;
                                for (int e = 0; e < 4; ++e) {
                                    double u = 0.0;
                                    if (n < d.N && c < d.C) {
                                        const float *gk = w + ((size_t)n * d.C + c) * 9;
                                        for (int r = 0; r < 3; ++r)
                                            for (int s = 0; s < 3; ++s) u += G[q][r] * (double)gk[r * 3 + s] * G[e][s];
                                    }
                                    *dst++ = (float)u;
                                }
                            }
        return;
    }
    for (int by = 0; by < g.grid_y; ++by)
        for (int chunk = 0; chunk < g.nchunks; ++chunk)
            for (int mbl = 0; mbl < mbw; ++mbl)
                for (int cg = 0; cg < ncg; ++cg)
                    for (int tap = 0; tap < taps; ++tap)
                        for (int l = 0; l < 64; ++l) {
                            const int n = by * g.MT + mbl * t.mf + l % t.mf;
                            const int c = chunk * t.cch + cg * g.kc + l / t.mf;
                            *dst++ = (n < d.N && c < d.C) ? w[((size_t)n * d.C + c) * taps + tap] : 0.0f;
                        }
}

// ---------------------------------------------------------------------------
// Analytic model
// ---------------------------------------------------------------------------
namespace {

// Calibration constants of the latency model.  The defaults were fitted to a measured sweep of every
// launchable tile of the 28 benchmark layers on one MI355X (python -m tdc_amd.fit_model); they can be
// replaced at run time through tdc_model_set_constants, e.g. for another CDNA part.  They play the role
// of num_sm / num_threads / the (a, b, c) weights / the keep-ratio in the reference's model
// (2080Ti-evaluation/TDC-LAYERS-MODELING/model.py:265-266,278).
struct ModelConst {
    double launch_us = 1.474;           // device time of an empty kernel in a back-to-back stream
    double setup_clk = 1479;          // kernel arguments and index arithmetic before the first copy is issued
    double copy_latency_clk = 798.12;   // first byte of a global->LDS copy (L2 / memory-side cache)
    double copy_bytes_per_clk = 42.0036;   // sustained global->LDS rate of one CU
    double l2_bytes_per_clk = 12019.7;   // whole-chip L2->CU rate when every CU copies at once
    double lds_bytes_per_clk = 41.148;   // LDS traffic of the split-K reduction
    double sync_clk = 275.2;            // one workgroup barrier
    double store_bytes_per_clk = 2.827;  // per CU, short runs per channel
    double kstep_issue_clk = 4.36679;      // vector-ALU / LDS-issue cycles per operand read, not hidden under MFMAs
    double pass_overhead_clk = 371.876;   // per wave and pass: copy issue, pointer set-up, pipeline fill
    double wave_setup_clk = 778.32;      // prologue cycles added per extra wave sharing a SIMD
    double ksplit_clk = 3381.18;         // split across workgroups: write-through, ticket round trip, read-back
    double copy_issue_clk = 100.5;      // a wave is held this long by every global->LDS copy instruction it issues
    double lds_read_clk = 1.44;        // LDS busy cycles per conflict-free operand read of one wave
    double wino_kstep_clk = 16.788;      // Winograd: cycles per MFMA that the input transform adds on top of the operand reads
    double gw_latency_clk = 1040.3;       // alg 2: the first weights come from L2 into registers after the input copy is under way
    double stream_setup_clk = 459;      // alg 3: index arithmetic before the requests go out (no copy tables, no stages)
    double stream_latency_clk = 774;    // alg 3: round trip of the first request, global memory -> registers
};
ModelConst MC;
std::shared_mutex MC_mutex;   // readers: every model evaluation; writer: tdc_model_set_constants
constexpr int kNumModelConst = 18;

double *mc_field(int i) {
    switch (i) {
        case 0: return &MC.launch_us;
        case 1: return &MC.setup_clk;
        case 2: return &MC.copy_latency_clk;
        case 3: return &MC.copy_bytes_per_clk;
        case 4: return &MC.l2_bytes_per_clk;
        case 5: return &MC.lds_bytes_per_clk;
        case 6: return &MC.sync_clk;
        case 7: return &MC.store_bytes_per_clk;
        case 8: return &MC.kstep_issue_clk;
        case 9: return &MC.pass_overhead_clk;
        case 10: return &MC.wave_setup_clk;
        case 11: return &MC.ksplit_clk;
        case 12: return &MC.copy_issue_clk;
        case 13: return &MC.lds_read_clk;
        case 14: return &MC.wino_kstep_clk;
        case 15: return &MC.gw_latency_clk;
        case 16: return &MC.stream_setup_clk;
        case 17: return &MC.stream_latency_clk;
        default: return nullptr;
    }
}

}  // namespace

struct CompiledKernel { const char *name; int regs, sgprs, waves; };
// hipcc's resource report for the convolution kernels of this build (written by the Makefile from the compile of
// conv_staged.hip and conv_stream.hip): name, VGPRs + AGPRs per lane, scalar registers, waves per SIMD.
static const CompiledKernel compiled_kernels[] = {
#include "kernel_registers.inc"
};

static const CompiledKernel *compiled_kernel(const KernelId &k) {
    static const std::map<std::string, const CompiledKernel *> by_name = [] {
        std::map<std::string, const CompiledKernel *> m;
        for (const CompiledKernel &c : compiled_kernels) m[c.name] = &c;
        return m;
    }();
    const auto it = by_name.find(kernel_name(k));
    return it == by_name.end() ? nullptr : it->second;
}

// Waves of this kernel that fit one SIMD, as the compiler works it out from the registers of the compiled kernel:
// 512 vector registers per lane shared by a SIMD's waves (handed out in blocks of 8), at most 8 waves, and 800 scalar
// registers in blocks of 16 — the staged kernel needs 106 (112 allocated), which leaves room for 7 waves, not 8, so
// a 1024-thread workgroup of it is alone on its compute unit however few vector registers it uses (the HIP runtime's
// occupancy query says the same).
int kernel_waves_per_simd(const KernelId &k) {
    const CompiledKernel *c = compiled_kernel(k);
    if (!c) return 0;
    const Machine &m = machine();
    const int by_vgpr = m.vgprs_per_simd_lane / ((c->regs + 7) / 8 * 8);
    const int by_sgpr = 800 / ((c->sgprs + 15) / 16 * 16);
    return std::min(std::min(m.max_waves_per_simd, by_vgpr), std::min(by_sgpr, c->waves));
}

KernelId kernel_id_with_head(const tdc_tile &t) {
    KernelId k;
    if (t.alg != 4 || t.ks != 1 || t.wk < 1 || t.cch % (4 * t.wk) != 0) return k;
    const int cg = t.cch / (4 * t.wk);
    if (cg != 1 && cg != 2 && cg != 4) return k;
    k.family = KernelId::STREAM_3x3;
    k.p[0] = cg; k.p[1] = 0; k.p[2] = 3; k.p[3] = 1;
    return k;
}

int wino_stream_max_waves(int groups) { return (groups >= 1 && groups <= 4) ? 16 : 0; }

KernelId kernel_id_for(const tdc_tile &t, int KH, int KW, int dilation, int stride, bool extras) {
    KernelId k;
    if (t.alg == 5) {
        if (extras || KH != 3 || KW != 3 || dilation != 1 || stride != 1 || t.mf != 16 || t.mb != 1 || t.nb != 1 || t.wn != 1 ||
            t.wm < 1 || t.wk < 1 || t.ks != 1 || t.cch % (4 * t.wk) != 0)
            return k;
        const int cg = t.cch / (4 * t.wk);
        const int maxw = wino_stream_max_waves(cg);
        if (!maxw || t.wm * t.wk > maxw) return k;
        k.family = KernelId::STREAM_WINO;
        k.p[0] = cg; k.p[1] = maxw;
        return k;
    }
    if (t.alg == 4 || t.alg == 6) {
        // (`extras` can only mean a fused tail here, which the one kernel carries)
        if (KH != 3 || KW != 3 || dilation != 1 || t.mf != 16 || t.mb != 1 || t.wm < 1 || t.wn != 1 || t.wk < 1 ||
            t.wm * t.wk > 16 || t.cch % (4 * t.wk) != 0)
            return k;
        const int cg = t.cch / (4 * t.wk);
        if ((cg != 1 && cg != 2 && cg != 4) || (extras && t.ks > 1)) return k;
        const bool row = stride == 1 && t.tw == 14;   // one row of 14 pixels: the taps of a filter row are lane shifts
        if (t.nb != 1) {
            // several pixel blocks per wave: row tiles, no extras, no split across workgroups
            if ((t.nb != 2 && t.nb != 4) || !row || extras || t.ks > 1) return k;
            if (t.alg == 6 && t.nb == 4 && cg == 4) return k;
        }
        k.family = KernelId::STREAM_3x3;
        k.p[0] = cg;
        k.p[1] = t.alg == 6 ? 2 : row;
        k.p[2] = extras ? 2 : t.ks > 1 ? 1 : 0;
        k.p[3] = t.nb;
        return k;
    }
    if (t.alg == 3) {
        // (`extras` here can only mean the input affine: the host refuses a fused tail for this path)
        if (KH != 1 || KW != 1 || t.mf != 16 || t.mb != 1 || t.nb != 1 || t.wm != 1 || t.wn != 1 || t.wk < 1 ||
            t.cch % (16 * t.wk) != 0)
            return k;
        const int nq = t.cch / (16 * t.wk);
        if ((nq != 1 && nq != 2 && nq != 4 && nq != 8) || t.wk > (nq == 8 ? 8 : 16) || (stride > 1 && t.ks > 1)) return k;
        k.family = KernelId::STREAM_1x1;
        k.p[0] = nq; k.p[1] = extras; k.p[2] = stride > 1 ? 2 : t.ks > 1 ? 1 : 0;
        return k;
    }
    if (t.mf != 16 && t.mf != 32) return k;
    if (t.mb < 1 || t.mb > 2 || t.nb < 1 || t.nb > 2) return k;
    int taps;
    if (t.alg == 1) {
        if (extras || KH != 3 || KW != 3 || dilation != 1 || t.mf != 16 || t.mb != 1 || t.nb != 1) return k;
        taps = TAPS_WINO;
    } else if (t.alg == 2) {
        if (extras || KH != 3 || KW != 3 || dilation != 1 || t.mb != 1 || t.nb != 1) return k;
        taps = TAPS_3x3G;
    } else if (t.alg == 0) {
        taps = (KH == 3 && KW == 3 && dilation == 1) ? TAPS_3x3 : (KH == 1 && KW == 1) ? TAPS_1x1
             : (KH == 7 && KW == 7 && dilation == 1 && !extras) ? TAPS_7x7   // (the network stems; built without the extras)
                                                                : TAPS_GENERIC;
    } else {
        return k;
    }
    k.family = KernelId::STAGED;
    k.p[0] = t.mf; k.p[1] = t.mb; k.p[2] = t.nb; k.p[3] = taps;
    k.p[4] = taps == TAPS_WINO ? 12 : (t.mb == 2 && t.nb == 2) ? 8 : 16;   // launch bound in waves
    k.p[5] = extras;
    return k;
}

std::string kernel_name(const KernelId &k) {
    char buf[96];
    const char *tf[2] = {"false", "true"};
    switch (k.family) {
        case KernelId::STAGED:
            std::snprintf(buf, sizeof buf, "tdc_conv_mfma_kernel<%d, %d, %d, %d, %d, %s>", k.p[0], k.p[1], k.p[2], k.p[3], k.p[4], tf[k.p[5] != 0]);
            break;
        case KernelId::STREAM_1x1:
            std::snprintf(buf, sizeof buf, "tdc_conv1x1_stream_kernel<%d, %s, %d>", k.p[0], tf[k.p[1] != 0], k.p[2]);
            break;
        case KernelId::STREAM_3x3:
            if (k.p[3] > 1) std::snprintf(buf, sizeof buf, "tdc_conv3x3_stream_rownb_kernel<%d, %d, %s>", k.p[0], k.p[3], tf[k.p[1] == 2]);
            else std::snprintf(buf, sizeof buf, "tdc_conv3x3_stream_kernel<%d, %d, %d>", k.p[0], k.p[1], k.p[2]);
            break;
        case KernelId::STREAM_WINO:
            std::snprintf(buf, sizeof buf, "tdc_wino3x3_stream_kernel<%d, %d>", k.p[0], k.p[1]);
            break;
        default: return "";
    }
    return buf;
}

// Registers per lane of the compiled instantiation (hipcc's kernel-resource-usage report: VGPRs + AGPRs), rounded up
// to the allocation granule of 8; 0 for a kernel the library does not hold.  The reference measures occupancy per
// candidate by compiling and probing each (2080Ti-evaluation/Gen-occupancy/template.cu:277-284); here the candidates
// share about a hundred instantiations, whose report the build compiles into this file.
int kernel_vgprs(const KernelId &k) {
    const CompiledKernel *c = compiled_kernel(k);
    return c ? (c->regs + 7) / 8 * 8 : 0;
}

bool model_evaluate(const tdc_conv_desc &d, const tdc_tile &t, tdc_tile_info &info, std::string *why, int tail_N) {
    Geometry g;
    if (!make_geometry(d, t, g, why, tail_N)) return false;
    const Machine &m = machine();
    std::shared_lock<std::shared_mutex> constants_lock(MC_mutex);
    std::memset(&info, 0, sizeof(info));
    info.tile = t;
    info.grid_x = g.grid_x;
    info.grid_y = g.grid_y;
    info.grid_z = g.grid_z;
    info.block_threads = g.threads;
    info.lds_bytes = g.lds_bytes;
    info.nchunks = g.nchunks;
    info.th = g.TH;
    // (a fused tail needs the instantiation with the extras; an input affine, which the model does not know of, too)
    const KernelId kid = kernel_id_for(t, d.KH, d.KW, d.dilation, d.stride, tail_N > 0);
    info.vgpr_estimate = kernel_vgprs(kid);
    if (info.vgpr_estimate <= 0) {
        if (why) *why = "no kernel instantiated for this tile";
        return false;
    }

    // --- occupancy (replaces cudaOccupancyMaxActiveBlocksPerMultiprocessor) ---
    const int waves_simd_vgpr = kernel_waves_per_simd(kid);   // registers per lane, and scalar registers per wave
    const int wg_waves_per_simd = ceil_div(g.waves, m.simds_per_cu);
    const int wg_by_vgpr = waves_simd_vgpr / wg_waves_per_simd;
    const int wg_by_lds = m.lds_bytes_per_cu / std::max(g.lds_bytes, 1);
    // (the staged kernels are never resident more than eight times per CU; the streamed one has no stage to hold)
    int wg_per_cu = std::min(std::min(wg_by_vgpr, wg_by_lds), t.alg >= 3 ? 32 : 8);
    if (wg_per_cu < 1) {
        if (why) *why = "tile does not fit one compute unit";
        return false;
    }
    info.wg_per_cu = wg_per_cu;
    info.waves_per_simd = wg_per_cu * wg_waves_per_simd;

    // --- algorithmic work and roofline ---------------------------------------
    const double P = (double)g.P;
    info.flops = 2.0 * P * d.C * d.N * g.taps * d.batch;
    info.bytes = 4.0 * ((double)d.batch * ((double)d.C * d.H * d.W + (double)d.N * P) +
                        (double)g.taps * d.C * d.N);
    if (tail_N > 0) {   // the intermediate never leaves the chip
        info.flops += 2.0 * P * d.N * tail_N * d.batch;
        info.bytes += 4.0 * ((double)d.batch * ((double)tail_N - d.N) * P + (double)d.N * tail_N);
    }
    info.roof_us = std::max(info.bytes / (m.hbm_tbps * 1e6), info.flops / (m.fp32_tflops * 1e6));

    // --- per-workgroup costs (clock cycles of one CU) ------------------------
    const long long n_wg = (long long)g.grid_x * g.grid_y * g.grid_z;
    const double mfma_clk = (t.mf == 32) ? 64.0 : 32.0;
    const double ksteps_pass = (double)(g.cpw / g.kc) * g.ktaps;
    // One wave's matrix-core time per pass; the LDS reads of a K-step (one A and
    // one B word per lane per block row/column) must fit under it.
    // (Winograd: the register transform of the input patch shares the wave's issue slots with its MFMAs)
    const double mfma_pass = ksteps_pass * t.mb * t.nb * (mfma_clk + (t.alg == 1 ? MC.wino_kstep_clk : 0.0));
    const double copy_bytes_pass = (double)g.stage_floats * 4.0;
    const double red_bytes = t.wk > 1 ? (double)t.wk * g.MT * g.PT * 4.0 * 2.0 : 0.0;
    // (the Winograd epilogue stores four pixels per instruction where tile and image width are multiples of four,
    //  two where the image width is even: cheaper per byte than single-pixel stores)
    const double store_width = t.alg != 1 ? 1.0 : ((g.TW | g.Wo) % 4 == 0) ? 0.6 : (g.Wo % 2 == 0) ? 0.85 : 1.0;
    const double out_bytes = (double)g.MT * g.PT * 4.0 * store_width;

    // Copy instructions of one pass (64 elements each) and how long issuing them holds a wave: the first
    // pass is dealt to every wave; later ones to the loader waves if there are any, else to everybody.
    const int ncomp = t.wm * t.wn * t.wk;
    const double n_instr = (double)g.in_stage_floats / (64.0 * g.VW) + (t.alg ? 0.0 : std::ceil(g.wslab_floats / 256.0));
    const double issue_first = std::ceil(n_instr / g.waves) * MC.copy_issue_clk;
    const double issue_steady = std::ceil(n_instr / (t.wl ? t.wl : g.waves)) * MC.copy_issue_clk;
    const int comp_waves_per_simd = ceil_div(ncomp, m.simds_per_cu);

    auto wg_time = [&](int r, long long concurrent_wgs) {
        if (t.alg == 5) {
            // like the streamed direct kernel: set-up, one round trip, the bytes at the achieved fill rate, the requests
            // of a wave one after the other, the MFMA chains of the waves that share a SIMD (the transform's vector work
            // mostly hides under them), output transform and drain, the reduction, the store.  Per input channel and 16
            // output channels 1 KiB of transformed weights; per input channel four rows of 128 bytes.
            // (fitted to 60 timed tiles of 13 shapes, 6 % mean error)
            const double chip_share =
                MC.l2_bytes_per_clk / std::max<double>(1.0, (double)std::min<long long>(concurrent_wgs, m.cus));
            const double rate = std::min(1.31 * MC.copy_bytes_per_clk, chip_share);
            const double bytes = (double)t.cch * (t.wm * 1024.0 + 512.0) * r;
            const double groups = (double)t.cch / (4.0 * t.wk);
            const double waves_simd = std::ceil((double)g.waves * r / m.simds_per_cu);
            double clk = MC.stream_setup_clk + MC.stream_latency_clk + 65.0 * (waves_simd - 1.0) + bytes / rate +
                         groups * 8.0 * 21.4 + waves_simd * groups * 16.0 * (mfma_clk + 10.0);
            clk += 1.6 * MC.sync_clk + 1000.0;   // MFMA drain, output transform, park, barrier
            const double rounds = std::ceil((double)g.MT * 32.0 / g.threads);
            clk += rounds * (110.0 + 8.0 * t.wk) + out_bytes * r / 200.0;
            return clk;
        }
        if (t.alg == 4 || t.alg == 6) {
            // as below; per input channel 576 bytes of weights and nine 64-byte rows of input (the rows of
            // neighbouring taps mostly hit in the L1, so they count for less than their size)
            const double chip_share =
                MC.l2_bytes_per_clk / std::max<double>(1.0, (double)std::min<long long>(concurrent_wgs, m.cus));
            // (fitted to 364 timed tiles of 35 shapes, 7 % mean error: the achieved fill rate is lower than that of the
            //  1x1 path; the nine taps of a lane are separate requests that mostly hit in the L1, three requests and lane
            //  shifts where a tile is one row of 14 pixels)
            const double rate = std::min(0.59 * MC.copy_bytes_per_clk, chip_share);
            const bool row_mode = d.stride == 1 && t.tw == 14;
            // (nb pixel blocks per wave: the input rows of every block, the weights once)
            // (alg 6: the window of the tile once, 16 bytes per slot)
            const double in_bytes_ch = t.alg == 6 ? 16.0 * g.win_rows * g.win_L * 0.7 : t.nb * (row_mode ? 0.28 : 0.66) * 576.0;
            const double bytes = (double)t.cch * t.wm * (576.0 + in_bytes_ch) * r;
            const double groups = (double)t.cch / (4.0 * t.wk);
            const double waves_simd = std::ceil((double)g.waves * r / m.simds_per_cu);
            // a wave issues its requests one after the other (about 21 cycles each): fewer groups per wave start sooner
            // (288 cycles per group: a wave's own nine MFMAs per block run one after the other)
            // (alg 6: one or two requests per group for the window, then its way through LDS: a write, nine reads)
            const double in_requests = t.alg == 6 ? (double)g.win_nreq : t.nb * (row_mode ? 3.0 : 9.0);
            double clk = MC.stream_setup_clk + MC.stream_latency_clk + 288.0 * groups + 65.0 * (waves_simd - 1.0) + bytes / rate +
                         groups * (3.0 + in_requests) * 21.4 + (t.alg == 6 ? 150.0 + 40.0 * groups * (t.nb > 1 ? 1.5 * t.nb : 1.0) : 0.0);
            // the MFMAs of the extra blocks no longer hide under the requests: the matrix pipe of a SIMD serves its waves in turn
            if (t.nb > 1) {
                clk += waves_simd * groups * 9.0 * (t.nb - 1) * mfma_clk;
                // all threads share the final sum and store; a workgroup of few waves walks its blocks in several rounds
                const double rounds = std::ceil((double)t.wm * t.nb * 256.0 / g.threads);
                clk += (rounds - 1.0) * (110.0 + 8.0 * t.wk);
            }
            if (t.wk > 1) clk += 1.6 * MC.sync_clk;
            if (tail_N > 0) {
                // park the columns, a barrier, the first touch of the tail's weights, its blocks dealt over the waves
                const double blocks = std::ceil((double)ceil_div(tail_N, 16) / g.waves);
                clk += MC.sync_clk + MC.stream_latency_clk + blocks * (g.tail_ng * 40.0 + 64.0) +
                       (double)tail_N * d.N * 4.0 * r / rate + (double)tail_N * 64.0 * r / 200.0;
                return clk;
            }
            if (t.ks > 1) clk += MC.ksplit_clk + 1000.0 * (t.ks - 2) + (double)t.ks * 1024.0 * r / rate;   // (timed: each slice past the second adds 0.4 us)
            clk += out_bytes * r / 200.0;
            return clk;
        }
        if (t.alg == 3) {
            // every wave requests its whole share up front and works through it as it arrives: one round trip, the
            // bytes at the CU's (or the chip's) fill rate, two chains of dependent MFMAs, the reduction over the waves
            const double chip_share =
                MC.l2_bytes_per_clk / std::max<double>(1.0, (double)std::min<long long>(concurrent_wgs, m.cus));
            const double rate = std::min(MC.copy_bytes_per_clk, chip_share);
            const double bytes = (double)t.cch * (64.0 + 64.0) * r;   // weights and input of one 16x16 block
            const double runs = (double)t.cch / (16.0 * t.wk);
            const double waves_simd = std::ceil((double)g.waves * r / m.simds_per_cu);
            // (fitted to 71 timed tiles of 23 shapes: the requests of all resident waves overlap, so only the bytes,
            //  a little per extra wave and half an MFMA time per K-step show; the stores are hidden)
            double clk = MC.stream_setup_clk + MC.stream_latency_clk + 20.0 * (waves_simd - 1.0) + bytes / (0.87 * rate) +
                         runs * 4.0 * 0.5 * mfma_clk * waves_simd;
            if (t.wk > 1) clk += 1.5 * MC.sync_clk;
            if (t.ks > 1) clk += MC.ksplit_clk + 1000.0 * (t.ks - 2) + (double)t.ks * 1024.0 * r / rate;   // (timed: each slice past the second adds 0.4 us)
            clk += out_bytes * r / 64.0;
            return clk;
        }
        // r workgroups share one CU: matrix time and the issue cycles of the operand reads add up per
        // SIMD; copies share the CU's fill rate and, chip-wide, the L2.
        const double waves_simd = (double)comp_waves_per_simd * r;
        // A wave alone on its SIMD stalls on every operand read and while it issues copies; with several
        // waves per SIMD those gaps are filled by the others until the matrix pipe itself is the limit.
        // (wino = 2: the A operands do not come from the LDS)
        const double a_reads = t.alg == 2 ? 0.25 * t.mb : (double)t.mb;
        const double stall = ksteps_pass * (a_reads + t.nb * g.b_ways) * MC.kstep_issue_clk + MC.pass_overhead_clk;
        const double alone = mfma_pass + stall;
        // ... or the LDS: every operand read keeps it busy for lds_read_clk cycles, a conflicting one longer.
        const double lds_busy = ksteps_pass * ((t.alg == 2 ? 0.0 : (double)t.mb) + t.nb * g.b_ways) * MC.lds_read_clk * ncomp * r;
        const double pipe = std::max(mfma_pass * waves_simd, lds_busy) + MC.pass_overhead_clk;
        const double compute = std::max(alone, pipe) + MC.sync_clk;
        const double compute_issuing = std::max(alone + issue_steady, pipe) + MC.sync_clk;
        const double chip_share =
            MC.l2_bytes_per_clk / std::max<double>(1.0, (double)std::min<long long>(concurrent_wgs, m.cus));
        const double rate = std::min(MC.copy_bytes_per_clk, chip_share);
        const double copy = copy_bytes_pass * r / rate;
        // First pass is exposed; afterwards the copy of pass i+1 runs under the MFMAs of pass i.
        double clk = MC.setup_clk + MC.wave_setup_clk * ((double)wg_waves_per_simd * r - 1.0) + issue_first +
                     MC.copy_latency_clk + copy + (t.alg == 2 ? MC.gw_latency_clk : 0.0);
        clk += compute;  // last pass: nothing left to hide
        if (g.cps > 1) {
            const double pass = t.wl ? std::max(compute, std::max(issue_steady, copy) + MC.copy_latency_clk)
                                     : std::max(compute_issuing, copy + MC.copy_latency_clk);
            clk += (g.cps - 1) * pass;
        }
        clk += red_bytes * r / MC.lds_bytes_per_clk + out_bytes * r / MC.store_bytes_per_clk +
               (t.wk > 1 ? 2.0 * MC.sync_clk : 0.0);
        // Split across workgroups: the partial tile goes to the workspace (the store above), and the
        // workgroup that draws the last ticket reads all ks partials back before the real store.
        if (t.ks > 1)
            clk += MC.ksplit_clk + MC.copy_latency_clk + (double)t.ks * out_bytes / rate +
                   out_bytes / MC.store_bytes_per_clk;
        // Fused tail: park the tile, one more barrier, the first touch of the tail's weights, then the 16x16
        // blocks of the small GEMM dealt over the waves, and the tail's own store.
        if (tail_N > 0) {
            const double blocks = std::ceil((double)ceil_div(tail_N, 16) * (g.PT / 16) / g.waves);
            clk += out_bytes * r / MC.lds_bytes_per_clk + MC.sync_clk + MC.copy_latency_clk +
                   blocks * (g.tail_ng * 32.0 + 64.0) * r + (double)tail_N * g.PT * 4.0 * r / MC.store_bytes_per_clk -
                   out_bytes * r / MC.store_bytes_per_clk;
        }
        return clk;
    };
    const long long slots = (long long)m.cus * wg_per_cu;
    const long long full = n_wg / slots;
    const long long rem = n_wg % slots;
    double clk = (double)full * wg_time(wg_per_cu, slots);
    if (rem) clk += wg_time((int)((rem + m.cus - 1) / m.cus), rem);
    info.pred_us = MC.launch_us + clk / (m.clock_ghz * 1e3);
    info.pred_l2_bytes = (double)n_wg * g.cps * copy_bytes_pass;
    return true;
}

std::vector<tdc_tile> model_enumerate(const tdc_conv_desc &d, int tail_N) {
    std::vector<tdc_tile> out;
    if (!check_desc(d, nullptr)) return out;
    const bool flat = (d.KH == 1 && d.KW == 1 && d.stride == 1 && d.pad == 0);
    const int He = flat ? 1 : d.H, We = flat ? d.H * d.W : d.W;
    const int Ho = (He + 2 * d.pad - d.dilation * (d.KH - 1) - 1) / d.stride + 1;
    const int Wo = (We + 2 * d.pad - d.dilation * (d.KW - 1) - 1) / d.stride + 1;
    const int P = Ho * Wo;
    static const int mfs[] = {16, 32};
    static const int wks[] = {1, 2, 4, 8, 16};
    static const int wms[] = {1, 2, 4};
    static const int wns[] = {1, 2, 4};
    // streamed 1x1 candidates: the input channels in runs of 16, 1, 2, 4 or 8 runs per wave
    if (d.KH == 1 && d.KW == 1 && d.pad == 0 && tail_N == 0 && !std::getenv("TDC_EXPERIMENT_NO_STREAMED_1X1")) {
        // (a split of the input channels over ks workgroups only where the layer leaves most of the chip idle)
        for (int ks : {1, 2, 4, 8}) {
            if (ks > 1 && !flat) break;
            const int runs = ceil_div(ceil_div(d.C, ks), 16);
            for (int per_wave : {8, 4, 2, 1}) {
                if (per_wave > runs) continue;   // (more than half of such a wave's channels would be padding)
                const int wk = ceil_div(runs, per_wave);
                if (wk > 16) continue;
                tdc_tile t{16, 1, 1, 1, 1, wk, 16 * per_wave * wk, std::min(16, P), ks, 0, 3};
                Geometry g;
                if (!make_geometry(d, t, g, nullptr, 0)) continue;
                if (ks > 1 && (long long)g.grid_x * g.grid_y * g.grid_z > 2LL * machine().cus) continue;
                out.push_back(t);
            }
        }
    }
    // streamed 3x3 candidates: 1, 2 or 4 groups of four channels per wave, a few shapes of the 16-pixel tile
    if (d.KH == 3 && d.KW == 3 && d.dilation == 1 && !std::getenv("TDC_EXPERIMENT_NO_STREAMED_3X3")) {
        std::vector<int> tws;
        for (int tw : {16, 14, 8, 7, 4, std::min(16, Wo)}) {
            if (tw > std::min(16, Wo) || std::find(tws.begin(), tws.end(), tw) != tws.end()) continue;
            const int th = std::min(16 / tw, Ho);
            const double util = (double)P / ((double)ceil_div(Wo, tw) * ceil_div(Ho, th) * 16);
            if (util < 0.6 && tw != std::min(16, Wo)) continue;
            tws.push_back(tw);
        }
        // (a fused tail needs every output channel in the workgroup: one wave per block of 16 and channel slice)
        const int wm = tail_N > 0 ? ceil_div(d.N, 16) : 1;
        for (int ks : {1, 2, 4, 8}) {
            if (ks > 1 && tail_N > 0) break;
            const int groups_slice = ceil_div(ceil_div(d.C, ks), 4);
            for (int per_wave : {4, 2, 1}) {
                if (per_wave > groups_slice) continue;
                const int wk = ceil_div(groups_slice, per_wave);
                if (wm * wk > 16) continue;
                for (int tw : tws) {
                    tdc_tile t{16, 1, 1, wm, 1, wk, 4 * per_wave * wk, tw, ks, 0, 4};
                    Geometry g;
                    if (!make_geometry(d, t, g, nullptr, tail_N)) continue;
                    if (ks > 1 && (long long)g.grid_x * g.grid_y * g.grid_z > 2LL * machine().cus) continue;
                    out.push_back(t);
                    // the same tile with its input window loaded in 128-bit pieces and passed through LDS
                    if (d.pad <= 1 && d.stride <= 2 && !std::getenv("TDC_EXPERIMENT_NO_STREAMED_WINDOW")) {
                        tdc_tile t6 = t;
                        t6.alg = 6;
                        if (make_geometry(d, t6, g, nullptr, tail_N)) out.push_back(t6);
                    }
                    // the same tile with 2 or 4 neighbouring 14-pixel row tiles per workgroup, sharing the weights in
                    // registers (where the image row has that many)
                    if (tw == 14 && d.stride == 1 && ks == 1 && tail_N == 0 && !std::getenv("TDC_EXPERIMENT_NO_STREAMED_NB"))
                        for (int nb : {2, 4}) {
                            if (ceil_div(Wo, 14) < nb) continue;
                            t.nb = nb;
                            if (make_geometry(d, t, g, nullptr, 0) &&
                                kernel_id_for(t, 3, 3, 1, 1, false).family != KernelId::NONE)
                                out.push_back(t);
                            // ... and with the rows of all blocks loaded as one window through LDS
                            if (d.pad <= 1 && !std::getenv("TDC_EXPERIMENT_NO_STREAMED_WINDOW")) {
                                tdc_tile t6 = t;
                                t6.alg = 6;
                                if (make_geometry(d, t6, g, nullptr, 0) &&
                                    kernel_id_for(t6, 3, 3, 1, 1, false).family != KernelId::NONE)
                                    out.push_back(t6);
                            }
                        }
                }
            }
        }
    }
    // streamed Winograd candidates: 3x3 / stride 1 / pad 1, even width, all input channels in one pass.  Offered for single
    // images only: the kernel is built for the latency of one small launch, and at batch 8 its timing alone misleads the
    // measured selection (DenseNet-121's 64 -> 16 @56x56 core at batch 8: 6.9 us alone against 8.1 us for the staged
    // Winograd tile, but the network ran 2.5 % slower with it); a forced tile still runs any batch.
    if (d.batch == 1 && d.KH == 3 && d.KW == 3 && d.stride == 1 && d.dilation == 1 && d.pad == 1 && d.W % 2 == 0 && tail_N == 0 &&
        !std::getenv("TDC_EXPERIMENT_NO_STREAMED_WINOGRAD")) {
        const int groups_total = ceil_div(d.C, 4);
        for (int wm : {1, 2}) {
            if (16 * wm > round_up(d.N, 16)) continue;
            for (int per_wave : {4, 3, 2, 1}) {
                if (per_wave > groups_total) continue;
                const int wk = ceil_div(groups_total, per_wave);
                if (wm * wk > wino_stream_max_waves(per_wave)) continue;
                if (per_wave * wk - groups_total >= per_wave) continue;   // an idle wave
                tdc_tile t{16, 1, 1, wm, 1, wk, 4 * per_wave * wk, 28, 1, 0, 5};
                Geometry g;
                if (make_geometry(d, t, g, nullptr, 0)) out.push_back(t);
            }
        }
    }
    // Winograd candidates for 3x3 / stride 1 convolutions with enough pixels to fill tile lanes
    if (d.KH == 3 && d.KW == 3 && d.stride == 1 && d.dilation == 1 && tail_N == 0 && !std::getenv("TDC_EXPERIMENT_NO_WINOGRAD")) {
        const int Wt = ceil_div(Wo, 2), Ht = ceil_div(Ho, 2);
        for (int wm : wms)
            for (int wn : wns)
                for (int wk : wks) {
                    if (wm * wn * wk > 8) continue;
                    if (16 * wm > round_up(d.N, 16)) continue;
                    const int lanes = 16 * wn;
                    if (lanes > round_up(Wt * Ht, 16)) continue;
                    std::vector<int> tws;
                    for (int tw = 1; tw <= std::min(Wt, lanes); ++tw) {
                        const bool pow2 = (tw & (tw - 1)) == 0;
                        const bool widest = (tw == std::min(Wt, lanes));
                        if (!(widest || (pow2 && tw >= 2) || (Wt % tw == 0 && tw >= 2))) continue;
                        const int th = std::min(lanes / tw, Ht);
                        const double util = (double)(Wt * Ht) / ((double)ceil_div(Wt, tw) * ceil_div(Ht, th) * lanes);
                        if (util < 0.7 && !widest) continue;
                        tws.push_back(tw);
                    }
                    const int granule = 4 * wk;
                    std::vector<int> cchs;
                    for (int div : {1, 2, 4, 8}) {
                        const int cch = round_up(ceil_div(d.C, div), granule);
                        if (std::find(cchs.begin(), cchs.end(), cch) == cchs.end()) cchs.push_back(cch);
                    }
                    for (int fixed : {16, 32})
                        if (fixed % granule == 0 && fixed < round_up(d.C, granule) &&
                            std::find(cchs.begin(), cchs.end(), fixed) == cchs.end())
                            cchs.push_back(fixed);
                    const long long max_wgs = 4LL * machine().cus;
                    for (int tw : tws)
                        for (int cch : cchs)
                            for (int ks : {1, 2, 4})
                                for (int wl : {0, 2, 4}) {
                                    tdc_tile t{16, 1, 1, wm, wn, wk, cch, tw, ks, wl, 1};
                                    Geometry g;
                                    if (!make_geometry(d, t, g, nullptr, 0)) continue;
                                    if (ks > 1 && (long long)g.grid_x * g.grid_y * g.grid_z > max_wgs) continue;
                                    if (wl > 0 && g.cps < 2) continue;
                                    out.push_back(t);
                                }
                }
    }
    const bool global_weights = d.KH == 3 && d.KW == 3 && d.dilation == 1 && tail_N == 0 &&
                                !std::getenv("TDC_EXPERIMENT_NO_GLOBAL_WEIGHTS");
    for (int mf : mfs) {
        const int kc = (mf == 32) ? 2 : 4;
        for (int mb = 1; mb <= 2; ++mb)
            for (int nb = 1; nb <= 2; ++nb)
                for (int wm : wms)
                    for (int wn : wns)
                        for (int wk : wks) {
                            const int maxw = (mb == 2 && nb == 2) ? 8 : 16;
                            if (wm * wn * wk > maxw) continue;
                            if (mf * mb * wm > round_up(d.N, mf)) continue;  // do not tile past the problem
                            const int PT = mf * nb * wn;
                            if (PT > round_up(P, mf)) continue;
                            // Tile widths: the whole row, and power-of-two or exact-divisor widths
                            // that keep at least 70 % of the pixel lanes on real pixels.
                            std::vector<int> tws;
                            for (int tw = 1; tw <= std::min(Wo, PT); ++tw) {
                                const bool pow2 = (tw & (tw - 1)) == 0;
                                const bool widest = (tw == std::min(Wo, PT));
                                if (flat && !widest) continue;  // one row of pixels: nothing to gain from narrower runs
                                if (!(widest || (pow2 && tw >= 4) || (Wo % tw == 0 && tw >= 4))) continue;
                                const int th = std::min(PT / tw, Ho);
                                const double util = (double)P / ((double)ceil_div(Wo, tw) * ceil_div(Ho, th) * PT);
                                if (util < 0.7 && !widest) continue;
                                tws.push_back(tw);
                            }
                            const int granule = kc * wk;
                            const int c_full = round_up(d.C, granule);
                            std::vector<int> cchs;
                            for (int div : {1, 2, 4, 8}) {
                                const int cch = round_up(ceil_div(d.C, div), granule);
                                if (std::find(cchs.begin(), cchs.end(), cch) == cchs.end()) cchs.push_back(cch);
                            }
                            for (int fixed : {16, 32})
                                if (fixed % granule == 0 && fixed < c_full &&
                                    std::find(cchs.begin(), cchs.end(), fixed) == cchs.end())
                                    cchs.push_back(fixed);
                            // Splitting the passes over several workgroups only pays while the
                            // layer has fewer tiles than the chip has room for.
                            const long long max_wgs = 4LL * machine().cus;
                            for (int tw : tws)
                                for (int cch : cchs)
                                    for (int ks : {1, 2, 4, 8})
                                        for (int wl : {0, 1, 2, 4}) {
                                            tdc_tile t{mf, mb, nb, wm, wn, wk, cch, tw, ks, wl, 0};
                                            Geometry g;
                                            if (!make_geometry(d, t, g, nullptr, tail_N)) continue;
                                            if (ks > 1 && (long long)g.grid_x * g.grid_y * g.grid_z > max_wgs) continue;
                                            if (wl > 0 && g.cps < 2) continue;  // loaders only work from the second pass on
                                            out.push_back(t);
                                            // the same tile with its weights read from global memory
                                            if (global_weights && mb == 1 && nb == 1) {
                                                t.alg = 2;
                                                if (make_geometry(d, t, g, nullptr, 0)) out.push_back(t);
                                            }
                                        }
                        }
    }
    return out;
}

int model_constants(double *out, int cap) {
    std::shared_lock<std::shared_mutex> lock(MC_mutex);
    for (int i = 0; i < kNumModelConst && i < cap; ++i) out[i] = *mc_field(i);
    return kNumModelConst;
}

bool model_set_constants(const double *in, int n) {
    if (n != kNumModelConst) return false;
    for (int i = 0; i < n; ++i)
        if (!(in[i] > 0.0)) return false;
    std::unique_lock<std::shared_mutex> lock(MC_mutex);
    for (int i = 0; i < n; ++i) *mc_field(i) = in[i];
    return true;
}

bool model_select(const tdc_conv_desc &d, tdc_tile_info &best, std::string *why, int tail_N) {
    if (!check_desc(d, why)) return false;
    std::vector<tdc_tile> cands = model_enumerate(d, tail_N);
    bool have = false;
    for (const tdc_tile &t : cands) {
        tdc_tile_info info;
        if (!model_evaluate(d, t, info, nullptr, tail_N)) continue;
        if (!have || info.pred_us < best.pred_us) {
            best = info;
            have = true;
        }
    }
    if (!have && why) {
        // say why the plainest tile cannot be launched: that is the limit the shape runs into
        const tdc_tile plain{16, 1, 1, 1, 1, 1, 4, 1, 1, 0, 0};
        Geometry g;
        std::string reason;
        *why = make_geometry(d, plain, g, &reason, tail_N) ? "no launchable tile for this shape"
                                                             : "no launchable tile for this shape: " + reason;
    }
    return have;
}

}  // namespace tdc
