// Launch geometry and the closed-form gfx950 tile model.
//
// The reference chooses (TH, TW, TC) per layer either from a measured sweep
// (2080Ti-evaluation/TDC-LAYERS-ORACLE/gen_from_occupancy.py:51-66) or from an
// analytic score that still needs a table of measured CUDA occupancies
// (2080Ti-evaluation/TDC-LAYERS-MODELING/model.py:136-156,209-235;
// 2080Ti-evaluation/Gen-occupancy/template.cu:277-284).  This file is the
// self-contained counterpart for one MI355X: occupancy comes from the register
// and LDS footprint of the tile, latency from MFMA issue cycles per SIMD, the
// L1 fill rate for the staged input and streamed weights, and wave quantisation
// over 256 compute units.  Host-only code: it runs without a GPU.
#include <algorithm>
#include <cmath>
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
    if ((long long)d.C * d.H * d.W >= (1LL << 31) || (long long)d.N * d.H * d.W >= (1LL << 31))
        return fail("per-image tensor exceeds 2^31 elements");
    return true;
}

// LDS channel stride: the lanes of one ds_read that belong to different input
// channels of an MFMA K-step must fall into different banks.  With 4-byte banks
// a stride of 32 (mod 64) separates the two halves of a 32x32x2 step and a
// stride of 16 (mod 64) separates the four quarters of a 16x16x4 step.
static int pad_channel_stride(int raw, int mf) {
    const int want = (mf == 32) ? 32 : 16;
    int cs = raw;
    while (cs % 64 != want) ++cs;
    return cs;
}

bool make_geometry(const tdc_conv_desc &d, const tdc_tile &t, Geometry &g, std::string *why) {
    auto fail = [&](const std::string &m) {
        if (why) *why = m;
        return false;
    };
    if (!check_desc(d, why)) return false;
    if (t.mf != 32 && t.mf != 16) return fail("tile.mf must be 16 or 32");
    if (t.mb < 1 || t.mb > 2 || t.nb < 1 || t.nb > 2) return fail("tile.mb / tile.nb must be 1 or 2");
    if (t.wm < 1 || t.wn < 1 || t.wk < 1) return fail("tile.wm / wn / wk must be >= 1");
    g = Geometry();
    g.max_waves_kernel = (t.mb == 2 && t.nb == 2) ? 8 : 16;
    g.waves = t.wm * t.wn * t.wk;
    if (g.waves > g.max_waves_kernel) return fail("too many waves per workgroup for this tile");
    g.threads = g.waves * 64;
    g.Ho = (d.H + 2 * d.pad - d.dilation * (d.KH - 1) - 1) / d.stride + 1;
    g.Wo = (d.W + 2 * d.pad - d.dilation * (d.KW - 1) - 1) / d.stride + 1;
    g.P = g.Ho * g.Wo;
    g.kc = (t.mf == 32) ? 2 : 4;
    g.taps = d.KH * d.KW;
    g.PT = t.mf * t.nb * t.wn;
    g.MT = t.mf * t.mb * t.wm;
    g.grid_x = ceil_div(g.P, g.PT);
    g.grid_y = ceil_div(d.N, g.MT);
    g.grid_z = d.batch;
    if (g.grid_y > 65535 || g.grid_z > 65535) return fail("grid too large");
    const bool one_by_one = (d.KH == 1 && d.KW == 1);
    const int granule = g.kc * t.wk * (one_by_one ? 4 : 1);
    if (t.cch < granule || t.cch % granule != 0)
        return fail("tile.cch must be a positive multiple of kc*wk (x4 for 1x1 filters)");
    g.cpw = t.cch / t.wk;
    g.nchunks = ceil_div(d.C, t.cch);
    g.c_pad = g.nchunks * t.cch;
    g.n_pad = g.grid_y * g.MT;
    // LDS rows are filled with VW-wide vectors: the left halo and the row stride
    // are rounded up so that every image row starts on a vector boundary.
    g.VW = (d.W % 4 == 0) ? 4 : (d.W % 2 == 0) ? 2 : 1;
    g.PL = round_up(d.pad, g.VW);
    g.RS = round_up(g.PL + d.W + d.pad, g.VW);
    int nrows = 0;
    for (int bx = 0; bx < g.grid_x; ++bx) {
        const int p0 = bx * g.PT;
        const int pl = std::min(p0 + g.PT, g.P) - 1;
        const int span = pl / g.Wo - p0 / g.Wo;
        nrows = std::max(nrows, span * d.stride + (d.KH - 1) * d.dilation + 1);
    }
    g.nrows = nrows;
    g.CS = pad_channel_stride(nrows * g.RS, t.mf);
    const long long in_bytes = (long long)t.cch * g.CS * 4;
    const long long red_bytes = t.wk > 1 ? (long long)t.wk * g.MT * g.PT * 4 : 0;
    const long long lds = std::max(in_bytes, red_bytes);
    if (lds > machine().lds_bytes_per_cu) return fail("tile needs more than 160 KiB of LDS");
    g.lds_bytes = (int)lds;
    return true;
}

size_t packed_weight_floats(const Geometry &g, int mf) {
    return (size_t)(g.n_pad / mf) * (size_t)(g.c_pad / g.kc) * (size_t)g.taps * 64;
}

void pack_weights(const tdc_conv_desc &d, const Geometry &g, int mf, const float *w, float *packed) {
    const int nmblk = g.n_pad / mf;
    const int ncg = g.c_pad / g.kc;
    const int taps = g.taps;
    for (int mblk = 0; mblk < nmblk; ++mblk) {
        for (int cg = 0; cg < ncg; ++cg) {
            for (int tap = 0; tap < taps; ++tap) {
                float *dst = packed + (((size_t)mblk * ncg + cg) * taps + tap) * 64;
                for (int l = 0; l < 64; ++l) {
                    const int n = mblk * mf + l % mf;
                    const int c = cg * g.kc + l / mf;
                    dst[l] = (n < d.N && c < d.C) ? w[((size_t)n * d.C + c) * taps + tap] : 0.0f;
                }
            }
        }
    }
}

// ---------------------------------------------------------------------------
// Analytic model
// ---------------------------------------------------------------------------
namespace {

struct ModelConst {
    double launch_us = 1.6;        // empty-kernel device time incl. dispatch ramp
    double l1_bytes_per_clk = 64;  // per-CU vector memory fill rate
    double mem_latency_clk = 1800; // first-byte latency of a dependent fetch (L2/MALL)
    double lds_bytes_per_clk = 128;
    double sync_clk = 200;
};
const ModelConst MC;

int estimate_vgprs(const tdc_tile &t, int taps) {
    const int nacc = (t.mf == 32) ? 16 : 4;
    int regs = nacc * t.mb * t.nb;             // accumulators
    if (taps == 9) regs += 2 * 9 * t.mb + 9 * t.nb;   // two weight buffers + row of B
    else if (taps == 1) regs += 2 * 4 * t.mb + 4 * t.nb;
    else regs += t.mb + t.nb;
    regs += 28;                                 // addresses, indices, staging temporaries
    return round_up(regs, 8);
}

}  // namespace

bool model_evaluate(const tdc_conv_desc &d, const tdc_tile &t, tdc_tile_info &info, std::string *why) {
    Geometry g;
    if (!make_geometry(d, t, g, why)) return false;
    const Machine &m = machine();
    std::memset(&info, 0, sizeof(info));
    info.tile = t;
    info.grid_x = g.grid_x;
    info.grid_y = g.grid_y;
    info.grid_z = g.grid_z;
    info.block_threads = g.threads;
    info.lds_bytes = g.lds_bytes;
    info.nchunks = g.nchunks;
    info.vgpr_estimate = estimate_vgprs(t, g.taps);

    // --- occupancy (replaces cudaOccupancyMaxActiveBlocksPerMultiprocessor) ---
    const int waves_simd_vgpr = std::min(m.max_waves_per_simd, m.vgprs_per_simd_lane / info.vgpr_estimate);
    const int wg_waves_per_simd = ceil_div(g.waves, m.simds_per_cu);
    const int wg_by_vgpr = waves_simd_vgpr / wg_waves_per_simd;
    const int wg_by_lds = m.lds_bytes_per_cu / std::max(g.lds_bytes, 1);
    int wg_per_cu = std::min(wg_by_vgpr, wg_by_lds);
    if (wg_per_cu < 1) {
        if (why) *why = "tile does not fit one compute unit";
        return false;
    }
    wg_per_cu = std::min(wg_per_cu, 8);
    info.wg_per_cu = wg_per_cu;
    info.waves_per_simd = wg_per_cu * wg_waves_per_simd;

    // --- algorithmic work and roofline ---------------------------------------
    const double P = g.P;
    info.flops = 2.0 * P * d.C * d.N * g.taps * d.batch;
    info.bytes = 4.0 * ((double)d.batch * ((double)d.C * d.H * d.W + (double)d.N * P) +
                        (double)g.taps * d.C * d.N);
    info.roof_us = std::max(info.bytes / (m.hbm_tbps * 1e6), info.flops / (m.fp32_tflops * 1e6));

    // --- per-workgroup costs (clock cycles of one CU) ------------------------
    const double mfma_clk = (t.mf == 32) ? 64.0 : 32.0;
    const double ksteps_wave = (double)g.nchunks * (g.cpw / g.kc) * g.taps;
    const double mfma_wave = ksteps_wave * t.mb * t.nb * mfma_clk;       // one wave's matrix-core time
    const double stage_bytes = (double)g.c_pad * g.nrows * g.RS * 4.0;   // input slab of one WG
    const double weight_bytes = ksteps_wave * t.mb * 256.0 * g.waves;    // streamed by all waves of one WG
    const double red_bytes = t.wk > 1 ? (double)t.wk * g.MT * g.PT * 4.0 * 2.0 : 0.0;
    const double out_bytes = (double)g.MT * g.PT * 4.0;

    const long long n_wg = (long long)g.grid_x * g.grid_y * g.grid_z;
    auto round_clk = [&](int r) {
        // r workgroups share one CU: matrix time adds up per SIMD, fills share the L1 port.
        const double mfma = mfma_wave * wg_waves_per_simd * r;
        const double wfill = weight_bytes * r / MC.l1_bytes_per_clk;
        const double sfill = stage_bytes * r / MC.l1_bytes_per_clk;
        // Staging of one workgroup overlaps other workgroups' MFMAs only when r > 1.
        const double stage = MC.mem_latency_clk * g.nchunks + (r > 1 ? 0.5 : 1.0) * sfill +
                             2.0 * MC.sync_clk * g.nchunks;
        const double epi = red_bytes * r / MC.lds_bytes_per_clk + out_bytes * r / MC.l1_bytes_per_clk +
                           (t.wk > 1 ? 2.0 * MC.sync_clk : 0.0) + 300.0;
        return stage + std::max(mfma + MC.mem_latency_clk * 0.25, wfill + MC.mem_latency_clk) + epi;
    };
    const long long slots = (long long)m.cus * wg_per_cu;
    const long long full = n_wg / slots;
    const long long rem = n_wg % slots;
    double clk = (double)full * round_clk(wg_per_cu);
    if (rem) clk += round_clk((int)ceil_div((int)rem, m.cus));
    info.pred_us = MC.launch_us + clk / (m.clock_ghz * 1e3);
    info.pred_hbm_bytes = (double)n_wg * (stage_bytes + weight_bytes) + (double)d.batch * d.N * P * 4.0;
    return true;
}

std::vector<tdc_tile> model_enumerate(const tdc_conv_desc &d) {
    std::vector<tdc_tile> out;
    std::string why;
    if (!check_desc(d, &why)) return out;
    const Machine &m = machine();
    const int Ho = (d.H + 2 * d.pad - d.dilation * (d.KH - 1) - 1) / d.stride + 1;
    const int Wo = (d.W + 2 * d.pad - d.dilation * (d.KW - 1) - 1) / d.stride + 1;
    const int P = Ho * Wo;
    const bool one_by_one = (d.KH == 1 && d.KW == 1);
    static const int mfs[] = {32, 16};
    static const int wks[] = {1, 2, 4, 8, 16};
    static const int wms[] = {1, 2, 4};
    static const int wns[] = {1, 2, 4};
    for (int mf : mfs) {
        const int kc = (mf == 32) ? 2 : 4;
        for (int mb = 1; mb <= 2; ++mb)
            for (int nb = 1; nb <= 2; ++nb)
                for (int wm : wms)
                    for (int wn : wns)
                        for (int wk : wks) {
                            const int maxw = (mb == 2 && nb == 2) ? 8 : 16;
                            if (wm * wn * wk > maxw) continue;
                            // Do not tile past the problem.
                            if (mf * mb * wm > round_up(d.N, mf)) continue;
                            if (mf * nb * wn > round_up(P, mf)) continue;
                            const int granule = kc * wk * (one_by_one ? 4 : 1);
                            const int c_full = round_up(d.C, granule);
                            // Candidate LDS pass sizes: everything at once, or the largest
                            // slab that leaves room for 1, 2 or 4 workgroups per CU.
                            int last = -1;
                            for (int share = 0; share <= 3; ++share) {
                                int cch;
                                if (share == 0) {
                                    cch = c_full;
                                } else {
                                    const int budget = m.lds_bytes_per_cu / (1 << (share - 1));
                                    tdc_tile probe{mf, mb, nb, wm, wn, wk, granule};
                                    Geometry gp;
                                    if (!make_geometry(d, probe, gp, nullptr)) continue;
                                    const int fit = budget / (gp.CS * 4);
                                    cch = std::min(c_full, (fit / granule) * granule);
                                    if (cch < granule) continue;
                                    // Prefer an even split of the channels over a ragged last pass.
                                    const int passes = ceil_div(d.C, cch);
                                    cch = round_up(ceil_div(d.C, passes), granule);
                                }
                                if (cch == last) continue;
                                tdc_tile t{mf, mb, nb, wm, wn, wk, cch};
                                Geometry g;
                                if (!make_geometry(d, t, g, nullptr)) continue;
                                bool dup = false;
                                for (const tdc_tile &o : out)
                                    if (!std::memcmp(&o, &t, sizeof(t))) { dup = true; break; }
                                if (dup) continue;
                                out.push_back(t);
                                last = cch;
                            }
                        }
    }
    return out;
}

bool model_select(const tdc_conv_desc &d, tdc_tile_info &best, std::string *why) {
    if (!check_desc(d, why)) return false;
    std::vector<tdc_tile> cands = model_enumerate(d);
    bool have = false;
    for (const tdc_tile &t : cands) {
        tdc_tile_info info;
        if (!model_evaluate(d, t, info, nullptr)) continue;
        if (!have || info.pred_us < best.pred_us) {
            best = info;
            have = true;
        }
    }
    if (!have && why) *why = "no launchable tile for this shape";
    return have;
}

}  // namespace tdc
