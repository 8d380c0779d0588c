// Streamed Winograd F(2x2,3x3) convolution (tile.alg = 5): 3x3 / stride 1 / pad 1 / even image width.
//
// One workgroup owns 16*WM output channels of one TILE ROW block: two output rows x 28 output columns = 14 tiles of
// 2x2 pixels, one tile per pixel lane (lanes 14 and 15 of a quarter carry the block's halo columns only).  Its WK
// waves split the input channels, CG groups of four channels each (lane quarter k = channel 4g + k).  Nothing is
// staged in LDS and there is no pass loop: a wave requests everything it needs at once, straight into registers,
//   * per group the 16 transformed weights U = G g G^T of its (output channel, input channel) pairs: four 128-bit
//     loads from the packed weights (same packing as the staged Winograd path, one pass);
//   * per group the four input rows under the tile row, each as ONE 64-bit load per lane: lane j of a quarter loads
//     the column pair (28*bx - 2 + 2j, +1), so the 16 lanes cover columns 28*bx - 2 .. 28*bx + 29 exactly once.  Tile
//     j needs columns 2j-1 .. 2j+2 of the block = the second word of pair j, both words of pair j+1 and the first of
//     pair j+2: its neighbours' registers, fetched with row_shl lane shifts (DPP) instead of overlapping loads.
// Against the direct streamed kernel this moves 4 rows x 128 bytes of input per four channels and 28 x 2 outputs where
// that one moves 3 rows x 64 bytes per 14 outputs, and issues 16 MFMAs per four channels and 56 pixels instead of 36.
// The input transform V = B^T d B is done on the loaded pairs BEFORE the shifts (rows first: it is the same for both
// words of a pair), so a group costs 36 vector-ALU operations next to its 16 MFMAs.
// After its last group a wave turns its 16 accumulators into 2x2 outputs (Y = A^T M A, in registers: all 16
// positions of a tile sit in one lane) and parks them in LDS; all threads of the workgroup then add the WK slices in
// slice order (bit-reproducible) and store pairs of pixels with bias, residual and ReLU fused.
#include "conv_device.hpp"

namespace tdc {

typedef float f2_t __attribute__((ext_vector_type(2)));
typedef unsigned u2_t __attribute__((ext_vector_type(2)));

// lane j of a 16-lane row takes the value of lane j + 1 / j + 2 (zero past the row)
__device__ __forceinline__ float shl1(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x101, 0xf, 0xf, true));
}

// Four groups per wave would need 142 registers per lane with everything requested up front; the operands of the third
// and fourth group are requested when the first and second have been consumed instead, which keeps the kernel inside
// the 128 registers that let two 8-wave workgroups share a compute unit.
template <int CG, int MAXW>
__global__ void __launch_bounds__(MAXW * 64) tdc_wino3x3_stream_kernel(const ConvKParams p) {
    constexpr int NOW = CG < 4 ? CG : 2;   // groups requested before the first MFMA
    extern __shared__ __align__(16) float lds[];
    TDC_STAMP_DECL;
    TDC_STAMP(0);   // entry
    touch_kernel_arguments();
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    // die-aware decoding of the one-dimensional launch, as in the other kernels
    const int logical = (int)(blockIdx.x & 7u) * p.xcd_chunk + (int)(blockIdx.x >> 3);
    if (logical >= p.n_wg) return;
    const int q1 = fdiv(logical, p.fd_g1);
    const int r1 = logical - q1 * p.fd_g1.d;
    const int img = fdiv(q1, p.fd_g2);
    const int r2 = q1 - img * p.fd_g2.d;
    const int bx = p.channel_major ? r1 : r2;  // tile-row block
    const int by = p.channel_major ? r2 : r1;  // channel tile
    const int tile_y = fdiv(bx, p.fd_ntx);     // tile row: output rows 2*tile_y, 2*tile_y + 1
    const int tile_x = bx - tile_y * p.ntx;    // block of 28 output columns in that row
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
    // packed weights: [channel tile][block of the workgroup][group][quarter][lane][4], 4 KiB per group
    const int a_soff = (((by * p.WM + wmi) * (p.CCH >> 2)) + wki * CG) * 4096;
    f4_t u[CG][4];
    f2_t xin[CG][4];
    auto load_weights = [&](int g) {
#pragma unroll
        for (int q = 0; q < 4; ++q)
            u[g][q] = __builtin_bit_cast(f4_t, __builtin_amdgcn_raw_buffer_load_b128(w_rsrc, lane * 16, a_soff + g * 4096 + q * 1024, 0));
    };
    load_weights(0);   // (they depend on nothing but the block index and the wave)
    __builtin_amdgcn_sched_barrier(0);

    const int k = lane >> 4, j = lane & 15;
    const unsigned chan_bytes = (unsigned)(p.H * p.W) * 4u;
    const unsigned base = (unsigned)(wki * (4 * CG) + k) * chan_bytes;   // this lane's first channel
    const int iy0 = 2 * tile_y - 1;
    const int ix = tile_x * 28 - 2 + 2 * j;             // first column of this lane's pair
    const bool col_ok = (unsigned)ix < (unsigned)(p.W - 1);   // (W is even: a pair lies inside the row or outside it)
    unsigned roff[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        const bool ok = col_ok && (unsigned)(iy0 + r) < (unsigned)p.H;
        const unsigned m = ok ? 0xffffffffu : 0u;
        roff[r] = ((unsigned)((iy0 + r) * p.W + ix) * 4u & m) | ((unsigned)OOB_OFFSET & ~m);
    }
    auto load_input = [&](int g) {
#pragma unroll
        for (int r = 0; r < 4; ++r)   // (the whole offset goes through the range-checked vector operand)
            xin[g][r] = __builtin_bit_cast(f2_t, __builtin_amdgcn_raw_buffer_load_b64(
                in_rsrc, (int)(roff[r] + base + (unsigned)(4 * g) * chan_bytes), 0, 0));
    };
#pragma unroll
    for (int g = 0; g < NOW; ++g) {
        if (g > 0) load_weights(g);
        load_input(g);
        __builtin_amdgcn_sched_barrier(0);   // requests in the order the MFMAs consume them
    }
    __builtin_amdgcn_sched_barrier(0);
    TDC_STAMP(1);   // every request issued

    f4_t acc[16];
#pragma unroll
    for (int x = 0; x < 16; ++x) acc[x] = (f4_t){0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int g = 0; g < CG; ++g) {
        // rows of B^T d on both words of the pair (B^T = [1 0 -1 0; 0 1 1 0; 0 -1 1 0; 0 1 0 -1])
        f2_t t[4];
        t[0] = xin[g][0] - xin[g][2];
        t[1] = xin[g][1] + xin[g][2];
        t[2] = xin[g][2] - xin[g][1];
        t[3] = xin[g][1] - xin[g][3];
        float v[16];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            // columns: d0 = second word here, d1 / d2 = the pair one lane up, d3 = first word two lanes up
            const float X = t[i][0], Y = t[i][1];
            v[i * 4 + 0] = Y - shl1(Y);            // d0 - d2
            v[i * 4 + 1] = shl1(X + Y);            // d1 + d2
            v[i * 4 + 2] = shl1(Y - X);            // d2 - d1
            v[i * 4 + 3] = shl1(X - shl1(X));      // d1 - d3
        }
#pragma unroll
        for (int x = 0; x < 16; ++x)
            acc[x] = __builtin_amdgcn_mfma_f32_16x16x4f32(u[g][x >> 2][x & 3], v[x], acc[x], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);   // group by group, as the data arrives
        if (g + NOW < CG) {                  // this group's registers are free: request the group NOW further on
            load_weights(g + NOW);
            load_input(g + NOW);
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    TDC_STAMP(4);   // MFMAs issued
    // Output transform Y = A^T M A, A^T = [1 1 1 0; 0 1 -1 -1], per accumulator register (= output channel); parked as
    // [slice][channel of the workgroup][row 0/1][32 columns]
    const int MT = 16 * p.WM;
#pragma unroll
    for (int c4 = 0; c4 < 4; ++c4) {
        float sr[4][2];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            sr[i][0] = acc[i * 4 + 0][c4] + acc[i * 4 + 1][c4] + acc[i * 4 + 2][c4];
            sr[i][1] = acc[i * 4 + 1][c4] - acc[i * 4 + 2][c4] - acc[i * 4 + 3][c4];
        }
        const int ml = wmi * 16 + 4 * k + c4;
        f2_t *dst = reinterpret_cast<f2_t *>(lds + (wki * MT + ml) * 64 + 2 * j);
        dst[0] = (f2_t){sr[0][0] + sr[1][0] + sr[2][0], sr[0][1] + sr[1][1] + sr[2][1]};
        dst[16] = (f2_t){sr[1][0] - sr[2][0] - sr[3][0], sr[1][1] - sr[2][1] - sr[3][1]};
    }
    __syncthreads();
    TDC_STAMP(5);   // everybody's partial outputs are in LDS
    const int nthreads = blockDim.x;
    const int total = MT * 32;   // pairs of pixels
    const int wstride = MT * 64;
    // wide loads and stores where the addresses allow it
    const bool vec_ok = ((reinterpret_cast<unsigned long long>(p.out) | reinterpret_cast<unsigned long long>(p.resid)) & 7ull) == 0 &&
                        ((p.out_bstride | p.resid_bstride | (long long)p.P) & 1) == 0;
    for (int idx = tid; idx < total; idx += nthreads) {
        const int ml = idx >> 5, dy = (idx >> 4) & 1, jp = idx & 15;
        const int ch = by * MT + ml;
        const int oy = 2 * tile_y + dy, ox = tile_x * 28 + 2 * jp;
        const bool ok = ch < p.N && jp < 14 && oy < p.Ho && ox < p.Wo;
        const long long o = ok ? (long long)ch * p.P + oy * p.Wo + ox : 0;
        // (bias and residual are requested before the partial sums are read and arrive under those reads)
        const float bv = p.bias ? p.bias[min(ch, p.N - 1)] : 0.0f;
        f2_t rv = (f2_t){0.0f, 0.0f};
        if (resid) {
            if (vec_ok) rv = *reinterpret_cast<const f2_t *>(resid + o);
            else rv = (f2_t){resid[o], resid[o + (ok ? 1 : 0)]};
        }
        const f2_t *src = reinterpret_cast<const f2_t *>(lds + ml * 64 + dy * 32 + 2 * jp);
        f2_t val = (f2_t){0.0f, 0.0f};
        // four reads in flight at a time; the additions stay in slice order
        for (int w0 = 0; w0 < p.WK; w0 += 4) {
            f2_t part[4];
#pragma unroll
            for (int s = 0; s < 4; ++s) part[s] = src[(min(w0 + s, p.WK - 1) * wstride) >> 1];
#pragma unroll
            for (int s = 0; s < 4; ++s)
                if (w0 + s < p.WK) val += part[s];
        }
        if (ok) {
            val += bv;
            val += rv;
            if (p.relu) {
                val[0] = fmaxf(val[0], 0.0f);
                val[1] = fmaxf(val[1], 0.0f);
            }
            if (vec_ok) store_out(out + o, val);
            else {
                store_out(out + o, val[0]);
                store_out(out + o + 1, val[1]);
            }
        }
    }
    TDC_STAMP(6);   // stores issued
    TDC_STAMP_FLUSH(p, logical, wave, lane);
}

// ---------------------------------------------------------------------------
// Instantiation table: KernelId{STREAM_WINO, {CG, MAXW}} -> function, all built for 16 waves per workgroup (128 registers
// per lane).
// ---------------------------------------------------------------------------
typedef void (*kernel_fn)(const ConvKParams);

const void *wino_stream_kernel_function(const KernelId &k) {
    kernel_fn fn = nullptr;
    if (k.family == KernelId::STREAM_WINO) {
        const int cg = k.p[0], maxw = k.p[1];
        if (cg == 1 && maxw == 16) fn = tdc_wino3x3_stream_kernel<1, 16>;
        if (cg == 2 && maxw == 16) fn = tdc_wino3x3_stream_kernel<2, 16>;
        if (cg == 3 && maxw == 16) fn = tdc_wino3x3_stream_kernel<3, 16>;
        if (cg == 4 && maxw == 16) fn = tdc_wino3x3_stream_kernel<4, 16>;
    }
    return reinterpret_cast<const void *>(fn);
}

}  // namespace tdc
