// Window-stationary int8 convolution (the 3x3 body of ResNet-like nets and BASELINE config 2; any
// stride, maps of any width through column tiles) on v_mfma_i32_32x32x32_i8
// (the 16x16x64 form runs at half the rate on this part).
//
// Same arithmetic as the generic implicit GEMM in conv2d_i8.hip (exact int32 sums of
// cpu::Conv2DQuantizedCore, src/kernels/cpu/quantized/conv2d_quantized_core.cpp:18-147), but
// a different data movement:
//   * one workgroup (4 wavefronts) owns a tile of TH output rows x TW output columns x 128 output
//     channels; wavefront w owns channels [32w, 32w+32) and all positions of the tile (layers with
//     at most 64 / 32 output channels: 64 / 32 channels, the other wavefronts taking further
//     positions of a 2x / 4x larger tile).  Rows are counted across the whole batch (image n's rows
//     follow image n-1's), so a tile may straddle two images: their staged rows are contiguous in
//     memory, and a position in the second image just reads the window hs - ho*stride rows further
//     down.  Tiles therefore need not divide the image height.  TW is the whole row where the row
//     and its window fit, else a multiple of 32 columns.  A 1x1 layer reading a buffer without halo
//     is tiled as rows of one pixel (the plan's view of the map): any run of consecutive pixels;
//   * per 64-channel block the input *window* that all KH*KW taps of the tile read
//     (((TH-1)*stride + (KH-1)*dil + 1) rows x ((TW-1)*stride + (KW-1)*dil + 1) columns) is copied
//     once into LDS (double buffered, one block ahead, 80-byte pixel stride = bank-conflict-free
//     16-byte reads); every tap is then a shifted read of the same LDS data, so activations cross
//     L2 -> CU once, not KH*KW times, and the K loop needs one barrier per channel block, not per
//     K-step.  A 1x1 layer has one K-step per channel block, too short to cover the window's L2
//     latency one block ahead: its windows hold up to 4 channel blocks per pixel (pixel stride
//     64*blocks + 16) and the blocks of a window are walked like taps;
//   * weights never touch LDS: each wavefront streams its own rows from the packed
//     buffer (1 KiB contiguous per MFMA operand) into a 4-deep register ring, three
//     K-steps ahead of use.
// K order is (channel block, kh, kw); K-steps are padded with zero weights to a multiple
// of the ring depth.
//
// MFMA operand layout (v_mfma_i32_32x32x32_i8): lane l supplies row/column l%32 and the 16
// K bytes of group l/32 (two MFMAs, "halves", cover a 64-byte K-step); accumulator register r
// of lane l is row 8*(r/4) + 4*(l/32) + r%4, column l%32.  Rows = cout, columns = positions.
#include "conv2d_i8_ws_kernel.hpp"

#include <algorithm>

namespace tsx {
namespace {

// packed[ks][frag][half][lane][16]: ks = cb*taps + tap; frag = cout/32; lane l: cout frag*32 + l%32,
// channels cb*64 + half*32 + (l/32)*16 + 0..15.  K-steps >= cblocks*taps, rows >= cout, channels >= c: zero.
__global__ __launch_bounds__(256) void ws_pack_kernel(const int8_t *__restrict__ w, int cout, int c, int taps,
                                                     int cblocks, int ksteps_p, int coutp,
                                                     int8_t *__restrict__ packed) {
    const int frags = coutp / 32;
    const int64_t total = int64_t(ksteps_p) * frags * 2 * 64;
    const int64_t id = int64_t(blockIdx.x) * blockDim.x + threadIdx.x;
    if (id >= total) return;
    const int lane = int(id % 64);
    const int half = int((id / 64) % 2);
    const int frag = int((id / 128) % frags);
    const int ks = int(id / 128 / frags);
    const int cb = ks / taps, tap = ks % taps;
    const int co = frag * 32 + lane % 32;
    const int c0 = cb * 64 + half * 32 + (lane / 32) * 16;
    uint32_t words[4] = {0, 0, 0, 0};
    if (co < cout && cb < cblocks) {
#pragma unroll
        for (int j = 0; j < 16; ++j) {
            const int ci = c0 + j;
            const int v = ci < c ? w[(int64_t(co) * c + ci) * taps + tap] : 0;
            words[j / 4] |= uint32_t(v & 0xff) << (8 * (j % 4));
        }
    }
    *reinterpret_cast<uint4 *>(packed + id * 16) = make_uint4(words[0], words[1], words[2], words[3]);
}


}  // namespace

WsPlan ws_plan(const WsGeom &g_in) {
    WsPlan pl{};
    pl.ok = false;
    // A 1x1 layer reading a buffer without halo is a plain [positions][channels] matrix: rows mean nothing,
    // so it is tiled as rows of ONE pixel (ho*wo of them per image) -- a tile is then any number of
    // consecutive pixels, chosen below as whole fragments whatever the map's width (3136 = 56x56 positions
    // per image give 128-position tiles with no padding; a 608-wide map is no obstacle).
    WsGeom g = g_in;
    if (g.kh == 1 && g.kw == 1 && g.hs == g.ho && g.ws == g.wo && int64_t(g.n) * g.ho * g.wo < (int64_t(1) << 31)) {
        g.ho = g.hs = g_in.ho * g_in.wo;
        g.wo = g.ws = 1;
    }
    pl.ho = g.ho;
    pl.wo = g.wo;
    pl.hs = g.hs;
    pl.ws = g.ws;
    // A tile is TH output rows of the batch-wide row sequence x TW output columns (whole rows when they fit),
    // at most MAX_NT fragments of 32 positions per wavefront.  Candidates are ranked by a model of the busiest
    // CU's time in units of one fragment's work,
    //     (rounds of resident workgroups) x (overlap factor) x (0.5 + fragments x slow),
    // where 0.5 is the per-workgroup fixed cost and slow = 1.45 for tiles of more than 4 fragments
    // (one workgroup per CU, so one wavefront per SIMD with nothing to hide its LDS/L2 waits).  The
    // constants come from a sweep over 32x256x28x28 (1/2/4/8-row tiles: 35 / 30.5 / 23.0 / 23.4 us) and the
    // layers of a ResNet-50-shaped network, whose small maps want many small workgroups: 196 workgroups of 4
    // fragments per wavefront (60 CUs idle) take 11.7 us on 32x512x28x28 -> 128 channels, 392 of 2 take 9.4.
    // Ties go to the fewest total fragments (least padding).
    constexpr int MAX_NT = 7;
    // few output channels: fewer wavefronts along cout, the others take more positions of a larger tile
    const int wm = g.cout <= 32 ? 1 : g.cout <= 64 ? 2 : 4, wn = 4 / wm;
    const int cap = 32 * MAX_NT * wn;
    if (g.wo < 1 || g.sh < 1 || g.sw < 1) return pl;
    const int wrap = g.hs - g.ho * g.sh;
    const int bm = 32 * WS_FM * wm;
    // GEMM weights are packed once for every kernel that may read them: rows padded to 128
    const int coutp = g.gemm ? (g.cout + 127) / 128 * 128 : (g.cout + bm - 1) / bm * bm;
    const int ksteps_p = (g.cblocks * g.kh * g.kw + RING - 1) / RING * RING;
    double best_cost = -1;
    int64_t best_frags = 0;
    // tile widths: the whole row where it (and its window) fits, else multiples of 32 columns (a fragment is
    // then one run of a row)
    const bool tiny_k = g.cblocks * g.kh * g.kw <= 2;
    auto consider = [&](int tw) {
        const int ctiles = (g.wo + tw - 1) / tw;
        const int wc = (tw - 1) * g.sw + (g.kw - 1) * g.dil_w + 1;
        for (int t = 1; t <= g.ho && t * tw <= cap; ++t) {
            const int nt = ((t * tw + 31) / 32 + wn - 1) / wn;   // fragments per wavefront
            const int64_t tiles = (int64_t(g.n) * g.ho + t - 1) / t * ctiles;
            const bool straddle = g.ho % t != 0;
            const int wr = (t - 1) * g.sh + (g.kh - 1) * g.dil_h + 1 + (straddle && wrap > 0 ? wrap : 0);
            const int wp = wr * wc;
            if (wp > MAX_WP || size_t(2) * wp * PIX > 65536) continue;   // two windows must fit 64 KiB of LDS
            const int64_t wgs = tiles * (coutp / bm);
            const int64_t frags = tiles * nt * wn;
            // workgroups of up to 2 fragments per wavefront fit three to a CU, up to 4 two, larger ones one; those
            // resident together overlap (each further one adds about half of a lone workgroup's time), the rest
            // run in rounds -- so a layer that leaves CUs idle with large tiles takes tiles of half the size
            const int64_t per_cu = (wgs + 255) / 256;
            const int resident = nt <= 2 ? 3 : nt <= 4 ? 2 : 1;
            const int64_t rounds = (per_cu + resident - 1) / resident;
            const double together = 1.0 + 0.5 * double(std::min<int64_t>(per_cu, resident) - 1);
            const double cost = double(rounds) * together * (0.5 + nt * (nt > 4 ? 1.45 : 1.0));
            // One or two K-steps (a 1x1 layer on 64 or 128 channels): the workgroup is all epilogue, its time is the
            // store traffic of its tile, and what pays is many small workgroups in flight per CU -- measured on
            // 32x64x56x56 -> 256 channels: 63 us with 4 fragments per wavefront and a residual join, 55 us with 2.
            if (tiny_k && nt > 2) continue;
            if (best_cost < 0 || cost < best_cost || (cost == best_cost && frags < best_frags)) {
                best_cost = cost;
                best_frags = frags;
                pl.th = t;
                pl.tw = tw;
                pl.ctiles = ctiles;
                pl.nt = nt;
                pl.tiles = tiles;
                pl.wr = wr;
                pl.wc = wc;
                pl.wp = wp;
            }
        }
    };
    if (g.wo <= cap) consider(g.wo);
    if (best_cost < 0)
        for (int tw = 32; tw <= cap && tw < g.wo; tw += 32) consider(tw);
    if (best_cost < 0 || pl.tiles >= (int64_t(1) << 31)) return pl;
    pl.wm = wm;
    // 1x1 layers: as many channel blocks per window as divide the layer's, fit the fill registers and LDS
    pl.cbs = 1;
    if (g.kh == 1 && g.kw == 1)
        for (int c = 4; c > 1; c >>= 1)
            if (g.cblocks % c == 0 && pl.wp * 4 * c <= MAX_FILL * WS_THREADS && size_t(2) * pl.wp * (64 * c + 16) <= 65536) {
                pl.cbs = c;
                break;
            }
    pl.ksteps_p = ksteps_p;
    pl.coutp = coutp;
    pl.packed_bytes = size_t(pl.ksteps_p) * pl.coutp * 64;
    pl.ok = true;
    fl_plan(g_in, &pl);   // layers the flat-tile kernel suits better (same packed weights)
    rs_plan(g_in, &pl);   // ... and the weight-stationary one
    return pl;
}

int ws_pack_weights(const WsGeom &g, const WsPlan &pl, const int8_t *w_oihw, int c, int8_t *packed, hipStream_t stream) {
    const int64_t threads = int64_t(pl.packed_bytes / 16);
    hipLaunchKernelGGL(ws_pack_kernel, dim3(unsigned(ceil_div(threads, 256))), dim3(256), 0, stream, w_oihw, g.cout, c,
                       g.kh * g.kw, g.cblocks, pl.ksteps_p, pl.coutp, packed);
    TSX_LAUNCH_CHECK("ws_pack_kernel");
    return 0;
}

int ws_launch(const WsGeom &g, const WsPlan &pl, const int8_t *xs, const int8_t *packed, const EpiParams &ep,
              hipStream_t stream) {
    if (rs_takes(pl, ep, int64_t(g.n) * g.cout * g.ho * g.wo)) return rs_launch(g, pl, xs, packed, ep, stream);
    if (pl.flat) return fl_launch(g, pl, xs, packed, ep, stream);
    WsParams p{};
    static_cast<EpiParams &>(p) = ep;
    p.xs = xs;
    p.wp = packed;
    p.n = g.n;
    p.cout = g.cout;
    p.coutp = pl.coutp;
    p.ho = pl.ho;   // the plan's view of the map (1-pixel rows for 1x1 layers)
    p.wo = pl.wo;
    p.hs = pl.hs;
    p.ws = pl.ws;
    p.cp = g.cp;
    p.cblocks = g.cblocks;
    p.kh = g.kh;
    p.kw = g.kw;
    p.dil_h = g.dil_h;
    p.dil_w = g.dil_w;
    p.th = pl.th;
    p.wr = pl.wr;
    p.wc = pl.wc;
    p.wpix = pl.wp;
    p.ksteps_p = pl.ksteps_p;
    p.ksteps = g.cblocks * g.kh * g.kw;
    p.wm = pl.wm;
    p.tw = pl.tw;
    p.ctiles = pl.ctiles;
    p.sh = g.sh;
    p.sw = g.sw;
    p.pix = 64 * pl.cbs + 16;
    p.chunk_shift = pl.cbs == 4 ? 4 : pl.cbs == 2 ? 3 : 2;
    p.stage_bytes = 64 * pl.cbs;
    p.tap_row = g.dil_h * pl.wc * p.pix;
    p.tap_col = g.dil_w * p.pix;
    if (pl.cbs > 1) {          // the blocks of a window take the place of taps
        p.cblocks = g.cblocks / pl.cbs;
        p.kh = 1;
        p.kw = pl.cbs;
        p.tap_row = 0;
        p.tap_col = 64;
    }
    // an output of L2 size or more that no fused consumer reads: stream it
    p.stream_out = (!ep.residual && !ep.st_out && ep.out_f32 && int64_t(g.n) * g.cout * g.ho * g.wo * 4 >= (int64_t(16) << 20)) ? 1 : 0;
    p.rowmajor = g.gemm ? 1 : 0;
    if (g.gemm) p.stream_out = 0;
    p.wc_magic = div_magic(p.wc, MAX_WP);
    p.tw_magic = div_magic(p.tw, 4 * 7 * 32);
    p.ow_magic = div_magic(ep.o_w, int64_t(p.ho) * p.wo);
    const int bm = 32 * WS_FM * pl.wm;
    const dim3 grid(unsigned(pl.tiles), unsigned((g.cout + bm - 1) / bm));
    // two window buffers (one channel block ahead); a layer whose channels fit one window never swaps and takes one:
    // more workgroups per CU where the window is large (stride-2 3x3 layers on 32 or 64 channels)
    const size_t lds_bytes = size_t(p.cblocks > 1 ? 2 : 1) * pl.wp * (64 * pl.cbs + 16);
    switch (pl.nt) {
        case 1: return ws_launch_nt<1>(p, grid, lds_bytes, stream);
        case 2: return ws_launch_nt<2>(p, grid, lds_bytes, stream);
        case 3: return ws_launch_nt<3>(p, grid, lds_bytes, stream);
        case 4: return ws_launch_nt<4>(p, grid, lds_bytes, stream);
        case 5: return ws_launch_nt<5>(p, grid, lds_bytes, stream);
        case 6: return ws_launch_nt<6>(p, grid, lds_bytes, stream);
        case 7: return ws_launch_nt<7>(p, grid, lds_bytes, stream);
    }
    return fail(TSX_E_INVALID, "conv_i8_ws: unsupported fragment count %d", pl.nt);
}

}  // namespace tsx
