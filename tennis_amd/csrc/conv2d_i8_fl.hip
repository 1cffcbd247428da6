// Flat-tile int8 convolution for layers with more than one tap whose whole-row window fits LDS (the 3x3
// body of ResNet-like networks and BASELINE config 2).  Same arithmetic, staged input, packed weights,
// window-in-LDS data movement and epilogue as the window-stationary kernel in conv2d_i8_ws.hip (exact int32
// sums of cpu::Conv2DQuantizedCore, src/kernels/cpu/quantized/conv2d_quantized_core.cpp:18-147); what
// differs is how output positions are dealt to workgroups:
//   * positions are the flat list (n, oh, ow) over the whole batch, cut into tiles of F consecutive
//     32-position fragments wherever rows and images happen to end -- no fragment is padded, whatever the
//     map's width (28 x 28: 784 positions = 24.5 fragments per image, 784 per batch of 32).  The window is the
//     run of staged rows from the tile's first output row to its last (plus the taps' reach and the halo rows
//     between two images); a fragment's 32 positions of one channel are 128 contiguous output bytes;
//   * a workgroup is 8 wavefronts on 128 output channels: wavefronts 0-3 take the tile's first NTA
//     fragments, 4-7 the other NTB, one of each kind per SIMD.  One workgroup per CU, so placement is known:
//     F = NTA + NTB fragment-channel blocks per SIMD.  With NTA = NTB + 1 the short wavefronts store their
//     output while the long ones run their last fragment's share of K;
//   * tiles are numbered so that each XCD (own L2) gets a contiguous run of them: neighbouring tiles share
//     halo rows, and the weights are fetched once per XCD.
#include "conv2d_i8_fl_kernel.hpp"

#include <cstdlib>
#include <cstring>

#include <atomic>


namespace tsx {

void fl_plan(const WsGeom &g, WsPlan *pl) {
    pl->flat = false;
    if (!pl->ok || g.gemm || g.kh * g.kw <= 1 || pl->wm != 4) return;
    // TSX_CONV_I8_FLAT, read at every plan: "0" keeps every layer on the window-stationary kernel; "force" takes
    // this kernel wherever the geometry allows, whatever the cost model says, with the largest tile that fits (tests
    // of the kernel on small layers); "forceNM" the same with tiles of N + M fragments only
    const char *e = std::getenv("TSX_CONV_I8_FLAT");
    if (e && e[0] == '0') return;
    const bool force = e && e[0] == 'f';
    const int only = force && std::strlen(e) == 7 ? (e[5] - '0') * 10 + (e[6] - '0') : 0;
    const int64_t positions = int64_t(g.n) * g.ho * g.wo;
    if (positions >= (int64_t(1) << 31) - 256) return;
    if (pl->packed_bytes >= (size_t(1) << 31)) return;   // the kernel addresses the weights with 32-bit offsets
    const int wrap = g.hs - g.ho * g.sh;
    const int wc = (g.wo - 1) * g.sw + (g.kw - 1) * g.dil_w + 1;
    if (wc > g.ws) return;
    // Measured against the window-stationary kernel, the flat tiles pay on large layers that fill most of the
    // chip with tiles of 6 to 8 fragments in one round (BASELINE config 2: 24.9 -> 23.4 us; the large 3x3
    // layers of the YOLOv4-shaped network); small maps (ResNet's 14x14 and 7x7 layers, under 200 workgroups of
    // short tiles) run 1-20 % slower on it and stay where they were.  The smaller splits remain instantiated
    // for the planner to use once that changes.
    // (the first three are the planner's; the smaller ones are instantiated for layers forced onto this kernel)
    static const int splits[7][2] = {{3, 3}, {4, 3}, {4, 4}, {3, 2}, {2, 2}, {2, 1}, {1, 1}};
    // One workgroup per CU: the busiest CU's time, in units of one fragment x 32 channels on one SIMD, is
    //     rounds x (fixed + F)
    // -- the same form as the window-stationary plan's model, whose workgroups pair up on a CU.
    double best = -1;
    for (int si = 0; si < (force ? 7 : 3); ++si) {
        const int *s = splits[si];
        if (only && s[0] * 10 + s[1] != only) continue;
        const int f = s[0] + s[1];
        // rows between a tile's first and last position, and image ends in between (worst tile)
        const int dr = (f * 32) % g.wo == 0 ? f * 32 / g.wo - 1 : (f * 32 + g.wo - 2) / g.wo;
        const int crossings = (dr + g.ho - 1) / g.ho;
        const int wr = dr * g.sh + (wrap > 0 ? wrap * crossings : 0) + (g.kh - 1) * g.dil_h + 1;
        const int wp = wr * wc;
        // LDS bytes per window row.  A fragment's 32 consecutive positions are consecutive window pixels (80 bytes
        // apart: any 16 of them fall into distinct banks) except where an output row ends and the next position
        // sits wc - wo + 1 pixels further: the row pitch is padded so that the first pixel of the next row lands
        // on the banks the pixel behind the row's last would have used (pitch = wo * sw * 80 modulo 256), and
        // the reads of a fragment that spans two rows stay conflict-free.
        int rowp = wc * FL_PIX;
        rowp += ((g.wo * g.sw * FL_PIX - rowp) % 256 + 256) % 256;
        if (wp > FL_MAX_WP || size_t(2) * wr * rowp > size_t(FL_MAX_LDS)) continue;
        const int64_t tiles = (positions + f * 32 - 1) / (f * 32);
        const int64_t wgs = tiles * (pl->coutp / 128);
        if (wgs < 160 && !force) continue;
        // forced: the largest tile that fits
        const double cost = force ? double(16 - f) : double((wgs + 255) / 256) * (0.75 + f);
        if (best < 0 || cost < best) {
            best = cost;
            pl->fl_nta = s[0];
            pl->fl_ntb = s[1];
            pl->fl_wr = wr;
            pl->fl_wc = wc;
            pl->fl_wp = wp;
            pl->fl_tiles = tiles;
            // every channel block's window in LDS at once where they fit: no barrier in the K loop
            pl->fl_rowp = rowp;
            pl->fl_resident = size_t(g.cblocks) * wr * rowp <= size_t(FL_MAX_LDS);
        }
    }
    if (best < 0) return;
    // the window-stationary plan's cost in the same units: its 4-wavefront workgroups sit two to a CU
    const int64_t ws_wgs = pl->tiles * (pl->coutp / 128);
    const double ws_cost = double((ws_wgs + 511) / 512) * 2 * (0.5 + pl->nt * (pl->nt > 4 ? 1.45 : 1.0));
    if (best <= ws_cost || force) pl->flat = true;
}

int fl_launch(const WsGeom &g, const WsPlan &pl, const int8_t *xs, const int8_t *packed, const EpiParams &ep,
              hipStream_t stream) {
    FlParams p{};
    static_cast<EpiParams &>(p) = ep;
    p.xs = xs;
    p.wp = packed;
    p.n = g.n;
    p.cout = g.cout;
    p.coutp = pl.coutp;
    p.ho = g.ho;
    p.wo = g.wo;
    p.hs = g.hs;
    p.ws = g.ws;
    p.cp = g.cp;
    p.cblocks = g.cblocks;
    p.kh = g.kh;
    p.kw = g.kw;
    p.sh = g.sh;
    p.sw = g.sw;
    p.frags = pl.fl_nta + pl.fl_ntb;
    p.wc = pl.fl_wc;
    p.wpix = pl.fl_wp;
    p.wr = pl.fl_wr;
    p.rowp = pl.fl_rowp;
    p.ksteps_p = pl.ksteps_p;
    p.ksteps = g.cblocks * g.kh * g.kw;
    p.tap_row = g.dil_h * pl.fl_rowp;
    p.tap_col = g.dil_w * FL_PIX;
    p.tiles = int(pl.fl_tiles);
    p.tiles_per_xcd = int((pl.fl_tiles + 7) / 8);
    p.positions = int(int64_t(g.n) * g.ho * g.wo);
    p.resident = pl.fl_resident ? 1 : 0;
    p.wc_magic = div_magic(p.wc, FL_MAX_WP);
    p.wo_magic = div_magic(p.wo, p.positions);
    p.ho_magic = div_magic(p.ho, int64_t(g.n) * g.ho);
    p.howo_magic = div_magic(p.ho * p.wo, p.positions);
    // an output of L2 size or more that no fused consumer reads: stream it
    p.stream_out = (!ep.residual && !ep.st_out && ep.out_f32 && int64_t(g.n) * g.cout * g.ho * g.wo * 4 >= (int64_t(16) << 20)) ? 1 : 0;
    const dim3 grid(unsigned(p.tiles_per_xcd * 8), unsigned((g.cout + 127) / 128));
    const size_t lds_bytes = size_t(pl.fl_resident ? g.cblocks : 2) * pl.fl_wr * pl.fl_rowp;
    const int key = pl.fl_nta * 10 + pl.fl_ntb;
    switch (key) {
        case 11: return fl_launch_nt<1, 1>(p, grid, lds_bytes, stream);
        case 21: return fl_launch_nt<2, 1>(p, grid, lds_bytes, stream);
        case 22: return fl_launch_nt<2, 2>(p, grid, lds_bytes, stream);
        case 32: return fl_launch_nt<3, 2>(p, grid, lds_bytes, stream);
        case 33: return fl_launch_nt<3, 3>(p, grid, lds_bytes, stream);
        case 43: return fl_launch_nt<4, 3>(p, grid, lds_bytes, stream);
        case 44: return fl_launch_nt<4, 4>(p, grid, lds_bytes, stream);
    }
    return fail(TSX_E_INVALID, "conv_i8_fl: unsupported fragment split %d+%d", pl.fl_nta, pl.fl_ntb);
}

}  // namespace tsx
