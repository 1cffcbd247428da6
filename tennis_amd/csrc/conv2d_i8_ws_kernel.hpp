// The window-stationary int8 convolution kernel itself (see conv2d_i8_ws.hip for the data movement it
// implements).  Included by one translation unit per fragment count NT, each of which defines
// TSX_WS_NT and gets the specialisation ws_launch_nt<TSX_WS_NT>: the kernel is fully unrolled over its
// fragments, so compiling the seven counts side by side is what keeps the build time down.
#pragma once
#include "igemm_i8.hpp"

namespace tsx {

constexpr int RING = 4;         // A register ring depth (K-steps)
constexpr int PIX = 80;         // LDS bytes per window pixel (64 + 16 pad) when a window holds one channel block
constexpr int WS_THREADS = 256;
constexpr int WS_FM = 1;        // 32-cout fragments per wavefront
constexpr int MAX_FILL = 7;     // window chunks per thread per channel block
constexpr int SMALL_FILL = 4;   // ... of the kernels compiled for small windows (fewer registers: one more workgroup per CU)
constexpr int MAX_WP = MAX_FILL * WS_THREADS / 4;   // 448 window pixels

struct WsParams : EpiParams {
    const int8_t *xs;   // staged activations [n][hs][ws][cp]
    const int8_t *wp;   // packed weights [ks_p][coutp/32][2 halves][64 lanes][16]
    int n, cout, coutp, ho, wo, hs, ws, cp, cblocks, kh, kw, dil_h, dil_w;
    int th, wr, wc, wpix, ksteps_p;
    int ksteps;       // K-steps that hold weights (ksteps_p: padded to the A-ring size with zero steps)
    int wm;           // wavefronts along cout (4, 2 or 1: the other factor of 4 splits the tile's positions)
    int tw, ctiles;   // tile width in output columns, column tiles per row (1: whole rows)
    int sh, sw;       // strides
    // a window holds `cbs` channel blocks per pixel: pix = 64*cbs + 16 bytes, 4*cbs = 1 << chunk_shift chunks;
    // a tap is tap_row/tap_col bytes further into the window per kernel row / column (for cbs > 1 the "taps"
    // are the window's channel blocks: kh = 1, kw = cbs, tap_col = 64)
    int pix, chunk_shift, stage_bytes, tap_row, tap_col;
    int stream_out;   // fp32 output written with streaming stores
    int rowmajor;     // GEMM: output index position * cout + channel, row_scale[position] applied behind dq
    // per-lane divisions by uniform divisors as one multiply-high (div_magic / udiv)
    unsigned wc_magic, tw_magic, ow_magic;
};


// One specialisation per fragment count, each defined by its own translation unit.
template <int NT>
int ws_launch_nt(const WsParams &p, dim3 grid, size_t lds_bytes, hipStream_t stream);
template <> int ws_launch_nt<1>(const WsParams &, dim3, size_t, hipStream_t);
template <> int ws_launch_nt<2>(const WsParams &, dim3, size_t, hipStream_t);
template <> int ws_launch_nt<3>(const WsParams &, dim3, size_t, hipStream_t);
template <> int ws_launch_nt<4>(const WsParams &, dim3, size_t, hipStream_t);
template <> int ws_launch_nt<5>(const WsParams &, dim3, size_t, hipStream_t);
template <> int ws_launch_nt<6>(const WsParams &, dim3, size_t, hipStream_t);
template <> int ws_launch_nt<7>(const WsParams &, dim3, size_t, hipStream_t);

#ifdef TSX_WS_NT
namespace {

// EXTRA = false compiles the residual input and the staged-layout output out of the epilogue (fewer
// registers for the plain dequant + bias + activation case); STREAM selects streaming fp32 stores.
//
// Up to 4 position fragments the kernel is compiled for two wavefronts per SIMD (at most 256 registers): the
// layers that take these tiles are bound by their epilogue's memory traffic (residual in, fp32 and staged int8
// out), and a second resident workgroup per CU is worth more there than registers.
// NT counts the position fragments of ONE wavefront; a tile holds (4 / wm) x NT of them.
//
// ROWM = true is the GEMM form (a 1x1 layer over one "image" of m one-pixel rows): the output is
// [position][cout] row-major, and row_scale[position] multiplies behind dq (the per-row activation scale of a
// quantized inner product).  A lane's accumulators 4g..4g+3 are 4 consecutive channels of its position, so
// the fp32 output goes out as 16-byte stores; lanes l and l+32 and the four g complete a 128-byte line.
//
// FILL = chunks of 16 window bytes a thread copies per channel block (MAX_FILL, or SMALL_FILL for windows that need
// no more: with up to 2 fragments the kernel then fits four wavefronts per SIMD, and the layers bound by their
// epilogue's memory latency -- the residual joins on large maps -- keep a fourth workgroup in flight per CU).
//
// LOOK: the B operands go through a register ring as deep as the weights', read RING - 1 K-steps ahead of their
// MFMAs.  A wavefront with one fragment spends 2 MFMAs (64 cycles) on a K-step, half of an LDS read's latency: read
// one half-step ahead (the other form), the small maps at the end of a network -- under one wavefront per SIMD,
// nothing else to issue -- ran at one K-step per two LDS latencies.
template <int NT, int FM, bool EXTRA, bool STREAM, bool ROWM, int FILL, bool LOOK, bool MISHX = false>
__global__ __launch_bounds__(WS_THREADS) __attribute__((amdgpu_waves_per_eu(NT <= 4 ? 2 : 1))) void conv_i8_ws_kernel(WsParams p_in) {
    WsParams p = p_in;
    if (!EXTRA) {
        p.residual = nullptr;
        p.st_out = nullptr;
    }
    if (!ROWM) p.row_scale = nullptr;
    extern __shared__ __attribute__((aligned(16))) int8_t lds[];   // 2 x wpix x PIX
    // the wavefront's index as a scalar: what derives from it (first cout, tile bases, the choice of epilogue path)
    // then stays in scalar registers and branches uniformly
    const int tid = threadIdx.x, lane = tid % 64, wave = __builtin_amdgcn_readfirstlane(tid / 64);
    const int rtile = blockIdx.x / p.ctiles;
    const int col0 = (blockIdx.x - rtile * p.ctiles) * p.tw;   // first output column of the tile
    const int row0 = rtile * p.th;           // first output row of the tile, counted over the whole batch
    const int img = row0 / p.ho;             // image of the tile's first row
    const int th0 = row0 - img * p.ho;       // ... and that row inside it
    const int rows_total = p.n * p.ho;
    // staged rows from where output row `ho` of an image would start to the next image's first row
    const int wrap = p.hs - p.ho * p.sh;
    const int wave_m = wave & (p.wm - 1);                            // position along cout
    const int pos0 = (p.wm == 4 ? 0 : p.wm == 2 ? wave >> 1 : wave) * (NT * 32);   // first tile position of this wavefront
    const int m0 = (blockIdx.y * p.wm + wave_m) * (32 * FM);         // first cout of this wavefront
    const int taps = p.kh * p.kw;
    const int win_bytes = p.wpix * p.pix;

    // ---- window fill bookkeeping: chunk q = tid + i*256 -> pixel q / chunks-per-pixel, 16-byte chunk q % ...
    // A uniform 64-bit base (the window's first staged row and column) plus one 32-bit byte offset per chunk: the
    // loads then take the base from scalar registers and need no address arithmetic of their own.
    const int n_fill = ((p.wpix << p.chunk_shift) + WS_THREADS - 1) / WS_THREADS;   // <= FILL, uniform
    // window row r is staged row (img * hs + th0 * stride) + r of the batch-wide staged row sequence
    const int64_t row_base = int64_t(img) * p.hs + th0 * p.sh;
    const int col_base = col0 * p.sw;
    const int row_last = int(min(int64_t(p.n) * p.hs - 1 - row_base, int64_t(1) << 20));   // last tile: rows no stored output uses
    const int col_last = p.ws - 1 - col_base;                                               // last column tile: likewise
    const int8_t *xs_base = p.xs + (row_base * p.ws + col_base) * p.cp;
    unsigned fill_off[FILL];
    int fill_dst[FILL];
    static_for<0, FILL>([&](auto ic) {
        constexpr int i = decltype(ic)::value;
        fill_off[i] = 0;
        fill_dst[i] = 0;
        if (i < n_fill) {
            const int q = tid + i * WS_THREADS;
            int pix = q >> p.chunk_shift;
            const int chunk = q & ((1 << p.chunk_shift) - 1);
            if (pix >= p.wpix) pix = p.wpix - 1;   // duplicates rewrite the same bytes
            const int wrow = udiv(pix, p.wc, p.wc_magic);
            const int wcol = pix - __mul24(wrow, p.wc);
            // 24-bit multiplies (full rate): window rows, staged widths and pixel sizes are far below 2^24
            fill_off[i] = unsigned(__mul24(__mul24(min(wrow, row_last), p.ws) + min(wcol, col_last), p.cp) + chunk * 16);
            fill_dst[i] = __mul24(pix, p.pix) + chunk * 16;
        }
    });
    v4i wreg[FILL];   // native vectors: arrays of HIP's uint4 struct do not stay in registers

    auto window_load = [&](int cb) __attribute__((always_inline)) {
        const int8_t *base = xs_base + cb * p.stage_bytes;
        static_for<0, FILL>([&](auto ic) {
            constexpr int i = decltype(ic)::value;
            if (i < n_fill) {
                // the empty statement keeps the offset's widening next to the load, where instruction selection
                // folds it into the scalar-base addressing mode
                unsigned off = fill_off[i];
                asm volatile("" : "+v"(off));
                wreg[i] = *reinterpret_cast<const v4i *>(base + off);
            }
        });
    };
    auto window_store = [&](int buf) __attribute__((always_inline)) {
        static_for<0, FILL>([&](auto ic) {
            constexpr int i = decltype(ic)::value;
            if (i < n_fill) *reinterpret_cast<v4i *>(&lds[buf * win_bytes + fill_dst[i]]) = wreg[i];
        });
    };

    // the first window's loads leave before anything else is computed: their latency covers the rest of the set-up
    window_load(0);

    // ---- B operand addresses: fragment j, lane l -> tile position j*32 + l%32, K group l/32
    int b_base[NT];
    static_for<0, NT>([&](auto jc) {
        constexpr int j = decltype(jc)::value;
        int pos = pos0 + j * 32 + lane % 32;
        if (pos >= p.th * p.tw) pos = 0;       // padding positions: computed, never stored
        const int r = udiv(pos, p.tw, p.tw_magic), tc = pos - __mul24(r, p.tw);
        const int wrow = r * p.sh + (th0 + r >= p.ho ? wrap : 0);   // positions of the next image sit below its halo rows
        b_base[j] = __mul24(__mul24(wrow, p.wc) + __mul24(tc, p.sw), p.pix) + (lane / 32) * 16;
    });

    // ---- A ring: the wavefront's FM fragments (32 cout each) x 2 halves of K-step ks, 1 KiB each
    const int8_t *a_ptr = p.wp + (int64_t(m0 / 32) * 128 + lane) * 16;
    const int64_t a_kstride = int64_t(p.coutp / 32) * 128 * 16;
    v4i areg[RING][2 * FM];
    auto a_load = [&](auto slot, int ks) __attribute__((always_inline)) {
        constexpr int s = decltype(slot)::value;
        if (ks >= p.ksteps) ks = p.ksteps - 1;   // beyond the last K-step: its lines again, never used
        const int8_t *src = a_ptr + ks * a_kstride;
        static_for<0, 2 * FM>([&](auto fc) {
            constexpr int f = decltype(fc)::value;
            areg[s][f] = *reinterpret_cast<const v4i *>(src + f * 1024);
        });
    };

    v16i acc[FM][NT];
    static_for<0, FM>([&](auto ic) {
        static_for<0, NT>([&](auto jc) {
            static_for<0, 16>([&](auto rc) { acc[decltype(ic)::value][decltype(jc)::value][decltype(rc)::value] = 0; });
        });
    });

    // ---- prologue (the first window is on its way)
    static_for<0, RING - 1>([&](auto sc) { a_load(sc, decltype(sc)::value); });

    // ---- epilogue operands, fetched while the first window is in flight: a wavefront that meets them only behind
    // its K-loop waits a full memory latency there, with nothing else on its SIMD to hide it
    const int tile_pos = p.th * p.tw;
    const int howo = p.ho * p.wo;
    const int64_t count = int64_t(p.n) * p.cout * howo;
    // hot case: no raw accumulators wanted, every element inside the activation's SIMD-body range,
    // a tensor small enough for 32-bit lane offsets, and -- for the requantized output -- one
    // quantize group per image (or a single scale whose round-half-even bulk covers everything),
    // so the consumer's scale is uniform for this tile and needs no per-element division
    const bool want_q = p.out_i8 || p.st_out;
    const bool q_uniform = !want_q || (p.n_qscales == 1 ? p.q_bulk8 == count : p.q_group_len == int64_t(p.cout) * howo);
    // the GEMM form stores 4 consecutive channels at once, and its quantize groups are rows, not images
    const bool rowm_ok = !ROWM || (!want_q && p.cout % 4 == 0 && reinterpret_cast<uintptr_t>(p.out_f32) % 16 == 0);
    const bool fast = (p.out_f32 || want_q) && !p.out_acc && p.act_body == count && count < (int64_t(1) << 30) && q_uniform && rowm_ok;
    // a tile may end in the next image: one consumer scale per image, selected per lane
    const float q_scale_a = (fast && want_q) ? p.q_scales[p.n_qscales == 1 ? 0 : img] : 0.f;
    const float q_scale_b = (fast && want_q) ? p.q_scales[p.n_qscales == 1 ? 0 : min(img + 1, p.n - 1)] : 0.f;
    const bool q_even = p.n_qscales == 1;   // single-scale quantize rounds half to even in its bulk
    // the wavefront's dequantize scales and biases are read behind the K-loop; touching their lines now leaves them
    // in the caches by then (one load per array: 32 channels per fragment)
    float touch = 0.f;
    static_for<0, FM>([&](auto fc) {
        const int co = min(m0 + decltype(fc)::value * 32 + lane % 32, p.cout - 1);
        if (p.dq) touch += p.dq[co];
        if (p.bias) touch += p.bias[co];
    });
    asm volatile("; epilogue operands touched" ::"v"(touch));

    window_store(0);
    __syncthreads();
    int cb = 0, tap = 0, kc = 0, buf = 0;
    int cb_ks = 0;   // K-steps the B read pointer has passed (LOOK)
    // byte offset of the current tap in the LDS windows (buffer + kernel row and column), stepped with the taps: a
    // column on, or to the first column of the next kernel row
    int toff = 0;
    const int row_step = p.tap_row - (p.kw - 1) * p.tap_col;
    if (p.cblocks > 1) window_load(1);   // block cb+1, in flight during block cb's taps

    auto b_read = [&](v4i(&dst)[NT], int off) __attribute__((always_inline)) {
        static_for<0, NT>([&](auto jc) {
            constexpr int j = decltype(jc)::value;
            dst[j] = *reinterpret_cast<const v4i *>(&lds[b_base[j] + off]);
        });
    };
    int ks = 0;
    if constexpr (LOOK) {
        // ---- K-loop with the B ring: slot u holds both halves of K-step (round start + u).  The read pointer runs
        // RING - 1 K-steps ahead of the MFMAs and is the one that swaps the windows when it enters a channel block.
        v4i bq[RING][2][NT];
        auto b_ahead = [&](auto slot) __attribute__((always_inline)) {
            constexpr int sl = decltype(slot)::value;
            b_read(bq[sl][0], toff);
            b_read(bq[sl][1], toff + 32);
            ++cb_ks;
            ++tap;
            if (++kc == p.kw) {
                kc = 0;
                toff += row_step;
            } else {
                toff += p.tap_col;
            }
            if (tap == taps) {
                tap = 0;
                kc = 0;
                ++cb;
                if (cb_ks < p.ksteps) {      // no window swap behind the last K-step (reads beyond it stay where they are)
                    window_store(buf ^ 1);
                    __syncthreads();
                    buf ^= 1;
                    const int next = cb + 1 < p.cblocks ? cb + 1 : p.cblocks - 1;
                    window_load(next);
                }
                toff = buf * win_bytes;
            }
        };
        static_for<0, RING - 1>([&](auto sc) { b_ahead(sc); });
        auto k_step = [&](auto uc, auto prefetch) __attribute__((always_inline)) {
            constexpr int u = decltype(uc)::value;
            if (decltype(prefetch)::value) a_load(std::integral_constant<int, (u + RING - 1) % RING>{}, ks + RING - 1);
            b_ahead(std::integral_constant<int, (u + RING - 1) % RING>{});
            static_for<0, 2>([&](auto hc) {
                constexpr int h = decltype(hc)::value;
                static_for<0, FM>([&](auto ic) {
                    constexpr int i = decltype(ic)::value;
                    static_for<0, NT>([&](auto jc) {
                        constexpr int j = decltype(jc)::value;
                        acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(areg[u][i * 2 + h], bq[u][h][j], acc[i][j], 0, 0, 0);
                    });
                });
            });
            ++ks;
        };
        while (ks + RING <= p.ksteps) static_for<0, RING>([&](auto uc) { k_step(uc, std::true_type{}); });
        const int left = p.ksteps - ks;
        static_for<0, RING - 1>([&](auto uc) {
            if (decltype(uc)::value < left) k_step(uc, std::false_type{});
        });
    } else {
        // B fragments are read one half-step ahead of the MFMAs that use them (one wavefront per
        // SIMD: nothing else hides the LDS latency).
        v4i b0[NT], b1[NT];
        b_read(b0, toff);

        // One K-step: both halves' MFMAs, the B reads one half-step ahead, the window swap on a channel-block boundary.
        // PREFETCH: also load the weights of the K-step RING-1 ahead into the ring slot the previous step freed.
        auto k_step = [&](auto uc, auto prefetch) __attribute__((always_inline)) {
            constexpr int u = decltype(uc)::value;
            if (decltype(prefetch)::value) a_load(std::integral_constant<int, (u + RING - 1) % RING>{}, ks + RING - 1);
            b_read(b1, toff + 32);                       // second half of this K-step
            static_for<0, FM>([&](auto ic) {
                constexpr int i = decltype(ic)::value;
                static_for<0, NT>([&](auto jc) {
                    constexpr int j = decltype(jc)::value;
                    acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(areg[u][i * 2], b0[j], acc[i][j], 0, 0, 0);
                });
            });
            // advance (cb, tap); on a channel-block boundary swap in the next window (none behind the last K-step)
            ++ks;
            ++tap;
            if (++kc == p.kw) {
                kc = 0;
                toff += row_step;
            } else {
                toff += p.tap_col;
            }
            if (tap == taps) {
                tap = 0;
                kc = 0;
                ++cb;
                if (ks < p.ksteps) {
                    window_store(buf ^ 1);
                    __syncthreads();
                    buf ^= 1;
                    const int next = cb + 1 < p.cblocks ? cb + 1 : p.cblocks - 1;
                    window_load(next);
                }
                toff = buf * win_bytes;
            }
            b_read(b0, toff);                            // first half of the next K-step
            static_for<0, FM>([&](auto ic) {
                constexpr int i = decltype(ic)::value;
                static_for<0, NT>([&](auto jc) {
                    constexpr int j = decltype(jc)::value;
                    acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(areg[u][i * 2 + 1], b1[j], acc[i][j], 0, 0, 0);
                });
            });
        };
        // whole rounds of the ring, then the K-steps left over: their weights are in the ring already (the steps
        // ahead of the last round), and the zero steps that pad the packed weights to a whole round are not multiplied
        while (ks + RING <= p.ksteps) static_for<0, RING>([&](auto uc) { k_step(uc, std::true_type{}); });
        const int left = p.ksteps - ks;
        static_for<0, RING - 1>([&](auto uc) {
            if (decltype(uc)::value < left) k_step(uc, std::false_type{});
        });
    }


    // ---- epilogue: accumulator register r of lane l = cout 8*(r/4) + 4*(l/32) + r%4, position l%32
    static_for<0, FM>([&](auto fc) {
        constexpr int f = decltype(fc)::value;
        const int cf = m0 + f * 32;   // first cout of this fragment (uniform)
        // fast: all 32 channels exist, the loads need no bounds and combine into 16-byte ones
        const bool fast_f = fast && cf + 32 <= p.cout;
        // Loads without per-element branches: the fast case needs no bounds (consecutive channels combine into
        // 16-byte loads); otherwise the index is clamped, and what a channel beyond cout loads is never stored.
        float dq[16], bias[16];
        static_for<0, 16>([&](auto rc) {
            dq[decltype(rc)::value] = 0.f;
            bias[decltype(rc)::value] = 0.f;
        });
        const int co_lane = cf + 4 * (lane / 32);
        if (fast_f) {
            if (p.dq) static_for<0, 16>([&](auto rc) {
                constexpr int r = decltype(rc)::value;
                dq[r] = (p.dq + cf)[4 * (lane / 32) + 8 * (r / 4) + (r % 4)];
            });
            if (p.bias) static_for<0, 16>([&](auto rc) {
                constexpr int r = decltype(rc)::value;
                bias[r] = (p.bias + cf)[4 * (lane / 32) + 8 * (r / 4) + (r % 4)];
            });
        } else {
            if (p.dq) static_for<0, 16>([&](auto rc) {
                constexpr int r = decltype(rc)::value;
                dq[r] = p.dq[min(co_lane + 8 * (r / 4) + (r % 4), p.cout - 1)];
            });
            if (p.bias) static_for<0, 16>([&](auto rc) {
                constexpr int r = decltype(rc)::value;
                bias[r] = p.bias[min(co_lane + 8 * (r / 4) + (r % 4), p.cout - 1)];
            });
        }
        // One branch around the fragments, not one per fragment: inside it the compiler knows what is still in
        // flight, and a fragment does not wait for the stores of the one before it.
        if (fast_f) {
            // the other branch of a residual join: the loads of every fragment are in flight before the first use
            float res[NT][16];
            if (EXTRA && p.residual) {
                const int64_t tile_base = (int64_t(img) * p.cout + cf) * howo;
                static_for<0, NT>([&](auto jc) {
                    constexpr int j = decltype(jc)::value;
                    const int pos = pos0 + j * 32 + lane % 32;
                    const int tr = udiv(pos, p.tw, p.tw_magic), ow = col0 + pos - tr * p.tw;
                    const bool wrapped = th0 + tr >= p.ho;                 // this position belongs to the next image
                    const int oh = th0 + tr - (wrapped ? p.ho : 0);
                    const bool pos_ok = pos < tile_pos && row0 + tr < rows_total && ow < p.wo;
                    const unsigned lane_off = unsigned((wrapped ? p.cout * howo : 0) + (4 * (lane / 32)) * howo + oh * p.wo + ow);
                    static_for<0, 16>([&](auto rc) {
                        constexpr int r = decltype(rc)::value;
                        constexpr int dco = 8 * (r / 4) + (r % 4);
                        res[j][r] = pos_ok ? (p.residual + tile_base + int64_t(dco) * howo)[lane_off] : 0.f;
                    });
                });
            }
            static_for<0, NT>([&](auto jc) {
                constexpr int j = decltype(jc)::value;
                const int pos = pos0 + j * 32 + lane % 32;
                const int tr = udiv(pos, p.tw, p.tw_magic), ow = col0 + pos - tr * p.tw;
                const bool wrapped = th0 + tr >= p.ho;                 // this position belongs to the next image
                const int oh = th0 + tr - (wrapped ? p.ho : 0);
                const bool pos_ok = pos < tile_pos && row0 + tr < rows_total && ow < p.wo;
                const float q_scale = wrapped ? q_scale_b : q_scale_a;
                // uniform base in scalar registers + one 32-bit lane offset: no per-store address math
                const int64_t tile_base = (int64_t(img) * p.cout + cf) * howo;
                const unsigned lane_off = unsigned((wrapped ? p.cout * howo : 0) + (4 * (lane / 32)) * howo + oh * p.wo + ow);
                if (pos_ok) {
                    // One pass per epilogue term over the fragment's 16 accumulators, each behind a single
                    // uniform branch: testing the (uniform) options per element costs more instructions than
                    // the arithmetic itself.
                    float v[16];
                    static_for<0, 16>([&](auto rc) {
                        constexpr int r = decltype(rc)::value;
                        v[r] = __fmul_rn(float(acc[f][j][r]), dq[r]);
                    });
                    if (ROWM && p.row_scale) {
                        const float rs = p.row_scale[row0 + tr];
                        static_for<0, 16>([&](auto rc) {
                            constexpr int r = decltype(rc)::value;
                            v[r] = __fmul_rn(v[r], rs);
                        });
                    }
                    if (p.bias) static_for<0, 16>([&](auto rc) {
                        constexpr int r = decltype(rc)::value;
                        v[r] = __fadd_rn(v[r], bias[r]);
                    });
                    if (EXTRA && p.residual && !p.res_after) static_for<0, 16>([&](auto rc) {
                        constexpr int r = decltype(rc)::value;
                        v[r] = __fadd_rn(v[r], res[j][r]);
                    });
                    if (p.act == TSX_ACT_RELU) {
                        static_for<0, 16>([&](auto rc) {
                            constexpr int r = decltype(rc)::value;
                            v[r] = v[r] > 0.f ? v[r] : 0.f;
                        });
                    } else if (p.act == TSX_ACT_LEAKY_RELU) {
                        static_for<0, 16>([&](auto rc) {
                            constexpr int r = decltype(rc)::value;
                            v[r] = apply_act_conv_i8(v[r], TSX_ACT_LEAKY_RELU, p.slope, true);
                        });
                    } else if (MISHX && p.act == TSX_ACT_MISH) {
                        // nothing but the requantized values leaves: the exact form only where it decides a rounding (the
                        // largest tile has no registers left for it)
                        if (NT < 7 && !ROWM && !p.out_f32 && want_q) mish_fragment_for_rounding(v, res[j], EXTRA && p.residual && p.res_after, q_scale);
                        else mish_fragment(v);
                    } else if (p.act == TSX_ACT_MISH_FAST) {
                        static_for<0, 16>([&](auto rc) {
                            constexpr int r = decltype(rc)::value;
                            v[r] = apply_act_conv_i8(v[r], TSX_ACT_MISH_FAST, 0.f, true);
                        });
                    }
                    if (EXTRA && p.residual && p.res_after) static_for<0, 16>([&](auto rc) {
                        constexpr int r = decltype(rc)::value;
                        v[r] = __fadd_rn(v[r], res[j][r]);
                    });
                    if (ROWM) {
                        // row-major [position][cout]: one 16-byte store per group of 4 accumulators
                        float *o = p.out_f32 + cf + unsigned((row0 + tr) * p.cout + 4 * (lane / 32));
                        static_for<0, 4>([&](auto gc) {
                            constexpr int g4 = decltype(gc)::value;
                            typedef float v4f __attribute__((ext_vector_type(4)));
                            const v4f q4 = {v[4 * g4], v[4 * g4 + 1], v[4 * g4 + 2], v[4 * g4 + 3]};
                            *reinterpret_cast<v4f *>(o + 8 * g4) = q4;
                        });
                    } else if (p.out_f32) static_for<0, 16>([&](auto rc) {
                        constexpr int r = decltype(rc)::value;
                        constexpr int dco = 8 * (r / 4) + (r % 4);
                        // streaming store for large plain outputs: lines that never become dirty in L2 need no
                        // write-back burst when the kernel ends; outputs a following kernel reads stay cached
                        float *o = &(p.out_f32 + tile_base + int64_t(dco) * howo)[lane_off];
                        if (STREAM) __builtin_nontemporal_store(v[r], o);
                        else *o = v[r];
                    });
                    if (!ROWM && want_q) {
                        // the 16 requantized values as 4 dwords of 4 consecutive channels (quantize_pack: the value of
                        // quantize_value, converted, clamped and packed by one instruction)
                        uint32_t word[4] = {0u, 0u, 0u, 0u};
                        if (q_even) static_for<0, 16>([&](auto rc) {
                            constexpr int r = decltype(rc)::value;
                            word[r / 4] = quantize_pack<r % 4>(__fmul_rn(v[r], q_scale), true, word[r / 4]);
                        });
                        else static_for<0, 16>([&](auto rc) {
                            constexpr int r = decltype(rc)::value;
                            word[r / 4] = quantize_pack<r % 4>(__fmul_rn(v[r], q_scale), false, word[r / 4]);
                        });
                        static_for<0, 4>([&](auto gc) { word[decltype(gc)::value] ^= 0x80808080u; });
                        if (p.out_i8) static_for<0, 16>([&](auto rc) {
                            constexpr int r = decltype(rc)::value;
                            constexpr int dco = 8 * (r / 4) + (r % 4);
                            (p.out_i8 + tile_base + int64_t(dco) * howo)[lane_off] = int8_t(word[r / 4] >> (8 * (r % 4)));
                        });
                        if (EXTRA && p.st_out) {
                            // consumer's staged layout [pixel][channel].  Accumulator registers 4g..4g+3 of a lane are 4
                            // consecutive channels of one pixel (one dword); the pixel's other 16 channels of this
                            // fragment sit in lane +-32.  Two half-wave swaps leave every lane with 16 consecutive
                            // channels -- lower half cf..cf+15, upper half cf+16..cf+31 -- for one 16-byte store
                            // (4-byte stores at a pixel stride cost an L2 request each).
                            // swap(a, b): a's upper half-wave <-> b's lower half-wave
                            const auto s02 = __builtin_amdgcn_permlane32_swap(word[0], word[2], false, false);
                            const auto s13 = __builtin_amdgcn_permlane32_swap(word[1], word[3], false, false);
                            // the consumer's buffer is addressed by the real row/column (this kernel's rows may be virtual)
                            const int pix = oh * p.wo + ow;
                            const int roh = p.wo == p.o_w ? oh : udiv(pix, p.o_w, p.ow_magic);
                            const int row_ = p.wo == p.o_w ? ow : pix - roh * p.o_w;
                            const int up = p.st_up == 2 ? 2 : 1;   // 2: a nearest-neighbour resize by 2 folded into the store
                            int8_t *dst = p.st_out + ((int64_t(img + (wrapped ? 1 : 0)) * p.st_hs + up * roh + p.st_pt) * p.st_ws + up * row_ + p.st_pl) * p.st_cp +
                                          cf + 16 * (lane / 32);
                            const v4i packed = {int(s02[0]), int(s02[1]), int(s13[0]), int(s13[1])};
                            *reinterpret_cast<v4i *>(dst) = packed;
                            if (up == 2) {
                                *reinterpret_cast<v4i *>(dst + p.st_cp) = packed;
                                *reinterpret_cast<v4i *>(dst + int64_t(p.st_ws) * p.st_cp) = packed;
                                *reinterpret_cast<v4i *>(dst + int64_t(p.st_ws + 1) * p.st_cp) = packed;
                            }
                        }
                    }
                }
            });
        } else {
            static_for<0, NT>([&](auto jc) {
                constexpr int j = decltype(jc)::value;
                const int pos = pos0 + j * 32 + lane % 32;
                const int tr = udiv(pos, p.tw, p.tw_magic), ow = col0 + pos - tr * p.tw;
                const bool wrapped = th0 + tr >= p.ho;                 // this position belongs to the next image
                const int oh = th0 + tr - (wrapped ? p.ho : 0);
                const bool pos_ok = pos < tile_pos && row0 + tr < rows_total && ow < p.wo;
                const int co0 = cf + 4 * (lane / 32);
                const int64_t base = ROWM ? int64_t(row0 + tr) * p.cout + co0
                                          : (int64_t(img + (wrapped ? 1 : 0)) * p.cout + co0) * howo + oh * p.wo + ow;
                const int64_t co_stride = ROWM ? 1 : howo;
                const float rs = (ROWM && p.row_scale && pos_ok) ? p.row_scale[row0 + tr] : 0.f;
                static_for<0, 16>([&](auto rc) {
                    constexpr int r = decltype(rc)::value;
                    constexpr int dco = 8 * (r / 4) + (r % 4);
                    if (pos_ok && co0 + dco < p.cout)
                        emit<MISHX>(p, acc[f][j][r], base + int64_t(dco) * co_stride, dq[r], bias[r], rs);
                });
            });
        }
    });
}

}  // namespace

template <>
int ws_launch_nt<TSX_WS_NT>(const WsParams &p, dim3 grid, size_t lds_bytes, hipStream_t stream) {
    constexpr int NT = TSX_WS_NT;
    // ROWM: the GEMM form of the epilogue; EXTRA: residual input and/or staged int8 output; STREAM: a large
    // fp32 output nothing reads back soon
    // small windows of small tiles: the variant with fewer fill registers
    const bool small_fill = NT <= 2 && ((p.wpix << p.chunk_shift) + WS_THREADS - 1) / WS_THREADS <= SMALL_FILL;
    // one fragment per wavefront, a K of two rounds or more, and few enough workgroups that a SIMD holds one or
    // two wavefronts: the B ring (more registers: three workgroups per CU)
    const bool look = NT == 1 && small_fill && p.ksteps >= 2 * RING && int64_t(grid.x) * grid.y <= 1024;
#define TSX_WS_LAUNCH(EXTRA, STREAM, ROWM, MISHX)                                                                      \
    do {                                                                                                               \
        constexpr int F = NT <= 2 ? SMALL_FILL : MAX_FILL;                                                             \
        if (NT == 1 && look)                                                                                           \
            hipLaunchKernelGGL((conv_i8_ws_kernel<NT, WS_FM, EXTRA, STREAM, ROWM, F, NT == 1, MISHX>), grid,           \
                               dim3(WS_THREADS), lds_bytes, stream, p);                                                \
        else if (NT <= 2 && small_fill)                                                                                \
            hipLaunchKernelGGL((conv_i8_ws_kernel<NT, WS_FM, EXTRA, STREAM, ROWM, F, false, MISHX>), grid,             \
                               dim3(WS_THREADS), lds_bytes, stream, p);                                                \
        else                                                                                                           \
            hipLaunchKernelGGL((conv_i8_ws_kernel<NT, WS_FM, EXTRA, STREAM, ROWM, MAX_FILL, false, MISHX>), grid,      \
                               dim3(WS_THREADS), lds_bytes, stream, p);                                                \
    } while (0)
    // the exact Mish: one instantiation (with every other epilogue term) that only its layers run
    if (p.act == TSX_ACT_MISH) {
        if (p.rowmajor) return fail(TSX_E_INVALID, "conv_i8_ws: the exact Mish is not compiled into the row-major form");
        TSX_WS_LAUNCH(true, false, false, true);
    }
    else if (p.rowmajor) TSX_WS_LAUNCH(false, false, true, false);
    else if (p.residual || p.st_out) TSX_WS_LAUNCH(true, false, false, false);
    else if (p.stream_out) TSX_WS_LAUNCH(false, true, false, false);
    else TSX_WS_LAUNCH(false, false, false, false);
#undef TSX_WS_LAUNCH
    TSX_LAUNCH_CHECK("conv_i8_ws_kernel");
    return 0;
}
#endif  // TSX_WS_NT

}  // namespace tsx
