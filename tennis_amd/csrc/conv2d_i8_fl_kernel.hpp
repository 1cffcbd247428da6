// The flat-tile int8 convolution kernel (see conv2d_i8_fl.hip for the data movement it implements).
// Included by one translation unit per fragment split (NTA, NTB), each of which defines TSX_FL_NTA and
// TSX_FL_NTB and gets the specialisation fl_launch_nt<NTA, NTB>.
#pragma once
#include "igemm_i8.hpp"

#include <atomic>

namespace tsx {

constexpr int FL_RING = 4;        // A register ring depth (K-steps); the packed weights are padded to it
constexpr int FL_PIX = 80;        // LDS bytes per window pixel (64 channels + 16 pad: conflict-free 16-byte reads)
constexpr int FL_THREADS = 512;   // 8 wavefronts: two per SIMD
constexpr int FL_MAX_FILL = 4;    // window chunks per thread per channel block
constexpr int FL_MAX_WP = FL_MAX_FILL * FL_THREADS / 4;   // 512 window pixels
constexpr int FL_MAX_LDS = 160 * 1024;                    // LDS of one CU, all of it available to one workgroup

struct FlParams : EpiParams {
    const int8_t *xs;   // staged activations [n][hs][ws][cp]
    const int8_t *wp;   // packed weights [ks_p][coutp/32][2 halves][64 lanes][16]
    int n, cout, coutp, ho, wo, hs, ws, cp, cblocks, kh, kw;
    int sh, sw;
    int frags;              // position fragments per tile (NTA + NTB)
    int wc, wpix;           // window columns, window pixels
    int wr, rowp;           // window rows; LDS bytes per window row (>= wc * FL_PIX, see fl_plan)
    int ksteps_p;
    int ksteps;             // K-steps that hold weights (ksteps_p: padded to the A-ring size with zero steps)
    int tap_row, tap_col;   // bytes into the window per kernel row / column
    int tiles, tiles_per_xcd;
    int positions;          // n * ho * wo
    int stream_out;         // fp32 output written with streaming stores
    int resident;           // every channel block's window in LDS at once (cblocks buffers instead of 2)
    // per-lane divisions by uniform divisors as one multiply-high (div_magic / udiv)
    unsigned wc_magic, wo_magic, ho_magic, howo_magic;
};

template <int NTA, int NTB>
int fl_launch_nt(const FlParams &p, dim3 grid, size_t lds_bytes, hipStream_t stream);
template <> int fl_launch_nt<1, 1>(const FlParams &, dim3, size_t, hipStream_t);
template <> int fl_launch_nt<2, 1>(const FlParams &, dim3, size_t, hipStream_t);
template <> int fl_launch_nt<2, 2>(const FlParams &, dim3, size_t, hipStream_t);
template <> int fl_launch_nt<3, 2>(const FlParams &, dim3, size_t, hipStream_t);
template <> int fl_launch_nt<3, 3>(const FlParams &, dim3, size_t, hipStream_t);
template <> int fl_launch_nt<4, 3>(const FlParams &, dim3, size_t, hipStream_t);
template <> int fl_launch_nt<4, 4>(const FlParams &, dim3, size_t, hipStream_t);

#if defined(TSX_FL_NTA) && defined(TSX_FL_NTB)
namespace {

// The work of one wavefront: NT position fragments (tile fragments frag0 .. frag0 + NT - 1) x 32 output
// channels, all of K.  Every wavefront of the workgroup also copies its share of each channel block's window.
//
// RESIDENT: the windows of ALL channel blocks are copied into LDS before the K loop (they fit: one buffer per
// block), so the loop holds no barrier and no window traffic -- only the weight stream into registers, the
// LDS operand reads and the MFMAs -- and the wavefronts of a workgroup run through it independently.  The
// wavefronts that finish first store their output while the others still multiply.  Otherwise the window
// is double buffered, one channel block ahead, with one barrier per block.
template <int NT, bool EXTRA, bool STREAM, bool RESIDENT, bool MISHX>
__device__ __forceinline__ void fl_wave(const FlParams &p, int8_t *lds, int tile, int wave_m, int frag0) {
    const int tid = threadIdx.x, lane = tid % 64;
    const int P0 = tile * p.frags * 32;   // first flat position (n, oh, ow) of the tile
    const int R0 = udiv(P0, p.wo, p.wo_magic);   // its row in the batch-wide row sequence
    const int img0 = udiv(R0, p.ho, p.ho_magic);
    const int srow0 = img0 * p.hs + (R0 - img0 * p.ho) * p.sh;   // staged row of window row 0
    // staged rows from where output row `ho` of an image would start to the next image's first row
    const int wrap = p.hs - p.ho * p.sh;
    const int m0 = (blockIdx.y * 4 + wave_m) * 32;   // first cout of this wavefront
    const int taps = p.kh * p.kw;
    const int win_bytes = p.wr * p.rowp;

    // ---- window fill bookkeeping: chunk q = tid + i*512 -> pixel q / 4, 16-byte chunk q % 4
    // A uniform 64-bit base (the window's first staged row) plus one 32-bit byte offset per chunk: the loads take
    // the base from scalar registers and need no address arithmetic of their own.
    const int n_fill = (p.wpix * 4 + FL_THREADS - 1) / FL_THREADS;   // <= FL_MAX_FILL, uniform
    const int row_last = int(min(int64_t(p.n) * p.hs - 1 - srow0, int64_t(1) << 20));   // last tile: rows no stored output uses
    const int8_t *xs_base = p.xs + int64_t(srow0) * p.ws * p.cp;
    unsigned fill_off[FL_MAX_FILL];
    int fill_dst[FL_MAX_FILL];
    static_for<0, FL_MAX_FILL>([&](auto ic) {
        constexpr int i = decltype(ic)::value;
        fill_off[i] = 0;
        fill_dst[i] = 0;
        if (i < n_fill) {
            const int q = tid + i * FL_THREADS;
            int pix = q >> 2;
            const int chunk = q & 3;
            if (pix >= p.wpix) pix = p.wpix - 1;   // duplicates rewrite the same bytes
            const int wrow = udiv(pix, p.wc, p.wc_magic);
            const int wcol = pix - __mul24(wrow, p.wc);
            // 24-bit multiplies (full rate): window rows, staged widths and pixel sizes are far below 2^24
            fill_off[i] = unsigned(__mul24(__mul24(min(wrow, row_last), p.ws) + wcol, p.cp) + chunk * 16);
            fill_dst[i] = __mul24(wrow, p.rowp) + wcol * FL_PIX + chunk * 16;
        }
    });
    v4i wreg[FL_MAX_FILL];

    // the empty statement keeps the offset's widening next to the load, where instruction selection folds it
    // into the scalar-base addressing mode
    auto fill_load = [&](int i, int cb) __attribute__((always_inline)) {
        unsigned off = fill_off[i];
        asm volatile("" : "+v"(off));
        return *reinterpret_cast<const v4i *>(xs_base + cb * 64 + off);
    };
    auto window_load = [&](int cb) __attribute__((always_inline)) {
        static_for<0, FL_MAX_FILL>([&](auto ic) {
            constexpr int i = decltype(ic)::value;
            if (i < n_fill) wreg[i] = fill_load(i, cb);
        });
    };
    auto window_store = [&](int buf) __attribute__((always_inline)) {
        static_for<0, FL_MAX_FILL>([&](auto ic) {
            constexpr int i = decltype(ic)::value;
            if (i < n_fill) *reinterpret_cast<v4i *>(&lds[buf * win_bytes + fill_dst[i]]) = wreg[i];
        });
    };

    // the first window's loads leave before anything else is computed: their latency covers the rest of the set-up
    window_load(0);

    // ---- B operand addresses: fragment j, lane l -> flat position P0 + (frag0 + j)*32 + l%32, K group l/32
    int b_base[NT];
    static_for<0, NT>([&](auto jc) {
        constexpr int j = decltype(jc)::value;
        int pp = P0 + (frag0 + j) * 32 + lane % 32;
        if (pp >= p.positions) pp = P0;       // beyond the last position: computed, never stored
        const int R = udiv(pp, p.wo, p.wo_magic), ow = pp - R * p.wo;
        const int img = udiv(R, p.ho, p.ho_magic);
        const int wrow = (R - R0) * p.sh + wrap * (img - img0);   // later images sit below their halo rows
        b_base[j] = __mul24(wrow, p.rowp) + __mul24(ow, p.sw * FL_PIX) + (lane / 32) * 16;
    });

    // ---- A ring: 2 halves of K-step ks for the wavefront's 32 output channels, 1 KiB each.  Buffer loads:
    // descriptor and K-step offset stay in scalar registers, the lane supplies one constant 32-bit offset
    // (per-lane 64-bit addresses cost a 64-bit multiply-add per load and measurably more time and power).
    const int frag_u = __builtin_amdgcn_readfirstlane(m0 / 32);
    const __amdgpu_buffer_rsrc_t a_rsrc =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<int8_t *>(p.wp), 0, 0x7fffffff, 0x00020000);
    const int a_lane = lane * 16;
    const int a_frag = frag_u * 2048;
    const int a_kstride = (p.coutp / 32) * 2048;   // packed weights are below 2 GiB (checked by the launcher)
    v4i areg[FL_RING][2];
    auto a_load = [&](auto slot, int ks) __attribute__((always_inline)) {
        constexpr int s = decltype(slot)::value;
        if (ks >= p.ksteps) ks = p.ksteps - 1;   // beyond the last K-step: its lines again, never used
        const int so = a_frag + ks * a_kstride;
        areg[s][0] = __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(a_rsrc, a_lane, so, 0));
        areg[s][1] = __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(a_rsrc, a_lane, so + 1024, 0));
    };

    v16i acc[NT];
    static_for<0, NT>([&](auto jc) {
        static_for<0, 16>([&](auto rc) { acc[decltype(jc)::value][decltype(rc)::value] = 0; });
    });

    // ---- prologue
    static_for<0, FL_RING - 1>([&](auto sc) { a_load(sc, decltype(sc)::value); });
    int cb = 0, tap = 0, kr = 0, kc = 0, buf = 0;
    // RESIDENT: block 0's window first -- the K loop starts as soon as it is in LDS -- with the next three
    // blocks' loads already in flight behind it; those are stored (and any further blocks fetched) when this
    // wavefront leaves block 0, behind the loop's only barrier.
    v4i wbat[3][FL_MAX_FILL];
    if (RESIDENT) {
        static_for<0, 3>([&](auto bc) {
            constexpr int b = decltype(bc)::value;
            const int c = 1 + b < p.cblocks ? 1 + b : p.cblocks - 1;
            static_for<0, FL_MAX_FILL>([&](auto ic) {
                constexpr int i = decltype(ic)::value;
                if (i < n_fill) wbat[b][i] = fill_load(i, c);
            });
        });
    }
    window_store(0);
    __syncthreads();
    if (!RESIDENT && p.cblocks > 1) window_load(1);   // block cb+1, in flight during block cb's taps

    v4i b0[NT], b1[NT];
    auto b_read = [&](v4i(&dst)[NT], int off) __attribute__((always_inline)) {
        static_for<0, NT>([&](auto jc) {
            constexpr int j = decltype(jc)::value;
            dst[j] = *reinterpret_cast<const v4i *>(&lds[b_base[j] + off]);
        });
    };
    int toff = 0;   // buf * win_bytes + tap shift
    b_read(b0, toff);

    // One K-step: both halves' MFMAs, the B reads one half-step ahead, the window change on a channel-block
    // boundary.  PREFETCH: also load the weights of the K-step FL_RING-1 ahead into the slot the previous step freed.
    int ks = 0;
    auto k_step = [&](auto uc, auto prefetch) __attribute__((always_inline)) {
        constexpr int u = decltype(uc)::value;
        if (decltype(prefetch)::value) a_load(std::integral_constant<int, (u + FL_RING - 1) % FL_RING>{}, ks + FL_RING - 1);
        b_read(b1, toff + 32);                       // second half of this K-step
        static_for<0, NT>([&](auto jc) {
            constexpr int j = decltype(jc)::value;
            acc[j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(areg[u][0], b0[j], acc[j], 0, 0, 0);
        });
        ++ks;
        ++tap;
        if (++kc == p.kw) {
            kc = 0;
            ++kr;
        }
        if (tap == taps) {
            tap = 0;
            kr = 0;
            kc = 0;
            ++cb;
            if (RESIDENT) {
                if (cb == 1 && p.cblocks > 1) {
                    static_for<0, 3>([&](auto bc) {
                        constexpr int b = decltype(bc)::value;
                        const int c = 1 + b < p.cblocks ? 1 + b : p.cblocks - 1;
                        static_for<0, FL_MAX_FILL>([&](auto ic) {
                            constexpr int i = decltype(ic)::value;
                            if (i < n_fill) *reinterpret_cast<v4i *>(&lds[c * win_bytes + fill_dst[i]]) = wbat[b][i];
                        });
                    });
                    for (int c = 4; c < p.cblocks; ++c) {   // more than four blocks: the rest, one round trip each
                        window_load(c);
                        window_store(c);
                    }
                    __syncthreads();
                }
                buf = cb < p.cblocks ? cb : p.cblocks - 1;   // the read ahead behind the last K-step stays in the last block
            } else if (ks < p.ksteps) {                      // no window change behind the last K-step
                window_store(buf ^ 1);
                __syncthreads();
                buf ^= 1;
                const int next = cb + 1 < p.cblocks ? cb + 1 : p.cblocks - 1;
                window_load(next);
            }
        }
        toff = buf * win_bytes + kr * p.tap_row + kc * p.tap_col;
        b_read(b0, toff);                            // first half of the next K-step
        static_for<0, NT>([&](auto jc) {
            constexpr int j = decltype(jc)::value;
            acc[j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(areg[u][1], b1[j], acc[j], 0, 0, 0);
        });
    };
    // whole rounds of the ring, then the K-steps left over: their weights are in the ring already (the steps
    // ahead of the last round), and the zero steps that pad the packed weights to a whole round are not multiplied
    while (ks + FL_RING <= p.ksteps) static_for<0, FL_RING>([&](auto uc) { k_step(uc, std::true_type{}); });
    const int left = p.ksteps - ks;
    static_for<0, FL_RING - 1>([&](auto uc) {
        if (decltype(uc)::value < left) k_step(uc, std::false_type{});
    });


    // ---- epilogue: accumulator register r of lane l = cout 8*(r/4) + 4*(l/32) + r%4, position l%32
    const int howo = p.ho * p.wo;
    const int64_t count = int64_t(p.n) * p.cout * howo;
    // hot case: no raw accumulators wanted, every element inside the activation's SIMD-body range, a tensor
    // small enough for 32-bit lane offsets, and -- for the requantized output -- one quantize group per image
    // (or a single scale whose round-half-even bulk covers everything)
    const bool want_q = p.out_i8 || p.st_out;
    const bool q_uniform = !want_q || (p.n_qscales == 1 ? p.q_bulk8 == count : p.q_group_len == int64_t(p.cout) * howo);
    const bool fast = (p.out_f32 || want_q) && !p.out_acc && p.act_body == count && count < (int64_t(1) << 30) && q_uniform;
    const bool q_even = p.n_qscales == 1;   // single-scale quantize rounds half to even in its bulk
    const int cf = m0;                      // first cout of this wavefront's fragment (uniform)
    // Loads without per-element branches: the fast case needs no bounds (consecutive channels combine into
    // 16-byte loads); otherwise the index is clamped, and what a channel beyond cout loads is never stored.
    const bool fast_f = fast && cf + 32 <= p.cout;
    float dq[16], bias[16];
    static_for<0, 16>([&](auto rc) {
        dq[decltype(rc)::value] = 0.f;
        bias[decltype(rc)::value] = 0.f;
    });
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
        const int co_lane = cf + 4 * (lane / 32);
        if (p.dq) static_for<0, 16>([&](auto rc) {
            constexpr int r = decltype(rc)::value;
            dq[r] = p.dq[min(co_lane + 8 * (r / 4) + (r % 4), p.cout - 1)];
        });
        if (p.bias) static_for<0, 16>([&](auto rc) {
            constexpr int r = decltype(rc)::value;
            bias[r] = p.bias[min(co_lane + 8 * (r / 4) + (r % 4), p.cout - 1)];
        });
    }
    // per fragment: the lane's position as image and pixel
    int pimg[NT], prem[NT];
    bool pok[NT];
    static_for<0, NT>([&](auto jc) {
        constexpr int j = decltype(jc)::value;
        const int pp = P0 + (frag0 + j) * 32 + lane % 32;
        pok[j] = pp < p.positions;
        const int ps = pok[j] ? pp : P0;
        pimg[j] = udiv(ps, howo, p.howo_magic);
        prem[j] = ps - pimg[j] * howo;
    });
    if (fast_f) {
        // uniform base in scalar registers + one 32-bit lane offset: no per-store address math
        const int64_t base = int64_t(cf) * howo;
        // the other branch of a residual join: the loads of every fragment are in flight before the first use
        float res[NT][16];
        if (EXTRA && p.residual) {
            static_for<0, NT>([&](auto jc) {
                constexpr int j = decltype(jc)::value;
                const unsigned lane_off = unsigned(pimg[j] * p.cout * howo + (4 * (lane / 32)) * howo + prem[j]);
                static_for<0, 16>([&](auto rc) {
                    constexpr int r = decltype(rc)::value;
                    constexpr int dco = 8 * (r / 4) + (r % 4);
                    res[j][r] = pok[j] ? (p.residual + base + int64_t(dco) * howo)[lane_off] : 0.f;
                });
            });
        }
        static_for<0, NT>([&](auto jc) {
            constexpr int j = decltype(jc)::value;
            if (!pok[j]) return;
            const unsigned lane_off = unsigned(pimg[j] * p.cout * howo + (4 * (lane / 32)) * howo + prem[j]);
            // One pass per epilogue term over the fragment's 16 accumulators, each behind one uniform branch.
            float v[16];
            static_for<0, 16>([&](auto rc) {
                constexpr int r = decltype(rc)::value;
                v[r] = __fmul_rn(float(acc[j][r]), dq[r]);
            });
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
                // nothing but the requantized values leaves: the exact form only where it decides a rounding
                if (!p.out_f32 && want_q)
                    mish_fragment_for_rounding(v, res[j], EXTRA && p.residual && p.res_after, p.q_scales[p.n_qscales == 1 ? 0 : pimg[j]]);
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
            if (p.out_f32) static_for<0, 16>([&](auto rc) {
                constexpr int r = decltype(rc)::value;
                constexpr int dco = 8 * (r / 4) + (r % 4);
                // streaming store for large plain outputs: lines that never become dirty in L2 need no
                // write-back burst when the kernel ends; outputs a following kernel reads stay cached
                float *o = &(p.out_f32 + base + int64_t(dco) * howo)[lane_off];
                if (STREAM) __builtin_nontemporal_store(v[r], o);
                else *o = v[r];
            });
            if (want_q) {
                const float q_scale = p.q_scales[p.n_qscales == 1 ? 0 : pimg[j]];
                int qv[16];
                if (q_even) static_for<0, 16>([&](auto rc) {
                    constexpr int r = decltype(rc)::value;
                    qv[r] = quantize_value(__fmul_rn(v[r], q_scale), true);
                });
                else static_for<0, 16>([&](auto rc) {
                    constexpr int r = decltype(rc)::value;
                    qv[r] = quantize_value(__fmul_rn(v[r], q_scale), false);
                });
                if (p.out_i8) static_for<0, 16>([&](auto rc) {
                    constexpr int r = decltype(rc)::value;
                    constexpr int dco = 8 * (r / 4) + (r % 4);
                    (p.out_i8 + base + int64_t(dco) * howo)[lane_off] = int8_t(qv[r]);
                });
                if (EXTRA && p.st_out) {
                    // consumer's staged layout [pixel][channel]: registers 4g..4g+3 of a lane are 4 consecutive
                    // channels of one pixel, the pixel's other 16 channels of this fragment sit in lane +-32.  Two
                    // half-wave swaps leave every lane with 16 consecutive channels for one 16-byte store.
                    uint32_t word[4];
                    static_for<0, 4>([&](auto gc) {
                        constexpr int g4 = decltype(gc)::value;
                        word[g4] = uint32_t(qv[4 * g4] & 0xff) | (uint32_t(qv[4 * g4 + 1] & 0xff) << 8) |
                                   (uint32_t(qv[4 * g4 + 2] & 0xff) << 16) | (uint32_t(qv[4 * g4 + 3] & 0xff) << 24);
                    });
                    const auto s02 = __builtin_amdgcn_permlane32_swap(word[0], word[2], false, false);
                    const auto s13 = __builtin_amdgcn_permlane32_swap(word[1], word[3], false, false);
                    const int oh = udiv(prem[j], p.wo, p.wo_magic), ow = prem[j] - oh * p.wo;
                    const int up = p.st_up == 2 ? 2 : 1;   // 2: a nearest-neighbour resize by 2 folded into the store
                    int8_t *dst = p.st_out + ((int64_t(pimg[j]) * p.st_hs + up * oh + p.st_pt) * p.st_ws + up * ow + p.st_pl) * p.st_cp +
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
        });
    } else {
        static_for<0, NT>([&](auto jc) {
            constexpr int j = decltype(jc)::value;
            const int co0 = cf + 4 * (lane / 32);
            const int64_t base = (int64_t(pimg[j]) * p.cout + co0) * howo + prem[j];
            static_for<0, 16>([&](auto rc) {
                constexpr int r = decltype(rc)::value;
                constexpr int dco = 8 * (r / 4) + (r % 4);
                if (pok[j] && co0 + dco < p.cout) emit<MISHX>(p, acc[j][r], base + int64_t(dco) * howo, dq[r], bias[r], 0.f);
            });
        });
    }
}

// A workgroup of 8 wavefronts owns a tile of NTA + NTB position fragments x 128 output channels: wavefront w
// takes channels [32 (w%4), +32) and the first NTA fragments (w < 4) or the last NTB (w >= 4), so each SIMD
// hosts one wavefront of either kind.  With NTA > NTB the short wavefronts reach their epilogue while the
// long ones still multiply: part of the output leaves under the K loop.
// EXTRA = false compiles the residual input and the staged-layout output out of the epilogue; STREAM selects
// streaming fp32 stores.
template <int NTA, int NTB, bool EXTRA, bool STREAM, bool RESIDENT, bool MISHX = false>
__global__ __launch_bounds__(FL_THREADS) void conv_i8_fl_kernel(FlParams p_in) {
    FlParams p = p_in;
    if (!EXTRA) {
        p.residual = nullptr;
        p.st_out = nullptr;
    }
    p.row_scale = nullptr;
    extern __shared__ __attribute__((aligned(16))) int8_t lds[];   // (RESIDENT ? cblocks : 2) x wpix x FL_PIX
    // Workgroups are dealt round-robin to the 8 XCDs, each with its own L2: give every XCD a contiguous run of
    // tiles, so the halo rows two neighbouring tiles share are fetched from HBM once.  gridDim.x is a multiple
    // of 8, so the workgroups of one tile (blockIdx.y) land on the same XCD too.
    const int tile = (blockIdx.x & 7) * p.tiles_per_xcd + (blockIdx.x >> 3);
    if (tile >= p.tiles) return;   // the whole workgroup leaves
    // the wavefront's index as a scalar: what derives from it stays in scalar registers and branches uniformly
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / 64);
    // The long wavefronts get the SIMD's issue priority: they run through K at the MFMA pipe's pace while the
    // short ones fill the gaps, finish first although they hold more fragments, and store the larger part of
    // the tile's output under the other group's K loop.
    if (wave < 4) {
        __builtin_amdgcn_s_setprio(3);
        fl_wave<NTA, EXTRA, STREAM, RESIDENT, MISHX>(p, lds, tile, wave, 0);
    } else {
        fl_wave<NTB, EXTRA, STREAM, RESIDENT, MISHX>(p, lds, tile, wave - 4, NTA);
    }
}

}  // namespace

template <>
int fl_launch_nt<TSX_FL_NTA, TSX_FL_NTB>(const FlParams &p, dim3 grid, size_t lds_bytes, hipStream_t stream) {
    constexpr int NTA = TSX_FL_NTA, NTB = TSX_FL_NTB;
    // more than 64 KiB of dynamic LDS (up to the CU's 160 KiB) has to be granted per kernel and device
    static std::atomic<bool> granted[2][4][64];
    int dev = 0;
    TSX_HIP(hipGetDevice(&dev));
#define TSX_FL_LAUNCH(EXTRA, STREAM, RESIDENT, SLOT)                                                          \
    do {                                                                                                      \
        auto kernel = conv_i8_fl_kernel<NTA, NTB, EXTRA, STREAM, RESIDENT, SLOT == 3>;                        \
        if (lds_bytes > 65536 && dev < 64 && !granted[RESIDENT][SLOT][dev].load()) {                          \
            TSX_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),                               \
                                        hipFuncAttributeMaxDynamicSharedMemorySize, FL_MAX_LDS));             \
            granted[RESIDENT][SLOT][dev].store(true);                                                         \
        }                                                                                                     \
        hipLaunchKernelGGL(kernel, grid, dim3(FL_THREADS), lds_bytes, stream, p);                             \
    } while (0)
    // (slot 3: the instantiation with the exact Mish, which only its layers run)
    if (p.resident) {
        if (p.act == TSX_ACT_MISH) TSX_FL_LAUNCH(true, false, true, 3);
        else if (p.residual || p.st_out) TSX_FL_LAUNCH(true, false, true, 0);
        else if (p.stream_out) TSX_FL_LAUNCH(false, true, true, 1);
        else TSX_FL_LAUNCH(false, false, true, 2);
    } else {
        if (p.act == TSX_ACT_MISH) TSX_FL_LAUNCH(true, false, false, 3);
        else if (p.residual || p.st_out) TSX_FL_LAUNCH(true, false, false, 0);
        else if (p.stream_out) TSX_FL_LAUNCH(false, true, false, 1);
        else TSX_FL_LAUNCH(false, false, false, 2);
    }
#undef TSX_FL_LAUNCH
    TSX_LAUNCH_CHECK("conv_i8_fl_kernel");
    return 0;
}
#endif  // TSX_FL_NTA && TSX_FL_NTB

}  // namespace tsx
