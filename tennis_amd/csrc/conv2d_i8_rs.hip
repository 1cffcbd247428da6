// Weight-stationary int8 convolution for large multi-tap layers on 256 input channels (BASELINE config 2:
// 32x256x28x28 * 256x256x3x3).  Same arithmetic, staged input and packed weights as the window-stationary and
// flat-tile kernels (exact int32 sums of cpu::Conv2DQuantizedCore,
// src/kernels/cpu/quantized/conv2d_quantized_core.cpp:18-147, dequantized as its lines 81-106 do); what differs
// is which operand stays put:
//   * a workgroup is 4 wavefronts, one per SIMD, on 64 output channels and a run of F consecutive 32-position
//     fragments of the batch-wide flat position list (n, oh, ow).  Wavefront s multiplies only channel block s
//     (64 input channels x KH x KW taps: a quarter of K) and keeps ITS weights for all 64 output channels in
//     registers for the whole kernel: 2 x KH*KW x 2 MFMA operands of 16 bytes per lane (144 registers for 3x3),
//     loaded once.  The K loop therefore streams nothing but activations;
//   * activations come from a ring of staged rows in LDS, one ring per wavefront holding that wavefront's 64
//     channels only: a wavefront fills and reads its own ring, so the window needs no workgroup barrier.  Rows
//     are loaded three fragments ahead of their first use and enter the ring two ahead;
//   * per fragment a wavefront issues KH*KW x 2 x 2 MFMAs (32x32x32) into 2 accumulators; the four wavefronts'
//     partial sums (exact integers, any order) meet in LDS, and wavefront s finishes a quarter of the
//     fragment's outputs -- dequantize, bias, activation, store -- while the MFMAs of the NEXT fragment run.
//     Output therefore leaves the chip as a steady stream under the multiplication instead of one burst
//     behind it; only the last fragment's epilogue is exposed.
// One barrier per fragment (partial sums double buffered).  MFMA operand layout as in conv2d_i8_ws.hip: lane l
// supplies row / column l%32 and the 16 K bytes of group l/32; accumulator register r of lane l is output
// channel 8*(r/4) + 4*(l/32) + r%4, position l%32.
#include "igemm_i8.hpp"

#include <atomic>
#include <cstdlib>

namespace tsx {

constexpr int RS_PIX = 80;        // LDS bytes per ring pixel (64 channels + 16 pad: conflict-free 16-byte reads)
constexpr int RS_THREADS = 256;   // 4 wavefronts, one per SIMD
constexpr int RS_FILLN = 2;       // 16-byte chunks per lane per ring row: rows of up to 32 window pixels
constexpr int RS_MAXNEW = 4;      // staged rows that may enter the ring per fragment
constexpr int RS_PRO = 8;         // staged rows the first two fragments of a tile may need (= the largest ring)
constexpr int RS_BR = 6;          // B operand register ring (divides the 2 x taps sub-steps of a fragment)
constexpr int RS_LOOK = 5;        // sub-steps a B operand is read ahead of its MFMAs
constexpr int RS_XBUF = 65536;    // partial-sum exchange: [4 finishers][2 parities][4 sources][2 fragments][1 KiB]
constexpr int RS_MAX_LDS = 160 * 1024;

struct RsParams : EpiParams {
    const int8_t *xs;   // staged activations [n][hs][ws][cp]
    const int8_t *wp;   // packed weights [kstep][coutp/32][2 halves][64 lanes][16], K order (channel block, kh, kw)
    int n, cout, coutp, ho, wo, hs, ws, cp;
    int sh, sw, dil_h, dil_w;
    int frags;            // fragments per tile
    int total_frags;      // ceil(positions / 32)
    int positions;        // n * ho * wo
    int ptiles, ctiles, tiles, tiles_per_xcd;
    int nr_mask;          // ring rows - 1 (ring rows: 4 or 8)
    int rowp, wc;         // LDS bytes per ring row, window pixels per row
    int ring_bytes;       // (nr_mask + 1) * rowp
    unsigned xs_bytes, out_bytes;
    unsigned wo_magic, ho_magic;
#ifdef TSX_RS_STAMPS
    unsigned long long *stamps;   // [workgroup][wavefront][24][wall clock, shader clock]
    int stamp_slots;
#endif
};
#ifdef TSX_RS_STAMPS
void debug_phase_stamps(unsigned long long **buffer, int *slots);
#endif

namespace {

// floor(n / d) by the host's magic number (div_magic; the plan takes this kernel only where one exists)
__device__ __forceinline__ int mdiv(int n, unsigned magic) { return int(__umulhi(unsigned(n), magic)); }

// Keeps the computation of v where it is written: a value that only feeds one arm of a select would otherwise be
// sunk into a conditional block of its own, and a branch ends the scheduling region around it.
__device__ __forceinline__ int pinned(int v) {
    asm volatile("" : "+v"(v));
    return v;
}

__device__ __forceinline__ void lds_fence_barrier() {
    // LDS traffic only: global loads and stores stay in flight across the barrier
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

// ACT: 0 = none / relu / leaky_relu picked by uniform selects, 1 = relu, 2 = Mish
template <int KH, int KW, bool STREAM, int ACT>
__global__ __launch_bounds__(RS_THREADS) __attribute__((amdgpu_waves_per_eu(1, 1))) void conv_i8_rs_kernel(RsParams p) {
    constexpr int TAPS = KH * KW, SUB = 2 * TAPS;
    static_assert(SUB % RS_BR == 0, "the B ring must divide a fragment's sub-steps");
    static_assert(SUB >= 18, "a fragment's sub-steps carry the other duties of the wavefront: 18 of them");
    extern __shared__ __attribute__((aligned(16))) int8_t lds[];
    // Workgroups are dealt round-robin to the 8 XCDs (own L2 each): every XCD gets a contiguous run of tiles, and
    // the cout tiles of one run of positions are neighbours in it.
    const int tile = (blockIdx.x & 7) * p.tiles_per_xcd + (blockIdx.x >> 3);
    if (tile >= p.tiles) return;
    const int ptile = tile / p.ctiles, ctile = tile - ptile * p.ctiles;
    const int lane = threadIdx.x % 64;
    const int s = __builtin_amdgcn_readfirstlane(threadIdx.x / 64);   // wavefront = channel block = finished quarter
    const int f0 = ptile * p.frags;
    const int f1 = min(f0 + p.frags, p.total_frags);
    const int cf = ctile * 64;
    const int howo = p.ho * p.wo;
#ifdef TSX_RS_STAMPS
    int stamp_k = 0;
    auto stamp = [&]() __attribute__((always_inline)) {
        const int slot = ((blockIdx.x * 4 + s) * 24 + stamp_k) * 2;
        if (p.stamps && lane == 0 && stamp_k < 24 && slot + 2 <= p.stamp_slots) {
            p.stamps[slot] = wall_clock64();
            p.stamps[slot + 1] = clock64();
        }
        ++stamp_k;
    };
#define RS_STAMP() stamp()
#else
#define RS_STAMP() ((void)0)
#endif
    RS_STAMP();

    // ---- LDS map: 4 rings | 4 x 1 KiB dump (target of predicated-off ring stores) | exchange buffers
    const int ring_base = s * p.ring_bytes;
    const int dump_addr = 4 * p.ring_bytes + s * 1024 + lane * 16;
    const int xlane = 4 * p.ring_bytes + 4096 + lane * 16;

    const __amdgpu_buffer_rsrc_t xs_rsrc =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<int8_t *>(p.xs), 0, p.xs_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t w_rsrc =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<int8_t *>(p.wp), 0, 0x7fffffff, 0x00020000);
    const __amdgpu_buffer_rsrc_t out_rsrc =
        __builtin_amdgcn_make_buffer_rsrc(p.out_f32, 0, p.out_bytes, 0x00020000);

    // uniform: last staged row (+1) that fragment f reads, f clamped to this tile
    auto rows_end = [&](int f) __attribute__((always_inline)) {
        f = min(f, f1 - 1);
        const int pp = min(f * 32 + 31, p.positions - 1);
        const int R = mdiv(pp, p.wo_magic);
        const int img = mdiv(R, p.ho_magic);
        return img * p.hs + (R - img * p.ho) * p.sh + (KH - 1) * p.dil_h + 1;
    };
    // Ring fill of one staged row: lane l moves chunks l and l + 64 (pixel q / 4, 16 bytes q % 4 of this wavefront's
    // 64 channels).  The row's place in memory and in the ring is uniform (scalar offsets); what a lane adds is
    // constant.  Predicated without branches: an out-of-range buffer offset fetches nothing, and the store of a row
    // that is not wanted goes to the dump.
    int fill_src[RS_FILLN], fill_pix[RS_FILLN];
    bool fill_on[RS_FILLN];
    static_for<0, RS_FILLN>([&](auto jc) {
        constexpr int j = decltype(jc)::value;
        const int q = lane + 64 * j, pix = q >> 2, chunk = q & 3;
        fill_on[j] = pix < p.wc;
        fill_src[j] = fill_on[j] ? pix * p.cp + s * 64 + chunk * 16 : int(0x80000000u);
        fill_pix[j] = ring_base + pix * RS_PIX + chunk * 16;
    });
    const int row_bytes = p.ws * p.cp;
    auto fill_load = [&](int g, bool need, int j) __attribute__((always_inline)) {
        return __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(
                                           xs_rsrc, need ? fill_src[j] : int(0x80000000u), g * row_bytes, 0));
    };
    auto fill_store = [&](int g, bool need, int j, const v4i &v) __attribute__((always_inline)) {
        const int dst = pinned(fill_pix[j] + (g & p.nr_mask) * p.rowp);
        *reinterpret_cast<v4i *>(&lds[(need && fill_on[j]) ? dst : dump_addr]) = v;
    };

    // ---- prologue 1: the ring rows of the tile's first two fragments (in flight first: they are needed first)
    {
        const int pp0 = f0 * 32;
        const int R0 = mdiv(pp0, p.wo_magic);
        const int img0 = mdiv(R0, p.ho_magic);
        const int g_first = img0 * p.hs + (R0 - img0 * p.ho) * p.sh;
        const int g_end = rows_end(f0 + 1);
        v4i pro[RS_PRO][RS_FILLN];
        static_for<0, RS_PRO>([&](auto ic) {
            constexpr int i = decltype(ic)::value;
            static_for<0, RS_FILLN>([&](auto jc) {
                constexpr int j = decltype(jc)::value;
                pro[i][j] = fill_load(min(g_first + i, g_end - 1), g_first + i < g_end, j);
            });
        });
        static_for<0, RS_PRO>([&](auto ic) {
            constexpr int i = decltype(ic)::value;
            static_for<0, RS_FILLN>([&](auto jc) {
                constexpr int j = decltype(jc)::value;
                fill_store(g_first + i, g_first + i < g_end, j, pro[i][j]);
            });
        });
    }
    int rows_hi = rows_end(f0 + 1);   // staged rows below this are (being) loaded

    // ---- prologue 2: this wavefront's weights, K-step by K-step in the order the MFMAs use them
    v4i A[2][TAPS][2];
    {
        const int kstride = (p.coutp / 32) * 2048;
        const int frag_off = (cf / 32) * 2048;
        static_for<0, TAPS>([&](auto kc_) {
            constexpr int k = decltype(kc_)::value;
            static_for<0, 2>([&](auto hc) {
                constexpr int h = decltype(hc)::value;
                static_for<0, 2>([&](auto cc) {
                    constexpr int c = decltype(cc)::value;
                    const int so = (s * TAPS + k) * kstride + frag_off + c * 2048 + h * 1024;
                    A[c][k][h] = __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(w_rsrc, lane * 16, so, 0));
                });
            });
        });
        // The weights live in the accumulation registers' half of the file (an MFMA reads its A operand from either
        // half): with the accumulators that is 208 of its 256, and the other half is left to everything that other
        // instructions touch.  Left to itself the allocator keeps them in the general half and, short of registers
        // there, parks freshly loaded ring rows in this one -- behind a wait for the load in the middle of the MFMAs.
        static_for<0, TAPS>([&](auto kc_) {
            constexpr int k = decltype(kc_)::value;
            static_for<0, 2>([&](auto hc) {
                constexpr int h = decltype(hc)::value;
                static_for<0, 2>([&](auto cc) {
                    constexpr int c = decltype(cc)::value;
                    v4i &w = A[c][k][h];
                    asm volatile("" : "+a"(w));
                });
            });
        });
    }

    // ---- per-lane constants of the finishing quarter: register (c, i) is channel cf + 32c + 8s + 4(l/32) + i
    float dqv[2][4], bv[2][4];
    unsigned cmask[2][4];   // 0, or the out-of-range bit for a channel beyond cout
    static_for<0, 2>([&](auto cc) {
        constexpr int c = decltype(cc)::value;
        static_for<0, 4>([&](auto ic) {
            constexpr int i = decltype(ic)::value;
            const int co = cf + 32 * c + 8 * s + 4 * (lane / 32) + i;
            cmask[c][i] = co < p.cout ? 0u : 0x80000000u;
            dqv[c][i] = p.dq[min(co, p.cout - 1)];
            bv[c][i] = p.bias ? p.bias[min(co, p.cout - 1)] : -0.f;   // v + (-0) = v, bit for bit: no bias, no branch
        });
    });
    // dequantize -> bias -> activation of one sum, without branches (each would end a scheduling region of the
    // fragment loop): relu and leaky_relu in their SIMD-body forms (src/kernels/cpu/relu.cpp:30-52,
    // leaky_relu.cpp:41-66; rs_takes admits only tensors that lie in the body), picked by uniform selects
    const bool is_relu = p.act == TSX_ACT_RELU, is_leaky = p.act == TSX_ACT_LEAKY_RELU;
    const float slope = p.slope;
    auto finish = [&](int sum, float dq, float bias) __attribute__((always_inline)) {
        const float v = __fadd_rn(__fmul_rn(float(sum), dq), bias);
        if constexpr (ACT == 2) {
            return apply_act_conv_i8(v, TSX_ACT_MISH, 0.f, true);
        } else if constexpr (ACT == 1) {
            return v > 0.f ? v : 0.f;
        } else {
            const float mx = v > 0.f ? v : 0.f;
            const float mn = v < 0.f ? v : 0.f;
            const float leaky = __builtin_fmaf(slope, mn, mx);
            return is_relu ? mx : is_leaky ? leaky : v;
        }
    };

    // ---- fragment decode: LDS address of the lane's pixel per kernel row, and its place in the output
    struct Frag {
        int ra[KH];          // ring address of (kernel row kr, kernel column 0), 16 K bytes of group lane/32
        unsigned out_off;    // byte offset of (image, channel 4(l/32), pixel) in the output, or out of range
    };
    struct Half {            // the first half of a decode
        int pp, img, g0, col;
        bool ok;
    };
    auto decode_a = [&](int f, Half &h) __attribute__((always_inline)) {
        int pp = f * 32 + lane % 32;
        h.ok = pp < p.positions && f < f1;
        pp = min(pp, p.positions - 1);
        const int R = mdiv(pp, p.wo_magic), ow = pp - R * p.wo;
        const int img = mdiv(R, p.ho_magic), oh = R - img * p.ho;
        h.pp = pp;
        h.img = img;
        h.g0 = img * p.hs + oh * p.sh;
        h.col = ring_base + ow * p.sw * RS_PIX + (lane / 32) * 16;
    };
    auto decode_b = [&](const Half &h, Frag &fr) __attribute__((always_inline)) {
        static_for<0, KH>([&](auto rc) {
            constexpr int kr = decltype(rc)::value;
            fr.ra[kr] = ((h.g0 + kr * p.dil_h) & p.nr_mask) * p.rowp + h.col;
        });
        const unsigned off = unsigned(pinned(((h.img * p.cout + 4 * (lane / 32)) * howo + (h.pp - h.img * howo)) * 4));
        fr.out_off = h.ok ? off : 0x80000000u;
    };
    const int tap_col = p.dil_w * RS_PIX;
    auto b_addr = [&](const Frag &fr, int sub) __attribute__((always_inline)) {
        const int k = sub / 2, h = sub % 2;
        return fr.ra[k / KW] + (k % KW) * tap_col + h * 32;
    };

    Frag cur, nxt;
    {
        Half h;
        decode_a(f0, h);
        decode_b(h, cur);
        decode_a(f0 + 1, h);
        decode_b(h, nxt);
    }
    v4i breg[RS_BR];
    static_for<0, RS_LOOK>([&](auto jc) {
        constexpr int j = decltype(jc)::value;
        breg[j % RS_BR] = *reinterpret_cast<const v4i *>(&lds[b_addr(cur, j)]);
    });

    v16i acc[2][2];
    unsigned prev_off = 0x80000000u;   // out_off of the fragment whose sums wait in the other accumulator set
    // Ring rows travel memory -> registers in one fragment and registers -> LDS at the end of the NEXT one: a load has
    // two fragments' worth of MFMAs (about a microsecond) to arrive before anything waits for it.  Two register sets,
    // one per fragment parity; set 1 starts with the rows of the tile's third fragment (the first fragment stores it).
    v4i fill[2][RS_MAXNEW][RS_FILLN];
    int fill_g0[2] = {0, 0}, fill_g1[2] = {0, 0};
    fill_g0[1] = rows_hi;
    fill_g1[1] = rows_end(f0 + 2);
    rows_hi = max(rows_hi, fill_g1[1]);
    static_for<0, RS_MAXNEW>([&](auto rc) {
        constexpr int r = decltype(rc)::value;
        static_for<0, RS_FILLN>([&](auto jc) {
            constexpr int j = decltype(jc)::value;
            fill[1][r][j] = fill_load(fill_g0[1] + r, fill_g0[1] + r < fill_g1[1], j);
        });
    });

    // exchange of the partial sums of accumulator set PAR: every wavefront writes its 2 x 16 registers as four
    // quarters, one per finishing wavefront; the finisher reads the four sources of its quarter.  The lane's base
    // addresses are pinned: from an address whose alignment it cannot see the compiler keeps the 16-byte accesses the
    // types promise (one whose visible terms are only 4-byte multiples is split into 8-byte accesses with an
    // address computation each).
    const int xw_base = pinned(xlane + s * 2048), xr_base = pinned(xlane + s * 8192);
    auto xchg_write = [&](auto parc, auto qc) __attribute__((always_inline)) {
        constexpr int PAR = decltype(parc)::value, q = decltype(qc)::value;
        static_for<0, 2>([&](auto cc) {
            constexpr int c = decltype(cc)::value;
            const v4i v = {acc[PAR][c][4 * q], acc[PAR][c][4 * q + 1], acc[PAR][c][4 * q + 2], acc[PAR][c][4 * q + 3]};
            *reinterpret_cast<v4i *>(&lds[xw_base + ((PAR * 4 + q) * 8 + c) * 1024]) = v;
        });
    };
    auto xchg_read = [&](auto parc, v4i(&part)[4][2]) __attribute__((always_inline)) {
        constexpr int PAR = decltype(parc)::value;
        static_for<0, 4>([&](auto wc_) {
            constexpr int w = decltype(wc_)::value;
            static_for<0, 2>([&](auto cc) {
                constexpr int c = decltype(cc)::value;
                part[w][c] = *reinterpret_cast<const v4i *>(&lds[xr_base + (PAR * 32 + w * 2 + c) * 1024]);
            });
        });
    };
    auto finish_store = [&](auto cc, auto ec, const v4i(&part)[4][2]) __attribute__((always_inline)) {
        constexpr int c = decltype(cc)::value, e = decltype(ec)::value;
        const int sum = (part[0][c][e] + part[1][c][e]) + (part[2][c][e] + part[3][c][e]);
        const float v = finish(sum, dqv[c][e], bv[c][e]);
        const int soff = ((cf + 32 * c + 8 * s + e) * howo) * 4;
#ifdef TSX_RS_NOSTORE   // timing experiments only
        if (v == 1.2345f)
#endif
        __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, v), out_rsrc, int(prev_off | cmask[c][e]), soff,
                                              STREAM ? 2 : 0);
    };

    // The work of one fragment, written sub-step by sub-step (one B operand read LOOK sub-steps ahead, two MFMAs)
    // with the other duties of the wavefront dealt over the sub-steps in between -- the scheduler may not move
    // anything across a sub-step's end, and a sub-step has room for about 14 vector instructions beside its MFMAs:
    //   1, 2    ring rows of fragment f+3: loads issued (two rows each)
    //   2-5     partial sums of fragment f-1 -> exchange buffer, a quarter each             (PREV)
    //   6       barrier                                                                      (PREV)
    //   6, 7    decode of fragment f+2's addresses
    //   7       the four partial sums of this wavefront's quarter <- LDS                     (PREV)
    //   8-15    sum, dequantize, bias, activation, store: one output register per sub-step   (PREV)
    //   16, 17  ring rows of fragment f+2 (loaded during the fragment before this one) -> LDS (two rows each)
    auto fragment = [&](auto parc, auto prevc, int f) __attribute__((always_inline)) {
        constexpr int PAR = decltype(parc)::value;
#ifdef TSX_RS_ABL_NOPREV
        constexpr bool PREV = false;
#else
        constexpr bool PREV = decltype(prevc)::value;
#endif
        v4i part[4][2];
        Frag nn;
        Half nh;
        static_for<0, SUB>([&](auto ic) {
            constexpr int i = decltype(ic)::value;
            // B operand LOOK sub-steps ahead: this fragment's, or the next one's first
#ifdef TSX_RS_ABL_NOB   // timing experiments only
            if (f < 0)
#endif
            if constexpr (i + RS_LOOK < SUB)
                breg[(i + RS_LOOK) % RS_BR] = *reinterpret_cast<const v4i *>(&lds[b_addr(cur, i + RS_LOOK)]);
            else
                breg[(i + RS_LOOK) % RS_BR] = *reinterpret_cast<const v4i *>(&lds[b_addr(nxt, i + RS_LOOK - SUB)]);
            static_for<0, 2>([&](auto cc) {
                constexpr int c = decltype(cc)::value;
                if constexpr (i == 0) {
                    v16i zero;
                    static_for<0, 16>([&](auto rc) { zero[decltype(rc)::value] = 0; });
                    acc[PAR][c] = __builtin_amdgcn_mfma_i32_32x32x32_i8(A[c][0][0], breg[0], zero, 0, 0, 0);
                } else {
                    acc[PAR][c] = __builtin_amdgcn_mfma_i32_32x32x32_i8(A[c][i / 2][i % 2], breg[i % RS_BR], acc[PAR][c], 0, 0, 0);
                }
            });
            if constexpr (i == 0) {
                fill_g0[PAR] = rows_hi;
                fill_g1[PAR] = rows_end(f + 3);
                rows_hi = max(rows_hi, fill_g1[PAR]);
            }
#ifdef TSX_RS_ABL_NOFILL
            if (f < 0)
#endif
            if constexpr (i == 1 || i == 2) {
                static_for<0, RS_MAXNEW / 2>([&](auto rc) {
                    constexpr int r = (i - 1) * (RS_MAXNEW / 2) + decltype(rc)::value;
                    static_for<0, RS_FILLN>([&](auto jc) {
                        constexpr int j = decltype(jc)::value;
                        fill[PAR][r][j] = fill_load(fill_g0[PAR] + r, fill_g0[PAR] + r < fill_g1[PAR], j);
                    });
                });
            }
#ifdef TSX_RS_ABL_NOXW
            if (f < 0)
#endif
            if constexpr (PREV && i >= 2 && i < 6) xchg_write(std::integral_constant<int, PAR ^ 1>{}, std::integral_constant<int, i - 2>{});
#ifdef TSX_RS_ABL_NOBAR
            if (f < 0)
#endif
            if constexpr (PREV && i == 6) lds_fence_barrier();
            if constexpr (i == 6) decode_a(f + 2, nh);
            if constexpr (i == 7) decode_b(nh, nn);
#ifdef TSX_RS_ABL_NOXR
            if (f < 0)
#endif
            if constexpr (PREV && i == 7) xchg_read(std::integral_constant<int, PAR ^ 1>{}, part);
#ifdef TSX_RS_ABL_NOEPI
            if (f < 0)
#endif
            if constexpr (PREV && i >= 8 && i < 16)
                finish_store(std::integral_constant<int, (i - 8) / 4>{}, std::integral_constant<int, (i - 8) % 4>{}, part);
#ifdef TSX_RS_ABL_NOFILL
            if (f < 0)
#endif
            if constexpr (i == 16 || i == 17) {
                static_for<0, RS_MAXNEW / 2>([&](auto rc) {
                    constexpr int r = (i - 16) * (RS_MAXNEW / 2) + decltype(rc)::value;
                    static_for<0, RS_FILLN>([&](auto jc) {
                        constexpr int j = decltype(jc)::value;
                        fill_store(fill_g0[PAR ^ 1] + r, fill_g0[PAR ^ 1] + r < fill_g1[PAR ^ 1], j, fill[PAR ^ 1][r][j]);
                    });
                });
            }
            __builtin_amdgcn_sched_barrier(0);
        });
        prev_off = cur.out_off;
        cur = nxt;
        nxt = nn;
    };

    int f = f0;
    RS_STAMP();
    fragment(std::integral_constant<int, 0>{}, std::false_type{}, f);
    RS_STAMP();
    ++f;
    while (f + 1 < f1) {
        fragment(std::integral_constant<int, 1>{}, std::true_type{}, f);
        RS_STAMP();
        fragment(std::integral_constant<int, 0>{}, std::true_type{}, f + 1);
        RS_STAMP();
        f += 2;
    }
    // the last fragment's sums: the same exchange and epilogue without MFMAs beside them
    auto drain = [&](auto parc) __attribute__((always_inline)) {
        static_for<0, 4>([&](auto qc) { xchg_write(parc, qc); });
        lds_fence_barrier();
        v4i part[4][2];
        xchg_read(parc, part);
        static_for<0, 2>([&](auto cc) {
            static_for<0, 4>([&](auto ec) { finish_store(cc, ec, part); });
        });
    };
    if (f < f1) {
        fragment(std::integral_constant<int, 1>{}, std::true_type{}, f);
        RS_STAMP();
        drain(std::integral_constant<int, 1>{});
    } else {
        drain(std::integral_constant<int, 0>{});
    }
#ifdef TSX_RS_STAMPS
    RS_STAMP();                       // stores issued
    __builtin_amdgcn_s_waitcnt(0);    // ... and left
    RS_STAMP();
#endif
}

}  // namespace

// Which layers take this kernel: 3x3 taps on exactly four channel blocks (193..256 input channels), more than 64
// output channels, window rows of at most 32 pixels, and rows that enter the ring no faster than the kernel loads
// them -- checked by walking every tile the way the kernel does.
void rs_plan(const WsGeom &g, WsPlan *pl) {
    pl->rs = false;
    if (!pl->ok || g.gemm || g.kh != 3 || g.kw != 3 || g.cblocks != 4 || pl->wm != 4) return;
    static const int mode = [] {
        const char *e = std::getenv("TSX_CONV_I8_RS");   // "0": never; "force": wherever the geometry allows (tests)
        return !e ? 0 : e[0] == '0' ? 0 : e[0] == 'f' ? 2 : 1;   // off unless asked for, until it beats the flat-tile kernel
    }();
    if (mode == 0) return;
    const int64_t positions = int64_t(g.n) * g.ho * g.wo;
    if (positions >= (int64_t(1) << 31) - 256) return;
    if (pl->packed_bytes >= (size_t(1) << 31)) return;
    if (int64_t(g.n) * g.hs * g.ws * g.cp >= (int64_t(1) << 31)) return;      // 32-bit buffer offsets
    if (int64_t(g.n) * g.cout * g.ho * g.wo >= (int64_t(1) << 29)) return;     // ... for the output as well
    if (!div_magic(g.wo, positions + 64) || !div_magic(g.ho, int64_t(g.n) * g.ho + 64)) return;   // the kernel divides by these
    const int wc = (g.wo - 1) * g.sw + (g.kw - 1) * g.dil_w + 1;
    if (wc > g.ws || wc * 4 > 64 * RS_FILLN) return;
    int rowp = wc * RS_PIX;
    rowp += ((g.wo * g.sw * RS_PIX - rowp) % 256 + 256) % 256;   // see fl_plan: conflict-free reads across a row's end
    const int total_frags = int((positions + 31) / 32);
    const int ctiles = (g.cout + 63) / 64;
    // one round of workgroups where the layer allows: as many position tiles as leave every CU at most one
    int frags = (total_frags + std::max(1, 256 / ctiles) - 1) / std::max(1, 256 / ctiles);
    if (mode == 2) frags = std::min(frags, 5);
    else if (frags < 8 || frags > 64) return;   // the weights (36 KiB per wavefront) are loaded once per tile
    frags = std::max(frags, 2);
    const int ptiles = (total_frags + frags - 1) / frags;
    if (mode != 2 && int64_t(ptiles) * ctiles < 160) return;
    // walk the tiles: rows the first two fragments need, rows entering per fragment, rows alive at once
    auto row_of = [&](int64_t pp) {
        const int64_t R = pp / g.wo, img = R / g.ho;
        return int(img * g.hs + (R - img * g.ho) * g.sh);
    };
    int need_nr = 0;
    for (int t = 0; t < ptiles; ++t) {
        const int f0 = t * frags, f1 = std::min(f0 + frags, total_frags);
        auto first = [&](int f) { return row_of(int64_t(std::min(f, f1 - 1)) * 32); };
        auto end = [&](int f) {
            return row_of(std::min<int64_t>(int64_t(std::min(f, f1 - 1)) * 32 + 31, positions - 1)) + (g.kh - 1) * g.dil_h + 1;
        };
        const int pro = end(f0 + 1) - first(f0);
        if (pro > RS_PRO) return;
        need_nr = std::max(need_nr, pro);
        for (int f = f0; f < f1; ++f) {
            if (end(f + 2) - end(f + 1) > RS_MAXNEW) return;
            need_nr = std::max(need_nr, end(f + 2) - first(f + 1));   // rows of f+2 enter while f+1's are read
        }
    }
    const int nr = need_nr <= 4 ? 4 : need_nr <= 8 ? 8 : 0;
    if (!nr) return;
    const size_t lds = size_t(4) * nr * rowp + 4096 + RS_XBUF;
    if (lds > size_t(RS_MAX_LDS)) return;
    pl->rs = true;
    pl->rs_frags = frags;
    pl->rs_ptiles = ptiles;
    pl->rs_nr = nr;
    pl->rs_rowp = rowp;
    pl->rs_wc = wc;
    pl->rs_lds = int(lds);
}

// Epilogues this kernel writes: fp32 NCHW with dequantize scales, optional bias and activation, every element in
// the activation's SIMD-body range.  Everything else stays on the other kernels (same packed weights).
bool rs_takes(const WsPlan &pl, const EpiParams &ep, int64_t count) {
    return pl.rs && ep.out_f32 && ep.dq && !ep.out_i8 && !ep.out_acc && !ep.st_out && !ep.residual && !ep.row_scale &&
           ep.act_body == count;
}

int rs_launch(const WsGeom &g, const WsPlan &pl, const int8_t *xs, const int8_t *packed, const EpiParams &ep,
              hipStream_t stream) {
    RsParams p{};
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
    p.sh = g.sh;
    p.sw = g.sw;
    p.dil_h = g.dil_h;
    p.dil_w = g.dil_w;
    p.frags = pl.rs_frags;
    p.positions = int(int64_t(g.n) * g.ho * g.wo);
    p.total_frags = (p.positions + 31) / 32;
    p.ptiles = pl.rs_ptiles;
    p.ctiles = (g.cout + 63) / 64;
    p.tiles = p.ptiles * p.ctiles;
    p.tiles_per_xcd = (p.tiles + 7) / 8;
    p.nr_mask = pl.rs_nr - 1;
    p.rowp = pl.rs_rowp;
    p.wc = pl.rs_wc;
    p.ring_bytes = pl.rs_nr * pl.rs_rowp;
    p.xs_bytes = unsigned(int64_t(g.n) * g.hs * g.ws * g.cp);
    p.out_bytes = unsigned(int64_t(g.n) * g.cout * g.ho * g.wo * 4);
    p.wo_magic = div_magic(p.wo, int64_t(p.positions) + 64);
    p.ho_magic = div_magic(p.ho, int64_t(g.n) * g.ho + 64);
#ifdef TSX_RS_STAMPS
    debug_phase_stamps(&p.stamps, &p.stamp_slots);
#endif
    // an output of L2 size or more that no fused consumer reads: stream it
#ifdef TSX_RS_ABL_CACHED
    const bool stream_out = false;
#else
    const bool stream_out = int64_t(p.out_bytes) >= (int64_t(16) << 20);
#endif
    const dim3 grid(unsigned(p.tiles_per_xcd * 8));
    const size_t lds_bytes = size_t(pl.rs_lds);
    static std::atomic<bool> granted[2][3][64];
    int dev = 0;
    TSX_HIP(hipGetDevice(&dev));
#define TSX_RS_LAUNCH(STREAM, ACT)                                                                             \
    do {                                                                                                       \
        auto kernel = conv_i8_rs_kernel<3, 3, STREAM, ACT>;                                                    \
        if (dev < 64 && !granted[STREAM][ACT][dev].load()) {                                                   \
            TSX_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),                                \
                                        hipFuncAttributeMaxDynamicSharedMemorySize, RS_MAX_LDS));              \
            granted[STREAM][ACT][dev].store(true);                                                             \
        }                                                                                                      \
        hipLaunchKernelGGL(kernel, grid, dim3(RS_THREADS), lds_bytes, stream, p);                              \
    } while (0)
    const int act = ep.act == TSX_ACT_MISH ? 2 : ep.act == TSX_ACT_RELU ? 1 : 0;
    if (stream_out) {
        if (act == 2) TSX_RS_LAUNCH(true, 2);
        else if (act == 1) TSX_RS_LAUNCH(true, 1);
        else TSX_RS_LAUNCH(true, 0);
    } else {
        if (act == 2) TSX_RS_LAUNCH(false, 2);
        else if (act == 1) TSX_RS_LAUNCH(false, 1);
        else TSX_RS_LAUNCH(false, 0);
    }
#undef TSX_RS_LAUNCH
    TSX_LAUNCH_CHECK("conv_i8_rs_kernel");
    return 0;
}

}  // namespace tsx
