// Weight-stationary int8 convolution for large 3x3 layers on 256 input channels (BASELINE config 2:
// 32x256x28x28 * 256x256x3x3).  Same arithmetic, staged input and packed weights as the window-stationary and
// flat-tile kernels (exact int32 sums of cpu::Conv2DQuantizedCore,
// src/kernels/cpu/quantized/conv2d_quantized_core.cpp:18-147, dequantized as its lines 81-106 do); what differs
// is which operand stays put and who does what:
//   * a workgroup owns 64 output channels and a run of F consecutive 32-position fragments of the batch-wide flat
//     position list (n, oh, ow).  It is 8 wavefronts, two per SIMD: a MULTIPLYING wavefront and a SERVING one.
//     A wavefront cannot issue anything else while one of its own MFMAs runs, so the two kinds are kept apart: the
//     multiplying wavefront issues MFMAs, the LDS reads that feed them and little else, and everything that can be
//     done by someone else is issued by its neighbour on the SIMD in the shadow of those MFMAs;
//   * multiplying wavefront s handles channel block s (64 input channels x 9 taps: a quarter of K) and keeps ITS
//     weights for all 64 output channels in registers for the whole kernel (2 x 9 x 2 MFMA operands of 16 bytes
//     per lane, 144 registers, loaded once): the K loop streams nothing but activations.  Per fragment it issues
//     36 MFMAs (32x32x32) into 2 accumulators and writes them, as four quarters, to an exchange buffer in LDS;
//   * serving wavefront s keeps the ring of staged rows in LDS that multiplying wavefront s reads (that block's 64
//     channels only; rows are loaded three fragments ahead of their first use and enter the ring two ahead), sums
//     the four partial sums (exact integers, any order) of quarter s of the previous fragment's outputs,
//     dequantizes, adds the bias, applies the activation and stores -- so output leaves the chip as a steady stream
//     under the multiplication instead of one burst behind it; only the last fragment's epilogue is exposed.  It
//     also works out the LDS addresses of the fragments to come and hands them over through LDS.
// Two barriers per fragment: one when the multiplying wavefronts have read a fragment's last operand (behind it the
// serving wavefronts may overwrite ring rows and the multiplying ones the exchange buffer), one when the partial
// sums and the new ring rows are in LDS.  MFMA operand layout as in conv2d_i8_ws.hip: lane l supplies row / column
// l%32 and the 16 K bytes of group l/32; accumulator register r of lane l is output channel 8*(r/4) + 4*(l/32) +
// r%4, position l%32.
#include "igemm_i8.hpp"
#ifdef TSX_MEASUREMENT_AIDS
#include "tsx_aids.h"
#endif

#include <algorithm>
#include <atomic>
#include <cstdlib>

namespace tsx {

constexpr int RS_PIX = 80;        // LDS bytes per ring pixel (64 channels + 16 pad: conflict-free 16-byte reads)
constexpr int RS_THREADS = 512;   // 8 wavefronts: a multiplying and a serving one per SIMD
constexpr int RS_FILLN = 2;       // 16-byte chunks per lane per ring row: rows of up to 32 window pixels
constexpr int RS_MAXNEW = 2;      // staged rows loaded for the ring per fragment (the fill runs ahead of the need)
constexpr int RS_PRO = 8;         // staged rows the first two fragments of a tile may need (= the largest ring)
constexpr int RS_BR = 6;          // B operand register ring (divides the 18 sub-steps of a fragment)
constexpr int RS_LOOK = 5;        // sub-steps a B operand is read ahead of its MFMAs
constexpr int RS_XBUF = 32768;    // partial-sum exchange, one of two: [4 finishers][4 sources][2 accumulators][1 KiB]
constexpr int RS_A_GENERAL = 3;   // MFMA operands of the second accumulator's weights (of 18) that live in the general register half, with all of the first's
constexpr int RS_ABUF = 8192;     // fragment addresses: [4 wavefronts][2 parities][1 KiB]
constexpr int RS_MAX_LDS = 160 * 1024;

struct RsParams : EpiParams {
    const int8_t *xs;   // staged activations [n][hs][ws][cp]
    const int8_t *wp;   // packed weights [kstep][coutp/32][2 halves][64 lanes][16], K order (channel block, kh, kw)
    int n, cout, coutp, ho, wo, hs, ws, cp;
    int sh, sw, dil_h;
    int frags;            // fragments per tile
    int total_frags;      // ceil(positions / 32)
    int positions;        // n * ho * wo
    int ptiles, ctiles, tiles, tiles_per_xcd;
    int nr_mask;          // ring rows - 1 (ring rows: 4 or 8)
    int rowp, wc;         // LDS bytes per ring row, window pixels per row
    int ring_bytes;       // (nr_mask + 1) * rowp
    unsigned xs_bytes, out_bytes;
    unsigned wo_magic, ho_magic;
#ifdef TSX_MEASUREMENT_AIDS
    unsigned long long *stamps;   // [workgroup][wavefront][24][wall clock, shader clock]
    int stamp_slots;
#endif
};
#ifdef TSX_MEASUREMENT_AIDS
// the buffer tsx_debug_phase_stamps named (null = off)
static std::atomic<unsigned long long *> g_stamps{nullptr};
static std::atomic<size_t> g_stamp_slots{0};
#endif

namespace {

// floor(n / d) by the host's magic number (div_magic; the plan takes this kernel only where one exists)
__device__ __forceinline__ int mdiv(int n, unsigned magic) { return int(__umulhi(unsigned(n), magic)); }

// Keeps the computation of v where it is written and hides what it was computed from: a value that only feeds one
// arm of a select would otherwise be sunk into a conditional block of its own (a branch ends the scheduling region
// around it), and an LDS address whose visible terms are only 4-byte multiples loses the 16-byte accesses its type
// promises (they are split into 8-byte ones with an address computation each).
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

// ACT: 0 = none / relu / leaky_relu picked by uniform selects, 1 = relu, 2 = Mish in its fast form
template <bool STREAM, int ACT>
__global__ __launch_bounds__(RS_THREADS) __attribute__((amdgpu_waves_per_eu(2, 2))) void conv_i8_rs_kernel(RsParams p) {
    constexpr int KH = 3, KW = 3, TAPS = KH * KW, SUB = 2 * TAPS;
    static_assert(SUB % RS_BR == 0, "the B ring must divide a fragment's sub-steps");
    extern __shared__ __attribute__((aligned(16))) int8_t lds[];
    // Workgroups are dealt round-robin to the 8 XCDs (own L2 each): every XCD gets a contiguous run of tiles, and
    // the cout tiles of one run of positions are neighbours in it.
    const int tile = (blockIdx.x & 7) * p.tiles_per_xcd + (blockIdx.x >> 3);
    if (tile >= p.tiles) return;
    const int ptile = tile / p.ctiles, ctile = tile - ptile * p.ctiles;
    const int lane = threadIdx.x % 64;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / 64);
    const int s = wave & 3;            // channel block (multiplying) / finished quarter (serving); also the SIMD
    const bool serving = wave >= 4;
    const int f0 = ptile * p.frags;
    const int f1 = min(f0 + p.frags, p.total_frags);
    const int cf = ctile * 64;
    const int howo = p.ho * p.wo;

    // ---- LDS map: 4 rings | 4 x 1 KiB dump (target of predicated-off ring stores) | exchange | fragment addresses
    const int ring_base = s * p.ring_bytes;
    const int dump_addr = 4 * p.ring_bytes + s * 1024 + lane * 16;
    const int xbuf = 4 * p.ring_bytes + 4096;
    const int abuf = pinned(xbuf + 2 * RS_XBUF + s * 2048 + lane * 16);

#ifdef TSX_MEASUREMENT_AIDS
    int stamp_k = 0;
    auto stamp = [&]() __attribute__((always_inline)) {
        const int slot = ((blockIdx.x * 8 + wave) * 24 + stamp_k) * 2;
        if (p.stamps && lane == 0 && stamp_k < 24 && slot + 2 <= p.stamp_slots) {
            p.stamps[slot] = wall_clock64();
            p.stamps[slot + 1] = clock64();
        }
        ++stamp_k;
    };
#define RS_STAMP() stamp()
// per fragment / round as well with -DTSX_MEASUREMENT_AIDS=2: the stamps inside the loops cost the kernel a quarter of
// its speed, so the measurement build leaves them out and divides the loop's time by its fragments
#if TSX_MEASUREMENT_AIDS >= 2
#define RS_STAMP_FINE() stamp()
#else
#define RS_STAMP_FINE() ((void)0)
#endif
#else
#define RS_STAMP() ((void)0)
#define RS_STAMP_FINE() ((void)0)
#endif
    RS_STAMP();

    // ---- fragment decode: LDS address of the lane's pixel per kernel row (what the multiplying wavefront needs),
    // and the lane's place in the output (what the serving one needs)
    auto decode = [&](int f, int (&ra)[KH], unsigned &out_off) __attribute__((always_inline)) {
        int pp = f * 32 + lane % 32;
        const bool ok = pp < p.positions && f < f1;
        pp = min(pp, p.positions - 1);
        const int R = mdiv(pp, p.wo_magic), ow = pp - R * p.wo;
        const int img = mdiv(R, p.ho_magic), oh = R - img * p.ho;
        const int g0 = img * p.hs + oh * p.sh;
        const int col = ring_base + ow * p.sw * RS_PIX + (lane / 32) * 16;
        static_for<0, KH>([&](auto rc) {
            constexpr int kr = decltype(rc)::value;
            ra[kr] = ((g0 + kr * p.dil_h) & p.nr_mask) * p.rowp + col;
        });
        const unsigned off = unsigned(pinned(((img * p.cout + 4 * (lane / 32)) * howo + (pp - img * howo)) * 4));
        out_off = ok ? off : 0x80000000u;
    };

    if (!serving) {
        // ================================================================ the multiplying wavefront
        const __amdgpu_buffer_rsrc_t w_rsrc =
            __builtin_amdgcn_make_buffer_rsrc(const_cast<int8_t *>(p.wp), 0, 0x7fffffff, 0x00020000);
        // this wavefront's weights, K-step by K-step in the order the MFMAs use them
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
        }
        int cur[KH], nxt[KH];
        {
            unsigned unused;
            decode(f0, cur, unused);
            decode(f0 + 1, nxt, unused);
        }
        // Where the weights live: most of them in the accumulation registers' half of the file next to the
        // accumulators (an MFMA reads its A operand from either half), the rest in the general one.  The serving
        // wavefronts run the same kernel and need their registers in the general half; a wavefront's budget
        // (256 at two per SIMD) is the sum of the largest demand on either half.
        static_for<0, TAPS>([&](auto kc_) {
            constexpr int k = decltype(kc_)::value;
            static_for<0, 2>([&](auto hc) {
                constexpr int h = decltype(hc)::value;
                v4i &w0 = A[0][k][h];
                asm volatile("" : "+v"(w0));
                v4i &w1 = A[1][k][h];
                if constexpr (2 * k + h < RS_A_GENERAL) asm volatile("" : "+v"(w1));
                else asm volatile("" : "+a"(w1));
            });
        });
        lds_fence_barrier();   // the ring rows of the first two fragments and the third's addresses are in LDS
        RS_STAMP();
        auto b_read = [&](const int (&ra)[KH], auto subc) __attribute__((always_inline)) {
            constexpr int sub = decltype(subc)::value, k = sub / 2, h = sub % 2;
            return *reinterpret_cast<const v4i *>(&lds[ra[k / KW] + (k % KW) * RS_PIX + h * 32]);
        };
        v4i breg[RS_BR];
        static_for<0, RS_LOOK>([&](auto jc) { breg[decltype(jc)::value % RS_BR] = b_read(cur, jc); });
        v16i acc[2][2];
        const int xw_base = pinned(xbuf + s * 2048 + lane * 16);
        // partial sums of accumulator set PAR, quarter q of accumulator c -> exchange buffer PAR
        auto xchg_write = [&](auto parc, auto ic) __attribute__((always_inline)) {
            constexpr int PAR = decltype(parc)::value, q = decltype(ic)::value / 2, c = decltype(ic)::value % 2;
            const v4i v = {acc[PAR][c][4 * q], acc[PAR][c][4 * q + 1], acc[PAR][c][4 * q + 2], acc[PAR][c][4 * q + 3]};
            *reinterpret_cast<v4i *>(&lds[xw_base + PAR * RS_XBUF + (q * 8 + c) * 1024]) = v;
        };
        // One fragment: 18 sub-steps of one B operand read (LOOK sub-steps ahead) and two MFMAs.  A store to LDS
        // holds the MFMA pipe up for some twenty cycles however it is placed, and eight in a row for four hundred:
        // the previous fragment's partial sums (the other accumulator set) leave one store per sub-step.
        auto fragment = [&](auto parc, auto prevc, int f) __attribute__((always_inline)) {
            constexpr int PAR = decltype(parc)::value;
            constexpr bool PREV = decltype(prevc)::value;
            v4i nn4;
            static_for<0, SUB>([&](auto ic) {
                constexpr int i = decltype(ic)::value;
                if constexpr (i + RS_LOOK < SUB) breg[(i + RS_LOOK) % RS_BR] = b_read(cur, std::integral_constant<int, i + RS_LOOK>{});
                else breg[(i + RS_LOOK) % RS_BR] = b_read(nxt, std::integral_constant<int, i + RS_LOOK - SUB>{});
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
                // the addresses of fragment f+2, worked out by the serving wavefront two fragments ago
                if constexpr (i == 1) nn4 = *reinterpret_cast<const v4i *>(&lds[abuf + (f & 1) * 1024]);
                if constexpr (PREV && i >= 2 && i < 10) xchg_write(std::integral_constant<int, PAR ^ 1>{}, std::integral_constant<int, i - 2>{});
                // Every operand of this fragment has been read (the last one a whole sub-step ago) and the previous
                // fragment's partial sums are in LDS: behind this barrier the serving wavefronts overwrite the ring
                // rows this fragment alone used and finish the previous fragment.
                if constexpr (i == SUB - RS_LOOK - 1) lds_fence_barrier();
                __builtin_amdgcn_sched_barrier(0);
            });
            static_for<0, KH>([&](auto rc) {
                constexpr int kr = decltype(rc)::value;
                cur[kr] = nxt[kr];
                nxt[kr] = nn4[kr];
            });
            RS_STAMP_FINE();
        };
        int f = f0;
        fragment(std::integral_constant<int, 0>{}, std::false_type{}, f);
        ++f;
        while (f + 1 < f1) {
            fragment(std::integral_constant<int, 1>{}, std::true_type{}, f);
            fragment(std::integral_constant<int, 0>{}, std::true_type{}, f + 1);
            f += 2;
        }
        // the last fragment's partial sums have no MFMAs to leave under
        if (f < f1) {
            fragment(std::integral_constant<int, 1>{}, std::true_type{}, f);
            static_for<0, 8>([&](auto ic) { xchg_write(std::integral_constant<int, 1>{}, ic); });
        } else {
            static_for<0, 8>([&](auto ic) { xchg_write(std::integral_constant<int, 0>{}, ic); });
        }
        RS_STAMP();
        lds_fence_barrier();
        return;
    }

    // ==================================================================== the serving wavefront
    const __amdgpu_buffer_rsrc_t xs_rsrc =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<int8_t *>(p.xs), 0, p.xs_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t out_rsrc = __builtin_amdgcn_make_buffer_rsrc(p.out_f32, 0, p.out_bytes, 0x00020000);
    // uniform: last staged row (+1) that fragment f reads, f clamped to this tile
    auto rows_end = [&](int f) __attribute__((always_inline)) {
        f = min(f, f1 - 1);
        const int pp = min(f * 32 + 31, p.positions - 1);
        const int R = mdiv(pp, p.wo_magic);
        const int img = mdiv(R, p.ho_magic);
        return img * p.hs + (R - img * p.ho) * p.sh + (KH - 1) * p.dil_h + 1;
    };
    // uniform: first staged row that fragment f reads, f clamped to this tile
    auto rows_first = [&](int f) __attribute__((always_inline)) {
        f = min(f, f1 - 1);
        const int R = mdiv(f * 32, p.wo_magic);
        const int img = mdiv(R, p.ho_magic);
        return img * p.hs + (R - img * p.ho) * p.sh;
    };
    const int tile_rows_end = rows_end(f1 - 1);
    const int ring_rows = p.nr_mask + 1;
    // Ring fill of one staged row: lane l moves chunks l and l + 64 (pixel q / 4, 16 bytes q % 4 of this block's 64
    // channels).  The row's place in memory and in the ring is uniform (scalar offsets); what a lane adds is
    // constant; a lane beyond the row's pixels fetches nothing (out-of-range buffer offset) and stores to the dump.
    int fill_src[RS_FILLN], fill_dst[RS_FILLN];
    bool fill_on[RS_FILLN];
    static_for<0, RS_FILLN>([&](auto jc) {
        constexpr int j = decltype(jc)::value;
        const int q = lane + 64 * j, pix = q >> 2, chunk = q & 3;
        fill_on[j] = pix < p.wc;
        fill_src[j] = fill_on[j] ? pix * p.cp + s * 64 + chunk * 16 : int(0x80000000u);
        fill_dst[j] = ring_base + pix * RS_PIX + chunk * 16;
    });
    const int row_bytes = p.ws * p.cp;
    auto fill_load = [&](int g, bool need, int j) __attribute__((always_inline)) {
        return __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(
                                           xs_rsrc, need ? fill_src[j] : int(0x80000000u), g * row_bytes, 0));
    };
    auto fill_store = [&](int g, int j, const v4i &v) __attribute__((always_inline)) {
        const int dst = pinned(fill_dst[j] + (g & p.nr_mask) * p.rowp);
        *reinterpret_cast<v4i *>(&lds[fill_on[j] ? dst : dump_addr]) = v;
    };

    // ---- prologue: as many rows as the ring holds, from the tile's first
    int rows_hi;   // staged rows below this are in the ring (or on their way)
    {
        const int g_first = rows_first(f0);
        const int g_end = min(g_first + ring_rows, tile_rows_end);
        v4i pro[RS_PRO][RS_FILLN];
        static_for<0, RS_PRO>([&](auto ic) {
            constexpr int i = decltype(ic)::value;
            static_for<0, RS_FILLN>([&](auto jc) {
                constexpr int j = decltype(jc)::value;
                pro[i][j] = fill_load(min(g_first + i, g_end - 1), true, j);   // rows beyond the last: the last again
            });
        });
        static_for<0, RS_PRO>([&](auto ic) {
            constexpr int i = decltype(ic)::value;
            static_for<0, RS_FILLN>([&](auto jc) {
                constexpr int j = decltype(jc)::value;
                fill_store(min(g_first + i, g_end - 1), j, pro[i][j]);
            });
        });
        rows_hi = g_end;
    }
    // The fill runs ahead of the need: round r loads up to RS_MAXNEW rows -- as far as the ring will have room when
    // they are stored, at the start of round r+2 behind the barrier that tells that nobody reads fragment r+1's rows
    // any more (a row may replace one that lies below fragment r+2's first).  A load has two fragments' MFMAs to
    // arrive (with one, the round was as long as the load's latency); two register sets, one per round parity.  The
    // plan takes this kernel only where this schedule has every fragment's rows in the ring in time (rs_plan walks
    // it).  The loads are a fixed number per round, predicated (an out-of-range offset fetches nothing), and so are
    // the output stores issued behind them: the wait for the loads can then be counted (one counter covers loads and
    // stores) and never waits for a store.
    v4i fill[2][RS_MAXNEW][RS_FILLN];
    int fill_g0[2] = {rows_hi, rows_hi}, fill_n[2] = {0, 0};
    auto fill_issue = [&](auto setc, int r) __attribute__((always_inline)) {
        constexpr int S = decltype(setc)::value;
        fill_g0[S] = rows_hi;
        fill_n[S] = max(min(min(rows_first(r + 2) + ring_rows, tile_rows_end) - rows_hi, RS_MAXNEW), 0);
        rows_hi += fill_n[S];
        static_for<0, RS_MAXNEW>([&](auto rc) {
            constexpr int r = decltype(rc)::value;
            static_for<0, RS_FILLN>([&](auto jc) {
                constexpr int j = decltype(jc)::value;
                fill[S][r][j] = fill_load(fill_g0[S] + r, r < fill_n[S], j);
            });
        });
    };
    auto fill_commit = [&](auto setc) __attribute__((always_inline)) {
        constexpr int S = decltype(setc)::value;
        // every loaded register counts as used here, wanted or not: a register whose row is not wanted would
        // otherwise be handed to another value while its load is still in flight, and that value's first write
        // would wait for the load in the middle of the round
        static_for<0, RS_MAXNEW>([&](auto rc) {
            static_for<0, RS_FILLN>([&](auto jc) {
                v4i &v = fill[S][decltype(rc)::value][decltype(jc)::value];
                asm volatile("" : "+v"(v));
            });
        });
        static_for<0, RS_MAXNEW>([&](auto rc) {
            constexpr int r = decltype(rc)::value;
            if (r < fill_n[S]) static_for<0, RS_FILLN>([&](auto jc) {
                constexpr int j = decltype(jc)::value;
                fill_store(fill_g0[S] + r, j, fill[S][r][j]);
            });
        });
    };
    // fragment addresses for the multiplying wavefront of this SIMD: slot f & 1 holds those of fragment f
    auto publish = [&](int f, unsigned &out_off) __attribute__((always_inline)) {
        int ra[KH];
        decode(f, ra, out_off);
        const v4i v = {ra[0], ra[1], ra[2], 0};
        *reinterpret_cast<v4i *>(&lds[abuf + (f & 1) * 1024]) = v;
    };

    // ---- per-lane constants of the finished quarter: register (c, i) is channel cf + 32c + 8s + 4(l/32) + i
    float dqv[2][4], bv[2][4];
    const int co_lane = cf + 8 * s + 4 * (lane / 32);
    static_for<0, 2>([&](auto cc) {
        constexpr int c = decltype(cc)::value;
        static_for<0, 4>([&](auto ic) {
            constexpr int i = decltype(ic)::value;
            const int co = co_lane + 32 * c + i;
            dqv[c][i] = p.dq[min(co, p.cout - 1)];
            bv[c][i] = p.bias ? p.bias[min(co, p.cout - 1)] : -0.f;   // v + (-0) = v, bit for bit: no bias, no branch
        });
    });
    // dequantize -> bias -> activation of one sum: relu and leaky_relu in their SIMD-body forms
    // (src/kernels/cpu/relu.cpp:30-52, leaky_relu.cpp:41-66; rs_takes admits only tensors that lie in the body)
    const bool is_relu = p.act == TSX_ACT_RELU, is_leaky = p.act == TSX_ACT_LEAKY_RELU;
    const float slope = p.slope;
    auto finish = [&](int sum, float dq, float bias) __attribute__((always_inline)) {
        const float v = __fadd_rn(__fmul_rn(float(sum), dq), bias);
        if constexpr (ACT == 2) {
            return apply_act_conv_i8(v, TSX_ACT_MISH_FAST, 0.f, true);
        } else if constexpr (ACT == 1) {
            return v > 0.f ? v : 0.f;
        } else {
            const float mx = v > 0.f ? v : 0.f;
            const float mn = v < 0.f ? v : 0.f;
            const float leaky = __builtin_fmaf(slope, mn, mx);
            return is_relu ? mx : is_leaky ? leaky : v;
        }
    };
    // the four partial sums of this wavefront's quarter (exchange buffer `par`) -> fp32 output at lane offset `off`
    const int xr_base = pinned(xbuf + s * 8192 + lane * 16);
    auto finish_quarter = [&](auto fullc, int par, unsigned off) __attribute__((always_inline)) {
        constexpr bool FULL = decltype(fullc)::value;   // all 64 channels of the tile exist
        const int xr = xr_base + par * RS_XBUF;
        static_for<0, 2>([&](auto cc) {
            constexpr int c = decltype(cc)::value;
            v4i part[4];
            static_for<0, 4>([&](auto wc_) {
                constexpr int w = decltype(wc_)::value;
                part[w] = *reinterpret_cast<const v4i *>(&lds[xr + (w * 2 + c) * 1024]);
            });
            static_for<0, 4>([&](auto ec) {
                constexpr int e = decltype(ec)::value;
                const int sum = (part[0][e] + part[1][e]) + (part[2][e] + part[3][e]);
                const float v = finish(sum, dqv[c][e], bv[c][e]);
                const int soff = ((cf + 32 * c + 8 * s + e) * howo) * 4;
                // a channel beyond cout: out-of-range offset, nothing is written
                const unsigned o = (FULL || co_lane + 32 * c + e < p.cout) ? off : 0x80000000u;
                __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, v), out_rsrc, int(o), soff, STREAM ? 2 : 0);
            });
        });
    };

    const bool full_tile = cf + 64 <= p.cout;
    auto finish_fragment = [&](int par, unsigned off) __attribute__((always_inline)) {
        if (full_tile) finish_quarter(std::true_type{}, par, off);
        else finish_quarter(std::false_type{}, par, off);
    };

    // The serving wavefront decodes every fragment three ahead of the multiplication; the output offsets it finds on
    // the way wait in a queue until the fragment's sums arrive, two rounds behind the multiplication:
    // off_a = fragment r-2, ... off_e = fragment r+2.
    unsigned off_a = 0x80000000u, off_b = 0x80000000u, off_c, off_d, off_e;
    {
        int unused[KH];
        decode(f0, unused, off_c);
        decode(f0 + 1, unused, off_d);
    }
    publish(f0 + 2, off_e);
    lds_fence_barrier();   // the multiplying wavefronts' first barrier
    RS_STAMP();

    // One fragment of the multiplying wavefronts = one round here, from the barrier in fragment r-1 to the one in
    // fragment r.
    // One fragment of the multiplying wavefronts = one round here, from the barrier in fragment r-1 to the one in
    // fragment r; PAR = parity of r - f0.
    auto round = [&](auto parc, int r) __attribute__((always_inline)) {
        constexpr int PAR = decltype(parc)::value;
        fill_commit(std::integral_constant<int, PAR>{});         // rows of fragment r+1, loaded two rounds ago
        fill_issue(std::integral_constant<int, PAR>{}, r);
        finish_fragment(PAR, off_a);   // fragment r-2: its sums came in during fragment r-1 (none yet: the offset is
                                       // out of range and nothing is written)
        unsigned off_f;
        publish(r + 3, off_f);
        off_a = off_b;
        off_b = off_c;
        off_c = off_d;
        off_d = off_e;
        off_e = off_f;
        lds_fence_barrier();
        RS_STAMP_FINE();
    };
    fill_issue(std::integral_constant<int, 1>{}, f0 - 1);   // the set that round f0+1 stores
    for (int r = f0; r < f1; r += 2) {
        round(std::integral_constant<int, 0>{}, r);
        if (r + 1 < f1) round(std::integral_constant<int, 1>{}, r + 1);
    }
    RS_STAMP();
    // off_a = fragment f1-2, off_b = fragment f1-1
    if (f1 - 2 >= f0) finish_fragment((f1 - f0) & 1, off_a);
    lds_fence_barrier();   // the last fragment's partial sums
    finish_fragment((f1 - 1 - f0) & 1, off_b);
#ifdef TSX_MEASUREMENT_AIDS
    RS_STAMP();                       // stores issued
    __builtin_amdgcn_s_waitcnt(0);    // ... and left
    RS_STAMP();
#endif
}

}  // namespace

// Which layers take this kernel: 3x3 taps (any stride, rows of any dilation) on exactly four channel blocks (193..256
// input channels), more than 64 output channels, window rows of at most 32 pixels, and rows that enter the ring no faster than the kernel loads
// them -- checked by walking every tile the way the kernel does.
void rs_plan(const WsGeom &g, WsPlan *pl) {
    pl->rs = false;
    if (!pl->ok || g.gemm || g.kh != 3 || g.kw != 3 || g.dil_w != 1 || g.cblocks != 4 || pl->wm != 4) return;
    // TSX_CONV_I8_RS, read at every plan: "0" never; "force" wherever the geometry allows, with tiles of at most 5
    // fragments, "forceN" with tiles of N (2..9) fragments (tests of the kernel on small layers); otherwise the layers
    // measured to gain
    const char *e = std::getenv("TSX_CONV_I8_RS");
    const int mode = !e ? 1 : e[0] == '0' ? 0 : e[0] == 'f' ? 2 : 1;
    const int forced_frags = mode == 2 && e[5] >= '2' && e[5] <= '9' && !e[6] ? e[5] - '0' : 0;
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
    if (mode == 2) frags = forced_frags ? forced_frags : std::min(frags, 5);
    else if (frags < 8 || frags > 64) return;   // the weights (36 KiB per wavefront) are loaded once per tile
    frags = std::max(frags, 2);
    const int ptiles = (total_frags + frags - 1) / frags;
    if (mode != 2 && int64_t(ptiles) * ctiles < 160) return;
    // walk every tile through the kernel's fill schedule: the smallest ring with which each fragment's rows are
    // there in time
    auto row_of = [&](int64_t pp) {
        const int64_t R = pp / g.wo, img = R / g.ho;
        return int(img * g.hs + (R - img * g.ho) * g.sh);
    };
    int nr = 0;
    for (const int ring : {4, 8}) {
        bool ok = true;
        for (int t = 0; t < ptiles && ok; ++t) {
            const int f0 = t * frags, f1 = std::min(f0 + frags, total_frags);
            auto first = [&](int f) { return row_of(int64_t(std::min(f, f1 - 1)) * 32); };
            auto end = [&](int f) {
                return row_of(std::min<int64_t>(int64_t(std::min(f, f1 - 1)) * 32 + 31, positions - 1)) + (g.kh - 1) * g.dil_h + 1;
            };
            const int tile_end = end(f1 - 1);
            int rows_hi = std::min(first(f0) + ring, tile_end);          // the prologue
            ok = rows_hi >= end(f0 + 1) && end(f0 + 1) - first(f0) <= ring;
            for (int r = f0 - 1; r < f1 && ok; ++r) {                    // round r loads; its rows are stored in round r+2
                rows_hi += std::max(std::min(std::min(first(r + 2) + ring, tile_end) - rows_hi, RS_MAXNEW), 0);
                ok = rows_hi >= end(r + 3)                               // fragment r+3 reads them behind round r+2's barrier
                     && end(r + 3) - first(r + 2) <= ring;               // ... while fragment r+2's are still in use
            }
        }
        if (ok) {
            nr = ring;
            break;
        }
    }
    if (!nr) return;
    const size_t lds = size_t(4) * nr * rowp + 4096 + 2 * RS_XBUF + RS_ABUF;
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
// the activation's SIMD-body range; of the two forms of Mish the fast one (the exact one's double-precision chain
// does not fit beside the serving wavefronts' row registers).  Everything else stays on the other kernels (same
// packed weights).
bool rs_takes(const WsPlan &pl, const EpiParams &ep, int64_t count) {
    return pl.rs && ep.out_f32 && ep.dq && !ep.out_i8 && !ep.out_acc && !ep.st_out && !ep.residual && !ep.row_scale &&
           ep.act_body == count && ep.act != TSX_ACT_MISH;
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
#ifdef TSX_MEASUREMENT_AIDS
    p.stamps = g_stamps.load();
    p.stamp_slots = int(g_stamp_slots.load());
#endif
    // an output of L2 size or more that no fused consumer reads: stream it
    const bool stream_out = int64_t(p.out_bytes) >= (int64_t(16) << 20);
    const dim3 grid(unsigned(p.tiles_per_xcd * 8));
    const size_t lds_bytes = size_t(pl.rs_lds);
    static std::atomic<bool> granted[2][3][64];
    int dev = 0;
    TSX_HIP(hipGetDevice(&dev));
#define TSX_RS_LAUNCH(STREAM, ACT)                                                                             \
    do {                                                                                                       \
        auto kernel = conv_i8_rs_kernel<STREAM, ACT>;                                                    \
        if (dev < 64 && !granted[STREAM][ACT][dev].load()) {                                                   \
            TSX_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),                                \
                                        hipFuncAttributeMaxDynamicSharedMemorySize, RS_MAX_LDS));              \
            granted[STREAM][ACT][dev].store(true);                                                             \
        }                                                                                                      \
        hipLaunchKernelGGL(kernel, grid, dim3(RS_THREADS), lds_bytes, stream, p);                              \
    } while (0)
    const int act = ep.act == TSX_ACT_MISH_FAST ? 2 : ep.act == TSX_ACT_RELU ? 1 : 0;
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

#ifdef TSX_MEASUREMENT_AIDS
extern "C" int tsx_debug_phase_stamps(void *buffer_dev, size_t bytes) {
    if (buffer_dev && (bytes < 8 * 24 * 16 || reinterpret_cast<uintptr_t>(buffer_dev) % 8 != 0))
        return tsx::fail(TSX_E_INVALID, "debug_phase_stamps: buffer must be 8-byte aligned and hold at least one workgroup's stamps");
    tsx::g_stamp_slots.store(buffer_dev ? bytes / 8 : 0);
    tsx::g_stamps.store(static_cast<unsigned long long *>(buffer_dev));
    return 0;
}
#endif
