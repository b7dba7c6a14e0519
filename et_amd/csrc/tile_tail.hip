// Layer tail (encoder/encoder.cu:33-44: O_linear, skip + LayerNorm, MLP1 with
// GELU, MLP2, skip + LayerNorm) as PAIRS of workgroups over one row panel.
//
// Why.  With one workgroup per 32-row panel every CU streams the whole of the
// three weight matrices (2.1 MB at BERT-base / 80 %) through the L2 -> CU path
// for 32 rows of work, two MFMAs per kilobyte, and a workgroup is one chain of
// dependent phases with nothing beside it on its CU.  Here the hidden dimension
// of the feed-forward block is split over the two workgroups of a pair:
// workgroup `half` of panel P runs the projection and the first LayerNorm on
// the panel (both do: 11 % duplicated work), then the first feed-forward linear
// for ITS half of the hidden columns and the second linear over those columns
// only.  Two panel heights are built (template parameter MS, 16-row subtiles
// per panel): 64 rows - four MFMAs per kilobyte of W, a CU streams 1.2 MB
// instead of 2.1, one workgroup per CU - and 32 rows - 77 KB of LDS, so that two
// workgroups share a CU and one's waits are the other's issue slots.  Neither
// beats the one-workgroup form of tile_linear.hip at BERT-base sizes (8192
// rows, 80 % pruned: 74 and 89 us against 53): with hidden buffers of 192
// columns, which is what fits, a segment of the second linear is one or two
// tile pairs long and the per-segment work (flush, hand-over, start vector)
// outweighs what the split saves.  Both stay available as an option
// (et_tuning_set "tile_tail_pair") and are tested like the default.
//
// The two partial sums of a panel meet without any workgroup waiting for the
// other one.  The first half of the panel's rows is finished by whoever arrives
// second at that row-half's counter, the second half likewise; a workgroup
// visits the other row-half first.  At a row-half it looks at the counter: zero
// means the partner has not published yet, so it writes its own fp32 partial
// (scratch) and adds one to the counter - if the add returns one the partner
// arrived in between.  Whoever finds (or gets) one reads the partner's partial,
// adds the two, runs bias + skip + LayerNorm 2 on those rows, stores them and
// resets the counter.  When the pair runs in step each workgroup writes one
// row-half, reads one and normalises one; when one is late the other leaves
// both of its partials and exits, and the late one finishes both.  No spin, no
// assumption that the partner is resident.  a + b == b + a in fp32, so the
// bits do not depend on who finishes.
//
// Inside a workgroup (8 waves).  LDS holds the panel and two 192-column hidden
// buffers INTERLEAVED per row (row stride = panel width + 2 x 208 halves, which
// keeps ds_read_b128 conflict-free), so a tile's X operand is "lane's row base
// + one byte offset" whether it multiplies the panel (projection, first
// linear) or a hidden buffer (second linear): one stage body serves all three.
// Every wave walks ONE continuous stream of tile pairs that the host lays out
// for it at plan time (its block-rows of the projection; then, per 192-column
// phase p, one or two hidden block-rows of the first linear and its output
// block-rows of the second linear over chunk p, the first linear one phase
// ahead), through a register pipeline of 4 or 8 pairs that never drains.  Where
// a segment of the stream ends, a control word that travels with the segment's
// last pair (next to its operand offsets, so it costs no memory request of its
// own) says what to do with the finished sums: GELU and store into a hidden
// buffer, or add into one of the wave's output accumulators; and which LDS
// event counter to wait for or to signal (hidden buffer complete / hidden
// buffer free), exactly as an s_barrier would order them but without stopping
// a wave that is not a whole phase ahead.  Waits are bounded; a wave that gives
// up sets the process's wait-status word, which the next launch reports.  Both
// LayerNorms run on the accumulators where they are (a panel row's columns are
// spread over the 8 waves; row sums meet in LDS), so no staging tile is needed
// for them.
#include "tile_plan.h"

#include <algorithm>
#include <cstring>
#include <type_traits>

namespace et {

#ifndef TT_NWAVES
#define TT_NWAVES 8
#endif
constexpr int TT_WAVES = TT_NWAVES;       // 8: two per SIMD and workgroup; 12: three (64-row panels: 168 registers each)
static_assert(TT_WAVES == 8 || TT_WAVES == 12, "eight or twelve waves");
// A panel has 16 * MS rows, MS = 4 or 2 (template parameter of the kernel): 64 rows, one workgroup per CU,
// or 32 rows, two workgroups per CU (either the two of a panel or of two different ones), whose chains of
// dependent phases overlap.
constexpr int TT_HB = 12;                 // hidden block-rows per phase
constexpr int TT_HC = 16 * TT_HB;         // hidden columns per phase
constexpr int TT_HW = (TT_HC + 16) * 2;   // bytes of one hidden buffer inside an LDS row
constexpr int TT_MAX_PHASES = 16;         // per half: counters F[16], S[16]
constexpr int TT_MAX_PANELS = 8192;       // counters per program: 2 per panel
// Tile pairs in flight per wave: 8 where a wave has 256 registers (eight waves, 64-row panels), else 4.  The
// host lays every stream out as a multiple of TT_PAD pairs, which suits both.
constexpr int TT_PAD = 8;
constexpr int tt_depth(int ms) { return (TT_WAVES == 8 && ms == 4) ? 8 : 4; }
// stages the X fragments are read ahead of their MFMAs
#ifndef TT_XA
#define TT_XA 1
#endif

template <int D, int MS = 4> struct TtGeom {
    static constexpr int NB = (D / 16 + TT_WAVES - 1) / TT_WAVES; // output block-rows per wave
    static constexpr int XW = (D + ((D & 31) ? 0 : 16)) * 2;      // bytes of the panel part of an LDS row
    static constexpr int RS = XW + 2 * TT_HW;                     // LDS row stride, == 32 (mod 64)
    static constexpr int CT = 16 * MS * RS;                       // event counters: F[16], S[16]
    static constexpr int ZV = CT + 2 * TT_MAX_PHASES * 4;         // 16 zero floats
    static constexpr int MISC = ZV + 64;                          // workgroup broadcasts
    static constexpr int BI = MISC + 64;                          // first linear's bias (halves), 32 B per block-row
    static_assert(RS % 64 == 32, "row stride must be == 32 (mod 64) bytes");
};
constexpr int TT_BI_BYTES = 32; // per hidden block-row

// A pair's record in the stream: 16 bytes, {offset of tile A, control, offset of
// tile B, control} - lanes 0-31 read the first half, lanes 32-63 the second.  An
// offset is the LDS byte offset of the tile's X columns inside the lane's row
// (panel part or a hidden buffer).  The control word is 0 except on the last
// pair of a segment:
//   bit 0      set
//   bit 1      the segment is a hidden block-row of the first linear (GELU, store)
//   bits 2-4   accumulator the sums are added to (7: none)
//   bits 5-8   slot of the hidden block-row in its 192-column buffer
//   bits 9-12  phase p of the segment (buffer p & 1, counters F[p] / S[p])
//   bit 13     wait for S[p - 2] (all waves) before the hidden store
//   bit 14     signal F[p] (hidden block-row) or S[p] (second linear) afterwards
//   bit 15     before the NEXT segment's first operand is read, wait for
//   bits 16-19   F[p'] to reach
//   bits 20-23   this count minus one
//   bits 24-31 what the next segment's sums start from: 255 zeros, else the
//              bias of hidden block-row (index inside this half)
constexpr int TT_C_SET = 1, TT_C_HID = 2, TT_C_WAITF = 1 << 13, TT_C_SIG = 1 << 14, TT_C_WAITN = 1 << 15;

struct TtArgs {
    const f16 *pairs;
    const int *rec;
    const int *wtab; // per (half, wave): projection pair base, stages; feed-forward pair base, stages; first start vector; initial wait
    const f16 *attn, *input;
    f16 *Y;
    const f16 *biasO, *bias1, *bias2, *g1, *b1, *g2, *b2;
    unsigned long long *ws;
    int *sync;   // per panel: two row-half counters
    int *status; // set when a bounded wait gives up
    int M, npanels, per_xcd, spin;
    int hb0[2], nb1h[2]; // first hidden block-row and count per half
};

template <int I> using tt_ic = std::integral_constant<int, I>;
template <int B, int E, class F>
__device__ __forceinline__ void tt_static_for(F &&f) {
    if constexpr (B < E) {
        f(tt_ic<B>());
        tt_static_for<B + 1, E>(f);
    }
}

// One pair's operands: 16 bytes of W per lane, the lane's X offset and the
// control word.  The pair's address is wave-uniform and the lane's part a 32-bit
// offset kept opaque in place, so the loads need no vector address arithmetic.
__device__ __forceinline__ void tt_load_pair(const char *wq, const char *rq, unsigned &lo, unsigned &lw,
                                             f16x8 &w, int &o, int &c) {
    typedef int i32x2 __attribute__((ext_vector_type(2)));
    asm("" : "+v"(lo), "+v"(lw));
    const i32x2 r = *reinterpret_cast<const i32x2 *>(rq + lo);
    o = r[0];
    c = r[1];
    w = *reinterpret_cast<const f16x8 *>(wq + lw);
}

// A wave's LDS operations are executed in the order it issued them, so an add
// that follows the wave's stores in program order is seen after them by
// everyone: no wait for the stores (a release fence would be an s_waitcnt, i.e.
// an LDS round trip per signal), only a barrier for the compiler.
__device__ __forceinline__ void tt_signal(unsigned *ctr, int lane) {
    asm volatile("" ::: "memory");
    if (lane == 0)
        __hip_atomic_fetch_add(ctr, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    asm volatile("" ::: "memory");
}
// Bounded: after `spin` polls the wave sets the status word and goes on (the
// result of this launch is then wrong, and the next launch reports it).
__device__ __forceinline__ void tt_wait(unsigned *ctr, unsigned target, int spin, int *status, int lane) {
    for (int s = 0;; s++) {
        if ((unsigned)__builtin_amdgcn_readfirstlane(
                (int)__hip_atomic_load(ctr, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP)) >= target)
            break;
        if (s >= spin) {
            if (lane == 0)
                __hip_atomic_store(status, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
            break;
        }
        __builtin_amdgcn_s_sleep(1);
    }
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

// Sum over the four lanes l, l^16, l^32, l^48, result in all four (gfx950 row
// swaps in the vector ALU; the empty asm keeps the optimiser from reasoning
// about the swapped copies).
__device__ __forceinline__ float tt_xor_sum_16_32(float v) {
    unsigned a = __builtin_bit_cast(unsigned, v), b = a;
    asm("" : "+v"(b));
    auto r = __builtin_amdgcn_permlane32_swap(a, b, false, false);
    unsigned x0 = r[0], x1 = r[1];
    asm("v_add_f32 %0, %0, %1" : "+v"(x0) : "v"(x1));
    unsigned y1 = x0;
    asm("" : "+v"(y1));
    auto q = __builtin_amdgcn_permlane16_swap(x0, y1, false, false);
    unsigned z0 = q[0], z1 = q[1];
    asm("v_add_f32 %0, %0, %1" : "+v"(z0) : "v"(z1));
    return __builtin_bit_cast(float, z0);
}

template <int RS, int MS>
__device__ __forceinline__ void tt_read_x(f16x8 (&x)[MS], const char *xl, int off) {
    const char *p = xl + off;
#pragma unroll
    for (int k = 0; k < MS; k++)
        x[k] = *reinterpret_cast<const f16x8 *>(p + k * 16 * RS);
}

// The stream: n stages (a multiple of DEPTH), pair q's operands in slot q %
// DEPTH of w / o / c (the first DEPTH requested by the caller), X fragments
// read TT_XA stages ahead, MS MFMAs per stage into cur[] (one per 16-row
// subtile).  at_end(ctl, reread) runs where a stage finishes a segment (its
// pair's control word is not 0); reread() reads the fragments of the pairs that
// are already on their way once more, for a handler that has to wait before
// they may be read.
template <int RS, int MS, int DEPTH, class AtEnd>
__device__ __forceinline__ void tt_stream(const char *xl, const char *wq, const char *rq, int n,
                                          unsigned &lane_lo, unsigned &lane_lw, f16x8 (&w)[DEPTH],
                                          int (&o)[DEPTH], int (&c)[DEPTH], f32x4 (&cur)[MS],
                                          AtEnd &&at_end) {
    constexpr int NX = TT_XA + 1;
    static_assert(DEPTH % NX == 0 && TT_XA < DEPTH, "fragment buffers rotate inside the unrolled group");
    f16x8 xf[NX][MS];
#pragma unroll
    for (int i = 0; i < TT_XA; i++)
        tt_read_x<RS, MS>(xf[i], xl, o[i]);
    const char *wp = wq + DEPTH * 1024, *rp = rq + DEPTH * 16;
    for (int q = 0; q < n; q += DEPTH) {
        tt_static_for<0, DEPTH>([&](auto ic) {
            constexpr int I = decltype(ic)::value;
            tt_read_x<RS, MS>(xf[(I + TT_XA) % NX], xl, o[(I + TT_XA) % DEPTH]);
            // keep the reads above the MFMAs (the scheduler otherwise sinks them
            // and every stage waits out the LDS latency)
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int k = 0; k < MS; k++)
                cur[k] = mfma16x16x32(w[I], xf[I % NX][k], cur[k]);
            const int ctl = __builtin_amdgcn_readfirstlane(c[I]);
            // pair q + I + DEPTH (unconditional: the stream is followed by spare pairs)
            tt_load_pair(wp + I * 1024, rp + I * 16, lane_lo, lane_lw, w[I], o[I], c[I]);
            if (ctl != 0)
                at_end(ctl, [&]() {
#pragma unroll
                    for (int i = 1; i <= TT_XA; i++)
                        tt_read_x<RS, MS>(xf[(I + i) % NX], xl, o[(I + i) % DEPTH]);
                });
        });
        wp += DEPTH * 1024;
        rp += DEPTH * 16;
    }
}

// a += c with tied operands: the sum replaces the accumulator in its own
// registers.  (Left to the compiler, the accumulators of the NB cases below are
// shuffled between registers at every merge.  The case number in the text also
// keeps the optimiser from sinking the NB blocks into one that addresses acc[]
// with a run-time index, i.e. through scratch memory.)
template <int K>
__device__ __forceinline__ void tt_add_tied(f32x4 &a, const f32x4 &c) {
    float a0 = a[0], a1 = a[1], a2 = a[2], a3 = a[3];
    asm volatile("v_add_f32 %0, %0, %4 ; accumulator %8\n\tv_add_f32 %1, %1, %5\n\t"
                 "v_add_f32 %2, %2, %6\n\tv_add_f32 %3, %3, %7"
                 : "+v"(a0), "+v"(a1), "+v"(a2), "+v"(a3)
                 : "v"(c[0]), "v"(c[1]), "v"(c[2]), "v"(c[3]), "n"(K));
    a = f32x4{a0, a1, a2, a3};
}
// acc[j] += cur for a wave-uniform run-time j (no accumulator for j >= NB).  A
// sequence of independent ifs with something opaque between them: as an if /
// else chain it becomes a switch whose lowering copies the accumulators around.
template <int NB, int MS>
__device__ __forceinline__ void tt_acc_add(f32x4 (&acc)[NB][MS], int j, const f32x4 (&cur)[MS]) {
    tt_static_for<0, NB>([&](auto kc) {
        constexpr int k = decltype(kc)::value;
        if (j == k) {
#pragma unroll
            for (int ms = 0; ms < MS; ms++)
                tt_add_tied<k>(acc[k][ms], cur[ms]);
        }
        asm volatile("; after case %0" ::"n"(k));
    });
}

// Skip + LayerNorm on values held in the accumulator layout: lane (c16, g4) of
// wave w holds, per block-row j and 16-row subtile ms, columns 16*(NB*w + j) +
// 4*g4 .. +3 of panel row 16*(ms0 + ms) + c16, already as x = half(y) + skip
// (zeros in block-rows beyond the matrix).  The math of skip_layernorm.hip (fp32
// mean, two-pass biased variance, eps 1e-6; kernels/skip_layernorm.cu:4-43).  A
// row's partial sums of the eight waves meet in the hidden-buffer part of that
// row in LDS (free whenever this runs) and are added in wave order.  Two
// workgroup barriers.
template <int D, int NMS>
__device__ __forceinline__ void tt_ln(f16x4 (&x)[TtGeom<D>::NB][NMS], int ms0,
                                      const f16x4 (&gam)[TtGeom<D>::NB], const f16x4 (&bet)[TtGeom<D>::NB],
                                      char *smem, int wave, int c16, int g4, int nvalid) {
    constexpr int NB = TtGeom<D>::NB, RS = TtGeom<D>::RS, XW = TtGeom<D>::XW;
    typedef _Float16 h2 __attribute__((ext_vector_type(2)));
    const float inv_n = 1.0f / (float)D;
    float mean[NMS], rstd[NMS];
    auto total = [&](int ms, int at) {
        const f32x4 *p = reinterpret_cast<const f32x4 *>(smem + (16 * (ms0 + ms) + c16) * RS + XW + at);
        const f32x4 a0 = p[0], a1 = p[1];
        float t = ((a0[0] + a0[1]) + (a0[2] + a0[3])) + ((a1[0] + a1[1]) + (a1[2] + a1[3]));
        if constexpr (TT_WAVES == 12) {
            const f32x4 a2 = p[2];
            t += (a2[0] + a2[1]) + (a2[2] + a2[3]);
        }
        return t;
    };
#pragma unroll
    for (int ms = 0; ms < NMS; ms++) {
        float s = 0.f;
#pragma unroll
        for (int j = 0; j < NB; j++) {
            s = __builtin_amdgcn_fdot2(h2{x[j][ms][0], x[j][ms][1]}, h2{(f16)1, (f16)1}, s, false);
            s = __builtin_amdgcn_fdot2(h2{x[j][ms][2], x[j][ms][3]}, h2{(f16)1, (f16)1}, s, false);
        }
        s = tt_xor_sum_16_32(s);
        if (g4 == 0)
            *reinterpret_cast<float *>(smem + (16 * (ms0 + ms) + c16) * RS + XW + wave * 4) = s;
    }
    __syncthreads();
#pragma unroll
    for (int ms = 0; ms < NMS; ms++)
        mean[ms] = total(ms, 0) * inv_n;
#pragma unroll
    for (int ms = 0; ms < NMS; ms++) {
        float v = 0.f;
#pragma unroll
        for (int j = 0; j < NB; j++) {
            float vj = 0.f;
#pragma unroll
            for (int r = 0; r < 4; r++) {
                const float d = (float)x[j][ms][r] - mean[ms];
                vj += d * d;
            }
            v += j < nvalid ? vj : 0.f; // (a block-row beyond the matrix is not part of the row)
        }
        v = tt_xor_sum_16_32(v);
        if (g4 == 0)
            *reinterpret_cast<float *>(smem + (16 * (ms0 + ms) + c16) * RS + XW + 64 + wave * 4) = v;
    }
    __syncthreads();
#pragma unroll
    for (int ms = 0; ms < NMS; ms++) {
        rstd[ms] = rsqrtf(total(ms, 64) * inv_n + 1e-6f);
        const float shift = -mean[ms] * rstd[ms];
#pragma unroll
        for (int j = 0; j < NB; j++)
#pragma unroll
            for (int r = 0; r < 4; r++) // ((x - mean) * rstd) * gamma + beta, the first step as one fma
                x[j][ms][r] = (f16)(__builtin_fmaf((float)x[j][ms][r], rstd[ms], shift) * (float)gam[j][r] +
                                    (float)bet[j][r]);
    }
}

template <int D, int MS>
__global__ void __launch_bounds__(TT_WAVES * 64, MS == 2 ? 4 : 1) tile_tail_pair_kernel(const TtArgs a) {
    using G = TtGeom<D, MS>;
    constexpr int NB = G::NB, RS = G::RS, XW = G::XW, nbrD = D / 16;
    constexpr int TT_BM = 16 * MS, TT_DEPTH = tt_depth(MS), HS = MS / 2; // rows; pairs in flight; subtiles per row-half
    extern __shared__ __attribute__((aligned(16))) unsigned char tt_smem[];
    char *const smem = reinterpret_cast<char *>(tt_smem);
    // the two workgroups of a panel get neighbouring slots of ONE XCD (hardware
    // round-robins consecutive workgroup ids over the 8 XCDs): they fetch the
    // same panel and exchange their partial sums through that XCD's L2
    const int vid = (blockIdx.x & 7) * a.per_xcd + (blockIdx.x >> 3);
    const int panel = vid >> 1, half = vid & 1;
    if (panel >= a.npanels)
        return;
    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lane = tid & 63, c16 = lane & 15, g4 = lane >> 4, khalf8 = (g4 & 1) * 8, hi = lane >> 5;
    const int m0 = panel * TT_BM;
    unsigned *const ctr = reinterpret_cast<unsigned *>(smem + G::CT);
    int *const misc = reinterpret_cast<int *>(smem + G::MISC);
    const int nvalid = min(max(nbrD - NB * wave, 0), NB); // this wave's block-rows inside the matrix

    // the panel (attention output): DMA, wave w takes rows w, w + 8, ...
    {
        constexpr int PCPR = D / 8; // 16-byte pieces per row, <= 124
        for (int r = wave; r < TT_BM; r += TT_WAVES)
            if (m0 + r < a.M) {
                const f16 *src = a.attn + (size_t)(m0 + r) * D;
                f16 *dst = reinterpret_cast<f16 *>(smem + r * RS);
                if (lane < PCPR)
                    load_lds16(src + lane * 8, dst);
                if (PCPR > 64 && 64 + lane < PCPR)
                    load_lds16(src + (64 + lane) * 8, dst + 512);
            }
    }
    if (tid < 2 * TT_MAX_PHASES)
        ctr[tid] = 0u;
    if (tid >= 64 && tid < 80)
        reinterpret_cast<float *>(smem + G::ZV)[tid - 64] = 0.f;
    {
        const int hb0 = half ? a.hb0[1] : a.hb0[0], nb1h = half ? a.nb1h[1] : a.nb1h[0];
        f16 *bi = reinterpret_cast<f16 *>(smem + G::BI);
        for (int i = tid; i < nb1h * 16; i += TT_WAVES * 64)
            bi[i] = a.bias1[hb0 * 16 + i];
    }
    typedef const __attribute__((address_space(4))) int *ScalarInts;
    const ScalarInts wt = (ScalarInts)a.wtab + (half * TT_WAVES + wave) * 8;
    const int o_base = wt[0], o_n = wt[1], f_base = wt[2], f_n = wt[3], f_init = wt[4], f_wait0 = wt[5];
    unsigned lane_lo = hi * 8u, lane_lw = (hi * 256 + c16 * 16 + khalf8) * 2u;
    const char *const pairs = reinterpret_cast<const char *>(a.pairs);
    const char *const recs = reinterpret_cast<const char *>(a.rec);
    f16x8 w[TT_DEPTH];
    int o[TT_DEPTH], c[TT_DEPTH];
#pragma unroll
    for (int i = 0; i < TT_DEPTH; i++)
        tt_load_pair(pairs + (size_t)(o_base + i) * 1024, recs + (size_t)(o_base + i) * 16, lane_lo, lane_lw, w[i],
                     o[i], c[i]);
    __builtin_amdgcn_s_waitcnt(0x0F70); // vmcnt(0): this wave's part of the panel has landed
    __syncthreads();

    f32x4 acc[NB][MS], cur[MS];
#pragma unroll
    for (int j = 0; j < NB; j++)
#pragma unroll
        for (int ms = 0; ms < MS; ms++)
            acc[j][ms] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int ms = 0; ms < MS; ms++)
        cur[ms] = f32x4{0.f, 0.f, 0.f, 0.f};
    const char *const xl = smem + c16 * RS + khalf8 * 2;

    // ---- the projection: this wave's NB block-rows over the whole panel ----
    tt_stream<RS, MS, TT_DEPTH>(xl, pairs + (size_t)o_base * 1024, recs + (size_t)o_base * 16, o_n, lane_lo, lane_lw,
                                w, o, c, cur, [&](int ctl, auto &&) {
                                    tt_acc_add<NB, MS>(acc, (ctl >> 2) & 7, cur);
#pragma unroll
                                    for (int ms = 0; ms < MS; ms++)
                                        cur[ms] = f32x4{0.f, 0.f, 0.f, 0.f};
                                });

    // ---- bias + skip (the layer input) + LayerNorm 1, written over the panel ----
    {
        // every operand is requested before any is used, from addresses that are
        // legal for all lanes (block-rows beyond the matrix read column 0 and are
        // zeroed afterwards): one memory latency for the whole step
        f16x4 x[NB][MS], gam[NB], bet[NB], bo[NB];
#pragma unroll
        for (int j = 0; j < NB; j++) {
            const int col = j < nvalid ? (NB * wave + j) * 16 + g4 * 4 : 0;
            bo[j] = *reinterpret_cast<const f16x4 *>(a.biasO + col);
            gam[j] = *reinterpret_cast<const f16x4 *>(a.g1 + col);
            bet[j] = *reinterpret_cast<const f16x4 *>(a.b1 + col);
#pragma unroll
            for (int ms = 0; ms < MS; ms++)
                x[j][ms] = *reinterpret_cast<const f16x4 *>(
                    a.input + (size_t)min(m0 + 16 * ms + c16, a.M - 1) * D + col);
        }
#pragma unroll
        for (int j = 0; j < NB; j++) {
            const f32x4 bf = __builtin_convertvector(bo[j], f32x4);
            const f16x4 zero = f16x4{0, 0, 0, 0};
#pragma unroll
            for (int ms = 0; ms < MS; ms++) {
                // half(acc + bias) is the linear's output as the reference stores it; the
                // skip connection is added in half (kernels/skip_layernorm.cu:20)
                const f16x4 v = __builtin_convertvector(acc[j][ms] + bf, f16x4) + x[j][ms];
                x[j][ms] = j < nvalid ? v : zero;
            }
        }
        // the first pairs of the feed-forward stream travel under the LayerNorm
#pragma unroll
        for (int i = 0; i < TT_DEPTH; i++)
            tt_load_pair(pairs + (size_t)(f_base + i) * 1024, recs + (size_t)(f_base + i) * 16, lane_lo, lane_lw,
                         w[i], o[i], c[i]);
        tt_ln<D, MS>(x, 0, gam, bet, smem, wave, c16, g4, nvalid);
        // (every wave has passed a barrier since its last read of the attention panel)
#pragma unroll
        for (int j = 0; j < NB; j++)
            if (j < nvalid)
#pragma unroll
                for (int ms = 0; ms < MS; ms++)
                    *reinterpret_cast<f16x4 *>(smem + (16 * ms + c16) * RS + ((NB * wave + j) * 16 + g4 * 4) * 2) =
                        x[j][ms];
    }
#pragma unroll
    for (int j = 0; j < NB; j++)
#pragma unroll
        for (int ms = 0; ms < MS; ms++)
            acc[j][ms] = f32x4{0.f, 0.f, 0.f, 0.f};
    __syncthreads(); // the feed-forward input panel is complete

    // ---- the feed-forward block over this half of the hidden columns ----
    {
        auto start_vector = [&](int idx) { // what a segment's sums start from: zeros or a hidden block-row's bias
            f32x4 init = f32x4{0.f, 0.f, 0.f, 0.f};
            if (idx != 255) // (most segments start from zeros: no LDS round trip for those)
                init = __builtin_convertvector(
                    *reinterpret_cast<const f16x4 *>(smem + G::BI + idx * TT_BI_BYTES + g4 * 8), f32x4);
#pragma unroll
            for (int ms = 0; ms < MS; ms++)
                cur[ms] = init;
        };
        start_vector(f_init);
        if (f_wait0 >= 0)
            tt_wait(ctr + (f_wait0 & 15), (unsigned)(f_wait0 >> 8), a.spin, a.status, lane);
        tt_stream<RS, MS, TT_DEPTH>(
            xl, pairs + (size_t)f_base * 1024, recs + (size_t)f_base * 16, f_n, lane_lo, lane_lw, w, o, c, cur,
            [&](int ctl, auto &&reread) {
                const int p = (ctl >> 9) & 15;
                if (ctl & TT_C_HID) {
                    // a finished hidden block-row (its bias was the starting value): GELU,
                    // rounded to half as the reference stores it, into the hidden buffer
                    if (ctl & TT_C_WAITF) { // ... once everyone has finished reading what it held before
                        tt_wait(ctr + TT_MAX_PHASES + p - 2, TT_WAVES, a.spin, a.status, lane);
                    }
                    char *hp = smem + c16 * RS + (XW + (p & 1) * TT_HW + ((ctl >> 5) & 15) * 32) + g4 * 8;
#pragma unroll
                    for (int ms = 0; ms < MS; ms++) {
                        *reinterpret_cast<f16x4 *>(hp + ms * 16 * RS) =
                            gelu4(__builtin_convertvector(cur[ms], f16x4));
                        __builtin_amdgcn_sched_barrier(0); // one subtile at a time: few temporaries
                    }
                }
                // (not in an else branch: as a part of that if / else the accumulators were
                // given a second set of registers behind the handler; a hidden block-row's
                // control word names accumulator 7, which does not exist)
                tt_acc_add<NB, MS>(acc, (ctl >> 2) & 7, cur);
                if (ctl & TT_C_SIG)
                    tt_signal(ctr + ((ctl & TT_C_HID) ? p : TT_MAX_PHASES + p), lane);
                if (ctl & TT_C_WAITN) {
                    // the next segment multiplies a hidden buffer: wait until it is complete
                    // and read the next pair's fragments again
                    tt_wait(ctr + ((ctl >> 16) & 15), (unsigned)((ctl >> 20) & 15) + 1u, a.spin, a.status, lane);
                    reread();
                }
                start_vector((int)((unsigned)ctl >> 24));
            });
    }

    // ---- the two halves' partial sums meet; bias + skip + LayerNorm 2; store ----
    f16x4 b2[NB], gam[NB], bet[NB];
#pragma unroll
    for (int j = 0; j < NB; j++) {
        const int col = j < nvalid ? (NB * wave + j) * 16 + g4 * 4 : 0;
        b2[j] = *reinterpret_cast<const f16x4 *>(a.bias2 + col);
        gam[j] = *reinterpret_cast<const f16x4 *>(a.g2 + col);
        bet[j] = *reinterpret_cast<const f16x4 *>(a.b2 + col);
    }
    // Scratch of (panel, half, row-half): [wave][j][subtile][piece][lane] 8-byte
    // words, coalesced both ways.  Every access to it is an agent-scope atomic
    // (relaxed): such a store is complete at the device's coherence point when the
    // wave's memory counter says so, and such a load does not take a stale line
    // from another XCD's L2 - the data of one row-half costs what it is, not a
    // write-back and invalidation of the whole L2 as a device-scope fence would.
    // Order: all waves wait for their stores, barrier, THEN thread 0 touches the
    // counter; a reader loads only after the barrier behind thread 0's counter read.
    constexpr size_t PART = (size_t)TT_WAVES * NB * HS * 2 * 64; // words per (panel, half, row-half)
    auto publish = [&](int h) {
        unsigned long long *dst =
            a.ws + ((size_t)(panel * 2 + half) * 2 + h) * PART + (size_t)wave * NB * HS * 2 * 64 + lane;
#pragma unroll
        for (int j = 0; j < NB; j++)
#pragma unroll
            for (int m2 = 0; m2 < HS; m2++) {
                const f32x4 v = h ? acc[j][HS + m2] : acc[j][m2]; // (selected, not indexed: acc stays in registers)
                typedef float f32x2 __attribute__((ext_vector_type(2)));
                __hip_atomic_store(dst + ((j * HS + m2) * 2 + 0) * 64,
                                   __builtin_bit_cast(unsigned long long, f32x2{v[0], v[1]}), __ATOMIC_RELAXED,
                                   __HIP_MEMORY_SCOPE_AGENT);
                __hip_atomic_store(dst + ((j * HS + m2) * 2 + 1) * 64,
                                   __builtin_bit_cast(unsigned long long, f32x2{v[2], v[3]}), __ATOMIC_RELAXED,
                                   __HIP_MEMORY_SCOPE_AGENT);
            }
        __builtin_amdgcn_s_waitcnt(0x0F70); // vmcnt(0): this wave's stores are complete
    };
    auto finish = [&](int h) {
        const unsigned long long *src =
            a.ws + ((size_t)(panel * 2 + (1 - half)) * 2 + h) * PART + (size_t)wave * NB * HS * 2 * 64 + lane;
        typedef float f32x2 __attribute__((ext_vector_type(2)));
        f32x4 other[NB][HS];
#pragma unroll
        for (int j = 0; j < NB; j++)
#pragma unroll
            for (int m2 = 0; m2 < HS; m2++) {
                const f32x2 lo = __builtin_bit_cast(
                    f32x2, __hip_atomic_load(src + ((j * HS + m2) * 2 + 0) * 64, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
                const f32x2 hi2 = __builtin_bit_cast(
                    f32x2, __hip_atomic_load(src + ((j * HS + m2) * 2 + 1) * 64, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
                other[j][m2] = f32x4{lo[0], lo[1], hi2[0], hi2[1]};
            }
        f16x4 x[NB][HS];
#pragma unroll
        for (int j = 0; j < NB; j++) {
            const f32x4 bf = __builtin_convertvector(b2[j], f32x4);
            const f16x4 zero = f16x4{0, 0, 0, 0};
#pragma unroll
            for (int m2 = 0; m2 < HS; m2++) {
                const int col = j < nvalid ? (NB * wave + j) * 16 + g4 * 4 : 0;
                const f16x4 sk = *reinterpret_cast<const f16x4 *>(smem + (16 * (HS * h + m2) + c16) * RS + col * 2);
                const f32x4 mine = h ? acc[j][HS + m2] : acc[j][m2];
                const f16x4 v = __builtin_convertvector((mine + other[j][m2]) + bf, f16x4) + sk;
                x[j][m2] = j < nvalid ? v : zero;
            }
        }
        tt_ln<D, HS>(x, HS * h, gam, bet, smem, wave, c16, g4, nvalid);
        // in place over the skip operand (each lane overwrites what it read), then
        // whole rows leave with 16-byte stores
#pragma unroll
        for (int j = 0; j < NB; j++)
            if (j < nvalid)
#pragma unroll
                for (int m2 = 0; m2 < HS; m2++)
                    *reinterpret_cast<f16x4 *>(smem + (16 * (HS * h + m2) + c16) * RS +
                                               ((NB * wave + j) * 16 + g4 * 4) * 2) = x[j][m2];
        __syncthreads();
        constexpr int PR = D / 8;
        for (int i = tid; i < 16 * HS * PR; i += TT_WAVES * 64) {
            const int r = 16 * HS * h + i / PR, cc = i % PR;
            if (m0 + r < a.M)
                *reinterpret_cast<u32x4 *>(a.Y + (size_t)(m0 + r) * D + cc * 8) =
                    *reinterpret_cast<const u32x4 *>(smem + r * RS + cc * 16);
        }
        if (tid == 0) // ready for the next launch
            __hip_atomic_store(a.sync + 2 * panel + h, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    };
    const int other_h = 1 - half;
    publish(other_h); // the partner finishes that row-half unless it has long gone
    __syncthreads();  // (also: every wave has left the hidden buffers)
    if (tid == 0) {
        // one round trip: arrive at the other row-half's counter, look at the own one
        misc[0] = __hip_atomic_fetch_add(a.sync + 2 * panel + other_h, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        misc[1] = __hip_atomic_load(a.sync + 2 * panel + half, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    __syncthreads();
    const int arrived_other = misc[0]; // 1: the partner's partial of that row-half was there first: finish it here
    int arrived_own = misc[1];         // 1: the partner's partial of the own row-half is in scratch
    if (arrived_own == 0) {
        // not yet: leave the own partial as well; whoever adds second finishes
        publish(half);
        __syncthreads();
        if (tid == 0)
            misc[2] = __hip_atomic_fetch_add(a.sync + 2 * panel + half, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __syncthreads();
        arrived_own = misc[2];
    }
    if (arrived_own != 0)
        finish(half);
    if (arrived_other != 0) {
        __syncthreads(); // (the statistics area and the broadcast words are free again)
        finish(other_h);
    }
}

// ---------------------------------------------------------------------------
// host side: the program
// ---------------------------------------------------------------------------
struct TailProgram {
    int D = 0, Hd = 0;
    int nphase[2] = {0, 0}, hb0[2] = {0, 0}, nb1h[2] = {0, 0};
    f16 *d_pairs = nullptr;
    int *d_rec = nullptr, *d_wtab = nullptr, *d_sync = nullptr;
    size_t npairs = 0; // including padding (for reports)
};

void tail_program_destroy(TailProgram *p) {
    if (!p)
        return;
    et_free(p->d_pairs);
    et_free(p->d_rec);
    et_free(p->d_wtab);
    et_free(p->d_sync);
    delete p;
}

// et_tuning_set("tile_tail_pair"): 0 never, 1 where there are enough panels (32-row panels), 2 wherever it
// applies with 64-row panels, 3 wherever it applies with 32-row panels
static int g_tail_pair = 0;
static int tail_ms() { return g_tail_pair == 2 ? 4 : 2; } // 16-row subtiles per panel
static int g_tail_spin = 1 << 22;    // et_tuning_set("tile_wait_spin"): polls before a bounded LDS wait gives up
void set_tail_pair(int v) { g_tail_pair = v; }
bool tail_pair_forced() { return g_tail_pair >= 2; }
bool tail_pair_enabled() { return g_tail_pair != 0; }
void set_tail_spin(int v) { g_tail_spin = v < 0 ? (1 << 22) : v; }
int tail_spin() { return g_tail_spin; }

static int tail_geom(int D, int *nb, int *xw) {
    if (D <= 0 || D % 16 || D / 16 > 6 * TT_WAVES)
        return 0;
    *nb = (D / 16 + TT_WAVES - 1) / TT_WAVES;
    *xw = (D + ((D & 31) ? 0 : 16)) * 2;
    return 1;
}

// LDS bytes of a workgroup: the rows, the event counters, zeros and broadcast words, the first linear's bias
static size_t tail_lds_bytes(int xw, int ms, int nb1h) {
    return (size_t)16 * ms * (xw + 2 * TT_HW) + 2 * TT_MAX_PHASES * 4 + 128 + (size_t)nb1h * TT_BI_BYTES;
}

// which panel widths the kernel is built for
static bool tail_width_built(int D) { return D == 768 || D == 512 || D == 256; }

bool tail_pair_applies(const et_tile_plan *pO, const et_tile_plan *p1, const et_tile_plan *p2) {
    if (!pO || !p1 || !p2 || !g_tail_pair)
        return false;
    const int D = pO->out_feat, Hd = p1->out_feat;
    if (pO->in_feat != D || p1->in_feat != D || p2->in_feat != Hd || p2->out_feat != D || !tail_width_built(D) ||
        Hd % 16)
        return false;
    const int nchunk = (Hd + TT_HC - 1) / TT_HC, per_half = (nchunk + 1) / 2;
    if (nchunk < 2 || per_half > TT_MAX_PHASES || per_half * TT_HB > 255)
        return false;
    int nb, xw;
    if (!tail_geom(D, &nb, &xw))
        return false;
    return tail_lds_bytes(xw, tail_ms(), per_half * TT_HB) <= 160 * 1024;
}

size_t tail_ws_bytes_for(int D, int rows) {
    int nb, xw;
    if (rows <= 0 || !tail_width_built(D) || !tail_geom(D, &nb, &xw))
        return 0;
    // per (panel, half, row-half): waves x block-rows x subtiles of the row-half x 64 lanes x 4 floats; enough
    // for either panel height
    size_t need = 0;
    for (int ms = 2; ms <= 4; ms += 2) {
        const size_t npanels = ((size_t)rows + 16 * ms - 1) / (16 * ms);
        need = std::max(need, npanels * 4 * ((size_t)TT_WAVES * nb * (ms / 2) * 64 * 4) * sizeof(float));
    }
    return need;
}

size_t tail_pair_ws_bytes(const et_tile_plan *pO, const et_tile_plan *p1, const et_tile_plan *p2, int M) {
    if (!tail_pair_applies(pO, p1, p2) || M <= 0)
        return 0;
    return tail_ws_bytes_for(pO->out_feat, M);
}

namespace {
// one wave's stream while it is being laid out
struct Segment {
    int end;                 // pair index inside the stream, exclusive
    bool hidden;             // a hidden block-row of the first linear
    int j, slot, p;          // accumulator; slot in the hidden buffer; phase
    bool wait_store, signal; // wait for S[p - 2] before the hidden store; signal F[p] / S[p] afterwards
    int init;                // what its sums start from (255: zeros)
    int wait_p, wait_n;      // before its first operand is read: F[wait_p] has to reach wait_n (wait_p < 0: nothing)
};
struct ProgBuilder {
    std::vector<uint16_t> pairs; // 512 halves per pair
    std::vector<int> rec;        // 4 ints per pair: offset A, control, offset B, control
    size_t npairs() const { return rec.size() / 4; }

    // tiles of block-row bn of plan pl with column in [lo, hi), two per pair
    // (an odd last one gets an all-zero partner at its own offset); returns pairs added
    template <class OffsetOf>
    int add_tiles(const et_tile_plan *pl, int bn, int lo, int hi, OffsetOf &&offset_of) {
        int cnt = 0, last = 0;
        auto put = [&](int off, const uint16_t *tile) {
            rec.push_back(off);
            rec.push_back(0);
            if (tile)
                pairs.insert(pairs.end(), tile, tile + 256);
            else
                pairs.insert(pairs.end(), 256, (uint16_t)0);
            cnt++;
        };
        for (int i = pl->h_row_ptr[bn]; i < pl->h_row_ptr[bn + 1]; i++) {
            const int col = pl->h_col[i];
            if (col < lo || col >= hi)
                continue;
            last = offset_of(col);
            put(last, &pl->h_data[(size_t)i * 256]);
        }
        if (cnt & 1)
            put(last, nullptr);
        return cnt / 2;
    }
    void add_zero_pair(int offset) {
        const int r[4] = {offset, 0, offset, 0};
        rec.insert(rec.end(), r, r + 4);
        pairs.insert(pairs.end(), 512, (uint16_t)0);
    }
    // control words of a finished stream that starts at pair `base`
    void seal(size_t base, const std::vector<Segment> &segs) {
        for (size_t i = 0; i < segs.size(); i++) {
            const Segment &g = segs[i];
            int ctl = TT_C_SET | (g.hidden ? TT_C_HID : 0) | ((g.hidden ? 7 : g.j) << 2) | (g.slot << 5) | (g.p << 9) |
                      (g.wait_store ? TT_C_WAITF : 0) | (g.signal ? TT_C_SIG : 0);
            int next_init = 255;
            if (i + 1 < segs.size()) {
                const Segment &nx = segs[i + 1];
                next_init = nx.init;
                if (nx.wait_p >= 0)
                    ctl |= TT_C_WAITN | (nx.wait_p << 16) | ((nx.wait_n - 1) << 20);
            }
            ctl |= (int)((unsigned)next_init << 24);
            const size_t q = base + g.end - 1;
            rec[q * 4 + 1] = rec[q * 4 + 3] = ctl;
        }
    }
};
} // namespace

int tail_pair_prepare(const et_tile_plan *pO, const et_tile_plan *p1, et_tile_plan *p2) {
    ET_REQUIRE(tail_pair_applies(pO, p1, p2), ET_ERR_UNSUPPORTED, "layer tail (pairs): these plans do not qualify");
    if (p2->tail && p2->tail_uid[0] == pO->uid && p2->tail_uid[1] == p1->uid)
        return ET_OK;
    tail_program_destroy(p2->tail);
    p2->tail = nullptr;
    const int D = pO->out_feat, Hd = p1->out_feat, nbrD = D / 16, nbr1 = Hd / 16;
    int NB, XW;
    tail_geom(D, &NB, &XW);
    const int RS = XW + 2 * TT_HW;
    const int nchunk = (Hd + TT_HC - 1) / TT_HC;
    TailProgram *P = new TailProgram();
    P->D = D;
    P->Hd = Hd;
    const int c0[2] = {0, (nchunk + 1) / 2};
    P->nphase[0] = c0[1];
    P->nphase[1] = nchunk - c0[1];
    for (int h = 0; h < 2; h++) {
        P->hb0[h] = c0[h] * TT_HB;
        P->nb1h[h] = std::min(nbr1, (c0[h] + P->nphase[h]) * TT_HB) - P->hb0[h];
    }

    ProgBuilder B;
    std::vector<int> wtab(2 * TT_WAVES * 8, 0);
    for (int h = 0; h < 2; h++)
        for (int w = 0; w < TT_WAVES; w++) {
            int *wt = &wtab[(h * TT_WAVES + w) * 8];
            std::vector<Segment> segs;
            // ---- projection: block-rows NB*w .. NB*w + NB - 1 ----
            size_t base = B.npairs();
            wt[0] = (int)base;
            for (int j = 0; j < NB; j++) {
                const int bn = NB * w + j;
                if (bn >= nbrD)
                    continue;
                if (B.add_tiles(pO, bn, 0, D, [](int col) { return col * 2; }) > 0)
                    segs.push_back(Segment{(int)(B.npairs() - base), false, j, 0, 0, false, false, 255, -1, 0});
            }
            if (!segs.empty()) {
                while ((B.npairs() - base) % TT_PAD)
                    B.add_zero_pair(0);
                segs.back().end = (int)(B.npairs() - base); // the padding belongs to the last segment
            }
            wt[1] = (int)(B.npairs() - base);
            B.seal(base, segs);
            // ---- feed-forward: F(0) F(1) S(0) F(2) S(1) ... F(n-1) S(n-2) S(n-1) ----
            segs.clear();
            base = B.npairs();
            wt[2] = (int)base;
            const int np = P->nphase[h];
            auto first = [&](int p) { // F(p): this wave's one or two hidden block-rows of chunk c0 + p
                // twelve waves: slot s of the chunk's 12 goes to wave s.  Eight waves: to wave
                // (s + 4p) mod 8 - four waves have two block-rows in a phase, and they are the
                // other four in the next one
                for (int s = 0; s < TT_HB; s++) {
                    const int hb = (c0[h] + p) * TT_HB + s;
                    if ((TT_WAVES == 12 ? s : (s + 4 * p) % TT_WAVES) != w || hb >= nbr1)
                        continue;
                    if (B.add_tiles(p1, hb, 0, D, [](int col) { return col * 2; }) == 0)
                        B.add_zero_pair(0); // bias only: one pair of zeros so that the segment exists
                    segs.push_back(Segment{(int)(B.npairs() - base), true, 7, s, p, p >= 2, true, hb - P->hb0[h], -1, 0});
                }
            };
            auto second = [&](int p) { // S(p): this wave's output block-rows over hidden chunk c0 + p
                const int c = c0[h] + p, lo = c * TT_HC, hi = std::min(lo + TT_HC, Hd);
                const int nF = std::min(TT_HB, nbr1 - c * TT_HB); // hidden block-rows of the chunk, each signalled once
                const int hbase = XW + (p & 1) * TT_HW;
                const size_t nseg0 = segs.size();
                for (int j = 0; j < NB; j++) {
                    const int bn = NB * w + j;
                    if (bn >= nbrD)
                        continue;
                    if (B.add_tiles(p2, bn, lo, hi, [&](int col) { return hbase + (col - lo) * 2; }) == 0)
                        continue;
                    segs.push_back(Segment{(int)(B.npairs() - base), false, j, 0, p, false, false, 255, -1, 0});
                }
                if (segs.size() == nseg0) { // nothing of this chunk in the wave's block-rows: the phase is still signalled
                    B.add_zero_pair(hbase);
                    segs.push_back(Segment{(int)(B.npairs() - base), false, 0, 0, p, false, false, 255, -1, 0});
                }
                segs[nseg0].wait_p = p; // the phase's first segment reads the hidden buffer: F[p] complete
                segs[nseg0].wait_n = nF;
                segs.back().signal = true; // its last one signals S[p]
            };
            for (int p = 0; p < np; p++) {
                if (p == 0)
                    first(0);
                if (p + 1 < np)
                    first(p + 1);
                second(p);
            }
            while ((B.npairs() - base) % TT_PAD)
                B.add_zero_pair(XW + ((np - 1) & 1) * TT_HW);
            segs.back().end = (int)(B.npairs() - base);
            wt[3] = (int)(B.npairs() - base);
            wt[4] = segs.front().init;
            wt[5] = segs.front().wait_p >= 0 ? (segs.front().wait_p | (segs.front().wait_n << 8)) : -1;
            B.seal(base, segs);
        }
    P->npairs = B.npairs();
    for (int i = 0; i < 2 * TT_PAD; i++) // the last stages of a stream request up to depth - 1 pairs past its end
        B.add_zero_pair(0);
    // every offset must address the panel or a hidden buffer of the lane's row
    for (size_t q = 0; q < B.npairs(); q++)
        for (int t = 0; t < 2; t++) {
            const int v = B.rec[q * 4 + 2 * t];
            if (v < 0 || v + 32 > RS) {
                tail_program_destroy(P);
                set_error("layer tail (pairs): internal error, operand offset %d outside the LDS row", v);
                return ET_ERR_FORMAT;
            }
        }

    int rc = ET_OK;
    auto up = [&](void **dst, const void *hsrc, size_t bytes) {
        if (rc != ET_OK)
            return;
        rc = et_malloc(dst, std::max<size_t>(bytes, 16));
        if (rc == ET_OK && bytes)
            rc = et_memcpy_h2d(*dst, hsrc, bytes);
    };
    up((void **)&P->d_pairs, B.pairs.data(), B.pairs.size() * 2);
    up((void **)&P->d_rec, B.rec.data(), B.rec.size() * 4);
    up((void **)&P->d_wtab, wtab.data(), wtab.size() * 4);
    const std::vector<int> zeros(2 * TT_MAX_PANELS, 0);
    up((void **)&P->d_sync, zeros.data(), zeros.size() * 4);
    if (rc != ET_OK) {
        tail_program_destroy(P);
        return rc;
    }
    p2->tail = P;
    p2->tail_uid[0] = pO->uid;
    p2->tail_uid[1] = p1->uid;
    return ET_OK;
}

template <auto KERN>
static hipError_t tt_allow_lds(size_t lds) {
    static size_t allowed[16] = {};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 16)
        return hipFuncSetAttribute(reinterpret_cast<const void *>(KERN), hipFuncAttributeMaxDynamicSharedMemorySize,
                                   (int)lds);
    if (lds <= allowed[dev])
        return hipSuccess;
    const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(KERN),
                                             hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e == hipSuccess)
        allowed[dev] = lds;
    return e;
}

template <int D, int MS>
static int tt_launch(const TtArgs &a, size_t lds, hipStream_t st) {
    constexpr auto k = &tile_tail_pair_kernel<D, MS>;
    ET_HIP(tt_allow_lds<k>(lds));
    hipLaunchKernelGGL(k, dim3(a.per_xcd * 8), dim3(TT_WAVES * 64), lds, st, a);
    return launch_status("layer tail (pairs) launch");
}

int tail_pair_launch(const et_tile_plan *pO, const et_tile_plan *p1, const et_tile_plan *p2, f16 *Y,
                     const f16 *attn, const f16 *input, const f16 *gamma1, const f16 *beta1,
                     const f16 *gamma2, const f16 *beta2, int M, void *ws, hipStream_t st) {
    const TailProgram *P = p2->tail;
    ET_REQUIRE(P && p2->tail_uid[0] == pO->uid && p2->tail_uid[1] == p1->uid, ET_ERR_INVALID_ARG,
               "layer tail (pairs): no program for these plans (et_tile_plan_tail_prepare)");
    const int ms = tail_ms(), bm = 16 * ms;
    const int npanels = (M + bm - 1) / bm;
    ET_REQUIRE(npanels <= TT_MAX_PANELS, ET_ERR_UNSUPPORTED, "layer tail (pairs): %d rows, at most %d", M,
               TT_MAX_PANELS * bm);
    ET_REQUIRE(ws && aligned16(ws), ET_ERR_INVALID_ARG, "layer tail (pairs): scratch missing or misaligned");
    int *status = wait_status_device();
    ET_REQUIRE(status, ET_ERR_HIP, "layer tail (pairs): no wait-status word");
    const int rc = check_wait_status("layer tail (pairs)");
    if (rc != ET_OK)
        return rc;
    TtArgs a;
    memset(&a, 0, sizeof(a));
    a.pairs = P->d_pairs;
    a.rec = P->d_rec;
    a.wtab = P->d_wtab;
    a.attn = attn;
    a.input = input;
    a.Y = Y;
    a.biasO = pO->d_bias;
    a.bias1 = p1->d_bias;
    a.bias2 = p2->d_bias;
    a.g1 = gamma1;
    a.b1 = beta1;
    a.g2 = gamma2;
    a.b2 = beta2;
    a.ws = static_cast<unsigned long long *>(ws);
    a.sync = P->d_sync;
    a.status = status;
    a.M = M;
    a.npanels = npanels;
    a.per_xcd = 2 * ((npanels + 7) / 8);
    a.spin = g_tail_spin;
    for (int h = 0; h < 2; h++) {
        a.hb0[h] = P->hb0[h];
        a.nb1h[h] = P->nb1h[h];
    }
    int nb, xw;
    tail_geom(P->D, &nb, &xw);
    const size_t lds = tail_lds_bytes(xw, ms, std::max(P->nb1h[0], P->nb1h[1]));
    switch (P->D * 8 + ms) {
    case 768 * 8 + 4: return tt_launch<768, 4>(a, lds, st);
    case 512 * 8 + 4: return tt_launch<512, 4>(a, lds, st);
    case 256 * 8 + 4: return tt_launch<256, 4>(a, lds, st);
    case 768 * 8 + 2: return tt_launch<768, 2>(a, lds, st);
    case 512 * 8 + 2: return tt_launch<512, 2>(a, lds, st);
    case 256 * 8 + 2: return tt_launch<256, 2>(a, lds, st);
    default: break;
    }
    set_error("layer tail (pairs): width %d is not built", P->D);
    return ET_ERR_UNSUPPORTED;
}

} // namespace et
