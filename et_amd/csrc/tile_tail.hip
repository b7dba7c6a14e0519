// Layer tail (encoder/encoder.cu:33-44: O_linear, skip + LayerNorm, MLP1 with
// GELU, MLP2, skip + LayerNorm) as PAIRS of workgroups over 64-row panels.
//
// Why.  With one workgroup per 32-row panel every CU streams the whole of the
// three weight matrices (2.1 MB at BERT-base / 80 %) through the L2 -> CU path
// for 32 rows of work, two MFMAs per kilobyte, and all CUs together saturate
// the L2s.  Here a panel has 64 rows (four MFMAs per kilobyte of W) and the
// hidden dimension of the feed-forward block is split over the two workgroups
// of a pair: workgroup `half` of panel P runs the projection and the first
// LayerNorm on the panel (both do: 11 % duplicated work), then the first
// feed-forward linear for ITS half of the hidden columns and the second linear
// over those columns only.  A CU streams 1.2 MB of W instead of 2.1.
//
// The two partial sums of a panel meet without any workgroup waiting for the
// other one.  Rows 0-31 of the panel are finished by whoever arrives second at
// that row-half's counter, rows 32-63 likewise; a workgroup visits the other
// row-half first.  At a row-half it looks at the counter: zero means the
// partner has not published yet, so it writes its own fp32 partial (scratch),
// fences, and adds one to the counter - if the add returns one the partner
// arrived in between.  Whoever finds (or gets) one reads the partner's partial,
// adds the two, runs bias + skip + LayerNorm 2 on those 32 rows, stores them
// and resets the counter.  When the pair runs in step each workgroup writes one
// row-half, reads one and normalises one; when one is late the other leaves
// both of its partials and exits, and the late one finishes both.  No spin, no
// assumption that the partner is resident.  a + b == b + a in fp32, so the
// bits do not depend on who finishes.
//
// Inside a workgroup (8 waves, two per SIMD, 256 registers each).  LDS holds the panel and two 192-column hidden
// buffers INTERLEAVED per row (row stride = panel width + 2 x 208 halves, which
// keeps ds_read_b128 conflict-free), so a tile's X operand is "lane's row base
// + one byte offset" whether it multiplies the panel (projection, first
// linear) or a hidden buffer (second linear): one stage body serves all three.
// Every wave walks ONE continuous stream of tile pairs that the host lays out
// for it at plan time (its 6 block-rows of the projection; then, per 192-column
// phase p, one or two hidden block-rows of the first linear and its 6 output block-rows
// of the second linear over chunk p, the first linear one phase ahead), through
// a 4-deep register pipeline that never drains.  Where a segment of the stream
// ends a descriptor says what to do with the finished 64 x 16 sums: GELU and
// store into a hidden buffer, or add into one of the wave's output
// accumulators; and which LDS event counter to wait for or to signal (hidden
// buffer complete / hidden buffer free), exactly as an s_barrier would order
// them but without stopping a wave that is not a whole phase ahead.  Waits are
// bounded; a wave that gives up sets the process's wait-status word, which the
// next launch reports.  Both LayerNorms run on the accumulators where they are
// (a panel row's 768 columns are spread over the 8 waves; row sums meet in
// LDS), so no staging tile is needed for them.
#include "tile_plan.h"

#include <algorithm>
#include <cstring>
#include <type_traits>

namespace et {

constexpr int TT_WAVES = 8;               // two per SIMD: 256 registers each (accumulators for 6 block-rows x 64 rows)
constexpr int TT_BM = 64;                 // panel rows
constexpr int TT_HB = 12;                 // hidden block-rows per phase
constexpr int TT_HC = 16 * TT_HB;         // hidden columns per phase
constexpr int TT_HW = (TT_HC + 16) * 2;   // bytes of one hidden buffer inside an LDS row
constexpr int TT_MAX_PHASES = 16;         // per half: counters F[16], S[16]
constexpr int TT_MAX_PANELS = 8192;       // counters per program: 2 per panel
constexpr int TT_DESC = 8;                // ints per segment descriptor

template <int D> struct TtGeom {
    static constexpr int NB = (D / 16 + TT_WAVES - 1) / TT_WAVES; // output block-rows per wave
    static constexpr int XW = (D + ((D & 31) ? 0 : 16)) * 2;      // bytes of the panel part of an LDS row
    static constexpr int RS = XW + 2 * TT_HW;                     // LDS row stride, == 32 (mod 64)
    static constexpr int CT = TT_BM * RS;                         // event counters: F[16], S[16]
    static constexpr int ZV = CT + 2 * TT_MAX_PHASES * 4;         // 16 zero floats
    static constexpr int MISC = ZV + 64;                          // workgroup broadcasts
    static constexpr int BI = MISC + 64;                          // first linear's bias as fp32, 64 B per block-row
    static_assert(RS % 64 == 32, "row stride must be == 32 (mod 64) bytes");
};

// segment descriptor (TT_DESC ints): [0] end (pair index in the wave's stream, exclusive), [1] kind | j << 8
// (kind 0: add into accumulator j, 1: GELU into a hidden buffer), [2] hidden byte offset inside an LDS row,
// [3] LDS byte offset of the 64-byte vector the running sums start from (zeros, or the block-row's bias),
// [4] counter to wait for before the hidden store (byte offset | target << 16, -1 none), [5] counter to signal
// afterwards (byte offset, -1 none), [6] counter to wait for before the NEXT segment's first operand is read
struct TtArgs {
    const f16 *pairs;
    const int *off;
    const int *desc;
    const int *wtab; // per (half, wave): projection pair base, stages, descriptor base; feed-forward ditto; initial wait
    const f16 *attn, *input;
    f16 *Y;
    const f16 *biasO, *bias1, *bias2, *g1, *b1, *g2, *b2;
    float *ws;
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

// One pair's operands: 16 bytes of W per lane and the lane's X offset.  The
// pair's address is wave-uniform and the lane's part a 32-bit offset kept
// opaque in place, so the loads need no vector address arithmetic.
__device__ __forceinline__ void tt_load_pair(const char *wq, const char *oq, unsigned &lo, unsigned &lw,
                                             f16x8 &w, int &o) {
    asm("" : "+v"(lo), "+v"(lw));
    o = *reinterpret_cast<const int *>(oq + lo);
    w = *reinterpret_cast<const f16x8 *>(wq + lw);
}

__device__ __forceinline__ void tt_signal(unsigned *ctr, int lane) {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local"); // this wave's LDS traffic first
    if (lane == 0)
        __hip_atomic_fetch_add(ctr, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
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

template <int RS>
__device__ __forceinline__ void tt_read_x(f16x8 (&x)[4], const char *xl, int off) {
    const char *p = xl + off;
#pragma unroll
    for (int k = 0; k < 4; k++)
        x[k] = *reinterpret_cast<const f16x8 *>(p + k * 16 * RS);
}

// The stream: n stages (a multiple of 4), pair q's operands in w[q % 4] / o[q % 4]
// (the first four requested by the caller), X fragments read one stage ahead,
// four MFMAs per stage into cur[0..3] (one per 16-row subtile).  at_end(xn, on)
// runs where a stage finishes the segment that ends at `send`; xn / on are the
// fragments and the offset of the NEXT pair, for a handler that has to wait
// before they may be read.
template <int RS, class AtEnd>
__device__ __forceinline__ void tt_stream(const char *xl, const char *wq, const char *oq, int n,
                                          unsigned &lane_lo, unsigned &lane_lw, f16x8 (&w)[4], int (&o)[4],
                                          f32x4 (&cur)[4], int &send, AtEnd &&at_end) {
    f16x8 xf[2][4];
    tt_read_x<RS>(xf[0], xl, o[0]);
    const char *wp = wq + 4 * 1024, *op = oq + 4 * 8;
    for (int q = 0; q < n; q += 4) {
        tt_static_for<0, 4>([&](auto ic) {
            constexpr int I = decltype(ic)::value, SN = (I + 1) & 3, P = I & 1;
            tt_read_x<RS>(xf[P ^ 1], xl, o[SN]);
            // keep the reads above the MFMAs (the scheduler otherwise sinks them
            // and every stage waits out the LDS latency)
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int k = 0; k < 4; k++)
                cur[k] = mfma16x16x32(w[I], xf[P][k], cur[k]);
            // pair q + I + 4 (unconditional: the stream is followed by spare pairs)
            tt_load_pair(wp + I * 1024, op + I * 8, lane_lo, lane_lw, w[I], o[I]);
            if (q + I + 1 == send)
                at_end(xf[P ^ 1], o[SN]);
        });
        wp += 4 * 1024;
        op += 4 * 8;
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
template <int NB>
__device__ __forceinline__ void tt_acc_add(f32x4 (&acc)[NB][4], int j, const f32x4 (&cur)[4]) {
    tt_static_for<0, NB>([&](auto kc) {
        constexpr int k = decltype(kc)::value;
        if (j == k) {
            tt_add_tied<k>(acc[k][0], cur[0]);
            tt_add_tied<k>(acc[k][1], cur[1]);
            tt_add_tied<k>(acc[k][2], cur[2]);
            tt_add_tied<k>(acc[k][3], cur[3]);
        }
        asm volatile("; after case %0" ::"n"(k));
    });
}

// Skip + LayerNorm on values held in the accumulator layout: lane (c16, g4) of
// wave w holds, per block-row j and 16-row subtile ms, columns 16*(NB*w + j) +
// 4*g4 .. +3 of panel row 16*(ms0 + ms) + c16, already as x = half(y) + skip.
// The math of skip_layernorm.hip (fp32 mean, two-pass biased variance, eps
// 1e-6; kernels/skip_layernorm.cu:4-43).  A row's partial sums of the eight waves
// meet in the hidden-buffer part of that row in LDS (free whenever this runs)
// and are added in wave order.  Two workgroup barriers.
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
        static_assert(TT_WAVES == 8, "eight partial sums per row");
        const f32x4 a0 = p[0], a1 = p[1];
        return ((a0[0] + a0[1]) + (a0[2] + a0[3])) + ((a1[0] + a1[1]) + (a1[2] + a1[3]));
    };
#pragma unroll
    for (int ms = 0; ms < NMS; ms++) {
        float s = 0.f;
#pragma unroll
        for (int j = 0; j < NB; j++) { // (block-rows beyond the matrix hold zeros)
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
        for (int j = 0; j < NB; j++)
            if (j < nvalid) {
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    const float d = (float)x[j][ms][r] - mean[ms];
                    v += d * d;
                }
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

template <int D>
__global__ void __launch_bounds__(TT_WAVES * 64) tile_tail_pair_kernel(const TtArgs a) {
    using G = TtGeom<D>;
    constexpr int NB = G::NB, RS = G::RS, nbrD = D / 16;
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

    // the panel (attention output): DMA, wave w takes rows w, w + 12, ...
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
        float *bi = reinterpret_cast<float *>(smem + G::BI);
        for (int i = tid; i < nb1h * 16; i += TT_WAVES * 64)
            bi[i] = (float)a.bias1[hb0 * 16 + i];
    }
    typedef const __attribute__((address_space(4))) int *ScalarInts;
    const ScalarInts wt = (ScalarInts)a.wtab + (half * TT_WAVES + wave) * 8;
    const int o_base = __builtin_amdgcn_readfirstlane(wt[0]), o_n = __builtin_amdgcn_readfirstlane(wt[1]),
              o_desc = __builtin_amdgcn_readfirstlane(wt[2]), f_base = __builtin_amdgcn_readfirstlane(wt[3]),
              f_n = __builtin_amdgcn_readfirstlane(wt[4]), f_desc = __builtin_amdgcn_readfirstlane(wt[5]),
              f_wait0 = __builtin_amdgcn_readfirstlane(wt[6]);
    const ScalarInts dsc = (ScalarInts)a.desc;
    // (descriptor words are wave-uniform; saying so keeps every branch on them scalar)
#define TT_U(x_) __builtin_amdgcn_readfirstlane(x_)
    unsigned lane_lo = hi * 4u, lane_lw = (hi * 256 + c16 * 16 + khalf8) * 2u;
    const char *const pairs = reinterpret_cast<const char *>(a.pairs);
    const char *const offs = reinterpret_cast<const char *>(a.off);
    f16x8 w[4];
    int o[4];
#pragma unroll
    for (int i = 0; i < 4; i++)
        tt_load_pair(pairs + (size_t)(o_base + i) * 1024, offs + (size_t)(o_base + i) * 8, lane_lo, lane_lw, w[i],
                     o[i]);
    __builtin_amdgcn_s_waitcnt(0x0F70); // vmcnt(0): this wave's part of the panel has landed
    __syncthreads();

    f32x4 acc[NB][4], cur[4];
#pragma unroll
    for (int j = 0; j < NB; j++)
#pragma unroll
        for (int ms = 0; ms < 4; ms++)
            acc[j][ms] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int ms = 0; ms < 4; ms++)
        cur[ms] = f32x4{0.f, 0.f, 0.f, 0.f};
    const char *const xl = smem + c16 * RS + khalf8 * 2;

    // ---- the projection: this wave's NB block-rows over the whole panel ----
    {
        int seg = 0;
        int d_kind = TT_U(dsc[(size_t)o_desc * TT_DESC + 1]);
        int send = TT_U(dsc[(size_t)o_desc * TT_DESC]);
        int n_end = TT_U(dsc[(size_t)(o_desc + 1) * TT_DESC]), n_kind = TT_U(dsc[(size_t)(o_desc + 1) * TT_DESC + 1]);
        tt_stream<RS>(xl, pairs + (size_t)o_base * 1024, offs + (size_t)o_base * 8, o_n, lane_lo, lane_lw, w, o, cur,
                      send, [&](f16x8(&)[4], int) {
                          tt_acc_add<NB>(acc, d_kind >> 8, cur);
#pragma unroll
                          for (int ms = 0; ms < 4; ms++)
                              cur[ms] = f32x4{0.f, 0.f, 0.f, 0.f};
                          d_kind = n_kind;
                          send = n_end;
                          seg++;
                          n_end = TT_U(dsc[(size_t)(o_desc + seg + 1) * TT_DESC]);
                          n_kind = TT_U(dsc[(size_t)(o_desc + seg + 1) * TT_DESC + 1]);
                      });
    }
    // the first pairs of the feed-forward stream travel under the LayerNorm
#pragma unroll
    for (int i = 0; i < 4; i++)
        tt_load_pair(pairs + (size_t)(f_base + i) * 1024, offs + (size_t)(f_base + i) * 8, lane_lo, lane_lw, w[i],
                     o[i]);

    // ---- bias + skip (the layer input) + LayerNorm 1, written over the panel ----
    {
        f16x4 x[NB][4], gam[NB], bet[NB];
#pragma unroll
        for (int j = 0; j < NB; j++) {
            const int col = (NB * wave + j) * 16 + g4 * 4;
            f16x4 bo = f16x4{0, 0, 0, 0};
            gam[j] = bet[j] = bo;
            if (j < nvalid) {
                bo = *reinterpret_cast<const f16x4 *>(a.biasO + col);
                gam[j] = *reinterpret_cast<const f16x4 *>(a.g1 + col);
                bet[j] = *reinterpret_cast<const f16x4 *>(a.b1 + col);
            }
            const f32x4 bf = __builtin_convertvector(bo, f32x4);
#pragma unroll
            for (int ms = 0; ms < 4; ms++) {
                f16x4 sk = f16x4{0, 0, 0, 0};
                if (j < nvalid)
                    sk = *reinterpret_cast<const f16x4 *>(
                        a.input + (size_t)min(m0 + 16 * ms + c16, a.M - 1) * D + col);
                // half(acc + bias) is the linear's output as the reference stores it; the
                // skip connection is added in half (kernels/skip_layernorm.cu:20)
                x[j][ms] = __builtin_convertvector(acc[j][ms] + bf, f16x4) + sk;
            }
        }
        tt_ln<D, 4>(x, 0, gam, bet, smem, wave, c16, g4, nvalid);
        // (every wave has passed a barrier since its last read of the attention panel)
#pragma unroll
        for (int j = 0; j < NB; j++)
            if (j < nvalid)
#pragma unroll
                for (int ms = 0; ms < 4; ms++)
                    *reinterpret_cast<f16x4 *>(smem + (16 * ms + c16) * RS + ((NB * wave + j) * 16 + g4 * 4) * 2) =
                        x[j][ms];
    }
#pragma unroll
    for (int j = 0; j < NB; j++)
#pragma unroll
        for (int ms = 0; ms < 4; ms++)
            acc[j][ms] = f32x4{0.f, 0.f, 0.f, 0.f};
    __syncthreads(); // the feed-forward input panel is complete

    // ---- the feed-forward block over this half of the hidden columns ----
    {
        int seg = 0;
        int send, d_kind, d_hoff, d_wf, d_sig, d_wn;
        int n_end, n_kind, n_hoff, n_init, n_wf, n_sig, n_wn;
        {
            const ScalarInts p = dsc + (size_t)f_desc * TT_DESC;
            send = TT_U(p[0]), d_kind = TT_U(p[1]), d_hoff = TT_U(p[2]), d_wf = TT_U(p[4]), d_sig = TT_U(p[5]),
            d_wn = TT_U(p[6]);
            const f32x4 init = *reinterpret_cast<const f32x4 *>(smem + p[3] + g4 * 16);
#pragma unroll
            for (int ms = 0; ms < 4; ms++)
                cur[ms] = init;
            const ScalarInts pn = p + TT_DESC;
            n_end = TT_U(pn[0]), n_kind = TT_U(pn[1]), n_hoff = TT_U(pn[2]), n_init = TT_U(pn[3]), n_wf = TT_U(pn[4]),
            n_sig = TT_U(pn[5]), n_wn = TT_U(pn[6]);
        }
        if (f_wait0 >= 0)
            tt_wait(ctr + ((f_wait0 & 0xffff) >> 2), (unsigned)f_wait0 >> 16, a.spin, a.status, lane);
        tt_stream<RS>(
            xl, pairs + (size_t)f_base * 1024, offs + (size_t)f_base * 8, f_n, lane_lo, lane_lw, w, o, cur, send,
            [&](f16x8(&xn)[4], int on) {
                if ((d_kind & 0xff) == 1) {
                    // a finished hidden block-row (its bias was the starting value): GELU,
                    // rounded to half as the reference stores it, into the hidden buffer
                    if (d_wf >= 0) // ... once everyone has finished reading what it held before
                        tt_wait(ctr + ((d_wf & 0xffff) >> 2), (unsigned)d_wf >> 16, a.spin, a.status, lane);
                    char *hp = smem + c16 * RS + d_hoff + g4 * 8;
#pragma unroll
                    for (int ms = 0; ms < 4; ms++) {
                        *reinterpret_cast<f16x4 *>(hp + ms * 16 * RS) =
                            gelu4(__builtin_convertvector(cur[ms], f16x4));
                        __builtin_amdgcn_sched_barrier(0); // one subtile at a time: few temporaries
                    }
                }
                // (not in an else branch: as a part of that if / else the accumulators were
                // given a second set of registers behind the handler; a hidden block-row's
                // descriptor carries j = 255, which matches no accumulator)
                tt_acc_add<NB>(acc, d_kind >> 8, cur);
                if (d_sig >= 0)
                    tt_signal(ctr + (d_sig >> 2), lane);
                if (d_wn >= 0) {
                    // the next segment multiplies a hidden buffer: wait until it is complete
                    // and read the next pair's fragments again
                    tt_wait(ctr + ((d_wn & 0xffff) >> 2), (unsigned)d_wn >> 16, a.spin, a.status, lane);
                    tt_read_x<RS>(xn, xl, on);
                }
                const f32x4 init = *reinterpret_cast<const f32x4 *>(smem + n_init + g4 * 16);
#pragma unroll
                for (int ms = 0; ms < 4; ms++)
                    cur[ms] = init;
                send = n_end, d_kind = n_kind, d_hoff = n_hoff, d_wf = n_wf, d_sig = n_sig, d_wn = n_wn;
                seg++;
                const ScalarInts pn = dsc + (size_t)(f_desc + seg + 1) * TT_DESC;
                n_end = TT_U(pn[0]), n_kind = TT_U(pn[1]), n_hoff = TT_U(pn[2]), n_init = TT_U(pn[3]), n_wf = TT_U(pn[4]),
                n_sig = TT_U(pn[5]), n_wn = TT_U(pn[6]);
            });
#undef TT_U
    }

    // ---- the two halves' partial sums meet; bias + skip + LayerNorm 2; store ----
    f16x4 b2[NB], gam[NB], bet[NB];
#pragma unroll
    for (int j = 0; j < NB; j++) {
        const int col = (NB * wave + j) * 16 + g4 * 4;
        b2[j] = gam[j] = bet[j] = f16x4{0, 0, 0, 0};
        if (j < nvalid) {
            b2[j] = *reinterpret_cast<const f16x4 *>(a.bias2 + col);
            gam[j] = *reinterpret_cast<const f16x4 *>(a.g2 + col);
            bet[j] = *reinterpret_cast<const f16x4 *>(a.b2 + col);
        }
    }
    __syncthreads(); // every wave has left the hidden buffers
    // scratch of (panel, half, row-half): [wave][j][subtile][lane] float4, coalesced both ways
    constexpr size_t PART = (size_t)TT_WAVES * NB * 2 * 64 * 4; // floats per (panel, half, row-half)
    for (int visit = 0; visit < 2; visit++) {
        const int h = visit == 0 ? 1 - half : half; // the other workgroup's row-half first
        int *const cnt = a.sync + 2 * panel + h;
        if (tid == 0)
            misc[0] = __hip_atomic_load(cnt, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __syncthreads();
        int arrived = misc[0]; // 1: the partner's partial of this row-half is in scratch
        if (arrived == 0) {
            f32x4 *dst = reinterpret_cast<f32x4 *>(a.ws + ((size_t)(panel * 2 + half) * 2 + h) * PART) +
                         (size_t)wave * NB * 2 * 64 + lane;
#pragma unroll
            for (int j = 0; j < NB; j++)
#pragma unroll
                for (int m2 = 0; m2 < 2; m2++)
                    dst[(j * 2 + m2) * 64] = h ? acc[j][2 + m2] : acc[j][m2]; // (selected, not indexed: acc stays in registers)
            __threadfence(); // the partial is visible to the device before the counter says so
            __syncthreads();
            if (tid == 0)
                misc[1] = __hip_atomic_fetch_add(cnt, 1, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_AGENT);
            __syncthreads();
            arrived = misc[1];
        }
        if (arrived != 0) { // (workgroup-uniform)
            __threadfence();
            const f32x4 *src =
                reinterpret_cast<const f32x4 *>(a.ws + ((size_t)(panel * 2 + (1 - half)) * 2 + h) * PART) +
                (size_t)wave * NB * 2 * 64 + lane;
            f16x4 x[NB][2];
#pragma unroll
            for (int j = 0; j < NB; j++) {
                const f32x4 bf = __builtin_convertvector(b2[j], f32x4);
#pragma unroll
                for (int m2 = 0; m2 < 2; m2++) {
                    f32x4 other = f32x4{0.f, 0.f, 0.f, 0.f};
                    f16x4 sk = f16x4{0, 0, 0, 0};
                    if (j < nvalid) {
                        other = src[(j * 2 + m2) * 64];
                        sk = *reinterpret_cast<const f16x4 *>(smem + (16 * (2 * h + m2) + c16) * RS +
                                                              ((NB * wave + j) * 16 + g4 * 4) * 2);
                    }
                    const f32x4 mine = h ? acc[j][2 + m2] : acc[j][m2];
                    x[j][m2] = __builtin_convertvector((mine + other) + bf, f16x4) + sk;
                }
            }
            tt_ln<D, 2>(x, 2 * h, gam, bet, smem, wave, c16, g4, nvalid);
            // in place over the skip operand (each lane overwrites what it read), then
            // whole rows leave with 16-byte stores
#pragma unroll
            for (int j = 0; j < NB; j++)
                if (j < nvalid)
#pragma unroll
                    for (int m2 = 0; m2 < 2; m2++)
                        *reinterpret_cast<f16x4 *>(smem + (16 * (2 * h + m2) + c16) * RS +
                                                   ((NB * wave + j) * 16 + g4 * 4) * 2) = x[j][m2];
            __syncthreads();
            constexpr int PR = D / 8;
            for (int i = tid; i < 32 * PR; i += TT_WAVES * 64) {
                const int r = 32 * h + i / PR, c = i % PR;
                if (m0 + r < a.M)
                    *reinterpret_cast<u32x4 *>(a.Y + (size_t)(m0 + r) * D + c * 8) =
                        *reinterpret_cast<const u32x4 *>(smem + r * RS + c * 16);
            }
            if (tid == 0) // ready for the next launch
                __hip_atomic_store(cnt, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        __syncthreads(); // misc[] is free again
    }
}

// ---------------------------------------------------------------------------
// host side: the program
// ---------------------------------------------------------------------------
struct TailProgram {
    int D = 0, Hd = 0;
    int nphase[2] = {0, 0}, hb0[2] = {0, 0}, nb1h[2] = {0, 0};
    f16 *d_pairs = nullptr;
    int *d_off = nullptr, *d_desc = nullptr, *d_wtab = nullptr, *d_sync = nullptr;
    size_t lds_bytes = 0;
    size_t npairs = 0; // including padding (for reports)
};

void tail_program_destroy(TailProgram *p) {
    if (!p)
        return;
    et_free(p->d_pairs);
    et_free(p->d_off);
    et_free(p->d_desc);
    et_free(p->d_wtab);
    et_free(p->d_sync);
    delete p;
}

static int g_tail_pair = 1;          // et_tuning_set("tile_tail_pair"): 0 never, 1 where it pays, 2 wherever it applies
static int g_tail_spin = 1 << 22;    // et_tuning_set("tile_wait_spin"): polls before a bounded LDS wait gives up
void set_tail_pair(int v) { g_tail_pair = v; }
bool tail_pair_forced() { return g_tail_pair >= 2; }
void set_tail_spin(int v) { g_tail_spin = v < 0 ? (1 << 22) : v; }
int tail_spin() { return g_tail_spin; }

static int tail_geom(int D, int *nb, int *xw) {
    if (D <= 0 || D % 16 || D / 16 > 6 * TT_WAVES)
        return 0;
    *nb = (D / 16 + TT_WAVES - 1) / TT_WAVES;
    *xw = (D + ((D & 31) ? 0 : 16)) * 2;
    return 1;
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
    if (nchunk < 2 || per_half > TT_MAX_PHASES)
        return false;
    int nb, xw;
    if (!tail_geom(D, &nb, &xw))
        return false;
    const size_t lds = (size_t)TT_BM * (xw + 2 * TT_HW) + 2 * TT_MAX_PHASES * 4 + 128 + (size_t)per_half * TT_HB * 64;
    return lds <= 160 * 1024;
}

size_t tail_pair_ws_bytes(const et_tile_plan *pO, const et_tile_plan *p1, const et_tile_plan *p2, int M) {
    if (!tail_pair_applies(pO, p1, p2) || M <= 0)
        return 0;
    int nb, xw;
    tail_geom(pO->out_feat, &nb, &xw);
    const size_t npanels = ((size_t)M + TT_BM - 1) / TT_BM;
    return npanels * 4 * ((size_t)TT_WAVES * nb * 2 * 64 * 4) * sizeof(float);
}

size_t tail_ws_bytes_for(int D, int rows) {
    int nb, xw;
    if (rows <= 0 || !tail_width_built(D) || !tail_geom(D, &nb, &xw))
        return 0;
    const size_t npanels = ((size_t)rows + TT_BM - 1) / TT_BM;
    return npanels * 4 * ((size_t)TT_WAVES * nb * 2 * 64 * 4) * sizeof(float);
}

namespace {
struct ProgBuilder {
    std::vector<uint16_t> pairs; // 512 halves per pair
    std::vector<int> off;        // 2 ints per pair
    std::vector<int> desc;       // TT_DESC ints per segment
    size_t npairs() const { return off.size() / 2; }
    int nseg() const { return (int)(desc.size() / TT_DESC); }

    // tiles of block-row bn of plan pl with column in [lo, hi), two per pair
    // (an odd last one gets an all-zero partner at its own offset); returns pairs added
    template <class OffsetOf>
    int add_tiles(const et_tile_plan *pl, int bn, int lo, int hi, OffsetOf &&offset_of) {
        int cnt = 0, last = 0;
        for (int i = pl->h_row_ptr[bn]; i < pl->h_row_ptr[bn + 1]; i++) {
            const int col = pl->h_col[i];
            if (col < lo || col >= hi)
                continue;
            last = offset_of(col);
            off.push_back(last);
            pairs.insert(pairs.end(), pl->h_data.begin() + (size_t)i * 256, pl->h_data.begin() + (size_t)i * 256 + 256);
            cnt++;
        }
        if (cnt & 1) {
            off.push_back(last);
            pairs.insert(pairs.end(), 256, (uint16_t)0);
            cnt++;
        }
        return cnt / 2;
    }
    void add_zero_pair(int offset) {
        off.push_back(offset);
        off.push_back(offset);
        pairs.insert(pairs.end(), 512, (uint16_t)0);
    }
    void add_desc(int end, int kind, int j, int hoff, int init, int wf, int sig) {
        const int d[TT_DESC] = {end, kind | (j << 8), hoff, init, wf, sig, -1, 0};
        desc.insert(desc.end(), d, d + TT_DESC);
    }
    void sentinel(int init) { add_desc(0x7fffffff, 0, 0, 0, init, -1, -1); }
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
    const int RS = XW + 2 * TT_HW, CT = TT_BM * RS, ZV = CT + 2 * TT_MAX_PHASES * 4, BI = ZV + 128;
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
    P->lds_bytes = (size_t)BI + (size_t)std::max(P->nb1h[0], P->nb1h[1]) * 64;

    ProgBuilder B;
    std::vector<int> wtab(2 * TT_WAVES * 8, 0);
    for (int h = 0; h < 2; h++)
        for (int w = 0; w < TT_WAVES; w++) {
            int *wt = &wtab[(h * TT_WAVES + w) * 8];
            // ---- projection: block-rows NB*w .. NB*w + NB - 1 ----
            size_t base = B.npairs();
            wt[0] = (int)base;
            wt[2] = B.nseg();
            int segs = 0;
            for (int j = 0; j < NB; j++) {
                const int bn = NB * w + j;
                if (bn >= nbrD)
                    continue;
                if (B.add_tiles(pO, bn, 0, D, [](int col) { return col * 2; }) > 0) {
                    B.add_desc((int)(B.npairs() - base), 0, j, 0, ZV, -1, -1);
                    segs++;
                }
            }
            if (segs) {
                while ((B.npairs() - base) % 4)
                    B.add_zero_pair(0);
                B.desc[B.desc.size() - TT_DESC] = (int)(B.npairs() - base); // the padding belongs to the last segment
            }
            wt[1] = (int)(B.npairs() - base);
            B.sentinel(ZV);
            // ---- feed-forward: F(0) F(1) S(0) F(2) S(1) ... F(n-1) S(n-2) S(n-1) ----
            base = B.npairs();
            wt[3] = (int)base;
            wt[5] = B.nseg();
            wt[6] = -1;
            const int np = P->nphase[h];
            int last_desc = -1; // index of the stream's latest descriptor
            auto ctrF = [](int p) { return 4 * p; };
            auto ctrS = [](int p) { return 4 * (TT_MAX_PHASES + p); };
            auto first = [&](int p) { // F(p): this wave's one or two hidden block-rows of chunk c0 + p
                // slot s of the chunk's 12 goes to wave (s + 4p) mod 8: four waves have two
                // block-rows in a phase, and they are the other four in the next one
                for (int s = 0; s < TT_HB; s++) {
                    const int hb = (c0[h] + p) * TT_HB + s;
                    if ((s + 4 * p) % TT_WAVES != w || hb >= nbr1)
                        continue;
                    if (B.add_tiles(p1, hb, 0, D, [](int col) { return col * 2; }) == 0)
                        B.add_zero_pair(0); // bias only: one pair of zeros so that the segment exists
                    const int wf = p >= 2 ? (ctrS(p - 2) | (TT_WAVES << 16)) : -1;
                    last_desc = B.nseg();
                    B.add_desc((int)(B.npairs() - base), 1, 255, XW + (p & 1) * TT_HW + s * 32,
                               BI + (hb - P->hb0[h]) * 64, wf, ctrF(p));
                }
            };
            auto second = [&](int p) { // S(p): this wave's output block-rows over hidden chunk c0 + p
                const int c = c0[h] + p, lo = c * TT_HC, hi = std::min(lo + TT_HC, Hd);
                const int nF = std::min(TT_HB, nbr1 - c * TT_HB); // hidden block-rows of the chunk, each signalled once
                const int wait = ctrF(p) | (nF << 16);
                const int hbase = XW + (p & 1) * TT_HW;
                bool any = false;
                auto begin_phase = [&]() {
                    if (any)
                        return;
                    any = true;
                    if (last_desc >= 0)
                        B.desc[(size_t)last_desc * TT_DESC + 6] = wait;
                    else
                        wt[6] = wait;
                };
                for (int j = 0; j < NB; j++) {
                    const int bn = NB * w + j;
                    if (bn >= nbrD)
                        continue;
                    if (B.add_tiles(p2, bn, lo, hi, [&](int col) { return hbase + (col - lo) * 2; }) == 0)
                        continue;
                    begin_phase();
                    last_desc = B.nseg();
                    B.add_desc((int)(B.npairs() - base), 0, j, 0, ZV, -1, -1);
                }
                if (!any) { // nothing of this chunk in the wave's block-rows: the phase still has to be signalled
                    B.add_zero_pair(hbase);
                    begin_phase();
                    last_desc = B.nseg();
                    B.add_desc((int)(B.npairs() - base), 0, 0, 0, ZV, -1, -1);
                }
                B.desc[(size_t)last_desc * TT_DESC + 5] = ctrS(p); // the phase's last segment signals S[p]
            };
            for (int p = 0; p < np; p++) {
                if (p == 0)
                    first(0);
                if (p + 1 < np)
                    first(p + 1);
                second(p);
            }
            while ((B.npairs() - base) % 4)
                B.add_zero_pair(XW + ((np - 1) & 1) * TT_HW);
            B.desc[(size_t)last_desc * TT_DESC] = (int)(B.npairs() - base);
            wt[4] = (int)(B.npairs() - base);
            B.sentinel(ZV);
        }
    B.sentinel(ZV); // (a handler reads one descriptor past its stream's sentinel)
    P->npairs = B.npairs();
    for (int i = 0; i < 8; i++) // the last stages of a stream request up to seven pairs past its end
        B.add_zero_pair(0);
    // every offset must address the panel or a hidden buffer of the lane's row
    for (int v : B.off)
        if (v < 0 || v + 32 > RS) {
            tail_program_destroy(P);
            set_error("layer tail (pairs): internal error, operand offset %d outside the LDS row", v);
            return ET_ERR_FORMAT;
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
    up((void **)&P->d_off, B.off.data(), B.off.size() * 4);
    up((void **)&P->d_desc, B.desc.data(), B.desc.size() * 4);
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

template <int D>
static int tt_launch(const TtArgs &a, size_t lds, hipStream_t st) {
    constexpr auto k = &tile_tail_pair_kernel<D>;
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
    const int npanels = (M + TT_BM - 1) / TT_BM;
    ET_REQUIRE(npanels <= TT_MAX_PANELS, ET_ERR_UNSUPPORTED, "layer tail (pairs): %d rows, at most %d", M,
               TT_MAX_PANELS * TT_BM);
    ET_REQUIRE(ws && aligned16(ws), ET_ERR_INVALID_ARG, "layer tail (pairs): scratch missing or misaligned");
    int *status = wait_status_device();
    ET_REQUIRE(status, ET_ERR_HIP, "layer tail (pairs): no wait-status word");
    const int rc = check_wait_status("layer tail (pairs)");
    if (rc != ET_OK)
        return rc;
    TtArgs a;
    memset(&a, 0, sizeof(a));
    a.pairs = P->d_pairs;
    a.off = P->d_off;
    a.desc = P->d_desc;
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
    a.ws = static_cast<float *>(ws);
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
    switch (P->D) {
    case 768: return tt_launch<768>(a, P->lds_bytes, st);
    case 512: return tt_launch<512>(a, P->lds_bytes, st);
    case 256: return tt_launch<256>(a, P->lds_bytes, st);
    default: break;
    }
    set_error("layer tail (pairs): width %d is not built", P->D);
    return ET_ERR_UNSUPPORTED;
}

} // namespace et
