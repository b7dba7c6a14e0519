// Tensor-tile pruned linear (and the dense row-compacted linear) for gfx950.
//
// Computes Y[M x N] = X[M x K] * W^T + bias (optionally followed by GELU) where
// W[N x K] is stored as its surviving 16x16 tiles (tile_mat: CSR over
// block-rows of 16 output features, kernels/linear.cu:54-101 in the
// reference), or dense row-major for the row-pruned linear
// (kernels/linear.cu:18-34).
//
// Mapping.  A workgroup of 8 waves owns 32 rows of X (two 16-row MFMA
// subtiles) and a group of 8*NB consecutive block-rows of W.  The 32 x KC
// panel of X lives in LDS; each wave walks the tile list of its NB block-rows
// and issues v_mfma_f32_16x16x32_f16 with TWO arbitrary surviving tiles
// concatenated along k (a surviving tile is exactly one k=16 slice): lanes
// 0-31 carry the first tile of the pair, lanes 32-63 the second.  The W
// operand of a pair is one coalesced 1 KB global read reused for both row
// subtiles; the X operand is gathered from LDS at the tile's column offset.
// The product is formed transposed (D = W_tile * X^T) so that a lane ends up
// with four consecutive output features of one row, which makes the
// half-precision staging write 8 bytes wide.  Results are staged in LDS and
// written with 16-byte row-contiguous stores, because at >= 80 % sparsity a
// linear on its own is bound by the Y write.
// K larger than the LDS panel is walked in chunks of KC columns; plans sort
// each block-row's tiles by column and carry a per-chunk CSR so a chunk only
// touches its own tiles (TL_PLAN); raw unsorted input with K > one panel falls
// back to filtering the whole list per chunk (TL_FILTER).
//
// Kernels in this file: tile_linear_resident_kernel (K in one panel: persistent
// workgroups, 32- or 64-row panels, optional LayerNorm epilogue),
// tile_linear_plan_kernel (K in chunks), tile_linear_chunked_ln_kernel (K in
// chunks + LayerNorm, double-buffered panels with a fetching wave),
// tile_ffn_fused_kernel (feed-forward block / whole layer tail in one launch,
// hidden activations in LDS), tile_linear_generic_kernel (raw and dense input).
#include "tile_plan.h"

#include <algorithm>
#include <type_traits>
#include <cstdlib>
#include <cstring>
#include <numeric>
#include <vector>

namespace et {

void set_attn_variant(int v);
void set_attn_vwin(int v);
void set_attn_packed(int v);
void set_ln_rows(int v);
void set_tail_pair(int v);
void set_tail_spin(int v);
int tail_spin();

constexpr int TL_THREADS = 512;
constexpr int TL_WAVES = 8;
constexpr int TL_BM = 32;
constexpr int TL_PAD = 16;       // halves; LDS row stride == 32 (mod 64) bytes: measured conflict-free for ds_read_b128
constexpr int TL_MAX_PANEL = 992;  // single-panel K limit: 32*(992+16)*2 B < 64 KB
constexpr int TL_CHUNK = 768;
constexpr int TL_MAX_LIN = 4;

// TL_PLAN: plan layout (see et_tile_plan_create): tiles ordered (chunk,
//          block-row, column), every (chunk, block-row) segment padded to an
//          even tile count with an all-zero tile, cptr[c*nbr + bn] in tiles.
// TL_RAW:  caller's tile_mat as is (any order inside a block-row, odd counts),
//          K fits one LDS panel; cptr is row_ptr.
// TL_FILTER: caller's tile_mat, K walked in chunks by filtering every list.
// TL_DENSE: W row-major [N x K] (the row-pruned linear's compacted rows).
enum { TL_PLAN = 0, TL_RAW = 1, TL_FILTER = 2, TL_DENSE = 3 };

struct TlProblem {
    f16 *Y;
    const int *cptr;
    const int *row_offset; // element column offset per tile
    const f16 *data;       // tile data, or dense row-major W for TL_DENSE
    const f16 *bias;
    int N;
    int nbr; // N / 16
    int ntile = 0; // surviving tiles where known (plans), 0 otherwise
};

// kernel arguments; per-linear fields as separate arrays that are only ever
// indexed with constants (a dynamically indexed by-value struct would be
// copied to scratch memory)
struct TlArgs {
    f16 *Y[TL_MAX_LIN];
    const int *cptr[TL_MAX_LIN];
    const int *row_offset[TL_MAX_LIN];
    const f16 *data[TL_MAX_LIN];
    const f16 *bias[TL_MAX_LIN];
    int N[TL_MAX_LIN];
    const f16 *X;
    int nlin, M, K, KC, nchunk, ncg, total, per_xcd;
    int ipw; // plan kernel: consecutive work items per (persistent) workgroup
    // fused skip + LayerNorm epilogue (plan kernels with LN = true)
    const f16 *skip, *gamma, *beta;
    const f16 *gamma2, *beta2; // second LayerNorm of the fused layer tail
    int *status;               // fused feed-forward kernels: set when a bounded LDS wait gives up
    int spin;                  // ... after this many polls
};
#define TL_SEL(f) (lin == 0 ? a.f[0] : lin == 1 ? a.f[1] : lin == 2 ? a.f[2] : a.f[3])

// tanh-form GELU of kernels/linear.cu:36-48: x^3 in half, the tanh argument
// and 0.5(1+tanh u) in fp32, rounded to half, times x in half.
// 0.5(1+tanh u) == 1 - 1/(exp(2u)+1).
__device__ __forceinline__ f16 gelu_h(f16 v) {
    const f16 x2 = v * v;
    const f16 x3 = v * x2;
    const float x = (float)v;
    const float u2 = 1.5957691216057308f * (x + 0.044715f * (float)x3); // 2u
    const float e = __builtin_amdgcn_exp2f(u2 * 1.4426950408889634f);
    const float t = 1.0f - __builtin_amdgcn_rcpf(e + 1.0f);
    return v * (f16)t;
}

// what every variant shares: workgroup -> (row panel, linear, column group)
struct TlCtx {
    int lin, cg, m0, wave, lane, c16, g4, khalf8, hi, ldx, bn_wg, bn0, ld_r, ld_c;
};

__device__ __forceinline__ bool tl_context(const TlArgs &a, int nb, TlCtx &x) {
    // Workgroups that share a row panel of X get consecutive ids on ONE XCD
    // (hardware round-robins consecutive workgroup ids over the 8 XCDs), so
    // the panel is fetched into that XCD's L2 once.
    const int pid = (blockIdx.x & 7) * a.per_xcd + (blockIdx.x >> 3);
    if (pid >= a.total)
        return false;
    const int per_rp = a.ncg * a.nlin;
    const int rp = pid / per_rp;
    const int rest = pid - rp * per_rp;
    x.lin = rest / a.ncg;
    x.cg = rest - x.lin * a.ncg;
    x.m0 = rp * TL_BM;
    x.wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    x.lane = threadIdx.x & 63;
    x.c16 = x.lane & 15;
    x.g4 = x.lane >> 4;
    x.khalf8 = (x.g4 & 1) * 8;
    x.hi = x.lane >> 5;
    x.ldx = a.KC + ((a.KC & 31) ? 0 : TL_PAD);
    x.bn_wg = x.cg * (TL_WAVES * nb);
    x.bn0 = x.bn_wg + x.wave * nb;
    x.ld_r = threadIdx.x >> 4; // 0..31: panel row this thread stages
    x.ld_c = threadIdx.x & 15;
    return true;
}

// bias (+GELU), round to half, stage in LDS (the X panel's storage), then
// 16-byte row-contiguous stores
template <int NB, bool GELU>
__device__ __forceinline__ void tl_epilogue(const TlArgs &a, const TlCtx &x, f16 *xs, f16 *Y, int N,
                                            int nbr, const f32x4 (&acc)[NB][2], const f16x4 (&b4)[NB]) {
    __syncthreads(); // every wave is done reading the X panel
    constexpr int BNW = TL_WAVES * NB * 16; // output columns per workgroup
    constexpr int ldy = BNW + TL_PAD;
    f16 *ys = xs;
#pragma unroll
    for (int j = 0; j < NB; j++) {
        const int bn = x.bn0 + j;
        if (bn >= nbr)
            continue;
        const int ncol = (bn - x.bn_wg) * 16 + x.g4 * 4;
#pragma unroll
        for (int ms = 0; ms < 2; ms++) {
            f16x4 o;
#pragma unroll
            for (int r = 0; r < 4; r++) {
                const f16 v = (f16)(acc[j][ms][r] + (float)b4[j][r]);
                o[r] = GELU ? gelu_h(v) : v;
            }
            *reinterpret_cast<f16x4 *>(ys + (ms * 16 + x.c16) * ldy + ncol) = o;
        }
    }
    __syncthreads();
    const int col0 = x.bn_wg * 16;
    const int wcols = min(BNW, N - col0);
    const int cpr = wcols >> 3;
    if (x.m0 + x.ld_r < a.M) {
        u32x4 *dst = reinterpret_cast<u32x4 *>(Y + (size_t)(x.m0 + x.ld_r) * N + col0);
        const u32x4 *src = reinterpret_cast<const u32x4 *>(ys + x.ld_r * ldy);
        for (int cc = x.ld_c; cc < cpr; cc += 16)
            dst[cc] = src[cc];
    }
}

// Per-wave epilogue: bias (+GELU), round to half, transpose through a
// wave-private LDS tile (32 rows x 16*NB columns, no barrier: a wave's LDS
// operations execute in order), then 16-byte stores of 32*NB contiguous bytes
// per row.  Waves never wait for each other here, so one wave's stores overlap
// the other waves' MFMAs.
template <int NB> constexpr int tl_wave_stage_halves() { return TL_BM * (16 * NB + 8); }

template <int NB, bool GELU, bool STORE = true>
__device__ __forceinline__ void tl_epilogue_wave(const TlArgs &a, const TlCtx &x, f16 *stage, f16 *Y,
                                                 int N, int nbr, const f32x4 (&acc)[NB][2],
                                                 const f16x4 (&b4)[NB]) {
    constexpr int lds = 16 * NB + 8; // halves per staged row
#pragma unroll
    for (int j = 0; j < NB; j++) {
#pragma unroll
        for (int ms = 0; ms < 2; ms++) {
            f16x4 o;
#pragma unroll
            for (int r = 0; r < 4; r++) {
                const f16 v = (f16)(acc[j][ms][r] + (float)b4[j][r]);
                o[r] = GELU ? gelu_h(v) : v;
            }
            *reinterpret_cast<f16x4 *>(stage + (ms * 16 + x.c16) * lds + j * 16 + x.g4 * 4) = o;
        }
    }
    if (!STORE)
        return;
    // valid block-rows of this wave (the last column group may be partial)
    const int nvalid = min(NB, nbr - x.bn0);
    if (nvalid <= 0)
        return;
    const int cpr = 2 * nvalid; // 16-byte chunks per row
    f16 *ybase = Y + (size_t)x.m0 * N + x.bn0 * 16;
#pragma unroll
    for (int t = 0; t < NB; t++) {
        const int i = x.lane + 64 * t;
        const int r = i / (2 * NB), c = i - r * (2 * NB);
        if (c < cpr && x.m0 + r < a.M) {
            const u32x4 v = *reinterpret_cast<const u32x4 *>(stage + r * lds + c * 8);
            *reinterpret_cast<u32x4 *>(ybase + (size_t)r * N + c * 8) = v;
        }
    }
}

// ---------------------------------------------------------------------------
// The pair stream shared by the plan kernels.
//
// A wave owns NB CONSECUTIVE block-rows, and the plan stores tiles in (chunk,
// block-row) order with even segments, so the wave's work for a chunk is ONE
// contiguous run of tile pairs [q0, qend): 1 KB of W per pair at an address
// linear in the pair index, plus one int per half-wave giving the LDS byte
// offset of that tile's X columns.  The run is consumed through a TL_DEPTH-stage
// register pipeline (stage = pair index mod TL_DEPTH) with unconditional loads
// in the main loop, so TL_DEPTH pairs are always in flight per wave and the
// waits are counted, not drained; only the last stages of a run test whether
// there is still a pair to request.  X operands are read from LDS one stage
// ahead.  Products accumulate into one running 32x16 accumulator; when the
// stream crosses a block-row boundary (a scalar compare per pair) flush(j,
// cur0, cur1) receives block-row j's finished sums.  All control flow in here
// is wave-uniform and straight-line per stage: loops or conditional loads
// would make the compiler drain every load instead of counting.
// ---------------------------------------------------------------------------
#ifndef TL_DEPTH
#define TL_DEPTH 4
#endif
// Wave priority while a stream runs (0 outside and inside a flush): waves that
// are streaming issue their loads and MFMAs ahead of waves that sit in the
// vector-ALU work of a GELU flush or a LayerNorm (layer tail: -2 %).
#ifndef TL_PRIO
#define TL_PRIO 1
#endif
static_assert(TL_DEPTH % 2 == 0, "the X operand ping-pong needs an even pipeline depth");

template <int I> using tl_ic = std::integral_constant<int, I>;
template <int B, int E, class F>
__device__ __forceinline__ void tl_static_for(F &&f) {
    if constexpr (B < E) {
        f(tl_ic<B>());
        tl_static_for<B + 1, E>(f);
    }
}

// the first TL_DEPTH pairs of a stream (an empty stream still loads pair q0:
// the plan keeps a spare pair behind the last one)
// One pair's operands: 16 bytes of W per lane and the lane's X offset.  The
// pair's address is wave-uniform (scalar registers) and the lane's part a
// 32-bit offset, so the loads need no vector address arithmetic.
// lo / lw: the lane's byte offsets into a pair's two ints and its 1 KB of W
__device__ __forceinline__ void tl_load_pair_at(const char *wq, const char *oq, unsigned &lo,
                                                unsigned &lw, f16x8 &w, int &o) {
    // (the empty asm, in place on variables that live across the whole stream,
    // makes the lane offsets look freshly computed: otherwise the compiler folds
    // them into loop-invariant 64-bit vector addresses and pays two 64-bit
    // vector adds per pair instead of using scalar base + 32-bit lane offset)
    asm("" : "+v"(lo), "+v"(lw));
    o = *reinterpret_cast<const int *>(oq + lo);
    w = *reinterpret_cast<const f16x8 *>(wq + lw);
}
__device__ __forceinline__ void tl_load_pair(const f16 *data, const int *poff, int q, unsigned lane_w,
                                             unsigned hi, f16x8 &w, int &o) {
    unsigned lo = hi * 4u, lw = lane_w * 2u;
    tl_load_pair_at(reinterpret_cast<const char *>(data) + (size_t)q * 1024,
                    reinterpret_cast<const char *>(poff) + (size_t)q * 8, lo, lw, w, o);
}

__device__ __forceinline__ void tl_preload(const f16 *data, const int *poff, unsigned lane_w, unsigned hi,
                                           int q0, int qlast, f16x8 (&w)[TL_DEPTH], int (&o)[TL_DEPTH]) {
#pragma unroll
    for (int i = 0; i < TL_DEPTH; i++)
        tl_load_pair(data, poff, min(q0 + i, qlast), lane_w, hi, w[i], o[i]);
}


// bvec: lane j holds the first pair of block-row j, lane NB the end of the
// last one (read back with v_readlane)
template <int NB, class Flush>
__device__ __forceinline__ void tl_stream(const char *xlane, int xrow16, const f16 *data,
                                          const int *poff, unsigned lane_w, unsigned hi, int q0,
                                          int qend, int qlast, int bvec, f16x8 (&w)[TL_DEPTH],
                                          int (&o)[TL_DEPTH], Flush &&flush
) {
    if (q0 >= qend)
        return;
    __builtin_amdgcn_s_setprio(TL_PRIO);
    f32x4 cur0 = f32x4{0.f, 0.f, 0.f, 0.f}, cur1 = f32x4{0.f, 0.f, 0.f, 0.f};
    int j = 0;
    int bend = __builtin_amdgcn_readlane(bvec, 1);
#pragma unroll
    for (int t = 0; t < NB - 1; t++) { // leading empty block-rows
        j += (bend == q0 && j + 1 < NB) ? 1 : 0;
        bend = __builtin_amdgcn_readlane(bvec, j + 1);
    }
    f16x8 xa[2], xb[2];
    xa[0] = *reinterpret_cast<const f16x8 *>(xlane + o[0]);
    xb[0] = *reinterpret_cast<const f16x8 *>(xlane + o[0] + xrow16);
    xa[1] = xb[1] = f16x8{0, 0, 0, 0, 0, 0, 0, 0};
    int q = q0;
    // running (wave-uniform) addresses of pair q + TL_DEPTH: a stage adds a
    // constant, which goes into the load's immediate offset
    const char *wp = reinterpret_cast<const char *>(data) + (size_t)(q0 + TL_DEPTH) * 1024;
    const char *op = reinterpret_cast<const char *>(poff) + (size_t)(q0 + TL_DEPTH) * 8;
    unsigned lane_lo = hi * 4u, lane_lw = lane_w * 2u;
    auto stage = [&](auto ic, auto always) {
        constexpr int I = decltype(ic)::value;
        constexpr int S = I % TL_DEPTH, SN = (I + 1) % TL_DEPTH, P = I & 1;
        xa[P ^ 1] = *reinterpret_cast<const f16x8 *>(xlane + o[SN]);
        xb[P ^ 1] = *reinterpret_cast<const f16x8 *>(xlane + o[SN] + xrow16);
        // keep the reads above the MFMAs: left alone, the scheduler sinks them
        // to the end of the stage and every stage then waits out the LDS latency
        __builtin_amdgcn_sched_barrier(0);
        cur0 = mfma16x16x32(w[S], xa[P], cur0);
        cur1 = mfma16x16x32(w[S], xb[P], cur1);
        // pair q + I + TL_DEPTH; the last stages of a stream request nothing:
        // a request still in flight when the stream ends would make the next
        // use of these registers wait out a full memory latency
        if (decltype(always)::value || q + I + TL_DEPTH < qend)
            tl_load_pair_at(wp + I * 1024, op + I * 8, lane_lo, lane_lw, w[S], o[S]);
        if (q + I + 1 == bend) { // block-row j is complete
            __builtin_amdgcn_s_setprio(0);
            flush(j, cur0, cur1);
            __builtin_amdgcn_s_setprio(TL_PRIO);
            cur0 = f32x4{0.f, 0.f, 0.f, 0.f};
            cur1 = f32x4{0.f, 0.f, 0.f, 0.f};
            j++;
            bend = __builtin_amdgcn_readlane(bvec, min(j + 1, NB));
#pragma unroll
            for (int t = 0; t < NB - 2; t++) { // skip empty block-rows
                j += (bend == q + I + 1 && j + 1 < NB) ? 1 : 0;
                bend = __builtin_amdgcn_readlane(bvec, min(j + 1, NB));
            }
        }
    };
    for (; q + 2 * TL_DEPTH <= qend; q += TL_DEPTH) { // straight-line body: counted waits
        tl_static_for<0, TL_DEPTH>([&](auto ic) { stage(ic, std::true_type()); });
        wp += TL_DEPTH * 1024;
        op += TL_DEPTH * 8;
    }
    tl_static_for<0, 2 * TL_DEPTH - 1>([&](auto ic) {
        if (q + decltype(ic)::value < qend)
            stage(ic, std::false_type());
    });
    __builtin_amdgcn_s_setprio(0);
}

// The same stream over a 64-row panel: every W pair is used for four 16-row
// subtiles (four MFMAs per kilobyte of W instead of two: the stream is bound by
// delivering W, so this is what raises its throughput).  flush(j, c0..c3).
template <int NB, class Flush>
__device__ __forceinline__ void tl_stream64(const char *xlane, int xrow16, const f16 *data,
                                          const int *poff, unsigned lane_w, unsigned hi, int q0,
                                          int qend, int qlast, int bvec, f16x8 (&w)[TL_DEPTH],
                                          int (&o)[TL_DEPTH], Flush &&flush
) {
    if (q0 >= qend)
        return;
    f32x4 cur0 = f32x4{0.f, 0.f, 0.f, 0.f}, cur1 = cur0, cur2 = cur0, cur3 = cur0;
    int j = 0;
    int bend = __builtin_amdgcn_readlane(bvec, 1);
#pragma unroll
    for (int t = 0; t < NB - 1; t++) { // leading empty block-rows
        j += (bend == q0 && j + 1 < NB) ? 1 : 0;
        bend = __builtin_amdgcn_readlane(bvec, j + 1);
    }
    f16x8 xa[2], xb[2], xc[2], xd[2];
    xa[0] = *reinterpret_cast<const f16x8 *>(xlane + o[0]);
    xb[0] = *reinterpret_cast<const f16x8 *>(xlane + o[0] + xrow16);
    xc[0] = *reinterpret_cast<const f16x8 *>(xlane + o[0] + 2 * xrow16);
    xd[0] = *reinterpret_cast<const f16x8 *>(xlane + o[0] + 3 * xrow16);
    xa[1] = xb[1] = xc[1] = xd[1] = f16x8{0, 0, 0, 0, 0, 0, 0, 0};
    int q = q0;
    // running (wave-uniform) addresses of pair q + TL_DEPTH: a stage adds a
    // constant, which goes into the load's immediate offset
    const char *wp = reinterpret_cast<const char *>(data) + (size_t)(q0 + TL_DEPTH) * 1024;
    const char *op = reinterpret_cast<const char *>(poff) + (size_t)(q0 + TL_DEPTH) * 8;
    unsigned lane_lo = hi * 4u, lane_lw = lane_w * 2u;
    auto stage = [&](auto ic, auto always) {
        constexpr int I = decltype(ic)::value;
        constexpr int S = I % TL_DEPTH, SN = (I + 1) % TL_DEPTH, P = I & 1;
        xa[P ^ 1] = *reinterpret_cast<const f16x8 *>(xlane + o[SN]);
        xb[P ^ 1] = *reinterpret_cast<const f16x8 *>(xlane + o[SN] + xrow16);
        xc[P ^ 1] = *reinterpret_cast<const f16x8 *>(xlane + o[SN] + 2 * xrow16);
        xd[P ^ 1] = *reinterpret_cast<const f16x8 *>(xlane + o[SN] + 3 * xrow16);
        // keep the reads above the MFMAs: left alone, the scheduler sinks them
        // to the end of the stage and every stage then waits out the LDS latency
        __builtin_amdgcn_sched_barrier(0);
        cur0 = mfma16x16x32(w[S], xa[P], cur0);
        cur1 = mfma16x16x32(w[S], xb[P], cur1);
        cur2 = mfma16x16x32(w[S], xc[P], cur2);
        cur3 = mfma16x16x32(w[S], xd[P], cur3);
        // pair q + I + TL_DEPTH; the last stages of a stream request nothing:
        // a request still in flight when the stream ends would make the next
        // use of these registers wait out a full memory latency
        if (decltype(always)::value || q + I + TL_DEPTH < qend)
            tl_load_pair_at(wp + I * 1024, op + I * 8, lane_lo, lane_lw, w[S], o[S]);
        if (q + I + 1 == bend) { // block-row j is complete
            flush(j, cur0, cur1, cur2, cur3);
            cur0 = cur1 = cur2 = cur3 = f32x4{0.f, 0.f, 0.f, 0.f};
            j++;
            bend = __builtin_amdgcn_readlane(bvec, min(j + 1, NB));
#pragma unroll
            for (int t = 0; t < NB - 2; t++) { // skip empty block-rows
                j += (bend == q + I + 1 && j + 1 < NB) ? 1 : 0;
                bend = __builtin_amdgcn_readlane(bvec, min(j + 1, NB));
            }
        }
    };
    for (; q + 2 * TL_DEPTH <= qend; q += TL_DEPTH) { // straight-line body: counted waits
        tl_static_for<0, TL_DEPTH>([&](auto ic) { stage(ic, std::true_type()); });
        wp += TL_DEPTH * 1024;
        op += TL_DEPTH * 8;
    }
    tl_static_for<0, 2 * TL_DEPTH - 1>([&](auto ic) {
        if (q + decltype(ic)::value < qend)
            stage(ic, std::false_type());
    });
}

// flush for kernels that keep NB static accumulators: acc[j] += cur with a
// 0/1 mask per accumulator (branch-free; a branch per j makes the compiler
// keep a copy of every accumulator per pipeline stage)
template <int NB>
__device__ __forceinline__ void tl_flush_acc(f32x4 (&acc)[NB][2], int j, f32x4 cur0, f32x4 cur1) {
#pragma unroll
    for (int k = 0; k < NB; k++) {
        const float mk = (k == j) ? 1.0f : 0.0f;
#pragma unroll
        for (int r = 0; r < 4; r++) {
            acc[k][0][r] = __builtin_fmaf(cur0[r], mk, acc[k][0][r]);
            acc[k][1][r] = __builtin_fmaf(cur1[r], mk, acc[k][1][r]);
        }
    }
}

// The same with a branch per accumulator instead of NB masked multiply-adds
// (eight adds per flush instead of 8 NB fused multiply-adds and NB selects).
// Two things keep the compiler from undoing it: the adds are inline assembly
// with tied operands (the sum replaces the accumulator in its own registers;
// otherwise every accumulator gets a second set of registers behind the
// branches), and the cases are independent ifs with something opaque between
// them (as an if / else chain they become a switch, whose lowering copies the
// accumulators around or addresses them through scratch memory).
template <int K>
__device__ __forceinline__ void tl_add_tied(f32x4 &a, const f32x4 &c) {
    float a0 = a[0], a1 = a[1], a2 = a[2], a3 = a[3];
    asm volatile("v_add_f32 %0, %0, %4 ; accumulator %8\n\tv_add_f32 %1, %1, %5\n\t"
                 "v_add_f32 %2, %2, %6\n\tv_add_f32 %3, %3, %7"
                 : "+v"(a0), "+v"(a1), "+v"(a2), "+v"(a3)
                 : "v"(c[0]), "v"(c[1]), "v"(c[2]), "v"(c[3]), "n"(K));
    a = f32x4{a0, a1, a2, a3};
}
template <int NB>
__device__ __forceinline__ void tl_flush_acc_branch(f32x4 (&acc)[NB][2], int j, const f32x4 &cur0, const f32x4 &cur1) {
    tl_static_for<0, NB>([&](auto kc) {
        constexpr int k = decltype(kc)::value;
        if (j == k) {
            tl_add_tied<k>(acc[k][0], cur0);
            tl_add_tied<k>(acc[k][1], cur1);
        }
        asm volatile("; after case %0" ::"n"(k));
    });
}

// Fused skip connection + LayerNorm over a workgroup's 32 finished rows (the
// math of skip_layernorm.hip: x = half(y + skip), fp32 mean and biased
// two-pass variance, eps 1e-6).  The workgroup covers the whole row: wave k's
// staging tile holds columns [k*16*NB, (k+1)*16*NB), k < NW.  Wave w of the NLW
// waves that take part normalises rows w, w+NLW, ..., a row spread over its 64
// lanes in 16-byte pieces.  The operands that come from global memory (the
// skip rows, gamma, beta) are requested by tl_ln_fetch, which a wave calls
// BEFORE the barrier that ends the staging writes, so that their latency runs
// under the wait for the other waves.
template <int NB, int NW, int NLW>
struct TlLnOperands {
    static constexpr int NCH = (NW * NB * 2 + 63) / 64;    // 16-byte pieces per lane and row
    static constexpr int ROWS = (TL_BM + NLW - 1) / NLW;   // rows per wave
    f16x8 skip[ROWS][NCH], gamma[NCH], beta[NCH];
};

// (skip0 / Y0 point at the panel's first row, in global memory or in LDS, with
// row pitches ldskip / ldy in halves)
template <int NB, int NW, int NLW>
__device__ __forceinline__ void tl_ln_fetch_at(TlLnOperands<NB, NW, NLW> &op, int M, int wave, int lane,
                                               int m0, int N, const f16 *skip0, long ldskip,
                                               const f16 *gamma, const f16 *beta) {
    constexpr int NCH = TlLnOperands<NB, NW, NLW>::NCH;
    constexpr int ROWS = TlLnOperands<NB, NW, NLW>::ROWS;
    const int npiece = N >> 3;
#pragma unroll
    for (int i = 0; i < NCH; i++) {
        const int ch = min(lane + 64 * i, npiece - 1); // (clamped pieces are never used)
#pragma unroll
        for (int k = 0; k < ROWS; k++) {
            const long r = min((long)wave + k * NLW, (long)M - 1 - m0);
            op.skip[k][i] = *reinterpret_cast<const f16x8 *>(skip0 + r * ldskip + ch * 8);
        }
        op.gamma[i] = *reinterpret_cast<const f16x8 *>(gamma + ch * 8);
        op.beta[i] = *reinterpret_cast<const f16x8 *>(beta + ch * 8);
    }
}

template <int NB, int NW, int NLW>
__device__ __forceinline__ void tl_ln_fetch(TlLnOperands<NB, NW, NLW> &op, const TlArgs &a, int wave,
                                            int lane, int m0, int N) {
    tl_ln_fetch_at(op, a.M, wave, lane, m0, N, a.skip + (long)m0 * N, (long)N, a.gamma, a.beta);
}

template <int NB, int NW, int NLW>
__device__ __forceinline__ void tl_ln_rows_at(const TlLnOperands<NB, NW, NLW> &op, int M,
                                              const f16 *stage0, int wave, int lane, int m0, int N,
                                              f16 *Y0, long ldy);

template <int NB, int NW, int NLW>
__device__ __forceinline__ void tl_ln_rows(const TlLnOperands<NB, NW, NLW> &op, const TlArgs &a,
                                           const f16 *stage0, int wave, int lane, int m0, f16 *Y, int N) {
    tl_ln_rows_at(op, a.M, stage0, wave, lane, m0, N, Y + (long)m0 * N, (long)N);
}

template <int NB, int NW, int NLW>
__device__ __forceinline__ void tl_ln_rows_at(const TlLnOperands<NB, NW, NLW> &op, int M,
                                              const f16 *stage0, int wave, int lane, int m0, int N,
                                              f16 *Y0, long ldy) {
    constexpr int lds = 16 * NB + 8;
    constexpr int NCH = TlLnOperands<NB, NW, NLW>::NCH;
    constexpr int ROWS = TlLnOperands<NB, NW, NLW>::ROWS;
    const int npiece = N >> 3;
    const float inv_n = 1.0f / (float)N;
    const f16x8 zero8 = f16x8{0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
    for (int k = 0; k < ROWS; k++) {
        const int r = wave + k * NLW;
        if (r >= TL_BM || m0 + r >= M)
            break;
        f16x8 xv[NCH];
        float sum = 0.f;
#pragma unroll
        for (int i = 0; i < NCH; i++) {
            const int ch = lane + 64 * i;
            xv[i] = zero8;
            if (ch < npiece) {
                const int tile = ch / (2 * NB), c = ch - tile * (2 * NB);
                const f16x8 y = *reinterpret_cast<const f16x8 *>(
                    stage0 + tile * tl_wave_stage_halves<NB>() + r * lds + c * 8);
                xv[i] = y + op.skip[k][i]; // half add, one rounding (kernels/skip_layernorm.cu:20)
            }
            // (pairs of halves summed in fp32 by the dot-product unit: no conversions)
            typedef _Float16 h2 __attribute__((ext_vector_type(2)));
#pragma unroll
            for (int j = 0; j < 8; j += 2)
                sum = __builtin_amdgcn_fdot2(h2{xv[i][j], xv[i][j + 1]}, h2{(f16)1, (f16)1}, sum, false);
        }
        const float mean = wave_sum(sum) * inv_n;
        float var = 0.f;
#pragma unroll
        for (int i = 0; i < NCH; i++)
            if (lane + 64 * i < npiece) {
#pragma unroll
                for (int j = 0; j < 8; j++) {
                    const float d = (float)xv[i][j] - mean;
                    var += d * d;
                }
            }
        const float rstd = rsqrtf(wave_sum(var) * inv_n + 1e-6f);
        const float shift = -mean * rstd;
#pragma unroll
        for (int i = 0; i < NCH; i++) {
            const int ch = lane + 64 * i;
            if (ch < npiece) {
                f16x8 o;
#pragma unroll
                for (int j = 0; j < 8; j++) // ((x - mean) * rstd) * gamma + beta, the first step as one fma
                    o[j] = (f16)(__builtin_fmaf((float)xv[i][j], rstd, shift) * (float)op.gamma[i][j] +
                                 (float)op.beta[i][j]);
                *reinterpret_cast<f16x8 *>(Y0 + r * ldy + ch * 8) = o;
            }
        }
    }
}

// ---------------------------------------------------------------------------
// Plan kernel (the fast path).
//
// Work items are (row panel, linear, column group) triples, numbered with the
// row panel slowest.  A workgroup is persistent over `ipw` consecutive items:
// as long as the row panel does not change (and K fits one chunk) the X panel
// stays in LDS, so it is fetched once for several column groups, and because
// every wave stages its output through a private LDS tile the waves never
// meet at a barrier between items - one wave's stores overlap the others'
// MFMAs and the next item's weight loads.
//
// Within an item a wave owns NB CONSECUTIVE block-rows, and the plan stores
// tiles in (chunk, block-row) order with even segments, so the wave's work for
// a chunk is ONE contiguous stream of tile pairs: 1 KB of W per pair at an
// address that is linear in the pair index, plus one int per half-wave giving
// the LDS byte offset of that tile's X columns.  The stream is consumed
// through a fixed 4-stage register pipeline (stage = pair index mod 4, see
// tl_stream), so four pairs are always in flight per wave and the waits are
// counted, not drained.  Products accumulate
// into one running 32x16 accumulator; when the stream crosses a block-row
// boundary (a scalar compare per pair) it is added into that block-row's
// static accumulator.
// ---------------------------------------------------------------------------

template <int NB, bool GELU, int NW, bool LN>
__global__ void __launch_bounds__(NW * 64) tile_linear_plan_kernel(const TlArgs a) {
    extern __shared__ __attribute__((aligned(16))) unsigned char tl_smem[];
    f16 *xs = reinterpret_cast<f16 *>(tl_smem);
    // Workgroups with consecutive virtual ids run on ONE XCD (hardware
    // round-robins consecutive workgroup ids over the 8 XCDs), so the column
    // groups of a row panel that do not fit one workgroup share that XCD's L2.
    const int vid = (blockIdx.x & 7) * a.per_xcd + (blockIdx.x >> 3);
    const int it0 = vid * a.ipw;
    const int it1 = min(it0 + a.ipw, a.total);
    if (it0 >= it1)
        return;
    TlCtx x;
    x.wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    x.lane = threadIdx.x & 63;
    x.c16 = x.lane & 15;
    x.g4 = x.lane >> 4;
    x.khalf8 = (x.g4 & 1) * 8;
    x.hi = x.lane >> 5;
    x.ldx = a.KC + ((a.KC & 31) ? 0 : TL_PAD);
    const int hi = x.hi, lane = x.lane;
    const char *xlane = reinterpret_cast<const char *>(xs + x.c16 * x.ldx + x.khalf8);
    const int xrow16 = 16 * x.ldx * 2; // bytes between the two 16-row subtiles
    f16 *const stage0 = xs + TL_BM * x.ldx;
    f16 *const stage = stage0 + x.wave * tl_wave_stage_halves<NB>();
    const int per_rp = a.ncg * a.nlin;

    // X panel staging: global -> LDS directly (global_load_lds_dwordx4: lane L
    // of the issuing wave writes 16 bytes at  base + 16*L, the source address is
    // free per lane).  Wave w fills panel rows 4w..4w+3, each row as one 64-lane
    // and one partial instruction; no VGPRs are held and nothing waits until the
    // barrier.  Rows at or beyond M are left unwritten: a panel row only feeds
    // the output row of the same index, which is never stored.
#define TL_PANEL_LOAD(c_)                                                                         \
    {                                                                                             \
        const int pk0 = (c_) * a.KC;                                                              \
        const int pcpr = min(a.KC, a.K - pk0) >> 3; /* 16-byte chunks per row, <= 124 */          \
        _Pragma("unroll") for (int rr = 0; rr < TL_BM / NW; rr++) {                               \
            const int row = x.wave * (TL_BM / NW) + rr;                                           \
            if (x.m0 + row < a.M) {                                                               \
                const f16 *src = a.X + (size_t)(x.m0 + row) * a.K + pk0;                          \
                f16 *dstrow = xs + row * x.ldx;                                                   \
                if (lane < pcpr)                                                                  \
                    load_lds16(src + lane * 8, dstrow);                                           \
                if (64 + lane < pcpr)                                                             \
                    load_lds16(src + (64 + lane) * 8, dstrow + 512);                              \
            }                                                                                     \
        }                                                                                         \
    }

    int panel_rp = -1; // row panel currently in LDS (single-chunk problems only)
    bool lds_used = false;
    for (int it = it0; it < it1; it++) {
        const int rp = it / per_rp;
        const int rest = it - rp * per_rp;
        const int lin = rest / a.ncg;
        x.lin = lin;
        x.cg = rest - lin * a.ncg;
        x.m0 = rp * TL_BM;
        x.bn_wg = x.cg * (NW * NB);
        x.bn0 = x.bn_wg + x.wave * NB;
        f16 *const Yp = TL_SEL(Y);
        const int *const cptr = TL_SEL(cptr);
        const int *const poff = TL_SEL(row_offset); // LDS byte offset per tile (chunk-local column * 2)
        const f16 *const data = TL_SEL(data);
        const f16 *const bias = TL_SEL(bias);
        const int N = TL_SEL(N);
        const int nbr = N >> 4;

        f32x4 acc[NB][2];
        f16x4 b4[NB];
#pragma unroll
        for (int j = 0; j < NB; j++) {
            acc[j][0] = f32x4{0.f, 0.f, 0.f, 0.f};
            acc[j][1] = f32x4{0.f, 0.f, 0.f, 0.f};
            b4[j] = f16x4{0, 0, 0, 0};
            if (x.bn0 + j < nbr)
                b4[j] = *reinterpret_cast<const f16x4 *>(bias + (x.bn0 + j) * 16 + x.g4 * 4);
        }
        const unsigned lane_w = hi * 256 + x.c16 * 16 + x.khalf8; // lane's halves inside a 1 KB tile pair

        for (int c = 0; c < a.nchunk; c++) {
            // pair-index boundaries of the wave's block-rows: lane j holds the end
            // of block-row j (read back with v_readlane)
            const int bidx = c * nbr + min(x.bn0 + min(lane, NB), nbr);
            const int bvec = cptr[bidx] >> 1;

            const bool reload = a.nchunk > 1 || rp != panel_rp; // workgroup-uniform
            if (reload) {
                // (The load, its wait and both barriers stay in this one block:
                // with the wait further down, behind the first weight loads,
                // the compiler loses track of the DMA and drains every load in
                // the pipelined loop below instead of counting.)
                if (lds_used)
                    __syncthreads(); // every wave is done with the previous panel
                TL_PANEL_LOAD(c)
                lds_used = true;
                __builtin_amdgcn_s_waitcnt(0x0F70); // vmcnt(0): this wave's part has landed
                __syncthreads();                    // ... and everyone else's
            }
            // the first pairs of the stream
            const int q0 = __builtin_amdgcn_readfirstlane(bvec);
            const int qend = __builtin_amdgcn_readlane(bvec, NB);
            const int qlast = max(qend - 1, q0);
            f16x8 w[TL_DEPTH];
            int o[TL_DEPTH];
            tl_preload(data, poff, lane_w, hi, q0, qlast, w, o);
            tl_stream<NB>(xlane, xrow16, data, poff, lane_w, hi, q0, qend, qlast, bvec, w, o,
                          [&](int j, f32x4 c0, f32x4 c1) { tl_flush_acc<NB>(acc, j, c0, c1); });
        }
        panel_rp = a.nchunk > 1 ? -1 : rp;
        tl_epilogue_wave<NB, GELU, !LN>(a, x, stage, Yp, N, nbr, acc, b4);
        if constexpr (LN) {
            TlLnOperands<NB, NW, NW> lnop;
            tl_ln_fetch(lnop, a, x.wave, lane, x.m0, N);
            __syncthreads(); // every wave's part of the rows is staged
            tl_ln_rows(lnop, a, stage0, x.wave, lane, x.m0, Yp, N);
            lds_used = true; // (the next item's panel load starts with a barrier)
        }
    }
#undef TL_PANEL_LOAD
}

// ---------------------------------------------------------------------------
// Resident-panel kernel: the plan kernel for K that fits one LDS panel (every
// BERT-base linear except FFN2).  Same tile stream and 4-stage pipeline as
// above, with three differences that take work off the critical path of a
// wave:
//  * a finished block-row is converted (bias, GELU, half) and written to the
//    wave's staging tile right where the stream crosses its boundary, so there
//    are no per-block-row accumulators to fold into and the conversion work
//    overlaps the weight loads already in flight;
//  * the next item's block-row boundaries and bias are requested before the
//    current item's stream starts, and its first four weight pairs before the
//    current item's output tile is stored - a wave sees one memory latency per
//    item instead of three;
//  * items that share the row panel reuse it without any barrier.
// ---------------------------------------------------------------------------
// Workgroup barrier that orders LDS traffic only.  __syncthreads() also fences
// global memory, which would make every wave drain the weight pairs it has
// just requested; this one is for hand-overs of LDS buffers.
__device__ __forceinline__ void tl_barrier_lds() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

struct TlItem {
    int rp, lin, cg, bn0, nbr, N;
    f16 *Y;
    const int *cptr;
    const int *poff;
    const f16 *data;
    const f16 *bias;
};

// one finished 32x16 block-row tile -> wave-private staging tile
template <bool GELU>
__device__ __forceinline__ void tl_stage_tile(f16 *dst, int lds, f32x4 c0, f32x4 c1, f16x4 bj) {
    const f32x4 bf = __builtin_convertvector(bj, f32x4);
    f16x4 o0 = __builtin_convertvector(c0 + bf, f16x4);
    f16x4 o1 = __builtin_convertvector(c1 + bf, f16x4);
    if (GELU) {
        o0 = gelu4(o0);
        o1 = gelu4(o1);
    }
    *reinterpret_cast<f16x4 *>(dst) = o0;
    *reinterpret_cast<f16x4 *>(dst + 16 * lds) = o1;
}

template <int NB, bool GELU, int NW, bool LN, int BM = TL_BM>
__global__ void __launch_bounds__(NW * 64) tile_linear_resident_kernel(const TlArgs a) {
    // BM = 64: 64-row panels and items (tl_stream64: four MFMAs per streamed W
    // pair), one workgroup per CU - the panel and the 64-row staging tiles fill
    // the LDS.  Chosen by the launcher where enough 64-row items exist.
    static_assert(BM == TL_BM || (BM == 2 * TL_BM && !LN), "64-row panels: without the LayerNorm epilogue");
    extern __shared__ __attribute__((aligned(16))) unsigned char tl_smem[];
    f16 *xs = reinterpret_cast<f16 *>(tl_smem);
    const int vid = (blockIdx.x & 7) * a.per_xcd + (blockIdx.x >> 3); // see tile_linear_plan_kernel
    const int it0 = vid * a.ipw;
    const int it1 = min(it0 + a.ipw, a.total);
    if (it0 >= it1)
        return;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int lane = threadIdx.x & 63;
    const int c16 = lane & 15, g4 = lane >> 4, khalf8 = (g4 & 1) * 8, hi = lane >> 5;
    const int ldx = a.KC + ((a.KC & 31) ? 0 : TL_PAD);
    const char *xlane = reinterpret_cast<const char *>(xs + c16 * ldx + khalf8);
    const int xrow16 = 16 * ldx * 2; // bytes between the two 16-row subtiles
    constexpr int lds = 16 * NB + 8; // halves per staged row
    f16 *const stage0 = xs + BM * ldx;
    f16 *const stage = stage0 + wave * (BM * (16 * NB + 8));
    f16 *const stage_lane = stage + c16 * lds + g4 * 4;
    const int lane_w = hi * 256 + c16 * 16 + khalf8; // lane's halves inside a 1 KB tile pair

    // pair-index boundaries of a wave's block-rows: lane j holds the start of
    // block-row j, lane NB the end of the last one (read back with v_readlane)
#define TL_BVEC(t_) ((t_).cptr[min((t_).bn0 + min(lane, NB), (t_).nbr)] >> 1)
    // (block-rows beyond the matrix read the last block-row's bias; their
    // output is never stored)
#define TL_BIAS(dst_, t_)                                                                         \
    _Pragma("unroll") for (int k = 0; k < NB; k++)                                                \
        dst_[k] = *reinterpret_cast<const f16x4 *>(                                               \
            (t_).bias + min((t_).bn0 + k, (t_).nbr - 1) * 16 + g4 * 4);
    // wave w fills panel rows (BM/NW)w ... (see tile_linear_plan_kernel)
#define TL_PANEL(rp_)                                                                             \
    {                                                                                             \
        const int pcpr = a.K >> 3;                                                                \
        constexpr int RPW = (BM + NW - 1) / NW; /* panel rows per wave */                         \
        _Pragma("unroll") for (int rr = 0; rr < RPW; rr++) {                                      \
            const int prow = wave * RPW + rr;                                                     \
            const int row = (rp_) * BM + prow;                                                    \
            if (row < a.M && (BM % NW == 0 || prow < BM)) {                                       \
                const f16 *src = a.X + (size_t)row * a.K;                                         \
                f16 *dstrow = xs + prow * ldx;                                                    \
                if (lane < pcpr)                                                                  \
                    load_lds16(src + lane * 8, dstrow);                                           \
                if (64 + lane < pcpr)                                                             \
                    load_lds16(src + (64 + lane) * 8, dstrow + 512);                              \
            }                                                                                     \
        }                                                                                         \
        __builtin_amdgcn_s_waitcnt(0x0F70); /* vmcnt(0): this wave's part has landed */           \
        __syncthreads();                    /* ... and everyone else's */                         \
    }
    // the first pairs of an item's stream
#define TL_PRELOAD(t_, bvec_)                                                                     \
    {                                                                                             \
        q0 = __builtin_amdgcn_readfirstlane(bvec_);                                               \
        qend = __builtin_amdgcn_readlane(bvec_, NB);                                              \
        qlast = max(qend - 1, q0);                                                                \
        wdata = (t_).data;                                                                        \
        wpoff = (t_).poff;                                                                        \
        tl_preload(wdata, wpoff, lane_w, hi, q0, qlast, w, o);                                    \
    }

    // Per-linear arguments are read from the kernel-argument segment with a
    // run-time index (scalar loads).  Indexing the by-value struct itself would
    // make the compiler copy it to scratch memory, and chains of selects over
    // its constant-indexed elements compile to long branch ladders.
    typedef const __attribute__((address_space(4))) char *KArg;
    const KArg ka = (KArg)__builtin_amdgcn_kernarg_segment_ptr(); // TlArgs is the only argument
#define TL_KARG(type_, field_, lin_)                                                              \
    (*(const __attribute__((address_space(4))) type_ *)(ka + offsetof(TlArgs, field_) +           \
                                                         (lin_) * sizeof(type_)))
    auto tl_item = [&](int rp, int lin, int cg) {
        TlItem t;
        t.rp = rp;
        t.lin = lin;
        t.cg = cg;
        t.bn0 = (cg * NW + wave) * NB;
        typedef f16 *YPtr;
        typedef const int *IPtr;
        typedef const f16 *HPtr;
        t.Y = TL_KARG(YPtr, Y, lin);
        t.cptr = TL_KARG(IPtr, cptr, lin);
        t.poff = TL_KARG(IPtr, row_offset, lin);
        t.data = TL_KARG(HPtr, data, lin);
        t.bias = TL_KARG(HPtr, bias, lin);
        t.N = TL_KARG(int, N, lin);
        t.nbr = t.N >> 4;
        return t;
    };
    // the item after t in (row panel, linear, column group) order
    auto tl_next = [&](const TlItem &t) {
        const bool cw = t.cg + 1 == a.ncg;
        const bool lw = cw && t.lin + 1 == a.nlin;
        return tl_item(t.rp + (lw ? 1 : 0), lw ? 0 : t.lin + (cw ? 1 : 0), cw ? 0 : t.cg + 1);
    };
    const int per_rp = a.ncg * a.nlin;
    const int rp0 = it0 / per_rp, rest0 = it0 - rp0 * per_rp;
    TlItem cur = tl_item(rp0, rest0 / a.ncg, rest0 % a.ncg);

    int bvec = TL_BVEC(cur);
    f16x4 b4[NB];
    TL_BIAS(b4, cur)
    TL_PANEL(cur.rp)
    int q0, qend, qlast;
    const f16 *wdata;
    const int *wpoff;
    f16x8 w[TL_DEPTH];
    int o[TL_DEPTH];
    TL_PRELOAD(cur, bvec)

    for (int it = it0;; it++) {
        const bool has_next = it + 1 < it1;
        const TlItem nxt = tl_next(cur); // (past the last item: a valid linear, never run)
        const int bvec_n = TL_BVEC(nxt);
        f16x4 b4n[NB];
        TL_BIAS(b4n, nxt)

        // a finished block-row goes straight to the wave's staging tile
        // bias of block-row j as a 0/1-masked sum (exact); a chain of selects
        // over b4[] would be turned into an indexed load and put the array into
        // scratch memory
        auto bias_of = [&](int j) {
            f16x4 bj = f16x4{0, 0, 0, 0};
#pragma unroll
            for (int k = 0; k < NB; k++)
                bj += b4[k] * ((j == k) ? (f16)1 : (f16)0);
            return bj;
        };
        if constexpr (BM == TL_BM) {
            tl_stream<NB>(xlane, xrow16, wdata, wpoff, lane_w, hi, q0, qend, qlast, bvec, w, o,
                          [&](int j, f32x4 c0, f32x4 c1) {
                              tl_stage_tile<GELU>(stage_lane + j * 16, lds, c0, c1, bias_of(j));
                          });
        } else {
            tl_stream64<NB>(xlane, xrow16, wdata, wpoff, lane_w, hi, q0, qend, qlast, bvec, w, o,
                            [&](int j, f32x4 c0, f32x4 c1, f32x4 c2, f32x4 c3) {
                                const f16x4 bj = bias_of(j);
                                tl_stage_tile<GELU>(stage_lane + j * 16, lds, c0, c1, bj);
                                tl_stage_tile<GELU>(stage_lane + 32 * lds + j * 16, lds, c2, c3, bj);
                            });
        }
        // block-rows without any tile: bias only
#pragma unroll
        for (int k = 0; k < NB; k++)
            if (__builtin_amdgcn_readlane(bvec, k) == __builtin_amdgcn_readlane(bvec, k + 1)) {
#pragma unroll
                for (int h = 0; h < BM / TL_BM; h++)
                    tl_stage_tile<GELU>(stage_lane + h * 32 * lds + k * 16, lds, f32x4{0.f, 0.f, 0.f, 0.f},
                                        f32x4{0.f, 0.f, 0.f, 0.f}, b4[k]);
            }

        const bool same_panel = has_next && nxt.rp == cur.rp;
        if (same_panel)
            TL_PRELOAD(nxt, bvec_n)

        if constexpr (LN) {
            // the workgroup holds whole rows: skip connection + LayerNorm here
            TlLnOperands<NB, NW, NW> lnop;
            tl_ln_fetch(lnop, a, wave, lane, cur.rp * BM, cur.N);
            __syncthreads(); // every wave's part of the rows is staged
            tl_ln_rows(lnop, a, stage0, wave, lane, cur.rp * BM, cur.Y, cur.N);
            if (has_next && same_panel)
                __syncthreads(); // the staging tiles are free again
        } else {
            // staging tile -> Y: 16-byte stores of 32*NB contiguous bytes per row
            const int nvalid = min(NB, cur.nbr - cur.bn0); // the last column group may be partial
            const int cpr = 2 * nvalid;                    // 16-byte chunks per row
            const int m0 = cur.rp * BM;
            f16 *ybase = cur.Y + (size_t)m0 * cur.N + cur.bn0 * 16;
#pragma unroll
            for (int t = 0; t < NB * (BM / TL_BM); t++) {
                const int i = lane + 64 * t;
                const int r = i / (2 * NB), c = i - r * (2 * NB);
                if (c < cpr && m0 + r < a.M) {
                    const u32x4 v = *reinterpret_cast<const u32x4 *>(stage + r * lds + c * 8);
                    *reinterpret_cast<u32x4 *>(ybase + (size_t)r * cur.N + c * 8) = v;
                }
            }
        }
        if (!has_next)
            break;
        if (!same_panel) {
            __syncthreads(); // every wave is done with the previous panel
            TL_PANEL(nxt.rp)
            TL_PRELOAD(nxt, bvec_n)
        }
        cur = nxt;
        bvec = bvec_n;
#pragma unroll
        for (int k = 0; k < NB; k++)
            b4[k] = b4n[k];
    }
#undef TL_PRELOAD
#undef TL_PANEL
#undef TL_BIAS
#undef TL_BVEC
#undef TL_KARG
}

// ---------------------------------------------------------------------------
// Chunked fused kernel: linear + skip + LayerNorm for K beyond one LDS panel
// (FFN2 of BERT-base, K = 3072, N = 768).  One workgroup per row panel holds
// whole rows: twelve computing waves of NB block-rows each and a thirteenth
// wave that does nothing but fetch.  K is walked in chunks through two LDS
// panel buffers; the fetching wave requests chunk c+1 (global -> LDS DMA) as
// soon as the computing waves have left chunk c-1, so the fetch runs under
// chunk c's MFMAs.  It has to be a wave of its own: loads return in order
// within a wave, so a panel request in a computing wave's queue would hold
// back every weight pair requested after it.  One LDS-only barrier per chunk
// hands over both "chunk c has landed" and "buffer (c+1)&1 is free".  The
// computing waves run the pair stream and 4-stage pipeline of the plan kernel,
// restarted per chunk with the first pairs requested before the barrier.
// ---------------------------------------------------------------------------
constexpr int TL_CWAVES = 12;
constexpr int TL_CTHREADS = (TL_CWAVES + 1) * 64;

template <int NB>
__global__ void __launch_bounds__(TL_CTHREADS) tile_linear_chunked_ln_kernel(const TlArgs a) {
    extern __shared__ __attribute__((aligned(16))) unsigned char tl_smem[];
    f16 *xs = reinterpret_cast<f16 *>(tl_smem);
    const int rp = (blockIdx.x & 7) * a.per_xcd + (blockIdx.x >> 3);
    if (rp >= a.total)
        return;
    TlCtx x;
    x.lin = 0;
    x.cg = 0;
    x.m0 = rp * TL_BM;
    x.wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    x.lane = threadIdx.x & 63;
    x.c16 = x.lane & 15;
    x.g4 = x.lane >> 4;
    x.khalf8 = (x.g4 & 1) * 8;
    x.hi = x.lane >> 5;
    x.ldx = a.KC + ((a.KC & 31) ? 0 : TL_PAD);
    x.bn_wg = 0;
    x.bn0 = x.wave * NB;
    x.ld_r = x.ld_c = 0;
    const int lane = x.lane;
    const int pbuf = TL_BM * x.ldx; // halves per panel buffer
    f16 *const stage0 = xs + 2 * pbuf;
    f16 *const Yp = a.Y[0];
    const int N = a.N[0];
    const int nbr = N >> 4;

    if (x.wave == TL_CWAVES) {
        // ---- the fetching wave ----
#define TL_FETCH(c_)                                                                              \
    {                                                                                             \
        const int pk0 = (c_) * a.KC;                                                              \
        const int pcpr = min(a.KC, a.K - pk0) >> 3; /* 16-byte pieces per row, <= 124 */          \
        f16 *dst = xs + ((c_) & 1) * pbuf;                                                        \
        const int nrow = min(TL_BM, a.M - x.m0);                                                  \
        for (int row = 0; row < nrow; row++) {                                                    \
            const f16 *src = a.X + (size_t)(x.m0 + row) * a.K + pk0;                              \
            if (lane < pcpr)                                                                      \
                load_lds16(src + lane * 8, dst + row * x.ldx);                                    \
            if (64 + lane < pcpr)                                                                 \
                load_lds16(src + (64 + lane) * 8, dst + row * x.ldx + 512);                       \
        }                                                                                         \
    }
        TL_FETCH(0)
        __builtin_amdgcn_s_waitcnt(0x0F70); // vmcnt(0)
        if (a.nchunk > 1)
            TL_FETCH(1)
        tl_barrier_lds(); // chunk 0 is in LDS
        for (int c = 1; c < a.nchunk; c++) {
            __builtin_amdgcn_s_waitcnt(0x0F70); // chunk c has landed
            tl_barrier_lds();                   // ... and every wave has left chunk c-1
            if (c + 1 < a.nchunk)
                TL_FETCH(c + 1)
        }
#undef TL_FETCH
    } else {
        // ---- the computing waves ----
        const int *const cptr = a.cptr[0];
        const int hi = x.hi;
        f32x4 acc[NB][2];
        f16x4 b4[NB];
#pragma unroll
        for (int j = 0; j < NB; j++) {
            acc[j][0] = f32x4{0.f, 0.f, 0.f, 0.f};
            acc[j][1] = f32x4{0.f, 0.f, 0.f, 0.f};
            b4[j] = f16x4{0, 0, 0, 0};
            if (x.bn0 + j < nbr)
                b4[j] = *reinterpret_cast<const f16x4 *>(a.bias[0] + (x.bn0 + j) * 16 + x.g4 * 4);
        }
        const int xrow16 = 16 * x.ldx * 2; // bytes between the two 16-row subtiles
        const f16 *const data = a.data[0];
        const int *const poff = a.row_offset[0];
        const unsigned lane_w = hi * 256 + x.c16 * 16 + x.khalf8; // lane's halves inside a 1 KB tile pair
        // pair-index boundaries of the wave's block-rows in the current chunk
        // (see tile_linear_plan_kernel); the next chunk's are requested a chunk ahead
        int bvec = cptr[min(x.bn0 + min(lane, NB), nbr)] >> 1;

        for (int c = 0; c < a.nchunk; c++) {
            const char *xlane =
                reinterpret_cast<const char *>(xs + (c & 1) * pbuf + x.c16 * x.ldx + x.khalf8);
            const int q0 = __builtin_amdgcn_readfirstlane(bvec);
            const int qend = __builtin_amdgcn_readlane(bvec, NB);
            const int qlast = max(qend - 1, q0);
            f16x8 w[TL_DEPTH];
            int o[TL_DEPTH];
            tl_preload(data, poff, lane_w, hi, q0, qlast, w, o);
            const int cn = min(c + 1, a.nchunk - 1);
            const int bvec_n = cptr[cn * nbr + min(x.bn0 + min(lane, NB), nbr)] >> 1;
            const int bcur = bvec;
            tl_barrier_lds();

            tl_stream<NB>(xlane, xrow16, data, poff, lane_w, hi, q0, qend, qlast, bcur, w, o,
                          [&](int j, f32x4 c0, f32x4 c1) { tl_flush_acc<NB>(acc, j, c0, c1); });
            bvec = bvec_n;
        }
        f16 *stage = stage0 + x.wave * tl_wave_stage_halves<NB>();
        tl_epilogue_wave<NB, false, false>(a, x, stage, Yp, N, nbr, acc, b4);
    }
    TlLnOperands<NB, TL_CWAVES, TL_CWAVES + 1> lnop;
    tl_ln_fetch(lnop, a, x.wave, lane, x.m0, N);
    __syncthreads(); // every computing wave's part of the rows is staged
    tl_ln_rows(lnop, a, stage0, x.wave, lane, x.m0, Yp, N);
}

// ---------------------------------------------------------------------------
// Fused feed-forward block: Y = LayerNorm(skip + W2 * gelu(W1 * X + b1) + b2)
// in ONE launch (encoder/encoder.cu:36-44 runs it as MLP1, MLP2 and
// skip_layernorm with the [rows x ffn] intermediate written to and read back
// from memory).  One workgroup of 16 waves per 32-row panel keeps the panel of
// X in LDS and walks the hidden dimension in chunks of the second plan's
// chunk width: phase p computes hidden columns [p*KC, (p+1)*KC) with the first
// linear (bias, GELU, rounded to half exactly like the stored intermediate)
// into one of two LDS buffers, then multiplies that buffer with chunk p of the
// second linear into register accumulators that live across all phases.  The
// hidden activations never leave the CU.  Each wave owns NB block-rows of
// either linear per phase.  The first linear runs one phase ahead of the
// second, and the hand-overs ("hidden buffer p is complete", "everyone has
// finished reading it") are event counters in LDS rather than barriers, so a
// wave only ever waits when it is a whole stream ahead of the slowest wave.
// WITH_O: the attention output projection with its skip connection and
// LayerNorm (encoder/encoder.cu:33-35) runs first on the same panel, and its
// normalised rows replace the panel in LDS - steps 6-10 of a layer in one
// launch.
// arguments: [linear 0 = projection (WITH_O),] then the first feed-forward
// linear (N = hidden width) and the second (N = output width, Y = output);
// K = input width, KC / nchunk = the second plan's chunking; skip / gamma /
// beta belong to the first LayerNorm that runs, gamma2 / beta2 to the second.
// ---------------------------------------------------------------------------
#ifdef TL_FFN_MASKED_FLUSH
#define TL_FFN_FLUSH(acc_, j_, c0_, c1_) tl_flush_acc<NB>(acc_, j_, c0_, c1_)
#else
#define TL_FFN_FLUSH(acc_, j_, c0_, c1_) tl_flush_acc_branch<NB>(acc_, j_, c0_, c1_)
#endif
constexpr int TL_FFN_WAVES = 16;
constexpr int TL_FFN_MAX_PHASES = 16;

// Workgroup-local event counters in LDS: every wave adds one when it has
// finished a step, and a wave that needs everyone's result waits for the
// count.  Unlike s_barrier this lets a wave run ahead with other work and
// wait only when it is a whole step ahead of the slowest wave.
__device__ __forceinline__ void tl_signal(unsigned *ctr, int lane) {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local"); // this wave's LDS writes first
    if (lane == 0)
        __hip_atomic_fetch_add(ctr, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
}
// The wait is bounded (about 4 million polls by default, tens of milliseconds):
// should a wave ever fail to signal, the waiting wave sets the process's
// wait-status word and goes on - the kernel ends with a wrong result instead of
// hanging the GPU, and the next launch of a fused kernel reports ET_ERR_HIP.
// Every launch site checks on the host that the phase count fits the counters
// (tile_launch_ffn).
__device__ __forceinline__ void tl_wait_count(unsigned *ctr, unsigned target, int spin, int *status, int lane) {
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

template <int NB, bool WITH_O>
__global__ void __launch_bounds__(TL_FFN_WAVES * 64) tile_ffn_fused_kernel(const TlArgs a) {
    constexpr int L1 = WITH_O ? 1 : 0, L2 = L1 + 1; // the two feed-forward linears
    extern __shared__ __attribute__((aligned(16))) unsigned char tl_smem[];
    f16 *xs = reinterpret_cast<f16 *>(tl_smem);
    const int rp = (blockIdx.x & 7) * a.per_xcd + (blockIdx.x >> 3);
    if (rp >= a.total)
        return;
    constexpr int NW = TL_FFN_WAVES;
    TlCtx x;
    x.lin = 1;
    x.cg = 0;
    x.m0 = rp * TL_BM;
    x.wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    x.lane = threadIdx.x & 63;
    x.c16 = x.lane & 15;
    x.g4 = x.lane >> 4;
    x.khalf8 = (x.g4 & 1) * 8;
    x.hi = x.lane >> 5;
    x.ldx = a.K + ((a.K & 31) ? 0 : TL_PAD);
    x.bn_wg = 0;
    x.bn0 = x.wave * NB;
    x.ld_r = x.ld_c = 0;
    const int wave = x.wave, lane = x.lane, c16 = x.c16, g4 = x.g4, hi = x.hi;
    const int ldx = x.ldx;
    const int ldh = a.KC + ((a.KC & 31) ? 0 : TL_PAD);
    f16 *const hs = xs + TL_BM * ldx; // two hidden buffers behind the X panel
    const int hbuf = TL_BM * ldh;
    // event counters behind the hidden buffers: [p] first linear of phase p
    // done, [TL_FFN_MAX_PHASES + p] second linear of phase p done
    unsigned *const ctr = reinterpret_cast<unsigned *>(hs + 2 * hbuf);
    const int N1 = a.N[L1], N2 = a.N[L2], nbr1 = N1 >> 4, nbr2 = N2 >> 4;
    const int hbr = a.KC >> 4; // hidden block-rows per phase
    const unsigned lane_w = hi * 256 + c16 * 16 + x.khalf8;

    // the X panel: wave w fetches rows 2w and 2w+1
    {
        const int pcpr = a.K >> 3;
#pragma unroll
        for (int rr = 0; rr < TL_BM / NW; rr++) {
            const int r = wave * (TL_BM / NW) + rr;
            if (x.m0 + r < a.M) {
                const f16 *src = a.X + (size_t)(x.m0 + r) * a.K;
                if (lane < pcpr)
                    load_lds16(src + lane * 8, xs + r * ldx);
                if (64 + lane < pcpr)
                    load_lds16(src + (64 + lane) * 8, xs + r * ldx + 512);
            }
        }
    }
    if (threadIdx.x < 2 * TL_FFN_MAX_PHASES)
        ctr[threadIdx.x] = 0;
    const int *const cptr1 = a.cptr[L1], *const cptr2 = a.cptr[L2];
    const f16 *const data1 = a.data[L1], *const data2 = a.data[L2];
    const int *const poff1 = a.row_offset[L1], *const poff2 = a.row_offset[L2];
    // pair-index boundaries of the wave's block-rows (lane j: start of block-row
    // j, lane NB: end of the last one); block-rows past the phase's range or the
    // matrix are empty
    // (read with scalar loads: they do not queue behind the weight pairs in
    // flight, and no wait for them drains those)
    typedef const __attribute__((address_space(4))) int *ScalarInts;
    auto bvec_of = [&](ScalarInts base, int i0, int lim) {
        int v = 0;
#pragma unroll
        for (int k = NB; k >= 0; k--) {
            const int s = base[min(i0 + k, lim)] >> 1;
            v = (lane == k) ? s : v;
        }
        return v;
    };
#define TL_FFN_BVEC1(p_) bvec_of((ScalarInts)cptr1, (p_) * hbr + wave * NB, min(((p_) + 1) * hbr, nbr1))
#define TL_FFN_BVEC2(p_) bvec_of((ScalarInts)cptr2 + (p_) * nbr2, wave * NB, nbr2)
#define TL_FFN_BIAS1(dst_, p_)                                                                    \
    _Pragma("unroll") for (int k = 0; k < NB; k++)                                                \
        dst_[k] = *reinterpret_cast<const f16x4 *>(                                               \
            a.bias[L1] + min((p_) * hbr + wave * NB + k, nbr1 - 1) * 16 + g4 * 4);
    f32x4 acc[NB][2];
#pragma unroll
    for (int j = 0; j < NB; j++) {
        acc[j][0] = f32x4{0.f, 0.f, 0.f, 0.f};
        acc[j][1] = f32x4{0.f, 0.f, 0.f, 0.f};
    }
    const char *const xlane1 = reinterpret_cast<const char *>(xs + c16 * ldx + x.khalf8);
    const int xrow1 = 16 * ldx * 2, xrow2 = 16 * ldh * 2;

    // One stream of the first linear: hidden columns of phase p_ (bias, GELU,
    // half) into hidden buffer p_ & 1.  w_/o_ hold its first pairs already.
#define TL_FFN_FIRST(p_, bvec_, b1_, w_, o_)                                                      \
    {                                                                                             \
        f16 *const hlane = hs + ((p_) & 1) * hbuf + c16 * ldh + wave * NB * 16 + g4 * 4;          \
        const int q0_ = __builtin_amdgcn_readfirstlane(bvec_), qe_ = __builtin_amdgcn_readlane(bvec_, NB); \
        tl_stream<NB>(xlane1, xrow1, data1, poff1, lane_w, hi, q0_, qe_, max(qe_ - 1, q0_), bvec_, w_, o_, \
                      [&](int j, f32x4 c0, f32x4 c1) {                                            \
                          f16x4 bj = f16x4{0, 0, 0, 0};                                           \
                          _Pragma("unroll") for (int k = 0; k < NB; k++)                          \
                              bj += b1_[k] * ((j == k) ? (f16)1 : (f16)0);                        \
                          tl_stage_tile<true>(hlane + j * 16, ldh, c0, c1, bj);                   \
                      });                                                              \
        /* block-rows of this phase without any tile: bias only */                                \
        const int lim1 = min(((p_) + 1) * hbr, nbr1);                                             \
        _Pragma("unroll") for (int k = 0; k < NB; k++)                                            \
            if ((p_) * hbr + wave * NB + k < lim1 &&                                              \
                __builtin_amdgcn_readlane(bvec_, k) == __builtin_amdgcn_readlane(bvec_, k + 1))   \
                tl_stage_tile<true>(hlane + k * 16, ldh, f32x4{0.f, 0.f, 0.f, 0.f},               \
                                    f32x4{0.f, 0.f, 0.f, 0.f}, b1_[k]);                           \
        tl_signal(ctr + (p_), lane);                                                              \
    }
#define TL_FFN_PRELOAD(data_, poff_, bvec_, w_, o_)                                               \
    {                                                                                             \
        const int q0_ = __builtin_amdgcn_readfirstlane(bvec_), qe_ = __builtin_amdgcn_readlane(bvec_, NB); \
        tl_preload(data_, poff_, lane_w, hi, q0_, max(qe_ - 1, q0_), w_, o_);                     \
    }

    // Stream order (F = first linear, S = second).  Half of the waves run
    // F(0) F(1) S(0) F(2) S(1) ... S(last), the first linear one phase ahead;
    // the other half F(0) S(0) F(1) S(1) ...  Both orders respect "S(p) after
    // every wave's F(p)" and "F(p+2) after every wave's S(p)" (the hidden buffer
    // it overwrites), what a wave waits for was usually finished a stream ago,
    // and at most times the two halves of a SIMD's waves are in different kinds
    // of stream: F streams load the vector ALU (GELU), S streams hardly do.
    // Register set A serves F(0) and every S, set B every later F.
    f16x8 wA[TL_DEPTH], wB[TL_DEPTH];
    int oA[TL_DEPTH], oB[TL_DEPTH];
    int bvecF = TL_FFN_BVEC1(0);
    f16x4 b1[NB];
    TL_FFN_BIAS1(b1, 0)
    int bvecFn = TL_FFN_BVEC1(min(1, a.nchunk - 1));
    f16x4 b1n[NB];
    TL_FFN_BIAS1(b1n, min(1, a.nchunk - 1))
    int bvecS = TL_FFN_BVEC2(0);
    __builtin_amdgcn_s_waitcnt(0x0F70); // vmcnt(0): this wave's part of the panel has landed
    if constexpr (WITH_O) {
        // Linear 0 (the attention output projection) with its skip connection
        // and LayerNorm comes first: the panel just fetched holds the attention
        // output, and the normalised rows (rounded to half, as the reference
        // stores them) replace it in LDS as the feed-forward block's input and
        // as the skip operand of the final LayerNorm.
        const int NO = a.N[0], nbrO = NO >> 4; // == K
        const int bvecO = bvec_of((ScalarInts)a.cptr[0], wave * NB, nbrO);
        f16x4 bO[NB];
#pragma unroll
        for (int j = 0; j < NB; j++) {
            bO[j] = f16x4{0, 0, 0, 0};
            if (x.bn0 + j < nbrO)
                bO[j] = *reinterpret_cast<const f16x4 *>(a.bias[0] + (x.bn0 + j) * 16 + g4 * 4);
        }
        TL_FFN_PRELOAD(a.data[0], a.row_offset[0], bvecO, wB, oB)
        tl_barrier_lds(); // the whole panel has landed; the counters are zero
        {
            const int q0_ = __builtin_amdgcn_readfirstlane(bvecO), qe_ = __builtin_amdgcn_readlane(bvecO, NB);
            tl_stream<NB>(xlane1, xrow1, a.data[0], a.row_offset[0], lane_w, hi, q0_, qe_, max(qe_ - 1, q0_),
                          bvecO, wB, oB,
                          [&](int j, f32x4 c0, f32x4 c1) { TL_FFN_FLUSH(acc, j, c0, c1); });
        }
        TL_FFN_PRELOAD(data1, poff1, bvecF, wA, oA)
        TlLnOperands<NB, NW, NW> lnop1; // (requested here: their latency runs under the wait for the other waves)
        tl_ln_fetch_at(lnop1, a.M, wave, lane, x.m0, NO, a.skip + (long)x.m0 * NO, (long)NO, a.gamma, a.beta);
        // staging tiles in the hidden buffers, which nobody uses yet
        tl_epilogue_wave<NB, false, false>(a, x, hs + wave * tl_wave_stage_halves<NB>(), nullptr, NO, nbrO, acc,
                                           bO);
#pragma unroll
        for (int j = 0; j < NB; j++) {
            acc[j][0] = f32x4{0.f, 0.f, 0.f, 0.f};
            acc[j][1] = f32x4{0.f, 0.f, 0.f, 0.f};
        }
        tl_barrier_lds(); // every wave's part is staged, and everyone has left the attention panel
        tl_ln_rows_at(lnop1, a.M, hs, wave, lane, x.m0, NO, xs, (long)ldx);
    } else {
        TL_FFN_PRELOAD(data1, poff1, bvecF, wA, oA)
    }
    tl_barrier_lds(); // the feed-forward input panel is complete (and the counters are zero)
    if (a.nchunk > 1)
        TL_FFN_PRELOAD(data1, poff1, bvecFn, wB, oB)
    TL_FFN_FIRST(0, bvecF, b1, wA, oA)

    const int behind = (wave >> 2) & 1; // (a SIMD's waves are w, w+4, w+8, w+12)
    for (int p = 0; p < a.nchunk; p++) {
        const int bvecSn = TL_FFN_BVEC2(min(p + 1, a.nchunk - 1));
        TL_FFN_PRELOAD(data2, poff2, bvecS, wA, oA) // S(p), a stream ahead (unless no F runs in between)
        const int fq = p + 1 - behind; // the first-linear phase this wave runs before S(p)
        if (fq >= 1 && fq < a.nchunk) {
            const int bvecF2 = TL_FFN_BVEC1(min(fq + 1, a.nchunk - 1)); // (scalar loads, used after the stream)
            if (fq >= 2) // F(fq) overwrites the buffer that S(fq-2) read
                tl_wait_count(ctr + TL_FFN_MAX_PHASES + fq - 2, NW, a.spin, a.status, lane);
            TL_FFN_FIRST(fq, bvecFn, b1n, wB, oB)
            bvecFn = bvecF2;
            if (fq + 1 < a.nchunk) { // F(fq+1), a stream (or two) ahead
                TL_FFN_PRELOAD(data1, poff1, bvecFn, wB, oB)
                TL_FFN_BIAS1(b1n, fq + 1)
            }
        }
        tl_wait_count(ctr + p, NW, a.spin, a.status, lane); // hidden buffer p & 1 is complete
        {
            const char *const xlane2 =
                reinterpret_cast<const char *>(hs + (p & 1) * hbuf + c16 * ldh + x.khalf8);
            const int q0_ = __builtin_amdgcn_readfirstlane(bvecS), qe_ = __builtin_amdgcn_readlane(bvecS, NB);
            tl_stream<NB>(xlane2, xrow2, data2, poff2, lane_w, hi, q0_, qe_, max(qe_ - 1, q0_), bvecS, wA, oA,
                          [&](int j, f32x4 c0, f32x4 c1) { TL_FFN_FLUSH(acc, j, c0, c1); });
            tl_signal(ctr + TL_FFN_MAX_PHASES + p, lane);
        }
        bvecS = bvecSn;
    }
#undef TL_FFN_BVEC1
#undef TL_FFN_BVEC2
#undef TL_FFN_BIAS1
#undef TL_FFN_FIRST
#undef TL_FFN_PRELOAD

    // output rows -> staging tiles over the (now unused) panel and hidden
    // buffers, then skip connection + LayerNorm over whole rows
    TlLnOperands<NB, NW, NW> lnop;
    if constexpr (WITH_O) // the skip operand is the panel in LDS
        tl_ln_fetch_at(lnop, a.M, wave, lane, x.m0, N2, xs, (long)ldx, a.gamma2, a.beta2);
    else
        tl_ln_fetch(lnop, a, wave, lane, x.m0, N2);
    f16x4 b2[NB];
#pragma unroll
    for (int j = 0; j < NB; j++) {
        b2[j] = f16x4{0, 0, 0, 0};
        if (x.bn0 + j < nbr2)
            b2[j] = *reinterpret_cast<const f16x4 *>(a.bias[L2] + (x.bn0 + j) * 16 + g4 * 4);
    }
    tl_barrier_lds(); // every wave has left the hidden buffers
    f16 *const stage0 = WITH_O ? hs : xs;
    tl_epilogue_wave<NB, false, false>(a, x, stage0 + wave * tl_wave_stage_halves<NB>(), a.Y[L2], N2, nbr2,
                                       acc, b2);
    __syncthreads(); // every wave's part of the rows is staged
    tl_ln_rows(lnop, a, stage0, wave, lane, x.m0, a.Y[L2], N2);
}

// ---------------------------------------------------------------------------
// Generic kernel: the caller's own tile_mat (TL_RAW / TL_FILTER) or a dense
// row-major weight (TL_DENSE).  Same mapping, plain per-block-row loops with
// per-lane predicates.
// ---------------------------------------------------------------------------
template <int NB, bool GELU, int MODE>
__global__ void __launch_bounds__(TL_THREADS) tile_linear_generic_kernel(const TlArgs a) {
    extern __shared__ __attribute__((aligned(16))) unsigned char tl_smem[];
    f16 *xs = reinterpret_cast<f16 *>(tl_smem);
    TlCtx x;
    if (!tl_context(a, NB, x))
        return;
    const int lin = x.lin;
    f16 *const Yp = TL_SEL(Y);
    const int *const cptr = TL_SEL(cptr);
    const int *const roff = TL_SEL(row_offset);
    const f16 *const data = TL_SEL(data);
    const f16 *const bias = TL_SEL(bias);
    const int N = TL_SEL(N);
    const int nbr = N >> 4;
    const int hi = x.hi;

    f32x4 acc[NB][2];
    f16x4 b4[NB];
#pragma unroll
    for (int j = 0; j < NB; j++) {
        acc[j][0] = f32x4{0.f, 0.f, 0.f, 0.f};
        acc[j][1] = f32x4{0.f, 0.f, 0.f, 0.f};
        b4[j] = f16x4{0, 0, 0, 0};
        if (x.bn0 + j < nbr)
            b4[j] = *reinterpret_cast<const f16x4 *>(bias + (x.bn0 + j) * 16 + x.g4 * 4);
    }
    const f16 *xlane = xs + x.c16 * x.ldx + x.khalf8;
    const int xrow16 = 16 * x.ldx;
    const bool rowok = (x.m0 + x.ld_r) < a.M;
    const u32x4 *xsrc = reinterpret_cast<const u32x4 *>(a.X + (size_t)(x.m0 + x.ld_r) * a.K);
    u32x4 *xdst = reinterpret_cast<u32x4 *>(xs + x.ld_r * x.ldx);
    const f16x8 zero8 = f16x8{0, 0, 0, 0, 0, 0, 0, 0};

    for (int c = 0; c < a.nchunk; c++) {
        const int k0 = c * a.KC;
        const int kc = min(a.KC, a.K - k0);
        if (c > 0)
            __syncthreads();
        {
            const int cpr = kc >> 3;
            u32x4 pv[8];
#pragma unroll
            for (int u = 0; u < 8; u++) {
                const int cc = x.ld_c + 16 * u;
                pv[u] = u32x4{0u, 0u, 0u, 0u};
                if (rowok && cc < cpr)
                    pv[u] = xsrc[(k0 >> 3) + cc];
            }
#pragma unroll
            for (int u = 0; u < 8; u++) {
                const int cc = x.ld_c + 16 * u;
                if (cc < cpr)
                    xdst[cc] = pv[u];
            }
        }
        __syncthreads();
#pragma unroll
        for (int j = 0; j < NB; j++) {
            const int bn = x.bn0 + j;
            if (bn >= nbr)
                continue;
            if (MODE == TL_DENSE) {
                const f16 *wrow = data + (size_t)(bn * 16 + x.c16) * a.K + k0 + x.khalf8;
                const int nt = kc >> 4;
                for (int i = 0; i < nt; i += 2) {
                    const bool ok = i + hi < nt;
                    const int off = (ok ? i + hi : i) * 16;
                    f16x8 w = zero8;
                    if (ok)
                        w = *reinterpret_cast<const f16x8 *>(wrow + off);
                    const f16x8 x0 = *reinterpret_cast<const f16x8 *>(xlane + off);
                    const f16x8 x1 = *reinterpret_cast<const f16x8 *>(xlane + off + xrow16);
                    acc[j][0] = mfma16x16x32(w, x0, acc[j][0]);
                    acc[j][1] = mfma16x16x32(w, x1, acc[j][1]);
                }
            } else {
                const int fs = cptr[bn];
                const int fe = cptr[bn + 1];
                const f16 *wlane = data + x.c16 * 16 + x.khalf8;
                for (int i = fs; i < fe; i += 2) {
                    const int ti = min(i + hi, fe - 1);
                    const int off = roff[ti] - k0;
                    const bool ok = (i + hi < fe) && off >= 0 && off < kc;
                    if (MODE == TL_FILTER && __builtin_amdgcn_ballot_w64(ok) == 0)
                        continue;
                    f16x8 w = zero8, x0 = zero8, x1 = zero8;
                    if (ok) {
                        w = *reinterpret_cast<const f16x8 *>(wlane + (size_t)ti * 256);
                        x0 = *reinterpret_cast<const f16x8 *>(xlane + off);
                        x1 = *reinterpret_cast<const f16x8 *>(xlane + off + xrow16);
                    }
                    acc[j][0] = mfma16x16x32(w, x0, acc[j][0]);
                    acc[j][1] = mfma16x16x32(w, x1, acc[j][1]);
                }
            }
        }
    }
    tl_epilogue<NB, GELU>(a, x, xs, Yp, N, nbr, acc, b4);
}

// ---------------------------------------------------------------------------
// Few rows (a single short sequence).  Such a launch is a chain of memory
// latencies, not a stream: the kernels above give a wave one (32-row panel,
// block-row) unit whose tile pairs it requests TL_DEPTH at a time, one round
// trip to memory per TL_DEPTH pairs and one more per K chunk of the panel
// (BERT-base FFN2 on 128 rows: 20 us).  Here a workgroup of 16 waves takes a
// 16-row panel with ALL of its K columns in LDS (16 x 3072 halves = 97 KB) and
// 16/SPLIT block-rows; the pairs of a block-row are split over SPLIT waves (by
// K chunk and by pair ranges inside a chunk - with the whole row of X in LDS
// any partition works), and a wave requests up to TL_SK_D pairs at once, which
// covers its whole share in the dense BERT-base cases: the panel and all of W
// arrive in one round trip.  The SPLIT partial sums meet in LDS and are added
// in a fixed order, so the result does not depend on timing.
// ---------------------------------------------------------------------------
constexpr int TL_SK_WAVES = 16;
constexpr int TL_SK_BM = 16; // rows per panel
constexpr int TL_SK_D = 12;  // pairs in flight per wave

template <bool GELU, int SPLIT>
__global__ void __launch_bounds__(TL_SK_WAVES * 64) tile_linear_splitk_kernel(const TlArgs a) {
    constexpr int BR = TL_SK_WAVES / SPLIT; // block-rows per workgroup
    extern __shared__ __attribute__((aligned(16))) unsigned char tl_smem[];
    f16 *xs = reinterpret_cast<f16 *>(tl_smem);
    const int vid = (blockIdx.x & 7) * a.per_xcd + (blockIdx.x >> 3); // a panel's workgroups on one XCD
    if (vid >= a.total)
        return;
    const int per_rp = a.ncg * a.nlin;
    const int rp = vid / per_rp, rest = vid - rp * per_rp;
    const int lin = rest / a.ncg, grp = rest - lin * a.ncg;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int lane = threadIdx.x & 63;
    const int c16 = lane & 15, g4 = lane >> 4, khalf8 = (g4 & 1) * 8, hi = lane >> 5;
    const int ldx = a.K + ((a.K & 31) ? 0 : TL_PAD); // row stride == 32 (mod 64) bytes
    const int m0 = rp * TL_SK_BM;
    f16 *const Yp = TL_SEL(Y);
    const int *const cptr = TL_SEL(cptr);
    const int *const poff = TL_SEL(row_offset);
    const f16 *const data = TL_SEL(data);
    const f16 *const bias = TL_SEL(bias);
    const int N = TL_SEL(N);
    const int nbr = N >> 4;

    // the panel: wave w fetches row w (DMA, 16 bytes per lane and instruction)
    if (m0 + wave < a.M) {
        const f16 *src = a.X + (size_t)(m0 + wave) * a.K;
        f16 *dstrow = xs + wave * ldx;
        const int pcpr = a.K >> 3;
        for (int c0 = 0; c0 < pcpr; c0 += 64)
            if (c0 + lane < pcpr)
                load_lds16(src + (c0 + lane) * 8, dstrow + c0 * 8);
    }
    const int j = wave % BR, sp = wave / BR; // block-row of the group, split
    const int bn = grp * BR + j;
    // this wave's pairs: chunk ck of the plan, part `sub` of `spc` of the block-row's segment there
    const int spc = SPLIT / a.nchunk; // (nchunk divides SPLIT)
    const int ck = sp / spc, sub = sp - ck * spc;
    int qa = 0, qb = 0;
    f16x4 b4 = f16x4{0, 0, 0, 0};
    if (bn < nbr) {
        const int p0 = cptr[ck * nbr + bn] >> 1, p1 = cptr[ck * nbr + bn + 1] >> 1;
        const int len = p1 - p0;
        qa = p0 + len * sub / spc;
        qb = p0 + len * (sub + 1) / spc;
        b4 = *reinterpret_cast<const f16x4 *>(bias + bn * 16 + g4 * 4);
    }
    qa = __builtin_amdgcn_readfirstlane(qa);
    qb = __builtin_amdgcn_readfirstlane(qb);
    // Pairs at or beyond qb are replaced by the plan's spare pair (all-zero W,
    // behind the last real pair): every slot loads and multiplies, nothing
    // inside a round is conditional.
    const int qsp = __builtin_amdgcn_readfirstlane(cptr[a.nchunk * nbr] >> 1);
    const unsigned lane_w = hi * 256 + c16 * 16 + khalf8;
    f16x8 w[TL_SK_D];
    int o[TL_SK_D];
    // (requested while the panel is still arriving: loads return in order, the
    // wait below covers both)
#pragma unroll
    for (int i = 0; i < TL_SK_D; i++)
        tl_load_pair(data, poff, qa + i < qb ? qa + i : qsp, lane_w, hi, w[i], o[i]);
    __builtin_amdgcn_s_waitcnt(0x0F70); // vmcnt(0)
    __syncthreads();

    // chunk-local column offsets of a multi-chunk plan -> offsets in the full row
    const char *xlane = reinterpret_cast<const char *>(xs + c16 * ldx + khalf8) + (size_t)ck * a.KC * 2;
    f32x4 acc0 = f32x4{0.f, 0.f, 0.f, 0.f}, acc1 = f32x4{0.f, 0.f, 0.f, 0.f};
    for (int q = qa;;) {
#pragma unroll
        for (int i = 0; i < TL_SK_D; i += 2) { // two accumulators: two independent MFMA chains
            acc0 = mfma16x16x32(w[i], *reinterpret_cast<const f16x8 *>(xlane + o[i]), acc0);
            acc1 = mfma16x16x32(w[i + 1], *reinterpret_cast<const f16x8 *>(xlane + o[i + 1]), acc1);
        }
        q += TL_SK_D;
        if (q >= qb)
            break;
#pragma unroll
        for (int i = 0; i < TL_SK_D; i++)
            tl_load_pair(data, poff, q + i < qb ? q + i : qsp, lane_w, hi, w[i], o[i]);
    }
    const f32x4 acc = acc0 + acc1;

    // partial sums -> LDS (behind the panel), summed by the first wave of each block-row
    f32x4 *red = reinterpret_cast<f32x4 *>(xs + TL_SK_BM * ldx);
    red[(sp * BR + j) * 64 + lane] = acc;
    __syncthreads();
    if (sp == 0 && bn < nbr) {
        f32x4 t = red[j * 64 + lane];
#pragma unroll
        for (int k = 1; k < SPLIT; k++)
            t += red[(k * BR + j) * 64 + lane];
        f16x4 ov = __builtin_convertvector(t + __builtin_convertvector(b4, f32x4), f16x4);
        if (GELU)
            ov = gelu4(ov);
        if (m0 + c16 < a.M)
            *reinterpret_cast<f16x4 *>(Yp + (size_t)(m0 + c16) * N + bn * 16 + g4 * 4) = ov;
    }
}

#undef TL_SEL

// ---------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------
// Dynamic LDS above the 64 KB default has to be allowed per kernel.  The call
// goes to the driver, so it is made only when a kernel needs more than it was
// last given (one record per kernel instance and device).
template <auto KERN>
static hipError_t allow_lds(size_t lds) {
    static size_t allowed[16] = {};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 16)
        return hipFuncSetAttribute(reinterpret_cast<const void *>(KERN),
                                   hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (lds <= allowed[dev])
        return hipSuccess;
    const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(KERN),
                                             hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e == hipSuccess)
        allowed[dev] = lds;
    return e;
}

template <int NB, bool GELU, int MODE>
static void launch_inst(const TlArgs &a, size_t lds, hipStream_t st) {
    const dim3 grid(a.per_xcd * 8), block(TL_THREADS);
    if constexpr (MODE == TL_PLAN) {
        // (block-rows per wave beyond 3 never paid off for the plan kernels)
        constexpr int PNB = NB > 3 ? 3 : NB;
        if (a.nchunk == 1)
            hipLaunchKernelGGL((tile_linear_resident_kernel<PNB, GELU, TL_WAVES, false>), grid, block, lds, st, a);
        else
            hipLaunchKernelGGL((tile_linear_plan_kernel<PNB, GELU, TL_WAVES, false>), grid, block, lds, st, a);
    } else {
        hipLaunchKernelGGL((tile_linear_generic_kernel<NB, GELU, MODE>), grid, block, lds, st, a);
    }
}

template <bool GELU, int MODE>
static void launch_nb(int nb, const TlArgs &a, size_t lds, hipStream_t st) {
    switch (nb) {
    case 1: launch_inst<1, GELU, MODE>(a, lds, st); break;
    case 2: launch_inst<2, GELU, MODE>(a, lds, st); break;
    case 3: launch_inst<3, GELU, MODE>(a, lds, st); break;
    case 4: launch_inst<4, GELU, MODE>(a, lds, st); break;
    default: launch_inst<6, GELU, MODE>(a, lds, st); break;
    }
}

// Fused linear + skip + LayerNorm: one workgroup of 16 waves covers whole rows.
constexpr int TL_LN_WAVES = 16;

template <int NB>
static int launch_ln_inst(const TlArgs &a, size_t lds, hipStream_t st) {
    const dim3 grid(a.per_xcd * 8), block(TL_LN_WAVES * 64);
    if (a.nchunk == 1) {
        constexpr auto k = &tile_linear_resident_kernel<NB, false, TL_LN_WAVES, true>;
        ET_HIP(allow_lds<k>(lds));
        hipLaunchKernelGGL(k, grid, block, lds, st, a);
    } else {
        constexpr auto k = &tile_linear_plan_kernel<NB, false, TL_LN_WAVES, true>;
        ET_HIP(allow_lds<k>(lds));
        hipLaunchKernelGGL(k, grid, block, lds, st, a);
    }
    return launch_status("tile_linear+LayerNorm launch");
}

// block-rows per wave of the fused kernel for a matrix of nbr block-rows; 0 if
// the rows do not fit one workgroup (then the caller runs the two kernels)
static int ln_block_rows(int nbr) {
    const int need = (nbr + TL_LN_WAVES - 1) / TL_LN_WAVES;
    return need <= 3 ? need : need == 4 ? 4 : need <= 6 ? 6 : 0;
}

template <int NB>
static int launch_chunked_ln_inst(const TlArgs &a, size_t lds, hipStream_t st) {
    constexpr auto k = &tile_linear_chunked_ln_kernel<NB>;
    ET_HIP(allow_lds<k>(lds));
    hipLaunchKernelGGL(k, dim3(a.per_xcd * 8), dim3(TL_CTHREADS), lds, st, a);
    return launch_status("tile_linear+LayerNorm (chunked) launch");
}

static int g_tile_ln_chunked = 1;
static int g_tile_fuse_ffn = 2; // et_tuning_set("tile_fuse_ffn"): 1 feed-forward block, 2 whole layer tail

// LDS bytes of the fused feed-forward kernel: X panel, two hidden buffers (the
// output staging tiles reuse their storage)
static size_t ffn_lds_bytes(int K1, int KC2) {
    const size_t ldx = K1 + ((K1 & 31) ? 0 : TL_PAD), ldh = KC2 + ((KC2 & 31) ? 0 : TL_PAD);
    size_t panels = (size_t)TL_BM * (ldx + 2 * ldh) * sizeof(f16) + 2 * TL_FFN_MAX_PHASES * sizeof(unsigned);
    const size_t staging = (size_t)TL_FFN_WAVES * TL_BM * (16 * 3 + 8) * sizeof(f16);
    return std::max(panels, staging);
}

// pO: the attention output projection in front of the block (the whole layer
// tail in one launch), or null
static int tile_launch_ffn(const TlProblem *pO, const TlProblem &p1, const TlProblem &p2, const f16 *X,
                           int M, int K1, int KC2, int nchunk2, const f16 *skip, const f16 *gamma,
                           const f16 *beta, const f16 *gamma2, const f16 *beta2, hipStream_t st) {
    // the kernel's LDS event counters cover TL_FFN_MAX_PHASES phases: every launch passes through here
    ET_REQUIRE(nchunk2 >= 1 && nchunk2 <= TL_FFN_MAX_PHASES, ET_ERR_UNSUPPORTED,
               "fused feed-forward: %d phases, the kernel covers %d", nchunk2, TL_FFN_MAX_PHASES);
    // a wave of an earlier launch that gave up an LDS wait left a wrong result behind: say so once
    int *const status = wait_status_device();
    ET_REQUIRE(status, ET_ERR_HIP, "fused feed-forward: no wait-status word");
    {
        const int rc = check_wait_status("fused feed-forward");
        if (rc != ET_OK)
            return rc;
    }
    TlArgs a;
    memset(&a, 0, sizeof(a));
    a.status = status;
    a.spin = tail_spin();
    const TlProblem *ps[3] = {pO ? pO : &p1, pO ? &p1 : &p2, &p2};
    for (int i = 0; i < TL_MAX_LIN; i++) {
        const TlProblem &p = *ps[std::min(i, 2)];
        a.Y[i] = p.Y;
        a.cptr[i] = p.cptr;
        a.row_offset[i] = p.row_offset;
        a.data[i] = p.data;
        a.bias[i] = p.bias;
        a.N[i] = p.N;
    }
    a.X = X;
    a.nlin = pO ? 3 : 2;
    a.gamma2 = gamma2;
    a.beta2 = beta2;
    a.M = M;
    a.K = K1;
    a.KC = KC2;
    a.nchunk = nchunk2;
    a.ncg = 1;
    a.total = (M + TL_BM - 1) / TL_BM;
    a.ipw = 1;
    a.per_xcd = (a.total + 7) / 8;
    a.skip = skip;
    a.gamma = gamma;
    a.beta = beta;
    const size_t lds = ffn_lds_bytes(K1, KC2);
    if (pO) {
        constexpr auto k = &tile_ffn_fused_kernel<3, true>;
        ET_HIP(allow_lds<k>(lds));
        hipLaunchKernelGGL(k, dim3(a.per_xcd * 8), dim3(TL_FFN_WAVES * 64), lds, st, a);
    } else {
        constexpr auto k = &tile_ffn_fused_kernel<3, false>;
        ET_HIP(allow_lds<k>(lds));
        hipLaunchKernelGGL(k, dim3(a.per_xcd * 8), dim3(TL_FFN_WAVES * 64), lds, st, a);
    }
    return launch_status("fused feed-forward launch");
}

static int tile_launch_ln(const TlProblem &p, const f16 *X, int M, int K, int KC, int nchunk,
                          const f16 *skip, const f16 *gamma, const f16 *beta, hipStream_t st) {
    TlArgs a;
    memset(&a, 0, sizeof(a));
    for (int i = 0; i < TL_MAX_LIN; i++) {
        a.Y[i] = p.Y;
        a.cptr[i] = p.cptr;
        a.row_offset[i] = p.row_offset;
        a.data[i] = p.data;
        a.bias[i] = p.bias;
        a.N[i] = p.N;
    }
    a.X = X;
    a.nlin = 1;
    a.M = M;
    a.K = K;
    a.KC = KC;
    a.nchunk = nchunk;
    a.ncg = 1;
    a.total = (M + TL_BM - 1) / TL_BM;
    a.ipw = 1;
    a.per_xcd = (a.total + 7) / 8;
    a.skip = skip;
    a.gamma = gamma;
    a.beta = beta;
    const size_t lds_x = (size_t)TL_BM * (KC + ((KC & 31) ? 0 : TL_PAD)) * sizeof(f16);
    // K in chunks and rows narrow enough for twelve waves of <= 4 block-rows:
    // the double-buffered kernel with a fetching wave
    const int cnb = (p.nbr + TL_CWAVES - 1) / TL_CWAVES;
    if (nchunk > 1 && cnb <= 4 && g_tile_ln_chunked) {
        const size_t lds = 2 * lds_x + (size_t)TL_CWAVES * TL_BM * (16 * cnb + 8) * sizeof(f16);
        switch (cnb) {
        case 1: return launch_chunked_ln_inst<1>(a, lds, st);
        case 2: return launch_chunked_ln_inst<2>(a, lds, st);
        case 3: return launch_chunked_ln_inst<3>(a, lds, st);
        default: return launch_chunked_ln_inst<4>(a, lds, st);
        }
    }
    const int nb = ln_block_rows(p.nbr);
    const size_t lds = lds_x + (size_t)TL_LN_WAVES * TL_BM * (16 * nb + 8) * sizeof(f16);
    switch (nb) {
    case 1: return launch_ln_inst<1>(a, lds, st);
    case 2: return launch_ln_inst<2>(a, lds, st);
    case 3: return launch_ln_inst<3>(a, lds, st);
    case 4: return launch_ln_inst<4>(a, lds, st);
    default: return launch_ln_inst<6>(a, lds, st);
    }
}

// Tuning knobs (et_tuning_set): 0 = automatic.
static int g_tile_nb = 0;
static int g_tile_min_wgs = 512;
static int g_tile_ipw = 0;
static int g_tile_fuse_ln = 1;
static int g_tile_ln_min_panels = 96;
// the layer tail in one launch: from fewer panels than the linear + LayerNorm kernels (measured on
// BERT-base at 80 %: one launch 42 us for any count below one per CU, step by step 37 / 43 / 54 us
// at 52 / 80 / 95 panels)
static int g_tile_tail_min_panels = 72;

// Block-rows per wave.  Measured on the BERT-base shapes (rows 4096..8192):
// three block-rows per wave is the best trade between panel re-reads (fewer
// with larger NB) and register pressure / workgroup count (better with
// smaller NB); small problems fall back to smaller NB to get enough
// workgroups for 256 CUs.
static int choose_nb(int nrp, int nbr_max, int nlin) {
    const int forced = g_tile_nb;
    if (forced == 1 || forced == 2 || forced == 3 || forced == 4 || forced == 6)
        return forced;
    const int cand[3] = {3, 2, 1};
    for (int i = 0; i < 3; i++) {
        const int nb = cand[i];
        const int ncg = (nbr_max + TL_WAVES * nb - 1) / (TL_WAVES * nb);
        if ((long)nrp * ncg * nlin >= g_tile_min_wgs)
            return nb;
    }
    return 1;
}

constexpr int TL_BM64 = 2 * TL_BM;
static int g_tile_bm64 = 1; // et_tuning_set("tile_bm64")
// rows from which the row-pruned linear runs the register-blocked GEMM (et_tuning_set("row_gemm_min_rows");
// below, 128 x 128 blocks leave most CUs without work and the tile kernels win)
static int g_row_gemm_min_rows = 1024;

static int g_tile_splitk_k1 = 0;
static int g_tile_splitk_rows = -1; // et_tuning_set("tile_splitk_rows"): row count up to which the few-rows kernel runs, -1 automatic

template <int NB, bool GELU, int NW = TL_WAVES>
static int launch_resident64(const TlArgs &a, size_t lds, hipStream_t st) {
    constexpr auto k = &tile_linear_resident_kernel<NB, GELU, NW, false, TL_BM64>;
    ET_HIP(allow_lds<k>(lds));
    hipLaunchKernelGGL(k, dim3(a.per_xcd * 8), dim3(NW * 64), lds, st, a);
    return launch_status("tile_linear (64-row panels) launch");
}

static int tile_launch(const TlProblem *probs, int nlin, const f16 *X, int M, int K,
                       int KC, int nchunk, bool gelu, int mode, hipStream_t st) {
    TlArgs a;
    memset(&a, 0, sizeof(a));
    int nbr_max = 0;
    for (int i = 0; i < TL_MAX_LIN; i++) {
        const TlProblem &p = probs[i < nlin ? i : 0];
        a.Y[i] = p.Y;
        a.cptr[i] = p.cptr;
        a.row_offset[i] = p.row_offset;
        a.data[i] = p.data;
        a.bias[i] = p.bias;
        a.N[i] = p.N;
        if (i < nlin)
            nbr_max = std::max(nbr_max, p.nbr);
    }
    a.X = X;
    a.nlin = nlin;
    a.M = M;
    a.K = K;
    a.KC = KC;
    a.nchunk = nchunk;
    // Few rows and K in several chunks: up to 128 rows, up to 256 where at
    // least three quarters of the tiles survive (each 16-row panel streams W
    // once more, which a long dense stream repays for longer than a short one).
    // With K in one chunk the kernels below are as fast.
    int sk_rows = g_tile_splitk_rows;
    if (sk_rows < 0) {
        const long all_tiles = (long)nbr_max * (K / 16);
        sk_rows = nlin == 1 && 4L * probs[0].ntile >= 3 * all_tiles ? 256 : 128;
    }
    if (mode == TL_PLAN && M <= sk_rows && (nchunk == 2 || nchunk == 4 || nchunk == 8 || g_tile_splitk_k1) &&
        (nchunk == 1 || nchunk == 2 || nchunk == 4 || nchunk == 8) && g_tile_nb == 0) {
        // few rows: 16-row panels with the whole of K in LDS, a block-row's pairs split over 4 or 8 waves
        const int split = nchunk == 1 ? 4 : 8;
        const int br = TL_SK_WAVES / split;
        const size_t lds_sk = (size_t)TL_SK_BM * (K + ((K & 31) ? 0 : TL_PAD)) * sizeof(f16) +
                              (size_t)TL_SK_WAVES * 64 * sizeof(f32x4);
        if (lds_sk <= 160 * 1024) {
            a.ncg = (nbr_max + br - 1) / br;
            a.total = ((M + TL_SK_BM - 1) / TL_SK_BM) * a.ncg * nlin;
            a.ipw = 1;
            a.per_xcd = (a.total + 7) / 8;
            const dim3 grid(a.per_xcd * 8), block(TL_SK_WAVES * 64);
#define TL_SK_LAUNCH(GELU_, SPLIT_)                                                               \
    {                                                                                             \
        constexpr auto k = &tile_linear_splitk_kernel<GELU_, SPLIT_>;                                        \
        ET_HIP(allow_lds<k>(lds_sk));     \
        hipLaunchKernelGGL(k, grid, block, lds_sk, st, a);                                        \
    }
            if (split == 4) {
                if (gelu) TL_SK_LAUNCH(true, 4) else TL_SK_LAUNCH(false, 4)
            } else {
                if (gelu) TL_SK_LAUNCH(true, 8) else TL_SK_LAUNCH(false, 8)
            }
#undef TL_SK_LAUNCH
            return launch_status("tile_linear (few rows) launch");
        }
    }
    if (mode == TL_PLAN && nchunk == 1 && g_tile_bm64 && g_tile_nb == 0) {
        // 64-row panels, one workgroup per CU: twice the rows per kilobyte of W
        // streamed.  Needs the panel and one 64-row staging tile per wave in LDS
        // and at least two items per CU.  Twelve waves of two block-rows (where
        // the LDS holds their staging tiles: K <= 784), or eight waves of three
        // or of two, and d consecutive items of a panel per workgroup: the
        // combination with the least estimated time (a round of workgroups costs
        // the panel load, 2/3 of a 24-block-row item, plus its items).  Twelve
        // waves come first and win ties: the same items as eight waves of three,
        // with three waves per SIMD instead of two to cover the stream's waits
        // (Q/K/V of the benchmark: 20 -> 17.5 us).
        const int cus = std::max(et_device_cu_count(), 1);
        const int nrp64 = (M + TL_BM64 - 1) / TL_BM64;
        static const int cand[3][2] = {{12, 2}, {8, 3}, {8, 2}}; // waves, block-rows per wave
        double best = 0.0;
        int best_c = -1, best_d = 1, best_ncg = 1;
        size_t best_lds = 0;
        for (int c = 0; c < 3; c++) {
            const int nw = cand[c][0], nb = cand[c][1];
            if (nw == 12 && g_tile_bm64 == 4)
                continue; // (tuning: eight waves only)
            const size_t lds64 = (size_t)TL_BM64 * (KC + ((KC & 31) ? 0 : TL_PAD)) * sizeof(f16) +
                                 (size_t)nw * TL_BM64 * (16 * nb + 8) * sizeof(f16);
            const int ncg64 = (nbr_max + nw * nb - 1) / (nw * nb);
            const long items = (long)nrp64 * ncg64 * nlin;
            if (lds64 > 160 * 1024 || items < (g_tile_bm64 == 2 ? 1L : 2L * cus))
                continue;
            const int per_rp = ncg64 * nlin;
            for (int d = 1; d <= per_rp; d++) {
                if (per_rp % d)
                    continue;
                const long nwg = items / d, rounds = (nwg + cus - 1) / cus;
                const double cost = (double)rounds * (2.0 / 3.0 + d * (nw * nb) / 24.0);
                if (best_c < 0 || cost < best * 0.999) {
                    best = cost;
                    best_c = c;
                    best_d = d;
                    best_ncg = ncg64;
                    best_lds = lds64;
                }
            }
        }
        if (best_c >= 0) {
            a.ncg = best_ncg;
            a.total = nrp64 * best_ncg * nlin;
            a.ipw = g_tile_ipw > 0 ? g_tile_ipw : best_d;
            a.per_xcd = ((a.total + a.ipw - 1) / a.ipw + 7) / 8;
            if (best_c == 0)
                return gelu ? launch_resident64<2, true, 12>(a, best_lds, st)
                            : launch_resident64<2, false, 12>(a, best_lds, st);
            if (best_c == 1)
                return gelu ? launch_resident64<3, true>(a, best_lds, st) : launch_resident64<3, false>(a, best_lds, st);
            return gelu ? launch_resident64<2, true>(a, best_lds, st) : launch_resident64<2, false>(a, best_lds, st);
        }
    }
    const int nrp = (M + TL_BM - 1) / TL_BM;
    const int nb = choose_nb(nrp, nbr_max, nlin);
    a.ncg = (nbr_max + TL_WAVES * nb - 1) / (TL_WAVES * nb);
    a.total = nrp * a.ncg * nlin;
    a.ipw = 1;
    if (mode == TL_PLAN && nchunk == 1) {
        // Persistent workgroups: d items of one row panel per workgroup, d a
        // divisor of the items per panel.  A workgroup costs one panel fetch
        // (about 2/3 of an item) plus d items, and the launch runs in
        // ceil(workgroups / resident slots) rounds; take the cheapest d.
        const int per_rp = a.ncg * nlin;
        const long slots = g_tile_min_wgs; // two workgroups per CU
        double best = 0.0;
        for (int d = 1; d <= per_rp; d++) {
            if (per_rp % d)
                continue;
            const long nwg = a.total / d;
            const long rounds = (nwg + slots - 1) / slots;
            const double cost = (double)rounds * (2.0 / 3.0 + d);
            if (a.ipw == 1 && d == 1) {
                best = cost;
            } else if (cost < best * 0.999) {
                best = cost;
                a.ipw = d;
            }
        }
        if (g_tile_ipw > 0)
            a.ipw = g_tile_ipw;
    }
    a.per_xcd = ((a.total + a.ipw - 1) / a.ipw + 7) / 8;
    const size_t lds_x = (size_t)TL_BM * (KC + ((KC & 31) ? 0 : TL_PAD)) * sizeof(f16);
    const size_t lds_y = (size_t)TL_BM * (TL_WAVES * nb * 16 + TL_PAD) * sizeof(f16);
    // plan kernel: panel + one private staging tile per wave; generic kernel:
    // the output tile reuses the panel's storage
    const size_t lds = mode == TL_PLAN
                           ? lds_x + (size_t)TL_WAVES * TL_BM * (16 * nb + 8) * sizeof(f16)
                           : std::max(lds_x, lds_y);
    if (mode == TL_PLAN) {
        if (gelu) launch_nb<true, TL_PLAN>(nb, a, lds, st);
        else launch_nb<false, TL_PLAN>(nb, a, lds, st);
    } else if (mode == TL_RAW) {
        if (gelu) launch_nb<true, TL_RAW>(nb, a, lds, st);
        else launch_nb<false, TL_RAW>(nb, a, lds, st);
    } else if (mode == TL_FILTER) {
        if (gelu) launch_nb<true, TL_FILTER>(nb, a, lds, st);
        else launch_nb<false, TL_FILTER>(nb, a, lds, st);
    } else {
        if (gelu) launch_nb<true, TL_DENSE>(nb, a, lds, st);
        else launch_nb<false, TL_DENSE>(nb, a, lds, st);
    }
    return launch_status("tile_linear launch");
}

static void chunking(int K, int *KC, int *nchunk) {
    if (K <= TL_MAX_PANEL) {
        *KC = K;
        *nchunk = 1;
    } else {
        *KC = TL_CHUNK;
        *nchunk = (K + TL_CHUNK - 1) / TL_CHUNK;
    }
}

static int raw_tile_linear(void *Y, const void *X, const int *row_ptr, const int *row_offset,
                           const void *data, int M, int N, int K, const void *bias,
                           bool gelu, void *stream, const char *who) {
    ET_REQUIRE(Y && X && row_ptr && bias, ET_ERR_INVALID_ARG, "%s: null pointer", who);
    ET_REQUIRE(M >= 0 && N > 0 && K > 0, ET_ERR_INVALID_ARG, "%s: M=%d N=%d K=%d", who, M, N, K);
    ET_REQUIRE(N % 16 == 0 && K % 16 == 0, ET_ERR_UNSUPPORTED,
               "%s: N=%d and K=%d must be multiples of 16", who, N, K);
    ET_REQUIRE(aligned16(Y) && aligned16(X) && aligned16(bias) && aligned16(data),
               ET_ERR_ALIGNMENT, "%s: Y, X, W_data and bias must be 16-byte aligned", who);
    if (M == 0)
        return ET_OK;
    TlProblem p;
    p.Y = static_cast<f16 *>(Y);
    p.cptr = row_ptr;
    p.row_offset = row_offset;
    p.data = static_cast<const f16 *>(data);
    p.bias = static_cast<const f16 *>(bias);
    p.N = N;
    p.nbr = N / 16;
    int KC, nchunk;
    chunking(K, &KC, &nchunk);
    return tile_launch(&p, 1, static_cast<const f16 *>(X), M, K, KC, nchunk, gelu,
                       nchunk == 1 ? TL_RAW : TL_FILTER, static_cast<hipStream_t>(stream));
}

} // namespace et

static int g_tail_pair_min_wgs = 0; // et_tuning_set("tile_tail_pair_min_wgs"): 0 = three quarters of the CUs

extern "C" int et_tuning_set(const char *key, int value) {
    if (key && !strcmp(key, "tile_splitk_k1")) {
        et::g_tile_splitk_k1 = value;
        return ET_OK;
    }
    if (key && !strcmp(key, "tile_splitk_rows")) {
        et::g_tile_splitk_rows = value;
        return ET_OK;
    }
    if (key && !strcmp(key, "row_gemm_min_rows")) {
        et::g_row_gemm_min_rows = value;
        return ET_OK;
    }
    if (key && !strcmp(key, "tile_nb")) {
        et::g_tile_nb = value;
        return ET_OK;
    }
    if (key && !strcmp(key, "tile_ipw")) {
        et::g_tile_ipw = value;
        return ET_OK;
    }
    if (key && !strcmp(key, "tile_bm64")) {
        et::g_tile_bm64 = value;
        return ET_OK;
    }
    if (key && !strcmp(key, "tile_tail_pair_min_wgs")) {
        g_tail_pair_min_wgs = value;
        return ET_OK;
    }
    if (key && !strcmp(key, "tile_tail_pair")) {
        et::set_tail_pair(value);
        return ET_OK;
    }
    if (key && !strcmp(key, "tile_wait_spin")) {
        et::set_tail_spin(value);
        return ET_OK;
    }
    if (key && !strcmp(key, "tile_fuse_ffn")) {
        et::g_tile_fuse_ffn = value;
        return ET_OK;
    }
    if (key && !strcmp(key, "tile_ln_chunked")) {
        et::g_tile_ln_chunked = value;
        return ET_OK;
    }
    if (key && !strcmp(key, "tile_ln_min_panels")) {
        et::g_tile_ln_min_panels = value > 0 ? value : 96;
        et::g_tile_tail_min_panels = value > 0 ? value : 72;
        return ET_OK;
    }
    if (key && !strcmp(key, "tile_fuse_ln")) {
        et::g_tile_fuse_ln = value;
        return ET_OK;
    }
    if (key && !strcmp(key, "tile_min_wgs")) {
        et::g_tile_min_wgs = value;
        return ET_OK;
    }
    if (key && !strcmp(key, "ln_rows")) {
        et::set_ln_rows(value);
        return ET_OK;
    }
    if (key && !strcmp(key, "attn_packed")) {
        et::set_attn_packed(value);
        return ET_OK;
    }
    if (key && !strcmp(key, "attn_vwin")) {
        et::set_attn_vwin(value);
        return ET_OK;
    }
    if (key && !strcmp(key, "attn_variant")) {
        et::set_attn_variant(value);
        return ET_OK;
    }
    et::set_error("et_tuning_set: unknown key");
    return ET_ERR_INVALID_ARG;
}

extern "C" int et_tile_spmm_add_bias(void *Y, const void *X, const int *W_row_ptr,
                                     const int *W_row_offset, const void *W_data, int M,
                                     int N, int K, const void *bias, void *stream) {
    return et::raw_tile_linear(Y, X, W_row_ptr, W_row_offset, W_data, M, N, K, bias, false,
                               stream, "et_tile_spmm_add_bias");
}

extern "C" int et_tile_spmm_add_bias_gelu(void *Y, const void *X, const int *W_row_ptr,
                                          const int *W_row_offset, const void *W_data,
                                          int M, int N, int K, const void *bias,
                                          void *stream) {
    return et::raw_tile_linear(Y, X, W_row_ptr, W_row_offset, W_data, M, N, K, bias, true,
                               stream, "et_tile_spmm_add_bias_gelu");
}

namespace et {
// dense_gemm.hip
int dense_gemm_launch(void *const *Ys, const void *X, const void *const *Ws, const void *const *biases,
                      const int *Ns, int nlin, int M, int K, bool gelu, hipStream_t st);
static int row_linear(void *out, const void *in, const void *weight, const void *bias, int M, int N,
                      int K, bool gelu, void *stream) {
    ET_REQUIRE(out && in && weight && bias, ET_ERR_INVALID_ARG, "et_row_spmm_add_bias: null pointer");
    ET_REQUIRE(M >= 0 && N > 0 && K > 0, ET_ERR_INVALID_ARG,
               "et_row_spmm_add_bias: M=%d N=%d K=%d", M, N, K);
    ET_REQUIRE(N % 16 == 0 && K % 16 == 0, ET_ERR_UNSUPPORTED,
               "et_row_spmm_add_bias: N=%d and K=%d must be multiples of 16", N, K);
    ET_REQUIRE(aligned16(out) && aligned16(in) && aligned16(weight) && aligned16(bias),
               ET_ERR_ALIGNMENT, "et_row_spmm_add_bias: pointers must be 16-byte aligned");
    if (M == 0)
        return ET_OK;
    if (g_row_gemm_min_rows > 0 && M >= g_row_gemm_min_rows) {
        const int rc = dense_gemm_launch(&out, in, &weight, &bias, &N, 1, M, K, gelu, static_cast<hipStream_t>(stream));
        if (rc != ET_ERR_UNSUPPORTED)
            return rc;
    }
    TlProblem p;
    p.Y = static_cast<f16 *>(out);
    p.cptr = nullptr;
    p.row_offset = nullptr;
    p.data = static_cast<const f16 *>(weight);
    p.bias = static_cast<const f16 *>(bias);
    p.N = N;
    p.nbr = N / 16;
    int KC, nchunk;
    chunking(K, &KC, &nchunk);
    return tile_launch(&p, 1, static_cast<const f16 *>(in), M, K, KC, nchunk, gelu, TL_DENSE,
                       static_cast<hipStream_t>(stream));
}
} // namespace et

extern "C" int et_row_spmm_prefers_gemm(int M, int N, int K) {
    return et::g_row_gemm_min_rows > 0 && M >= et::g_row_gemm_min_rows && N > 0 && N % 16 == 0 && K >= 32 &&
                   K % 32 == 0
               ? 1
               : 0;
}

extern "C" int et_row_spmm_add_bias_multi(void *const *outs, const void *in, const void *const *weights,
                                          const void *const *biases, const int *Ns, int n, int M, int K,
                                          void *stream) {
    using namespace et;
    ET_REQUIRE(outs && in && weights && biases && Ns, ET_ERR_INVALID_ARG, "et_row_spmm_add_bias_multi: null pointer");
    ET_REQUIRE(n >= 1 && n <= 3 && M >= 0 && K > 0, ET_ERR_INVALID_ARG, "et_row_spmm_add_bias_multi: n=%d M=%d K=%d",
               n, M, K);
    if (M == 0)
        return ET_OK;
    if (et_row_spmm_prefers_gemm(M, Ns[0], K)) {
        const int rc = dense_gemm_launch(outs, in, weights, biases, Ns, n, M, K, false, static_cast<hipStream_t>(stream));
        if (rc != ET_ERR_UNSUPPORTED)
            return rc;
    }
    for (int i = 0; i < n; i++) { // one after the other
        const int rc = row_linear(outs[i], in, weights[i], biases[i], M, Ns[i], K, false, stream);
        if (rc != ET_OK)
            return rc;
    }
    return ET_OK;
}

extern "C" int et_row_spmm_add_bias(void *out, const void *in, const void *weight,
                                    const void *bias, int M, int N, int K, void *stream) {
    return et::row_linear(out, in, weight, bias, M, N, K, false, stream);
}

extern "C" int et_row_spmm_add_bias_gelu(void *out, const void *in, const void *weight,
                                         const void *bias, int M, int N, int K, void *stream) {
    return et::row_linear(out, in, weight, bias, M, N, K, true, stream);
}

// ---------------------------------------------------------------------------
// plans
// ---------------------------------------------------------------------------
extern "C" int et_tile_plan_create(et_tile_plan **plan, int in_feat, int out_feat, int ntile,
                                   const void *data, const int *row_ptr,
                                   const int *row_offset, const void *bias) {
    using namespace et;
    ET_REQUIRE(plan && row_ptr && bias && (ntile == 0 || (data && row_offset)),
               ET_ERR_INVALID_ARG, "et_tile_plan_create: null pointer");
    *plan = nullptr;
    const int v = et_tile_mat_validate(out_feat, in_feat, ntile, row_ptr, row_offset);
    ET_REQUIRE(v == 0, ET_ERR_FORMAT, "et_tile_plan_create: malformed tile_mat (check %d)", v);
    const int nbr = out_feat / 16;
    int KC, nchunk;
    chunking(in_feat, &KC, &nchunk);
    // Plan layout: tiles ordered by (chunk, block-row, column); every
    // (chunk, block-row) segment padded to an even count with an all-zero
    // tile that reuses the segment's last column (so a pair never straddles
    // two block-rows and the kernel needs no odd-tail handling).
    std::vector<int> order(ntile);
    std::iota(order.begin(), order.end(), 0);
    for (int bn = 0; bn < nbr; bn++)
        std::stable_sort(order.begin() + row_ptr[bn], order.begin() + row_ptr[bn + 1],
                         [&](int x, int y) { return row_offset[x] < row_offset[y]; });
    std::vector<int> off, cptr((size_t)nbr * nchunk + 1);
    std::vector<uint16_t> packed;
    off.reserve(ntile + (size_t)nbr * nchunk);
    packed.reserve(((size_t)ntile + (size_t)nbr * nchunk) * 256);
    const uint16_t *src = static_cast<const uint16_t *>(data);
    for (int c = 0; c < nchunk; c++) {
        for (int bn = 0; bn < nbr; bn++) {
            cptr[(size_t)c * nbr + bn] = (int)off.size();
            int cnt = 0, last = 0;
            for (int i = row_ptr[bn]; i < row_ptr[bn + 1]; i++) {
                const int o = row_offset[order[i]];
                if (o / KC != c)
                    continue;
                off.push_back((o - c * KC) * 2);
                packed.insert(packed.end(), src + (size_t)order[i] * 256, src + (size_t)order[i] * 256 + 256);
                last = (o - c * KC) * 2;
                cnt++;
            }
            if (cnt & 1) {
                off.push_back(last);
                packed.insert(packed.end(), 256, (uint16_t)0);
            }
        }
    }
    cptr[(size_t)nbr * nchunk] = (int)off.size();
    // spare all-zero pairs behind the last one: the kernels request the first
    // pairs of a wave's stream before they know whether it is empty, and a
    // stream's last stages request up to 2*TL_DEPTH pairs past its end
    for (int i = 0; i < 2 * TL_DEPTH + 1; i++) {
        off.push_back(0);
        off.push_back(0);
        packed.insert(packed.end(), 512, (uint16_t)0);
    }

    et_tile_plan *p = new et_tile_plan();
    {
        static unsigned long long next_uid = 0;
        p->uid = ++next_uid;
    }
    // column-sorted host copy (the layer-tail program is built from it)
    p->h_row_ptr.assign(row_ptr, row_ptr + nbr + 1);
    p->h_col.resize(ntile);
    p->h_data.resize((size_t)ntile * 256);
    for (int i = 0; i < ntile; i++) {
        p->h_col[i] = row_offset[order[i]];
        memcpy(&p->h_data[(size_t)i * 256], src + (size_t)order[i] * 256, 512);
    }
    p->in_feat = in_feat;
    p->out_feat = out_feat;
    p->ntile = ntile;
    p->KC = KC;
    p->nchunk = nchunk;
    int rc = ET_OK;
    auto up = [&](void **dst, const void *h, size_t bytes) {
        if (rc != ET_OK)
            return;
        rc = et_malloc(dst, std::max<size_t>(bytes, 16));
        if (rc == ET_OK && bytes)
            rc = et_memcpy_h2d(*dst, h, bytes);
    };
    up((void **)&p->d_data, packed.data(), packed.size() * 2);
    up((void **)&p->d_cptr, cptr.data(), cptr.size() * 4);
    up((void **)&p->d_row_offset, off.data(), off.size() * 4);
    up((void **)&p->d_bias, bias, (size_t)out_feat * 2);
    if (rc != ET_OK) {
        et_tile_plan_destroy(p);
        return rc;
    }
    *plan = p;
    return ET_OK;
}

extern "C" void et_tile_plan_destroy(et_tile_plan *p) {
    if (!p)
        return;
    et_free(p->d_data);
    et_free(p->d_cptr);
    et_free(p->d_row_offset);
    et_free(p->d_bias);
    et::tail_program_destroy(p->tail);
    delete p;
}

extern "C" int et_tile_plan_query(const et_tile_plan *p, int *in_feat, int *out_feat,
                                  int *ntile, int *nchunk, int *chunk_cols) {
    ET_REQUIRE(p, ET_ERR_INVALID_ARG, "et_tile_plan_query: null plan");
    if (in_feat) *in_feat = p->in_feat;
    if (out_feat) *out_feat = p->out_feat;
    if (ntile) *ntile = p->ntile;
    if (nchunk) *nchunk = p->nchunk;
    if (chunk_cols) *chunk_cols = p->KC;
    return ET_OK;
}

extern "C" int et_tile_plan_run_multi(const et_tile_plan *const *plans, void *const *Ys, int n,
                                      const void *X, int M, void *stream) {
    using namespace et;
    ET_REQUIRE(plans && Ys && X, ET_ERR_INVALID_ARG, "et_tile_plan_run_multi: null pointer");
    ET_REQUIRE(n >= 1 && n <= TL_MAX_LIN, ET_ERR_INVALID_ARG, "et_tile_plan_run_multi: n=%d", n);
    ET_REQUIRE(M >= 0, ET_ERR_INVALID_ARG, "et_tile_plan_run_multi: M=%d", M);
    TlProblem pr[TL_MAX_LIN];
    for (int i = 0; i < n; i++) {
        ET_REQUIRE(plans[i] && Ys[i], ET_ERR_INVALID_ARG, "et_tile_plan_run_multi: null entry %d", i);
        ET_REQUIRE(plans[i]->in_feat == plans[0]->in_feat, ET_ERR_INVALID_ARG,
                   "et_tile_plan_run_multi: in_feat differs");
        ET_REQUIRE(aligned16(Ys[i]), ET_ERR_ALIGNMENT, "et_tile_plan_run_multi: Y not aligned");
        pr[i].Y = static_cast<f16 *>(Ys[i]);
        pr[i].cptr = plans[i]->d_cptr;
        pr[i].row_offset = plans[i]->d_row_offset;
        pr[i].data = plans[i]->d_data;
        pr[i].bias = plans[i]->d_bias;
        pr[i].N = plans[i]->out_feat;
        pr[i].nbr = plans[i]->out_feat / 16;
    }
    ET_REQUIRE(aligned16(X), ET_ERR_ALIGNMENT, "et_tile_plan_run_multi: X not aligned");
    if (M == 0)
        return ET_OK;
    return tile_launch(pr, n, static_cast<const f16 *>(X), M, plans[0]->in_feat, plans[0]->KC,
                       plans[0]->nchunk, false, TL_PLAN, static_cast<hipStream_t>(stream));
}

extern "C" int et_tile_plan_ln_fusable(const et_tile_plan *plan) {
    return plan && et::ln_block_rows(plan->out_feat / 16) != 0 && plan->out_feat % 8 == 0 &&
                   et::g_tile_fuse_ln != 0
               ? 1
               : 0;
}

// The fused kernels run one workgroup per 32-row panel; with few rows that
// leaves most CUs idle and the two-launch form (more, smaller workgroups) wins.
static bool ln_fusion_pays(int M) { return M >= 32 * et::g_tile_ln_min_panels; }
static bool tail_fusion_pays(int M) { return M >= 32 * et::g_tile_tail_min_panels; }

extern "C" int et_tile_plan_run_ln(const et_tile_plan *plan, void *Y, const void *X,
                                   const void *skip, const void *gamma, const void *beta, int M,
                                   void *stream) {
    using namespace et;
    ET_REQUIRE(plan && Y && X && skip && gamma && beta, ET_ERR_INVALID_ARG,
               "et_tile_plan_run_ln: null pointer");
    ET_REQUIRE(M >= 0, ET_ERR_INVALID_ARG, "et_tile_plan_run_ln: M=%d", M);
    ET_REQUIRE(aligned16(Y) && aligned16(X) && aligned16(skip) && aligned16(gamma) && aligned16(beta),
               ET_ERR_ALIGNMENT, "et_tile_plan_run_ln: pointers must be 16-byte aligned");
    if (M == 0)
        return ET_OK;
    const int nbr = plan->out_feat / 16;
    if (!et_tile_plan_ln_fusable(plan) || (!ln_fusion_pays(M) && Y != skip)) {
        // rows too wide for one workgroup, or too few of them: the two kernels, one after the other
        ET_REQUIRE(Y != skip, ET_ERR_INVALID_ARG,
                   "et_tile_plan_run_ln: Y must not alias skip for out_feat=%d", plan->out_feat);
        const int rc = et_tile_plan_run(plan, Y, X, M, 0, stream);
        if (rc != ET_OK)
            return rc;
        return et_skip_layernorm(Y, skip, gamma, beta, M, plan->out_feat, stream);
    }
    TlProblem pr;
    pr.Y = static_cast<f16 *>(Y);
    pr.cptr = plan->d_cptr;
    pr.row_offset = plan->d_row_offset;
    pr.data = plan->d_data;
    pr.bias = plan->d_bias;
    pr.N = plan->out_feat;
    pr.nbr = nbr;
    return tile_launch_ln(pr, static_cast<const f16 *>(X), M, plan->in_feat, plan->KC, plan->nchunk,
                          static_cast<const f16 *>(skip), static_cast<const f16 *>(gamma),
                          static_cast<const f16 *>(beta), static_cast<hipStream_t>(stream));
}

extern "C" int et_tile_plan_ffn_fusable(const et_tile_plan *p1, const et_tile_plan *p2) {
    using namespace et;
    if (!p1 || !p2 || !g_tile_fuse_ffn)
        return 0;
    return p1->nchunk == 1 && p2->in_feat == p1->out_feat && p2->nchunk <= TL_FFN_MAX_PHASES &&
                   p2->KC / 16 <= TL_FFN_WAVES * 3 &&
                   p2->out_feat / 16 <= TL_FFN_WAVES * 3 && p2->out_feat % 8 == 0 &&
                   ffn_lds_bytes(p1->in_feat, p2->KC) <= 160 * 1024
               ? 1
               : 0;
}

extern "C" int et_tile_plan_run_ffn_ln(const et_tile_plan *p1, const et_tile_plan *p2, void *Y,
                                       const void *X, void *hidden, const void *skip,
                                       const void *gamma, const void *beta, int M, void *stream) {
    using namespace et;
    ET_REQUIRE(p1 && p2 && Y && X && skip && gamma && beta, ET_ERR_INVALID_ARG,
               "et_tile_plan_run_ffn_ln: null pointer");
    ET_REQUIRE(M >= 0, ET_ERR_INVALID_ARG, "et_tile_plan_run_ffn_ln: M=%d", M);
    ET_REQUIRE(p2->in_feat == p1->out_feat, ET_ERR_INVALID_ARG,
               "et_tile_plan_run_ffn_ln: the second linear takes %d inputs, the first gives %d",
               p2->in_feat, p1->out_feat);
    ET_REQUIRE(aligned16(Y) && aligned16(X) && aligned16(skip) && aligned16(gamma) && aligned16(beta) &&
                   aligned16(hidden),
               ET_ERR_ALIGNMENT, "et_tile_plan_run_ffn_ln: pointers must be 16-byte aligned");
    if (M == 0)
        return ET_OK;
    const bool fusable = et_tile_plan_ffn_fusable(p1, p2) != 0;
    if (!fusable || (hidden && !ln_fusion_pays(M))) {
        // the three steps one after the other, through the caller's buffer
        ET_REQUIRE(hidden, ET_ERR_UNSUPPORTED,
                   "et_tile_plan_run_ffn_ln: these shapes need the hidden buffer (%d x %d halves)", M,
                   p1->out_feat);
        const int rc = et_tile_plan_run(p1, hidden, X, M, 1, stream);
        if (rc != ET_OK)
            return rc;
        return et_tile_plan_run_ln(p2, Y, hidden, skip, gamma, beta, M, stream);
    }
    TlProblem a, b;
    a.Y = nullptr;
    a.cptr = p1->d_cptr;
    a.row_offset = p1->d_row_offset;
    a.data = p1->d_data;
    a.bias = p1->d_bias;
    a.N = p1->out_feat;
    a.nbr = p1->out_feat / 16;
    b.Y = static_cast<f16 *>(Y);
    b.cptr = p2->d_cptr;
    b.row_offset = p2->d_row_offset;
    b.data = p2->d_data;
    b.bias = p2->d_bias;
    b.N = p2->out_feat;
    b.nbr = p2->out_feat / 16;
    return tile_launch_ffn(nullptr, a, b, static_cast<const f16 *>(X), M, p1->in_feat, p2->KC, p2->nchunk,
                           static_cast<const f16 *>(skip), static_cast<const f16 *>(gamma),
                           static_cast<const f16 *>(beta), nullptr, nullptr,
                           static_cast<hipStream_t>(stream));
}

extern "C" int et_tile_plan_tail_fusable(const et_tile_plan *pO, const et_tile_plan *p1,
                                         const et_tile_plan *p2) {
    return pO && et_tile_plan_ffn_fusable(p1, p2) && pO->nchunk == 1 && pO->in_feat == pO->out_feat &&
                   pO->out_feat == p1->in_feat && p2->out_feat == p1->in_feat &&
                   pO->out_feat / 16 <= et::TL_FFN_WAVES * 3 && et::g_tile_fuse_ffn >= 2
               ? 1
               : 0;
}

extern "C" int et_tile_plan_run_tail(const et_tile_plan *pO, const et_tile_plan *p1,
                                     const et_tile_plan *p2, void *Y, const void *attn, const void *input,
                                     void *mid, void *hidden, const void *gamma1, const void *beta1,
                                     const void *gamma2, const void *beta2, int M, void *stream) {
    using namespace et;
    ET_REQUIRE(pO && p1 && p2 && Y && attn && input && gamma1 && beta1 && gamma2 && beta2,
               ET_ERR_INVALID_ARG, "et_tile_plan_run_tail: null pointer");
    ET_REQUIRE(M >= 0, ET_ERR_INVALID_ARG, "et_tile_plan_run_tail: M=%d", M);
    ET_REQUIRE(pO->out_feat == p1->in_feat && p2->in_feat == p1->out_feat && p2->out_feat == p1->in_feat,
               ET_ERR_INVALID_ARG, "et_tile_plan_run_tail: the three linears do not chain (%d->%d, %d->%d, %d->%d)",
               pO->in_feat, pO->out_feat, p1->in_feat, p1->out_feat, p2->in_feat, p2->out_feat);
    ET_REQUIRE(aligned16(Y) && aligned16(attn) && aligned16(input) && aligned16(mid) && aligned16(hidden) &&
                   aligned16(gamma1) && aligned16(beta1) && aligned16(gamma2) && aligned16(beta2),
               ET_ERR_ALIGNMENT, "et_tile_plan_run_tail: pointers must be 16-byte aligned");
    if (M == 0)
        return ET_OK;
    if (!et_tile_plan_tail_fusable(pO, p1, p2) || (mid && !tail_fusion_pays(M))) {
        // step by step through the caller's buffers
        ET_REQUIRE(mid, ET_ERR_UNSUPPORTED,
                   "et_tile_plan_run_tail: these shapes need the mid buffer (%d x %d halves)", M, pO->out_feat);
        const int rc = et_tile_plan_run_ln(pO, mid, attn, input, gamma1, beta1, M, stream);
        if (rc != ET_OK)
            return rc;
        return et_tile_plan_run_ffn_ln(p1, p2, Y, mid, hidden, mid, gamma2, beta2, M, stream);
    }
    // The fused kernel runs one workgroup per CU and 32-row panel, in rounds of
    // as many panels as there are CUs.  A last round that would leave most CUs
    // idle costs as much as a full one: with the caller's buffers at hand those
    // rows run step by step instead (after the fused launch on the same stream;
    // rows are independent).
    if (mid && hidden) {
        const int cus = std::max(et_device_cu_count(), 1);
        const int panels = (M + TL_BM - 1) / TL_BM, full = panels / cus * cus, rem = panels - full;
        if (full > 0 && rem > 0 && rem < g_tile_tail_min_panels) {
            const int M1 = full * TL_BM;
            int rc = et_tile_plan_run_tail(pO, p1, p2, Y, attn, input, nullptr, nullptr, gamma1, beta1, gamma2,
                                           beta2, M1, stream);
            if (rc != ET_OK)
                return rc;
            const size_t off = (size_t)M1 * pO->out_feat; // all of Y, attn, input, mid are [rows x model width]
            f16 *midr = static_cast<f16 *>(mid) + off;
            rc = et_tile_plan_run_ln(pO, midr, static_cast<const f16 *>(attn) + off,
                                     static_cast<const f16 *>(input) + off, gamma1, beta1, M - M1, stream);
            if (rc != ET_OK)
                return rc;
            return et_tile_plan_run_ffn_ln(p1, p2, static_cast<f16 *>(Y) + off, midr, hidden, midr, gamma2, beta2,
                                           M - M1, stream);
        }
    }
    TlProblem o, a, b;
    o.Y = nullptr;
    o.cptr = pO->d_cptr;
    o.row_offset = pO->d_row_offset;
    o.data = pO->d_data;
    o.bias = pO->d_bias;
    o.N = pO->out_feat;
    o.nbr = pO->out_feat / 16;
    a.Y = nullptr;
    a.cptr = p1->d_cptr;
    a.row_offset = p1->d_row_offset;
    a.data = p1->d_data;
    a.bias = p1->d_bias;
    a.N = p1->out_feat;
    a.nbr = p1->out_feat / 16;
    b.Y = static_cast<f16 *>(Y);
    b.cptr = p2->d_cptr;
    b.row_offset = p2->d_row_offset;
    b.data = p2->d_data;
    b.bias = p2->d_bias;
    b.N = p2->out_feat;
    b.nbr = p2->out_feat / 16;
    return tile_launch_ffn(&o, a, b, static_cast<const f16 *>(attn), M, p1->in_feat, p2->KC, p2->nchunk,
                           static_cast<const f16 *>(input), static_cast<const f16 *>(gamma1),
                           static_cast<const f16 *>(beta1), static_cast<const f16 *>(gamma2),
                           static_cast<const f16 *>(beta2), static_cast<hipStream_t>(stream));
}

extern "C" int et_tile_plan_run(const et_tile_plan *plan, void *Y, const void *X, int M, int gelu,
                                void *stream) {
    using namespace et;
    ET_REQUIRE(plan && Y && X, ET_ERR_INVALID_ARG, "et_tile_plan_run: null pointer");
    ET_REQUIRE(M >= 0, ET_ERR_INVALID_ARG, "et_tile_plan_run: M=%d", M);
    ET_REQUIRE(aligned16(Y) && aligned16(X), ET_ERR_ALIGNMENT, "et_tile_plan_run: Y/X not aligned");
    if (M == 0)
        return ET_OK;
    TlProblem pr;
    pr.Y = static_cast<f16 *>(Y);
    pr.cptr = plan->d_cptr;
    pr.row_offset = plan->d_row_offset;
    pr.data = plan->d_data;
    pr.bias = plan->d_bias;
    pr.N = plan->out_feat;
    pr.nbr = plan->out_feat / 16;
    pr.ntile = plan->ntile;
    return tile_launch(&pr, 1, static_cast<const f16 *>(X), M, plan->in_feat, plan->KC,
                       plan->nchunk, gelu != 0, TL_PLAN, static_cast<hipStream_t>(stream));
}

// ---------------------------------------------------------------------------
// layer tail with caller-provided scratch: pairs of workgroups over 64-row
// panels (tile_tail.hip) where that applies and pays
// ---------------------------------------------------------------------------
extern "C" size_t et_tile_plan_tail_ws_bytes(const et_tile_plan *pO, const et_tile_plan *p1,
                                             const et_tile_plan *p2, int M) {
    return et::tail_pair_ws_bytes(pO, p1, p2, M);
}

extern "C" size_t et_tail_ws_bytes_for(int d_model, int rows) {
    // (nothing while the paired form is switched off: an encoder's workspace is then the reference's)
    return et::tail_pair_enabled() ? et::tail_ws_bytes_for(d_model, rows) : 0;
}

extern "C" int et_tile_plan_tail_prepare(const et_tile_plan *pO, const et_tile_plan *p1,
                                         const et_tile_plan *p2) {
    using namespace et;
    ET_REQUIRE(pO && p1 && p2, ET_ERR_INVALID_ARG, "et_tile_plan_tail_prepare: null plan");
    (void)wait_status_device(); // (allocated here rather than inside a run)
    if (!tail_pair_applies(pO, p1, p2))
        return ET_OK; // nothing to prepare: et_tile_plan_run_tail_ws will run the other kernels
    return tail_pair_prepare(pO, p1, const_cast<et_tile_plan *>(p2));
}

extern "C" int et_tile_plan_run_tail_ws(const et_tile_plan *pO, const et_tile_plan *p1,
                                        const et_tile_plan *p2, void *Y, const void *attn, const void *input,
                                        void *mid, void *hidden, const void *gamma1, const void *beta1,
                                        const void *gamma2, const void *beta2, int M, void *ws, size_t ws_bytes,
                                        void *stream) {
    using namespace et;
    ET_REQUIRE(pO && p1 && p2 && Y && attn && input && gamma1 && beta1 && gamma2 && beta2,
               ET_ERR_INVALID_ARG, "et_tile_plan_run_tail_ws: null pointer");
    if (ws && M > 0 && tail_pair_applies(pO, p1, p2)) {
        const size_t need = tail_pair_ws_bytes(pO, p1, p2, M);
        const int cus = std::max(et_device_cu_count(), 1);
        const int wgs = 2 * ((M + 63) / 64);
        const int min_wgs = g_tail_pair_min_wgs > 0 ? g_tail_pair_min_wgs : (3 * cus) / 4;
        if (ws_bytes >= need && (wgs >= min_wgs || !mid || tail_pair_forced())) {
            ET_REQUIRE(aligned16(Y) && aligned16(attn) && aligned16(input) && aligned16(gamma1) &&
                           aligned16(beta1) && aligned16(gamma2) && aligned16(beta2) && aligned16(ws),
                       ET_ERR_ALIGNMENT, "et_tile_plan_run_tail_ws: pointers must be 16-byte aligned");
            const int rc = tail_pair_prepare(pO, p1, const_cast<et_tile_plan *>(p2)); // (returns at once when prepared)
            if (rc != ET_OK)
                return rc;
            return tail_pair_launch(pO, p1, p2, static_cast<f16 *>(Y), static_cast<const f16 *>(attn),
                                    static_cast<const f16 *>(input), static_cast<const f16 *>(gamma1),
                                    static_cast<const f16 *>(beta1), static_cast<const f16 *>(gamma2),
                                    static_cast<const f16 *>(beta2), M, ws, static_cast<hipStream_t>(stream));
        }
    }
    return et_tile_plan_run_tail(pO, p1, p2, Y, attn, input, mid, hidden, gamma1, beta1, gamma2, beta2, M, stream);
}
