// Fused multi-head self-attention for gfx950: on-the-fly (scores never leave
// the CU), attention-aware pruned (compact Q/K/V column sets per head) and the
// score-matrix-in-memory variant, all from one key-tiled online-softmax kernel.
//
// Reference math (kernels/attention.cu:51-120): Qs = half(Q*scale),
// S = Qs K^T + mask, P = softmax_base2(S), Z = P V, per head, per 16-row query
// block, with the whole 16 x seq_len score block in shared memory.  Here the
// keys are walked in tiles of 64 with a running max / running sum, so LDS use
// is independent of seq_len and no S x S block exists anywhere.
//
// Layout trick: both contractions are issued TRANSPOSED.
//   S^T(keys x queries) = K_tile * Qs^T : A = K rows from LDS, B = Q fragment
//     held in registers for the whole kernel.  A lane (c = lane%16, g =
//     lane/16) then holds, for ONE query c, four consecutive keys 4g..4g+3 of
//     each 16-key subtile, so row max / row sum need only two cross-lane steps
//     (xor 16, xor 32) and the running statistics are per-lane scalars.
//   O^T(d x queries) = V^T * P^T : the P values a lane already holds are, as
//     they stand, the B operand (8 k-slots = 4 keys of subtile 2kk + 4 keys
//     of subtile 2kk+1); the matching A operand is a V^T fragment, which the
//     LDS transpose read (ds_read_b64_tr_b16) produces from a V tile kept in
//     its natural [key][d] layout (the pruned variant transposes V while
//     staging it instead).  P never goes through LDS and the O accumulator's
//     query index is again the lane's c, so the online rescale is a per-lane
//     multiply.
// K and V tiles of the unpruned variants are staged by DMA (global -> LDS
// without registers), double-buffered, one tile ahead of the MFMAs.
#include "common.h"

#include <cmath>
#include <mutex>
#include <type_traits>
#include <vector>

namespace et {

constexpr int AT_KT = 64; // keys per tile

struct AttnArgs {
    f16 *out;
    const f16 *Q, *K, *V, *QK, *mask;
    const int *seq_lens, *cu_seqlens;
    const int *qk_head_ptr, *v_col_id, *v_head_ptr;
    // optional: one bit per (16 query rows, 64-key tile) of the mask, set when
    // any of its elements is non-zero (et_attention_mask_summary); msum_words
    // 32-bit words per group of 16 rows
    const unsigned *msum;
    int msum_words;
    int ldq, ldv, ldo, seq_len, nhead, batch, nqb, total, per_xcd;
    // columns per head in Q, K, V and the output where that is not the kernel's
    // HD (any multiple of 16 below it; the register-staged kernel only): 0 = HD
    int head_width;
    // columns per head in Q and K where they are narrower than the head (compact Q / K with the same number of
    // kept columns in every head; register-staged kernel): 0 = the head's width
    int qk_width;
    float log2_scale, scale;
};

// eight (four) halves at p + d0 of which those at or beyond n read as zero.
// Whole groups are one load that needs no more than the 2-byte alignment of a
// half (compact operands start at arbitrary columns; the hardware takes
// unaligned multi-dword accesses to global memory), only a group that straddles
// n is fetched element by element.
typedef f16x8 f16x8_u __attribute__((aligned(2)));
typedef f16x4 f16x4_u __attribute__((aligned(2)));
__device__ __forceinline__ f16x8 load8_guard(const f16 *p, int d0, int n) {
    if (d0 + 8 <= n)
        return *reinterpret_cast<const f16x8_u *>(p + d0);
    f16x8 v;
#pragma unroll
    for (int j = 0; j < 8; j++)
        v[j] = (d0 + j < n) ? p[d0 + j] : (f16)0;
    return v;
}
__device__ __forceinline__ f16x4 load4_guard(const f16 *p, int d0, int n) {
    if (d0 + 4 <= n)
        return *reinterpret_cast<const f16x4_u *>(p + d0);
    f16x4 v;
#pragma unroll
    for (int j = 0; j < 4; j++)
        v[j] = (d0 + j < n) ? p[d0 + j] : (f16)0;
    return v;
}

// Maximum over the four lanes l, l^16, l^32, l^48 (a query's four key groups),
// result in all four.  gfx950's row-swap instructions exchange whole rows of 16
// lanes between two registers in the vector ALU, so no LDS round trip as with
// __shfl_xor.  (The empty asm statements keep the optimiser from reasoning
// about the swapped copies: it otherwise folds max(a, b) of the pair away.)
__device__ __forceinline__ float xor_max_16_32(float v) {
    unsigned a = __builtin_bit_cast(unsigned, v), b = a;
    asm("" : "+v"(b));
    auto r = __builtin_amdgcn_permlane32_swap(a, b, false, false); // a: lanes 0-31 twice, b: lanes 32-63 twice
    unsigned x0 = r[0], x1 = r[1];
    asm("v_max_f32 %0, %0, %1" : "+v"(x0) : "v"(x1));
    unsigned y1 = x0;
    asm("" : "+v"(y1));
    auto q = __builtin_amdgcn_permlane16_swap(x0, y1, false, false); // even rows twice, odd rows twice
    unsigned z0 = q[0], z1 = q[1];
    asm("v_max_f32 %0, %0, %1" : "+v"(z0) : "v"(z1));
    return __builtin_bit_cast(float, z0);
}

// 4 x 4 transpose of 8-byte pieces over the four lanes l, l+16, l+32, l+48: on entry piece j of the lane in
// row g (g = lane / 16) is element (g, j), on return it is element (j, g).  Two row-swap steps per dword.
__device__ __forceinline__ void transpose_pieces_4x4(f16x4 (&p)[4]) {
    typedef unsigned u32x2 __attribute__((ext_vector_type(2)));
    u32x2 pc[4];
#pragma unroll
    for (int j = 0; j < 4; j++)
        pc[j] = __builtin_bit_cast(u32x2, p[j]);
#pragma unroll
    for (int d = 0; d < 2; d++) {
        auto s01 = __builtin_amdgcn_permlane16_swap(pc[0][d], pc[1][d], false, false);
        auto s23 = __builtin_amdgcn_permlane16_swap(pc[2][d], pc[3][d], false, false);
        auto t02 = __builtin_amdgcn_permlane32_swap(s01[0], s23[0], false, false);
        auto t13 = __builtin_amdgcn_permlane32_swap(s01[1], s23[1], false, false);
        pc[0][d] = t02[0];
        pc[2][d] = t02[1];
        pc[1][d] = t13[0];
        pc[3][d] = t13[1];
    }
#pragma unroll
    for (int j = 0; j < 4; j++)
        p[j] = __builtin_bit_cast(f16x4, pc[j]);
}

// PLAIN: the launcher has established that there is no mask (or an all-zero
// one), every sequence has full length and seq_len is a multiple of the
// workgroup's query rows - no guards, no mask bookkeeping.
// Wave priority in the two MFMA sections of a key tile (0 in the softmax
// between them): a wave that has its scores or its P ready issues its MFMAs
// ahead of the waves that are in the vector-ALU part (-1 %).
#ifndef AT_PRIO
#define AT_PRIO 1
#endif

// HDK: width of a head in Q and K.  HDK < HD is attention-aware pruning with
// the same number of kept columns in every head: Q and K are compact
// [rows x nhead*HDK], head h at columns h*HDK, and the scores contract over
// HDK; V and the output keep HD columns per head.
// VWIN (pruned variant with dense Q/K and compact V whose row pitch is a
// multiple of 8): K and V are staged by DMA like the unpruned kernel.  A head's
// compact value columns [c0, c1) start at an arbitrary column, which DMA cannot
// address (16-byte pieces), so the tile holds the 16-byte-aligned WINDOW of 80
// columns that begins at c0 rounded down to 8; the product runs over the
// window's 16-column subtiles that reach into [c0, c1) (at most five), and the
// columns of the window that belong to neighbouring heads are never written.
// One workgroup's work: the NW*16*QS query rows of block qb of (sequence b, head h).
template <int HD, int QS, int NW, bool PRUNED, bool SHAREDQK, bool PLAIN = false, int HDK = HD, bool VWIN = false>
__device__ __forceinline__ void attention_block(const AttnArgs &a, const int b, const int h, const int qb) {
    static_assert(!PLAIN || ((!PRUNED || VWIN) && !SHAREDQK), "the plain form exists for the DMA-staged kernels only");
    static_assert(HDK == HD || (!PRUNED && !SHAREDQK && HDK % 32 == 0), "narrow Q/K heads: on-the-fly kernel only");
    static_assert(!VWIN || (PRUNED && HD == 64), "the value-window form exists for the pruned kernel with 64-wide heads");
    constexpr int AT_THREADS = NW * 64; // NW waves, each owning 16*QS query rows
    constexpr int AT_WAVES = NW;
    constexpr int DK = HDK / 32;   // k-steps of Q K^T
    constexpr int DV = VWIN ? 5 : HD / 16; // 16-wide column subtiles of the output (of the 80-column window)
    // LDS row strides.  K rows are read with ds_read_b128 by 16 lanes at a
    // time: a stride of 32 (mod 64) bytes is conflict-free (measured); V^T rows
    // are read with ds_read_b64, for which an odd multiple of 16 bytes is.
    constexpr int LDK = HDK + 16;
    constexpr int LDV = AT_KT + 8;
    constexpr int QB = AT_WAVES * 16 * QS; // queries per workgroup
    constexpr int LDO = HD + 8;
    // Unpruned operands are staged by DMA (global -> LDS, no registers) in their
    // natural [key][d] layout, K and V alike; the transposed V^T fragments the
    // second contraction needs are then produced by the LDS transpose read
    // (ds_read_b64_tr_b16).  The pruned variant gathers ragged column sets and
    // keeps the register path, which transposes V while storing it - except in
    // its value-window form (VWIN), which is DMA-staged as well.
    constexpr bool DMA = !PRUNED || VWIN;
    constexpr int LDVN = HD + 16; // V row stride in the natural layout (as LDK)
    constexpr int KBUF = AT_KT * LDK, VBUF = DMA ? AT_KT * LDVN : HD * LDV;
    constexpr int SM_KV = 2 * (KBUF + VBUF); // double-buffered key/value tiles
    constexpr int SM_O = QB * LDO;
    constexpr int SM = SM_KV > SM_O ? SM_KV : SM_O;
    extern __shared__ __attribute__((aligned(16))) unsigned char at_smem[];
    f16 *smem = reinterpret_cast<f16 *>(at_smem);
    static_assert(SM * 2 <= 160 * 1024, "LDS budget");

    const int bh = b * a.nhead + h;

    int row0, len, rows_alloc; // first row, valid rows, rows that exist for this sequence
    if (a.cu_seqlens) {
        row0 = a.cu_seqlens[b];
        len = a.cu_seqlens[b + 1] - row0;
        rows_alloc = len;
    } else {
        row0 = b * a.seq_len;
        len = a.seq_lens ? a.seq_lens[b] : a.seq_len;
        rows_alloc = a.seq_len;
    }
    len = min(max(len, 0), a.seq_len);
    const int q0 = qb * QB;
    if (q0 >= rows_alloc)
        return;

    int qc0 = h * HDK, nqk = HD, vc0 = h * HD, nv = HD;
    // head width of the data (HD unless the launcher says otherwise: heads of 48,
    // 80, 96 ... columns run as ragged heads of the next built width)
    const int hw = (PRUNED && !VWIN && a.head_width) ? a.head_width : HD;
    if (PRUNED && !VWIN && a.head_width) {
        qc0 = vc0 = h * hw;
        nqk = nv = hw;
    }
    if (PRUNED && !VWIN && a.qk_width) {
        qc0 = h * a.qk_width;
        nqk = a.qk_width;
    }
    if (PRUNED) {
        if (a.qk_head_ptr) {
            qc0 = a.qk_head_ptr[h];
            nqk = min(a.qk_head_ptr[h + 1] - qc0, HD);
        }
        if (a.v_head_ptr) {
            vc0 = a.v_head_ptr[h];
            nv = min(a.v_head_ptr[h + 1] - vc0, HD);
        }
    }
    // value window: vskip columns of a neighbouring head in front of the head's own nv
    int vskip = 0;
    if (VWIN) {
        // The window starts at the head's first column rounded down to 8, and never
        // beyond ldv - 8: a head that keeps no columns and sits at the very end
        // (v_head_ptr[h] == ldv) would otherwise start its window behind the row,
        // and the clamp of the staging offsets below (ldv - 8 - vc0) would go
        // negative.  The launcher guarantees ldv >= 8.
        const int w0 = min(vc0 & ~7, a.ldv - 8);
        vskip = vc0 - w0;
        vc0 = w0;
        nv += vskip; // columns of the window up to the head's last one
    }

    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lane = tid & 63;
    const int c16 = lane & 15;
    const int g4 = lane >> 4;
    f16 *obase = a.out + (size_t)row0 * a.ldo + h * hw;
    const f16x8 zero8 = f16x8{0, 0, 0, 0, 0, 0, 0, 0};

    if (q0 < len) {
        // ---- Q fragments (B operand of S^T), scaled in half like the reference
        f16x8 qf[QS][DK];
        const f16 sc = (f16)a.scale;
#pragma unroll
        for (int qs = 0; qs < QS; qs++) {
            const int q = q0 + (wave * QS + qs) * 16 + c16;
#pragma unroll
            for (int s = 0; s < DK; s++) {
                f16x8 v = zero8;
                if (!SHAREDQK && q < len) {
                    const f16 *qrow = a.Q + (size_t)(row0 + q) * a.ldq + qc0;
                    if (PRUNED && !VWIN)
                        v = load8_guard(qrow, s * 32 + g4 * 8, nqk);
                    else
                        v = *reinterpret_cast<const f16x8 *>(qrow + s * 32 + g4 * 8);
                }
                qf[qs][s] = v * sc;
            }
        }

        f32x4 ot[DV][QS];
        float m_run[QS];
        // What the key-tile loop needs of m_run in every tile, kept as state and touched only where a
        // maximum is raised (after the first tiles: almost never): the start vector of the score
        // products, four copies of -m (zero while the row has no maximum yet), and the amount a
        // tile's maximum has to exceed before the row's is raised (-inf until then, 8 binades after).
        // Only the plain form keeps them (there they save a dozen vector instructions per tile); with
        // mask handling they would be ten registers too many for three waves per SIMD, and the masked
        // forms work both out from m_run in every tile.
        constexpr bool KEEP_START = PLAIN;
        f32x4 neg_m4[QS];
        float raise_over[QS];
        f32x4 l_acc[QS]; // row sums of P, accumulated by the matrix unit (all 16 rows of the tile equal)
#pragma unroll
        for (int qs = 0; qs < QS; qs++) {
            m_run[qs] = -INFINITY;
            neg_m4[qs] = f32x4{-0.f, -0.f, -0.f, -0.f};
            raise_over[qs] = -INFINITY;
            l_acc[qs] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int d = 0; d < DV; d++)
                ot[d][qs] = f32x4{0.f, 0.f, 0.f, 0.f};
        }
        const bool mask_vec = a.mask && ((a.seq_len & 3) == 0) &&
                              ((reinterpret_cast<uintptr_t>(a.mask) & 7u) == 0);
        const bool qk_vec = SHAREDQK && ((a.seq_len & 3) == 0) &&
                            ((reinterpret_cast<uintptr_t>(a.QK) & 7u) == 0);
        const bool qk_vec16 = qk_vec && ((a.seq_len & 7) == 0) && ((reinterpret_cast<uintptr_t>(a.QK) & 15u) == 0);
        const float ls = a.log2_scale;

        // ---- key/value tile staging: global -> registers -> LDS.  The
        // registers of tile t+1 are in flight while tile t is being consumed.
        constexpr int CPR = HD / 8;                                        // 16-byte chunks per K row
        constexpr int NKL = (AT_KT * CPR + AT_THREADS - 1) / AT_THREADS;   // K chunks per thread
        constexpr int DQ = HD / 4;                                         // 4-wide column groups of V
        constexpr int NVW = ((AT_KT / 4) * DQ + AT_THREADS - 1) / AT_THREADS; // V 4x4 blocks per thread
        f16x8 kreg[NKL];
        f16x4 vreg[NVW][4];
        // FULL: every key of the tile is valid, so no per-lane bounds checks
        auto load_tile = [&](int kb, auto full_c) {
            constexpr bool FULL = decltype(full_c)::value;
            if (!SHAREDQK) {
#pragma unroll
                for (int i = 0; i < NKL; i++) {
                    const int idx = tid + i * AT_THREADS;
                    const int key = idx / CPR, dc = idx % CPR;
                    f16x8 v = zero8;
                    if ((AT_KT * CPR % AT_THREADS == 0 || idx < AT_KT * CPR) && (FULL || kb + key < len)) {
                        const f16 *krow = a.K + (size_t)(row0 + kb + key) * a.ldq + qc0;
                        if (PRUNED)
                            v = load8_guard(krow, dc * 8, nqk);
                        else
                            v = *reinterpret_cast<const f16x8 *>(krow + dc * 8);
                    }
                    kreg[i] = v;
                }
            }
#pragma unroll
            for (int i = 0; i < NVW; i++) {
                const int w = tid + i * AT_THREADS;
                const int dq = w % DQ, kq = w / DQ;
#pragma unroll
                for (int kk = 0; kk < 4; kk++) {
                    const int key = kb + kq * 4 + kk;
                    f16x4 v = f16x4{0, 0, 0, 0};
                    if (((AT_KT / 4) * DQ % AT_THREADS == 0 || w < (AT_KT / 4) * DQ) &&
                        (FULL || key < len)) { // rows at or beyond len read as zero
                        const f16 *vrow = a.V + (size_t)(row0 + key) * a.ldv + vc0;
                        if (PRUNED) {
                            v = load4_guard(vrow, dq * 4, nv);
                        } else {
                            v = *reinterpret_cast<const f16x4 *>(vrow + dq * 4);
                        }
                    }
                    vreg[i][kk] = v;
                }
            }
        };
        auto store_tile = [&](int buf) {
            f16 *ks = smem + buf * (KBUF + VBUF);
            f16 *vt = ks + KBUF;
            if (!SHAREDQK) {
#pragma unroll
                for (int i = 0; i < NKL; i++) {
                    const int idx = tid + i * AT_THREADS;
                    const int key = idx / CPR, dc = idx % CPR;
                    if (AT_KT * CPR % AT_THREADS == 0 || idx < AT_KT * CPR)
                        *reinterpret_cast<f16x8 *>(ks + key * LDK + dc * 8) = kreg[i];
                }
            }
#pragma unroll
            for (int i = 0; i < NVW; i++) { // V goes in transposed: [d][key]
                const int w = tid + i * AT_THREADS;
                const int dq = w % DQ, kq = w / DQ;
                if ((AT_KT / 4) * DQ % AT_THREADS == 0 || w < (AT_KT / 4) * DQ) {
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        const f16x4 t = f16x4{vreg[i][0][e], vreg[i][1][e], vreg[i][2][e], vreg[i][3][e]};
                        *reinterpret_cast<f16x4 *>(vt + (dq * 4 + e) * LDV + kq * 4) = t;
                    }
                }
            }
        };
        // DMA staging of one tile: every instruction moves 64 x 16 bytes to 1 KB
        // of consecutive LDS, so a lane's LDS position decides which (row,
        // column) it fetches; lanes that land in the row padding fetch the
        // row's first bytes.  Rows at or beyond len re-read the last valid row
        // (their scores are masked to -inf / their P is 0).
        // For a tile whose 64 keys all exist, a lane's source is "tile base + an
        // offset that never changes": the offsets are worked out once (byte
        // offsets in 32 bits, relative to the first row of the tile in K or V)
        // and an instruction then costs no address arithmetic in the vector ALU -
        // it was a quarter of the loop's vector instructions.
        constexpr int DMA_ROWBK = LDK * 2, DMA_ROWBV = LDVN * 2; // LDS bytes per row
        constexpr int DMA_NK = (DMA && !SHAREDQK) ? AT_KT * DMA_ROWBK / 1024 : 0;
        constexpr int DMA_NV = DMA ? AT_KT * DMA_ROWBV / 1024 : 0;
        constexpr int DMA_NTOT = DMA_NK + DMA_NV;
        constexpr int DMA_PW = DMA ? (DMA_NTOT + AT_WAVES - 1) / AT_WAVES : 1; // instructions per wave
        unsigned dma_off[DMA_PW];
        if (DMA) {
#pragma unroll
            for (int j = 0; j < DMA_PW; j++) {
                const int i = j * AT_WAVES + wave;
                const bool isv = i >= DMA_NK;
                const int ii = isv ? i - DMA_NK : i;
                const int p = ii * 1024 + lane * 16;
                const int rowb = isv ? DMA_ROWBV : DMA_ROWBK;
                const int row = p / rowb, cb = p - row * rowb;
                int col = cb < (isv ? HD : HDK) * 2 ? (cb >> 1) : 0;
                if (VWIN && isv) // all 80 columns of a window row are data; pieces past the row pitch re-read its last one
                    col = min(cb >> 1, a.ldv - 8 - vc0);
                dma_off[j] = (unsigned)((row * (isv ? a.ldv : a.ldq) + col) * 2);
            }
        }
        auto dma_tile = [&](int kb, int buf) {
            static_assert(!DMA || (AT_KT * DMA_ROWBK % 1024 == 0 && AT_KT * DMA_ROWBV % 1024 == 0),
                          "a tile is a whole number of DMA instructions");
            f16 *ks = smem + buf * (KBUF + VBUF);
            f16 *vs = ks + KBUF;
            if (PLAIN || kb + AT_KT <= len) { // (wave-uniform; always so in the plain form)
                const char *kbase = reinterpret_cast<const char *>(a.K + (size_t)(row0 + kb) * a.ldq + qc0);
                const char *vbase = reinterpret_cast<const char *>(a.V + (size_t)(row0 + kb) * a.ldv + vc0);
#pragma unroll
                for (int j = 0; j < DMA_PW; j++) {
                    const int i = j * AT_WAVES + wave;
                    if (DMA_NTOT % AT_WAVES != 0 && i >= DMA_NTOT)
                        break;
                    const bool isv = i >= DMA_NK;
                    const int ii = isv ? i - DMA_NK : i;
                    // (kept opaque in place: otherwise the offsets are folded into 64-bit vector
                    // addresses again, one 64-bit add per instruction and tile)
                    asm("" : "+v"(dma_off[j]));
                    load_lds16((isv ? vbase : kbase) + dma_off[j], (isv ? vs : ks) + ii * 512);
                }
                return;
            }
#pragma unroll
            for (int i0 = 0; i0 < DMA_NTOT; i0 += AT_WAVES) {
                const int i = i0 + wave;
                if (DMA_NTOT % AT_WAVES != 0 && i >= DMA_NTOT)
                    break;
                const bool isv = i >= DMA_NK;
                const int ii = isv ? i - DMA_NK : i;
                const int p = ii * 1024 + lane * 16;
                const int rowb = isv ? DMA_ROWBV : DMA_ROWBK;
                const int row = p / rowb, cb = p - row * rowb;
                const int rr = min(kb + row, len - 1);
                int col = cb < (isv ? HD : HDK) * 2 ? (cb >> 1) : 0;
                if (VWIN && isv)
                    col = min(cb >> 1, a.ldv - 8 - vc0);
                const f16 *src = isv ? a.V + (size_t)(row0 + rr) * a.ldv + vc0 + col
                                     : a.K + (size_t)(row0 + rr) * a.ldq + qc0 + col;
                load_lds16(src, (isv ? vs : ks) + ii * 512);
            }
        };
        typedef std::integral_constant<bool, true> yes_t;
        typedef std::integral_constant<bool, false> no_t;

        const int nt = (len + AT_KT - 1) / AT_KT;
        // all of this wave's query rows valid?  (wave-uniform)
        const bool wave_rows_ok = q0 + (wave + 1) * QS * 16 <= len;
        // value window: the output column (within the head) of every window column, -1 for the columns of
        // other heads; kept behind the tile buffers for the epilogue
        int *wcol = reinterpret_cast<int *>(at_smem + SM * 2);
        if (VWIN && tid < DV * 16) {
            int c = -1;
            if (tid >= vskip && tid < nv)
                c = (a.v_col_id ? a.v_col_id[vc0 + tid] : vc0 + tid) - h * HD;
            wcol[tid] = (c >= 0 && c < HD) ? c : -1;
        }
        if (DMA) {
            dma_tile(0, 0);
            __builtin_amdgcn_s_waitcnt(0x0F70); // vmcnt(0)
        } else {
            if (AT_KT <= len)
                load_tile(0, yes_t{});
            else
                load_tile(0, no_t{});
            store_tile(0);
        }
        __syncthreads();

        // Does key tile t hold a non-zero mask element for this wave's query
        // rows?  (wave-uniform; all-zero tiles skip the mask loads and adds,
        // which changes no result bit: s + 0 == s.)  The summary words of the
        // first 64 tiles are fetched once, up front; longer sequences do not
        // use the summary.
        unsigned mw0 = 0xFFFFFFFFu, mw1 = 0xFFFFFFFFu;
        if (a.msum && a.msum_words <= 2) {
            unsigned w0 = 0, w1 = 0;
#pragma unroll
            for (int qs = 0; qs < QS; qs++) {
                const int g = (q0 + (wave * QS + qs) * 16) >> 4;
                if (g * 16 < a.seq_len) {
                    w0 |= a.msum[(size_t)g * a.msum_words];
                    if (a.msum_words > 1)
                        w1 |= a.msum[(size_t)g * a.msum_words + 1];
                }
            }
            mw0 = __builtin_amdgcn_readfirstlane(w0);
            mw1 = __builtin_amdgcn_readfirstlane(w1);
        }
        auto tile_has_mask = [&](int t) -> bool {
            return t >= 64 || (((t < 32 ? mw0 : mw1) >> (t & 31)) & 1u);
        };

        // Additive mask values of one tile, in the score layout.  They are
        // requested one tile ahead (right after the previous tile consumed
        // its own) so the L2 latency is covered by a whole tile of work.
        f16x4 mk[QS][4];
        // Whole mask rows of a tile are 128 bytes, one cache line.  Where rows are 16-byte aligned a full tile's
        // values come as two 16-byte loads per lane that together read each of the 16 lines once (lane (row, g)
        // takes keys 16g .. 16g+15); the score layout wants keys 16k + 4g .. +3 for k = 0..3, i.e. the 4 x 4
        // transpose of the 8-byte pieces across the row's four lanes, done with row swaps when the values are
        // consumed (mk_blocked says that it is still due).  Four 8-byte loads per lane, the direct form, touch
        // every line four times from four requests: with twelve waves per CU the lines do not survive in L1
        // between them, and a dense mask then costs more L2 traffic than K and V together.
        const bool mask_vec16 = mask_vec && ((a.seq_len & 7) == 0) && ((reinterpret_cast<uintptr_t>(a.mask) & 15u) == 0);
        bool mk_blocked = false;
        auto load_mask = [&](int kb, auto fast_c) {
            constexpr bool FAST = decltype(fast_c)::value;
            mk_blocked = FAST && mask_vec16;
            if (FAST && mask_vec16) {
#pragma unroll
                for (int qs = 0; qs < QS; qs++) {
                    const int q = q0 + (wave * QS + qs) * 16 + c16;
                    const f16 *mrow = a.mask + (size_t)q * a.seq_len + kb + g4 * 16;
                    const f16x8 l0 = *reinterpret_cast<const f16x8 *>(mrow);
                    const f16x8 l1 = *reinterpret_cast<const f16x8 *>(mrow + 8);
                    mk[qs][0] = f16x4{l0[0], l0[1], l0[2], l0[3]};
                    mk[qs][1] = f16x4{l0[4], l0[5], l0[6], l0[7]};
                    mk[qs][2] = f16x4{l1[0], l1[1], l1[2], l1[3]};
                    mk[qs][3] = f16x4{l1[4], l1[5], l1[6], l1[7]};
                }
                return;
            }
#pragma unroll
            for (int qs = 0; qs < QS; qs++) {
                const int q = q0 + (wave * QS + qs) * 16 + c16;
#pragma unroll
                for (int ksub = 0; ksub < 4; ksub++) {
                    const int key = kb + ksub * 16 + g4 * 4;
                    const f16 *mrow = a.mask + (size_t)q * a.seq_len + key;
                    f16x4 v = f16x4{0, 0, 0, 0};
                    if (FAST) {
                        v = *reinterpret_cast<const f16x4 *>(mrow);
                    } else if (q < len) {
                        if (mask_vec && key + 3 < len) {
                            v = *reinterpret_cast<const f16x4 *>(mrow);
                        } else {
#pragma unroll
                            for (int r = 0; r < 4; r++)
                                if (key + r < len)
                                    v[r] = mrow[r];
                        }
                    }
                    mk[qs][ksub] = v;
                }
            }
        };
        const bool vec_ok = (!a.mask || mask_vec) && (!SHAREDQK || qk_vec);
        auto fast_tile = [&](int kb) { return kb + AT_KT <= len && wave_rows_ok && vec_ok; };
        bool has_mask_cur = !PLAIN && a.mask && tile_has_mask(0);
        if (has_mask_cur) {
            if (fast_tile(0))
                load_mask(0, yes_t{});
            else
                load_mask(0, no_t{});
        }

        // One key tile.  FAST: all 64 keys and all of the wave's query rows are
        // valid and the vector paths apply, so the body has no per-lane
        // predicates at all.
        bool has_mask_next = false;
        // (FAST and MASKED are wave-uniform run-time flags, not template
        // parameters: four inlined copies of this body made the register
        // allocator keep a second copy of every accumulator - 223 VGPRs against
        // 122 for one copy - which halved the waves per SIMD)
        auto tile_body = [&](int kb, const f16 *ks, const f16 *vt, const bool FAST, const bool MASKED) {
            // MASKED: this tile's mask values are in mk
            __builtin_amdgcn_s_setprio(AT_PRIO);
            // ---- scores, transposed: st[ksub][qs][r] = S[q = c16][key = 16 ksub + 4 g4 + r],
            // MINUS the row's running maximum: the matrix unit starts from -m
            // instead of zero, which costs nothing there and saves the vector
            // ALU one subtraction per score
            f32x4 st[4][QS];
            float m_ref[QS];
            f32x4 nm4[QS];
#pragma unroll
            for (int qs = 0; qs < QS; qs++) {
                if (KEEP_START) {
                    nm4[qs] = neg_m4[qs];
                    m_ref[qs] = -nm4[qs][0]; // (only used where a maximum is raised)
                } else {
                    m_ref[qs] = (m_run[qs] == -INFINITY) ? 0.f : m_run[qs];
                    nm4[qs] = f32x4{-m_ref[qs], -m_ref[qs], -m_ref[qs], -m_ref[qs]};
                }
            }
            if (!SHAREDQK) {
                // K fragments are read one 16-key subtile ahead of the MFMAs that
                // use them (two subtiles' worth of registers instead of four)
                f16x8 kfr[2][DK];
#pragma unroll
                for (int s = 0; s < DK; s++)
                    kfr[0][s] = *reinterpret_cast<const f16x8 *>(ks + c16 * LDK + s * 32 + g4 * 8);
#pragma unroll
                for (int ksub = 0; ksub < 4; ksub++) {
                    if (ksub + 1 < 4) {
#pragma unroll
                        for (int s = 0; s < DK; s++)
                            kfr[(ksub + 1) & 1][s] = *reinterpret_cast<const f16x8 *>(
                                ks + ((ksub + 1) * 16 + c16) * LDK + s * 32 + g4 * 8);
                    }
                    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                    for (int s = 0; s < DK; s++)
#pragma unroll
                        for (int qs = 0; qs < QS; qs++) // (the first step reads -m as its C operand: no copies)
                            st[ksub][qs] = mfma16x16x32(kfr[ksub & 1][s], qf[qs][s], s == 0 ? nm4[qs] : st[ksub][qs]);
                }
            } else if (FAST && qk_vec16) {
                // stored scores of a full tile: line-wise like the mask (128 bytes per query row and tile)
#pragma unroll
                for (int qs = 0; qs < QS; qs++) {
                    const int q = q0 + (wave * QS + qs) * 16 + c16;
                    const f16 *src = a.QK + ((size_t)bh * a.seq_len + q) * a.seq_len + kb + g4 * 16;
                    const f16x8 l0 = *reinterpret_cast<const f16x8 *>(src);
                    const f16x8 l1 = *reinterpret_cast<const f16x8 *>(src + 8);
                    f16x4 pc[4] = {f16x4{l0[0], l0[1], l0[2], l0[3]}, f16x4{l0[4], l0[5], l0[6], l0[7]},
                                   f16x4{l1[0], l1[1], l1[2], l1[3]}, f16x4{l1[4], l1[5], l1[6], l1[7]}};
                    transpose_pieces_4x4(pc);
#pragma unroll
                    for (int ksub = 0; ksub < 4; ksub++)
                        st[ksub][qs] = __builtin_convertvector(pc[ksub], f32x4) - m_ref[qs];
                }
            } else {
#pragma unroll
                for (int qs = 0; qs < QS; qs++) {
                    const int q = q0 + (wave * QS + qs) * 16 + c16;
#pragma unroll
                    for (int ksub = 0; ksub < 4; ksub++) {
                        const int key = kb + ksub * 16 + g4 * 4;
                        f32x4 v = f32x4{0.f, 0.f, 0.f, 0.f};
                        const f16 *src = a.QK + ((size_t)bh * a.seq_len + q) * a.seq_len + key;
                        if (FAST || (q < len && qk_vec && key + 3 < len)) {
                            const f16x4 t4 = *reinterpret_cast<const f16x4 *>(src);
#pragma unroll
                            for (int r = 0; r < 4; r++)
                                v[r] = (float)t4[r];
                        } else if (q < len) {
#pragma unroll
                            for (int r = 0; r < 4; r++)
                                if (key + r < len)
                                    v[r] = (float)src[r];
                        }
                        st[ksub][qs] = v - m_ref[qs];
                    }
                }
            }

            __builtin_amdgcn_s_setprio(0);
            // ---- mask, online softmax, pack P as the B operand.  The running
            // maximum is only raised when a row's new maximum exceeds it by
            // more than 8 binades (P then stays <= 256, exact enough in half),
            // so after the first tiles the accumulator rescale is skipped.
            f16x8 pf[QS][2];
            if (MASKED && mk_blocked) { // the line-wise loads hold key blocks per lane: into the score layout
#pragma unroll
                for (int qs = 0; qs < QS; qs++)
                    transpose_pieces_4x4(mk[qs]);
            }
            if (MASKED) {
                // (the multiplier is exactly 1.0 but opaque to the optimiser,
                // which would otherwise turn the fused form back into a
                // conversion and an add)
                float one = 1.0f;
                asm("" : "+s"(one));
#pragma unroll
                for (int qs = 0; qs < QS; qs++)
#pragma unroll
                    for (int ksub = 0; ksub < 4; ksub++)
#pragma unroll
                        for (int r = 0; r < 4; r++)
                            // (as a fused multiply-add by one: the mixed-precision
                            // form takes the half operand directly, no conversion)
                            st[ksub][qs][r] = __builtin_fmaf((float)mk[qs][ksub][r], one, st[ksub][qs][r]);
            }
            if (!PLAIN && a.mask) { // next tile's mask
                has_mask_next = kb + AT_KT < len && tile_has_mask((kb + AT_KT) / AT_KT);
                if (has_mask_next) {
                    if (fast_tile(kb + AT_KT))
                        load_mask(kb + AT_KT, yes_t{});
                    else
                        load_mask(kb + AT_KT, no_t{});
                }
            }
            // the lane's part of each row maximum (of s - m_ref); the row's other three
            // parts only matter when some row of the wave has to raise its maximum
            float pmx[QS];
            bool live = false;
#pragma unroll
            for (int qs = 0; qs < QS; qs++) {
                if (!FAST) {
#pragma unroll
                    for (int ksub = 0; ksub < 4; ksub++)
#pragma unroll
                        for (int r = 0; r < 4; r++)
                            if (kb + ksub * 16 + g4 * 4 + r >= len)
                                st[ksub][qs][r] = -INFINITY;
                }
                float mx = -INFINITY;
#pragma unroll
                for (int ksub = 0; ksub < 4; ksub++) {
                    mx = fmaxf(fmaxf(mx, st[ksub][qs][0]), st[ksub][qs][1]);
                    mx = fmaxf(fmaxf(mx, st[ksub][qs][2]), st[ksub][qs][3]);
                }
                pmx[qs] = mx;
                // does this tile add anything to the row?  Not if every score is 160 binades or more under a
                // maximum the row already has: every exp2 is then exactly zero in fp32 (so is P, and the sums
                // and the output do not change).
                live = live || m_run[qs] == -INFINITY || !(mx * ls < -160.0f);
            }
            // A tile that is dead for every row of the wave - the keys behind a padding mask - ends here: no
            // exponentials, no second product (wave-uniform; same bits as going through with P = 0).
            if (!PLAIN && __builtin_amdgcn_ballot_w64(live) == 0)
                return;
#pragma unroll
            for (int qs = 0; qs < QS; qs++) {
                float mx = pmx[qs];
                // (a row without a maximum yet takes its first finite one: raise_over is -inf then)
                auto raises = [&](float v) {
                    if (KEEP_START)
                        return v * ls > raise_over[qs];
                    return (m_run[qs] == -INFINITY) ? (v > -INFINITY) : (v * ls > 8.0f);
                };
                const bool up_lane = raises(mx);
                if (__builtin_amdgcn_ballot_w64(up_lane) != 0) {
                    mx = xor_max_16_32(mx);
                    const bool up = raises(mx);
                    const float m_new = up ? mx + m_ref[qs] : m_run[qs];
                    const float m_fin = (m_new == -INFINITY) ? 0.f : m_new;
                    const float alpha = __builtin_amdgcn_exp2f((m_run[qs] - m_fin) * ls); // 1 where unchanged
                    const float shift = m_fin - m_ref[qs];                                // 0 where unchanged
                    m_run[qs] = m_new;
                    if (KEEP_START) {
                        neg_m4[qs] = f32x4{-m_fin, -m_fin, -m_fin, -m_fin};
                        raise_over[qs] = (m_new == -INFINITY) ? -INFINITY : 8.0f;
                    }
                    l_acc[qs] *= alpha;
#pragma unroll
                    for (int d = 0; d < DV; d++)
                        ot[d][qs] *= alpha;
#pragma unroll
                    for (int ksub = 0; ksub < 4; ksub++)
                        st[ksub][qs] -= shift;
                }
                if (ls != 1.0f) { // (wave-uniform; base-2 softmax needs no multiplication at all)
#pragma unroll
                    for (int ksub = 0; ksub < 4; ksub++)
                        st[ksub][qs] *= ls;
                }
                f16x2 ph[8];
#pragma unroll
                for (int ksub = 0; ksub < 4; ksub++)
#pragma unroll
                    for (int r2 = 0; r2 < 2; r2++) {
                        const float p0 = __builtin_amdgcn_exp2f(st[ksub][qs][2 * r2]);
                        const float p1 = __builtin_amdgcn_exp2f(st[ksub][qs][2 * r2 + 1]);
                        typedef float f32x2 __attribute__((ext_vector_type(2)));
                        ph[ksub * 2 + r2] = __builtin_convertvector(f32x2{p0, p1}, f16x2);
                    }
#pragma unroll
                for (int kk = 0; kk < 2; kk++)
                    pf[qs][kk] = f16x8{ph[kk * 4 + 0][0], ph[kk * 4 + 0][1], ph[kk * 4 + 1][0], ph[kk * 4 + 1][1],
                                       ph[kk * 4 + 2][0], ph[kk * 4 + 2][1], ph[kk * 4 + 3][0], ph[kk * 4 + 3][1]};
            }

            __builtin_amdgcn_s_setprio(AT_PRIO);
            // ---- O^T += V^T P^T, V^T fragments read one 16-column subtile ahead
            {
                auto load_v = [&](int d, f16x8 (&dst)[2]) {
#pragma unroll
                    for (int kk = 0; kk < 2; kk++) {
                        f16x4 v0, v1;
                        if (DMA) {
                            // natural layout [key][d]: the transpose read hands lane
                            // c of a 16-lane group the 4 consecutive keys of column
                            // d0+c when lane i of the group addresses row i/4,
                            // columns 4(i%4)..+3.  The B operand's 8 k-slots are
                            // keys 4g..4g+3 of subtile 2kk and of subtile 2kk+1.
                            typedef short s16x4 __attribute__((ext_vector_type(4)));
                            typedef __attribute__((address_space(3))) s16x4 *lds4;
                            const f16 *vrow = vt + (kk * 32 + g4 * 4 + (c16 >> 2)) * LDVN + d * 16 + (c16 & 3) * 4;
                            v0 = __builtin_bit_cast(f16x4, __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds4)vrow));
                            v1 = __builtin_bit_cast(f16x4, __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds4)(vrow + 16 * LDVN)));
                        } else {
                            const f16 *vrow = vt + (d * 16 + c16) * LDV + kk * 32 + g4 * 4;
                            v0 = *reinterpret_cast<const f16x4 *>(vrow);
                            v1 = *reinterpret_cast<const f16x4 *>(vrow + 16);
                        }
                        dst[kk] = f16x8{v0[0], v0[1], v0[2], v0[3], v1[0], v1[1], v1[2], v1[3]};
                    }
                };
                f16x8 vfr[2][2];
                load_v(0, vfr[0]);
#pragma unroll
                for (int d = 0; d < DV; d++) {
                    // (a head that keeps nv < 64 value columns has nothing in the
                    // subtiles from ceil(nv / 16) on: wave-uniform skip)
                    if (PRUNED && d * 16 >= nv)
                        break;
                    if (d + 1 < DV)
                        load_v(d + 1, vfr[(d + 1) & 1]);
                    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                    for (int kk = 0; kk < 2; kk++)
#pragma unroll
                        for (int qs = 0; qs < QS; qs++)
                            ot[d][qs] = mfma16x16x32(vfr[d & 1][kk], pf[qs][kk], ot[d][qs]);
                }
                // the softmax denominators: ones^T P^T sums a query's 64
                // probabilities (as rounded to half for the product above)
                // without any vector adds or cross-lane steps
                const f16x8 ones8 = f16x8{1, 1, 1, 1, 1, 1, 1, 1};
#pragma unroll
                for (int kk = 0; kk < 2; kk++)
#pragma unroll
                    for (int qs = 0; qs < QS; qs++)
                        l_acc[qs] = mfma16x16x32(ones8, pf[qs][kk], l_acc[qs]);
            }
            __builtin_amdgcn_s_setprio(0);
        };

        for (int t = 0; t < nt; t++) {
            const int kb = t * AT_KT;
            const f16 *ks = smem + (t & 1) * (KBUF + VBUF);
            const f16 *vt = ks + KBUF;
            const bool more = t + 1 < nt;
            // tile t+1 goes into the other buffer (last read in iteration t-1,
            // which every wave left before the previous barrier) while tile t is
            // consumed: by DMA straight away, or through registers that are
            // stored after the tile body
            if (more) {
                if (DMA)
                    dma_tile(kb + AT_KT, (t + 1) & 1);
                else if (kb + 2 * AT_KT <= len)
                    load_tile(kb + AT_KT, yes_t{});
                else
                    load_tile(kb + AT_KT, no_t{});
            }
            if constexpr (PLAIN)
                tile_body(kb, ks, vt, true, false);
            else
                tile_body(kb, ks, vt, fast_tile(kb), has_mask_cur);
            has_mask_cur = has_mask_next;
            if (more) {
                if (DMA)
                    __builtin_amdgcn_s_waitcnt(0x0F70); // vmcnt(0): this wave's part of tile t+1 has landed
                else
                    store_tile((t + 1) & 1);
            }
            __syncthreads();
        }

        // ---- normalise and stage the output block in LDS (all waves are past
        // the loop's final barrier, so the tile buffers are free)
        f16 *os = smem;
        if (PRUNED) { // columns that no kept V column maps to must read as zero
            for (int i = tid; i < SM_O / 8; i += AT_THREADS)
                reinterpret_cast<f16x8 *>(os)[i] = zero8;
            __syncthreads();
        }
#pragma unroll
        for (int qs = 0; qs < QS; qs++) {
            const float l = l_acc[qs][0];
            const float inv = l > 0.f ? 1.0f / l : 0.f;
            const int ql = (wave * QS + qs) * 16 + c16;
#pragma unroll
            for (int d = 0; d < DV; d++) {
                f16x4 o;
#pragma unroll
                for (int r = 0; r < 4; r++)
                    o[r] = (f16)(ot[d][qs][r] * inv);
                if (VWIN) {
                    typedef int i32x4 __attribute__((ext_vector_type(4)));
                    const i32x4 c4 = *reinterpret_cast<const i32x4 *>(wcol + d * 16 + g4 * 4);
#pragma unroll
                    for (int r = 0; r < 4; r++)
                        if (c4[r] >= 0)
                            os[ql * LDO + c4[r]] = o[r];
                } else if (PRUNED) {
#pragma unroll
                    for (int r = 0; r < 4; r++) {
                        const int j = d * 16 + g4 * 4 + r;
                        if (j < nv) {
                            const int col = (a.v_col_id ? a.v_col_id[vc0 + j] : vc0 + j) - h * hw;
                            if (col >= 0 && col < hw)
                                os[ql * LDO + col] = o[r];
                        }
                    }
                } else {
                    *reinterpret_cast<f16x4 *>(os + ql * LDO + d * 16 + g4 * 4) = o;
                }
            }
        }
        __syncthreads();
        for (int idx = tid; idx < QB * CPR; idx += AT_THREADS) {
            const int ql = idx / CPR, dc = idx % CPR;
            const int q = q0 + ql;
            if (q < rows_alloc && dc * 8 < hw) {
                f16x8 v = zero8;
                if (q < len)
                    v = *reinterpret_cast<const f16x8 *>(os + ql * LDO + dc * 8);
                *reinterpret_cast<f16x8 *>(obase + (size_t)q * a.ldo + dc * 8) = v;
            }
        }
    } else {
        // whole query block is padding: rows exist (padded layout) and read as zero
        constexpr int CPR = HD / 8;
        for (int idx = tid; idx < QB * CPR; idx += AT_THREADS) {
            const int ql = idx / CPR, dc = idx % CPR;
            const int q = q0 + ql;
            if (q < rows_alloc && dc * 8 < hw)
                *reinterpret_cast<f16x8 *>(obase + (size_t)q * a.ldo + dc * 8) = zero8;
        }
    }
}

template <int HD, int QS, int NW, bool PRUNED, bool SHAREDQK, bool PLAIN = false, int HDK = HD, bool VWIN = false>
__global__ void __launch_bounds__(NW * 64, (QS == 1 && HD <= 64) ? 4 : 2) attention_kernel(const AttnArgs a) {
    // Workgroup ids go round-robin over the 8 XCDs.  XCD x works on the
    // (batch, head) pairs x, x+8, x+16, ... in that order, all query blocks of a
    // pair together (they share its K and V in that XCD's L2): with sequences of
    // different lengths every XCD gets an even mix, and pairs keep their order.
    const int xcd = blockIdx.x & 7, rest = blockIdx.x >> 3; // rest < per_xcd = ceil(pairs / 8) * nqb
    const int qb = rest % a.nqb;
    const int bh = (rest / a.nqb) * 8 + xcd;
    if (bh >= a.nhead * a.batch)
        return;
    attention_block<HD, QS, NW, PRUNED, SHAREDQK, PLAIN, HDK, VWIN>(a, bh / a.nhead, bh % a.nhead, qb);
}

// Packed sequences of different lengths (cu_seqlens): a grid of one workgroup per
// (sequence, head, query block of the LONGEST sequence) is mostly workgroups that
// find nothing to do, and dispatching those costs as much as the work of a batch
// of short sequences.  Here the grid is what the chip holds at once and every
// workgroup walks its share of the blocks that exist: XCD x owns the (sequence,
// head) pairs x, x+8, ... as above, their query blocks in order form that XCD's
// list, and workgroup k of the W on the XCD takes blocks k, k+W, k+2W, ... .
// A block's position in the list is found from the running block count per
// sequence, which every wave keeps in registers (lane l: sequences l, l+64, ...;
// at most 64*AT_PX sequences).
constexpr int AT_PX = 4;
template <int HD, int QS, int NW>
__global__ void __launch_bounds__(NW * 64, (QS == 1 && HD <= 64) ? 4 : 2) attention_packed_kernel(const AttnArgs a) {
    constexpr int QB = NW * 16 * QS;
    const int lane = threadIdx.x & 63;
    const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3, W = gridDim.x >> 3;
    int px[AT_PX], nbv[AT_PX]; // blocks before sequence (l + 64 r) in this XCD's list; its query blocks
    int run = 0;
#pragma unroll
    for (int r = 0; r < AT_PX; r++) {
        const int s = lane + 64 * r;
        int nb = 0, v = 0;
        if (s < a.batch) {
            const int len = min(max(a.cu_seqlens[s + 1] - a.cu_seqlens[s], 0), a.seq_len);
            nb = (len + QB - 1) / QB;
            const int h0 = (xcd - s * a.nhead) & 7; // first head of the sequence whose pair lands on this XCD
            v = h0 < a.nhead ? nb * ((a.nhead - h0 + 7) >> 3) : 0;
        }
        int inc = v; // inclusive scan over the 64 lanes
#pragma unroll
        for (int d = 1; d < 64; d <<= 1) {
            const int t = __shfl_up(inc, d, 64);
            inc += lane >= d ? t : 0;
        }
        px[r] = s < a.batch ? run + inc - v : 0x7fffffff;
        nbv[r] = nb;
        run += __shfl(inc, 63, 64);
    }
    run = __builtin_amdgcn_readfirstlane(run);
    for (int i = slot; i < run; i += W) {
        // the sequence: the last one whose first block is at or before i (the counts never decrease, and a
        // sequence without blocks on this XCD shares its successor's count and is passed over)
        int cnt = 0;
#pragma unroll
        for (int r = 0; r < AT_PX; r++)
            cnt += __builtin_popcountll(__builtin_amdgcn_ballot_w64(px[r] <= i));
        const int b = cnt - 1; // (cnt >= 1: the first sequence's count is 0)
        int first = 0, nb = 1;
#pragma unroll
        for (int r = 0; r < AT_PX; r++)
            if ((b >> 6) == r) {
                first = __builtin_amdgcn_readlane(px[r], b & 63);
                nb = __builtin_amdgcn_readlane(nbv[r], b & 63);
            }
        const int rem = i - first;
        const int h = ((xcd - b * a.nhead) & 7) + 8 * (rem / max(nb, 1));
        if (nb <= 0 || rem < 0 || b >= a.batch || h >= a.nhead)
            continue; // (cannot happen with consistent counts; never index past the operands)
        attention_block<HD, QS, NW, false, false, false, HD, false>(a, b, h, rem % nb);
        __syncthreads(); // the block's output staging in LDS is read before the next block's tiles land there
    }
}

// scaled Q K^T written to memory, [(b*nhead+h)][q][k]; one wave per 64 queries x 64 keys (the K fragments are
// fetched once and used for four tiles of 16 queries), transposed product so a lane owns 4 consecutive keys of
// one query.  A query's 64 scores of the tile are 128 bytes, one cache line: the lane's four 8-byte pieces are
// transposed over the query's four lanes so that every lane stores 32 contiguous bytes and the four of them the
// whole line (element-wise 2-byte stores of the same values took 129 us for batch 16 x seq 512, six times the
// time of writing 100 MB).
template <int HD>
__global__ void __launch_bounds__(256)
qk_scores_kernel(f16 *__restrict__ QK, const f16 *__restrict__ Q, const f16 *__restrict__ K,
                 int seq_len, int d_model, int nhead, float scale) {
    constexpr int DK = HD / 32;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int lane = threadIdx.x & 63, c16 = lane & 15, g4 = lane >> 4;
    const int bh = blockIdx.z, h = bh % nhead, b = bh / nhead;
    const int qb0 = blockIdx.y * 64;
    const int k0 = (blockIdx.x * 4 + wave) * 64;
    if (k0 >= seq_len)
        return;
    const size_t row0 = (size_t)b * seq_len;
    f16x8 kf[4][DK];
#pragma unroll
    for (int ksub = 0; ksub < 4; ksub++) {
        const int key = k0 + ksub * 16 + c16;
#pragma unroll
        for (int s = 0; s < DK; s++) {
            kf[ksub][s] = f16x8{0, 0, 0, 0, 0, 0, 0, 0};
            if (key < seq_len)
                kf[ksub][s] = *reinterpret_cast<const f16x8 *>(K + (row0 + key) * d_model + h * HD + s * 32 + g4 * 8);
        }
    }
    // whole lines: all 64 keys exist and rows start on 16-byte boundaries (wave-uniform)
    const bool lines = k0 + 64 <= seq_len && (seq_len & 7) == 0 && (reinterpret_cast<uintptr_t>(QK) & 15u) == 0;
    for (int qt = 0; qt < 4; qt++) {
        if (qb0 + qt * 16 >= seq_len)
            break;
        const int q = qb0 + qt * 16 + c16;
        f16x8 qf[DK];
#pragma unroll
        for (int s = 0; s < DK; s++) {
            qf[s] = f16x8{0, 0, 0, 0, 0, 0, 0, 0};
            if (q < seq_len)
                qf[s] = *reinterpret_cast<const f16x8 *>(Q + (row0 + q) * d_model + h * HD + s * 32 + g4 * 8);
        }
        f16x4 pc[4]; // piece ksub: keys k0 + 16 ksub + 4 g4 .. + 3 of query q
#pragma unroll
        for (int ksub = 0; ksub < 4; ksub++) {
            f32x4 acc = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int s = 0; s < DK; s++)
                acc = mfma16x16x32(kf[ksub][s], qf[s], acc);
            pc[ksub] = __builtin_convertvector(acc * scale, f16x4);
        }
        f16 *qrow = QK + ((size_t)bh * seq_len + q) * seq_len + k0;
        if (lines) {
            transpose_pieces_4x4(pc); // piece j: keys k0 + 16 g4 + 4 j .. + 3
            if (q < seq_len) {
                *reinterpret_cast<f16x8 *>(qrow + g4 * 16) =
                    f16x8{pc[0][0], pc[0][1], pc[0][2], pc[0][3], pc[1][0], pc[1][1], pc[1][2], pc[1][3]};
                *reinterpret_cast<f16x8 *>(qrow + g4 * 16 + 8) =
                    f16x8{pc[2][0], pc[2][1], pc[2][2], pc[2][3], pc[3][0], pc[3][1], pc[3][2], pc[3][3]};
            }
        } else if (q < seq_len) {
#pragma unroll
            for (int ksub = 0; ksub < 4; ksub++)
#pragma unroll
                for (int r = 0; r < 4; r++)
                    if (k0 + ksub * 16 + g4 * 4 + r < seq_len)
                        qrow[ksub * 16 + g4 * 4 + r] = pc[ksub][r];
        }
    }
}

// LDS bytes of one workgroup (mirrors the constants inside the kernel)
template <int HD, int QS, int NW, bool PRUNED, int HDK = HD, bool VWIN = false> constexpr size_t attn_lds_bytes() {
    // (must agree with the kernel's KBUF / VBUF)
    constexpr int KV = 2 * (AT_KT * (HDK + 16) + ((PRUNED && !VWIN) ? HD * (AT_KT + 8) : AT_KT * (HD + 16)));
    constexpr int O = NW * 16 * QS * (HD + 8);
    return sizeof(f16) * (size_t)(KV > O ? KV : O) + (VWIN ? 5 * 16 * sizeof(int) : 0); // (+ the window's column table)
}

template <int HD, int QS, int NW, bool PRUNED, bool SHAREDQK, bool PLAIN = false, int HDK = HD, bool VWIN = false>
static void attn_launch_one(const AttnArgs &a, hipStream_t st) {
    constexpr size_t lds = attn_lds_bytes<HD, QS, NW, PRUNED, HDK, VWIN>();
    auto kern = attention_kernel<HD, QS, NW, PRUNED, SHAREDQK, PLAIN, HDK, VWIN>;
    if (lds > 64 * 1024) { // above the default dynamic-LDS limit: opt in once per kernel
        static bool done = false;
        if (!done) {
            (void)hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
            done = true;
        }
    }
    hipLaunchKernelGGL(kern, dim3(a.per_xcd * 8), dim3(NW * 64), lds, st, a);
}

// packed sequences: as many workgroups (4 waves x 16 query rows) as the chip holds at once, or fewer
template <int HD>
static void attn_launch_packed(const AttnArgs &a, hipStream_t st) {
    // (32 query rows per wave need 207 registers here, two waves per SIMD: 63 us against 48 us on a batch of
    // 64 sequences of 32..512 rows)
    constexpr size_t lds = attn_lds_bytes<HD, 1, 4, false>();
    auto kern = attention_packed_kernel<HD, 1, 4>;
    if (lds > 64 * 1024) {
        static bool done = false;
        if (!done) {
            (void)hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
            done = true;
        }
    }
    const long resident = (long)std::max(et_device_cu_count(), 1) * (HD <= 64 ? 4 : 2);
    const long wgs = std::min<long>(resident, a.total);
    hipLaunchKernelGGL(kern, dim3((unsigned)((wgs + 7) / 8 * 8)), dim3(256), lds, st, a);
}

// variant 0: 4 waves x 32 query rows; 1: 8 waves x 16 rows; 2: 4 waves x 16 rows
template <int HD, bool PRUNED, bool SHAREDQK, int HDK = HD>
static void attn_launch_variant(int variant, bool plain, const AttnArgs &a, hipStream_t st) {
    if constexpr (!PRUNED && !SHAREDQK) {
        if (plain) {
            if (variant == 0)
                attn_launch_one<HD, 2, 4, false, false, true, HDK>(a, st);
            else if (variant == 1)
                attn_launch_one<HD, 1, 8, false, false, true, HDK>(a, st);
            else
                attn_launch_one<HD, 1, 4, false, false, true, HDK>(a, st);
            return;
        }
    }
    if (variant == 0)
        attn_launch_one<HD, 2, 4, PRUNED, SHAREDQK, false, HDK>(a, st);
    else if (variant == 1)
        attn_launch_one<HD, 1, 8, PRUNED, SHAREDQK, false, HDK>(a, st);
    else
        attn_launch_one<HD, 1, 4, PRUNED, SHAREDQK, false, HDK>(a, st);
}

static int g_attn_variant = -1; // et_tuning_set("attn_variant"): -1 = automatic
static int g_attn_packed = 1;   // et_tuning_set("attn_packed"): 0 = packed sequences run one workgroup per possible query block
static int g_attn_vwin = 1;     // et_tuning_set("attn_vwin"): 0 = pruned attention always stages through registers

static float head_scale(int hd) {
    // half(sqrt(1/head_dim)), kernels/attention.cu:126
    return (float)(f16)sqrtf(1.0f / (float)hd);
}

// ---- mask summary: one bit per (16 query rows, 64-key tile) ----------------
// One workgroup of four waves per group of 16 rows, wave w takes the tiles w, w+4, ...; per tile a lane tests 16
// elements (row lane/4, keys 16*(lane%4)..+15: two 16-byte loads where rows are 16-byte aligned) and the wave's
// ballot gives the bit.  (One wave per group with 2-byte loads took 22 us for a 512 x 512 mask, as long as the
// attention launch that the entry point without allocations puts behind it.)
__global__ void __launch_bounds__(256) mask_summary_kernel(const f16 *mask, int seq_len, unsigned *out,
                                                           int words) {
    extern __shared__ unsigned ms_bits[]; // `words` entries
    const int g = blockIdx.x;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    for (int w = threadIdx.x; w < words; w += 256)
        ms_bits[w] = 0;
    __syncthreads();
    const int row = g * 16 + (lane >> 2);
    const int nt = (seq_len + AT_KT - 1) / AT_KT;
    const uint16_t *m = reinterpret_cast<const uint16_t *>(mask);
    const bool vec = (seq_len & 7) == 0 && (reinterpret_cast<uintptr_t>(mask) & 15u) == 0;
    for (int t = wave; t < nt; t += 4) {
        bool nz = false; // anything but +0 / -0
        if (row < seq_len) {
            const int k0 = t * AT_KT + (lane & 3) * 16;
            if (vec && k0 + 16 <= seq_len) {
                const u32x4 *p = reinterpret_cast<const u32x4 *>(m + (size_t)row * seq_len + k0);
                const u32x4 v0 = p[0], v1 = p[1];
                nz = (((v0[0] | v0[1] | v0[2] | v0[3] | v1[0] | v1[1] | v1[2] | v1[3]) & 0x7FFF7FFFu) != 0);
            } else {
                for (int j = 0; j < 16; j++)
                    if (k0 + j < seq_len && (m[(size_t)row * seq_len + k0 + j] & 0x7FFFu) != 0)
                        nz = true;
            }
        }
        if (__builtin_amdgcn_ballot_w64(nz) != 0 && lane == 0)
            atomicOr(&ms_bits[t >> 5], 1u << (t & 31));
    }
    __syncthreads();
    for (int w = threadIdx.x; w < words; w += 256)
        out[(size_t)g * words + w] = ms_bits[w];
}

static int mask_summary_words(int seq_len) { return ((seq_len + AT_KT - 1) / AT_KT + 31) / 32; }

// summaries registered for a mask pointer (et_attention_mask_summary_attach)
struct MaskSummaryEntry {
    const void *mask;
    const unsigned *summary;
    int seq_len;
    bool all_zero; // no bit set: the mask adds nothing anywhere
};
static std::mutex g_msum_mutex;
static std::vector<MaskSummaryEntry> g_msum;

// returns whether the mask is known to be zero everywhere
static bool attach_mask_summary(AttnArgs &a) {
    a.msum = nullptr;
    a.msum_words = 0;
    if (!a.mask)
        return true;
    std::lock_guard<std::mutex> lock(g_msum_mutex);
    for (const MaskSummaryEntry &e : g_msum)
        if (e.mask == a.mask && e.seq_len == a.seq_len) {
            a.msum = e.summary;
            a.msum_words = mask_summary_words(a.seq_len);
            return e.all_zero;
        }
    return false;
}

// qk_width: columns per head in Q and K (0 = head_dim)
// given_summary: a summary of a.mask supplied by the caller of this function
// (it then replaces the lookup among the attached ones)
static int attention_check(const AttnArgs &a, int d_model, bool sharedqk, const char *who) {
    ET_REQUIRE(a.out && a.V, ET_ERR_INVALID_ARG, "%s: null pointer", who);
    ET_REQUIRE(sharedqk ? a.QK != nullptr : (a.Q && a.K), ET_ERR_INVALID_ARG, "%s: null pointer", who);
    ET_REQUIRE(a.seq_len > 0 && d_model > 0 && a.nhead > 0 && a.batch > 0, ET_ERR_INVALID_ARG,
               "%s: seq_len=%d d_model=%d nhead=%d batch=%d", who, a.seq_len, d_model, a.nhead, a.batch);
    ET_REQUIRE(d_model % a.nhead == 0, ET_ERR_INVALID_ARG, "%s: d_model %% nhead != 0", who);
    const int hd = d_model / a.nhead;
    ET_REQUIRE(hd % 16 == 0 && hd <= 128, ET_ERR_UNSUPPORTED,
               "%s: head_dim %d: multiples of 16 up to 128", who, hd);
    ET_REQUIRE(aligned16(a.out) && aligned16(a.Q) && aligned16(a.K) && aligned16(a.V),
               ET_ERR_ALIGNMENT, "%s: out/Q/K/V must be 16-byte aligned", who);
    return ET_OK;
}

static int attention_dispatch(AttnArgs a, int d_model, bool pruned, bool sharedqk,
                              hipStream_t st, const char *who, int qk_width = 0,
                              const unsigned *given_summary = nullptr) {
    {
        const int rc = attention_check(a, d_model, sharedqk, who);
        if (rc != ET_OK)
            return rc;
    }
    const int hd_data = d_model / a.nhead;
    // Kernels are built for heads of 32, 64 and 128 columns.  Any other multiple
    // of 16 up to 128 (the reference loops over head_dim in steps of 16,
    // kernels/attention.cu:86-90) runs on the register-staged kernel of the next
    // built width as ragged heads: it reads the columns beyond a head's end as
    // zeros and writes none of them.
    const bool odd_width = !(hd_data == 32 || hd_data == 64 || hd_data == 128);
    ET_REQUIRE(!odd_width || (hd_data % 16 == 0 && hd_data > 0 && hd_data < 128 && !sharedqk && !a.qk_head_ptr &&
                              !a.v_head_ptr && !a.cu_seqlens),
               ET_ERR_UNSUPPORTED,
               "%s: head_dim %d: multiples of 16 up to 128 (dense heads, padded batches) or 32 / 64 / 128", who, hd_data);
    const int hd = !odd_width ? hd_data : hd_data < 32 ? 32 : hd_data < 64 ? 64 : 128;
    if (odd_width) {
        pruned = true;
        a.head_width = hd_data;
    }
    if (!pruned) {
        ET_REQUIRE(a.ldq % 8 == 0 && a.ldv % 8 == 0, ET_ERR_ALIGNMENT,
                   "%s: d_model must be a multiple of 8", who);
    }
    a.ldo = d_model;
    a.scale = head_scale(hd_data);
    bool no_mask;
    if (given_summary && a.mask) {
        a.msum = given_summary;
        a.msum_words = mask_summary_words(a.seq_len);
        no_mask = false; // its bits are only known on the device
    } else {
        no_mask = attach_mask_summary(a);
    }
    // 128 query rows per workgroup when that still fills the chip, else 64
    int variant = 0;
    {
        const long wg128 = (long)((a.seq_len + 127) / 128) * a.nhead * a.batch;
        if (wg128 < 512)
            variant = 2;
        if (hd == 128)
            variant = 2;
        if (a.cu_seqlens)
            variant = 2; // packed sequences of different lengths: 64-row blocks waste fewer padded query rows
                         // (config-5 batch: 50 us against 53-57 us with 128-row blocks)
        if (g_attn_variant >= 0 && g_attn_variant <= 2 && !(hd == 128 && g_attn_variant == 0))
            variant = g_attn_variant;
    }
    const int QB = variant == 2 ? 64 : 128;
    const bool plain = no_mask && !a.seq_lens && !a.cu_seqlens && a.seq_len % QB == 0;
    a.nqb = (a.seq_len + QB - 1) / QB;
    a.total = a.nqb * a.nhead * a.batch;
    a.per_xcd = (a.nhead * a.batch + 7) / 8 * a.nqb;
#define ET_ATTN_CASE(HDV)                                                                         \
    if (hd == HDV) {                                                                              \
        if (sharedqk) attn_launch_variant<HDV, false, true>(variant, false, a, st);                     \
        else if (pruned) attn_launch_variant<HDV, true, false>(variant, false, a, st);                  \
        else attn_launch_variant<HDV, false, false>(variant, plain, a, st);                             \
    }
    if (qk_width && qk_width != hd_data) {
        ET_REQUIRE(qk_width > 0 && qk_width < hd_data && qk_width % 16 == 0 && !sharedqk && !a.qk_head_ptr &&
                       !a.v_head_ptr && !a.cu_seqlens,
                   ET_ERR_UNSUPPORTED, "%s: %d of %d columns per head in Q and K: a multiple of 16 below the head width",
                   who, qk_width, hd_data);
        if (hd == 64 && qk_width == 32 && !pruned) { // the DMA-staged kernel with a 32-wide K tile
            attn_launch_variant<64, false, false, 32>(variant, plain, a, st);
            return launch_status(who);
        }
        // any other width: ragged heads on the register-staged kernel
        pruned = true;
        a.qk_width = qk_width;
    }
    // packed sequences: the grid the chip holds, every workgroup walks its share of the query blocks that exist
    if (a.cu_seqlens && !pruned && !sharedqk && variant == 2 && a.batch <= 64 * AT_PX && g_attn_packed) {
        if (hd == 32)
            attn_launch_packed<32>(a, st);
        else if (hd == 64)
            attn_launch_packed<64>(a, st);
        else
            attn_launch_packed<128>(a, st);
        return launch_status(who);
    }
    // dense Q/K with compact V (the reference's pruned wiring): DMA-staged value windows
    if (pruned && hd == 64 && !a.qk_head_ptr && a.v_head_ptr && a.ldq % 8 == 0 && a.ldv % 8 == 0 && a.ldv >= 8 &&
        g_attn_vwin) {
        if (variant == 0 && plain)
            attn_launch_one<64, 2, 4, true, false, true, 64, true>(a, st);
        else if (variant == 0)
            attn_launch_one<64, 2, 4, true, false, false, 64, true>(a, st);
        else if (variant == 1)
            attn_launch_one<64, 1, 8, true, false, false, 64, true>(a, st);
        else if (plain)
            attn_launch_one<64, 1, 4, true, false, true, 64, true>(a, st);
        else
            attn_launch_one<64, 1, 4, true, false, false, 64, true>(a, st);
        return launch_status(who);
    }
    ET_ATTN_CASE(32)
    ET_ATTN_CASE(64)
    ET_ATTN_CASE(128)
#undef ET_ATTN_CASE
    return launch_status(who);
}

void set_attn_variant(int v) { g_attn_variant = v; }
void set_attn_vwin(int v) { g_attn_vwin = v; }
void set_attn_packed(int v) { g_attn_packed = v; }

} // namespace et

extern "C" int et_OTF_attention(void *out, const void *Q, const void *K, const void *V,
                                const void *mask, int seq_len, int d_model, int nhead, int batch,
                                const int *seq_lens, float log2_scale, void *stream) {
    using namespace et;
    AttnArgs a = {};
    a.out = static_cast<f16 *>(out);
    a.Q = static_cast<const f16 *>(Q);
    a.K = static_cast<const f16 *>(K);
    a.V = static_cast<const f16 *>(V);
    a.mask = static_cast<const f16 *>(mask);
    a.seq_lens = seq_lens;
    a.ldq = a.ldv = d_model;
    a.seq_len = seq_len;
    a.nhead = nhead;
    a.batch = batch;
    a.log2_scale = log2_scale;
    return attention_dispatch(a, d_model, false, false, static_cast<hipStream_t>(stream),
                              "et_OTF_attention");
}

// ---- the entry point that allocates nothing --------------------------------
// Its scratch memory is the summary of the mask (one bit per 16 query rows x 64
// keys), which the other entry points keep in a buffer that the caller
// allocates and attaches.  Every GPU holds its own copy of the array at its own
// address: the address is looked up once per device and only that pointer is
// ever handed to a kernel (the array's name is a host-side stand-in).
namespace et {
constexpr int NOALLOC_MAX_SEQ = 4096; // 64 key tiles: what the kernels' two summary words per row group cover
constexpr int NOALLOC_WORDS = (NOALLOC_MAX_SEQ / 16) * 2;
static __device__ __align__(256) unsigned scratch[NOALLOC_WORDS]; // 2 KiB
constexpr int NOALLOC_MAX_DEVICES = 64;
static unsigned *g_scratch_ptr[NOALLOC_MAX_DEVICES];
static std::mutex g_scratch_mutex;

static int noalloc_scratch(unsigned **ptr) {
    int dev = -1;
    ET_HIP(hipGetDevice(&dev));
    ET_REQUIRE(dev >= 0 && dev < NOALLOC_MAX_DEVICES, ET_ERR_UNSUPPORTED,
               "et_OTF_attention_noalloc: device index %d beyond %d", dev, NOALLOC_MAX_DEVICES);
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void *p = nullptr;
        ET_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
        ET_REQUIRE(p != nullptr, ET_ERR_HIP, "et_OTF_attention_noalloc: no address for the scratch array");
        g_scratch_ptr[dev] = static_cast<unsigned *>(p);
    }
    *ptr = g_scratch_ptr[dev];
    return ET_OK;
}
} // namespace et

extern "C" int et_OTF_attention_noalloc(void *out, const void *Q, const void *K, const void *V,
                                        const void *mask, int seq_len, int d_model, int nhead,
                                        int batch, const int *seq_lens, float log2_scale,
                                        void *stream) {
    using namespace et;
    AttnArgs a = {};
    a.out = static_cast<f16 *>(out);
    a.Q = static_cast<const f16 *>(Q);
    a.K = static_cast<const f16 *>(K);
    a.V = static_cast<const f16 *>(V);
    a.mask = static_cast<const f16 *>(mask);
    a.seq_lens = seq_lens;
    a.ldq = a.ldv = d_model;
    a.seq_len = seq_len;
    a.nhead = nhead;
    a.batch = batch;
    a.log2_scale = log2_scale;
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (!mask) // nothing to summarise: no scratch memory is touched
        return attention_dispatch(a, d_model, false, false, st, "et_OTF_attention_noalloc");
    {
        // everything the attention launch would refuse is refused before the scratch array is written
        const int rc = attention_check(a, d_model, false, "et_OTF_attention_noalloc");
        if (rc != ET_OK)
            return rc;
    }
    ET_REQUIRE(seq_len <= NOALLOC_MAX_SEQ, ET_ERR_UNSUPPORTED,
               "et_OTF_attention_noalloc: seq_len %d beyond the %d that the static scratch array covers",
               seq_len, NOALLOC_MAX_SEQ);
    unsigned *summary = nullptr;
    const int rc = noalloc_scratch(&summary);
    if (rc != ET_OK)
        return rc;
    // every word that the attention kernel reads for this seq_len is written
    // here first, so what an earlier call left in the array does not matter
    hipLaunchKernelGGL(mask_summary_kernel, dim3((seq_len + 15) / 16), dim3(256), mask_summary_words(seq_len) * sizeof(unsigned), st, a.mask, seq_len,
                       summary, mask_summary_words(seq_len));
    const int rs = launch_status("et_OTF_attention_noalloc summary launch");
    if (rs != ET_OK)
        return rs;
    return attention_dispatch(a, d_model, false, false, st, "et_OTF_attention_noalloc", 0, summary);
}

extern "C" int et_OTF_attention_summary(void *out, const void *Q, const void *K, const void *V,
                                        const void *mask, const void *mask_summary, int seq_len, int d_model,
                                        int nhead, int batch, const int *seq_lens, float log2_scale,
                                        void *stream) {
    using namespace et;
    AttnArgs a = {};
    a.out = static_cast<f16 *>(out);
    a.Q = static_cast<const f16 *>(Q);
    a.K = static_cast<const f16 *>(K);
    a.V = static_cast<const f16 *>(V);
    a.mask = static_cast<const f16 *>(mask);
    a.seq_lens = seq_lens;
    a.ldq = a.ldv = d_model;
    a.seq_len = seq_len;
    a.nhead = nhead;
    a.batch = batch;
    a.log2_scale = log2_scale;
    ET_REQUIRE(!mask_summary || mask, ET_ERR_INVALID_ARG, "et_OTF_attention_summary: a summary without a mask");
    return attention_dispatch(a, d_model, false, false, static_cast<hipStream_t>(stream), "et_OTF_attention_summary",
                              0, static_cast<const unsigned *>(mask_summary));
}

extern "C" int et_OTF_attention_qk_width(void *out, const void *Q, const void *K, const void *V,
                                         const void *mask, int qk_width, int seq_len, int d_model,
                                         int nhead, int batch, const int *seq_lens, float log2_scale,
                                         void *stream) {
    using namespace et;
    ET_REQUIRE(qk_width > 0 && nhead > 0, ET_ERR_INVALID_ARG, "et_OTF_attention_qk_width: qk_width=%d", qk_width);
    AttnArgs a = {};
    a.out = static_cast<f16 *>(out);
    a.Q = static_cast<const f16 *>(Q);
    a.K = static_cast<const f16 *>(K);
    a.V = static_cast<const f16 *>(V);
    a.mask = static_cast<const f16 *>(mask);
    a.seq_lens = seq_lens;
    a.ldq = nhead * qk_width;
    a.ldv = d_model;
    a.seq_len = seq_len;
    a.nhead = nhead;
    a.batch = batch;
    a.log2_scale = log2_scale;
    return attention_dispatch(a, d_model, false, false, static_cast<hipStream_t>(stream),
                              "et_OTF_attention_qk_width", qk_width);
}

extern "C" int et_OTF_attention_varlen(void *out, const void *Q, const void *K, const void *V,
                                       const void *mask, const int *cu_seqlens, int max_seq_len,
                                       int d_model, int nhead, int batch, float log2_scale,
                                       void *stream) {
    using namespace et;
    ET_REQUIRE(cu_seqlens, ET_ERR_INVALID_ARG, "et_OTF_attention_varlen: null cu_seqlens");
    AttnArgs a = {};
    a.out = static_cast<f16 *>(out);
    a.Q = static_cast<const f16 *>(Q);
    a.K = static_cast<const f16 *>(K);
    a.V = static_cast<const f16 *>(V);
    a.mask = static_cast<const f16 *>(mask);
    a.cu_seqlens = cu_seqlens;
    a.ldq = a.ldv = d_model;
    a.seq_len = max_seq_len;
    a.nhead = nhead;
    a.batch = batch;
    a.log2_scale = log2_scale;
    return attention_dispatch(a, d_model, false, false, static_cast<hipStream_t>(stream),
                              "et_OTF_attention_varlen");
}

extern "C" int et_Prune_attention(void *out, const void *Q, const void *K, const void *V,
                                  const int *qk_head_ptr, int ldqk, const int *v_col_id,
                                  const int *v_head_ptr, int ldv, const void *mask, int seq_len,
                                  int d_model, int nhead, int batch, const int *seq_lens,
                                  float log2_scale, void *stream) {
    using namespace et;
    AttnArgs a = {};
    a.out = static_cast<f16 *>(out);
    a.Q = static_cast<const f16 *>(Q);
    a.K = static_cast<const f16 *>(K);
    a.V = static_cast<const f16 *>(V);
    a.mask = static_cast<const f16 *>(mask);
    a.seq_lens = seq_lens;
    a.qk_head_ptr = qk_head_ptr;
    a.v_col_id = v_col_id;
    a.v_head_ptr = v_head_ptr;
    a.ldq = qk_head_ptr ? ldqk : d_model;
    a.ldv = v_head_ptr ? ldv : d_model;
    ET_REQUIRE(a.ldq > 0 && a.ldv > 0, ET_ERR_INVALID_ARG, "et_Prune_attention: ldqk=%d ldv=%d", ldqk, ldv);
    ET_REQUIRE(!v_col_id || v_head_ptr, ET_ERR_INVALID_ARG,
               "et_Prune_attention: v_col_id given without v_head_ptr");
    a.seq_len = seq_len;
    a.nhead = nhead;
    a.batch = batch;
    a.log2_scale = log2_scale;
    return attention_dispatch(a, d_model, true, false, static_cast<hipStream_t>(stream),
                              "et_Prune_attention");
}

extern "C" int et_sharedQK_attention(void *out, const void *QK, const void *V, const void *mask,
                                     int seq_len, int d_model, int nhead, int batch,
                                     const int *seq_lens, float log2_scale, void *stream) {
    using namespace et;
    AttnArgs a = {};
    a.out = static_cast<f16 *>(out);
    a.QK = static_cast<const f16 *>(QK);
    a.V = static_cast<const f16 *>(V);
    a.mask = static_cast<const f16 *>(mask);
    a.seq_lens = seq_lens;
    a.ldq = a.ldv = d_model;
    a.seq_len = seq_len;
    a.nhead = nhead;
    a.batch = batch;
    a.log2_scale = log2_scale;
    return attention_dispatch(a, d_model, false, true, static_cast<hipStream_t>(stream),
                              "et_sharedQK_attention");
}

extern "C" int et_qk_scores(void *QK, const void *Q, const void *K, int seq_len, int d_model,
                            int nhead, int batch, void *stream) {
    using namespace et;
    ET_REQUIRE(QK && Q && K, ET_ERR_INVALID_ARG, "et_qk_scores: null pointer");
    ET_REQUIRE(seq_len > 0 && d_model > 0 && nhead > 0 && batch > 0 && d_model % nhead == 0,
               ET_ERR_INVALID_ARG, "et_qk_scores: bad sizes");
    const int hd = d_model / nhead;
    ET_REQUIRE(hd == 32 || hd == 64 || hd == 128, ET_ERR_UNSUPPORTED,
               "et_qk_scores: head_dim %d not in {32,64,128}", hd);
    ET_REQUIRE(aligned16(Q) && aligned16(K) && d_model % 8 == 0, ET_ERR_ALIGNMENT,
               "et_qk_scores: Q/K must be 16-byte aligned");
    // scale = half(1/sqrt(head_dim)), encoder/encoder.cu:113
    const float scale = (float)(f16)(1.0f / sqrtf((float)hd));
    const dim3 grid((seq_len + 255) / 256, (seq_len + 63) / 64, batch * nhead), block(256);
    hipStream_t st = static_cast<hipStream_t>(stream);
    f16 *o = static_cast<f16 *>(QK);
    const f16 *q = static_cast<const f16 *>(Q), *k = static_cast<const f16 *>(K);
    if (hd == 32)
        hipLaunchKernelGGL(qk_scores_kernel<32>, grid, block, 0, st, o, q, k, seq_len, d_model, nhead, scale);
    else if (hd == 64)
        hipLaunchKernelGGL(qk_scores_kernel<64>, grid, block, 0, st, o, q, k, seq_len, d_model, nhead, scale);
    else
        hipLaunchKernelGGL(qk_scores_kernel<128>, grid, block, 0, st, o, q, k, seq_len, d_model, nhead, scale);
    return launch_status("et_qk_scores");
}

extern "C" size_t et_attention_mask_summary_bytes(int seq_len) {
    if (seq_len <= 0)
        return 0;
    return (size_t)((seq_len + 15) / 16) * et::mask_summary_words(seq_len) * sizeof(unsigned);
}

extern "C" int et_attention_mask_summary(const void *mask, int seq_len, void *summary, void *stream) {
    using namespace et;
    ET_REQUIRE(mask && summary, ET_ERR_INVALID_ARG, "et_attention_mask_summary: null pointer");
    ET_REQUIRE(seq_len > 0, ET_ERR_INVALID_ARG, "et_attention_mask_summary: seq_len=%d", seq_len);
    hipLaunchKernelGGL(mask_summary_kernel, dim3((seq_len + 15) / 16), dim3(256), mask_summary_words(seq_len) * sizeof(unsigned),
                       static_cast<hipStream_t>(stream), static_cast<const f16 *>(mask), seq_len,
                       static_cast<unsigned *>(summary), mask_summary_words(seq_len));
    return launch_status("et_attention_mask_summary launch");
}

extern "C" int et_attention_mask_summary_attach(const void *mask, int seq_len, const void *summary) {
    using namespace et;
    ET_REQUIRE(mask && seq_len > 0, ET_ERR_INVALID_ARG, "et_attention_mask_summary_attach: bad arguments");
    std::lock_guard<std::mutex> lock(g_msum_mutex);
    for (size_t i = 0; i < g_msum.size(); i++)
        if (g_msum[i].mask == mask && g_msum[i].seq_len == seq_len) {
            g_msum.erase(g_msum.begin() + i);
            break;
        }
    if (summary) {
        // read the summary back once: an all-zero mask selects the kernels
        // without any mask handling
        const size_t words = (size_t)((seq_len + 15) / 16) * mask_summary_words(seq_len);
        std::vector<unsigned> h(words);
        ET_HIP(hipDeviceSynchronize());
        ET_HIP(hipMemcpy(h.data(), summary, words * sizeof(unsigned), hipMemcpyDeviceToHost));
        bool all_zero = true;
        for (unsigned w : h)
            all_zero = all_zero && w == 0;
        g_msum.push_back({mask, static_cast<const unsigned *>(summary), seq_len, all_zero});
    }
    return ET_OK;
}
