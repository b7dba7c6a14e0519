// Dense GEMM for the row-pruned linear on gfx950:  Y[M x N] = X[M x K] W^T + b
// (+ GELU), W = the compacted surviving rows [N x K] row-major, fp16 storage,
// fp32 accumulate.  Replaces the cublasGemmEx call plus add_bias kernel of
// kernels/linear.cu:5-34.
//
// Both operands are contiguous along K, which is the layout the 16x16x32 MFMA
// wants for A and for B (8 consecutive k per lane), so neither is transposed.
// A workgroup of four waves (2 x 2) computes a 128 x 128 block, a wave 64 x 64
// = 4 x 4 MFMA tiles (16 fragment reads feed 32 MFMAs per K step of 64: the
// register blocking a streamed tile list cannot have).  The product is issued
// as W X^T so that a lane ends with four consecutive output features of one
// row.  K is walked in steps of 64 through two LDS buffers filled by DMA
// (global_load_lds_dwordx4, no registers) one step ahead.  A DMA instruction
// writes 64 x 16 bytes to consecutive LDS, the source address is free per
// lane: the 16-byte pieces of a row are stored XOR-swizzled by (row / 2) % 8,
// which makes the ds_read_b128 fragment reads conflict-free without padding
// (rows r and r + 2 would otherwise share their banks).
#include <cstring>

#include "common.h"

namespace et {

constexpr int DG_BN = 128, DG_BK = 64; // (the block has 64 WM rows, WM = 2 or 4 waves along M)
constexpr int DG_MAX_LIN = 3;

struct DgArgs {
    f16 *Y[DG_MAX_LIN];
    const f16 *W[DG_MAX_LIN];
    const f16 *bias[DG_MAX_LIN];
    int N[DG_MAX_LIN];
    int tile0[DG_MAX_LIN + 1]; // first column tile of each linear in the launch's tile list
    const f16 *X;
    int nlin, M, K, tiles_m, tiles_n, per_xcd, total;
};

// LDS position (in 16-byte pieces) of piece kc of row r in a [rows x 64] tile
__device__ __forceinline__ int dg_piece(int r, int kc) { return r * 8 + (kc ^ ((r >> 1) & 7)); }

// one operand tile: ROWS rows x 64 halves = ROWS / 8 DMA instructions, spread
// over the NW waves; rows beyond `rows_total` re-read the last row (their
// products are not stored)
template <int ROWS, int NW>
__device__ __forceinline__ void dg_fetch(f16 *lds, const f16 *src, int ld, int row0, int rows_total, int k0,
                                         int K, int wave, int lane) {
    static_assert((ROWS / 8) % NW == 0, "whole instructions per wave");
#pragma unroll
    for (int i = 0; i < ROWS / 8 / NW; i++) {
        const int inst = wave * (ROWS / 8 / NW) + i;
        const int p = inst * 64 + lane; // this lane's piece in the tile
        const int r = p >> 3, slot = p & 7;
        const int kc = slot ^ ((r >> 1) & 7);
        const int row = min(row0 + r, rows_total - 1);
        const int k = min(k0 + kc * 8, K - 8); // (pieces beyond K belong to a K step that is not multiplied)
        load_lds16(src + (size_t)row * ld + k, lds + inst * 512);
    }
}

template <bool GELU, int WM, int STAGES>
__global__ void __launch_bounds__(WM * 2 * 64) dense_gemm_kernel(const DgArgs a) {
    constexpr int NW = WM * 2, DG_BM = WM * 64;
    extern __shared__ __attribute__((aligned(16))) unsigned char dg_smem[];
    f16 *smem = reinterpret_cast<f16 *>(dg_smem);
    constexpr int XT = DG_BM * DG_BK, WT = DG_BN * DG_BK; // halves per operand tile
    constexpr int STAGE = XT + WT;
    constexpr int PER_WAVE = (DG_BM + DG_BN) / 8 / NW;    // DMA instructions per wave and K step
    // consecutive ids on one XCD walk the column tiles of one row tile: they
    // share the X tile in that XCD's L2, and W (small) is everywhere
    const int vid = (blockIdx.x & 7) * a.per_xcd + (blockIdx.x >> 3);
    if (vid >= a.total)
        return;
    const int tm = vid / a.tiles_n, tn_all = vid - tm * a.tiles_n;
    int lin = 0;
#pragma unroll
    for (int i = 1; i < DG_MAX_LIN; i++)
        lin += (i < a.nlin && tn_all >= a.tile0[i]) ? 1 : 0;
    const int tn = tn_all - (lin == 0 ? a.tile0[0] : lin == 1 ? a.tile0[1] : a.tile0[2]);
    f16 *const Y = lin == 0 ? a.Y[0] : lin == 1 ? a.Y[1] : a.Y[2];
    const f16 *const W = lin == 0 ? a.W[0] : lin == 1 ? a.W[1] : a.W[2];
    const f16 *const bias = lin == 0 ? a.bias[0] : lin == 1 ? a.bias[1] : a.bias[2];
    const int N = lin == 0 ? a.N[0] : lin == 1 ? a.N[1] : a.N[2];

    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int lane = threadIdx.x & 63;
    const int c16 = lane & 15, g4 = lane >> 4;
    const int wm = wave >> 1, wn = wave & 1; // the wave's 64 x 64 part of the block
    const int m0 = tm * DG_BM, n0 = tn * DG_BN;
    const int nk = (a.K + DG_BK - 1) / DG_BK;

    f32x4 acc[4][4]; // [feature subtile][row subtile]
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 4; j++)
            acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};

    // K step kt lives in stage kt % STAGES (X tile, W tile behind it); STAGES - 1
    // steps are requested ahead, so a step has the time of STAGES - 2 steps of
    // MFMAs (plus the other waves') to arrive
    auto fetch = [&](int kt) {
        f16 *xn = smem + (kt % STAGES) * STAGE;
        dg_fetch<DG_BM, NW>(xn, a.X, a.K, m0, a.M, kt * DG_BK, a.K, wave, lane);
        dg_fetch<DG_BN, NW>(xn + XT, W, a.K, n0, N, kt * DG_BK, a.K, wave, lane);
    };
#pragma unroll
    for (int t = 0; t < STAGES - 1; t++)
        if (t < nk)
            fetch(t);
    for (int kt = 0; kt < nk; kt++) {
        const f16 *xs = smem + (kt % STAGES) * STAGE;
        const f16 *ws = xs + XT;
        // this wave's pieces of step kt have landed (loads return in order: the
        // younger steps' instructions may still be out)
        if (STAGES > 2 && kt + STAGES - 1 <= nk)
            __builtin_amdgcn_s_waitcnt(0x0F70 | ((STAGES - 2) * PER_WAVE));
        else
            __builtin_amdgcn_s_waitcnt(0x0F70);
        __syncthreads(); // ... everyone's, and everyone is done with the stage that is refilled now
        if (kt + STAGES - 1 < nk)
            fetch(kt + STAGES - 1);
        const int ksteps = min(2, (a.K - kt * DG_BK) >> 5); // K is a multiple of 32
        for (int s = 0; s < ksteps; s++) {
            f16x8 xf[4], wf[4];
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const int r = wm * 64 + j * 16 + c16;
                xf[j] = *reinterpret_cast<const f16x8 *>(xs + dg_piece(r, s * 4 + g4) * 8);
            }
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const int r = wn * 64 + i * 16 + c16;
                wf[i] = *reinterpret_cast<const f16x8 *>(ws + dg_piece(r, s * 4 + g4) * 8);
            }
#pragma unroll
            for (int i = 0; i < 4; i++)
#pragma unroll
                for (int j = 0; j < 4; j++)
                    acc[i][j] = mfma16x16x32(wf[i], xf[j], acc[i][j]);
        }
    }
    __syncthreads(); // the tile buffers are free: they stage the output block

    // acc[i][j][r] = Y[row = m0 + wm*64 + j*16 + c16][col = n0 + wn*64 + i*16 + g4*4 + r]
    // -> the wave's 64 x 64 block in LDS ([row][64 halves + 8]), then 16-byte stores
    constexpr int LDO = 64 + 8;
    f16 *os = smem + wave * 64 * LDO;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const int col = n0 + wn * 64 + i * 16 + g4 * 4;
        f16x4 b4 = f16x4{0, 0, 0, 0};
        if (col < N)
            b4 = *reinterpret_cast<const f16x4 *>(bias + col);
        const f32x4 bf = __builtin_convertvector(b4, f32x4);
#pragma unroll
        for (int j = 0; j < 4; j++) {
            f16x4 ov = __builtin_convertvector(acc[i][j] + bf, f16x4);
            if (GELU)
                ov = gelu4(ov);
            *reinterpret_cast<f16x4 *>(os + (j * 16 + c16) * LDO + i * 16 + g4 * 4) = ov;
        }
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    // (the staging block is the wave's own: LDS operations of one wave execute in order)
#pragma unroll
    for (int t = 0; t < 8; t++) {
        const int p = t * 64 + lane; // 64 rows x 8 pieces
        const int r = p >> 3, pc = p & 7;
        const int row = m0 + wm * 64 + r, col = n0 + wn * 64 + pc * 8;
        if (row < a.M && col < N) { // N is a multiple of 16: a piece is inside or outside as a whole
            const u32x4 v = *reinterpret_cast<const u32x4 *>(os + r * LDO + pc * 8);
            *reinterpret_cast<u32x4 *>(Y + (size_t)row * N + col) = v;
        }
    }
}

template <bool GELU, int WM, int STAGES>
static int dg_launch_inst(DgArgs &a, hipStream_t st) {
    constexpr int BM = WM * 64;
    constexpr size_t lds = (size_t)STAGES * (BM + DG_BN) * DG_BK * sizeof(f16);
    static_assert((size_t)WM * 2 * 64 * (64 + 8) * sizeof(f16) <= lds, "the output staging fits the tile buffers");
    a.tiles_m = (a.M + BM - 1) / BM;
    a.total = a.tiles_m * a.tiles_n;
    a.per_xcd = (a.total + 7) / 8;
    constexpr auto k = &dense_gemm_kernel<GELU, WM, STAGES>;
    if (lds > 64 * 1024) {
        static bool done = false; // (asked of the driver once per kernel instance)
        if (!done) {
            ET_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(k), hipFuncAttributeMaxDynamicSharedMemorySize,
                                       (int)lds));
            done = true;
        }
    }
    hipLaunchKernelGGL(k, dim3(a.per_xcd * 8), dim3(WM * 2 * 64), lds, st, a);
    return launch_status("dense_gemm launch");
}

// nlin linears over the same X in one launch.  Returns ET_ERR_UNSUPPORTED where
// the shapes do not fit this kernel (the caller then takes the tile path).
int dense_gemm_launch(void *const *Ys, const void *X, const void *const *Ws, const void *const *biases,
                      const int *Ns, int nlin, int M, int K, bool gelu, hipStream_t st) {
    if (nlin < 1 || nlin > DG_MAX_LIN || K < 32 || K % 32 != 0 || M <= 0)
        return ET_ERR_UNSUPPORTED;
    DgArgs a;
    memset(&a, 0, sizeof(a));
    int tiles_n = 0;
    for (int i = 0; i < DG_MAX_LIN; i++) {
        const int s = i < nlin ? i : 0;
        if (Ns[s] <= 0 || Ns[s] % 16 != 0 || !aligned16(Ys[s]) || !aligned16(Ws[s]) || !aligned16(biases[s]))
            return ET_ERR_UNSUPPORTED;
        a.Y[i] = static_cast<f16 *>(Ys[s]);
        a.W[i] = static_cast<const f16 *>(Ws[s]);
        a.bias[i] = static_cast<const f16 *>(biases[s]);
        a.N[i] = Ns[s];
        a.tile0[i] = tiles_n;
        if (i < nlin)
            tiles_n += (Ns[s] + DG_BN - 1) / DG_BN;
    }
    a.tile0[DG_MAX_LIN] = tiles_n;
    if (!aligned16(X))
        return ET_ERR_UNSUPPORTED;
    a.X = static_cast<const f16 *>(X);
    a.nlin = nlin;
    a.M = M;
    a.K = K;
    a.tiles_n = tiles_n;
    // 128 x 128 blocks, four waves, two stages: 64 KB of LDS, two workgroups per
    // CU.  (Measured against 256 x 128 blocks of eight waves and against three
    // stages, both with one workgroup per CU: 10 to 30 % slower - the second
    // workgroup hides more latency than the deeper ring.)
    return gelu ? dg_launch_inst<true, 2, 2>(a, st) : dg_launch_inst<false, 2, 2>(a, st);
}

} // namespace et
