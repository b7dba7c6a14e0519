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
// half-precision staging write 8 bytes wide.  Results are staged in LDS (the
// X panel's storage is reused) and written with 16-byte row-contiguous
// stores, because at >= 80 % sparsity this op is bound by the Y write.
// K larger than the LDS panel is walked in chunks of KC columns; plans sort
// each block-row's tiles by column and carry a per-chunk CSR so a chunk only
// touches its own tiles (TL_CSR); raw unsorted input with K > one panel falls
// back to filtering the whole list per chunk (TL_FILTER).
#include "common.h"

#include <algorithm>
#include <cstdlib>
#include <cstring>
#include <numeric>
#include <vector>

namespace et {

constexpr int TL_THREADS = 512;
constexpr int TL_WAVES = 8;
constexpr int TL_BM = 32;
constexpr int TL_PAD = 8;        // halves; makes the LDS row stride an odd multiple of 16 B
constexpr int TL_MAX_PANEL = 1008; // single-panel K limit: 32*(1008+8)*2 B < 64 KB
constexpr int TL_CHUNK = 768;
constexpr int TL_MAX_LIN = 4;

enum { TL_CSR = 0, TL_FILTER = 1, TL_DENSE = 2 };

struct TlProblem {
    f16 *Y;
    const int *cptr;       // TL_CSR: per-(block-row,chunk) CSR; TL_FILTER: row_ptr
    const int *row_offset; // element column offset per tile
    const f16 *data;       // tile_mat data, or dense row-major W for TL_DENSE
    const f16 *bias;
    int N;
    int nbr; // N / 16
};

struct TlArgs {
    TlProblem p[TL_MAX_LIN];
    const f16 *X;
    int nlin, M, K, KC, nchunk, ncg, total, per_xcd;
};

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

template <int NB, bool GELU, int MODE>
__global__ void __launch_bounds__(TL_THREADS) tile_linear_kernel(const TlArgs a) {
    extern __shared__ __attribute__((aligned(16))) unsigned char tl_smem[];
    f16 *xs = reinterpret_cast<f16 *>(tl_smem);

    // Workgroups that share a row panel of X get consecutive ids on ONE XCD
    // (hardware round-robins consecutive workgroup ids over the 8 XCDs), so
    // the panel is fetched into that XCD's L2 once.
    const int pid = (blockIdx.x & 7) * a.per_xcd + (blockIdx.x >> 3);
    if (pid >= a.total)
        return;
    const int per_rp = a.ncg * a.nlin;
    const int rp = pid / per_rp;
    const int rest = pid - rp * per_rp;
    const int lin = rest / a.ncg;
    const int cg = rest - lin * a.ncg;
    TlProblem P = a.p[0];
    if (lin == 1) P = a.p[1];
    if (lin == 2) P = a.p[2];
    if (lin == 3) P = a.p[3];

    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int lane = threadIdx.x & 63;
    const int c16 = lane & 15;
    const int g4 = lane >> 4;
    const int khalf8 = (g4 & 1) * 8;
    const int hi = lane >> 5;
    const int m0 = rp * TL_BM;
    const int ldx = a.KC + TL_PAD;
    const int bn_wg = cg * (TL_WAVES * NB);
    const int bn0 = bn_wg + wave * NB;

    f32x4 acc[NB][2];
#pragma unroll
    for (int j = 0; j < NB; j++) {
        acc[j][0] = f32x4{0.f, 0.f, 0.f, 0.f};
        acc[j][1] = f32x4{0.f, 0.f, 0.f, 0.f};
    }

    const f16 *xlane = xs + c16 * ldx + khalf8;
    const int ld_r = threadIdx.x >> 4; // 0..31: panel row this thread stages
    const int ld_c = threadIdx.x & 15;

    for (int c = 0; c < a.nchunk; c++) {
        const int k0 = c * a.KC;
        const int kc = min(a.KC, a.K - k0);
        if (c > 0)
            __syncthreads();
        { // stage X[m0..m0+31][k0..k0+kc) into LDS, rows beyond M as zeros
            const int cpr = kc >> 3;
            const bool rowok = (m0 + ld_r) < a.M;
            const u32x4 *src = reinterpret_cast<const u32x4 *>(a.X + (size_t)(m0 + ld_r) * a.K + k0);
            u32x4 *dst = reinterpret_cast<u32x4 *>(xs + ld_r * ldx);
            for (int cc = ld_c; cc < cpr; cc += 16) {
                u32x4 v = u32x4{0u, 0u, 0u, 0u};
                if (rowok)
                    v = src[cc];
                dst[cc] = v;
            }
        }
        __syncthreads();

#pragma unroll
        for (int j = 0; j < NB; j++) {
            const int bn = bn0 + j;
            if (bn >= P.nbr)
                continue;
            if (MODE == TL_CSR) {
                const int s = P.cptr[bn * a.nchunk + c];
                const int e = P.cptr[bn * a.nchunk + c + 1];
                const f16 *wlane = P.data + c16 * 16 + khalf8;
                int i = s;
                f16x8 w_n = f16x8{0, 0, 0, 0, 0, 0, 0, 0};
                int off_n = 0;
                if (i + 1 < e) {
                    off_n = P.row_offset[i + hi];
                    w_n = *reinterpret_cast<const f16x8 *>(wlane + (size_t)(i + hi) * 256);
                }
                for (; i + 1 < e; i += 2) {
                    const f16x8 w = w_n;
                    const int off = off_n - k0;
                    if (i + 3 < e) {
                        off_n = P.row_offset[i + 2 + hi];
                        w_n = *reinterpret_cast<const f16x8 *>(wlane + (size_t)(i + 2 + hi) * 256);
                    }
                    const f16x8 x0 = *reinterpret_cast<const f16x8 *>(xlane + off);
                    const f16x8 x1 = *reinterpret_cast<const f16x8 *>(xlane + off + 16 * ldx);
                    acc[j][0] = mfma16x16x32(w, x0, acc[j][0]);
                    acc[j][1] = mfma16x16x32(w, x1, acc[j][1]);
                }
                if (i < e) { // odd tail: the upper half-wave multiplies by zero weights
                    const int off = P.row_offset[i] - k0;
                    f16x8 w = *reinterpret_cast<const f16x8 *>(wlane + (size_t)i * 256);
                    if (hi)
                        w = f16x8{0, 0, 0, 0, 0, 0, 0, 0};
                    const f16x8 x0 = *reinterpret_cast<const f16x8 *>(xlane + off);
                    const f16x8 x1 = *reinterpret_cast<const f16x8 *>(xlane + off + 16 * ldx);
                    acc[j][0] = mfma16x16x32(w, x0, acc[j][0]);
                    acc[j][1] = mfma16x16x32(w, x1, acc[j][1]);
                }
            } else if (MODE == TL_FILTER) {
                const int s = P.cptr[bn];
                const int e = P.cptr[bn + 1];
                const f16 *wlane = P.data + c16 * 16 + khalf8;
                for (int i = s; i < e; i += 2) {
                    const int ti = min(i + hi, e - 1);
                    const int off = P.row_offset[ti] - k0;
                    const bool ok = (i + hi < e) && off >= 0 && off < kc;
                    if (__builtin_amdgcn_ballot_w64(ok) == 0)
                        continue;
                    const f16x8 z = f16x8{0, 0, 0, 0, 0, 0, 0, 0};
                    f16x8 w = z, x0 = z, x1 = z;
                    if (ok) {
                        w = *reinterpret_cast<const f16x8 *>(wlane + (size_t)ti * 256);
                        x0 = *reinterpret_cast<const f16x8 *>(xlane + off);
                        x1 = *reinterpret_cast<const f16x8 *>(xlane + off + 16 * ldx);
                    }
                    acc[j][0] = mfma16x16x32(w, x0, acc[j][0]);
                    acc[j][1] = mfma16x16x32(w, x1, acc[j][1]);
                }
            } else { // TL_DENSE: every k-tile of the chunk, W row-major [N x K]
                const f16 *wlane = P.data + (size_t)(bn * 16 + c16) * a.K + k0 + khalf8;
                const int nt = kc >> 4;
                int i = 0;
                for (; i + 1 < nt; i += 2) {
                    const int off = (i + hi) * 16;
                    const f16x8 w = *reinterpret_cast<const f16x8 *>(wlane + off);
                    const f16x8 x0 = *reinterpret_cast<const f16x8 *>(xlane + off);
                    const f16x8 x1 = *reinterpret_cast<const f16x8 *>(xlane + off + 16 * ldx);
                    acc[j][0] = mfma16x16x32(w, x0, acc[j][0]);
                    acc[j][1] = mfma16x16x32(w, x1, acc[j][1]);
                }
                if (i < nt) {
                    const int off = i * 16;
                    f16x8 w = *reinterpret_cast<const f16x8 *>(wlane + off);
                    if (hi)
                        w = f16x8{0, 0, 0, 0, 0, 0, 0, 0};
                    const f16x8 x0 = *reinterpret_cast<const f16x8 *>(xlane + off);
                    const f16x8 x1 = *reinterpret_cast<const f16x8 *>(xlane + off + 16 * ldx);
                    acc[j][0] = mfma16x16x32(w, x0, acc[j][0]);
                    acc[j][1] = mfma16x16x32(w, x1, acc[j][1]);
                }
            }
        }
    }

    // ---- epilogue: bias (+GELU), round to half, stage in LDS, coalesced store
    __syncthreads(); // every wave is done reading the X panel
    constexpr int BNW = TL_WAVES * NB * 16; // output columns per workgroup
    constexpr int ldy = BNW + TL_PAD;
    f16 *ys = xs;
#pragma unroll
    for (int j = 0; j < NB; j++) {
        const int bn = bn0 + j;
        if (bn >= P.nbr)
            continue;
        const f16x4 b4 = *reinterpret_cast<const f16x4 *>(P.bias + bn * 16 + g4 * 4);
        const int ncol = (bn - bn_wg) * 16 + g4 * 4;
#pragma unroll
        for (int ms = 0; ms < 2; ms++) {
            f16x4 o;
#pragma unroll
            for (int r = 0; r < 4; r++) {
                const f16 v = (f16)(acc[j][ms][r] + (float)b4[r]);
                o[r] = GELU ? gelu_h(v) : v;
            }
            *reinterpret_cast<f16x4 *>(ys + (ms * 16 + c16) * ldy + ncol) = o;
        }
    }
    __syncthreads();
    {
        const int col0 = bn_wg * 16;
        const int wcols = min(BNW, P.N - col0);
        const int cpr = wcols >> 3;
        if (m0 + ld_r < a.M) {
            u32x4 *dst = reinterpret_cast<u32x4 *>(P.Y + (size_t)(m0 + ld_r) * P.N + col0);
            const u32x4 *src = reinterpret_cast<const u32x4 *>(ys + ld_r * ldy);
            for (int cc = ld_c; cc < cpr; cc += 16)
                dst[cc] = src[cc];
        }
    }
}

// ---------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------
template <int NB, bool GELU, int MODE>
static void launch_inst(const TlArgs &a, size_t lds, hipStream_t st) {
    hipLaunchKernelGGL((tile_linear_kernel<NB, GELU, MODE>), dim3(a.per_xcd * 8),
                       dim3(TL_THREADS), lds, st, a);
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

static int env_int(const char *name, int dflt) {
    const char *v = getenv(name);
    return (v && *v) ? atoi(v) : dflt;
}

// Block-rows per wave: the largest NB that still yields enough workgroups to
// fill 256 CUs a few times over.  ET_TILE_NB overrides (tuning aid).
static int choose_nb(int nrp, int nbr_max, int nlin) {
    static const int forced = env_int("ET_TILE_NB", 0);
    if (forced == 1 || forced == 2 || forced == 3 || forced == 4 || forced == 6)
        return forced;
    static const int want = env_int("ET_TILE_MIN_WGS", 1536);
    const int cand[5] = {6, 4, 3, 2, 1};
    for (int i = 0; i < 5; i++) {
        const int nb = cand[i];
        const int ncg = (nbr_max + TL_WAVES * nb - 1) / (TL_WAVES * nb);
        if ((long)nrp * ncg * nlin >= want)
            return nb;
    }
    return 1;
}

static int tile_launch(const TlProblem *probs, int nlin, const f16 *X, int M, int K,
                       int KC, int nchunk, bool gelu, int mode, hipStream_t st) {
    TlArgs a;
    memset(&a, 0, sizeof(a));
    int nbr_max = 0;
    for (int i = 0; i < nlin; i++) {
        a.p[i] = probs[i];
        nbr_max = std::max(nbr_max, probs[i].nbr);
    }
    for (int i = nlin; i < TL_MAX_LIN; i++)
        a.p[i] = probs[0];
    a.X = X;
    a.nlin = nlin;
    a.M = M;
    a.K = K;
    a.KC = KC;
    a.nchunk = nchunk;
    const int nrp = (M + TL_BM - 1) / TL_BM;
    const int nb = choose_nb(nrp, nbr_max, nlin);
    a.ncg = (nbr_max + TL_WAVES * nb - 1) / (TL_WAVES * nb);
    a.total = nrp * a.ncg * nlin;
    a.per_xcd = (a.total + 7) / 8;
    const size_t lds_x = (size_t)TL_BM * (KC + TL_PAD) * sizeof(f16);
    const size_t lds_y = (size_t)TL_BM * (TL_WAVES * nb * 16 + TL_PAD) * sizeof(f16);
    const size_t lds = std::max(lds_x, lds_y);
    if (mode == TL_CSR) {
        if (gelu) launch_nb<true, TL_CSR>(nb, a, lds, st);
        else launch_nb<false, TL_CSR>(nb, a, lds, st);
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
                       nchunk == 1 ? TL_CSR : TL_FILTER, static_cast<hipStream_t>(stream));
}

} // namespace et

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

extern "C" int et_row_spmm_add_bias(void *out, const void *in, const void *weight,
                                    const void *bias, int M, int N, int K, void *stream) {
    using namespace et;
    ET_REQUIRE(out && in && weight && bias, ET_ERR_INVALID_ARG, "et_row_spmm_add_bias: null pointer");
    ET_REQUIRE(M >= 0 && N > 0 && K > 0, ET_ERR_INVALID_ARG,
               "et_row_spmm_add_bias: M=%d N=%d K=%d", M, N, K);
    ET_REQUIRE(N % 16 == 0 && K % 16 == 0, ET_ERR_UNSUPPORTED,
               "et_row_spmm_add_bias: N=%d and K=%d must be multiples of 16", N, K);
    ET_REQUIRE(aligned16(out) && aligned16(in) && aligned16(weight) && aligned16(bias),
               ET_ERR_ALIGNMENT, "et_row_spmm_add_bias: pointers must be 16-byte aligned");
    if (M == 0)
        return ET_OK;
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
    return tile_launch(&p, 1, static_cast<const f16 *>(in), M, K, KC, nchunk, false, TL_DENSE,
                       static_cast<hipStream_t>(stream));
}

// ---------------------------------------------------------------------------
// plans
// ---------------------------------------------------------------------------
struct et_tile_plan {
    int in_feat, out_feat, ntile, KC, nchunk;
    et::f16 *d_data;
    int *d_cptr;
    int *d_row_offset;
    et::f16 *d_bias;
};

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
    // order each block-row's tiles by column; build the per-chunk CSR
    std::vector<int> order(ntile);
    std::iota(order.begin(), order.end(), 0);
    for (int bn = 0; bn < nbr; bn++)
        std::stable_sort(order.begin() + row_ptr[bn], order.begin() + row_ptr[bn + 1],
                         [&](int x, int y) { return row_offset[x] < row_offset[y]; });
    std::vector<int> off(ntile), cptr((size_t)nbr * nchunk + 1);
    std::vector<uint16_t> packed((size_t)ntile * 256);
    const uint16_t *src = static_cast<const uint16_t *>(data);
    for (int i = 0; i < ntile; i++) {
        off[i] = row_offset[order[i]];
        memcpy(&packed[(size_t)i * 256], src + (size_t)order[i] * 256, 512);
    }
    for (int bn = 0; bn < nbr; bn++) {
        int i = row_ptr[bn];
        for (int c = 0; c < nchunk; c++) {
            while (i < row_ptr[bn + 1] && off[i] < c * KC)
                i++;
            cptr[(size_t)bn * nchunk + c] = i;
        }
    }
    cptr[(size_t)nbr * nchunk] = ntile;

    et_tile_plan *p = new et_tile_plan();
    memset(p, 0, sizeof(*p));
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
                       plans[0]->nchunk, false, TL_CSR, static_cast<hipStream_t>(stream));
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
    return tile_launch(&pr, 1, static_cast<const f16 *>(X), M, plan->in_feat, plan->KC,
                       plan->nchunk, gelu != 0, TL_CSR, static_cast<hipStream_t>(stream));
}
