// Fused skip connection + LayerNorm for gfx950.
//
// Math of kernels/skip_layernorm.cu:4-43 (reference v1): x = half(a + skip),
// fp32 mean and biased two-pass variance over the row, rstd =
// rsqrt(var + 1e-6), y = (x-mean)*rstd*gamma + beta rounded to half, in place
// on `a`.  Pure streaming op: 3 x size x 2 bytes per row, so the layout aims
// at HBM bandwidth only — one wave64 per row, 16-byte loads per lane, the row
// kept in registers between the passes, shuffle reductions, no LDS.
#include "common.h"

namespace et {

template <bool NT>
__device__ __forceinline__ f16x8 ln_load(const f16 *row, int chunk) {
    if (NT)
        return __builtin_bit_cast(f16x8, __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(row) + chunk));
    return reinterpret_cast<const f16x8 *>(row)[chunk];
}

// One wave handles ROWS consecutive rows, one after the other; a row is held
// as NCH = ceil(size / 512) chunks of 8 halves per lane, chunk c of a row in
// lane c % 64 (the fused linear + LayerNorm kernels keep a row the same way,
// so the row statistics are summed in the same order and both give the same
// bits).  Only the last chunk can reach past the row: its lanes beyond the
// end load the row's last chunk instead (no branch around any load, so all of
// a row's loads are in flight together) and are masked out of the sums and the
// store.  The next row's loads are issued before the current row is reduced,
// so every wave keeps reads in flight while it computes and stores.
// NT: the row operands are loaded with the non-temporal hint - for launches
// whose operands exceed the last-level cache (streaming from HBM: 131072 rows
// of 768 98 -> 85 us); smaller ones are faster with ordinary loads (their
// operands are usually still cached from the kernel that produced them).
// NTS: the rows are also stored with the non-temporal hint - where the in/out
// operand alone is well beyond the last-level cache (524288 rows of 768:
// 440 -> 376 us, 5.5 -> 6.4 TB/s; up to 300 MB per operand the plain store is
// 2-4 % faster).
template <int NCH, int ROWS, bool NT, bool NTS = false>
__global__ void __launch_bounds__(256)
skip_layernorm_vec_kernel(f16 *__restrict__ in_out, const f16 *__restrict__ skip,
                          const f16 *__restrict__ gamma,
                          const f16 *__restrict__ beta, int num, int size, float inv_n) {
    typedef f16x8 vec;
    constexpr int CW = 8;
    typedef _Float16 h2 __attribute__((ext_vector_type(2)));
    const int wave = threadIdx.x >> 6;
    const int lane = threadIdx.x & 63;
    const long row0 = ((long)blockIdx.x * 4 + wave) * ROWS;
    if (row0 >= num)
        return;
    const int nchunk = size / CW;
    const bool last_ok = lane + (NCH - 1) * 64 < nchunk;
    int ci[NCH]; // this lane's chunk of each load
#pragma unroll
    for (int i = 0; i < NCH; i++)
        ci[i] = i == NCH - 1 ? min(lane + i * 64, nchunk - 1) : lane + i * 64;
    const vec *g = reinterpret_cast<const vec *>(gamma);
    const vec *b = reinterpret_cast<const vec *>(beta);
    vec zero;
#pragma unroll
    for (int j = 0; j < CW; j++)
        zero[j] = (f16)0;
    // an opaque 1.0: fma(x, one, -mean) on a half x is one mixed-precision
    // instruction, (float)x - mean is a conversion and a subtraction
    float one = 1.0f;
    asm("" : "+s"(one));

    vec an[NCH], sn[NCH]; // next row, raw
    // gamma and beta are requested together with the first row: asked for only
    // where they are used, after the reductions, each wave would wait out two
    // more memory latencies before its stores
    vec gg[NCH], bb[NCH];
#pragma unroll
    for (int i = 0; i < NCH; i++) {
        an[i] = ln_load<NT>(in_out + row0 * size, ci[i]);
        sn[i] = ln_load<NT>(skip + row0 * size, ci[i]);
    }
#pragma unroll
    for (int i = 0; i < NCH; i++) {
        gg[i] = g[ci[i]];
        bb[i] = b[ci[i]];
    }
#pragma unroll
    for (int r = 0; r < ROWS; r++) {
        const long row = row0 + r;
        if (row >= num)
            break;
        vec x[NCH];
        float sum = 0.f;
#pragma unroll
        for (int i = 0; i < NCH; i++) {
            x[i] = an[i] + sn[i]; // half add, one rounding (kernels/skip_layernorm.cu:20)
            if (i == NCH - 1)
                x[i] = last_ok ? x[i] : zero;
            // pairs of halves summed in fp32 by the dot-product unit
#pragma unroll
            for (int j = 0; j < CW; j += 2)
                sum = __builtin_amdgcn_fdot2(h2{x[i][j], x[i][j + 1]}, h2{(f16)1, (f16)1}, sum, false);
        }
        if (r + 1 < ROWS && row + 1 < num) {
#pragma unroll
            for (int i = 0; i < NCH; i++) {
                an[i] = ln_load<NT>(in_out + (row + 1) * size, ci[i]);
                sn[i] = ln_load<NT>(skip + (row + 1) * size, ci[i]);
            }
        }
        const float mean = wave_sum(sum) * inv_n;
        const float neg_mean = -mean;
        float var = 0.f;
#pragma unroll
        for (int i = 0; i < NCH; i++) {
            if (i < NCH - 1 || last_ok) {
#pragma unroll
                for (int j = 0; j < CW; j++) {
                    const float d = __builtin_fmaf((float)x[i][j], one, neg_mean); // x - mean, exactly
                    var += d * d;
                }
            }
        }
        const float rstd = rsqrtf(wave_sum(var) * inv_n + 1e-6f);
        const float shift = -mean * rstd;
        vec *a = reinterpret_cast<vec *>(in_out + row * size);
#pragma unroll
        for (int i = 0; i < NCH; i++) {
            vec y;
#pragma unroll
            for (int j = 0; j < CW; j++) // ((x - mean) * rstd) * gamma + beta, the first step as one fma
                y[j] = (f16)(__builtin_fmaf((float)x[i][j], rstd, shift) * (float)gg[i][j] + (float)bb[i][j]);
            if (i < NCH - 1 || last_ok) {
                if (NTS)
                    __builtin_nontemporal_store(__builtin_bit_cast(u32x4, y), reinterpret_cast<u32x4 *>(a) + ci[i]);
                else
                    a[ci[i]] = y;
            }
        }
    }
}

// The same for a compact operand: a[r][col_id[j]] = compact[r][j] for j < n,
// every other column of a zero (the output of a row-pruned linear,
// kernels/linear.cu:30-32, expanded to model width), out = LayerNorm(a + skip).
// One wave per row: the wave builds the expanded row in its own LDS strip
// (zero fill, then 2-byte scattered writes), reads it back in the chunk layout
// of the kernel above and goes on with the same arithmetic.
template <int NCH>
__global__ void __launch_bounds__(256)
scatter_skip_layernorm_kernel(f16 *__restrict__ out, const f16 *__restrict__ compact,
                              const int *__restrict__ col_id, int n, int ld_in,
                              const f16 *skip, const f16 *__restrict__ gamma,
                              const f16 *__restrict__ beta, int num, int size, float inv_n) {
    typedef f16x8 vec;
    typedef _Float16 h2 __attribute__((ext_vector_type(2)));
    extern __shared__ __attribute__((aligned(16))) unsigned char ln_smem[];
    const int wave = threadIdx.x >> 6;
    const int lane = threadIdx.x & 63;
    const long row = (long)blockIdx.x * 4 + wave;
    if (row >= num)
        return;
    f16 *strip = reinterpret_cast<f16 *>(ln_smem) + wave * (size + 8); // (the 8 halves behind a row take the writes of lanes past n)
    const int nchunk = size >> 3;
    const bool last_ok = lane + (NCH - 1) * 64 < nchunk;
    int ci[NCH];
#pragma unroll
    for (int i = 0; i < NCH; i++)
        ci[i] = i == NCH - 1 ? min(lane + i * 64, nchunk - 1) : lane + i * 64;
    const vec zero = vec{0, 0, 0, 0, 0, 0, 0, 0};
    float one = 1.0f;
    asm("" : "+s"(one));

    vec sn[NCH], gg[NCH], bb[NCH];
#pragma unroll
    for (int i = 0; i < NCH; i++)
        sn[i] = reinterpret_cast<const vec *>(skip + row * size)[ci[i]];
#pragma unroll
    for (int i = 0; i < NCH; i++) {
        gg[i] = reinterpret_cast<const vec *>(gamma)[ci[i]];
        bb[i] = reinterpret_cast<const vec *>(beta)[ci[i]];
    }
#pragma unroll
    for (int i = 0; i < NCH; i++)
        if (i < NCH - 1 || last_ok)
            reinterpret_cast<vec *>(strip)[ci[i]] = zero;
    // (LDS operations of one wave execute in order; the fences keep the compiler
    // from reordering the strip's writes and reads, which touch other lanes' data)
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    for (int j0 = lane * 8; j0 < n; j0 += 64 * 8) { // eight compact values per lane and step
        const vec v = *reinterpret_cast<const vec *>(compact + row * ld_in + j0);
#pragma unroll
        for (int k = 0; k < 8; k++) {
            const int c = col_id[min(j0 + k, n - 1)];
            strip[j0 + k < n ? c : size] = v[k];
        }
    }
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");

    vec x[NCH];
    float sum = 0.f;
#pragma unroll
    for (int i = 0; i < NCH; i++) {
        x[i] = reinterpret_cast<const vec *>(strip)[ci[i]] + sn[i]; // half add, one rounding
        if (i == NCH - 1)
            x[i] = last_ok ? x[i] : zero;
#pragma unroll
        for (int j = 0; j < 8; j += 2)
            sum = __builtin_amdgcn_fdot2(h2{x[i][j], x[i][j + 1]}, h2{(f16)1, (f16)1}, sum, false);
    }
    const float mean = wave_sum(sum) * inv_n;
    const float neg_mean = -mean;
    float var = 0.f;
#pragma unroll
    for (int i = 0; i < NCH; i++) {
        if (i < NCH - 1 || last_ok) {
#pragma unroll
            for (int j = 0; j < 8; j++) {
                const float d = __builtin_fmaf((float)x[i][j], one, neg_mean);
                var += d * d;
            }
        }
    }
    const float rstd = rsqrtf(wave_sum(var) * inv_n + 1e-6f);
    const float shift = -mean * rstd;
    vec *a = reinterpret_cast<vec *>(out + row * size);
#pragma unroll
    for (int i = 0; i < NCH; i++) {
        vec y;
#pragma unroll
        for (int j = 0; j < 8; j++)
            y[j] = (f16)(__builtin_fmaf((float)x[i][j], rstd, shift) * (float)gg[i][j] + (float)bb[i][j]);
        if (i < NCH - 1 || last_ok)
            a[ci[i]] = y;
    }
}

// Any size, any alignment: one wave per row, three passes over memory.
__global__ void __launch_bounds__(256)
skip_layernorm_generic_kernel(f16 *__restrict__ in_out, const f16 *__restrict__ skip,
                              const f16 *__restrict__ gamma,
                              const f16 *__restrict__ beta, int num, int size) {
    const int wave = threadIdx.x >> 6;
    const int lane = threadIdx.x & 63;
    const long row = (long)blockIdx.x * 4 + wave;
    if (row >= num)
        return;
    f16 *a = in_out + row * size;
    const f16 *s = skip + row * size;
    float sum = 0.f;
    for (int c = lane; c < size; c += 64) {
        const f16 x = a[c] + s[c];
        a[c] = x; // same lane re-reads it below
        sum += (float)x;
    }
    const float mean = wave_sum(sum) / (float)size;
    float var = 0.f;
    for (int c = lane; c < size; c += 64) {
        const float d = (float)a[c] - mean;
        var += d * d;
    }
    const float rstd = rsqrtf(wave_sum(var) / (float)size + 1e-6f);
    for (int c = lane; c < size; c += 64)
        a[c] = (f16)(((float)a[c] - mean) * rstd * (float)gamma[c] + (float)beta[c]);
}

int g_ln_rows = 0; // et_tuning_set("ln_rows"): 0 = automatic
void set_ln_rows(int v) { g_ln_rows = v; }

} // namespace et

extern "C" int et_skip_layernorm(void *in_out, const void *skip, const void *gamma,
                                 const void *beta, int num, int size, void *stream) {
    using namespace et;
    ET_REQUIRE(in_out && skip && gamma && beta, ET_ERR_INVALID_ARG,
               "et_skip_layernorm: null pointer");
    ET_REQUIRE(num >= 0 && size > 0, ET_ERR_INVALID_ARG,
               "et_skip_layernorm: num=%d size=%d", num, size);
    if (num == 0)
        return ET_OK;
    hipStream_t st = static_cast<hipStream_t>(stream);
    f16 *a = static_cast<f16 *>(in_out);
    const f16 *s = static_cast<const f16 *>(skip);
    const f16 *g = static_cast<const f16 *>(gamma);
    const f16 *b = static_cast<const f16 *>(beta);
    const dim3 block(256);
    const bool vec = (size % 8 == 0) && size <= 4096 && aligned16(in_out) &&
                     aligned16(skip) && aligned16(gamma) && aligned16(beta);
    if (!vec) {
        hipLaunchKernelGGL(skip_layernorm_generic_kernel, dim3((num + 3) / 4), block, 0, st, a, s, g, b, num, size);
    } else {
        const int nch8 = (size / 8 + 63) / 64;
        const float inv_n = 1.0f / (float)size;
        // rows per wave: enough waves to fill the chip first (256 CUs x 32 waves); two from there
        // (four rows per wave measured 4-5 % slower from 131072 rows up)
        // both operands together beyond the 256 MB last-level cache: streaming loads, two rows per wave
        const bool nt = g_ln_rows == 0 && (size_t)num * size * 4 > (size_t)256 << 20;
        // the in/out operand alone well beyond it (measured at 768 halves per row: 302 MB are 4 % faster
        // with plain stores, 403 MB 17 % faster with non-temporal ones)
        const bool nts = nt && (size_t)num * size * 2 > (size_t)320 << 20;
        const int rows = nt ? 2 : g_ln_rows > 0 ? g_ln_rows : (num >= 2 * 8192 ? 2 : 1);
        const dim3 grid((num + 4 * rows - 1) / (4 * rows));
#define ET_LN_CASE(NCH_)                                                                          \
    {                                                                                             \
    if (nts)                                                                                      \
        hipLaunchKernelGGL((skip_layernorm_vec_kernel<NCH_, 2, true, true>), grid, block, 0, st, a, s, g, b, num, size, inv_n); \
    else if (nt)                                                                                  \
        hipLaunchKernelGGL((skip_layernorm_vec_kernel<NCH_, 2, true>), grid, block, 0, st, a, s, g, b, num, size, inv_n); \
    else if (rows >= 4)                                                                           \
        hipLaunchKernelGGL((skip_layernorm_vec_kernel<NCH_, 4, false>), grid, block, 0, st, a, s, g, b, num, size, inv_n); \
    else if (rows >= 2)                                                                           \
        hipLaunchKernelGGL((skip_layernorm_vec_kernel<NCH_, 2, false>), grid, block, 0, st, a, s, g, b, num, size, inv_n); \
    else                                                                                          \
        hipLaunchKernelGGL((skip_layernorm_vec_kernel<NCH_, 1, false>), grid, block, 0, st, a, s, g, b, num, size, inv_n); \
    }
        {
            switch (nch8) { // size <= 4096: at most 8 chunks
            case 1: ET_LN_CASE(1) break;
            case 2: ET_LN_CASE(2) break;
            case 3: ET_LN_CASE(3) break;
            case 4: ET_LN_CASE(4) break;
            case 5: ET_LN_CASE(5) break;
            case 6: ET_LN_CASE(6) break;
            case 7: ET_LN_CASE(7) break;
            default: ET_LN_CASE(8) break;
            }
        }
#undef ET_LN_CASE
    }
    return launch_status("et_skip_layernorm launch");
}

extern "C" int et_scatter_skip_layernorm(void *out, const void *compact, const int *col_id, int n,
                                         int ld_in, const void *skip, const void *gamma,
                                         const void *beta, int num, int size, void *stream) {
    using namespace et;
    ET_REQUIRE(out && compact && col_id && skip && gamma && beta, ET_ERR_INVALID_ARG,
               "et_scatter_skip_layernorm: null pointer");
    ET_REQUIRE(num >= 0 && size > 0 && n >= 0 && n <= ld_in && n <= size, ET_ERR_INVALID_ARG,
               "et_scatter_skip_layernorm: num=%d size=%d n=%d ld_in=%d", num, size, n, ld_in);
    ET_REQUIRE(out != compact, ET_ERR_INVALID_ARG, "et_scatter_skip_layernorm: out must not alias compact");
    if (num == 0)
        return ET_OK;
    const bool vec = size % 8 == 0 && size <= 4096 && ld_in % 8 == 0 && n > 0 && aligned16(out) &&
                     aligned16(compact) && aligned16(skip) && aligned16(gamma) && aligned16(beta);
    if (!vec) { // the two steps, one after the other
        ET_REQUIRE(out != skip, ET_ERR_INVALID_ARG,
                   "et_scatter_skip_layernorm: out must not alias skip for these sizes");
        const int rc = et_scatter_cols(out, compact, col_id, num, n, ld_in, size, stream);
        return rc != ET_OK ? rc : et_skip_layernorm(out, skip, gamma, beta, num, size, stream);
    }
    hipStream_t st = static_cast<hipStream_t>(stream);
    const dim3 grid((num + 3) / 4), block(256);
    const size_t lds = (size_t)4 * (size + 8) * sizeof(f16);
    const float inv_n = 1.0f / (float)size;
#define ET_SLN_CASE(NCH_)                                                                         \
    hipLaunchKernelGGL((scatter_skip_layernorm_kernel<NCH_>), grid, block, lds, st,               \
                       static_cast<f16 *>(out), static_cast<const f16 *>(compact), col_id, n, ld_in, \
                       static_cast<const f16 *>(skip), static_cast<const f16 *>(gamma),           \
                       static_cast<const f16 *>(beta), num, size, inv_n);                         \
    break;
    switch ((size / 8 + 63) / 64) {
    case 1: ET_SLN_CASE(1)
    case 2: ET_SLN_CASE(2)
    case 3: ET_SLN_CASE(3)
    case 4: ET_SLN_CASE(4)
    case 5: ET_SLN_CASE(5)
    case 6: ET_SLN_CASE(6)
    case 7: ET_SLN_CASE(7)
    default: ET_SLN_CASE(8)
    }
#undef ET_SLN_CASE
    return launch_status("et_scatter_skip_layernorm launch");
}
