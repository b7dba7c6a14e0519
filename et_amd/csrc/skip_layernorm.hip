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

// One wave handles ROWS consecutive rows, one after the other; a row is held
// as NCH chunks of 8 halves per lane.  The next row's loads are issued before
// the current row is reduced, so every wave keeps reads in flight while it
// computes and stores (with one row per wave the whole grid is resident at
// once and all waves read, then all waves write).
template <int NCH, int ROWS>
__global__ void __launch_bounds__(256)
skip_layernorm_vec_kernel(f16 *__restrict__ in_out, const f16 *__restrict__ skip,
                          const f16 *__restrict__ gamma,
                          const f16 *__restrict__ beta, int num, int size) {
    const int wave = threadIdx.x >> 6;
    const int lane = threadIdx.x & 63;
    const long row0 = ((long)blockIdx.x * 4 + wave) * ROWS;
    if (row0 >= num)
        return;
    const int nchunk = size >> 3;
    const float inv_n = 1.0f / (float)size;
    const f16x8 *g = reinterpret_cast<const f16x8 *>(gamma);
    const f16x8 *b = reinterpret_cast<const f16x8 *>(beta);
    const f16x8 zero8 = f16x8{0, 0, 0, 0, 0, 0, 0, 0};

    f16x8 an[NCH], sn[NCH]; // next row, raw
#pragma unroll
    for (int i = 0; i < NCH; i++) {
        const int c = lane + i * 64;
        an[i] = zero8;
        sn[i] = zero8;
        if (c < nchunk) {
            an[i] = reinterpret_cast<const f16x8 *>(in_out + row0 * size)[c];
            sn[i] = reinterpret_cast<const f16x8 *>(skip + row0 * size)[c];
        }
    }
#pragma unroll
    for (int r = 0; r < ROWS; r++) {
        const long row = row0 + r;
        if (row >= num)
            break;
        f16x8 x[NCH];
        float sum = 0.f;
#pragma unroll
        for (int i = 0; i < NCH; i++) {
            x[i] = an[i] + sn[i]; // half add, one rounding (kernels/skip_layernorm.cu:20)
            // pairs of halves summed in fp32 by the dot-product unit (chunks
            // beyond the row are zero)
            typedef _Float16 h2 __attribute__((ext_vector_type(2)));
#pragma unroll
            for (int j = 0; j < 8; j += 2)
                sum = __builtin_amdgcn_fdot2(h2{x[i][j], x[i][j + 1]}, h2{(f16)1, (f16)1}, sum, false);
        }
        if (r + 1 < ROWS && row + 1 < num) {
#pragma unroll
            for (int i = 0; i < NCH; i++) {
                const int c = lane + i * 64;
                if (c < nchunk) {
                    an[i] = reinterpret_cast<const f16x8 *>(in_out + (row + 1) * size)[c];
                    sn[i] = reinterpret_cast<const f16x8 *>(skip + (row + 1) * size)[c];
                }
            }
        }
        const float mean = wave_sum(sum) * inv_n;
        float var = 0.f;
#pragma unroll
        for (int i = 0; i < NCH; i++) {
            const int c = lane + i * 64;
            if (c < nchunk) {
#pragma unroll
                for (int j = 0; j < 8; j++) {
                    const float d = (float)x[i][j] - mean;
                    var += d * d;
                }
            }
        }
        const float rstd = rsqrtf(wave_sum(var) * inv_n + 1e-6f);
        const float shift = -mean * rstd;
        f16x8 *a = reinterpret_cast<f16x8 *>(in_out + row * size);
#pragma unroll
        for (int i = 0; i < NCH; i++) {
            const int c = lane + i * 64;
            if (c < nchunk) {
                const f16x8 gg = g[c], bb = b[c];
                f16x8 y;
#pragma unroll
                for (int j = 0; j < 8; j++) // ((x - mean) * rstd) * gamma + beta, the first step as one fma
                    y[j] = (f16)(__builtin_fmaf((float)x[i][j], rstd, shift) * (float)gg[j] + (float)bb[j]);
                a[c] = y;
            }
        }
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
        const int nch = (size / 8 + 63) / 64;
        // rows per wave: enough waves to fill the chip first (256 CUs x 32 waves)
        const int rows = g_ln_rows > 0 ? g_ln_rows : (num >= 4 * 8192 ? 4 : num >= 2 * 8192 ? 2 : 1);
        const dim3 grid((num + 4 * rows - 1) / (4 * rows));
#define ET_LN_CASE(NCH_)                                                                          \
    if (rows >= 4)                                                                                \
        hipLaunchKernelGGL((skip_layernorm_vec_kernel<NCH_, 4>), grid, block, 0, st, a, s, g, b, num, size); \
    else if (rows >= 2)                                                                           \
        hipLaunchKernelGGL((skip_layernorm_vec_kernel<NCH_, 2>), grid, block, 0, st, a, s, g, b, num, size); \
    else                                                                                          \
        hipLaunchKernelGGL((skip_layernorm_vec_kernel<NCH_, 1>), grid, block, 0, st, a, s, g, b, num, size);
        if (nch <= 1) { ET_LN_CASE(1) }
        else if (nch <= 2) { ET_LN_CASE(2) }
        else if (nch <= 4) { ET_LN_CASE(4) }
        else { ET_LN_CASE(8) }
#undef ET_LN_CASE
    }
    return launch_status("et_skip_layernorm launch");
}
