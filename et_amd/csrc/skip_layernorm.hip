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
// as NCH = ceil(size / 512) chunks of 8 halves per lane, chunk c of a row in
// lane c % 64 (the fused linear + LayerNorm kernels keep a row the same way,
// so the row statistics are summed in the same order and both give the same
// bits).  Only the last chunk can reach past the row: its lanes beyond the
// end load the row's last chunk instead (no branch around any load, so all of
// a row's loads are in flight together) and are masked out of the sums and the
// store.  The next row's loads are issued before the current row is reduced,
// so every wave keeps reads in flight while it computes and stores.
template <int NCH, int ROWS>
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
        an[i] = reinterpret_cast<const vec *>(in_out + row0 * size)[ci[i]];
        sn[i] = reinterpret_cast<const vec *>(skip + row0 * size)[ci[i]];
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
                an[i] = reinterpret_cast<const vec *>(in_out + (row + 1) * size)[ci[i]];
                sn[i] = reinterpret_cast<const vec *>(skip + (row + 1) * size)[ci[i]];
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
            if (i < NCH - 1 || last_ok)
                a[ci[i]] = y;
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
        const int nch8 = (size / 8 + 63) / 64;
        const float inv_n = 1.0f / (float)size;
        // rows per wave: enough waves to fill the chip first (256 CUs x 32 waves)
        const int rows = g_ln_rows > 0 ? g_ln_rows : (num >= 4 * 8192 ? 4 : num >= 2 * 8192 ? 2 : 1);
        const dim3 grid((num + 4 * rows - 1) / (4 * rows));
#define ET_LN_CASE(NCH_)                                                                          \
    {                                                                                             \
    if (rows >= 4)                                                                                \
        hipLaunchKernelGGL((skip_layernorm_vec_kernel<NCH_, 4>), grid, block, 0, st, a, s, g, b, num, size, inv_n); \
    else if (rows >= 2)                                                                           \
        hipLaunchKernelGGL((skip_layernorm_vec_kernel<NCH_, 2>), grid, block, 0, st, a, s, g, b, num, size, inv_n); \
    else                                                                                          \
        hipLaunchKernelGGL((skip_layernorm_vec_kernel<NCH_, 1>), grid, block, 0, st, a, s, g, b, num, size, inv_n); \
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
