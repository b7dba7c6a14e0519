// Microbenchmarks of the three delivery paths that bound the tile kernels and
// the attention kernel on gfx950.  A library of its own (libet_microbench.so, next to
// this file; it is not part of the encoder's C ABI), loaded by bench.py --micro:
//   * LDS fragment reads (ds_read_b128 in the X-panel / K-tile access pattern),
//   * the weight stream (global_load_dwordx4, one kilobyte per wave request,
//     from a buffer that stays in L2),
//   * matrix-unit and vector-ALU co-execution: MFMAs and vector instructions
//     interleaved in ONE wave, against the same work in separate waves of a SIMD.
// Every kernel runs a fixed number of iterations; results are seconds, turned
// into bytes / instructions per nanosecond and CU by the caller.  The matrix
// unit's own loop (16 cycles per v_mfma_f32_16x16x32_f16 and SIMD) gives the
// clock that the other figures are quoted against.
#include "../csrc/common.h"

namespace et {

// MODE 0: the 16 rows x 4 k-groups pattern of a fragment read (lane: row c16 at `stride` bytes, 16 bytes at
// (lane / 16) * 16), 1: 64 lanes x 16 consecutive bytes
template <int MODE>
__global__ void __launch_bounds__(1024) mb_lds_kernel(float *out, int stride, int iters) {
    extern __shared__ __attribute__((aligned(16))) char mb_smem[];
    for (int i = threadIdx.x; i < 60000 / 4; i += blockDim.x)
        reinterpret_cast<float *>(mb_smem)[i] = (float)i;
    __syncthreads();
    const int lane = threadIdx.x & 63, c16 = lane & 15, g4 = lane >> 4;
    const unsigned base = MODE == 0 ? c16 * stride + g4 * 16 : lane * 16;
    f32x4 acc = {0, 0, 0, 0};
    for (int it = 0; it < iters; it++) {
        f32x4 v0, v1, v2, v3;
        asm volatile("ds_read_b128 %0, %1 offset:0" : "=v"(v0) : "v"(base));
        asm volatile("ds_read_b128 %0, %1 offset:32" : "=v"(v1) : "v"(base));
        asm volatile("ds_read_b128 %0, %1 offset:64" : "=v"(v2) : "v"(base));
        asm volatile("ds_read_b128 %0, %1 offset:96" : "=v"(v3) : "v"(base));
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        acc += v0 + v1 + v2 + v3;
    }
    out[blockIdx.x * blockDim.x + threadIdx.x] = acc[0] + acc[3];
}

// every wave walks its own part of `w` (bytes_per_wave, a multiple of 4 KB) `rounds` times, four
// one-kilobyte requests in flight
__global__ void __launch_bounds__(1024) mb_wstream_kernel(float *out, const f16 *w, int bytes_per_wave, int rounds) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const char *base = reinterpret_cast<const char *>(w) + (size_t)wave * bytes_per_wave + lane * 16;
    f16x8 acc = {0, 0, 0, 0, 0, 0, 0, 0};
    for (int r = 0; r < rounds; r++)
        for (int off = 0; off < bytes_per_wave; off += 4096) {
            const f16x8 a = *reinterpret_cast<const f16x8 *>(base + off);
            const f16x8 b = *reinterpret_cast<const f16x8 *>(base + off + 1024);
            const f16x8 c = *reinterpret_cast<const f16x8 *>(base + off + 2048);
            const f16x8 d = *reinterpret_cast<const f16x8 *>(base + off + 3072);
            acc += (a + b) + (c + d);
        }
    out[blockIdx.x * blockDim.x + threadIdx.x] = (float)acc[0] + (float)acc[7];
}

__device__ __forceinline__ float mb_mfma_loop(int iters, int lane) {
    f16x8 a, b;
    for (int i = 0; i < 8; i++) {
        a[i] = (f16)(lane * 0.01f + i);
        b[i] = (f16)(i * 0.5f);
    }
    f32x4 c0 = {0, 0, 0, 0}, c1 = c0, c2 = c0, c3 = c0;
    for (int it = 0; it < iters; it++) {
#pragma unroll
        for (int r = 0; r < 4; r++) {
            c0 = mfma16x16x32(a, b, c0);
            c1 = mfma16x16x32(a, b, c1);
            c2 = mfma16x16x32(a, b, c2);
            c3 = mfma16x16x32(a, b, c3);
        }
    }
    return c0[0] + c1[1] + c2[2] + c3[3];
}
__device__ __forceinline__ float mb_valu_loop(int iters, int lane) { // 64 v_fma_f32 per iteration
    float v[8];
    for (int i = 0; i < 8; i++)
        v[i] = lane * 0.001f + i;
    for (int it = 0; it < iters; it++) {
#pragma unroll
        for (int r = 0; r < 8; r++)
#pragma unroll
            for (int i = 0; i < 8; i++)
                asm volatile("v_fma_f32 %0, %0, %1, %1" : "+v"(v[i]) : "v"(1.0001f));
    }
    float s = 0;
    for (int i = 0; i < 8; i++)
        s += v[i];
    return s;
}
// 16 MFMAs and 64 FMAs per iteration, strictly alternating in one wave (1 MFMA, 4 FMAs)
__device__ __forceinline__ float mb_mixed_loop(int iters, int lane) {
    f16x8 a, b;
    for (int i = 0; i < 8; i++) {
        a[i] = (f16)(lane * 0.01f + i);
        b[i] = (f16)(i * 0.5f);
    }
    f32x4 c[4] = {{0, 0, 0, 0}, {0, 0, 0, 0}, {0, 0, 0, 0}, {0, 0, 0, 0}};
    float v[8];
    for (int i = 0; i < 8; i++)
        v[i] = lane * 0.001f + i;
    for (int it = 0; it < iters; it++) {
#pragma unroll
        for (int r = 0; r < 16; r++) {
            asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+v"(c[r & 3]) : "v"(a), "v"(b));
#pragma unroll
            for (int i = 0; i < 4; i++)
                asm volatile("v_fma_f32 %0, %0, %1, %1" : "+v"(v[(r & 1) * 4 + i]) : "v"(1.0001f));
        }
    }
    float s = c[0][0] + c[1][1] + c[2][2] + c[3][3];
    for (int i = 0; i < 8; i++)
        s += v[i];
    return s;
}
// MODE 0: every wave MFMAs, 1: every wave FMAs, 2: every wave the alternating mix, 3: waves 0-3 (one per
// SIMD) MFMAs and waves 4-7 (the same SIMDs) FMAs
template <int MODE>
__global__ void __launch_bounds__(1024) mb_coexec_kernel(float *out, int iters) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    float s;
    if (MODE == 0 || (MODE == 3 && wave < 4))
        s = mb_mfma_loop(iters, lane);
    else if (MODE == 2)
        s = mb_mixed_loop(iters, lane);
    else
        s = mb_valu_loop(iters, lane);
    out[blockIdx.x * blockDim.x + threadIdx.x] = s;
}

template <class Launch>
static int mb_time(Launch launch, double *seconds) {
    hipEvent_t e0 = nullptr, e1 = nullptr;
    hipError_t err = hipEventCreate(&e0);
    if (err == hipSuccess)
        err = hipEventCreate(&e1);
    float ms = 0.f;
    for (int rep = 0; rep < 3 && err == hipSuccess; rep++) { // the last of three launches counts
        err = hipEventRecord(e0, nullptr);
        if (err != hipSuccess)
            break;
        launch();
        err = hipEventRecord(e1, nullptr);
        if (err == hipSuccess)
            err = hipEventSynchronize(e1);
        if (err == hipSuccess)
            err = hipEventElapsedTime(&ms, e0, e1);
    }
    if (e0)
        (void)hipEventDestroy(e0);
    if (e1)
        (void)hipEventDestroy(e1);
    if (err != hipSuccess)
        return hip_fail(err, "microbenchmark timing");
    *seconds = ms * 1e-3;
    return launch_status("microbenchmark launch");
}

// device memory that is released on every way out
struct MbBuffer {
    void *p = nullptr;
    ~MbBuffer() {
        if (p)
            (void)hipFree(p);
    }
    hipError_t alloc(size_t bytes) { return hipMalloc(&p, bytes); }
};

} // namespace et

// what 0: LDS fragment reads (ds_read_b128); p0 = row stride in bytes of the 16-row x 64-byte fragment pattern, a
//         multiple of 16 (0: 64 x 16 consecutive bytes), p1 = waves per CU.  units = bytes read per CU.
// what 1: the weight stream: one-kilobyte global_load_dwordx4 requests, four in flight per wave, from 2 MiB that
//         stay in L2; p1 = waves per CU.  units = bytes requested per CU.
// what 2: matrix unit and vector ALU: p0 = 0 every wave issues MFMAs only, 1 v_fma_f32 only (four per MFMA of mode
//         0), 2 both, strictly alternating in every wave, 3 four waves MFMAs and four waves (on the same SIMDs) the
//         FMAs; p1 = waves per CU (modes 0-2).  units = v_mfma_f32_16x16x32_f16 per MFMA-issuing wave.
// seconds = duration of one launch on every CU of the device.  Allocates and synchronises.
extern "C" int et_microbench(int what, int p0, int p1, double *seconds, double *units_per_cu) {
    using namespace et;
    ET_REQUIRE(seconds && units_per_cu, ET_ERR_INVALID_ARG, "et_microbench: null pointer");
    // everything that can be refused is refused before anything is allocated
    ET_REQUIRE(what >= 0 && what <= 2, ET_ERR_INVALID_ARG, "et_microbench: what=%d", what);
    if (what == 0)
        ET_REQUIRE(p0 >= 0 && p0 % 16 == 0 && 15 * p0 + 64 + 112 <= 60000, ET_ERR_INVALID_ARG,
                   "et_microbench: stride %d (a multiple of 16 up to 3984)", p0);
    if (what == 2)
        ET_REQUIRE(p0 >= 0 && p0 <= 3, ET_ERR_INVALID_ARG, "et_microbench: mode %d", p0);
    const int cus = et_device_cu_count();
    ET_REQUIRE(cus > 0, ET_ERR_HIP, "et_microbench: no device");
    MbBuffer outb, wb;
    ET_HIP(outb.alloc((size_t)cus * 1024 * sizeof(float)));
    float *out = static_cast<float *>(outb.p);
    int rc = ET_OK;
    const int iters = 2000;
    if (what == 0) {
        const int waves = p1 > 0 && p1 <= 16 ? p1 : 16;
        if (p0 == 0)
            rc = mb_time([&] { hipLaunchKernelGGL(mb_lds_kernel<1>, dim3(cus), dim3(waves * 64), 60000, 0, out, 0, iters); }, seconds);
        else
            rc = mb_time([&] { hipLaunchKernelGGL(mb_lds_kernel<0>, dim3(cus), dim3(waves * 64), 60000, 0, out, p0, iters); }, seconds);
        *units_per_cu = (double)waves * iters * 4 * 1024; // bytes read per CU
    } else if (what == 1) { // every CU walks the same 2 MiB
        const int waves = p1 > 0 && p1 <= 16 ? p1 : 16;
        const int per_wave = (2 << 20) / 16, rounds = 8;
        ET_HIP(wb.alloc((size_t)16 * per_wave));
        ET_HIP(hipMemset(wb.p, 0, (size_t)16 * per_wave));
        const f16 *w = static_cast<const f16 *>(wb.p);
        rc = mb_time([&] { hipLaunchKernelGGL(mb_wstream_kernel, dim3(cus), dim3(waves * 64), 0, 0, out, w, per_wave, rounds); }, seconds);
        *units_per_cu = (double)waves * per_wave * rounds; // bytes requested per CU
    } else {
        const int waves = p0 == 3 ? 8 : (p1 > 0 && p1 <= 16 ? p1 : 4);
        switch (p0) {
        case 0: rc = mb_time([&] { hipLaunchKernelGGL(mb_coexec_kernel<0>, dim3(cus), dim3(waves * 64), 0, 0, out, iters); }, seconds); break;
        case 1: rc = mb_time([&] { hipLaunchKernelGGL(mb_coexec_kernel<1>, dim3(cus), dim3(waves * 64), 0, 0, out, iters); }, seconds); break;
        case 2: rc = mb_time([&] { hipLaunchKernelGGL(mb_coexec_kernel<2>, dim3(cus), dim3(waves * 64), 0, 0, out, iters); }, seconds); break;
        default: rc = mb_time([&] { hipLaunchKernelGGL(mb_coexec_kernel<3>, dim3(cus), dim3(waves * 64), 0, 0, out, iters); }, seconds); break;
        }
        *units_per_cu = (double)iters * 16; // MFMAs per MFMA wave (and 4x as many FMAs per FMA wave)
    }
    return rc;
}
