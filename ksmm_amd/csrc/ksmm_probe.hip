// Measurement aid: the rate at which the matrix cores multiply operands that are already in
// registers.  A benchmark prints it beside the kernels' own figures, as a copy kernel's rate is
// printed beside bandwidth-bound ones: with random operands the rate an MI355X sustains is well
// under the published peak (clock and power management), and no kernel can beat it.
// No counterpart in the reference.
#include "ksmm_mfma.h"

namespace ksmm {

namespace {

// 8 waves per CU, every wave 16 independent accumulator tiles' worth of work per iteration
// (two sub-steps of 8 MFMAs, as in the GEMM tiles), nothing but MFMAs in the loop.
template <int KIND>
__global__ __launch_bounds__(512, 1) void ks_mfma_probe_kernel(float *__restrict__ out, int iters, int random)
{
    const unsigned tid = threadIdx.x + blockIdx.x * 512u;
    auto rnd = [&](unsigned k) {
        unsigned s = (tid * 2654435761u + k * 40503u) * 1664525u + 1013904223u;
        s = s * 1664525u + 1013904223u;
        return random ? ((int)(s >> 16) % 2001 - 1000) / 1000.0f : 1.0f;  // uniform in [-1, 1], or all ones
    };
    float s = 0.f;
    if constexpr (KIND == 0) {  // v_mfma_f32_32x32x16_f16
        float16_t acc[8];
        half8_t a[4], b[4];
#pragma unroll
        for (int q = 0; q < 4; ++q)
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                a[q][i] = (half_t)rnd(q * 8 + i);
                b[q][i] = (half_t)(rnd(64 + q * 8 + i) * 0.125f);
            }
#pragma unroll
        for (int i = 0; i < 8; ++i)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][e] = 0.f;
        for (int it = 0; it < iters; ++it)
#pragma unroll
            for (int h = 0; h < 2; ++h)
#pragma unroll
                for (int i = 0; i < 8; ++i)
                    acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[(i >> 1) & 3], b[(i & 1) + 2 * h], acc[i], 0, 0, 0);
#pragma unroll
        for (int i = 0; i < 8; ++i) s += acc[i][0] + acc[i][7];
    } else {  // v_mfma_f32_16x16x4_f32
        float4_t acc[16];
        float a[4], b[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            a[q] = rnd(q);
            b[q] = rnd(64 + q) * 0.125f;
        }
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[i] = float4_t{0.f, 0.f, 0.f, 0.f};
        for (int it = 0; it < iters; ++it)
#pragma unroll
            for (int i = 0; i < 16; ++i)
                acc[i] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[i & 3], b[(i >> 2) & 3], acc[i], 0, 0, 0);
#pragma unroll
        for (int i = 0; i < 16; ++i) s += acc[i][0] + acc[i][3];
    }
    out[tid] = s;
}

}  // namespace

}  // namespace ksmm

extern "C" {

int64_t ksmm_mfma_probe_bytes(void) { return 256ll * 512 * (int64_t)sizeof(float); }

int ksmm_mfma_probe(int dtype, int iters, int random, void *out, int64_t out_bytes, double *flops, void *stream)
{
    using namespace ksmm;
    if (!out || !flops) return KSMM_ERR_NULL_POINTER;
    if (out_bytes < ksmm_mfma_probe_bytes() || ((uintptr_t)out & 3)) return KSMM_ERR_WORKSPACE;
    if (iters < 1 || iters > (1 << 24)) return KSMM_ERR_BAD_BATCH;
    const void *fn;
    double per_iter;  // flops per wave and iteration
    if (dtype == KSMM_F16) {
        fn = (const void *)ks_mfma_probe_kernel<0>;
        per_iter = 16 * 2.0 * 32 * 32 * 16;
    } else if (dtype == KSMM_F32) {
        fn = (const void *)ks_mfma_probe_kernel<1>;
        per_iter = 16 * 2.0 * 16 * 16 * 4;
    } else {
        return KSMM_ERR_BAD_DTYPE;
    }
    *flops = per_iter * iters * 256.0 * 8.0;
    void *args[] = {&out, &iters, &random};
    return hipLaunchKernel(fn, dim3(256), dim3(512), args, 0, (hipStream_t)stream) == hipSuccess ? KSMM_OK : KSMM_ERR_LAUNCH;
}

}  // extern "C"
