// Measurement aids of the benchmark, built into a library of their own (libksmm_bench.so): they
// are not part of the drop-in ABI.  (1) The rate at which the matrix cores multiply operands that
// are already in registers: with random operands the rate an MI355X sustains is well under the
// published peak (clock and power management), and no kernel can beat it.  (2) A copy that moves
// whole tiles with the addresses of a batch-size-last factor.  (3) A streaming copy with
// non-temporal loads and stores, the fastest way found to move bytes through this memory system.
// No counterpart in the reference.
#include "ksmm_mfma.h"
#include "ksmm_probe.h"

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


// A copy with the access pattern of a batch-size-last factor and nothing else: workgroup t moves
// the `rows` x `tile_bytes` tile of block (a_i, d_i) and batch tile nt from x to the same place
// in y, rows of a block being d rows apart.  Every load is issued before the first store, as in
// a kernel that needs the whole tile before it can produce an output row.  (With d = 1 and
// row_bytes = tile_bytes the same tiles lie in linear memory: the two rates differ little, and
// both are below a streaming copy with a few vectors per thread.)
constexpr int TC_MAX_PASSES = 48;
__global__ __launch_bounds__(256) void ks_tilecopy_probe_kernel(const uint4_t *__restrict__ x, uint4_t *__restrict__ y,
                                                           int rows, int d, int64_t row_chunks, int tile_chunks,
                                                           int n_tiles)
{
    const int tile = blockIdx.x, g = tile / n_tiles, nt = tile - g * n_tiles;
    const int a_i = g / d, d_i = g - a_i * d;
    const int rpp = 256 / tile_chunks;  // rows per pass
    const int rr = threadIdx.x / tile_chunks, cc = threadIdx.x - rr * tile_chunks;
    const int64_t chunk = (int64_t)nt * tile_chunks + cc;
    uint4_t v[TC_MAX_PASSES];
#pragma unroll
    for (int i = 0; i < TC_MAX_PASSES; ++i) {
        const int row = i * rpp + rr;
        if (row < rows && chunk < row_chunks) v[i] = x[((int64_t)(a_i * rows + row) * d + d_i) * row_chunks + chunk];
    }
#pragma unroll
    for (int i = 0; i < TC_MAX_PASSES; ++i) {
        const int row = i * rpp + rr;
        if (row < rows && chunk < row_chunks) y[((int64_t)(a_i * rows + row) * d + d_i) * row_chunks + chunk] = v[i];
    }
}

// Streaming copy: a persistent grid, every thread moves VPT 16-byte vectors per round (all loads
// of a round before its stores), consecutive threads consecutive vectors, non-temporal both ways.
constexpr int SC_VPT = 4;
__global__ __launch_bounds__(256) void ks_stream_copy_kernel(const uint4_t *__restrict__ x, uint4_t *__restrict__ y,
                                                        int64_t n_vec)
{
    const int64_t per_round = (int64_t)gridDim.x * 256 * SC_VPT;
    for (int64_t base = (int64_t)blockIdx.x * 256 * SC_VPT; base < n_vec; base += per_round) {
        uint4_t v[SC_VPT];
#pragma unroll
        for (int i = 0; i < SC_VPT; ++i) {
            const int64_t q = base + i * 256 + threadIdx.x;
            if (q < n_vec) v[i] = __builtin_nontemporal_load(x + q);
        }
#pragma unroll
        for (int i = 0; i < SC_VPT; ++i) {
            const int64_t q = base + i * 256 + threadIdx.x;
            if (q < n_vec) __builtin_nontemporal_store(v[i], y + q);
        }
    }
}

}  // namespace

}  // namespace ksmm

extern "C" {

int ksbench_stream_copy(const void *x, void *y, int64_t bytes, int workgroups, void *stream)
{
    using namespace ksmm;
    if (!x || !y) return KSMM_ERR_NULL_POINTER;
    if ((((uintptr_t)x | (uintptr_t)y) & 15) || bytes < 16 || bytes % 16) return KSMM_ERR_WORKSPACE;
    if (workgroups < 1 || workgroups > 65536) return KSMM_ERR_BAD_PATTERN;
    int64_t n_vec = bytes / 16;
    void *args[] = {(void *)&x, (void *)&y, &n_vec};
    return hipLaunchKernel((const void *)ks_stream_copy_kernel, dim3((unsigned)workgroups), dim3(256), args, 0,
                           (hipStream_t)stream) == hipSuccess
               ? KSMM_OK
               : KSMM_ERR_LAUNCH;
}

int64_t ksbench_mfma_probe_bytes(void) { return 256ll * 512 * (int64_t)sizeof(float); }

int ksbench_mfma_probe(int dtype, int iters, int random, void *out, int64_t out_bytes, double *flops, void *stream)
{
    using namespace ksmm;
    if (!out || !flops) return KSMM_ERR_NULL_POINTER;
    if (out_bytes < ksbench_mfma_probe_bytes() || ((uintptr_t)out & 3)) return KSMM_ERR_WORKSPACE;
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

int ksbench_tilecopy_probe(const void *x, void *y, int64_t row_bytes, int a, int rows, int d, int tile_bytes, void *stream)
{
    using namespace ksmm;
    if (!x || !y) return KSMM_ERR_NULL_POINTER;
    if (((uintptr_t)x | (uintptr_t)y) & 15) return KSMM_ERR_WORKSPACE;
    if (row_bytes < 16 || row_bytes % 16 || a < 1 || d < 1 || rows < 1) return KSMM_ERR_BAD_PATTERN;
    // a tile row is 16..4096 bytes, a power of two (256 threads take whole rows per pass)
    if (tile_bytes < 16 || tile_bytes > 4096 || (tile_bytes & (tile_bytes - 1))) return KSMM_ERR_BAD_PATTERN;
    const int tile_chunks = tile_bytes / 16;
    if (rows > TC_MAX_PASSES * (256 / tile_chunks)) return KSMM_ERR_BAD_PATTERN;
    const int64_t row_chunks = row_bytes / 16;
    const int64_t n_tiles = (row_chunks + tile_chunks - 1) / tile_chunks;
    const int64_t grid = (int64_t)a * d * n_tiles;
    if (grid > 0x7fffffffLL) return KSMM_ERR_TOO_LARGE;
    int n_tiles_i = (int)n_tiles, tc = tile_chunks;
    void *args[] = {(void *)&x, (void *)&y, &rows, &d, (void *)&row_chunks, &tc, &n_tiles_i};
    return hipLaunchKernel((const void *)ks_tilecopy_probe_kernel, dim3((unsigned)grid), dim3(256), args, 0,
                           (hipStream_t)stream) == hipSuccess
               ? KSMM_OK
               : KSMM_ERR_LAUNCH;
}

}  // extern "C"
