// Generic KS factor kernel: any (a, b, c, d), any batch, both layouts, every supported
// dtype combination.  One thread per output element; weights are read through the cache.
// It is the family of last resort for shapes the MFMA families do not cover (b or c not a
// multiple of the MFMA tile, odd batch sizes) and the simplest statement of the product on
// the device.
//
// For batch-size-last there is also a vector form for blocks of a few elements (b * c below
// about 100, e.g. the (1,2,4,7168) ... (1,16,32,896) factors of the reference's pattern list,
// where an MFMA tile would be almost empty): a thread owns 16 bytes of consecutive batch
// columns and up to BT outputs of one (a_i, d_i) block; it streams the c input rows once with
// 16-byte loads, multiplies by weights that are uniform over the workgroup and writes BT
// 16-byte (fp8 input: 32-byte) row pieces.  Pure streaming: HBM sees whole 16-byte vectors.
//
// Indexing follows the reference kernels' block arithmetic
// (src/ksmm_py/layer/kronecker_sparse/template_kernels_float.cuh:118-137, 328-347):
//   input feature  (a_i*c + c_i)*d + d_i,  output feature (a_i*b + b_i)*d + d_i,
//   weight element ((a_i*d + d_i)*c + c_i)*b + b_i.
#include "ksmm_common.h"

namespace ksmm {

template <typename TX, typename TW, typename TY, bool BS_LAST>
__global__ __launch_bounds__(256) void ks_generic_kernel(const TX *__restrict__ x,
                                                         const TW *__restrict__ w,
                                                         TY *__restrict__ y, int64_t batch, int a,
                                                         int b, int c, int d, Epi ep)
{
    const int64_t in_size = (int64_t)a * c * d;
    const int64_t out_size = (int64_t)a * b * d;
    // 1-D grid: blockIdx.x = slow * fast_blocks + fast_block
    const int64_t fast_extent = BS_LAST ? batch : out_size;
    const int64_t fast_blocks = (fast_extent + blockDim.x - 1) / blockDim.x;
    const int64_t slow = blockIdx.x / fast_blocks;
    const int64_t fast = (blockIdx.x - slow * fast_blocks) * blockDim.x + threadIdx.x;
    if (fast >= fast_extent) return;
    // bs_last: consecutive threads -> consecutive batch columns of one output row;
    // bs_first: consecutive threads -> consecutive output features of one batch row
    const int64_t n = BS_LAST ? fast : slow;
    const int64_t j = BS_LAST ? slow : fast;
    const int a_i = (int)(j / ((int64_t)b * d));
    const int rem = (int)(j - (int64_t)a_i * b * d);
    const int b_i = rem / d;
    const int d_i = rem - b_i * d;
    const TW *wp = w + ((int64_t)(a_i * d + d_i) * c) * b + b_i;
    float acc = 0.f;
    if (BS_LAST) {
        const TX *xp = x + ((int64_t)a_i * c * d + d_i) * batch + n;
        const int64_t xs = (int64_t)d * batch;
        for (int k = 0; k < c; ++k) acc += elem<TW>::load(wp + (int64_t)k * b) * elem<TX>::load(xp + k * xs);
        elem<TY>::store(y + j * batch + n, epi_finish(ep, acc, epi_bias<TY>(ep, (size_t)j)));
    } else {
        const TX *xp = x + n * in_size + (int64_t)a_i * c * d + d_i;
        for (int k = 0; k < c; ++k) acc += elem<TW>::load(wp + (int64_t)k * b) * elem<TX>::load(xp + (int64_t)k * d);
        elem<TY>::store(y + n * out_size + j, epi_finish(ep, acc, epi_bias<TY>(ep, (size_t)j)));
    }
}

template <typename TX> struct vec16;  // 16 bytes of inputs -> floats
template <> struct vec16<float> {
    static constexpr int N = 4;
    __device__ static __forceinline__ void unpack(const uint4_t &v, float (&f)[4])
    {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const uint32_t u = v[i];  // (a bit_cast of the element expression itself reads element 0)
            f[i] = __builtin_bit_cast(float, u);
        }
    }
};
template <> struct vec16<half_t> {
    static constexpr int N = 8;
    __device__ static __forceinline__ void unpack(const uint4_t &v, float (&f)[8])
    {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const uint32_t u = v[i];
            const half2_t h = __builtin_bit_cast(half2_t, u);
            f[2 * i] = (float)h[0];
            f[2 * i + 1] = (float)h[1];
        }
    }
};
template <> struct vec16<fp8_t> {
    static constexpr int N = 16;
    __device__ static __forceinline__ void unpack(const uint4_t &v, float (&f)[16])
    {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const uint32_t u = v[i];
            const half2_t lo = fp8x2_to_half2(u), hi = fp8x2_hi_to_half2(u);
            f[4 * i] = (float)lo[0];
            f[4 * i + 1] = (float)lo[1];
            f[4 * i + 2] = (float)hi[0];
            f[4 * i + 3] = (float)hi[1];
        }
    }
};

// batch-size-last, batch a multiple of the vector; blockIdx = ((g * n_blocks + nb) * b_chunks + bc)
template <typename TX, typename TW, typename TY, int BT>
__global__ __launch_bounds__(256) void ks_small_bl_kernel(const TX *__restrict__ x, const TW *__restrict__ w,
                                                          TY *__restrict__ y, int64_t batch, int a, int b, int c,
                                                          int d, Epi ep, int n_blocks, int b_chunks)
{
    constexpr int V = vec16<TX>::N;
    const int bc = blockIdx.x % b_chunks;
    const int rest = blockIdx.x / b_chunks;
    const int nb = rest % n_blocks, g = rest / n_blocks;  // g = a_i * d + d_i
    const int a_i = g / d, d_i = g - a_i * d;
    const int64_t n0 = ((int64_t)nb * 256 + threadIdx.x) * V;
    if (n0 >= batch) return;
    const int b0 = bc * BT;
    float acc[BT][V];
#pragma unroll
    for (int j = 0; j < BT; ++j)
#pragma unroll
        for (int e = 0; e < V; ++e) acc[j][e] = 0.f;
    const TX *xp = x + ((int64_t)a_i * c * d + d_i) * batch + n0;
    const int64_t xs = (int64_t)d * batch;
    const TW *wp = w + (int64_t)g * c * b + b0;  // uniform over the workgroup
#pragma unroll 4
    for (int k = 0; k < c; ++k) {
        float xf[V];
        vec16<TX>::unpack(*(const uint4_t *)(xp + k * xs), xf);
#pragma unroll
        for (int j = 0; j < BT; ++j) {
            const float wv = b0 + j < b ? elem<TW>::load(wp + (int64_t)k * b + j) : 0.f;
#pragma unroll
            for (int e = 0; e < V; ++e) acc[j][e] += wv * xf[e];
        }
    }
#pragma unroll
    for (int j = 0; j < BT; ++j) {
        if (b0 + j >= b) break;
        const int64_t feature = (int64_t)(a_i * b + b0 + j) * d + d_i;
        TY *yp = y + feature * batch + n0;
        const float bv = epi_bias<TY>(ep, (size_t)feature);
        if constexpr (sizeof(TY) == 4) {
            *(float4_t *)yp = float4_t{epi_finish(ep, acc[j][0], bv), epi_finish(ep, acc[j][1], bv),
                                       epi_finish(ep, acc[j][2], bv), epi_finish(ep, acc[j][3], bv)};
        } else {
#pragma unroll
            for (int h = 0; h < V / 8; ++h) {
                half8_t o;
#pragma unroll
                for (int e = 0; e < 8; ++e) o[e] = (half_t)epi_finish(ep, acc[j][8 * h + e], bv);
                *(half8_t *)(yp + 8 * h) = o;
            }
        }
    }
}

template <typename TX, typename TW, typename TY>
static void launch_small(const Problem &p, int64_t grid, int n_blocks, int b_chunks)
{
    hipLaunchKernelGGL((ks_small_bl_kernel<TX, TW, TY, 8>), dim3((unsigned)grid), dim3(256), 0, p.stream,
                       (const TX *)p.x, (const TW *)p.w, (TY *)p.y, p.batch, p.a, p.b, p.c, p.d, epi_of(p), n_blocks,
                       b_chunks);
}

template <typename TX, typename TW, typename TY>
static void launch_generic(const Problem &p, dim3 grid, dim3 block)
{
    if (p.bs_last)
        hipLaunchKernelGGL((ks_generic_kernel<TX, TW, TY, true>), grid, block, 0, p.stream,
                           (const TX *)p.x, (const TW *)p.w, (TY *)p.y, p.batch, p.a, p.b, p.c, p.d,
                           epi_of(p));
    else
        hipLaunchKernelGGL((ks_generic_kernel<TX, TW, TY, false>), grid, block, 0, p.stream,
                           (const TX *)p.x, (const TW *)p.w, (TY *)p.y, p.batch, p.a, p.b, p.c, p.d,
                           epi_of(p));
}

// variant 0: one thread per output; 1: the vector form (batch-size-last, batch a multiple of the
// 16-byte vector); -1: the vector form where it applies and the block is small
int generic_run(const Problem &p, int variant, bool launch, ksmm_tile *tile)
{
    if (variant > 1) return KSMM_ERR_BAD_ALGO;
    const int combo = combo_of(p.x_dtype, p.w_dtype, p.y_dtype);
    const int vec = 16 / (int)dtype_size(p.x_dtype);
    const bool vec_ok = p.bs_last && combo >= 0 && combo <= 2 && p.batch % vec == 0 &&
                        (((uintptr_t)p.x | (uintptr_t)p.y) & 15) == 0;
    if (variant == 1 && !vec_ok) return KSMM_ERR_BAD_ALGO;
    if (variant == 1 || (variant < 0 && vec_ok && (int64_t)p.b * p.c <= 1024)) {
        const int bt = 8;
        const int64_t n_blocks = (p.batch / vec + 255) / 256, b_chunks = (p.b + bt - 1) / bt;
        const int64_t grid = (int64_t)p.a * p.d * n_blocks * b_chunks;
        if (grid > 0x7fffffffLL) return KSMM_ERR_TOO_LARGE;
        if (tile) {
            tile->algo = KSMM_ALGO_GENERIC;
            tile->variant = 1;
            tile->tile_m = bt;
            tile->tile_n = 256 * vec;
            tile->tile_k = p.c;
            tile->tile_d = 1;
            tile->threads = 256;
            tile->lds_bytes = 0;
            tile->grid = grid;
        }
        if (!launch) return KSMM_OK;
        switch (combo) {
        case 0: launch_small<float, float, float>(p, grid, (int)n_blocks, (int)b_chunks); break;
        case 1: launch_small<half_t, half_t, half_t>(p, grid, (int)n_blocks, (int)b_chunks); break;
        default: launch_small<fp8_t, fp8_t, half_t>(p, grid, (int)n_blocks, (int)b_chunks); break;
        }
        return hipGetLastError() == hipSuccess ? KSMM_OK : KSMM_ERR_LAUNCH;
    }
    const int64_t out_size = (int64_t)p.a * p.b * p.d;
    const int threads = 256;
    dim3 block(threads, 1, 1);
    const int64_t fast = p.bs_last ? p.batch : out_size;
    const int64_t slow = p.bs_last ? out_size : p.batch;
    const int64_t nblocks = ((fast + threads - 1) / threads) * slow;
    if (nblocks > 0x7fffffffLL) return KSMM_ERR_TOO_LARGE;
    dim3 grid((unsigned)nblocks, 1, 1);
    if (tile) {
        tile->algo = KSMM_ALGO_GENERIC;
        tile->variant = 0;
        tile->tile_m = 1;
        tile->tile_n = p.bs_last ? threads : 1;
        tile->tile_k = p.c;
        tile->tile_d = 1;
        tile->threads = threads;
        tile->lds_bytes = 0;
        tile->grid = nblocks;
    }
    if (!launch) return KSMM_OK;
    switch (combo_of(p.x_dtype, p.w_dtype, p.y_dtype)) {
    case 0: launch_generic<float, float, float>(p, grid, block); break;
    case 1: launch_generic<half_t, half_t, half_t>(p, grid, block); break;
    case 2: launch_generic<fp8_t, fp8_t, half_t>(p, grid, block); break;
    case 3: launch_generic<half_t, fp8_t, half_t>(p, grid, block); break;
    default: return KSMM_ERR_BAD_DTYPE;
    }
    return hipGetLastError() == hipSuccess ? KSMM_OK : KSMM_ERR_LAUNCH;
}

}  // namespace ksmm
