// Generic KS factor kernel: any (a, b, c, d), any batch, both layouts, every supported
// dtype combination.  One thread per output element; weights are read through the cache.
// It is the family of last resort for shapes the MFMA families do not cover (b or c not a
// multiple of the MFMA tile, odd batch sizes) and the simplest statement of the product on
// the device.
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
                                                         int b, int c, int d, float scale)
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
        elem<TY>::store(y + j * batch + n, acc * scale);
    } else {
        const TX *xp = x + n * in_size + (int64_t)a_i * c * d + d_i;
        for (int k = 0; k < c; ++k) acc += elem<TW>::load(wp + (int64_t)k * b) * elem<TX>::load(xp + (int64_t)k * d);
        elem<TY>::store(y + n * out_size + j, acc * scale);
    }
}

template <typename TX, typename TW, typename TY>
static void launch_generic(const Problem &p, dim3 grid, dim3 block)
{
    if (p.bs_last)
        hipLaunchKernelGGL((ks_generic_kernel<TX, TW, TY, true>), grid, block, 0, p.stream,
                           (const TX *)p.x, (const TW *)p.w, (TY *)p.y, p.batch, p.a, p.b, p.c, p.d,
                           p.scale);
    else
        hipLaunchKernelGGL((ks_generic_kernel<TX, TW, TY, false>), grid, block, 0, p.stream,
                           (const TX *)p.x, (const TW *)p.w, (TY *)p.y, p.batch, p.a, p.b, p.c, p.d,
                           p.scale);
}

int generic_run(const Problem &p, int variant, bool launch, ksmm_tile *tile)
{
    if (variant > 0) return KSMM_ERR_BAD_ALGO;
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
