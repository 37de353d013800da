// Backward pass of one Kronecker-sparse factor y = K x (forward: ksmm_factor_forward).
//
//   dX = K^T dY   is itself a KS factor: pattern (a, c, b, d) with every b x c block transposed,
//                 so it runs on the forward kernels once the blocks are transposed (ks_block_transpose_kernel)
//   dW[a_i, b_i, c_i, d_i] = sum_n dY[a_i, b_i, d_i, n] * X[a_i, c_i, d_i, n]
//                 one (b x B) @ (B x c) product per (a_i, d_i) block, reduced over the batch:
//                 MFMA kernel for batch-size-last (operand rows are batch-contiguous, so both
//                 operands come straight from global memory in MFMA layout, no LDS), an
//                 LDS-tiled FMA kernel for everything else; every batch split writes its partial
//                 sums to a slice of its own in the workspace, and a finish kernel adds the slices
//                 in a fixed order, scales, converts and writes kernel format (a*d*c, b): the
//                 result is the same bit for bit from run to run (no atomics).
//
// The reference has no backward pass (src/ksmm_py/layer/kronecker_sparse/kernel.py:319-329 refers
// to an undefined symbol; forward_bmm.py:12-15 is `pass`); the definition above is the adjoint of
// its forward product (interface.py:108-113).
#include "ksmm_common.h"

namespace ksmm {

namespace {

// out block g (b x c, c contiguous)  <-  in block g (c x b, b contiguous); both in "kernel format"
// of their own pattern: in = (a*d*c, b) of (a,b,c,d), out = (a*d*b, c) of (a,c,b,d)
template <typename T>
__global__ __launch_bounds__(256) void ks_block_transpose_kernel(const T *__restrict__ in, T *__restrict__ out,
                                                                 int64_t total, int b, int c)
{
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;  // index into out
    if (i >= total) return;
    const int64_t g = i / ((int64_t)b * c);
    const int rem = (int)(i - g * b * c);
    const int bi = rem / c, ci = rem - bi * c;
    out[i] = in[(g * c + ci) * b + bi];
}

// dw[i] = scale * (sum of the slices); slices are n floats apart.  A workgroup takes 64 outputs;
// its four 64-thread groups add a quarter of the slices each, in slice order (eight loads in
// flight per thread), and the four partial sums are added in group order: the association is
// fixed by (splits) alone, so the result has the same bits on every run.
template <typename T>
__global__ __launch_bounds__(256) void ks_wgrad_finish_kernel(const float *__restrict__ acc, T *__restrict__ dw,
                                                              int64_t n, int splits, float scale)
{
    __shared__ float part[4][64];
    const int g = threadIdx.x >> 6, l = threadIdx.x & 63;
    const int64_t i = (int64_t)blockIdx.x * 64 + l;
    const int per = (splits + 3) / 4, k0 = g * per, k1 = min(k0 + per, splits);
    float s = 0.f;
    if (i < n) {
        int k = k0;
        for (; k + 8 <= k1; k += 8) {
            float v[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) v[j] = acc[(int64_t)(k + j) * n + i];
#pragma unroll
            for (int j = 0; j < 8; ++j) s += v[j];
        }
        for (; k < k1; ++k) s += acc[(int64_t)k * n + i];
    }
    part[g][l] = s;
    __syncthreads();
    if (g == 0 && i < n) dw[i] = (T)((((part[0][l] + part[1][l]) + part[2][l]) + part[3][l]) * scale);
}

template <typename T> struct wg_vec;
template <> struct wg_vec<float> {
    static constexpr int N = 4, MFMAS = 4;  // elements per 16-byte load; MFMAs fed by one load pair
    typedef float4_t type;
    __device__ static __forceinline__ float4_t mfma(int e, float4_t a, float4_t b, float4_t c)
    {
        return __builtin_amdgcn_mfma_f32_16x16x4f32(a[e], b[e], c, 0, 0, 0);
    }
};
template <> struct wg_vec<half_t> {
    static constexpr int N = 8, MFMAS = 2;
    typedef half8_t type;
    __device__ static __forceinline__ float4_t mfma(int e, half8_t a, half8_t b, float4_t c)
    {
        const half4_t ah = {a[4 * e], a[4 * e + 1], a[4 * e + 2], a[4 * e + 3]};
        const half4_t bh = {b[4 * e], b[4 * e + 1], b[4 * e + 2], b[4 * e + 3]};
        return __builtin_amdgcn_mfma_f32_16x16x16f16(ah, bh, c, 0, 0, 0);
    }
};

// Batch-size-last, batch a multiple of the 16-byte vector.  One wavefront owns a (16*MT) x (16*NT)
// tile of one block's b x c gradient and a range of batch columns.  Lane (r = lane % 16,
// q = lane / 16) loads N consecutive batch elements of operand row r at column n + N*q; MFMA e
// multiplies element group e of every lane, i.e. its k-set is {n + N*q + e ...}: the same set for
// both operands, and the order of a sum's terms is free.
// NTL: non-temporal loads, for blocks of a single tile (every operand row is read by one wave only;
// with several tiles per block the rows are shared through the caches)
template <typename T, int MT, int NT, bool NTL>
__global__ __launch_bounds__(256) void ks_wgrad_bl_kernel(const T *__restrict__ dy, const T *__restrict__ x,
                                                          float *__restrict__ acc_out, int batch, int a, int b,
                                                          int c, int d, int m_tiles, int n_tiles, int splits,
                                                          int cols_per_split, int64_t slice)
{
    typedef wg_vec<T> V;
    constexpr int STEP = 4 * V::N;  // batch columns per step (4 lane groups)
    const int lane = threadIdx.x & 63, r = lane & 15, q = lane >> 4;
    int64_t wave = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    const int split = (int)(wave % splits);
    wave /= splits;
    const int nt = (int)(wave % n_tiles);
    wave /= n_tiles;
    const int mt = (int)(wave % m_tiles);
    const int64_t g = wave / m_tiles;
    if (g >= (int64_t)a * d) return;
    const int a_i = (int)(g / d), d_i = (int)(g - (int64_t)a_i * d);
    const int m0 = mt * 16 * MT, c0 = nt * 16 * NT;
    const int n_begin = split * cols_per_split, n_end = min(batch, n_begin + cols_per_split);
    if (n_begin >= n_end) return;
    const size_t row_stride = (size_t)d * batch;
    // rows behind b (or c) are clamped to the last valid one and dropped at the end
    const T *ap[MT], *bp[NT];
#pragma unroll
    for (int i = 0; i < MT; ++i)
        ap[i] = dy + ((size_t)a_i * b * d + d_i) * batch + (size_t)min(m0 + 16 * i + r, b - 1) * row_stride;
#pragma unroll
    for (int j = 0; j < NT; ++j)
        bp[j] = x + ((size_t)a_i * c * d + d_i) * batch + (size_t)min(c0 + 16 * j + r, c - 1) * row_stride;
    float4_t acc[MT][NT];
#pragma unroll
    for (int i = 0; i < MT; ++i)
#pragma unroll
        for (int j = 0; j < NT; ++j) acc[i][j] = float4_t{0.f, 0.f, 0.f, 0.f};
    typedef typename V::type vec_t;
    // U sub-steps per iteration, all their loads issued before the first MFMA: a row is then read
    // in runs of U * 64 bytes, and the loads of the whole iteration are in flight together
    constexpr int U = (MT + NT) * 4 <= 24 ? 4 : 2;
    for (int n = n_begin; n < n_end; n += U * STEP) {
        vec_t av[U][MT], bv[U][NT];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int col = n + u * STEP + V::N * q;
            const bool live = col < n_end;          // whole vectors: batch and the split are multiples of N
            const int lcol = live ? col : n_begin;  // (a valid address; the value is zeroed)
#pragma unroll
            for (int i = 0; i < MT; ++i)
                av[u][i] = NTL ? __builtin_nontemporal_load((const vec_t *)(ap[i] + lcol)) : *(const vec_t *)(ap[i] + lcol);
#pragma unroll
            for (int j = 0; j < NT; ++j)
                bv[u][j] = NTL ? __builtin_nontemporal_load((const vec_t *)(bp[j] + lcol)) : *(const vec_t *)(bp[j] + lcol);
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            if (n + u * STEP + V::N * q >= n_end) {
#pragma unroll
                for (int i = 0; i < MT; ++i)
#pragma unroll
                    for (int e = 0; e < V::N; ++e) av[u][i][e] = 0;
#pragma unroll
                for (int j = 0; j < NT; ++j)
#pragma unroll
                    for (int e = 0; e < V::N; ++e) bv[u][j][e] = 0;
            }
#pragma unroll
            for (int e = 0; e < V::MFMAS; ++e)
#pragma unroll
                for (int i = 0; i < MT; ++i)
#pragma unroll
                    for (int j = 0; j < NT; ++j) acc[i][j] = V::mfma(e, av[u][i], bv[u][j], acc[i][j]);
        }
    }
    // D: lane holds column (c index) r and rows (b index) 4*q .. 4*q + 3 of each 16 x 16 tile
#pragma unroll
    for (int i = 0; i < MT; ++i)
#pragma unroll
        for (int j = 0; j < NT; ++j) {
            const int cc = c0 + 16 * j + r;
            if (cc >= c) continue;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int m = m0 + 16 * i + 4 * q + e;
                if (m < b) acc_out[(size_t)split * slice + ((size_t)g * c + cc) * b + m] = acc[i][j][e];
            }
        }
}

// Any layout, any batch: 16 x 16 threads compute a 16 x 16 tile of one block's gradient over a
// batch range, staging 16 x 16 element tiles of both operands in LDS (fp32 FMAs).
template <typename T, bool BS_LAST>
__global__ __launch_bounds__(256) void ks_wgrad_tiled_kernel(const T *__restrict__ dy, const T *__restrict__ x,
                                                             float *__restrict__ acc_out, int64_t batch, int a,
                                                             int b, int c, int d, int m_tiles, int n_tiles,
                                                             int splits, int64_t cols_per_split, int64_t slice)
{
    __shared__ float sa[16][17], sb[16][17];
    int64_t t = blockIdx.x;
    const int split = (int)(t % splits);
    t /= splits;
    const int nt = (int)(t % n_tiles);
    t /= n_tiles;
    const int mt = (int)(t % m_tiles);
    const int64_t g = t / m_tiles;
    const int a_i = (int)(g / d), d_i = (int)(g - (int64_t)a_i * d);
    const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;
    const int64_t in_size = (int64_t)a * c * d, out_size = (int64_t)a * b * d;
    const int64_t n_begin = split * cols_per_split, n_end = min(batch, n_begin + cols_per_split);
    // staging: thread (ty, tx) loads operand row ty, batch element n + tx (batch-size-last: tx runs
    // along the contiguous axis) or row tx, batch element n + ty (batch-size-first: features contiguous)
    const int lrow = BS_LAST ? ty : tx, lcol = BS_LAST ? tx : ty;
    const int m_ld = mt * 16 + lrow, c_ld = nt * 16 + lrow;
    const int64_t fa = ((int64_t)a_i * b + min(m_ld, b - 1)) * d + d_i;  // feature of dY
    const int64_t fb = ((int64_t)a_i * c + min(c_ld, c - 1)) * d + d_i;  // feature of X
    float acc = 0.f;
    for (int64_t n = n_begin; n < n_end; n += 16) {
        const int64_t nn = n + lcol;
        float va = 0.f, vb = 0.f;
        if (nn < n_end) {
            va = elem<T>::load(BS_LAST ? dy + fa * batch + nn : dy + nn * out_size + fa);
            vb = elem<T>::load(BS_LAST ? x + fb * batch + nn : x + nn * in_size + fb);
        }
        sa[lrow][lcol] = va;
        sb[lrow][lcol] = vb;
        __syncthreads();
#pragma unroll
        for (int k = 0; k < 16; ++k) acc += sa[tx][k] * sb[ty][k];
        __syncthreads();
    }
    const int m = mt * 16 + tx, cc = nt * 16 + ty;  // consecutive threads: consecutive b_i (contiguous in dW)
    if (m < b && cc < c) acc_out[(size_t)split * slice + ((size_t)g * c + cc) * b + m] = acc;
}

template <typename T> int launch_block_transpose(const void *w, void *wt, int64_t total, int b, int c, hipStream_t s)
{
    const int64_t blocks = (total + 255) / 256;
    if (blocks > 0x7fffffffLL) return KSMM_ERR_TOO_LARGE;
    hipLaunchKernelGGL((ks_block_transpose_kernel<T>), dim3((unsigned)blocks), dim3(256), 0, s, (const T *)w, (T *)wt,
                       total, b, c);
    return hipGetLastError() == hipSuccess ? KSMM_OK : KSMM_ERR_LAUNCH;
}

// Batch splits of the two weight-gradient kernels (every split is non-empty and writes a slice of
// a*b*c*d partial sums of its own): columns per split and their number.
// Weight gradient of large fp16 blocks (b and c multiples of 128), batch-size-last operands: a
// 128 x 128 tile of one block's gradient and a range of batch columns per workgroup (4 waves, 2 x 2,
// 64 x 64 each on v_mfma_f32_32x32x16_f16).  Both operands have the batch axis contiguous, so a slab
// of 64 columns is 128 rows x 128 bytes per operand: it goes through registers into LDS (16-byte
// chunks, the chunk index XORed with row / 2 so that the operand reads of 16 consecutive rows hit
// different banks), double-buffered, one barrier per slab.  Against the wave-per-tile kernel above,
// which re-reads every operand row once per 64 x 64 tile through L2 (1.85 GB for (1,1536,384,2) at
// batch 25088), the traffic drops to a quarter.  D = X-rows x dY-rows^T, so a lane holds one output
// feature m (contiguous in kernel format) and 16 inputs k.
constexpr int WG_TM = 128, WG_TN = 128, WG_TK = 64;
__global__ __launch_bounds__(256, 2) void ks_wgrad_gemm_h_kernel(const half_t *__restrict__ dy,
                                                                 const half_t *__restrict__ x,
                                                                 float *__restrict__ acc_out, int batch, int a, int b,
                                                                 int c, int d, int m_tiles, int n_tiles, int splits,
                                                                 int cols, int64_t slice)
{
    __shared__ __attribute__((aligned(16))) half_t sa[2][WG_TM * WG_TK], sb[2][WG_TN * WG_TK];
    int id = blockIdx.x;
    const int split = id % splits;
    id /= splits;
    const int mt = id % m_tiles;
    id /= m_tiles;
    const int nt = id % n_tiles, g = id / n_tiles;
    const int a_i = g / d, d_i = g - a_i * d;
    const int m0 = mt * WG_TM, n0 = nt * WG_TN;
    const int k_begin = split * cols, k_end = min(k_begin + cols, batch);
    const int tid = threadIdx.x, lane = tid & 63, l32 = lane & 31, lq = lane >> 5;
    const int wave = tid >> 6, wm = wave >> 1, wn = wave & 1;
    // staging: 4 vectors per operand and thread; vector v = tid + 256 * i is row v / 8, physical
    // chunk v % 8, which holds the logical chunk (v % 8) ^ ((row / 2) % 8)
    const half_t *ga[4], *gb[4];
    int lcol[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int v = tid + 256 * i, row = v >> 3, lc = (v & 7) ^ ((row >> 1) & 7);
        lcol[i] = lc * 8;
        ga[i] = dy + ((size_t)(a_i * b + m0 + row) * d + d_i) * batch + lc * 8;
        gb[i] = x + ((size_t)(a_i * c + n0 + row) * d + d_i) * batch + lc * 8;
    }
    uint4_t ra[4], rb[4];
    auto gload = [&](int k) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const bool in = k + lcol[i] < k_end;  // (k_end is a multiple of 8)
            ra[i] = in ? *(const uint4_t *)(ga[i] + k) : uint4_t{0u, 0u, 0u, 0u};
            rb[i] = in ? *(const uint4_t *)(gb[i] + k) : uint4_t{0u, 0u, 0u, 0u};
        }
    };
    auto lstore = [&](int buf) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            *(uint4_t *)(sa[buf] + (tid + 256 * i) * 8) = ra[i];
            *(uint4_t *)(sb[buf] + (tid + 256 * i) * 8) = rb[i];
        }
    };
    float16_t acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;
    if (k_begin < k_end) {
        gload(k_begin);
        lstore(0);
    }
    __syncthreads();
    int buf = 0;
    for (int k = k_begin; k < k_end; k += WG_TK) {
        const bool more = k + WG_TK < k_end;
        if (more) gload(k + WG_TK);
#pragma unroll
        for (int ks = 0; ks < WG_TK / 16; ++ks) {
            half8_t fx[2], fy[2];
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                const int rx = wn * 64 + i * 32 + l32, ry = wm * 64 + i * 32 + l32;
                fx[i] = *(const half8_t *)(sb[buf] + (rx * 8 + ((2 * ks + lq) ^ ((rx >> 1) & 7))) * 8);
                fy[i] = *(const half8_t *)(sa[buf] + (ry * 8 + ((2 * ks + lq) ^ ((ry >> 1) & 7))) * 8);
            }
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fx[i], fy[j], acc[i][j], 0, 0, 0);
        }
        if (more) lstore(buf ^ 1);
        __syncthreads();
        buf ^= 1;
    }
    // D[k'][m]: lane l32 = output feature m, rows k' = 8 * (e / 4) + 4 * lq + e % 4
    float *out = acc_out + (size_t)split * slice + (size_t)g * c * b;
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const int kk = n0 + wn * 64 + i * 32 + 8 * (e >> 2) + 4 * lq + (e & 3);
                const int m = m0 + wm * 64 + j * 32 + l32;
                out[(size_t)kk * b + m] = acc[i][j][e];
            }
}

bool wgrad_gemm_ok(int b, int c, int dtype) { return dtype == KSMM_F16 && b % WG_TM == 0 && c % WG_TN == 0; }

// batch ranges of the tiled kernel: two workgroups per CU, at least 8 slabs each
void wgrad_gemm_splits(int64_t batch, int64_t tiles, int64_t *splits_out, int64_t *cols_out)
{
    int64_t splits = (512 + tiles - 1) / tiles;
    const int64_t max_splits = (batch + 8 * WG_TK - 1) / (8 * WG_TK);
    if (splits > max_splits) splits = max_splits;
    if (splits < 1) splits = 1;
    int64_t cols = (batch + splits - 1) / splits;
    cols = (cols + WG_TK - 1) / WG_TK * WG_TK;
    *splits_out = (batch + cols - 1) / cols;
    *cols_out = cols;
}

void wgrad_bl_splits(int64_t batch, int64_t tiles, int step, int64_t *splits_out, int64_t *cols_out)
{
    // about 16 waves per CU; at least 4 loop iterations per wave
    int64_t splits = (4096 + tiles - 1) / tiles;
    const int64_t max_splits = (batch + 4 * step - 1) / (4 * step);
    if (splits > max_splits) splits = max_splits;
    if (splits < 1) splits = 1;
    int64_t cols = (batch + splits - 1) / splits;
    cols = (cols + step - 1) / step * step;
    *splits_out = (batch + cols - 1) / cols;
    *cols_out = cols;
}

void wgrad_tiled_splits(int64_t batch, int64_t tiles, int64_t *splits_out, int64_t *cols_out)
{
    int64_t splits = (2048 + tiles - 1) / tiles;
    const int64_t max_splits = (batch + 255) / 256;
    if (splits > max_splits) splits = max_splits;
    if (splits < 1) splits = 1;
    int64_t cols = (batch + splits - 1) / splits;
    cols = (cols + 15) / 16 * 16;
    *splits_out = (batch + cols - 1) / cols;
    *cols_out = cols;
}

// tile of the MFMA kernel for a block shape: 16 * t rows and columns
int wgrad_bl_tile(int b, int c)
{
    return (b <= 16 && c <= 16) ? 1 : (b <= 32 && c <= 32) ? 2 : (b % 64 && c % 64 && b % 48 == 0 && c % 48 == 0) ? 3 : 4;
}

bool wgrad_mfma_ok(const void *dy, const void *x, int64_t batch, int b, int c, int d, int dtype, int bs_last)
{
    const int vec = 16 / (int)dtype_size(dtype);
    return bs_last && batch % vec == 0 && ((((uintptr_t)dy | (uintptr_t)x) & 15) == 0) &&
           (int64_t)(b > c ? b : c) * d * batch < 0x7fffffffLL;
}

template <typename T, int MT, int NT>
int launch_wgrad_bl(const void *dy, const void *x, float *acc, int64_t batch, int a, int b, int c, int d,
                    hipStream_t s, int *splits_used)
{
    const int m_tiles = (b + 16 * MT - 1) / (16 * MT), n_tiles = (c + 16 * NT - 1) / (16 * NT);
    const int64_t tiles = (int64_t)a * d * m_tiles * n_tiles;
    constexpr int STEP = 16 * wg_vec<T>::N;  // columns per loop iteration of the kernel (four sub-steps)
    int64_t splits, cols;
    wgrad_bl_splits(batch, tiles, STEP, &splits, &cols);
    const int64_t waves = tiles * splits, blocks = (waves + 3) / 4;
    if (blocks > 0x7fffffffLL) return KSMM_ERR_TOO_LARGE;
    *splits_used = (int)splits;
    if (m_tiles == 1 && n_tiles == 1)
        hipLaunchKernelGGL((ks_wgrad_bl_kernel<T, MT, NT, true>), dim3((unsigned)blocks), dim3(256), 0, s, (const T *)dy,
                           (const T *)x, acc, (int)batch, a, b, c, d, m_tiles, n_tiles, (int)splits, (int)cols,
                           (int64_t)a * b * c * d);
    else
        hipLaunchKernelGGL((ks_wgrad_bl_kernel<T, MT, NT, false>), dim3((unsigned)blocks), dim3(256), 0, s, (const T *)dy,
                           (const T *)x, acc, (int)batch, a, b, c, d, m_tiles, n_tiles, (int)splits, (int)cols,
                           (int64_t)a * b * c * d);
    return hipGetLastError() == hipSuccess ? KSMM_OK : KSMM_ERR_LAUNCH;
}

template <typename T>
int launch_wgrad_tiled(const void *dy, const void *x, float *acc, int64_t batch, int a, int b, int c, int d,
                       int bs_last, hipStream_t s, int *splits_used)
{
    const int m_tiles = (b + 15) / 16, n_tiles = (c + 15) / 16;
    const int64_t tiles = (int64_t)a * d * m_tiles * n_tiles;
    int64_t splits, cols;
    wgrad_tiled_splits(batch, tiles, &splits, &cols);
    const int64_t blocks = tiles * splits;
    if (blocks > 0x7fffffffLL) return KSMM_ERR_TOO_LARGE;
    *splits_used = (int)splits;
    const int64_t slice = (int64_t)a * b * c * d;
    if (bs_last)
        hipLaunchKernelGGL((ks_wgrad_tiled_kernel<T, true>), dim3((unsigned)blocks), dim3(256), 0, s, (const T *)dy,
                           (const T *)x, acc, batch, a, b, c, d, m_tiles, n_tiles, (int)splits, cols, slice);
    else
        hipLaunchKernelGGL((ks_wgrad_tiled_kernel<T, false>), dim3((unsigned)blocks), dim3(256), 0, s, (const T *)dy,
                           (const T *)x, acc, batch, a, b, c, d, m_tiles, n_tiles, (int)splits, cols, slice);
    return hipGetLastError() == hipSuccess ? KSMM_OK : KSMM_ERR_LAUNCH;
}

int launch_wgrad_gemm(const void *dy, const void *x, float *acc, int64_t batch, int a, int b, int c, int d,
                      hipStream_t s, int *splits_used)
{
    const int m_tiles = b / WG_TM, n_tiles = c / WG_TN;
    const int64_t tiles = (int64_t)a * d * m_tiles * n_tiles;
    int64_t splits, cols;
    wgrad_gemm_splits(batch, tiles, &splits, &cols);
    const int64_t blocks = tiles * splits;
    if (blocks > 0x7fffffffLL) return KSMM_ERR_TOO_LARGE;
    *splits_used = (int)splits;
    hipLaunchKernelGGL(ks_wgrad_gemm_h_kernel, dim3((unsigned)blocks), dim3(256), 0, s, (const half_t *)dy,
                       (const half_t *)x, acc, (int)batch, a, b, c, d, m_tiles, n_tiles, (int)splits, (int)cols,
                       (int64_t)a * b * c * d);
    return hipGetLastError() == hipSuccess ? KSMM_OK : KSMM_ERR_LAUNCH;
}

}  // namespace

// wt <- the b x c blocks of w transposed: kernel format (a*d*b, c) of pattern (a, c, b, d)
int block_transpose_run(const void *w, void *wt, int a, int b, int c, int d, int dtype, hipStream_t stream)
{
    const int64_t total = (int64_t)a * b * c * d;
    switch (dtype) {
    case KSMM_F32: return launch_block_transpose<float>(w, wt, total, b, c, stream);
    case KSMM_F16: return launch_block_transpose<half_t>(w, wt, total, b, c, stream);
    case KSMM_FP8_E4M3: return launch_block_transpose<uint8_t>(w, wt, total, b, c, stream);
    default: return KSMM_ERR_BAD_DTYPE;
    }
}

// Floats of partial sums the weight gradient of this problem writes (slices of a*b*c*d, one per
// batch split), whichever kernel takes it: the larger of the two kernels' needs, so that the
// answer does not depend on pointer alignment.
int64_t wgrad_partial_floats(int64_t batch, int a, int b, int c, int d, int dtype)
{
    const int64_t n = (int64_t)a * b * c * d;
    int64_t splits, cols, most = 1;
    const int t = wgrad_bl_tile(b, c);
    const int64_t tiles_bl = (int64_t)a * d * ((b + 16 * t - 1) / (16 * t)) * ((c + 16 * t - 1) / (16 * t));
    wgrad_bl_splits(batch, tiles_bl, 16 * (16 / (int)dtype_size(dtype)), &splits, &cols);
    if (splits > most) most = splits;
    wgrad_tiled_splits(batch, (int64_t)a * d * ((b + 15) / 16) * ((c + 15) / 16), &splits, &cols);
    if (splits > most) most = splits;
    if (wgrad_gemm_ok(b, c, dtype)) {
        wgrad_gemm_splits(batch, (int64_t)a * d * (b / WG_TM) * (c / WG_TN), &splits, &cols);
        if (splits > most) most = splits;
    }
    return most * n;
}

// dw (kernel format, type `dtype`) <- scale * sum over the batch of dY x X^T per block; acc is an
// fp32 buffer of wgrad_partial_floats() elements.  kernel_used: 1 = MFMA kernel, 0 = tiled kernel.
int wgrad_run(const void *dy, const void *x, void *dw, float *acc, int64_t batch, int a, int b, int c, int d,
              int dtype, int bs_last, float scale, hipStream_t stream, int *kernel_used)
{
    const int64_t n = (int64_t)a * b * c * d;
    const int64_t fin_blocks = (n + 63) / 64;
    if (fin_blocks > 0x7fffffffLL) return KSMM_ERR_TOO_LARGE;
    const bool mfma_ok = wgrad_mfma_ok(dy, x, batch, b, c, d, dtype, bs_last);
    if (kernel_used) *kernel_used = mfma_ok ? 1 : 0;
    const int t = wgrad_bl_tile(b, c);
    int rc, splits = 1;
    if (dtype == KSMM_F32) {
        if (mfma_ok)
            rc = t == 1   ? launch_wgrad_bl<float, 1, 1>(dy, x, acc, batch, a, b, c, d, stream, &splits)
                 : t == 2 ? launch_wgrad_bl<float, 2, 2>(dy, x, acc, batch, a, b, c, d, stream, &splits)
                 : t == 3 ? launch_wgrad_bl<float, 3, 3>(dy, x, acc, batch, a, b, c, d, stream, &splits)
                          : launch_wgrad_bl<float, 4, 4>(dy, x, acc, batch, a, b, c, d, stream, &splits);
        else
            rc = launch_wgrad_tiled<float>(dy, x, acc, batch, a, b, c, d, bs_last, stream, &splits);
    } else if (dtype == KSMM_F16) {
        if (mfma_ok && wgrad_gemm_ok(b, c, dtype))
            rc = launch_wgrad_gemm(dy, x, acc, batch, a, b, c, d, stream, &splits);
        else if (mfma_ok)
            rc = t == 1   ? launch_wgrad_bl<half_t, 1, 1>(dy, x, acc, batch, a, b, c, d, stream, &splits)
                 : t == 2 ? launch_wgrad_bl<half_t, 2, 2>(dy, x, acc, batch, a, b, c, d, stream, &splits)
                 : t == 3 ? launch_wgrad_bl<half_t, 3, 3>(dy, x, acc, batch, a, b, c, d, stream, &splits)
                          : launch_wgrad_bl<half_t, 4, 4>(dy, x, acc, batch, a, b, c, d, stream, &splits);
        else
            rc = launch_wgrad_tiled<half_t>(dy, x, acc, batch, a, b, c, d, bs_last, stream, &splits);
    } else {
        return KSMM_ERR_BAD_DTYPE;
    }
    if (rc != KSMM_OK) return rc;
    if (dtype == KSMM_F32)
        hipLaunchKernelGGL((ks_wgrad_finish_kernel<float>), dim3((unsigned)fin_blocks), dim3(256), 0, stream, acc,
                           (float *)dw, n, splits, scale);
    else
        hipLaunchKernelGGL((ks_wgrad_finish_kernel<half_t>), dim3((unsigned)fin_blocks), dim3(256), 0, stream, acc,
                           (half_t *)dw, n, splits, scale);
    return hipGetLastError() == hipSuccess ? KSMM_OK : KSMM_ERR_LAUNCH;
}

}  // namespace ksmm
