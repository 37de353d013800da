// "Wave" family: bandwidth-bound path for small b x c blocks, batch-size-last layout.
//
// One wavefront owns one (a_i, d_i) block and a slab of batch columns.  The whole b x c weight
// block lives in registers as MFMA A-operands for the lifetime of the wave; the c input rows
// of the block are streamed straight from HBM with 8/16-byte loads along the batch axis (the
// contiguous axis in this layout), multiplied on the matrix cores with fp32 accumulation, and
// the b output rows are written back with 16-byte stores.  No LDS, no barriers: waves are
// independent, and latency is hidden by register double-buffering plus occupancy.
//
// MFMA operand layouts used (wave64, 16x16 output tile, lane l, q = l / 16, r = l % 16):
//   A (weights, M x K):  lane holds row r,    k = KL*q .. KL*q + KL-1
//   B (input,   K x N):  lane holds column r, k = KL*q .. KL*q + KL-1
//   D (output,  M x N):  lane holds column r, rows 4*q .. 4*q + 3
// with KL = 1 for v_mfma_f32_16x16x4_f32, 4 for v_mfma_f32_16x16x16_f16 and 8 for
// v_mfma_f32_16x16x32_f16.  A lane loads VEC consecutive batch columns of one input row, so
// it feeds VEC different 16-column MFMA tiles; tile v is made of columns {VEC*r + v}.  The
// same lane then owns VEC consecutive columns of every output row it holds, which makes the
// stores vectors as well.  For 16-bit MFMA operands a lane needs KL consecutive k of one
// column: it loads a KL x VEC block (KL rows) and transposes it in registers.
//
// Reference counterpart: kernel_bs_last_float / kernel_bs_last_half2
// (src/ksmm_py/layer/kronecker_sparse/template_kernels_float.cuh:297-491,
//  template_kernels_half.cuh:629-826), which stage both operands in shared memory and use
// scalar FMAs (and fp16 accumulation for half).
#include "ksmm_common.h"

namespace ksmm {

namespace {

template <int N> struct hvec;
template <> struct hvec<4> { typedef half4_t type; };
template <> struct hvec<8> { typedef half8_t type; };

// ---- row loaders: VEC consecutive batch columns of one input row, kept packed ------------
// raw_t<TX, VEC>: the dwords as loaded; unpack() turns them into VEC/2 dwords of fp16 pairs.
template <typename TX, int VEC> struct row_io;
template <int VEC> struct row_io<half_t, VEC> {
    static constexpr int RAW = VEC / 2;  // dwords per row load
    __device__ static __forceinline__ void load(const half_t *p, bool ok, uint32_t (&o)[RAW])
    {
        if constexpr (VEC == 8) {
            uint4_t v = {0, 0, 0, 0};
            if (ok) v = *(const uint4_t *)p;
            o[0] = v[0]; o[1] = v[1]; o[2] = v[2]; o[3] = v[3];
        } else {
            uint2_t v = {0, 0};
            if (ok) v = *(const uint2_t *)p;
            o[0] = v[0]; o[1] = v[1];
        }
    }
    __device__ static __forceinline__ void unpack(const uint32_t (&in)[RAW], uint32_t (&o)[VEC / 2])
    {
#pragma unroll
        for (int i = 0; i < RAW; ++i) o[i] = in[i];
    }
};
template <int VEC> struct row_io<fp8_t, VEC> {
    static constexpr int RAW = VEC / 4;
    __device__ static __forceinline__ void load(const fp8_t *p, bool ok, uint32_t (&o)[RAW])
    {
        if constexpr (VEC == 16) {
            uint4_t v = {0, 0, 0, 0};
            if (ok) v = *(const uint4_t *)p;
            o[0] = v[0]; o[1] = v[1]; o[2] = v[2]; o[3] = v[3];
        } else {
            uint2_t v = {0, 0};
            if (ok) v = *(const uint2_t *)p;
            o[0] = v[0]; o[1] = v[1];
        }
    }
    __device__ static __forceinline__ void unpack(const uint32_t (&in)[RAW], uint32_t (&o)[VEC / 2])
    {
#pragma unroll
        for (int i = 0; i < RAW; ++i) {
            o[2 * i] = __builtin_bit_cast(uint32_t, fp8x2_to_half2(in[i]));
            o[2 * i + 1] = __builtin_bit_cast(uint32_t, fp8x2_to_half2(in[i] >> 16));
        }
    }
};

// fp16 pair {column v of row A, column v of row B} from two packed rows
__device__ __forceinline__ uint32_t pick_pair(uint32_t row_a, uint32_t row_b, int odd)
{
    return odd ? __builtin_amdgcn_perm(row_b, row_a, 0x07060302u)
               : __builtin_amdgcn_perm(row_b, row_a, 0x05040100u);
}

template <int KL> struct mfma16;
template <> struct mfma16<4> {
    __device__ static __forceinline__ float4_t run(half4_t a, half4_t b, float4_t c)
    {
        return __builtin_amdgcn_mfma_f32_16x16x16f16(a, b, c, 0, 0, 0);
    }
};
template <> struct mfma16<8> {
    __device__ static __forceinline__ float4_t run(half8_t a, half8_t b, float4_t c)
    {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
    }
};

// ------------------------------------------------------------------------------------------
// fp32: v_mfma_f32_16x16x4_f32, VEC = 4 (16-byte loads and stores)
// MT = b / 16, KS = c / 4.  Each wave iteration covers 64 batch columns.
// ------------------------------------------------------------------------------------------
template <int MT, int KS, bool PREFETCH>
__global__ __launch_bounds__(256) void ks_wave_bl_f32(const float *__restrict__ x,
                                                     const float *__restrict__ w,
                                                     float *__restrict__ y, int batch, int a, int b,
                                                     int c, int d, float scale, int n_slabs,
                                                     int iters)
{
    constexpr int VEC = 4, TN = 16 * VEC;
    const int lane = threadIdx.x & 63;
    const int q = lane >> 4, r = lane & 15;
    const int wave = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    const int g = wave / n_slabs;  // block index a_i * d + d_i
    if (g >= a * d) return;
    const int slab = wave - g * n_slabs;
    const int a_i = g / d, d_i = g - a_i * d;

    // weights -> A operands, once per wave
    float areg[MT][KS];
    {
        const float *wg = w + (size_t)g * c * b;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks)
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) areg[mt][ks] = wg[(4 * ks + q) * b + 16 * mt + r];
    }
    const size_t row_stride = (size_t)d * batch;
    const float *xg = x + ((size_t)a_i * c * d + d_i) * batch + (size_t)q * row_stride;
    float *yg = y + ((size_t)a_i * b * d + d_i) * batch;

    int n = slab * iters * TN + VEC * r;
    float4_t xc[KS], xn[KS];
    auto load_tile = [&](float4_t(&dst)[KS], int col) {
        const bool ok = col < batch;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            float4_t v = {0.f, 0.f, 0.f, 0.f};
            if (ok) v = *(const float4_t *)(xg + (size_t)(4 * ks) * row_stride + col);
            dst[ks] = v;
        }
    };
    load_tile(xc, n);
    for (int it = 0; it < iters; ++it, n += TN) {
        if (n - VEC * r >= batch) break;  // uniform across the wave
        if (PREFETCH && it + 1 < iters) load_tile(xn, n + TN);
        float4_t acc[MT][VEC];
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int v = 0; v < VEC; ++v) acc[mt][v] = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int ks = 0; ks < KS; ++ks)
#pragma unroll
            for (int v = 0; v < VEC; ++v)
#pragma unroll
                for (int mt = 0; mt < MT; ++mt)
                    acc[mt][v] = __builtin_amdgcn_mfma_f32_16x16x4f32(areg[mt][ks], xc[ks][v],
                                                                      acc[mt][v], 0, 0, 0);
        if (n < batch) {
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    float4_t o = {acc[mt][0][i] * scale, acc[mt][1][i] * scale,
                                  acc[mt][2][i] * scale, acc[mt][3][i] * scale};
                    *(float4_t *)(yg + (size_t)(16 * mt + 4 * q + i) * row_stride + n) = o;
                }
        }
        if (PREFETCH) {
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) xc[ks] = xn[ks];
        } else if (it + 1 < iters) {
            load_tile(xc, n + TN);
        }
    }
}

// ------------------------------------------------------------------------------------------
// 16-bit MFMA path: x is fp16 or e4m3fn (decoded to fp16, exact), w is fp16 or e4m3fn,
// y is fp16.  MT = b / 16, KS = c / (4 * KL).  Each wave iteration covers 16 * VEC columns.
// ------------------------------------------------------------------------------------------
template <typename TX, typename TW, int MT, int KS, int KL, int VEC, bool PREFETCH>
__global__ __launch_bounds__(256) void ks_wave_bl_h(const TX *__restrict__ x,
                                                   const TW *__restrict__ w,
                                                   half_t *__restrict__ y, int batch, int a, int b,
                                                   int c, int d, float scale, int n_slabs, int iters)
{
    constexpr int TN = 16 * VEC, KSTEP = 4 * KL;
    typedef typename hvec<KL>::type frag_t;
    const int lane = threadIdx.x & 63;
    const int q = lane >> 4, r = lane & 15;
    const int wave = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    const int g = wave / n_slabs;
    if (g >= a * d) return;
    const int slab = wave - g * n_slabs;
    const int a_i = g / d, d_i = g - a_i * d;

    frag_t areg[MT][KS];
    {
        const TW *wg = w + (size_t)g * c * b;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks)
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
#pragma unroll
                for (int jj = 0; jj < KL; ++jj)
                    areg[mt][ks][jj] =
                        (half_t)elem<TW>::load(wg + (KSTEP * ks + KL * q + jj) * b + 16 * mt + r);
    }
    const size_t row_stride = (size_t)d * batch;
    const TX *xg = x + ((size_t)a_i * c * d + d_i) * batch + (size_t)(KL * q) * row_stride;
    half_t *yg = y + ((size_t)a_i * b * d + d_i) * batch;

    typedef row_io<TX, VEC> io;
    struct raw_t {
        uint32_t e[KS][KL][io::RAW];
    };
    struct tile_t {
        uint32_t e[KS][KL][VEC / 2];  // fp16 pairs: columns (2i, 2i+1) of row (ks, jj)
    };
    int n = slab * iters * TN + VEC * r;
    raw_t xn;
    tile_t xc;
    auto load_tile = [&](raw_t &dst, int col) {
        const bool ok = col < batch;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks)
#pragma unroll
            for (int jj = 0; jj < KL; ++jj)
                io::load(xg + (size_t)(KSTEP * ks + jj) * row_stride + col, ok, dst.e[ks][jj]);
    };
    auto unpack_tile = [&](const raw_t &src, tile_t &dst) {
#pragma unroll
        for (int ks = 0; ks < KS; ++ks)
#pragma unroll
            for (int jj = 0; jj < KL; ++jj) io::unpack(src.e[ks][jj], dst.e[ks][jj]);
    };
    load_tile(xn, n);
    for (int it = 0; it < iters; ++it, n += TN) {
        if (n - VEC * r >= batch) break;
        unpack_tile(xn, xc);
        if (PREFETCH && it + 1 < iters) load_tile(xn, n + TN);
        float4_t acc[MT][VEC];
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int v = 0; v < VEC; ++v) acc[mt][v] = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int ks = 0; ks < KS; ++ks)
#pragma unroll
            for (int v = 0; v < VEC; ++v) {
                // KL consecutive k of batch column VEC*r + v: in-register transpose
                uint32_t bw[KL / 2];
#pragma unroll
                for (int pp = 0; pp < KL / 2; ++pp)
                    bw[pp] = pick_pair(xc.e[ks][2 * pp][v / 2], xc.e[ks][2 * pp + 1][v / 2], v & 1);
                frag_t bf;
                if constexpr (KL == 8)
                    bf = __builtin_bit_cast(frag_t, uint4_t{bw[0], bw[1], bw[2], bw[3]});
                else
                    bf = __builtin_bit_cast(frag_t, uint2_t{bw[0], bw[1]});
#pragma unroll
                for (int mt = 0; mt < MT; ++mt)
                    acc[mt][v] = mfma16<KL>::run(areg[mt][ks], bf, acc[mt][v]);
            }
        if (n < batch) {
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    half_t *dst = yg + (size_t)(16 * mt + 4 * q + i) * row_stride + n;
                    constexpr int W = 8 < VEC ? 8 : VEC;  // halves per store (<= 16 bytes)
#pragma unroll
                    for (int v0 = 0; v0 < VEC; v0 += W) {
                        typename hvec<W>::type o;
#pragma unroll
                        for (int v = 0; v < W; ++v) o[v] = (half_t)(acc[mt][v0 + v][i] * scale);
                        *(typename hvec<W>::type *)(dst + v0) = o;
                    }
                }
        }
        if (!PREFETCH && it + 1 < iters) load_tile(xn, n + TN);
    }
}

// ---- instance table ---------------------------------------------------------------------
struct WaveInst {
    int b, c, vec, kl, prefetch;
    const void *fn;
};

typedef void (*f32_fn)(const float *, const float *, float *, int, int, int, int, int, float, int, int);
template <typename TX, typename TW>
using h_fn = void (*)(const TX *, const TW *, half_t *, int, int, int, int, int, float, int, int);

#define F32_INST(B_, C_, PF_) \
    {B_, C_, 4, 1, PF_, (const void *)(f32_fn)ks_wave_bl_f32<B_ / 16, C_ / 4, PF_>}
const WaveInst f32_insts[] = {
    F32_INST(48, 48, true),  F32_INST(48, 48, false), F32_INST(64, 64, true), F32_INST(64, 64, false),
    F32_INST(16, 16, true),  F32_INST(32, 32, true),
};

#define H_INST(TX_, TW_, B_, C_, KL_, VEC_, PF_)                            \
    {B_, C_, VEC_, KL_, PF_,                                                \
     (const void *)(h_fn<TX_, TW_>)ks_wave_bl_h<TX_, TW_, B_ / 16, C_ / (4 * KL_), KL_, VEC_, PF_>}
const WaveInst h_insts[] = {
    H_INST(half_t, half_t, 64, 64, 8, 4, true),  H_INST(half_t, half_t, 64, 64, 8, 8, true),
    H_INST(half_t, half_t, 64, 64, 8, 4, false), H_INST(half_t, half_t, 48, 48, 4, 4, true),
    H_INST(half_t, half_t, 48, 48, 4, 8, true),  H_INST(half_t, half_t, 16, 16, 4, 8, true),
    H_INST(half_t, half_t, 16, 16, 4, 4, true),  H_INST(half_t, half_t, 32, 32, 8, 8, true),
    H_INST(half_t, half_t, 96, 96, 8, 4, false),
};
const WaveInst hq_insts[] = {
    H_INST(half_t, fp8_t, 64, 64, 8, 4, true),  H_INST(half_t, fp8_t, 64, 64, 8, 8, true),
    H_INST(half_t, fp8_t, 64, 64, 8, 4, false), H_INST(half_t, fp8_t, 48, 48, 4, 4, true),
    H_INST(half_t, fp8_t, 48, 48, 4, 8, true),  H_INST(half_t, fp8_t, 16, 16, 4, 8, true),
    H_INST(half_t, fp8_t, 16, 16, 4, 4, true),  H_INST(half_t, fp8_t, 32, 32, 8, 8, true),
    H_INST(half_t, fp8_t, 96, 96, 8, 4, false),
};
const WaveInst q_insts[] = {
    H_INST(fp8_t, fp8_t, 64, 64, 8, 8, true),  H_INST(fp8_t, fp8_t, 64, 64, 8, 8, false),
    H_INST(fp8_t, fp8_t, 48, 48, 4, 8, true),  H_INST(fp8_t, fp8_t, 16, 16, 4, 16, true),
    H_INST(fp8_t, fp8_t, 16, 16, 4, 8, true),  H_INST(fp8_t, fp8_t, 32, 32, 8, 16, true),
    H_INST(fp8_t, fp8_t, 32, 32, 8, 8, true),
};

}  // namespace

int wave_run(const Problem &p, int variant, bool launch, ksmm_tile *tile)
{
    if (!p.bs_last) return KSMM_ERR_BAD_ALGO;
    const int combo = combo_of(p.x_dtype, p.w_dtype, p.y_dtype);
    const WaveInst *insts;
    int n_insts;
    switch (combo) {
    case 0: insts = f32_insts; n_insts = sizeof(f32_insts) / sizeof(WaveInst); break;
    case 1: insts = h_insts; n_insts = sizeof(h_insts) / sizeof(WaveInst); break;
    case 2: insts = q_insts; n_insts = sizeof(q_insts) / sizeof(WaveInst); break;
    case 3: insts = hq_insts; n_insts = sizeof(hq_insts) / sizeof(WaveInst); break;
    default: return KSMM_ERR_BAD_DTYPE;
    }
    // vector loads along the batch axis need every row start aligned to the vector
    // variant: bits 0-7 instance index (0xff: first that fits), bits 8-15 wave iterations
    // (0: heuristic); -1: everything automatic
    const int want = variant < 0 ? 0xff : (variant & 0xff);
    int iters = variant < 0 ? 0 : ((variant >> 8) & 0xff);
    int pick = -1;
    for (int i = 0; i < n_insts; ++i) {
        if (insts[i].b != p.b || insts[i].c != p.c) continue;
        if (p.batch % insts[i].vec) continue;
        if (want != 0xff && want != i) continue;
        pick = i;
        break;
    }
    if (pick < 0) return KSMM_ERR_BAD_ALGO;
    const WaveInst &in = insts[pick];
    const int tn = 16 * in.vec;
    const int64_t n_tiles = (p.batch + tn - 1) / tn;
    // columns per wave: enough wave-iterations to amortise the weight load, while keeping
    // several waves per SIMD busy on all 256 CUs
    const int64_t groups = (int64_t)p.a * p.d;
    if (iters == 0) {
        iters = 4;
        while (iters > 1 && groups * ((n_tiles + iters - 1) / iters) < 256 * 4 * 4) iters >>= 1;
    }
    const int64_t n_slabs = (n_tiles + iters - 1) / iters;
    const int64_t waves = groups * n_slabs;
    const int wpb = 4;
    const int64_t blocks = (waves + wpb - 1) / wpb;
    if (blocks > 0x7fffffffLL) return KSMM_ERR_TOO_LARGE;
    if (tile) {
        tile->algo = KSMM_ALGO_WAVE;
        tile->variant = pick;
        tile->tile_m = p.b;
        tile->tile_n = tn;
        tile->tile_k = p.c;
        tile->tile_d = 1;
        tile->threads = 64 * wpb;
        tile->lds_bytes = 0;
        tile->grid = blocks;
    }
    if (!launch) return KSMM_OK;
    void *args[] = {(void *)&p.x, (void *)&p.w, (void *)&p.y, nullptr, (void *)&p.a, (void *)&p.b,
                    (void *)&p.c, (void *)&p.d, (void *)&p.scale, nullptr, nullptr};
    int batch_i = (int)p.batch, n_slabs_i = (int)n_slabs;
    args[3] = &batch_i;
    args[9] = &n_slabs_i;
    args[10] = &iters;
    hipError_t e = hipLaunchKernel(in.fn, dim3((unsigned)blocks), dim3(64 * wpb), args, 0, p.stream);
    return e == hipSuccess ? KSMM_OK : KSMM_ERR_LAUNCH;
}

}  // namespace ksmm
