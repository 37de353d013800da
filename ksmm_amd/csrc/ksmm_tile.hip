// "Tile" family: LDS-staged MFMA kernel for b x c blocks that are real dense contractions.
//
// For one (a_i, d_i) block the factor is a GEMM  Y[b x B] = W[b x c] * X[c x B].  A workgroup
// computes a TM (outputs) x TN (batch) tile, looping over c in slabs of TK that are staged in
// LDS (double-buffered: the global loads of slab s+1 are in flight while slab s is multiplied).
// 32x32 MFMA tiles with fp32 accumulation: v_mfma_f32_32x32x2_f32 for fp32,
// v_mfma_f32_32x32x16_f16 for fp16 (e4m3fn operands are decoded to fp16 while they are
// written to LDS, which is exact).
//
// Layout handling.  Both operands of a 16-bit MFMA want 8 consecutive k per lane.  The weight
// is stored (c x b) with b contiguous and, batch-size-last, the input is (c x B) with B
// contiguous: both "k-outer".  They are copied to LDS as they are and read back with
// ds_read_b64_tr_b16, the gfx950 LDS transpose load (within 16 lanes, lane i receives
// element i of each of the four 32-byte rows the group addresses).  Batch-size-first input
// rows are already k-contiguous (d == 1) and are read with plain 16-byte LDS loads.  In both
// layouts A = X (rows = batch) and B = W (lanes = outputs):
//   bs_last : a lane holds 4 consecutive batch elements of one output; the tile is transposed
//             through LDS after the k loop and stored as 16-byte row pieces  -> y[(.)*d*B + n]
//   bs_first: the 32 lanes of a tile row store 32 consecutive outputs       -> y[n*out + (.)]
//
// Workgroup ids are remapped so that the workgroups that share an input tile (the TM-tiles of
// one batch tile) run on the same XCD and hit the same L2.
//
// Reference counterpart: kernel_bs_{first,last}_{float,half2,half4}
// (src/ksmm_py/layer/kronecker_sparse/template_kernels_float.cuh:85-491,
//  template_kernels_half.cuh:103-1092): same tiling idea (TILEX x TILEY output tile, TILEK
// slabs, double-buffered shared memory) with scalar FMAs and fp16 accumulation for half.
#include "ksmm_mfma.h"

namespace ksmm {

namespace {

template <typename CT, typename TX, typename TW, typename TY, bool BS_LAST, int TM, int TN, int TK,
          int WM, int WN>
struct TileCfg {
    static constexpr int THREADS = 64 * WM * WN;
    static constexpr int MT = TM / WM / 32, NT = TN / WN / 32;  // 32x32 MFMA tiles per wave
    static constexpr int LDW = pads<CT>::outer(TM);
    static constexpr int LDX = BS_LAST ? pads<CT>::outer(TN) : pads<CT>::inner(TK);
    static constexpr int W_ELEMS = TK * LDW;
    static constexpr int X_ELEMS = BS_LAST ? TK * LDX : TN * LDX;
    static constexpr int LDS_BYTES = 2 * (W_ELEMS + X_ELEMS) * (int)sizeof(CT);
    static constexpr int W_EPV = stage<TW, CT>::EPV, X_EPV = stage<TX, CT>::EPV;
    static constexpr int W_VECS = TK * TM / W_EPV, X_VECS = TK * TN / X_EPV;
    static constexpr int W_PER_T = (W_VECS + THREADS - 1) / THREADS, X_PER_T = (X_VECS + THREADS - 1) / THREADS;
    static_assert(TM % (32 * WM) == 0 && TN % (32 * WN) == 0, "wave tiling");
    static_assert(TK % compute<CT>::KSTEP == 0, "k slab");
    static_assert(TM % W_EPV == 0 && (BS_LAST ? TN % X_EPV == 0 : TK % X_EPV == 0), "vector width");
    static_assert(LDS_BYTES <= 160 * 1024, "LDS");
};

// RB ("ragged b"): b need not be a multiple of TM nor of the 16-byte weight vector.  The weight
// rows are then not 16-byte aligned: vectors that lie inside the block are fetched with one
// unaligned 16-byte load, the vector that straddles b element by element; columns behind b are
// zeros and are not stored.
template <typename CT, typename TX, typename TW, typename TY, bool BS_LAST, int TM, int TN, int TK,
          int WM, int WN, bool RB>
__global__ __launch_bounds__(64 * WM * WN) void ks_tile_kernel(const TX *__restrict__ x,
                                                              const TW *__restrict__ w,
                                                              TY *__restrict__ y, int batch, int a,
                                                              int b, int c, int d, Epi ep,
                                                              int m_tiles, int n_tiles, int blocks)
{
    typedef TileCfg<CT, TX, TW, TY, BS_LAST, TM, TN, TK, WM, WN> C;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    CT *const lds = (CT *)smem;
    auto ws = [&](int buf) { return lds + buf * C::W_ELEMS; };
    auto xs = [&](int buf) { return lds + 2 * C::W_ELEMS + buf * C::X_ELEMS; };

    // XCD-aware id: hardware deals consecutive workgroup ids round-robin to the 8 XCDs; give
    // each XCD a contiguous range of logical ids so that TM-tiles of one input tile share an L2.
    const int per_xcd = (blocks + 7) / 8;
    const int lid = (blockIdx.x % 8) * per_xcd + blockIdx.x / 8;
    if (lid >= blocks) return;
    const int mt_id = lid % m_tiles;
    const int rest = lid / m_tiles;
    const int nt_id = rest % n_tiles;
    const int g = rest / n_tiles;  // a_i * d + d_i
    const int a_i = g / d, d_i = g - a_i * d;
    const int m0 = mt_id * TM, n0 = nt_id * TN;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave / WN, wn = wave % WN;

    const size_t in_size = (size_t)a * c * d, out_size = (size_t)a * b * d;
    const TW *wg = w + (size_t)g * c * b + m0;  // row k: + k * b
    // x element (k, n): bs_last ((a_i*c + k)*d + d_i)*batch + n ; bs_first (d == 1) n*in + a_i*c + k
    const TX *xg = BS_LAST ? x + ((size_t)a_i * c * d + d_i) * batch : x + (size_t)a_i * c;
    const size_t x_kstride = BS_LAST ? (size_t)d * batch : 1;

    stage<TW, CT> wreg[C::W_PER_T];
    stage<TX, CT> xreg[C::X_PER_T];

    auto gload = [&](int k0) {
#pragma unroll
        for (int i = 0; i < C::W_PER_T; ++i) {
            const int v = tid + i * C::THREADS;
            if (C::W_VECS % C::THREADS == 0 || v < C::W_VECS) {
                const int kk = v / (TM / C::W_EPV), mm = (v % (TM / C::W_EPV)) * C::W_EPV;
                // batch-size-last: c need not be a multiple of TK; rows past the block are zeros
                if (BS_LAST && k0 + kk >= c) {
                    wreg[i].v = uint4_t{0u, 0u, 0u, 0u};
                } else if constexpr (RB) {
                    union {
                        uint4_t v;
                        TW e[C::W_EPV];
                    } u;
                    u.v = uint4_t{0u, 0u, 0u, 0u};
                    const TW *src = wg + (size_t)(k0 + kk) * b + mm;
                    if (m0 + mm + C::W_EPV <= b) {
                        // whole vector inside the block: one 16-byte load at element alignment
                        // (global memory takes unaligned vector accesses)
                        __builtin_memcpy(&u.v, src, 16);
                    } else {
#pragma unroll
                        for (int j = 0; j < C::W_EPV; ++j)
                            if (m0 + mm + j < b) u.e[j] = src[j];
                    }
                    wreg[i].v = u.v;
                } else {
                    wreg[i].load(wg + (size_t)(k0 + kk) * b + mm);
                }
            }
        }
#pragma unroll
        for (int i = 0; i < C::X_PER_T; ++i) {
            const int v = tid + i * C::THREADS;
            if (C::X_VECS % C::THREADS == 0 || v < C::X_VECS) {
                if (BS_LAST) {
                    const int kk = v / (TN / C::X_EPV), nn = (v % (TN / C::X_EPV)) * C::X_EPV;
                    // columns past the end are clamped to the last valid vector (never stored)
                    const int col = min(n0 + nn, batch - C::X_EPV);
                    if (k0 + kk >= c)
                        xreg[i].v = uint4_t{0u, 0u, 0u, 0u};
                    else
                        xreg[i].load(xg + (size_t)(k0 + kk) * x_kstride + col);
                } else {
                    const int nn = v / (TK / C::X_EPV), kk = (v % (TK / C::X_EPV)) * C::X_EPV;
                    const int row = min(n0 + nn, batch - 1);
                    xreg[i].load(xg + (size_t)row * in_size + k0 + kk);
                }
            }
        }
    };
    auto lstore = [&](int buf) {
#pragma unroll
        for (int i = 0; i < C::W_PER_T; ++i) {
            const int v = tid + i * C::THREADS;
            if (C::W_VECS % C::THREADS == 0 || v < C::W_VECS) {
                const int kk = v / (TM / C::W_EPV), mm = (v % (TM / C::W_EPV)) * C::W_EPV;
                wreg[i].store(ws(buf) + kk * C::LDW + mm);
            }
        }
#pragma unroll
        for (int i = 0; i < C::X_PER_T; ++i) {
            const int v = tid + i * C::THREADS;
            if (C::X_VECS % C::THREADS == 0 || v < C::X_VECS) {
                if (BS_LAST) {
                    const int kk = v / (TN / C::X_EPV), nn = (v % (TN / C::X_EPV)) * C::X_EPV;
                    xreg[i].store(xs(buf) + kk * C::LDX + nn);
                } else {
                    const int nn = v / (TK / C::X_EPV), kk = (v % (TK / C::X_EPV)) * C::X_EPV;
                    xreg[i].store(xs(buf) + nn * C::LDX + kk);
                }
            }
        }
    };

    float16_t acc[C::MT][C::NT];
#pragma unroll
    for (int i = 0; i < C::MT; ++i)
#pragma unroll
        for (int j = 0; j < C::NT; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

    const int steps = BS_LAST ? (c + TK - 1) / TK : c / TK;
    gload(0);
    lstore(0);
    __syncthreads();
    for (int s = 0; s < steps; ++s) {
        const int buf = s & 1;
        if (s + 1 < steps) gload((s + 1) * TK);
        const CT *wb = ws(buf), *xb = xs(buf);
#pragma unroll
        for (int k0 = 0; k0 < TK; k0 += compute<CT>::KSTEP) {
            typename frag<CT>::type fw[C::MT], fx[C::NT];
#pragma unroll
            for (int i = 0; i < C::MT; ++i)
                fw[i] = frag<CT>::k_outer(wb, C::LDW, (wm * C::MT + i) * 32, k0, lane);
#pragma unroll
            for (int j = 0; j < C::NT; ++j)
                fx[j] = BS_LAST ? frag<CT>::k_outer(xb, C::LDX, (wn * C::NT + j) * 32, k0, lane)
                                : frag<CT>::k_inner(xb, C::LDX, (wn * C::NT + j) * 32, k0, lane);
#pragma unroll
            for (int i = 0; i < C::MT; ++i)
#pragma unroll
                for (int j = 0; j < C::NT; ++j)
                    // A = input rows along the batch, B = weights: a lane ends up with 4 consecutive
                    // batch elements of one output feature (batch-size-last: the contiguous axis)
                    acc[i][j] = frag<CT>::mfma(fx[j], fw[i], acc[i][j]);
        }
        if (s + 1 < steps) lstore(buf ^ 1);
        __syncthreads();
    }

    // D tile: lane holds column (lane % 32) of the B operand (an output feature) and rows
    // 8*(e/4) + 4*(lane/32) + e%4 of the A operand (batch elements)
    const int l32 = lane & 31, lq = lane >> 5;
    if constexpr (BS_LAST) {
        // 4 consecutive batch elements per lane and 8-row group: the tile goes through LDS (the
        // staging buffers are free now) in passes of RPP rows and leaves as 16-byte row pieces
        constexpr int OES = (int)sizeof(TY), OEPC = 16 / OES;
        constexpr int RC = TN + OEPC;  // padded row, elements
        constexpr int RPP_RAW = C::LDS_BYTES / (RC * OES) / 32 * 32;
        constexpr int RPP = RPP_RAW > TM ? TM : RPP_RAW;
        constexpr int PASSES = (TM + RPP - 1) / RPP;
        constexpr int CPR = TN / OEPC;
        static_assert(RPP >= 32, "output pass");
        TY *const out = (TY *)smem;
#pragma unroll
        for (int pass = 0; pass < PASSES; ++pass) {
            if (pass > 0) __syncthreads();
#pragma unroll
            for (int i = 0; i < C::MT; ++i)
#pragma unroll
                for (int j = 0; j < C::NT; ++j) {
                    const int lrow = (wm * C::MT + i) * 32 + l32, rcol = (wn * C::NT + j) * 32 + 4 * lq;
                    if (lrow / RPP != pass) continue;  // uniform per wave (32-row tiles)
                    TY *dst = out + (lrow - pass * RPP) * RC + rcol;
                    // the lane's output feature (clamped: rows behind b are not stored)
                    const float bv = epi_bias<TY>(ep, ((size_t)a_i * b + min(m0 + lrow, b - 1)) * d + d_i);
#pragma unroll
                    for (int eg = 0; eg < 4; ++eg) {
                        float v[4];
#pragma unroll
                        for (int u = 0; u < 4; ++u) v[u] = epi_finish(ep, acc[i][j][4 * eg + u], bv);
                        if constexpr (sizeof(TY) == 4)
                            *(float4_t *)(dst + 8 * eg) = float4_t{v[0], v[1], v[2], v[3]};
                        else
                            *(half4_t *)(dst + 8 * eg) = half4_t{(half_t)v[0], (half_t)v[1], (half_t)v[2], (half_t)v[3]};
                    }
                }
            __syncthreads();
            for (int q = tid; q < RPP * CPR; q += C::THREADS) {
                const int r = q / CPR, cc = (q % CPR) * OEPC;
                const int row = pass * RPP + r;
                if (row >= TM) break;
                const int m = m0 + row, n = n0 + cc;
                if (n < batch && (!RB || m < b))
                    *(uint4_t *)(y + ((size_t)(a_i * b + m) * d + d_i) * batch + n) = *(const uint4_t *)(out + r * RC + cc);
            }
        }
    } else {
#pragma unroll
        for (int i = 0; i < C::MT; ++i)
#pragma unroll
            for (int j = 0; j < C::NT; ++j) {
                const int mb = m0 + (wm * C::MT + i) * 32, nb = n0 + (wn * C::NT + j) * 32;
                const float bv = epi_bias<TY>(ep, (size_t)a_i * b + min(mb + l32, b - 1));  // d == 1 in this layout
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    const int rr = 8 * (e >> 2) + 4 * lq + (e & 3);
                    const float v = epi_finish(ep, acc[i][j][e], bv);
                    const int n = nb + rr, m = mb + l32;
                    if (n < batch && (!RB || m < b)) elem<TY>::store(y + (size_t)n * out_size + (size_t)a_i * b + m, v);
                }
            }
    }
}

// ------------------------------------------------------------------------------------------
// Weight-stationary variant for mid-sized blocks (b*c elements fit the register file of one
// workgroup): a persistent workgroup owns one (a_i, d_i) block and a contiguous range of batch
// tiles.  The b x c weight block is staged through LDS once and kept in registers as MFMA
// operands (split over WM waves); after that LDS only holds input tiles with the whole c
// extent, double-buffered across batch tiles, so that the HBM loads of tile t+1 are in flight
// while tile t is multiplied and stored.  This is the bandwidth-bound regime: per tile the
// matrix cores need a fraction of the time HBM needs.
// ------------------------------------------------------------------------------------------
template <typename CT, typename TX, typename TW, typename TY, bool BS_LAST, int BB, int CC, int TN,
          int WM, int WN>
struct WsCfg {
    static constexpr int THREADS = 64 * WM * WN;
    static constexpr int KSTEP = compute<CT>::KSTEP;
    static constexpr int MT = BB / WM / 32, NT = TN / WN / 32, KS = CC / KSTEP;
    static constexpr int LDW = pads<CT>::outer(BB);
    static constexpr int LDX = BS_LAST ? pads<CT>::outer(TN) : pads<CT>::inner(CC);
    static constexpr int W_ELEMS = CC * LDW;
    static constexpr int X_ELEMS = BS_LAST ? CC * LDX : TN * LDX;
    static constexpr int LDS_ELEMS = (2 * X_ELEMS > W_ELEMS) ? 2 * X_ELEMS : W_ELEMS;
    static constexpr int LDS_BYTES = LDS_ELEMS * (int)sizeof(CT);
    static constexpr int W_EPV = stage<TW, CT>::EPV, X_EPV = stage<TX, CT>::EPV;
    static constexpr int W_VECS = CC * BB / W_EPV, X_VECS = CC * TN / X_EPV;
    static constexpr int X_PER_T = (X_VECS + THREADS - 1) / THREADS;
    static_assert(BB % (32 * WM) == 0 && TN % (32 * WN) == 0, "wave tiling");
    static_assert(CC % KSTEP == 0 && BB % W_EPV == 0, "block shape");
    static_assert(BS_LAST ? TN % X_EPV == 0 : CC % X_EPV == 0, "vector width");
    static_assert(LDS_BYTES <= 160 * 1024, "LDS");
};

template <typename CT, typename TX, typename TW, typename TY, bool BS_LAST, int BB, int CC, int TN,
          int WM, int WN>
__global__ __launch_bounds__(64 * WM * WN) void ks_ws_kernel(const TX *__restrict__ x,
                                                            const TW *__restrict__ w,
                                                            TY *__restrict__ y, int batch, int a,
                                                            int d, Epi ep, int wgs_per_group,
                                                            int n_tiles)
{
    typedef WsCfg<CT, TX, TW, TY, BS_LAST, BB, CC, TN, WM, WN> C;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    CT *const lds = (CT *)smem;
    const int g = blockIdx.x / wgs_per_group;  // a_i * d + d_i
    const int s = blockIdx.x - g * wgs_per_group;
    const int per = (n_tiles + wgs_per_group - 1) / wgs_per_group;
    const int t_begin = s * per, t_end = min(n_tiles, t_begin + per);
    if (t_begin >= t_end) return;
    const int a_i = g / d, d_i = g - a_i * d;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave / WN, wn = wave % WN;
    const size_t in_size = (size_t)a * CC * d, out_size = (size_t)a * BB * d;

    // ---- weights: global -> LDS (as stored, c x b) -> registers (MFMA operand layout) ----
    {
        const TW *wg = w + (size_t)g * CC * BB;
        // all loads first, then all LDS writes: one memory latency instead of one per vector
        constexpr int W_PER_T = (C::W_VECS + C::THREADS - 1) / C::THREADS;
        stage<TW, CT> r[W_PER_T];
#pragma unroll
        for (int i = 0; i < W_PER_T; ++i) {
            const int v = min(tid + i * C::THREADS, C::W_VECS - 1);
            r[i].load(wg + (size_t)(v / (BB / C::W_EPV)) * BB + (v % (BB / C::W_EPV)) * C::W_EPV);
        }
#pragma unroll
        for (int i = 0; i < W_PER_T; ++i) {
            const int v = min(tid + i * C::THREADS, C::W_VECS - 1);
            r[i].store(lds + (v / (BB / C::W_EPV)) * C::LDW + (v % (BB / C::W_EPV)) * C::W_EPV);
        }
    }
    __syncthreads();
    typename frag<CT>::type wreg[C::MT][C::KS];
#pragma unroll
    for (int i = 0; i < C::MT; ++i)
#pragma unroll
        for (int ks = 0; ks < C::KS; ++ks)
            wreg[i][ks] = frag<CT>::k_outer(lds, C::LDW, (wm * C::MT + i) * 32, ks * C::KSTEP, lane);
    __syncthreads();  // LDS is reused for the input tiles from here on

    const TX *xg = BS_LAST ? x + ((size_t)a_i * CC * d + d_i) * batch : x + (size_t)a_i * CC;
    const size_t x_kstride = BS_LAST ? (size_t)d * batch : 1;
    stage<TX, CT> xreg[C::X_PER_T];
    auto gload = [&](int t) {
        const int n0 = t * TN;
#pragma unroll
        for (int i = 0; i < C::X_PER_T; ++i) {
            const int v = tid + i * C::THREADS;
            if (C::X_VECS % C::THREADS == 0 || v < C::X_VECS) {
                if (BS_LAST) {
                    const int kk = v / (TN / C::X_EPV), nn = (v % (TN / C::X_EPV)) * C::X_EPV;
                    const int col = min(n0 + nn, batch - C::X_EPV);
                    xreg[i].load(xg + (size_t)kk * x_kstride + col);
                } else {
                    const int nn = v / (CC / C::X_EPV), kk = (v % (CC / C::X_EPV)) * C::X_EPV;
                    const int row = min(n0 + nn, batch - 1);
                    xreg[i].load(xg + (size_t)row * in_size + kk);
                }
            }
        }
    };
    auto lstore = [&](int buf) {
        CT *xb = lds + buf * C::X_ELEMS;
#pragma unroll
        for (int i = 0; i < C::X_PER_T; ++i) {
            const int v = tid + i * C::THREADS;
            if (C::X_VECS % C::THREADS == 0 || v < C::X_VECS) {
                if (BS_LAST) {
                    const int kk = v / (TN / C::X_EPV), nn = (v % (TN / C::X_EPV)) * C::X_EPV;
                    xreg[i].store(xb + kk * C::LDX + nn);
                } else {
                    const int nn = v / (CC / C::X_EPV), kk = (v % (CC / C::X_EPV)) * C::X_EPV;
                    xreg[i].store(xb + nn * C::LDX + kk);
                }
            }
        }
    };

    const int l32 = lane & 31, lq = lane >> 5;
    gload(t_begin);
    lstore(0);
    __syncthreads();
    for (int t = t_begin; t < t_end; ++t) {
        const int buf = (t - t_begin) & 1;
        if (t + 1 < t_end) gload(t + 1);
        const CT *xb = lds + buf * C::X_ELEMS;
        float16_t acc[C::MT][C::NT];
#pragma unroll
        for (int i = 0; i < C::MT; ++i)
#pragma unroll
            for (int j = 0; j < C::NT; ++j)
#pragma unroll
                for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;
#pragma unroll
        for (int ks = 0; ks < C::KS; ++ks) {
            typename frag<CT>::type fx[C::NT];
#pragma unroll
            for (int j = 0; j < C::NT; ++j)
                fx[j] = BS_LAST ? frag<CT>::k_outer(xb, C::LDX, (wn * C::NT + j) * 32, ks * C::KSTEP, lane)
                                : frag<CT>::k_inner(xb, C::LDX, (wn * C::NT + j) * 32, ks * C::KSTEP, lane);
#pragma unroll
            for (int i = 0; i < C::MT; ++i)
#pragma unroll
                for (int j = 0; j < C::NT; ++j)
                    acc[i][j] = BS_LAST ? frag<CT>::mfma(wreg[i][ks], fx[j], acc[i][j])
                                        : frag<CT>::mfma(fx[j], wreg[i][ks], acc[i][j]);
        }
        const int n0 = t * TN;
#pragma unroll
        for (int i = 0; i < C::MT; ++i)
#pragma unroll
            for (int j = 0; j < C::NT; ++j) {
                const int mb = (wm * C::MT + i) * 32, nb = n0 + (wn * C::NT + j) * 32;
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    const int rr = 8 * (e >> 2) + 4 * lq + (e & 3);
                    if (BS_LAST) {
                        const int m = mb + rr, n = nb + l32;
                        const size_t feature = (size_t)(a_i * BB + m) * d + d_i;
                        const float v = epi_finish(ep, acc[i][j][e], epi_bias<TY>(ep, feature));
                        if (n < batch) elem<TY>::store(y + feature * batch + n, v);
                    } else {
                        const int n = nb + rr, m = mb + l32;
                        const size_t feature = (size_t)a_i * BB + m;  // d == 1 in this layout
                        const float v = epi_finish(ep, acc[i][j][e], epi_bias<TY>(ep, feature));
                        if (n < batch) elem<TY>::store(y + (size_t)n * out_size + feature, v);
                    }
                }
            }
        if (t + 1 < t_end) lstore(buf ^ 1);
        __syncthreads();
    }
}

struct WsInst {
    int combo, bs_last, bb, cc, tn, threads, lds, wm;
    const void *fn;
};
#define WS_INST(COMBO_, CT_, TX_, TW_, TY_, BL_, BB_, CC_, TN_, WM_, WN_)                            \
    {COMBO_, BL_, BB_, CC_, TN_, 64 * WM_ * WN_,                                                    \
     WsCfg<CT_, TX_, TW_, TY_, BL_, BB_, CC_, TN_, WM_, WN_>::LDS_BYTES, WM_,                        \
     (const void *)ks_ws_kernel<CT_, TX_, TW_, TY_, BL_, BB_, CC_, TN_, WM_, WN_>}
#define WS_SET_H(COMBO_, TX_, TW_, BL_)                                                             \
    WS_INST(COMBO_, half_t, TX_, TW_, half_t, BL_, 192, 192, 64, 2, 2),                             \
        WS_INST(COMBO_, half_t, TX_, TW_, half_t, BL_, 192, 192, 128, 2, 2),                        \
        WS_INST(COMBO_, half_t, TX_, TW_, half_t, BL_, 128, 128, 64, 2, 2),                         \
        WS_INST(COMBO_, half_t, TX_, TW_, half_t, BL_, 128, 128, 128, 2, 2),                        \
        WS_INST(COMBO_, half_t, TX_, TW_, half_t, BL_, 96, 96, 128, 1, 4),                          \
        WS_INST(COMBO_, half_t, TX_, TW_, half_t, BL_, 64, 64, 128, 1, 4),                          \
        WS_INST(COMBO_, half_t, TX_, TW_, half_t, BL_, 64, 64, 64, 2, 2)
#define WS_SET_F32(BL_)                                                                             \
    WS_INST(0, float, float, float, float, BL_, 128, 128, 64, 2, 2),                                \
        WS_INST(0, float, float, float, float, BL_, 96, 96, 128, 1, 4),                             \
        WS_INST(0, float, float, float, float, BL_, 64, 64, 128, 1, 4),                             \
        WS_INST(0, float, float, float, float, BL_, 64, 64, 64, 2, 2)
const WsInst ws_insts[] = {
    WS_SET_F32(true),
    WS_SET_F32(false),
    WS_SET_H(1, half_t, half_t, true),
    WS_SET_H(1, half_t, half_t, false),
    WS_SET_H(2, fp8_t, fp8_t, true),
    WS_SET_H(2, fp8_t, fp8_t, false),
    WS_SET_H(3, half_t, fp8_t, true),
    WS_SET_H(3, half_t, fp8_t, false),
};
constexpr int N_WS_INSTS = sizeof(ws_insts) / sizeof(WsInst);

bool ws_fits(const WsInst &t, const Problem &p, int combo)
{
    if (t.combo != combo || t.bs_last != p.bs_last) return false;
    if (p.b != t.bb || p.c != t.cc) return false;
    const int x_epv = 16 / (int)dtype_size(p.x_dtype);
    if (p.bs_last) {
        if (p.batch % x_epv || p.batch < x_epv) return false;
    } else {
        if (p.d != 1) return false;
    }
    return true;
}

int ws_run(const Problem &p, int variant, int wgs_hint, bool launch, ksmm_tile *tile)
{
    const int combo = combo_of(p.x_dtype, p.w_dtype, p.y_dtype);
    int pick = -1;
    for (int i = 0; i < N_WS_INSTS; ++i) {
        if (variant >= 0 && variant != i) continue;
        if (ws_fits(ws_insts[i], p, combo)) {
            pick = i;
            break;
        }
    }
    if (pick < 0) return KSMM_ERR_BAD_ALGO;
    const WsInst &t = ws_insts[pick];
    const int64_t groups = (int64_t)p.a * p.d;
    const int64_t n_tiles = (p.batch + t.tn - 1) / t.tn;
    // persistent workgroups: about `target` per CU over all groups, never more than tiles
    const int per_cu = t.lds * 2 <= 160 * 1024 ? 2 : 1;
    int64_t wgs = wgs_hint > 0 ? wgs_hint : (256 * per_cu + groups - 1) / groups;
    if (wgs > n_tiles) wgs = n_tiles;
    if (wgs < 1) wgs = 1;
    const int64_t grid = groups * wgs;
    if (grid > 0x7fffffffLL) return KSMM_ERR_TOO_LARGE;
    if (tile) {
        tile->algo = KSMM_ALGO_TILE;
        tile->variant = (1 << 24) | pick;
        tile->tile_m = t.bb;
        tile->tile_n = t.tn;
        tile->tile_k = t.cc;
        tile->tile_d = 1;
        tile->threads = t.threads;
        tile->lds_bytes = t.lds;
        tile->grid = grid;
    }
    if (!launch) return KSMM_OK;
    if (ensure_dynamic_lds(t.fn, t.lds) != KSMM_OK) return KSMM_ERR_LAUNCH;
    int batch_i = (int)p.batch, wgs_i = (int)wgs, n_tiles_i = (int)n_tiles;
    Epi ep = epi_of(p);
    void *args[] = {(void *)&p.x, (void *)&p.w, (void *)&p.y, &batch_i, (void *)&p.a, (void *)&p.d,
                    &ep, &wgs_i, &n_tiles_i};
    hipError_t e = hipLaunchKernel(t.fn, dim3((unsigned)grid), dim3(t.threads), args, t.lds, p.stream);
    return e == hipSuccess ? KSMM_OK : KSMM_ERR_LAUNCH;
}

// ---- instance table -----------------------------------------------------------------------
struct TileInst {
    int combo, bs_last, tm, tn, tk, threads, lds;
    int ragged_b;
    int wm;
    const void *fn;
};

#define TILE_INST_R(COMBO_, CT_, TX_, TW_, TY_, BL_, TM_, TN_, TK_, WM_, WN_, RB_)                    \
    {COMBO_, BL_, TM_, TN_, TK_, 64 * WM_ * WN_,                                                    \
     TileCfg<CT_, TX_, TW_, TY_, BL_, TM_, TN_, TK_, WM_, WN_>::LDS_BYTES, RB_, WM_,                 \
     (const void *)ks_tile_kernel<CT_, TX_, TW_, TY_, BL_, TM_, TN_, TK_, WM_, WN_, RB_>}
#define TILE_INST(COMBO_, CT_, TX_, TW_, TY_, BL_, TM_, TN_, TK_, WM_, WN_)                          \
    TILE_INST_R(COMBO_, CT_, TX_, TW_, TY_, BL_, TM_, TN_, TK_, WM_, WN_, false)
#define TILE_SET_F32(BL_)                                                                           \
    TILE_INST(0, float, float, float, float, BL_, 128, 128, 16, 2, 2),                              \
        TILE_INST(0, float, float, float, float, BL_, 64, 128, 16, 1, 4),                           \
        TILE_INST(0, float, float, float, float, BL_, 32, 128, 16, 1, 4),                           \
        TILE_INST(0, float, float, float, float, BL_, 64, 256, 16, 1, 4),                           \
        TILE_INST(0, float, float, float, float, BL_, 128, 256, 16, 2, 2),                          \
        TILE_INST(0, float, float, float, float, BL_, 96, 128, 16, 1, 4)
#define TILE_SET_H(COMBO_, TX_, TW_, BL_)                                                           \
    TILE_INST(COMBO_, half_t, TX_, TW_, half_t, BL_, 128, 128, 32, 2, 2),                           \
        TILE_INST(COMBO_, half_t, TX_, TW_, half_t, BL_, 64, 128, 32, 1, 4),                        \
        TILE_INST(COMBO_, half_t, TX_, TW_, half_t, BL_, 32, 128, 32, 1, 4),                        \
        TILE_INST(COMBO_, half_t, TX_, TW_, half_t, BL_, 192, 128, 32, 2, 2),                       \
        TILE_INST(COMBO_, half_t, TX_, TW_, half_t, BL_, 128, 256, 32, 2, 2),                       \
        TILE_INST(COMBO_, half_t, TX_, TW_, half_t, BL_, 256, 256, 32, 2, 2),                       \
        TILE_INST(COMBO_, half_t, TX_, TW_, half_t, BL_, 64, 256, 64, 1, 4)

const TileInst tile_insts[] = {
    TILE_SET_F32(true),
    TILE_SET_F32(false),
    TILE_SET_H(1, half_t, half_t, true),
    TILE_SET_H(1, half_t, half_t, false),
    TILE_SET_H(2, fp8_t, fp8_t, true),
    TILE_SET_H(2, fp8_t, fp8_t, false),
    TILE_SET_H(3, half_t, fp8_t, true),
    TILE_SET_H(3, half_t, fp8_t, false),
    // b = 96 blocks, bs_last (appended: the indices above are referenced by the measured table)
    TILE_INST(1, half_t, half_t, half_t, half_t, true, 96, 128, 32, 1, 4),
    TILE_INST(1, half_t, half_t, half_t, half_t, true, 96, 256, 32, 1, 4),
    TILE_INST(2, half_t, fp8_t, fp8_t, half_t, true, 96, 128, 32, 1, 4),
    TILE_INST(2, half_t, fp8_t, fp8_t, half_t, true, 96, 256, 32, 1, 4),
    // any b (partial last TM-tile, unaligned weight rows), both layouts
    TILE_INST_R(0, float, float, float, float, true, 64, 256, 16, 1, 4, true),
    TILE_INST_R(0, float, float, float, float, true, 128, 256, 16, 2, 2, true),
    TILE_INST_R(0, float, float, float, float, false, 64, 256, 16, 1, 4, true),
    TILE_INST_R(0, float, float, float, float, false, 128, 256, 16, 2, 2, true),
    TILE_INST_R(1, half_t, half_t, half_t, half_t, true, 64, 256, 64, 1, 4, true),
    TILE_INST_R(1, half_t, half_t, half_t, half_t, true, 128, 256, 32, 2, 2, true),
    TILE_INST_R(1, half_t, half_t, half_t, half_t, false, 64, 256, 64, 1, 4, true),
    TILE_INST_R(1, half_t, half_t, half_t, half_t, false, 128, 256, 32, 2, 2, true),
    TILE_INST_R(2, half_t, fp8_t, fp8_t, half_t, true, 64, 256, 64, 1, 4, true),
    TILE_INST_R(2, half_t, fp8_t, fp8_t, half_t, true, 128, 256, 32, 2, 2, true),
    TILE_INST_R(2, half_t, fp8_t, fp8_t, half_t, false, 64, 256, 64, 1, 4, true),
    TILE_INST_R(2, half_t, fp8_t, fp8_t, half_t, false, 128, 256, 32, 2, 2, true),
    // the 16-bit ones on 8 waves (the planes of the instances above leave one workgroup of 4 waves per CU)
    TILE_INST_R(1, half_t, half_t, half_t, half_t, true, 128, 256, 32, 2, 4, true),
    TILE_INST_R(1, half_t, half_t, half_t, half_t, true, 64, 256, 64, 2, 4, true),
    TILE_INST_R(1, half_t, half_t, half_t, half_t, false, 128, 256, 32, 2, 4, true),
    TILE_INST_R(1, half_t, half_t, half_t, half_t, false, 64, 256, 64, 2, 4, true),
    TILE_INST_R(2, half_t, fp8_t, fp8_t, half_t, true, 128, 256, 32, 2, 4, true),
    TILE_INST_R(2, half_t, fp8_t, fp8_t, half_t, true, 64, 256, 64, 2, 4, true),
    TILE_INST_R(2, half_t, fp8_t, fp8_t, half_t, false, 128, 256, 32, 2, 4, true),
    TILE_INST_R(2, half_t, fp8_t, fp8_t, half_t, false, 64, 256, 64, 2, 4, true),
    TILE_INST_R(0, float, float, float, float, true, 128, 256, 16, 2, 4, true),
    TILE_INST_R(0, float, float, float, float, true, 64, 256, 16, 2, 4, true),
    TILE_INST_R(0, float, float, float, float, false, 128, 256, 16, 2, 4, true),
    TILE_INST_R(0, float, float, float, float, false, 64, 256, 16, 2, 4, true),
    // aligned b on 8 waves
    TILE_INST(1, half_t, half_t, half_t, half_t, true, 128, 256, 32, 2, 4),
    TILE_INST(1, half_t, half_t, half_t, half_t, false, 128, 256, 32, 2, 4),
    TILE_INST(2, half_t, fp8_t, fp8_t, half_t, true, 128, 256, 32, 2, 4),
    TILE_INST(2, half_t, fp8_t, fp8_t, half_t, false, 128, 256, 32, 2, 4),
    TILE_INST(0, float, float, float, float, true, 128, 256, 16, 2, 4),
    TILE_INST(0, float, float, float, float, false, 128, 256, 16, 2, 4),
};
constexpr int N_TILE_INSTS = sizeof(tile_insts) / sizeof(TileInst);

bool tile_fits(const TileInst &t, const Problem &p, int combo)
{
    if (t.combo != combo || t.bs_last != p.bs_last) return false;
    if (!p.bs_last && p.c % t.tk) return false;  // batch-size-last tiles zero-fill the K tail
    const int x_epv = 16 / (int)dtype_size(p.x_dtype), w_epv = 16 / (int)dtype_size(p.w_dtype);
    // 16-byte global vectors: weight rows (b elements) and input rows must keep alignment
    if (t.ragged_b) {
        if (p.b % t.tm == 0 && p.b % w_epv == 0) return false;  // the aligned instances are faster
        // blocks of a few elements fill a sliver of a 32 x 32 MFMA tile: the vector form of the
        // generic kernel is faster there (measured: (1,16,32,896) fp16 1.55 ms against 2.35 ms)
        if ((int64_t)p.b * p.c <= 1024) return false;
    } else if (p.b % t.tm || p.b % w_epv) {
        return false;
    }
    if (p.bs_last) {
        if (p.batch % x_epv || p.batch < x_epv) return false;
    } else {
        if (p.d != 1) return false;  // batch-size-first with d > 1 is not handled by this family
        if (((int64_t)p.a * p.c) % x_epv || p.c % x_epv) return false;
    }
    return true;
}

}  // namespace

int ktile_inst_count() { return N_TILE_INSTS; }

uint32_t ktile_inst_id(int i)
{
    if (i < 0 || i >= N_TILE_INSTS) return 0;
    const TileInst &t = tile_insts[i];
    const int v[8] = {t.combo, t.bs_last, t.tm, t.tn, t.tk, t.threads, t.ragged_b, t.wm};
    return inst_hash('K', v, 8);
}

int ws_inst_count() { return N_WS_INSTS; }

uint32_t ws_inst_id(int i)
{
    if (i < 0 || i >= N_WS_INSTS) return 0;
    const WsInst &t = ws_insts[i];
    const int v[7] = {t.combo, t.bs_last, t.bb, t.cc, t.tn, t.threads, t.wm};
    return inst_hash('V', v, 7);
}

int tile_run(const Problem &p, int variant, bool launch, ksmm_tile *tile)
{
    const int combo = combo_of(p.x_dtype, p.w_dtype, p.y_dtype);
    if (combo < 0) return KSMM_ERR_BAD_DTYPE;
    // variant layout: bits 24-27 sub-family (0 k-loop tiles, 1 weight-stationary, 2 stream,
    // 3 batch-size-first with d > 1, 4 direct-to-LDS GEMM), bits 0-7 instance (0xff: first that fits), bits 8-23 a
    // sub-family parameter (persistent workgroups per block); -1: everything automatic
    if (variant >= 0) {
        const int sub = (variant >> 24) & 15, inst = variant & 0xff, par = (variant >> 8) & 0xffff;
        if (sub == 4) return gemm_run(p, inst == 0xff ? -1 : inst, launch, tile);
        if (sub == 3) return tile_bf_run(p, inst == 0xff ? -1 : inst, launch, tile);
        if (sub == 2) return stream_run(p, (inst == 0xff ? 0x7f : inst) | (par << 7), launch, tile);
        if (sub == 1) return ws_run(p, inst == 0xff ? -1 : inst, par, launch, tile);
        variant = inst == 0xff ? -2 : inst;  // -2: heuristic among the k-loop tiles only
    } else {
        int rc = gemm_run(p, -1, launch, tile);  // large blocks: matrix-core-bound
        if (rc != KSMM_ERR_BAD_ALGO) return rc;
        if (!p.bs_last && p.d == 2) {
            rc = gemm_run(p, -6, launch, tile);  // 4-wave persistent GEMM tile, two workgroups per CU
            if (rc != KSMM_ERR_BAD_ALGO) return rc;
        }
        if (!p.bs_last && p.d > 1) return tile_bf_run(p, -1, launch, tile);
        rc = stream_run(p, -1, launch, tile);
        if (rc != KSMM_ERR_BAD_ALGO) return rc;
        rc = ws_run(p, -1, 0, launch, tile);
        if (rc != KSMM_ERR_BAD_ALGO) return rc;
        rc = gemm_run(p, -4, launch, tile);  // GEMM tiles with TM = 64
        if (rc != KSMM_ERR_BAD_ALGO) return rc;
        rc = gemm_run(p, -5, launch, tile);  // persistent GEMM tiles with a masked last TM-tile
        if (rc != KSMM_ERR_BAD_ALGO) return rc;
    }
    int pick = -1;
    if (variant >= 0) {
        if (variant < N_TILE_INSTS && tile_fits(tile_insts[variant], p, combo)) pick = variant;
    } else {  // -1 or -2
        // heuristic: the largest TM that divides b (fewest re-reads of the input), then a batch
        // tile that still leaves >= 2 workgroups per CU
        int64_t best_score = -1;
        for (int i = 0; i < N_TILE_INSTS; ++i) {
            const TileInst &t = tile_insts[i];
            if (!tile_fits(t, p, combo)) continue;
            const int64_t wgs = (int64_t)p.a * p.d * ((p.b + t.tm - 1) / t.tm) * ((p.batch + t.tn - 1) / t.tn);
            // (any b: between equal tiles the instance on 8 waves: with 4, the planes of the large tiles leave
            // one wave per SIMD; (16,1855,256,1) fp16 1343 -> 821 us, (64,455,64,1) 933 -> 533)
            // (the aligned 8-wave instances are named by the measured table only)
            int64_t score = (int64_t)t.tm * 1000 + t.tn + (t.ragged_b ? t.threads / 256 : 0);
            if (wgs < 512) score -= 100000;
            if (score > best_score) {
                best_score = score;
                pick = i;
            }
        }
    }
    // nothing else takes it: a GEMM tile that does not fill the chip still beats the generic kernel
    if (pick < 0) return variant == -1 ? gemm_run(p, -2, launch, tile) : KSMM_ERR_BAD_ALGO;
    const TileInst &t = tile_insts[pick];
    const int m_tiles = (p.b + t.tm - 1) / t.tm;
    const int64_t n_tiles = (p.batch + t.tn - 1) / t.tn;
    const int64_t blocks = (int64_t)p.a * p.d * m_tiles * n_tiles;
    const int64_t grid = (blocks + 7) / 8 * 8;
    if (grid > 0x7fffffffLL) return KSMM_ERR_TOO_LARGE;
    if (tile) {
        tile->algo = KSMM_ALGO_TILE;
        tile->variant = pick;
        tile->tile_m = t.tm;
        tile->tile_n = t.tn;
        tile->tile_k = t.tk;
        tile->tile_d = 1;
        tile->threads = t.threads;
        tile->lds_bytes = t.lds;
        tile->grid = grid;
    }
    if (!launch) return KSMM_OK;
    if (t.lds > 64 * 1024 && ensure_dynamic_lds(t.fn, t.lds) != KSMM_OK) return KSMM_ERR_LAUNCH;
    int batch_i = (int)p.batch, n_tiles_i = (int)n_tiles, blocks_i = (int)blocks, m_tiles_i = m_tiles;
    Epi ep = epi_of(p);
    void *args[] = {(void *)&p.x, (void *)&p.w, (void *)&p.y, &batch_i, (void *)&p.a, (void *)&p.b,
                    (void *)&p.c, (void *)&p.d, &ep, &m_tiles_i, &n_tiles_i, &blocks_i};
    hipError_t e = hipLaunchKernel(t.fn, dim3((unsigned)grid), dim3(t.threads), args, t.lds, p.stream);
    return e == hipSuccess ? KSMM_OK : KSMM_ERR_LAUNCH;
}

}  // namespace ksmm
