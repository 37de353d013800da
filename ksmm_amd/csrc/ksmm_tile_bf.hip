// Tile kernel for the batch-size-first layout with d > 1.
//
// Batch-size-first rows hold the features as (a_i, c_i, d_i) with d_i fastest, so for d > 1
// the c inputs of one (a_i, d_i) block are strided by d.  A workgroup therefore takes DD
// neighbouring blocks d_i = dg*DD .. dg*DD + DD-1 of one a_i at once (all of them when d = DD):
// it reads x[n][(a_i*c + k)*d + dg*DD ..] with 16-byte loads (one contiguous run per row when
// d = DD; one vector of DD elements per (row, k) when d > DD, which needs DD elements to fill
// the vector), splits the vectors by d_i while writing them to LDS (one k-contiguous plane
// per d_i), runs DD independent TM x TN x TK MFMA products against the DD weight blocks, and
// interleaves the DD results again in registers, so that a lane stores DD consecutive output
// features (16 bytes when d > DD).  Workgroups that read the same rows (the TM-tiles and the
// d-groups of one batch tile) get neighbouring ids on one XCD and share them through its L2.
//
// MFMA roles as in the batch-size-first case of the plain tile kernel: A = X (rows = batch),
// B = W (lanes = outputs), fp32 accumulation, 32x32 tiles.
//
// Reference counterpart: kernel_bs_first_float / kernel_bs_first_half2
// (src/ksmm_py/layer/kronecker_sparse/template_kernels_float.cuh:85-286,
//  template_kernels_half.cuh:103-299), which gather the strided inputs with scalar loads.
#include "ksmm_mfma.h"
#include <type_traits>

namespace ksmm {

namespace {

template <typename CT, int N> struct alignas(N * sizeof(CT)) pack_t {
    CT e[N];
};

// TX: the input's type in memory when it is not the compute type (e4m3fn, decoded to fp16 while the
// vectors are split into the planes)
template <typename CT, typename TW, int DD, int TM, int TN, int TK, int WM, int WN, typename TX = CT> struct BfCfg {
    static constexpr int THREADS = 64 * WM * WN;
    static constexpr int KSTEP = compute<CT>::KSTEP;
    static constexpr int MT = TM / WM / 32, NT = TN / WN / 32;
    static constexpr int EPV = 16 / (int)sizeof(TX);  // elements per 16-byte input vector
    static constexpr int KPV = EPV / DD;              // consecutive k per input vector
    static constexpr int LDW = pads<CT>::outer(TM);
    static constexpr int LDK = pads<CT>::inner(TK);
    static constexpr int W_ELEMS = DD * TK * LDW, X_ELEMS = DD * TN * LDK;
    static constexpr int LDS_BYTES = 2 * (W_ELEMS + X_ELEMS) * (int)sizeof(CT);
    static constexpr int W_EPV = stage<TW, CT>::EPV;
    static constexpr int W_VECS = DD * TK * TM / W_EPV, X_VECS = TN * TK * DD / EPV;
    static constexpr int W_PER_T = (W_VECS + THREADS - 1) / THREADS, X_PER_T = (X_VECS + THREADS - 1) / THREADS;
    static_assert(EPV % DD == 0 && KPV >= 1, "d must divide the 16-byte vector");
    static_assert(TM % (32 * WM) == 0 && TN % (32 * WN) == 0 && TK % KSTEP == 0, "wave tiling");
    static_assert(TM % W_EPV == 0 && TK % KPV == 0, "vector width");
    static_assert(LDS_BYTES <= 160 * 1024, "LDS");
};

__device__ __forceinline__ half_t bf_decode(half_t v) { return v; }
__device__ __forceinline__ float bf_decode(float v) { return v; }
__device__ __forceinline__ half_t bf_decode(fp8_t v) { return fp8_to_half(v.bits); }

template <typename CT, typename TW, typename TY, int DD, int TM, int TN, int TK, int WM, int WN, typename TX = CT>
__global__ __launch_bounds__(64 * WM * WN) void ks_tile_bf_kernel(const TX *__restrict__ x,
                                                                 const TW *__restrict__ w,
                                                                 TY *__restrict__ y, int batch, int a,
                                                                 int b, int c, int d, Epi ep,
                                                                 int m_tiles, int n_tiles, int blocks)
{
    typedef BfCfg<CT, TW, DD, TM, TN, TK, WM, WN, TX> C;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    CT *const lds = (CT *)smem;
    auto ws = [&](int buf, int dd) { return lds + buf * C::W_ELEMS + dd * TK * C::LDW; };
    auto xs = [&](int buf, int dd) { return lds + 2 * C::W_ELEMS + buf * C::X_ELEMS + dd * TN * C::LDK; };

    // workgroups that share an input tile (the TM-tiles of one batch tile) get consecutive
    // logical ids on one XCD
    const int per_xcd = (blocks + 7) / 8;
    const int lid = (blockIdx.x % 8) * per_xcd + blockIdx.x / 8;
    if (lid >= blocks) return;
    const int n_dg = d / DD;  // groups of DD blocks
    const int mt_id = lid % m_tiles;
    int rest = lid / m_tiles;
    const int dg = rest % n_dg;
    rest /= n_dg;
    const int nt_id = rest % n_tiles;
    const int a_i = rest / n_tiles;
    const int m0 = mt_id * TM, n0 = nt_id * TN;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave / WN, wn = wave % WN;
    const size_t in_size = (size_t)a * c * d, out_size = (size_t)a * b * d;
    const TX *xg = x + (size_t)a_i * c * d + dg * DD;  // + n * in_size + k * d + dd

    stage<TW, CT> wreg[C::W_PER_T];
    uint4_t xreg[C::X_PER_T];
    auto gload = [&](int k0) {
#pragma unroll
        for (int i = 0; i < C::W_PER_T; ++i) {
            const int v = tid + i * C::THREADS;
            if (C::W_VECS % C::THREADS == 0 || v < C::W_VECS) {
                const int per_dd = TK * TM / C::W_EPV;
                const int dd = v / per_dd, r = v % per_dd;
                const int kk = r / (TM / C::W_EPV), mm = (r % (TM / C::W_EPV)) * C::W_EPV;
                wreg[i].load(w + ((size_t)(a_i * d + dg * DD + dd) * c + k0 + kk) * b + m0 + mm);
            }
        }
#pragma unroll
        for (int i = 0; i < C::X_PER_T; ++i) {
            const int v = tid + i * C::THREADS;
            if (C::X_VECS % C::THREADS == 0 || v < C::X_VECS) {
                const int vpr = TK * DD / C::EPV;  // vectors per row
                const int nn = v / vpr, kk = (v % vpr) * C::KPV;
                const int row = min(n0 + nn, batch - 1);
                // KPV consecutive k share a vector only when d == DD (the host checks)
                xreg[i] = *(const uint4_t *)(xg + (size_t)row * in_size + (size_t)(k0 + kk) * d);
            }
        }
    };
    auto lstore = [&](int buf) {
#pragma unroll
        for (int i = 0; i < C::W_PER_T; ++i) {
            const int v = tid + i * C::THREADS;
            if (C::W_VECS % C::THREADS == 0 || v < C::W_VECS) {
                const int per_dd = TK * TM / C::W_EPV;
                const int dd = v / per_dd, r = v % per_dd;
                const int kk = r / (TM / C::W_EPV), mm = (r % (TM / C::W_EPV)) * C::W_EPV;
                wreg[i].store(ws(buf, dd) + kk * C::LDW + mm);
            }
        }
#pragma unroll
        for (int i = 0; i < C::X_PER_T; ++i) {
            const int v = tid + i * C::THREADS;
            if (C::X_VECS % C::THREADS == 0 || v < C::X_VECS) {
                const int vpr = TK * DD / C::EPV;
                const int nn = v / vpr, kk = (v % vpr) * C::KPV;
                // split the vector by d_i: element e is (k = kk + e / DD, d_i = e % DD)
                pack_t<TX, C::EPV> all = __builtin_bit_cast(pack_t<TX, C::EPV>, xreg[i]);
#pragma unroll
                for (int dd = 0; dd < DD; ++dd) {
                    pack_t<CT, C::KPV> part;
#pragma unroll
                    for (int q = 0; q < C::KPV; ++q) part.e[q] = bf_decode(all.e[q * DD + dd]);
                    *(pack_t<CT, C::KPV> *)(xs(buf, dd) + nn * C::LDK + kk) = part;
                }
            }
        }
    };

    float16_t acc[DD][C::MT][C::NT];
#pragma unroll
    for (int dd = 0; dd < DD; ++dd)
#pragma unroll
        for (int i = 0; i < C::MT; ++i)
#pragma unroll
            for (int j = 0; j < C::NT; ++j)
#pragma unroll
                for (int e = 0; e < 16; ++e) acc[dd][i][j][e] = 0.f;

    const int steps = c / TK;
    gload(0);
    lstore(0);
    __syncthreads();
    for (int s = 0; s < steps; ++s) {
        const int buf = s & 1;
        if (s + 1 < steps) gload((s + 1) * TK);
#pragma unroll
        for (int dd = 0; dd < DD; ++dd) {
            const CT *wb = ws(buf, dd), *xb = xs(buf, dd);
#pragma unroll
            for (int k0 = 0; k0 < TK; k0 += C::KSTEP) {
                typename frag<CT>::type fw[C::MT], fx[C::NT];
#pragma unroll
                for (int i = 0; i < C::MT; ++i)
                    fw[i] = frag<CT>::k_outer(wb, C::LDW, (wm * C::MT + i) * 32, k0, lane);
#pragma unroll
                for (int j = 0; j < C::NT; ++j)
                    fx[j] = frag<CT>::k_inner(xb, C::LDK, (wn * C::NT + j) * 32, k0, lane);
#pragma unroll
                for (int i = 0; i < C::MT; ++i)
#pragma unroll
                    for (int j = 0; j < C::NT; ++j)
                        acc[dd][i][j] = frag<CT>::mfma(fx[j], fw[i], acc[dd][i][j]);
            }
        }
        if (s + 1 < steps) lstore(buf ^ 1);
        __syncthreads();
    }

    // D tile: lane holds output column m = lane % 32, batch rows 8*(e/4) + 4*(lane/32) + e%4;
    // the DD results of one (n, m) are adjacent in y
    const int l32 = lane & 31, lq = lane >> 5;
#pragma unroll
    for (int i = 0; i < C::MT; ++i)
#pragma unroll
        for (int j = 0; j < C::NT; ++j) {
            const int m = m0 + (wm * C::MT + i) * 32 + l32;
            const int nb = n0 + (wn * C::NT + j) * 32;
            float bv[DD];  // bias of the lane's DD adjacent outputs
#pragma unroll
            for (int dd = 0; dd < DD; ++dd) bv[dd] = epi_bias<TY>(ep, ((size_t)a_i * b + m) * d + dg * DD + dd);
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const int n = nb + 8 * (e >> 2) + 4 * lq + (e & 3);
                pack_t<TY, DD> o;
#pragma unroll
                for (int dd = 0; dd < DD; ++dd) o.e[dd] = (TY)epi_finish(ep, acc[dd][i][j][e], bv[dd]);
                if (n < batch)
                    *(pack_t<TY, DD> *)(y + (size_t)n * out_size + ((size_t)a_i * b + m) * d + dg * DD) = o;
            }
        }
}

// ------------------------------------------------------------------------------------------
// Groups of 8 fp16 blocks with a register pipeline several slabs deep (TK = 16, one MFMA step
// per slab and block).  The plain kernel above keeps one slab in flight while it multiplies the
// previous one, and its padded planes leave room for one workgroup per CU: with 8 blocks per
// group a slab is 32 KB (half of it weights, which every batch tile reads again through L2),
// so it waits out a memory latency per slab.  Here
//  * a thread's loads of input slab s + PDX and weight slab s + PDW are issued before slab s is
//    multiplied (16 registers per slab and operand);
//  * eight neighbouring lanes read the 128 bytes (8 k x 8 d_i) a row holds per line, so a load
//    instruction touches 8 whole lines when d = 8; a thread gets k and k + 8 of its row, turns
//    the two vectors into 8 x (2 k of one d_i) with 8 byte permutes and writes them with
//    4-byte LDS stores.  Inside a slab k therefore sits at position 2 * (k % 8) + k / 8, in the
//    planes and in the weight rows alike (the order of a sum does not matter to the product);
//  * the planes are unpadded rows of 16 k, their two 16-byte halves swapped for rows 8..15 of
//    every 16 (the 16 rows a 16-byte operand read covers then fall on distinct banks);
// which brings LDS to 72 KB: two workgroups per CU, four slabs of 32 KB in flight.
// NG > 1: the workgroup takes NG neighbouring groups of 8 blocks with NG times the waves (each set
// of WM x WN waves multiplies one group), in slabs of TK = 8 (planes of 64 or 32 blocks at 16 k
// would not leave room for two LDS buffers; one 4-k MFMA step per slab and block).  With groups
// of 8 out of d = 64 a line of x is asked for by 8 workgroups for 16 bytes each, and a line of
// results is written in 8 pieces at 8 different times: that scatter, not the bytes, is what the
// groups of 8 wait for (fp16 (6,192,192,64) at batch 25088: 5.3 ms, and 2.5 ms when the same
// kernel reads and writes the same number of bytes as whole lines).  Here
//  * neighbouring lanes read the vectors of neighbouring groups: runs of 16 * NG bytes per
//    (row, k), whole runs of 8 k when the workgroup covers d;
//  * the results leave through LDS ([n][m][group], 16-byte pieces, the group xor-ed with bits of m so
//    that neighbouring lanes fall on distinct banks): runs of 16 * NG bytes per (row, m), or of
//    TM * d * 2 bytes when the workgroup covers d;
//  * the planes of a group start 256 / NG bytes apart in the banks (the lanes of one 4-byte
//    store differ in the group first).
// The accumulators of a workgroup are 8 * NG * TM * TN floats in 128 registers of 512 lanes, so
// the tile shrinks as NG grows and weights and rows are read again more often: 32 blocks
// (64-byte runs) on a 64 x 32 tile are the best trade (3.85 ms on the pattern above; 64 blocks
// on 32 x 32: 4.6 ms; 16 blocks on 64 x 64: 4.4 ms).
template <typename TX, typename TW, int TM, int TN, int WM, int WN, int PDX, int PDW, int NG = 1, int TK = 16>
__global__ __launch_bounds__(64 * WM * WN * NG, (WM * WN * NG >= 8 ? 1 : 2)) void ks_tile_bf8_kernel(const TX *__restrict__ x,
                                                                const TW *__restrict__ w,
                                                                half_t *__restrict__ y, int batch, int a,
                                                                int b, int c, int d, Epi ep,
                                                                int m_tiles, int n_tiles, int blocks)
{
    constexpr int DD = 8, DDA = DD * NG, KH = TK / 2, THREADS = 64 * WM * WN * NG;
    constexpr bool FL = NG > 1;  // whole lines: results leave through LDS
    constexpr int NBUF = 2;
    static_assert(TK == 16 || TK == 8, "one MFMA step per slab");
    constexpr int MT = TM / WM / 32, NT = TN / WN / 32;
    constexpr int LDW = TM == 32 ? 32 : pads<half_t>::outer(TM);  // (rows of 64 bytes: 4 k are 256 bytes, no padding needed)
    // (the chunks of a group start 256 / NG bytes apart in the banks: the lanes of one 4-byte store
    // differ in the chunk first)
    constexpr int XPAD = NG > 1 ? 128 / NG : 0;
    constexpr int W_ELEMS = DDA * TK * LDW, X_ELEMS = DDA * TN * TK + NG * XPAD;
    constexpr int W_EPV = stage<TW, half_t>::EPV;
    constexpr int W_VECS = DDA * TK * TM / W_EPV, W_PER_T = W_VECS / THREADS;
    constexpr int X_QUADS = NG * TN * TK / 2, XQ_PER_T = X_QUADS / THREADS;  // pairs (k, k + KH) of a row and chunk
    static_assert(W_VECS % THREADS == 0 && X_QUADS % THREADS == 0, "whole loads per thread");
    static_assert(TM % (32 * WM) == 0 && TN % (32 * WN) == 0, "wave tiling");
    static_assert(NBUF * (W_ELEMS + X_ELEMS) * 2 <= (WM * WN * NG >= 8 ? 160 : 80) * 1024, "8 waves per CU");
    static_assert((NG & (NG - 1)) == 0 && NG <= 8 && (!FL || TM * TN * DDA * 2 <= 160 * 1024), "chunks of a group");
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    half_t *const lds = (half_t *)smem;
    auto ws = [&](int buf, int dd) { return lds + buf * W_ELEMS + dd * TK * LDW; };
    auto xs = [&](int buf, int dd) { return lds + NBUF * W_ELEMS + buf * X_ELEMS + dd * TN * TK + (dd >> 3) * XPAD; };

    const int per_xcd = (blocks + 7) / 8;
    const int lid = (blockIdx.x % 8) * per_xcd + blockIdx.x / 8;
    if (lid >= blocks) return;
    const int n_dg = d / DDA;  // groups of DDA blocks
    const int mt_id = lid % m_tiles;
    int rest = lid / m_tiles;
    const int dg = rest % n_dg;
    rest /= n_dg;
    const int nt_id = rest % n_tiles;
    const int a_i = rest / n_tiles;
    const int m0 = mt_id * TM, n0 = nt_id * TN;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wg = wave / (WM * WN), wm = wave / WN % WM, wn = wave % WN;  // wg: the wave's chunk of 8 blocks
    const size_t in_size = (size_t)a * c * d, out_size = (size_t)a * b * d;

    stage<TW, half_t> wreg[PDW][W_PER_T];
    // one (row, k) of the group: 8 halves = 16 bytes, or 8 e4m3 bytes (decoded when they go to LDS)
    typedef typename std::conditional<sizeof(TX) == 2, uint4_t, uint2_t>::type xvec_t;
    xvec_t xreg[PDX][XQ_PER_T][2];
    // The loads of a slab are issued unconditionally: a branch around them would leave the
    // compiler two histories of the load counter to merge, and it would then wait for every
    // load in flight before it touches a register of the pipeline.  Behind the last slab
    // (live == false) every lane reads the first 16 bytes of the tile instead (one line): the
    // offsets are masked, not selected, so that no branch comes back.  Addresses are a uniform
    // base per tile plus a 32-bit offset per lane (the host checks that they fit).
    const TW *const wt = w + ((size_t)(a_i * d + dg * DDA) * c) * b + m0;
    const TX *const xt = x + (size_t)n0 * in_size + (size_t)a_i * c * d + dg * DDA;
    uint32_t woff[W_PER_T], xoff[XQ_PER_T];
#pragma unroll
    for (int i = 0; i < W_PER_T; ++i) {
        const int v = tid + i * THREADS;
        constexpr int per_dd = TK * TM / W_EPV;
        const int dd = v / per_dd, r = v % per_dd;
        const int kk = r / (TM / W_EPV), mm = (r % (TM / W_EPV)) * W_EPV;
        woff[i] = (uint32_t)((dd * c + kk) * b + mm);
    }
#pragma unroll
    for (int i = 0; i < XQ_PER_T; ++i) {
        const int v = tid + i * THREADS;
        // the chunk runs fastest: neighbouring lanes read neighbouring vectors of one line
        const int g = v % NG, k8 = v / NG % KH, nn = v / (KH * NG);
        xoff[i] = (uint32_t)(min(nn, batch - 1 - n0) * (uint32_t)in_size + k8 * d + g * DD);
    }
    auto live_mask = [](bool live) {
        int lv = live;
        asm volatile("" : "+v"(lv));  // opaque: stays a mask
        return 0u - (uint32_t)lv;
    };
    auto gload_w = [&](int slot, int k0, bool live) {
        const uint32_t mk = live_mask(live);
#pragma unroll
        for (int i = 0; i < W_PER_T; ++i) wreg[slot][i].load(wt + ((woff[i] + (uint32_t)(k0 * b)) & mk));
    };
    auto gload_x = [&](int slot, int k0, bool live) {
        const uint32_t mk = live_mask(live);
#pragma unroll
        for (int i = 0; i < XQ_PER_T; ++i)
#pragma unroll
            for (int j = 0; j < 2; ++j)
                // (32 fp16 blocks per workgroup: few workgroups share a line of x, and read without the
                // temporal hint it leaves more of L2 to the weights: (8,128,128,64) 2546 -> 2396 us,
                // (1,192,192,128) 1394 -> 1273; 1-6 % slower with 16 blocks, e4m3 input and in fp32)
                if constexpr (NG == 4 && sizeof(TX) == 2)
                    xreg[slot][i][j] = __builtin_nontemporal_load((const xvec_t *)(xt + ((xoff[i] + (uint32_t)((k0 + KH * j) * d)) & mk)));
                else
                    xreg[slot][i][j] = *(const xvec_t *)(xt + ((xoff[i] + (uint32_t)((k0 + KH * j) * d)) & mk));
    };
    auto lstore = [&](int wslot, int slot, int buf) {
#pragma unroll
        for (int i = 0; i < W_PER_T; ++i) {
            const int v = tid + i * THREADS;
            constexpr int per_dd = TK * TM / W_EPV;
            const int dd = v / per_dd, r = v % per_dd;
            const int kk = r / (TM / W_EPV), mm = (r % (TM / W_EPV)) * W_EPV;
            wreg[wslot][i].store(ws(buf, dd) + (2 * (kk % KH) + kk / KH) * LDW + mm);
        }
#pragma unroll
        for (int i = 0; i < XQ_PER_T; ++i) {
            const int v = tid + i * THREADS;
            const int g = v % NG, k8 = v / NG % KH, nn = v / (KH * NG);
            // k = k8 and k8 + 8 of row nn: positions 2 * k8 and 2 * k8 + 1, i.e. 4-byte piece k8 & 3
            // of the 16-byte half k8 >> 2 (swapped for rows 8..15 of every 16)
            // (TK = 8: k = k8 and k8 + 4 at positions 2 * k8 and 2 * k8 + 1 of a 16-byte row, its two
            // 8-byte halves swapped for rows 16..31 of every 32: the 32 rows an 8-byte operand read
            // covers then fall on distinct banks)
            half_t *const dst = xs(buf, g * DD) + nn * TK +
                                (TK == 16 ? ((((k8 >> 2) ^ ((nn >> 3) & 1)) << 3) | ((k8 & 3) << 1))
                                          : ((k8 ^ (2 * ((nn >> 4) & 1))) << 1));
            uint4_t c0, c1;  // register p: d_i = 2p (low half) and 2p + 1 (high half), as fp16
            if constexpr (sizeof(TX) == 2) {
                c0 = xreg[slot][i][0];
                c1 = xreg[slot][i][1];
            } else {
#pragma unroll
                for (int w2 = 0; w2 < 2; ++w2) {
                    c0[2 * w2] = __builtin_bit_cast(uint32_t, fp8x2_to_half2(xreg[slot][i][0][w2]));
                    c0[2 * w2 + 1] = __builtin_bit_cast(uint32_t, fp8x2_hi_to_half2(xreg[slot][i][0][w2]));
                    c1[2 * w2] = __builtin_bit_cast(uint32_t, fp8x2_to_half2(xreg[slot][i][1][w2]));
                    c1[2 * w2 + 1] = __builtin_bit_cast(uint32_t, fp8x2_hi_to_half2(xreg[slot][i][1][w2]));
                }
            }
#pragma unroll
            for (int p = 0; p < 4; ++p) {
                // register p of a vector holds d_i = 2p (low half) and 2p + 1 (high half)
                *(uint32_t *)(dst + (2 * p) * TN * TK) = __builtin_amdgcn_perm(c1[p], c0[p], 0x05040100u);
                *(uint32_t *)(dst + (2 * p + 1) * TN * TK) = __builtin_amdgcn_perm(c1[p], c0[p], 0x07060302u);
            }
        }
    };

    float16_t acc[DD][MT][NT];
#pragma unroll
    for (int dd = 0; dd < DD; ++dd)
#pragma unroll
        for (int i = 0; i < MT; ++i)
#pragma unroll
            for (int j = 0; j < NT; ++j)
#pragma unroll
                for (int e = 0; e < 16; ++e) acc[dd][i][j][e] = 0.f;

    const int l32 = lane & 31, lq = lane >> 5;
    int xrow[NT];  // the lane's operand inside a plane, in elements
#pragma unroll
    for (int j = 0; j < NT; ++j) {
        const int n = (wn * NT + j) * 32 + l32;
        xrow[j] = TK == 16 ? n * TK + ((lq ^ ((n >> 3) & 1)) << 3) : n * TK + 4 * (lq ^ ((n >> 4) & 1));
    }
    auto multiply = [&](int buf) {
#pragma unroll
        for (int dd = 0; dd < DD; ++dd) {
            const half_t *wb = ws(buf, wg * DD + dd), *xb = xs(buf, wg * DD + dd);
            if constexpr (TK == 16) {
                half8_t fw[MT], fx[NT];
#pragma unroll
                for (int i = 0; i < MT; ++i) fw[i] = frag<half_t>::k_outer(wb, LDW, (wm * MT + i) * 32, 0, lane);
#pragma unroll
                for (int j = 0; j < NT; ++j) fx[j] = *(const half8_t *)(xb + xrow[j]);
#pragma unroll
                for (int i = 0; i < MT; ++i)
#pragma unroll
                    for (int j = 0; j < NT; ++j) acc[dd][i][j] = frag<half_t>::mfma(fx[j], fw[i], acc[dd][i][j]);
            } else {
                // 8 k per slab: the lane's operand is 4 k (one transpose load, one 8-byte read)
                half4_t fw[MT], fx[NT];
#pragma unroll
                for (int i = 0; i < MT; ++i) fw[i] = frag<half_t>::k_outer4(wb, LDW, (wm * MT + i) * 32, 0, lane);
#pragma unroll
                for (int j = 0; j < NT; ++j) fx[j] = *(const half4_t *)(xb + xrow[j]);
#pragma unroll
                for (int i = 0; i < MT; ++i)
#pragma unroll
                    for (int j = 0; j < NT; ++j)
                        acc[dd][i][j] = __builtin_amdgcn_mfma_f32_32x32x8f16(fx[j], fw[i], acc[dd][i][j], 0, 0, 0);
            }
        }
    };

    const int steps = c / TK;
    // slab s: request weights PDW and input PDX slabs ahead into the slots slab s came from (it
    // went to LDS an iteration ago), multiply slab s, move slab s + 1 from its registers to
    // the other LDS buffer.  The weights come from L2 and get the shorter lead; they are
    // requested first, so that waiting for them leaves the younger input loads in flight.
    constexpr int PERIOD = PDX * PDW / (PDX % PDW == 0 ? PDW : PDW % PDX == 0 ? PDX : 1);
    static_assert(PERIOD % PDX == 0 && PERIOD % PDW == 0, "slots repeat after PERIOD slabs");
    auto slab = [&](int u, int s) {
        gload_w(u % PDW, (s + PDW) * TK, s + PDW < steps);
        gload_x(u % PDX, (s + PDX) * TK, s + PDX < steps);
        // (the permutes of the next slab's vectors must not move up here: they would wait for
        // that slab before this one is multiplied)
        __builtin_amdgcn_sched_barrier(0);
        multiply(s & 1);
        __builtin_amdgcn_sched_barrier(0);
        lstore((u + 1) % PDW, (u + 1) % PDX, (s & 1) ^ 1);  // behind the last slab: whatever the idle loads brought
        __syncthreads();
    };
#pragma unroll
    for (int u = 0; u < (PDX > PDW ? PDX : PDW); ++u) {
        if (u < PDW) gload_w(u, u * TK, u < steps);
        if (u < PDX) gload_x(u, u * TK, u < steps);
    }
    lstore(0, 0, 0);
    __syncthreads();
    int s = 0;
    for (; s + PERIOD <= steps; s += PERIOD) {
#pragma unroll
        for (int u = 0; u < PERIOD; ++u) slab(u, s + u);
    }
#pragma unroll
    for (int u = 0; u < PERIOD - 1; ++u)
        if (s + u < steps) slab(u, s + u);

    // D tile: lane holds output column m = lane % 32, batch rows 8*(e/4) + 4*(lane/32) + e%4;
    // the 8 results of one (n, m) are adjacent in y: one 16-byte store
    if constexpr (FL) {
        // the NG chunks of one (n, m) sit in NG waves and are adjacent in y, as are the m of one
        // row when the group is all of d
        uint4_t *const ot = (uint4_t *)smem;
        // (rows of m are 16 * NG bytes apart: 16 / NG consecutive m cover the banks once, so the
        // group is xor-ed with m / (16 / NG))
        auto okey = [](int ml) { return (ml * NG >> 4) & (NG - 1); };
#pragma unroll
        for (int i = 0; i < MT; ++i)
#pragma unroll
            for (int j = 0; j < NT; ++j) {
                const int ml = (wm * MT + i) * 32 + l32;
                float bv[DD];
#pragma unroll
                for (int dd = 0; dd < DD; ++dd)
                    bv[dd] = epi_bias<half_t>(ep, ((size_t)a_i * b + m0 + ml) * d + dg * DDA + wg * DD + dd);
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    const int nl = (wn * NT + j) * 32 + 8 * (e >> 2) + 4 * lq + (e & 3);
                    pack_t<half_t, DD> o;
#pragma unroll
                    for (int dd = 0; dd < DD; ++dd) o.e[dd] = (half_t)epi_finish(ep, acc[dd][i][j][e], bv[dd]);
                    ot[(nl * TM + ml) * NG + (wg ^ okey(ml))] = __builtin_bit_cast(uint4_t, o);
                }
            }
        __syncthreads();
        constexpr int PIECES = TN * TM * NG;
        static_assert(PIECES % THREADS == 0, "whole pieces per thread");
#pragma unroll 4
        for (int q = tid; q < PIECES; q += THREADS) {
            const int ch = q % NG, ml = q / NG % TM, nl = q / (NG * TM);
            if (n0 + nl < batch)
                *(uint4_t *)(y + (size_t)(n0 + nl) * out_size + ((size_t)a_i * b + m0 + ml) * d + dg * DDA + ch * DD) =
                    ot[(nl * TM + ml) * NG + (ch ^ okey(ml))];
        }
        return;
    }
#pragma unroll
    for (int i = 0; i < MT; ++i)
#pragma unroll
        for (int j = 0; j < NT; ++j) {
            const int m = m0 + (wm * MT + i) * 32 + l32;
            const int nb = n0 + (wn * NT + j) * 32;
            float bv[DD];
#pragma unroll
            for (int dd = 0; dd < DD; ++dd) bv[dd] = epi_bias<half_t>(ep, ((size_t)a_i * b + m) * d + dg * DD + dd);
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const int n = nb + 8 * (e >> 2) + 4 * lq + (e & 3);
                pack_t<half_t, DD> o;
#pragma unroll
                for (int dd = 0; dd < DD; ++dd) o.e[dd] = (half_t)epi_finish(ep, acc[dd][i][j][e], bv[dd]);
                if (n < batch)
                    *(pack_t<half_t, DD> *)(y + (size_t)n * out_size + ((size_t)a_i * b + m) * d + dg * DD) = o;
            }
        }
}

// The same pipeline for groups of 4 fp32 blocks (a 16-byte vector is one k of 4 d_i, so the
// vectors are split by plain 4-byte LDS stores and k keeps its place).  One MFMA step is 2 k:
// 32 steps per slab and wave, so this form is matrix-core-bound where the fp16 one waits for
// memory; what it buys over the plain kernel is a second wave per SIMD (64 KB of LDS, 64
// accumulator registers), which hides the LDS latency in front of every MFMA.  Plane rows are
// 16 floats, element k of row n at k ^ 2 * ((n / 4) % 8): the 32 rows an operand read covers
// fall on distinct banks.  Weight rows are unpadded too: the columns of odd k are XORed with 32,
// so the two rows an operand read covers use different bank halves.
// NG > 1: NG neighbouring groups of 4 blocks per workgroup with NG times the waves, slabs of 8 k,
// results staged through LDS, as in the 16-bit kernel above (runs of 16 * NG bytes both ways).
template <int TM, int TN, int WM, int WN, int PDX, int PDW, int NG = 1, int TK = 16>
__global__ __launch_bounds__(64 * WM * WN * NG, (WM * WN * NG >= 8 ? 1 : 2)) void ks_tile_bf4_kernel(const float *__restrict__ x,
                                                                const float *__restrict__ w,
                                                                float *__restrict__ y, int batch, int a,
                                                                int b, int c, int d, Epi ep,
                                                                int m_tiles, int n_tiles, int blocks)
{
    typedef float TW;
    constexpr int DD = 4, DDA = DD * NG, KH = TK / 2, THREADS = 64 * WM * WN * NG;
    constexpr bool FL = NG > 1;  // several groups per workgroup: results leave through LDS
    constexpr int XPAD = NG > 1 ? 64 / NG : 0;  // the groups start 256 / NG bytes apart in the banks
    static_assert(TK == 16 || TK == 8, "slab depth");
    constexpr int MT = TM / WM / 32, NT = TN / WN / 32;
    constexpr int LDW = TM;  // unpadded: columns of odd rows are XORed with 32 instead
    constexpr int WSW = TM >= 64 ? 32 : 0;  // (rows of 32 floats: two rows are the two bank halves as they are)
    constexpr int W_ELEMS = DDA * TK * LDW, X_ELEMS = DDA * TN * TK + NG * XPAD;
    constexpr int W_EPV = stage<float, float>::EPV;
    constexpr int W_VECS = DDA * TK * TM / W_EPV, W_PER_T = W_VECS / THREADS;
    constexpr int X_QUADS = NG * TN * TK / 2, XQ_PER_T = X_QUADS / THREADS;  // pairs (k, k + KH) of a row and group
    static_assert(W_VECS % THREADS == 0 && X_QUADS % THREADS == 0, "whole loads per thread");
    static_assert(TM % (32 * WM) == 0 && TN % (32 * WN) == 0, "wave tiling");
    static_assert(2 * (W_ELEMS + X_ELEMS) * 4 <= (WM * WN * NG >= 8 ? 160 : 80) * 1024, "8 waves per CU");
    static_assert((NG & (NG - 1)) == 0 && NG <= 8 && (!FL || TM * TN * DDA * 4 <= 160 * 1024), "groups of a workgroup");
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    float *const lds = (float *)smem;
    auto ws = [&](int buf, int dd) { return lds + buf * W_ELEMS + dd * TK * LDW; };
    auto xs = [&](int buf, int dd) { return lds + 2 * W_ELEMS + buf * X_ELEMS + dd * TN * TK + (dd >> 2) * XPAD; };

    const int per_xcd = (blocks + 7) / 8;
    const int lid = (blockIdx.x % 8) * per_xcd + blockIdx.x / 8;
    if (lid >= blocks) return;
    const int n_dg = d / DDA;  // groups of DDA blocks
    const int mt_id = lid % m_tiles;
    int rest = lid / m_tiles;
    const int dg = rest % n_dg;
    rest /= n_dg;
    const int nt_id = rest % n_tiles;
    const int a_i = rest / n_tiles;
    const int m0 = mt_id * TM, n0 = nt_id * TN;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wg = wave / (WM * WN), wm = wave / WN % WM, wn = wave % WN;  // wg: the wave's group of 4 blocks
    const size_t in_size = (size_t)a * c * d, out_size = (size_t)a * b * d;

    stage<float, float> wreg[PDW][W_PER_T];
    uint4_t xreg[PDX][XQ_PER_T][2];
    // The loads of a slab are issued unconditionally: a branch around them would leave the
    // compiler two histories of the load counter to merge, and it would then wait for every
    // load in flight before it touches a register of the pipeline.  Behind the last slab
    // (live == false) every lane reads the first 16 bytes of the tile instead (one line): the
    // offsets are masked, not selected, so that no branch comes back.  Addresses are a uniform
    // base per tile plus a 32-bit offset per lane (the host checks that they fit).
    const TW *const wt = w + ((size_t)(a_i * d + dg * DDA) * c) * b + m0;
    const float *const xt = x + (size_t)n0 * in_size + (size_t)a_i * c * d + dg * DDA;
    uint32_t woff[W_PER_T], xoff[XQ_PER_T];
#pragma unroll
    for (int i = 0; i < W_PER_T; ++i) {
        const int v = tid + i * THREADS;
        constexpr int per_dd = TK * TM / W_EPV;
        const int dd = v / per_dd, r = v % per_dd;
        const int kk = r / (TM / W_EPV), mm = (r % (TM / W_EPV)) * W_EPV;
        woff[i] = (uint32_t)((dd * c + kk) * b + mm);
    }
#pragma unroll
    for (int i = 0; i < XQ_PER_T; ++i) {
        const int v = tid + i * THREADS;
        // the group runs fastest: neighbouring lanes read neighbouring vectors of one line
        const int g = v % NG, k8 = v / NG % KH, nn = v / (KH * NG);
        xoff[i] = (uint32_t)(min(nn, batch - 1 - n0) * (uint32_t)in_size + k8 * d + g * DD);
    }
    auto live_mask = [](bool live) {
        int lv = live;
        asm volatile("" : "+v"(lv));  // opaque: stays a mask
        return 0u - (uint32_t)lv;
    };
    auto gload_w = [&](int slot, int k0, bool live) {
        const uint32_t mk = live_mask(live);
#pragma unroll
        for (int i = 0; i < W_PER_T; ++i) wreg[slot][i].load(wt + ((woff[i] + (uint32_t)(k0 * b)) & mk));
    };
    auto gload_x = [&](int slot, int k0, bool live) {
        const uint32_t mk = live_mask(live);
#pragma unroll
        for (int i = 0; i < XQ_PER_T; ++i)
#pragma unroll
            for (int j = 0; j < 2; ++j)
                xreg[slot][i][j] = *(const uint4_t *)(xt + ((xoff[i] + (uint32_t)((k0 + KH * j) * d)) & mk));
    };
    auto lstore = [&](int wslot, int slot, int buf) {
#pragma unroll
        for (int i = 0; i < W_PER_T; ++i) {
            const int v = tid + i * THREADS;
            constexpr int per_dd = TK * TM / W_EPV;
            const int dd = v / per_dd, r = v % per_dd;
            const int kk = r / (TM / W_EPV), mm = (r % (TM / W_EPV)) * W_EPV;
            wreg[wslot][i].store(ws(buf, dd) + kk * LDW + (mm ^ (WSW * (kk & 1))));
        }
#pragma unroll
        for (int i = 0; i < XQ_PER_T; ++i) {
            const int v = tid + i * THREADS;
            const int g = v % NG, k8 = v / NG % KH, nn = v / (KH * NG);
            // k = k8 and k8 + KH of row nn, element k at k ^ 2 * ((nn / 4) % 8) (rows of 8 k: k ^ 2 * ((nn / 8) % 4))
            float *const dst = xs(buf, g * DD) + nn * TK;
            const int fn = TK == 16 ? 2 * ((nn >> 2) & 7) : 2 * ((nn >> 3) & 3);
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                const uint4_t cj = xreg[slot][i][j];
#pragma unroll
                for (int dd = 0; dd < DD; ++dd) *(uint32_t *)(dst + dd * TN * TK + ((k8 + KH * j) ^ fn)) = cj[dd];
            }
        }
    };

    float16_t acc[DD][MT][NT];
#pragma unroll
    for (int dd = 0; dd < DD; ++dd)
#pragma unroll
        for (int i = 0; i < MT; ++i)
#pragma unroll
            for (int j = 0; j < NT; ++j)
#pragma unroll
                for (int e = 0; e < 16; ++e) acc[dd][i][j][e] = 0.f;

    const int l32 = lane & 31, lq = lane >> 5;
    int xrow[NT], xfn[NT];  // the lane's row inside a plane (elements) and its column swizzle
#pragma unroll
    for (int j = 0; j < NT; ++j) {
        const int n = (wn * NT + j) * 32 + l32;
        xrow[j] = n * TK;
        xfn[j] = TK == 16 ? 2 * ((n >> 2) & 7) : 2 * ((n >> 3) & 3);
    }
    // operands of MFMA step k0 + 2 are requested before the MFMAs of step k0 are issued
    auto multiply = [&](int buf) {
        float fw[2][DD][MT], fx[2][DD][NT];
        auto read = [&](int k0, float(&rw)[DD][MT], float(&rx)[DD][NT]) {
            int xcol[NT];
#pragma unroll
            for (int j = 0; j < NT; ++j) xcol[j] = xrow[j] + ((k0 + lq) ^ xfn[j]);
#pragma unroll
            for (int dd = 0; dd < DD; ++dd) {
                const float *wb = ws(buf, wg * DD + dd), *xb = xs(buf, wg * DD + dd);
#pragma unroll
                for (int i = 0; i < MT; ++i) rw[dd][i] = wb[(k0 + lq) * LDW + (((wm * MT + i) * 32 + l32) ^ (WSW * lq))];
#pragma unroll
                for (int j = 0; j < NT; ++j) rx[dd][j] = xb[xcol[j]];
            }
        };
        read(0, fw[0], fx[0]);
#pragma unroll
        for (int ks = 0; ks < TK / 2; ++ks) {
            if (ks + 1 < TK / 2) read(2 * ks + 2, fw[(ks + 1) & 1], fx[(ks + 1) & 1]);
            __builtin_amdgcn_sched_barrier(0);  // (the scheduler would sink the reads to their uses)
#pragma unroll
            for (int dd = 0; dd < DD; ++dd)
#pragma unroll
                for (int i = 0; i < MT; ++i)
#pragma unroll
                    for (int j = 0; j < NT; ++j)
                        acc[dd][i][j] = frag<float>::mfma(fx[ks & 1][dd][j], fw[ks & 1][dd][i], acc[dd][i][j]);
            __builtin_amdgcn_sched_barrier(0);
        }
    };

    const int steps = c / TK;
    // slab s: request weights PDW and input PDX slabs ahead into the slots slab s came from (it
    // went to LDS an iteration ago), multiply slab s, move slab s + 1 from its registers to
    // the other LDS buffer.  The weights come from L2 and get the shorter lead; they are
    // requested first, so that waiting for them leaves the younger input loads in flight.
    constexpr int PERIOD = PDX * PDW / (PDX % PDW == 0 ? PDW : PDW % PDX == 0 ? PDX : 1);
    static_assert(PERIOD % PDX == 0 && PERIOD % PDW == 0, "slots repeat after PERIOD slabs");
    auto slab = [&](int u, int s) {
        gload_w(u % PDW, (s + PDW) * TK, s + PDW < steps);
        gload_x(u % PDX, (s + PDX) * TK, s + PDX < steps);
        // (the LDS stores of the next slab must not move up here: they would wait for that slab
        // before this one is multiplied)
        __builtin_amdgcn_sched_barrier(0);
        multiply(s & 1);
        __builtin_amdgcn_sched_barrier(0);
        lstore((u + 1) % PDW, (u + 1) % PDX, (s & 1) ^ 1);  // behind the last slab: whatever the idle loads brought
        __syncthreads();
    };
#pragma unroll
    for (int u = 0; u < (PDX > PDW ? PDX : PDW); ++u) {
        if (u < PDW) gload_w(u, u * TK, u < steps);
        if (u < PDX) gload_x(u, u * TK, u < steps);
    }
    lstore(0, 0, 0);
    __syncthreads();
    int s = 0;
    for (; s + PERIOD <= steps; s += PERIOD) {
#pragma unroll
        for (int u = 0; u < PERIOD; ++u) slab(u, s + u);
    }
#pragma unroll
    for (int u = 0; u < PERIOD - 1; ++u)
        if (s + u < steps) slab(u, s + u);

    // D tile: lane holds output column m = lane % 32, batch rows 8*(e/4) + 4*(lane/32) + e%4;
    // the 4 results of one (n, m) are adjacent in y: one 16-byte store
    if constexpr (FL) {
        // the NG groups of one (n, m) sit in NG waves and are adjacent in y: the tile goes to LDS
        // as [n][m][group] (16-byte pieces, the group xor-ed with bits of m) and leaves in whole runs
        uint4_t *const ot = (uint4_t *)smem;
        // (rows of m are 16 * NG bytes apart: 16 / NG consecutive m cover the banks once, so the
        // group is xor-ed with m / (16 / NG))
        auto okey = [](int ml) { return (ml * NG >> 4) & (NG - 1); };
#pragma unroll
        for (int i = 0; i < MT; ++i)
#pragma unroll
            for (int j = 0; j < NT; ++j) {
                const int ml = (wm * MT + i) * 32 + l32;
                float bv[DD];
#pragma unroll
                for (int dd = 0; dd < DD; ++dd)
                    bv[dd] = epi_bias<float>(ep, ((size_t)a_i * b + m0 + ml) * d + dg * DDA + wg * DD + dd);
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    const int nl = (wn * NT + j) * 32 + 8 * (e >> 2) + 4 * lq + (e & 3);
                    pack_t<float, DD> o;
#pragma unroll
                    for (int dd = 0; dd < DD; ++dd) o.e[dd] = epi_finish(ep, acc[dd][i][j][e], bv[dd]);
                    ot[(nl * TM + ml) * NG + (wg ^ okey(ml))] = __builtin_bit_cast(uint4_t, o);
                }
            }
        __syncthreads();
        constexpr int PIECES = TN * TM * NG;
        static_assert(PIECES % THREADS == 0, "whole pieces per thread");
#pragma unroll 4
        for (int q = tid; q < PIECES; q += THREADS) {
            const int ch = q % NG, ml = q / NG % TM, nl = q / (NG * TM);
            if (n0 + nl < batch)
                *(uint4_t *)(y + (size_t)(n0 + nl) * out_size + ((size_t)a_i * b + m0 + ml) * d + dg * DDA + ch * DD) =
                    ot[(nl * TM + ml) * NG + (ch ^ okey(ml))];
        }
        return;
    }
#pragma unroll
    for (int i = 0; i < MT; ++i)
#pragma unroll
        for (int j = 0; j < NT; ++j) {
            const int m = m0 + (wm * MT + i) * 32 + l32;
            const int nb = n0 + (wn * NT + j) * 32;
            float bv[DD];
#pragma unroll
            for (int dd = 0; dd < DD; ++dd) bv[dd] = epi_bias<float>(ep, ((size_t)a_i * b + m) * d + dg * DD + dd);
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const int n = nb + 8 * (e >> 2) + 4 * lq + (e & 3);
                pack_t<float, DD> o;
#pragma unroll
                for (int dd = 0; dd < DD; ++dd) o.e[dd] = epi_finish(ep, acc[dd][i][j][e], bv[dd]);
                if (n < batch)
                    *(pack_t<float, DD> *)(y + (size_t)n * out_size + ((size_t)a_i * b + m) * d + dg * DD) = o;
            }
        }
}

// LDS of the whole-d form: one buffer of planes, or the staged result tile if that is larger
constexpr int bf8l_lds(int ng, int tk, int tm, int tn)
{
    const int ldw = tm == 32 ? 32 : pads<half_t>::outer(tm);
    const int planes = 2 * (2 * 8 * ng * (tk * ldw + tn * tk) + 256), out = tm * tn * 8 * ng * 2;
    return planes > out ? planes : out;
}
constexpr int bf4l_lds(int ng, int tk, int tm, int tn)
{
    const int planes = 2 * 4 * (4 * ng * (tk * tm + tn * tk) + 64), out = tm * tn * 4 * ng * 4;
    return planes > out ? planes : out;
}
struct BfInst {
    int combo, dd, tm, tn, tk, threads, lds, wm;
    const void *fn;
    int pd;  // slabs in flight in registers, input * 16 + weights (ks_tile_bf8_kernel); 0: the plain kernel
};
#define BF_INST(COMBO_, CT_, TW_, DD_, TM_, TN_, TK_, WM_, WN_)                                  \
    {COMBO_, DD_, TM_, TN_, TK_, 64 * WM_ * WN_, BfCfg<CT_, TW_, DD_, TM_, TN_, TK_, WM_, WN_>::LDS_BYTES, WM_, \
     (const void *)ks_tile_bf_kernel<CT_, TW_, CT_, DD_, TM_, TN_, TK_, WM_, WN_>}
// e4m3fn input and weights, fp16 planes and output
#define BF_INST_Q(DD_, TM_, TN_, TK_, WM_, WN_)                                                   \
    {2, DD_, TM_, TN_, TK_, 64 * WM_ * WN_, BfCfg<half_t, fp8_t, DD_, TM_, TN_, TK_, WM_, WN_, fp8_t>::LDS_BYTES, WM_, \
     (const void *)ks_tile_bf_kernel<half_t, fp8_t, half_t, DD_, TM_, TN_, TK_, WM_, WN_, fp8_t>}
#define BF_SET_H(COMBO_, TW_)                                                                    \
    BF_INST(COMBO_, half_t, TW_, 2, 128, 128, 32, 2, 2), BF_INST(COMBO_, half_t, TW_, 2, 256, 128, 32, 2, 2), \
        BF_INST(COMBO_, half_t, TW_, 2, 128, 256, 32, 2, 2), BF_INST(COMBO_, half_t, TW_, 2, 64, 128, 32, 1, 4), \
        BF_INST(COMBO_, half_t, TW_, 2, 32, 128, 32, 1, 4), BF_INST(COMBO_, half_t, TW_, 4, 64, 128, 32, 1, 4), \
        BF_INST(COMBO_, half_t, TW_, 4, 32, 128, 32, 1, 4)
// groups of 8 blocks out of any d that is a multiple of 8 (a 16-byte vector per row and k)
#define BF_SET_H8(COMBO_, TW_)                                                                   \
    BF_INST(COMBO_, half_t, TW_, 8, 64, 64, 32, 2, 2), BF_INST(COMBO_, half_t, TW_, 8, 64, 64, 16, 2, 2), \
        BF_INST(COMBO_, half_t, TW_, 8, 32, 128, 16, 1, 4), BF_INST(COMBO_, half_t, TW_, 8, 128, 64, 16, 4, 2)
#define BF8_INST(COMBO_, TX_, TW_, TM_, TN_, WM_, WN_, PDX_, PDW_)                                    \
    {COMBO_, 8, TM_, TN_, 16, 64 * WM_ * WN_,                                                    \
     2 * 2 * (8 * 16 * pads<half_t>::outer(TM_) + 8 * TN_ * 16), WM_,                            \
     (const void *)ks_tile_bf8_kernel<TX_, TW_, TM_, TN_, WM_, WN_, PDX_, PDW_>, PDX_ * 16 + PDW_}
#define BF4_INST(TM_, TN_, WM_, WN_, PDX_, PDW_)                                                 \
    {0, 4, TM_, TN_, 16, 64 * WM_ * WN_, 2 * 4 * (4 * 16 * TM_ + 4 * TN_ * 16), WM_,                 \
     (const void *)ks_tile_bf4_kernel<TM_, TN_, WM_, WN_, PDX_, PDW_>, PDX_ * 16 + PDW_}
#define BF8L_INST(COMBO_, TX_, TW_, NG_, TK_, TM_, TN_, WM_, WN_, PDX_, PDW_)                         \
    {COMBO_, 8 * NG_, TM_, TN_, TK_, 64 * WM_ * WN_ * NG_,                                       \
     bf8l_lds(NG_, TK_, TM_, TN_), WM_,                                                          \
     (const void *)ks_tile_bf8_kernel<TX_, TW_, TM_, TN_, WM_, WN_, PDX_, PDW_, NG_, TK_>, 256 + PDX_ * 16 + PDW_}
#define BF4L_INST(NG_, TK_, TM_, TN_, WM_, WN_, PDX_, PDW_)                                           \
    {0, 4 * NG_, TM_, TN_, TK_, 64 * WM_ * WN_ * NG_, bf4l_lds(NG_, TK_, TM_, TN_), WM_,            \
     (const void *)ks_tile_bf4_kernel<TM_, TN_, WM_, WN_, PDX_, PDW_, NG_, TK_>, 256 + PDX_ * 16 + PDW_}
#define BF8_SET(COMBO_, TX_, TW_)                                                                \
    BF8_INST(COMBO_, TX_, TW_, 64, 64, 2, 2, 2, 2), BF8_INST(COMBO_, TX_, TW_, 64, 128, 2, 4, 2, 2)
const BfInst bf_insts[] = {
    BF_SET_H(1, half_t),
    BF_SET_H(3, fp8_t),
    BF_INST(0, float, float, 2, 128, 128, 16, 2, 2),
    BF_INST(0, float, float, 2, 64, 128, 16, 1, 4),
    BF_INST(0, float, float, 2, 32, 128, 16, 1, 4),
    BF_INST(0, float, float, 4, 64, 128, 16, 1, 4),
    BF_INST(0, float, float, 4, 32, 128, 16, 1, 4),
    // appended (ids of the rows above stay): 16-bit groups of 8 blocks
    BF_SET_H8(1, half_t),
    BF_SET_H8(3, fp8_t),
    // the same groups with a register pipeline (ks_tile_bf8_kernel)
    BF8_SET(1, half_t, half_t),
    BF8_SET(3, half_t, fp8_t),
    // fp32 groups of 4 (ks_tile_bf4_kernel)
    BF4_INST(64, 64, 2, 2, 2, 2),
    BF4_INST(64, 128, 2, 4, 2, 2),
    // e4m3 input and weights: groups of 8 again (8-byte vectors, decoded on their way to LDS)
    BF8_SET(2, fp8_t, fp8_t),
    // e4m3 input and weights, d = 2 or 4 whole (a 16-byte vector is 8 or 4 k of every d_i)
    // ((1,768,192,2) at batch 25088: 62 us on the 64 x 128 tile, 67-71 on the larger ones; about
    // what the transposed route takes, without its workspace)
    BF_INST_Q(2, 64, 128, 32, 1, 4), BF_INST_Q(2, 128, 128, 32, 2, 2), BF_INST_Q(2, 256, 128, 32, 2, 2),
    BF_INST_Q(2, 32, 128, 32, 1, 4), BF_INST_Q(4, 64, 128, 32, 1, 4), BF_INST_Q(4, 32, 128, 32, 1, 4),
    // 32 or 16 blocks per workgroup (pipelined kernel with slabs of 8 k, 8 waves, one workgroup per CU)
    BF8L_INST(1, half_t, half_t, 4, 8, 64, 32, 2, 1, 2, 2), BF8L_INST(1, half_t, half_t, 4, 8, 32, 64, 1, 2, 2, 2),
    BF8L_INST(1, half_t, half_t, 2, 8, 64, 64, 2, 2, 2, 2),
    BF8L_INST(3, half_t, fp8_t, 4, 8, 64, 32, 2, 1, 2, 2), BF8L_INST(3, half_t, fp8_t, 4, 8, 32, 64, 1, 2, 2, 2),
    BF8L_INST(3, half_t, fp8_t, 2, 8, 64, 64, 2, 2, 2, 2),
    BF8L_INST(2, fp8_t, fp8_t, 4, 8, 64, 32, 2, 1, 2, 2), BF8L_INST(2, fp8_t, fp8_t, 4, 8, 32, 64, 1, 2, 2, 2),
    BF8L_INST(2, fp8_t, fp8_t, 2, 8, 64, 64, 2, 2, 2, 2),
    // fp32: 16 or 8 blocks per workgroup (32 blocks on a 32 x 32 tile never won; 8 blocks in slabs of
    // 16 k, which fit, were 2-8 % slower than in slabs of 8)
    BF4L_INST(4, 8, 64, 32, 2, 1, 2, 2), BF4L_INST(4, 8, 32, 64, 1, 2, 2, 2), BF4L_INST(2, 8, 64, 64, 2, 2, 2, 2),
    // 16-bit d = 4 and 2 whole on 8 waves (the 4-wave instances above leave one wave per SIMD when
    // their planes fill the LDS: fp16 (48,384,384,4) 4265 -> 3091 us on the 128 x 128 tile,
    // (64,256,256,4) 3246 -> 2204, (96,192,192,4) 2888 -> 2218 on 64 x 128 with slabs of 16)
    BF_INST(1, half_t, half_t, 4, 64, 128, 16, 2, 4), BF_INST(1, half_t, half_t, 4, 128, 128, 32, 2, 4),
    BF_INST(1, half_t, half_t, 4, 128, 128, 16, 2, 4), BF_INST(1, half_t, half_t, 4, 64, 64, 16, 2, 2),
    BF_INST(1, half_t, half_t, 2, 128, 128, 32, 2, 4), BF_INST(1, half_t, half_t, 2, 128, 256, 32, 2, 4),
    BF_INST(1, half_t, half_t, 2, 256, 128, 32, 4, 2),
    BF_INST(3, half_t, fp8_t, 4, 64, 128, 16, 2, 4), BF_INST(3, half_t, fp8_t, 4, 128, 128, 32, 2, 4),
    BF_INST(3, half_t, fp8_t, 2, 128, 128, 32, 2, 4),
    BF_INST_Q(4, 64, 128, 32, 2, 4), BF_INST_Q(4, 128, 128, 32, 2, 4), BF_INST_Q(2, 128, 128, 32, 2, 4),
    // fp32 groups of 4 on 128-row tiles, 8 waves (one slab in flight in registers: two spill); big d = 4
    // blocks 4-9 % faster than on 64 x 128 ((64,256,256,4) 8419 -> 7900 us, (32,128,128,4) 1240 -> 1122)
    BF4_INST(128, 64, 4, 2, 2, 2), BF4_INST(128, 128, 2, 4, 1, 1), BF4_INST(128, 128, 4, 2, 1, 1),
    // 16-bit groups of 8 on a 128 x 64 tile, 8 waves
    BF8_INST(1, half_t, half_t, 128, 64, 4, 2, 2, 2), BF8_INST(3, half_t, fp8_t, 128, 64, 4, 2, 2, 2),
    BF8_INST(2, fp8_t, fp8_t, 128, 64, 4, 2, 2, 2),
};
constexpr int N_BF_INSTS = sizeof(bf_insts) / sizeof(BfInst);

bool bf_fits(const BfInst &t, const Problem &p, int combo)
{
    if (t.combo != combo || p.bs_last || p.d % t.dd) return false;
    if (p.b % t.tm || p.c % t.tk) return false;
    const int x_epv = 16 / (int)dtype_size(p.x_dtype), w_epv = 16 / (int)dtype_size(p.w_dtype);
    // d > DD: the DD elements of one (row, k) must fill the 16-byte vector
    // (the pipelined e4m3 instances read 8-byte vectors: groups of 8 out of any multiple of 8)
    const int vec = (t.pd && combo == 2) ? 8 : x_epv;
    if (p.d != t.dd && (t.pd ? t.dd % vec != 0 : t.dd != vec)) return false;
    if (p.b % w_epv) return false;
    // rows of x start at multiples of in_size, slabs at multiples of TK * d: keep 16-byte alignment
    if (((int64_t)p.a * p.c * p.d) % vec || ((int64_t)p.c * p.d) % vec) return false;
    if (t.pd) {
        // 32-bit element offsets inside a tile: TN rows of x, DD blocks of w
        if ((int64_t)t.tn * p.a * p.c * p.d + (int64_t)p.c * p.d >= 0xffffffffLL) return false;
        if ((int64_t)t.dd * p.c * p.b >= 0xffffffffLL) return false;
    }
    return true;
}

}  // namespace

int bf_inst_count() { return N_BF_INSTS; }

uint32_t bf_inst_id(int i)
{
    if (i < 0 || i >= N_BF_INSTS) return 0;
    const BfInst &t = bf_insts[i];
    const int v[8] = {t.combo, t.dd, t.tm, t.tn, t.tk, t.threads, t.wm, t.pd};
    return inst_hash('B', v, t.pd ? 8 : 7);  // (ids of the plain instances predate the field)
}


// variant: index into the instance table (-1: heuristic)
int tile_bf_run(const Problem &p, int variant, bool launch, ksmm_tile *tile)
{
    const int combo = combo_of(p.x_dtype, p.w_dtype, p.y_dtype);
    int pick = -1;
    if (variant >= 0) {
        if (variant < N_BF_INSTS && bf_fits(bf_insts[variant], p, combo)) pick = variant;
    } else {
        int64_t best = -1;
        for (int i = 0; i < N_BF_INSTS; ++i) {
            const BfInst &t = bf_insts[i];
            if (!bf_fits(t, p, combo)) continue;
            // Groups out of a larger d: every line of x is shared by d/DD groups x b/TM tiles, and
            // the loads are 16-byte pieces d elements apart.  Against the transposed route (two
            // extra passes, but the fastest kernels in between) this wins while b x d stays
            // moderate: measured at batch 25088 on 33 patterns around these bounds with the
            // pipelined instances, time ratio 0.5-0.9 inside (fp16 (1,64,256,128) 1277 -> 765 us,
            // (1,512,128,16) 333 -> 257; fp32 (1,512,128,8) 466 -> 328) and 1.0-1.3 outside
            // ((1,768,192,24) fp16, (1,192,192,32) fp32, very long c).
            // 16-bit blocks of 512 x 512 and more (b at least 512) are matrix-core-bound: there
            // the batch-size-last GEMM tiles between two transposes beat this kernel (the
            // transposes move each operand once more, the GEMM tiles run at 2-3x its
            // matrix-core rate)
            // (e4m3 input: the bounds measured for it below)
            if (p.d == t.dd && combo != 0 && combo != 2 && p.b >= 512 && (int64_t)p.b * p.c >= 512 * 512) continue;
            // e4m3 input with d = 2 or 4 whole: measured against the transposed route on the 102
            // such patterns of the reference's list (batch 25088), the direct kernel wins (time
            // ratio 0.6-0.97) with short c or narrow blocks and loses (1.1-2.3) elsewhere: the
            // e4m3 GEMM tiles in the middle of the other route multiply at twice the rate
            // (with the instances on 8 waves, measured again on the 110 patterns that had stayed on
            // the other route: the direct kernel also wins, ratio 0.66-0.94, for d = 4 on blocks up to
            // 384 x 384 / 768 x 192 with b a multiple of 64 and c <= 384, and for d = 2 with b a
            // multiple of 128 up to 512 x 512 / 256 x 1024 / 1536 x 384; it loses, 1.1-1.8, on 96-row
            // blocks, c = 768 and blocks of 768 x 768 and more)
            if (combo == 2 && !t.pd) {
                const int64_t bc = (int64_t)p.b * p.c;
                const bool pays = p.d == 2 ? (p.c <= 128 || (p.c <= 256 && p.b <= 512) ||
                                              (p.b % 128 == 0 && (bc <= 262144 || (bc <= 589824 && p.c <= 384))))
                                           : (p.c <= 96 || (p.b <= 64 && p.a >= 3) ||
                                              (p.b % 64 == 0 && p.c <= 384 && (bc < 147456 || (bc == 147456 && (p.a >= 4 || p.c <= 192)))));
                if (!pays) continue;
            }
            const bool wide = t.pd >= 256;  // 32 or 16 blocks per workgroup
            // fp32 groups of 4 on 128-row tiles: the best choice on half of the patterns they fit and up
            // to 18 % behind the 64-row tiles on the others, with no simple bound between: named by the
            // measured table only
            if (combo == 0 && t.pd && !wide && t.tm == 128) continue;
            if (wide && combo == 0) {
                // fp32, measured the same way on the 161 patterns with d a multiple of 8: the
                // wider groups win from d = 16 on (0.61-0.98 of the time of the groups of 4; 8
                // blocks on 64 x 64 where b allows, else 16 blocks on 32 x 64), not at d = 8
                if (p.d < 16) continue;
            } else if (wide) {
                // Measured against the groups of 8 and the row kernel on the 141 patterns of the
                // reference's lists with d a multiple of 16 (batch 25088, fp16 and e4m3): 32 blocks
                // win from d = 64 on (time ratio 0.62-0.93) and, fp16, at d = 32 with short c
                // (0.88-0.90); 16 blocks win where d is not a multiple of 32 (d = 48: 0.79-0.98),
                // fp16 at d = 32 with longer c (0.77-0.90) and at d = 16 on wide short blocks
                // (0.90-0.97); elsewhere the groups of 8 stay within 3 %.
                const bool fits32 = p.d % 32 == 0 && (p.d >= 64 || (combo != 2 && p.c <= 128));
                const bool pays = t.dd == 32 ? fits32
                                             : (!fits32 && ((p.d % 32 != 0 && p.d >= 48) || (combo != 2 && p.d == 32) ||
                                                            (p.d == 16 && p.b >= 384 && p.c <= 192)));
                if (!pays) continue;
            }
            if (p.d != t.dd) {
                const int64_t bd = (int64_t)p.b * p.d;
                const bool pays = combo == 0 ? ((p.d <= 16 && p.b <= 192) || (bd <= 8192 && (p.d <= 16 || p.c <= 128)))
                                             : ((t.tm >= 64 || wide) && ((p.d <= 32 && p.b <= 384) ||
                                                               (p.c <= 256 && (p.b <= 192 ? p.d <= 128 : bd <= 12288))));
                if (!pays) continue;
            }
            const int64_t wgs = (int64_t)p.a * (p.d / t.dd) * (p.b / t.tm) * ((p.batch + t.tn - 1) / t.tn);
            // (between equal tiles the instance on more waves: two waves per SIMD where the planes
            // leave room for one workgroup per CU)
            int64_t score = (int64_t)t.tm * 1000 + t.tn + t.threads / 256;
            // the pipelined 64 x 64 form first (1.1-1.3x the plain instances on (1,192,192,8..16),
            // (4,128,128,8), (1,64,64,64) at batch 25088)
            if (t.pd && !wide && t.tn == 64 && wgs >= 512) score += 500000;
            if (wide && wgs >= 512) score += 600000;
            if (wgs < 512) score -= 100000;
            if (score > best) {
                best = score;
                pick = i;
            }
        }
    }
    if (pick < 0) return KSMM_ERR_BAD_ALGO;
    const BfInst &t = bf_insts[pick];
    const int m_tiles = p.b / t.tm;
    const int64_t n_tiles = (p.batch + t.tn - 1) / t.tn;
    const int64_t blocks = (int64_t)p.a * (p.d / t.dd) * m_tiles * n_tiles;
    const int64_t grid = (blocks + 7) / 8 * 8;
    if (grid > 0x7fffffffLL) return KSMM_ERR_TOO_LARGE;
    if (tile) {
        tile->algo = KSMM_ALGO_TILE;
        tile->variant = (3 << 24) | pick;
        tile->tile_m = t.tm;
        tile->tile_n = t.tn;
        tile->tile_k = t.tk;
        tile->tile_d = t.dd;
        tile->threads = t.threads;
        tile->lds_bytes = t.lds;
        tile->grid = grid;
    }
    if (!launch) return KSMM_OK;
    if (ensure_dynamic_lds(t.fn, t.lds) != KSMM_OK) return KSMM_ERR_LAUNCH;
    int batch_i = (int)p.batch, n_tiles_i = (int)n_tiles, blocks_i = (int)blocks, m_tiles_i = m_tiles;
    Epi ep = epi_of(p);
    void *args[] = {(void *)&p.x, (void *)&p.w, (void *)&p.y, &batch_i, (void *)&p.a, (void *)&p.b,
                    (void *)&p.c, (void *)&p.d, &ep, &m_tiles_i, &n_tiles_i, &blocks_i};
    hipError_t e = hipLaunchKernel(t.fn, dim3((unsigned)grid), dim3(t.threads), args, t.lds, p.stream);
    return e == hipSuccess ? KSMM_OK : KSMM_ERR_LAUNCH;
}

}  // namespace ksmm
