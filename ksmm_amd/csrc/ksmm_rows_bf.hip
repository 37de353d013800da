// "Row" kernels: batch-size-first layout, small b x c blocks, d > 1 (and d == 1 in groups of
// consecutive a_i, at the end of this comment).  The fp32 kernel first; the
// fp16 / e4m3 one further down has the same structure.
//
// In this layout a batch row holds, for one a_i, the c*d inputs of all d blocks interleaved
// (d_i fastest).  A workgroup owns one a_i, a group of DD consecutive d_i (all of them when
// d == DD) and every wgs-th tile of batch rows; it has one wavefront per d_i of its group, and
// each wavefront keeps the b x c weight block of its d_i in registers as MFMA operands
// (v_mfma_f32_16x16x4_f32, fp32 accumulation).  Row segments (c runs of DD contiguous floats,
// one run of c*d floats when d == DD) are copied to LDS with 16-byte loads, every wave picks
// the inputs of its own d_i out of LDS (stride DD), the DD result blocks are interleaved again
// in an LDS output tile, and the outputs of each row are written back as b runs of DD floats.
// HBM sees coalesced runs only; the stride-d gather the layout forces happens in LDS.
//
// The loads of the next two tiles are in flight (in registers) while a tile is multiplied and
// stored; tiles are dealt round-robin to the workgroups of an a_i, so that at any time they
// work on one compact window of memory.
//
// d == 1 with blocks of 16 x 16 or 32 x 32 (the last factor of a butterfly chain, (64,16,16,1)):
// the same kernel with the waves of a workgroup taking DD consecutive a_i, whose inputs are one
// contiguous run of DD * c elements per batch row; only the index arithmetic differs.
//
// Reference counterpart: kernel_bs_first_float
// (src/ksmm_py/layer/kronecker_sparse/template_kernels_float.cuh:85-286), whose strided scalar
// gathers from global memory (:156-161) make this the slowest layout of the reference
// (0.86 ms for (1,48,48,16) in kernel_bs_first_float.best:9).
#include "ksmm_common.h"
#include <type_traits>

namespace ksmm {

namespace {

// PL: the LDS tiles are split into one plane per d_i ([d_i][row][k], rows padded by 4, planes
// padded to 4 floats past a multiple of 64).  With d_i fastest all 64 lanes of an operand read
// or result write hit the same 4-byte slot of the 16-byte groups (16 banks at most: 4-way
// conflicts whatever the padding); in planes those accesses are conflict-free, and so are
// the four 4-byte stores / loads per 16-byte global vector that feed and drain them.
constexpr int plane_floats(int n) { return n + (68 - n % 64) % 64; }
// MS: waves per d_i, each holding BB / MS rows of the block (blocks whose weights do not fit the
// registers of one wave)
template <int BB, int CC, int DD, int TN, bool PL = false, int MS = 1> struct RowCfg {
    static constexpr int NW = DD * MS, THREADS = 64 * NW;
    static constexpr int MT = BB / 16 / MS, KS = CC / 4, NT = TN / 16;
    static constexpr int XROW = CC * DD, OROW = BB * DD;  // floats per row segment
    static constexpr int LDX = XROW + 4, LDO = OROW + 4;
    static constexpr int LDK = CC + 4, LDM = BB + 4;      // PL: rows of a plane
    static constexpr int PLANE_X = plane_floats(TN * LDK), PLANE_O = plane_floats(TN * LDM);
    static constexpr int X_FLOATS = PL ? DD * PLANE_X : TN * LDX, O_FLOATS = PL ? DD * PLANE_O : TN * LDO;
    static constexpr int X_VECS = TN * XROW / 4, O_VECS = TN * OROW / 4;
    static constexpr int X_PER_T = (X_VECS + THREADS - 1) / THREADS, O_PER_T = (O_VECS + THREADS - 1) / THREADS;
    static constexpr int LDS_BYTES = (2 * X_FLOATS + O_FLOATS) * 4;
    static_assert(!PL || DD % 4 == 0, "planes: a 16-byte vector is 4 d_i of one k");
    static_assert(BB % (16 * MS) == 0 && CC % 4 == 0 && TN % 16 == 0, "MFMA tiling");
    static_assert(NW <= 16 && XROW % 4 == 0 && OROW % 4 == 0, "shape");
    static_assert(LDS_BYTES <= 160 * 1024, "LDS");
};

// AG: d == 1 and the DD waves take DD consecutive a_i instead (their inputs are one contiguous run
// of DD * c elements of a batch row, block after block: the "stride" of a block's inputs is 1).
template <int BB, int CC, int DD, int TN, bool NT_STORE, bool PL = false, int MS = 1, bool AG = false>
__global__ __launch_bounds__(64 * DD * MS) void ks_rows_bf_kernel(const float *__restrict__ x,
                                                            const float *__restrict__ w,
                                                            float *__restrict__ y, int batch, int a,
                                                            int d, Epi ep, int wgs_per_a, int n_tiles)
{
    typedef RowCfg<BB, CC, DD, TN, PL, MS> C;
    static_assert(!(AG && PL), "planes are for interleaved blocks");
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    float *const xs = (float *)smem;                // [2][TN][LDX]; PL: [2][DD][PLANE_X]
    float *const os = xs + 2 * C::X_FLOATS;         // [TN][LDO]; PL: [DD][PLANE_O]
    // The d / DD workgroups that take the same tiles of one a_i read the same lines (a group's run
    // of DD elements is a piece of every line of a row): they get block indices that are equal
    // mod 8, i.e. one XCD and its L2.  (Dealt without that, whenever the workgroups per a_i are
    // not a multiple of 8, every XCD fetched the lines for its piece: (3,64,64,64) fp16 took 927 us
    // where (4,64,64,64) takes 425.)
    const int groups = AG ? 1 : d / DD;
    int a_i, d0, s;
    if (AG) {
        const int ag = blockIdx.x / wgs_per_a;
        s = blockIdx.x - ag * wgs_per_a;
        a_i = ag * DD;
        d0 = 0;
    } else {
        const int slot = blockIdx.x >> 3, grp = slot % groups;
        const int u = (slot / groups) * 8 + (blockIdx.x & 7);  // (a_i, share) pairs, 8 at a time
        if (u >= a * wgs_per_a) return;
        a_i = u / wgs_per_a;
        s = u - a_i * wgs_per_a;
        d0 = grp * DD;
    }
    const int t_begin = s, t_end = n_tiles, t_step = wgs_per_a;  // every wgs-th tile
    if (t_begin >= t_end) return;
    const int tid = threadIdx.x, lane = tid & 63, q = lane >> 4, r = lane & 15;
    const int wv = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int ms = wv / DD, dd = wv - ms * DD;  // this wave's row group and d_i
    const int m_off = ms * (BB / MS);
    const size_t in_size = (size_t)a * CC * d, out_size = (size_t)a * BB * d;

    // weights of block (a_i, dd): element (k, m) at ((a_i*d + dd)*c + k)*b + m -> A operands
    float wreg[C::MT][C::KS];
    {
        const float *wg = w + (size_t)(AG ? a_i + dd : a_i * d + d0 + dd) * CC * BB + m_off;
#pragma unroll
        for (int ks = 0; ks < C::KS; ++ks)
#pragma unroll
            for (int mt = 0; mt < C::MT; ++mt) wreg[mt][ks] = wg[(4 * ks + q) * BB + 16 * mt + r];
    }
    float bv[C::MT][4];  // bias of the outputs this lane holds: m = m_off + 16*mt + 4*q + i of d_i = d0 + dd
#pragma unroll
    for (int mt = 0; mt < C::MT; ++mt)
#pragma unroll
        for (int i = 0; i < 4; ++i)
            bv[mt][i] = epi_bias<float>(ep, AG ? (size_t)(a_i + dd) * BB + m_off + 16 * mt + 4 * q + i
                                               : ((size_t)a_i * BB + m_off + 16 * mt + 4 * q + i) * d + d0 + dd);

    // element e of a tile row (e = k * DD + j) lives at k * d + j behind the group's origin
    // (AG: e = j * c + k, at e)
    const float *xg = x + (size_t)a_i * CC * d + d0;
    float *yg = y + (size_t)a_i * BB * d + d0;
    auto row_off = [&](int e0) { return AG ? e0 : (e0 / DD) * d + e0 % DD; };
    float4_t xreg[2][C::X_PER_T];
    auto gload = [&](int t, auto P) {
#pragma unroll
        for (int i = 0; i < C::X_PER_T; ++i) {
            const int v = tid + i * C::THREADS;
            if (C::X_VECS % C::THREADS == 0 || v < C::X_VECS) {
                const int nn = v / (C::XROW / 4), e0 = (v % (C::XROW / 4)) * 4;
                const int row = min(t * TN + nn, batch - 1);
                xreg[decltype(P)::value][i] = *(const float4_t *)(xg + (size_t)row * in_size + row_off(e0));
            }
        }
    };
    auto lstore = [&](int buf, auto P) {
#pragma unroll
        for (int i = 0; i < C::X_PER_T; ++i) {
            const int v = tid + i * C::THREADS;
            if (C::X_VECS % C::THREADS == 0 || v < C::X_VECS) {
                const int nn = v / (C::XROW / 4), e0 = (v % (C::XROW / 4)) * 4;
                if constexpr (PL) {
                    float *dst = xs + buf * C::X_FLOATS + (e0 % DD) * C::PLANE_X + nn * C::LDK + e0 / DD;
#pragma unroll
                    for (int j = 0; j < 4; ++j) dst[j * C::PLANE_X] = xreg[decltype(P)::value][i][j];
                } else {
                    *(float4_t *)(xs + (buf * TN + nn) * C::LDX + e0) = xreg[decltype(P)::value][i];
                }
            }
        }
    };
    // one tile: its inputs are in LDS buffer `buf`; register set P is refilled with the tile
    // after the next one at the start, and set 1-P (the next tile) goes to the other LDS buffer
    // at the end
    auto do_tile = [&](int t, int buf, auto P) {
        typedef std::integral_constant<int, 1 - decltype(P)::value> Q;
        if (t + 2 * t_step < t_end) gload(t + 2 * t_step, P);
        const float *xb = xs + buf * C::X_FLOATS;
        float4_t acc[C::MT][C::NT];
#pragma unroll
        for (int mt = 0; mt < C::MT; ++mt)
#pragma unroll
            for (int nt = 0; nt < C::NT; ++nt) acc[mt][nt] = float4_t{0.f, 0.f, 0.f, 0.f};
        // B operand: lane (r, q) = input (k = 4*ks + q) of batch row 16*nt + r, for this d_i
        float xf[C::KS][C::NT];
#pragma unroll
        for (int ks = 0; ks < C::KS; ++ks)
#pragma unroll
            for (int nt = 0; nt < C::NT; ++nt)
                xf[ks][nt] = PL   ? xb[dd * C::PLANE_X + (16 * nt + r) * C::LDK + 4 * ks + q]
                             : AG ? xb[(16 * nt + r) * C::LDX + dd * CC + 4 * ks + q]
                                  : xb[(16 * nt + r) * C::LDX + (4 * ks + q) * DD + dd];
#pragma unroll
        for (int ks = 0; ks < C::KS; ++ks)
#pragma unroll
            for (int nt = 0; nt < C::NT; ++nt)
#pragma unroll
                for (int mt = 0; mt < C::MT; ++mt)
                    acc[mt][nt] = __builtin_amdgcn_mfma_f32_16x16x4f32(wreg[mt][ks], xf[ks][nt], acc[mt][nt], 0, 0, 0);
        // D: lane (r, q) holds batch row 16*nt + r, outputs m = 16*mt + 4*q + i
#pragma unroll
        for (int mt = 0; mt < C::MT; ++mt)
#pragma unroll
            for (int nt = 0; nt < C::NT; ++nt)
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    os[PL   ? dd * C::PLANE_O + (16 * nt + r) * C::LDM + m_off + 16 * mt + 4 * q + i
                       : AG ? (16 * nt + r) * C::LDO + dd * BB + m_off + 16 * mt + 4 * q + i
                            : (16 * nt + r) * C::LDO + (m_off + 16 * mt + 4 * q + i) * DD + dd] = epi_finish(ep, acc[mt][nt][i], bv[mt][i]);
        __syncthreads();
#pragma unroll
        for (int i = 0; i < C::O_PER_T; ++i) {
            const int v = tid + i * C::THREADS;
            if (C::O_VECS % C::THREADS == 0 || v < C::O_VECS) {
                const int nn = v / (C::OROW / 4), e0 = (v % (C::OROW / 4)) * 4;
                const int row = t * TN + nn;
                if (row < batch) {
                    float4_t o;
                    if constexpr (PL) {
                        const float *src = os + (e0 % DD) * C::PLANE_O + nn * C::LDM + e0 / DD;
#pragma unroll
                        for (int j = 0; j < 4; ++j) o[j] = src[j * C::PLANE_O];
                    } else {
                        o = *(const float4_t *)(os + nn * C::LDO + e0);
                    }
                    if (NT_STORE)
                        __builtin_nontemporal_store(o, (float4_t *)(yg + (size_t)row * out_size + row_off(e0)));
                    else
                        *(float4_t *)(yg + (size_t)row * out_size + row_off(e0)) = o;
                }
            }
        }
        if (t + t_step < t_end) lstore(buf ^ 1, Q{});
        __syncthreads();
    };

    gload(t_begin, std::integral_constant<int, 0>{});
    if (t_begin + t_step < t_end) gload(t_begin + t_step, std::integral_constant<int, 1>{});
    lstore(0, std::integral_constant<int, 0>{});
    __syncthreads();
    for (int t = t_begin; t < t_end; t += 2 * t_step) {
        do_tile(t, 0, std::integral_constant<int, 0>{});
        if (t + t_step < t_end) do_tile(t + t_step, 1, std::integral_constant<int, 1>{});
    }
}

// ---- the same for 16-bit and 8-bit inputs --------------------------------------------------
// fp16 or e4m3 inputs and weights, fp16 MFMA (v_mfma_f32_16x16x16_f16, e4m3 decoded exactly
// when an operand is picked out of LDS or loaded as a weight), fp32 accumulation, fp16
// output.  Row segments travel as 16-byte vectors (8 halves / 16 e4m3), so c * DD and b * DD
// must be multiples of the vector (and DD itself when d > DD: runs of DD elements).
template <typename TX, int BB, int CC, int DD, int TN, int MS = 1> struct RowCfgH {
    static constexpr int NW = DD * MS, THREADS = 64 * NW;
    static constexpr int ES = (int)sizeof(TX), EPV = 16 / ES;   // input element, elements per vector
    static constexpr int MT = BB / 16 / MS, KS = CC / 16, NT = TN / 16;
    static constexpr int XROW = CC * DD, OROW = BB * DD;         // elements per row segment
    static constexpr int LDX = XROW + EPV, LDO = OROW + 8;       // padded LDS rows (elements)
    static constexpr int X_VECS = TN * XROW / EPV, O_VECS = TN * OROW / 8;
    static constexpr int X_PER_T = (X_VECS + THREADS - 1) / THREADS, O_PER_T = (O_VECS + THREADS - 1) / THREADS;
    static constexpr int X_BYTES = 2 * TN * LDX * ES, LDS_BYTES = X_BYTES + TN * LDO * 2;
    static_assert(BB % (16 * MS) == 0 && CC % 16 == 0 && TN % 16 == 0, "MFMA tiling");
    static_assert(NW <= 16 && XROW % EPV == 0 && OROW % 8 == 0, "shape");
    static_assert(LDS_BYTES <= 160 * 1024, "LDS");
};

__device__ __forceinline__ half_t row_to_half(half_t v) { return v; }
__device__ __forceinline__ half_t row_to_half(fp8_t v) { return fp8_to_half(v.bits); }

template <typename TX, int BB, int CC, int DD, int TN, bool AG = false, int MS = 1>
__global__ __launch_bounds__(64 * DD * MS) void ks_rows_bf_h_kernel(const TX *__restrict__ x, const TX *__restrict__ w,
                                                              half_t *__restrict__ y, int batch, int a, int d,
                                                              Epi ep, int wgs_per_a, int n_tiles)
{
    typedef RowCfgH<TX, BB, CC, DD, TN, MS> C;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    TX *const xs = (TX *)smem;                         // [2][TN][LDX]
    half_t *const os = (half_t *)(smem + C::X_BYTES);  // [TN][LDO]
    // The d / DD workgroups that take the same tiles of one a_i read the same lines (a group's run
    // of DD elements is a piece of every line of a row): they get block indices that are equal
    // mod 8, i.e. one XCD and its L2.  (Dealt without that, whenever the workgroups per a_i are
    // not a multiple of 8, every XCD fetched the lines for its piece: (3,64,64,64) fp16 took 927 us
    // where (4,64,64,64) takes 425.)
    const int groups = AG ? 1 : d / DD;
    int a_i, d0, s;
    if (AG) {
        const int ag = blockIdx.x / wgs_per_a;
        s = blockIdx.x - ag * wgs_per_a;
        a_i = ag * DD;
        d0 = 0;
    } else {
        const int slot = blockIdx.x >> 3, grp = slot % groups;
        const int u = (slot / groups) * 8 + (blockIdx.x & 7);  // (a_i, share) pairs, 8 at a time
        if (u >= a * wgs_per_a) return;
        a_i = u / wgs_per_a;
        s = u - a_i * wgs_per_a;
        d0 = grp * DD;
    }
    const int t_begin = s, t_end = n_tiles, t_step = wgs_per_a;  // every wgs-th tile
    if (t_begin >= t_end) return;
    const int tid = threadIdx.x, lane = tid & 63, q = lane >> 4, r = lane & 15;
    const int wv = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int ms = wv / DD, dd = wv - ms * DD;  // this wave's row group of the block and its d_i inside the group
    const int m_off = ms * (BB / MS);
    const size_t in_size = (size_t)a * CC * d, out_size = (size_t)a * BB * d;

    // weights of block (a_i, d0 + dd): element (k, m) at ((a_i*d + d0 + dd)*c + k)*b + m;
    // A operand of sub-step ks: lane (r, q) holds k = 16*ks + 4*q .. + 3 of row m = m_off + 16*mt + r
    half4_t wreg[C::MT][C::KS];
    {
        const TX *wg = w + (size_t)(AG ? a_i + dd : a_i * d + d0 + dd) * CC * BB + m_off;
#pragma unroll
        for (int ks = 0; ks < C::KS; ++ks)
#pragma unroll
            for (int mt = 0; mt < C::MT; ++mt)
#pragma unroll
                for (int j = 0; j < 4; ++j) wreg[mt][ks][j] = row_to_half(wg[(16 * ks + 4 * q + j) * BB + 16 * mt + r]);
    }
    float bv[C::MT][4];  // bias of the outputs this lane holds: m = 16*mt + 4*q + i of d_i = d0 + dd
#pragma unroll
    for (int mt = 0; mt < C::MT; ++mt)
#pragma unroll
        for (int i = 0; i < 4; ++i)
            bv[mt][i] = epi_bias<half_t>(ep, AG ? (size_t)(a_i + dd) * BB + m_off + 16 * mt + 4 * q + i
                                                : ((size_t)a_i * BB + m_off + 16 * mt + 4 * q + i) * d + d0 + dd);

    const TX *xg = x + (size_t)a_i * CC * d + d0;
    half_t *yg = y + (size_t)a_i * BB * d + d0;
    auto row_off = [&](int e0) { return AG ? e0 : (e0 / DD) * d + e0 % DD; };
    uint4_t xreg[2][C::X_PER_T];
    auto gload = [&](int t, auto P) {
#pragma unroll
        for (int i = 0; i < C::X_PER_T; ++i) {
            const int v = tid + i * C::THREADS;
            if (C::X_VECS % C::THREADS == 0 || v < C::X_VECS) {
                const int nn = v / (C::XROW / C::EPV), e0 = (v % (C::XROW / C::EPV)) * C::EPV;
                const int row = min(t * TN + nn, batch - 1);
                xreg[decltype(P)::value][i] = *(const uint4_t *)(xg + (size_t)row * in_size + row_off(e0));
            }
        }
    };
    auto lstore = [&](int buf, auto P) {
#pragma unroll
        for (int i = 0; i < C::X_PER_T; ++i) {
            const int v = tid + i * C::THREADS;
            if (C::X_VECS % C::THREADS == 0 || v < C::X_VECS) {
                const int nn = v / (C::XROW / C::EPV), e0 = (v % (C::XROW / C::EPV)) * C::EPV;
                *(uint4_t *)(xs + (buf * TN + nn) * C::LDX + e0) = xreg[decltype(P)::value][i];
            }
        }
    };
    auto do_tile = [&](int t, int buf, auto P) {
        typedef std::integral_constant<int, 1 - decltype(P)::value> Q;
        if (t + 2 * t_step < t_end) gload(t + 2 * t_step, P);
        const TX *xb = xs + buf * TN * C::LDX;
        float4_t acc[C::MT][C::NT];
#pragma unroll
        for (int mt = 0; mt < C::MT; ++mt)
#pragma unroll
            for (int nt = 0; nt < C::NT; ++nt) acc[mt][nt] = float4_t{0.f, 0.f, 0.f, 0.f};
        // B operand: lane (r, q) = inputs k = 16*ks + 4*q .. + 3 of batch row 16*nt + r, for this d_i
        half4_t xf[C::KS][C::NT];
#pragma unroll
        for (int ks = 0; ks < C::KS; ++ks)
#pragma unroll
            for (int nt = 0; nt < C::NT; ++nt)
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    xf[ks][nt][j] = row_to_half(AG ? xb[(16 * nt + r) * C::LDX + dd * CC + 16 * ks + 4 * q + j]
                                                   : xb[(16 * nt + r) * C::LDX + (16 * ks + 4 * q + j) * DD + dd]);
#pragma unroll
        for (int ks = 0; ks < C::KS; ++ks)
#pragma unroll
            for (int nt = 0; nt < C::NT; ++nt)
#pragma unroll
                for (int mt = 0; mt < C::MT; ++mt)
                    acc[mt][nt] = __builtin_amdgcn_mfma_f32_16x16x16f16(wreg[mt][ks], xf[ks][nt], acc[mt][nt], 0, 0, 0);
        // D: lane (r, q) holds batch row 16*nt + r, outputs m = 16*mt + 4*q + i
#pragma unroll
        for (int mt = 0; mt < C::MT; ++mt)
#pragma unroll
            for (int nt = 0; nt < C::NT; ++nt)
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    os[AG ? (16 * nt + r) * C::LDO + dd * BB + m_off + 16 * mt + 4 * q + i
                          : (16 * nt + r) * C::LDO + (m_off + 16 * mt + 4 * q + i) * DD + dd] = (half_t)epi_finish(ep, acc[mt][nt][i], bv[mt][i]);
        __syncthreads();
#pragma unroll
        for (int i = 0; i < C::O_PER_T; ++i) {
            const int v = tid + i * C::THREADS;
            if (C::O_VECS % C::THREADS == 0 || v < C::O_VECS) {
                const int nn = v / (C::OROW / 8), e0 = (v % (C::OROW / 8)) * 8;
                const int row = t * TN + nn;
                if (row < batch) {
                    const uint4_t o = *(const uint4_t *)(os + nn * C::LDO + e0);
                    __builtin_nontemporal_store(o, (uint4_t *)(yg + (size_t)row * out_size + row_off(e0)));
                }
            }
        }
        if (t + t_step < t_end) lstore(buf ^ 1, Q{});
        __syncthreads();
    };

    gload(t_begin, std::integral_constant<int, 0>{});
    if (t_begin + t_step < t_end) gload(t_begin + t_step, std::integral_constant<int, 1>{});
    lstore(0, std::integral_constant<int, 0>{});
    __syncthreads();
    for (int t = t_begin; t < t_end; t += 2 * t_step) {
        do_tile(t, 0, std::integral_constant<int, 0>{});
        if (t + t_step < t_end) do_tile(t + t_step, 1, std::integral_constant<int, 1>{});
    }
}


struct RowInst {
    int combo, bb, cc, dd, tn, lds;
    int vec;  // elements per 16-byte vector of the input
    int nt;   // streaming (nontemporal) output stores
    const void *fn;
    int planes;  // fp32: LDS tiles split into one plane per d_i
    int ms = 1;  // fp32: waves per d_i (row groups of a tall block)
    int ag = 0;  // d == 1: the waves take dd consecutive a_i
};
#define ROW_INST_PL(BB_, CC_, DD_, TN_) \
    {0, BB_, CC_, DD_, TN_, RowCfg<BB_, CC_, DD_, TN_, true>::LDS_BYTES, 4, 1, (const void *)ks_rows_bf_kernel<BB_, CC_, DD_, TN_, true, true>, 1}
#define ROW_INST(BB_, CC_, DD_, TN_, NT_) \
    {0, BB_, CC_, DD_, TN_, RowCfg<BB_, CC_, DD_, TN_>::LDS_BYTES, 4, NT_, (const void *)ks_rows_bf_kernel<BB_, CC_, DD_, TN_, NT_>}
 // two waves per d_i, each with half of the block's rows
#define ROW_INST_MS(BB_, CC_, DD_, TN_, MS_) \
    {0, BB_, CC_, DD_, TN_, RowCfg<BB_, CC_, DD_, TN_, false, MS_>::LDS_BYTES, 4, 1, \
     (const void *)ks_rows_bf_kernel<BB_, CC_, DD_, TN_, true, false, MS_>, 0, MS_}
// d == 1: groups of DD_ consecutive blocks
#define ROW_INST_AG(BB_, CC_, DD_, TN_) \
    {0, BB_, CC_, DD_, TN_, RowCfg<BB_, CC_, DD_, TN_>::LDS_BYTES, 4, 1, \
     (const void *)ks_rows_bf_kernel<BB_, CC_, DD_, TN_, true, false, 1, true>, 0, 1, 1}
#define ROW_INST_AG_H(BB_, CC_, DD_, TN_) \
    {1, BB_, CC_, DD_, TN_, RowCfgH<half_t, BB_, CC_, DD_, TN_>::LDS_BYTES, 8, 1, \
     (const void *)ks_rows_bf_h_kernel<half_t, BB_, CC_, DD_, TN_, true>, 0, 1, 1}
#define ROW_INST_AG_Q(BB_, CC_, DD_, TN_) \
    {2, BB_, CC_, DD_, TN_, RowCfgH<fp8_t, BB_, CC_, DD_, TN_>::LDS_BYTES, 16, 1, \
     (const void *)ks_rows_bf_h_kernel<fp8_t, BB_, CC_, DD_, TN_, true>, 0, 1, 1}
#define ROW_SET_AG(M) M(16, 16, 16, 32), M(16, 16, 16, 64), M(16, 16, 8, 64), M(16, 16, 4, 128), M(32, 32, 8, 32), M(32, 32, 4, 64), \
    M(16, 16, 2, 128), M(16, 16, 1, 128)
#define ROW_SET_AG32(M) M(16, 16, 16, 16), M(16, 16, 16, 32), M(16, 16, 8, 32), M(16, 16, 4, 64), M(32, 32, 8, 16), M(32, 32, 4, 32), \
    M(16, 16, 2, 64), M(16, 16, 1, 128)
// 16-bit: MS_ waves per d_i, each with BB_ / MS_ rows of the block
#define ROW_INST_H_MS(BB_, CC_, DD_, TN_, MS_) \
    {1, BB_, CC_, DD_, TN_, RowCfgH<half_t, BB_, CC_, DD_, TN_, MS_>::LDS_BYTES, 8, 1, \
     (const void *)ks_rows_bf_h_kernel<half_t, BB_, CC_, DD_, TN_, false, MS_>, 0, MS_}
#define ROW_INST_Q_MS(BB_, CC_, DD_, TN_, MS_) \
    {2, BB_, CC_, DD_, TN_, RowCfgH<fp8_t, BB_, CC_, DD_, TN_, MS_>::LDS_BYTES, 16, 1, \
     (const void *)ks_rows_bf_h_kernel<fp8_t, BB_, CC_, DD_, TN_, false, MS_>, 0, MS_}
#define ROW_SET_AG_B(M) \
    M(48, 48, 4, 32), M(48, 48, 2, 64), M(48, 48, 1, 64), M(64, 64, 4, 32), M(64, 64, 2, 64), M(64, 64, 4, 64), \
    M(96, 96, 2, 32), M(96, 96, 4, 16), M(64, 64, 1, 64), M(32, 32, 2, 64), M(32, 32, 1, 128)
#define ROW_SET_AG32_B(M) \
    M(48, 48, 4, 16), M(48, 48, 2, 32), M(48, 48, 1, 64), M(64, 64, 4, 16), M(64, 64, 2, 32), M(64, 64, 4, 32), \
    M(64, 64, 1, 64), M(32, 32, 2, 64), M(32, 32, 1, 64)
#define ROW_INST_H(BB_, CC_, DD_, TN_)                                                                      \
    {1, BB_, CC_, DD_, TN_, RowCfgH<half_t, BB_, CC_, DD_, TN_>::LDS_BYTES, 8, 1,                          \
     (const void *)ks_rows_bf_h_kernel<half_t, BB_, CC_, DD_, TN_>}
#define ROW_INST_Q(BB_, CC_, DD_, TN_)                                                                      \
    {2, BB_, CC_, DD_, TN_, RowCfgH<fp8_t, BB_, CC_, DD_, TN_>::LDS_BYTES, 16, 1,                          \
     (const void *)ks_rows_bf_h_kernel<fp8_t, BB_, CC_, DD_, TN_>}
#define ROW_SET_16(M) \
    M(48, 48, 16, 16), M(48, 48, 8, 32), M(48, 48, 4, 64), M(48, 48, 12, 32), \
    M(48, 48, 6, 32), M(48, 48, 3, 64), M(48, 48, 2, 64), M(64, 64, 16, 16), \
    M(64, 64, 8, 32), M(64, 64, 4, 64), M(64, 64, 12, 16), M(64, 64, 6, 32), \
    M(64, 64, 3, 64), M(64, 64, 2, 64), M(96, 96, 8, 16), M(96, 96, 4, 32), \
    M(96, 96, 3, 32), M(96, 96, 6, 16), M(96, 96, 2, 32), M(48, 192, 8, 16), \
    M(48, 192, 4, 32), M(48, 192, 2, 16), M(48, 192, 3, 32), M(48, 192, 6, 16), \
    M(192, 48, 2, 32), M(192, 48, 8, 16), M(192, 48, 4, 32), M(192, 48, 3, 32), \
    M(192, 48, 6, 16), M(32, 32, 4, 64), M(192, 48, 2, 64), M(16, 16, 16, 64), \
    M(32, 32, 16, 32), M(32, 32, 8, 64), M(128, 128, 4, 16), M(128, 128, 2, 32)
#define ROW_SET_16B(M) \
    M(48, 48, 2, 16), M(48, 48, 3, 16), M(48, 48, 4, 16), M(48, 48, 6, 16), M(48, 48, 8, 16), \
    M(64, 64, 2, 16), M(64, 64, 3, 16), M(64, 64, 4, 16), M(64, 64, 6, 16), M(64, 64, 8, 16), \
    M(96, 96, 2, 16), M(96, 96, 3, 16), M(96, 96, 4, 16), M(192, 48, 2, 16), M(192, 48, 3, 16), \
    M(192, 48, 4, 16), M(48, 192, 3, 16), M(48, 192, 4, 16)
#define ROW_SET_16C(M) M(128, 128, 3, 16), M(128, 128, 3, 32), M(16, 16, 4, 64), M(16, 16, 4, 128)
const RowInst row_insts[] = {
    ROW_INST(48, 48, 16, 16, true), ROW_INST(48, 48, 8, 32, true), ROW_INST(48, 48, 4, 64, true),
    ROW_INST(64, 64, 8, 16, true),  ROW_INST(64, 64, 4, 32, true), ROW_INST(16, 16, 16, 32, true),
    ROW_INST(16, 16, 4, 128, true), ROW_INST(32, 32, 8, 32, true), ROW_INST(48, 48, 16, 16, false),
    // more group sizes (d = DD, or a multiple of DD when DD is a multiple of 4) and block shapes
    ROW_INST(48, 48, 12, 16, true), ROW_INST(48, 48, 6, 32, true),  ROW_INST(48, 48, 3, 64, true),
    ROW_INST(48, 48, 2, 64, true),  ROW_INST(64, 64, 12, 16, true), ROW_INST(64, 64, 6, 16, true),
    ROW_INST(64, 64, 3, 32, true),  ROW_INST(64, 64, 2, 64, true),  ROW_INST(96, 96, 4, 16, true),
    ROW_INST(96, 96, 3, 32, true),   ROW_INST(48, 192, 4, 16, true),
    ROW_INST(48, 192, 3, 16, true), ROW_INST(48, 192, 2, 16, true), ROW_INST(192, 48, 4, 16, true),
    ROW_INST(192, 48, 3, 32, true), ROW_INST(32, 32, 16, 16, true),
    // fp16, then e4m3: the same shapes
    ROW_SET_16(ROW_INST_H),
    ROW_SET_16(ROW_INST_Q),
    // fp32 again (appended: the measured table refers to the indices above): small groups with
    // small tiles, more workgroups per CU
    ROW_INST(48, 48, 2, 16, true), ROW_INST(48, 48, 3, 16, true), ROW_INST(48, 48, 4, 16, true), ROW_INST(64, 64, 2, 16, true),
    ROW_INST(64, 64, 3, 16, true), ROW_INST(64, 64, 4, 16, true), ROW_INST(96, 96, 3, 16, true), ROW_INST(192, 48, 3, 16, true),
    ROW_INST(48, 48, 6, 16, true), ROW_INST(48, 48, 8, 16, true),
    // the same for fp16 and e4m3
    ROW_SET_16B(ROW_INST_H),
    ROW_SET_16B(ROW_INST_Q),
    // fp32 with one LDS plane per d_i (groups of 4, 8, 16)
    ROW_INST_PL(48, 48, 16, 16), ROW_INST_PL(48, 48, 8, 32), ROW_INST_PL(48, 48, 8, 16), ROW_INST_PL(48, 48, 4, 64),
    ROW_INST_PL(48, 48, 4, 16), ROW_INST_PL(64, 64, 8, 16), ROW_INST_PL(64, 64, 4, 32), ROW_INST_PL(64, 64, 4, 16),
    ROW_INST_PL(16, 16, 16, 32), ROW_INST_PL(16, 16, 4, 128), ROW_INST_PL(32, 32, 8, 32), ROW_INST_PL(32, 32, 16, 16),
    ROW_INST_PL(96, 96, 4, 16), ROW_INST_PL(48, 192, 4, 16), ROW_INST_PL(192, 48, 4, 16),
    // 16-bit: three 128 x 128 blocks per workgroup (the down factor (1,128,128,3) of the reference's
    // ViT-S feed-forward, scripts/2_benchmark_ksvit_time.sh:48-50, in its default layout), and
    // 16 x 16 blocks in groups of four
    ROW_SET_16C(ROW_INST_H),
    ROW_SET_16C(ROW_INST_Q),
    // fp32 128 x 128 blocks: two waves per d_i
    ROW_INST_MS(128, 128, 3, 16, 2),
    // d == 1, small blocks: groups of consecutive a_i
    ROW_SET_AG32(ROW_INST_AG),
    ROW_SET_AG(ROW_INST_AG_H),
    ROW_SET_AG(ROW_INST_AG_Q),
    ROW_SET_AG32_B(ROW_INST_AG),
    ROW_SET_AG_B(ROW_INST_AG_H),
    ROW_SET_AG_B(ROW_INST_AG_Q),
    // 16-bit 128 x 128 blocks, three per workgroup, several waves per block
    // ((1,128,128,3) at batch 25088, fp16: 24.0 us on one wave per block, 15.6 on four with 32-row
    // tiles, 18-19 on two; e4m3 33.4 -> 18.8)
    ROW_INST_H_MS(128, 128, 3, 32, 4), ROW_INST_H_MS(128, 128, 3, 32, 2), ROW_INST_H_MS(128, 128, 3, 16, 2),
    ROW_INST_H_MS(128, 128, 3, 16, 4),
    ROW_INST_Q_MS(128, 128, 3, 32, 4), ROW_INST_Q_MS(128, 128, 3, 32, 2), ROW_INST_Q_MS(128, 128, 3, 16, 2),
    ROW_INST_Q_MS(128, 128, 3, 16, 4),
    // the same for groups of 4 and 2 blocks
    ROW_INST_H_MS(128, 128, 4, 16, 4), ROW_INST_H_MS(128, 128, 4, 32, 4), ROW_INST_H_MS(128, 128, 2, 32, 4),
    ROW_INST_H_MS(128, 128, 2, 32, 8),
    ROW_INST_Q_MS(128, 128, 4, 16, 4), ROW_INST_Q_MS(128, 128, 4, 32, 4), ROW_INST_Q_MS(128, 128, 2, 32, 4),
    ROW_INST_Q_MS(128, 128, 2, 32, 8),
    // fp32 128 x 128 blocks on four waves per block
    ROW_INST_MS(128, 128, 3, 16, 4), ROW_INST_MS(128, 128, 3, 32, 4),
};
constexpr int N_ROW_INSTS = sizeof(row_insts) / sizeof(RowInst);
constexpr int ROW_INST_BITS = 10, ROW_INST_ANY = (1 << ROW_INST_BITS) - 1;
static_assert(N_ROW_INSTS < ROW_INST_ANY, "the variant's instance field must hold every index");

}  // namespace

int rows_inst_count() { return N_ROW_INSTS; }

uint32_t rows_inst_id(int i)
{
    if (i < 0 || i >= N_ROW_INSTS) return 0;
    const RowInst &t = row_insts[i];
    const int v[9] = {t.combo, t.bb, t.cc, t.dd, t.tn, t.nt, t.planes, t.ms, t.ag};
    return inst_hash('R', v, t.ag ? 9 : t.ms > 1 ? 8 : t.planes ? 7 : 6);  // (ids of the other instances predate the fields)
}

// variant: bits 0-9 instance (all ones: first that fits), bits 10.. workgroups per a_i (0: heuristic)
int rows_bf_run(const Problem &p, int variant, bool launch, ksmm_tile *tile)
{
    const int combo = combo_of(p.x_dtype, p.w_dtype, p.y_dtype);
    if (p.bs_last || combo < 0 || combo > 2) return KSMM_ERR_BAD_ALGO;
    const int want = variant < 0 ? ROW_INST_ANY : (variant & ROW_INST_ANY);
    int64_t wgs = variant < 0 ? 0 : (variant >> ROW_INST_BITS);
    if (want != ROW_INST_ANY && want >= N_ROW_INSTS) return KSMM_ERR_BAD_ALGO;
    int pick = -1;
    for (int i = 0; i < N_ROW_INSTS; ++i) {
        if (want != ROW_INST_ANY && want != i) continue;
        const RowInst &t = row_insts[i];
        if (t.combo != combo || t.bb != p.b || t.cc != p.c) continue;
        if (want == ROW_INST_ANY && t.planes) continue;  // named by the table (or forced) only
        // 16-bit groups of 2 and 4 blocks on several waves per block: no faster than one wave per
        // block (fp16 (16,128,128,2) 150 against 138 us, (4,128,128,4) 78 against 70), named only
        if (want == ROW_INST_ANY && t.ms > 1 && combo != 0 && t.dd != 3) continue;
        // row segments start on 16-byte boundaries (output vectors: 4 floats / 8 halves)
        const int ovec = combo == 0 ? 4 : 8;
        if (((int64_t)p.a * p.c * p.d) % t.vec || ((int64_t)p.a * p.b * p.d) % ovec) continue;
        if (t.ag) {
            // d == 1: dd consecutive blocks per workgroup; the largest group that divides a (the
            // smallest tile among equals: more workgroups)
            if (p.d != 1 || p.a % t.dd) continue;
            // blocks up to 48 x 48 always; 64 x 64 in groups of four for fp32 and e4m3 and 96 x 96
            // for fp16 (measured against the tile and stream kernels these shapes had: fp32
            // (12,64,64,1) 53 -> 46 us, fp16 (8,96,96,1) 27 -> 20 us, fp32 (16,48,48,1) 122 -> 38 us;
            // fp16 64 x 64 stays on the stream kernel, 15 against 19 us); the rest when named
            const bool take = t.bb * t.cc <= 48 * 48 || (t.bb == 64 && t.cc == 64 && t.dd == 4 && combo != 1) ||
                              (t.bb == 96 && t.cc == 96 && combo == 1);
            if (want == ROW_INST_ANY && !take) continue;
            if (want != ROW_INST_ANY) {
                pick = i;
                break;
            }
            if (pick < 0 || t.dd > row_insts[pick].dd) pick = i;
            continue;
        }
        if (p.d == 1) continue;
        // 96 x 96 blocks and larger with d a multiple of 16 from 32 on (fp32) or of 32 from 64 on
        // (16-bit input): the tile kernel's groups of 16 / 32 blocks are faster at large batches
        // (fp32 (a,96,96,64) 0.64-0.82 of this kernel's time at batch 25088, (1,96,96,96) 0.61; fp16
        // (12,96,96,64) 0.68)
        // (within what that kernel takes before the transposed route: b * d <= 8192 in fp32, d <= 128)
        if (want == ROW_INST_ANY && t.bb >= 96 && t.bb <= 192 && t.cc >= 96 && t.cc <= 256 && p.batch >= 8192 &&
            (combo == 0 ? p.d >= 32 && p.d % 16 == 0 && (int64_t)p.b * p.d <= 8192
                        : p.d >= 64 && p.d % 32 == 0 && p.d <= 128))
            continue;
        // all d blocks in one workgroup, or groups of dd whose runs keep the 16-byte alignment
        const bool grouped_ok = t.dd % t.vec == 0 && t.dd % ovec == 0 && p.d % t.dd == 0;
        const int run_bytes = t.dd * (combo == 0 ? 4 : 2);  // output run of a group
        if (want != ROW_INST_ANY) {
            if (t.dd == p.d || grouped_ok) pick = i;
            break;
        }
        if (t.dd == p.d) {
            // all d blocks in one workgroup: the smallest batch tile (more workgroups per CU;
            // measured 10-55 % faster than the 32- and 64-row tiles for d <= 8), except for
            // 128 x 128 blocks, whose weights take longer to read than a small tile to multiply
            // ((1,128,128,3) at batch 25088: fp16 28.8 us with 16 rows, 23.9 with 32; e4m3 42.2 / 33.3)
            // (and more waves per block before larger tiles: 15.6 us on four waves per block)
            const bool larger = t.bb * t.cc >= 128 * 128;
            const RowInst *cur = pick >= 0 ? &row_insts[pick] : nullptr;
            // (then tiles that leave room for two workgroups' worth of LDS, then the larger tile:
            // fp32 on four waves per block 34.0 us with 16-row tiles, 45.8 with 32-row ones)
            auto rank = [](const RowInst &q) { return q.ms * 1000 + (q.lds <= 80 * 1024 ? 500 : 0) + q.tn; };
            if (!cur || cur->dd != p.d || (larger ? rank(t) > rank(*cur) : t.tn < cur->tn)) pick = i;
        } else if (pick >= 0 && row_insts[pick].dd == p.d) {
            // an exact match was found already
        } else if (grouped_ok && (run_bytes >= 32 || (combo == 0 && p.b <= p.c)) &&
                   (pick < 0 || t.dd > row_insts[pick].dd)) {
            // the largest group that divides d, unless an exact match follows; 16-byte runs
            // only for fp32 (groups of 4) where the output is not the larger side
            pick = i;
        }
    }
    if (pick < 0) return KSMM_ERR_BAD_ALGO;
    const RowInst &t = row_insts[pick];
    const int64_t n_tiles = (p.batch + t.tn - 1) / t.tn;
    const int64_t ag = t.ag ? p.a / t.dd : (int64_t)p.a * (p.d / t.dd);  // (a_i, group) pairs
    // one round of workgroups, 8 or more waves per CU
    const int nw = t.dd * t.ms;
    const int per_cu_lds = 160 * 1024 / t.lds, per_cu_waves = 16 / nw > 0 ? 16 / nw : 1;
    // (rounded down: a few workgroups beyond one round would cost a whole second round)
    if (wgs <= 0) {
        const int64_t round = 256 * (per_cu_lds < per_cu_waves ? per_cu_lds : per_cu_waves);
        wgs = round / ag;
        // the grid below is 8 * groups * ceil(a * wgs / 8) workgroups: keep that within the round too
        const int64_t groups = t.ag ? 1 : p.d / t.dd, units = 8 * (round / (8 * groups));
        if (!t.ag && units >= p.a && wgs > units / p.a) wgs = units / p.a;
    }
    if (wgs <= 0) wgs = 1;
    if (wgs > n_tiles) wgs = n_tiles;
    // (groups of one a_i that take the same tiles sit 8 block indices apart: see the kernels)
    const int64_t grid = t.ag ? ag * wgs : 8 * (int64_t)(p.d / t.dd) * (((int64_t)p.a * wgs + 7) / 8);
    if (grid > 0x7fffffffLL) return KSMM_ERR_TOO_LARGE;
    if (tile) {
        tile->algo = KSMM_ALGO_WAVE;
        tile->variant = 1000 + pick;
        tile->tile_m = t.bb;
        tile->tile_n = t.tn;
        tile->tile_k = t.cc;
        tile->tile_d = t.dd;
        tile->threads = 64 * nw;
        tile->lds_bytes = t.lds;
        tile->grid = grid;
    }
    if (!launch) return KSMM_OK;
    if (ensure_dynamic_lds(t.fn, t.lds) != KSMM_OK) return KSMM_ERR_LAUNCH;
    int batch_i = (int)p.batch, wgs_i = (int)wgs, n_tiles_i = (int)n_tiles;
    Epi ep = epi_of(p);
    void *args[] = {(void *)&p.x, (void *)&p.w, (void *)&p.y, &batch_i, (void *)&p.a, (void *)&p.d,
                    &ep, &wgs_i, &n_tiles_i};
    hipError_t e = hipLaunchKernel(t.fn, dim3((unsigned)grid), dim3(64 * nw), args, t.lds, p.stream);
    return e == hipSuccess ? KSMM_OK : KSMM_ERR_LAUNCH;
}

}  // namespace ksmm
