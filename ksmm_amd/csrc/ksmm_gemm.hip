// "GEMM" kernels of the tile family: the matrix-core-bound path for large b x c blocks.
//
// Same decomposition as the plain tile kernel (a workgroup computes a TM x TN tile of one
// (a_i, d_i) block, looping over c in slabs of TK), rebuilt around the two things that limited
// it: (1) the global loads of a slab were only one slab (~0.4 us of MFMA work) ahead, far less
// than the memory latency, and (2) staging registers.  Here both operands go straight to LDS
// with direct-to-LDS loads (global_load_lds_dwordx4) into a ring of ST slabs, so ST-1 slabs are
// in flight while one is multiplied; the waits are hand-counted s_waitcnt vmcnt(N) (the loop
// issues a fixed number of loads per slab and nothing else touches the counter).  Tiles are
// stored unpadded with an XOR swizzle of the 16-byte chunk index (direct-to-LDS loads write
// 64 consecutive chunks per wave instruction).  One barrier per slab.
//
// A wave computes up to 4 x 4 MFMA tiles of 32 x 32 (256 accumulator registers), which keeps
// the LDS operand traffic at half of what the LDS can deliver while the matrix cores run.
//
// The axis that is contiguous in the output runs along the MFMA rows, so that a lane holds 4
// consecutive output elements and the output tile can be transposed through LDS cheaply:
//   bs_last          : A = X (rows = batch),   B = W (lanes = outputs), any d
//   bs_first, d == 1 : A = W (rows = outputs), B = X (lanes = batch)
//   bs_first, d == 2 : as d == 1, but one workgroup computes both d_i blocks: an input row
//                      holds (k, d_i) pairs interleaved; each lane reads 16 consecutive halves
//                      and splits them into the two MFMA operands with 8 v_perm; the results
//                      of the two blocks are interleaved again in the output tile.
//
// Reference counterpart: kernel_bs_{first,last}_{float,half2,half4}
// (src/ksmm_py/layer/kronecker_sparse/template_kernels_float.cuh:85-491,
//  template_kernels_half.cuh:103-1092).
#include "ksmm_mfma.h"

#ifdef KSMM_PROFILE
// Phase timestamps of wave 0 of the first workgroups (standalone profiling builds only).
__device__ unsigned long long ksmm_gprof[256][64];
#define KG_STAMP(slot)                                                                    \
    do {                                                                                  \
        if (threadIdx.x == 0 && blockIdx.x < 256 && (slot) < 64)                          \
            ksmm_gprof[blockIdx.x][(slot)] = __builtin_amdgcn_s_memtime();                \
    } while (0)
#else
#define KG_STAMP(slot) do { } while (0)
#endif

namespace ksmm {

namespace {

constexpr int vmcnt_imm(int n) { return (n & 15) | (7 << 4) | (15 << 8) | (((n >> 4) & 3) << 14); }

__device__ __forceinline__ void dma16(const void *gptr, uint32_t lds_addr)
{
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off"
                 :
                 : "v"(gptr), "s"(lds_addr)
                 : "memory", "m0");
}

// Stage geometry.  W tile(s): DD x [TK][TM] k-outer.  X tile: bs_last [TK][TN] k-outer;
// bs_first [TN][TK*DD] k-inner (d_i interleaved when DD == 2).
template <typename CT, bool BS_LAST, int DD, int TM, int TN, int TK, int WM, int WN, int ST> struct GemmCfg {
    static constexpr int THREADS = 64 * WM * WN;
    static constexpr int ES = (int)sizeof(CT), EPC = 16 / ES;
    static constexpr int KSTEP = compute<CT>::KSTEP;
    static constexpr int MT = TM / WM / 32, NT = TN / WN / 32;
    static constexpr int W_CPR = TM / EPC;  // chunks per weight row
    static constexpr int X_CPR = BS_LAST ? TN / EPC : TK * DD / EPC;
    static constexpr int X_ROWS = BS_LAST ? TK : TN;
    static constexpr int W_CHUNKS = DD * TK * W_CPR, X_CHUNKS = X_ROWS * X_CPR;
    static constexpr int LW = W_CHUNKS / THREADS, LX = X_CHUNKS / THREADS, L = LW + LX;
    static constexpr int W_BYTES = W_CHUNKS * 16, X_BYTES = X_CHUNKS * 16, STAGE_BYTES = W_BYTES + X_BYTES;
    static constexpr int LDS_BYTES = ST * STAGE_BYTES;
    static constexpr int N_WAIT = (ST - 2) * L;
    static_assert(!BS_LAST || DD == 1, "DD > 1 is a batch-size-first variant");
    static_assert(ES == 2 || BS_LAST, "fp32 batch-size-first uses the plain tile kernel");
    static_assert(TM % (32 * WM) == 0 && TN % (32 * WN) == 0 && TK % KSTEP == 0, "wave tiling");
    static_assert(W_CHUNKS % THREADS == 0 && X_CHUNKS % THREADS == 0, "every wave issues L loads per slab");
    static_assert(W_CPR % (ES == 2 ? 8 : 16) == 0, "weight swizzle group");
    static_assert(BS_LAST ? X_CPR % (ES == 2 ? 8 : 16) == 0 : (X_CPR == 4 || X_CPR % 8 == 0), "input swizzle group");
    static_assert(ST >= 2 && N_WAIT <= 63 && LDS_BYTES <= 160 * 1024, "ring");
    static_assert(DD * MT * NT * 16 <= 256, "accumulators");
};

// chunk swizzles (applied to the global address a lane fetches and by the operand reads)
template <typename CT> __device__ __forceinline__ int swz_outer(int row) { return sizeof(CT) == 2 ? 2 * (row & 3) : 8 * (row & 1); }
template <int CPR> __device__ __forceinline__ int swz_inner(int row) { return CPR == 4 ? ((row >> 2) & 3) : (row & 7); }

// k-outer operand (weights always, input for bs_last): S[k][idx], row of COLS elements
template <typename CT, int COLS> struct outer_frag;
template <int COLS> struct outer_frag<half_t, COLS> {
    __device__ static __forceinline__ half8_t get(const half_t *s, int idx0, int k0, int lane)
    {
        const int kq = lane >> 5, i16 = lane & 15, hs = (lane >> 4) & 1;
        const int row = k0 + 8 * kq + (i16 >> 2);
        const int chunk = (idx0 >> 3) + 2 * hs + ((i16 & 3) >> 1);
        const half_t *p = s + row * COLS + ((chunk ^ (2 * ((i16 >> 2) & 3))) << 3) + 4 * (i16 & 1);
        typedef short4_t __attribute__((address_space(3))) * lds_ptr;
        short4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(p));
        short4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(p + 4 * COLS));
        typedef short short8_t __attribute__((ext_vector_type(8)));
        short8_t r = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
        return __builtin_bit_cast(half8_t, r);
    }
};
template <int COLS> struct outer_frag<float, COLS> {
    __device__ static __forceinline__ float get(const float *s, int idx0, int k0, int lane)
    {
        const int row = k0 + (lane >> 5), col = idx0 + (lane & 31);
        return s[row * COLS + ((((col >> 2) ^ (8 * (row & 1))) << 2) | (col & 3))];
    }
};

template <typename CT, typename TY, bool BS_LAST, int DD, int TM, int TN, int TK, int WM, int WN, int ST, int OCC>
__global__ __launch_bounds__(64 * WM * WN, OCC) void ks_gemm_kernel(const CT *__restrict__ x,
                                                              const CT *__restrict__ w,
                                                              TY *__restrict__ y, int batch, int a,
                                                              int b, int c, int d, float scale,
                                                              int m_tiles, int n_tiles, int blocks)
{
    typedef GemmCfg<CT, BS_LAST, DD, TM, TN, TK, WM, WN, ST> C;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    // XCD-aware id: TM-tiles of one input tile get consecutive logical ids on one XCD
    const int per_xcd = (blocks + 7) / 8;
    const int lid = (blockIdx.x % 8) * per_xcd + blockIdx.x / 8;
    if (lid >= blocks) return;
    const int mt_id = lid % m_tiles;
    const int rest = lid / m_tiles;
    const int nt_id = rest % n_tiles;
    const int g = rest / n_tiles;  // bs_last / d == 1: a_i * d + d_i;  DD == 2: a_i
    const int a_i = DD == 1 ? g / d : g, d_i = DD == 1 ? g - a_i * d : 0;
    const int m0 = mt_id * TM, n0 = nt_id * TN;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave / WN, wn = wave % WN;
    const size_t in_size = (size_t)a * c * d, out_size = (size_t)a * b * d;

    // ---- per-lane global addresses of the loads of one slab (k0 = 0) ----------------------
    const CT *wptr[C::LW];
    const CT *xptr[C::LX];
#pragma unroll
    for (int i = 0; i < C::LW; ++i) {
        const int q = tid + i * C::THREADS;
        const int dd = q / (TK * C::W_CPR), r = q % (TK * C::W_CPR);
        const int row = r / C::W_CPR, pc = r % C::W_CPR;
        const int col = (pc ^ swz_outer<CT>(row)) * C::EPC;
        const int blk = DD == 1 ? g : a_i * DD + dd;
        wptr[i] = w + ((size_t)blk * c + row) * b + m0 + col;
    }
#pragma unroll
    for (int i = 0; i < C::LX; ++i) {
        const int q = tid + i * C::THREADS;
        const int row = q / C::X_CPR, pc = q % C::X_CPR;
        if (BS_LAST) {
            const int col = (pc ^ swz_outer<CT>(row)) * C::EPC;
            xptr[i] = x + ((size_t)(a_i * c + row) * d + d_i) * batch + min(n0 + col, batch - C::EPC);
        } else {
            const int col = (pc ^ swz_inner<C::X_CPR>(row)) * C::EPC;
            xptr[i] = x + (size_t)min(n0 + row, batch - 1) * in_size + (size_t)a_i * c * DD + col;
        }
    }
    const size_t w_step = (size_t)TK * b;                                   // elements per slab
    const size_t x_step = BS_LAST ? (size_t)TK * d * batch : (size_t)TK * DD;
    const uint32_t lds_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char *)smem;
    auto issue = [&](int step, int stg) {
        const uint32_t dst = lds_base + stg * C::STAGE_BYTES + wave * 1024;
#pragma unroll
        for (int i = 0; i < C::LW; ++i) dma16(wptr[i] + step * w_step, dst + i * (C::THREADS * 16));
#pragma unroll
        for (int i = 0; i < C::LX; ++i)
            dma16(xptr[i] + step * x_step, dst + C::W_BYTES + i * (C::THREADS * 16));
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
    KG_STAMP(0);
#pragma unroll
    for (int p = 0; p < ST - 1; ++p) issue(min(p, steps - 1), p);
    KG_STAMP(1);

    // MFMA operands of sub-step k0 of the current slab
    typedef typename frag<CT>::type frag_t;
    auto load_frags = [&](const CT *wb, const CT *xb, int k0, frag_t(&fw)[DD][C::MT], frag_t(&fx)[DD][C::NT]) {
#pragma unroll
        for (int dd = 0; dd < DD; ++dd)
#pragma unroll
            for (int i = 0; i < C::MT; ++i)
                fw[dd][i] = outer_frag<CT, TM>::get(wb + dd * TK * TM, (wm * C::MT + i) * 32, k0, lane);
#pragma unroll
        for (int j = 0; j < C::NT; ++j) {
            const int idx0 = (wn * C::NT + j) * 32;
            if constexpr (BS_LAST) {
                fx[0][j] = outer_frag<CT, TN>::get(xb, idx0, k0, lane);
            } else if constexpr (DD == 1) {
                const int row = idx0 + (lane & 31), chunk = (k0 >> 3) + (lane >> 5);
                fx[0][j] = *(const half8_t *)(xb + row * (TK * DD) + ((chunk ^ swz_inner<C::X_CPR>(row)) << 3));
            } else {
                // 16 consecutive halves = 8 (k, d_i) pairs -> one operand per d_i
                const int row = idx0 + (lane & 31), chunk = 2 * ((k0 >> 3) + (lane >> 5));
                const int sw = swz_inner<C::X_CPR>(row);
                const uint4_t lo = *(const uint4_t *)(xb + row * (TK * DD) + ((chunk ^ sw) << 3));
                const uint4_t hi = *(const uint4_t *)(xb + row * (TK * DD) + (((chunk + 1) ^ sw) << 3));
                uint4_t e, o;
                e[0] = __builtin_amdgcn_perm(lo[1], lo[0], 0x05040100u);
                e[1] = __builtin_amdgcn_perm(lo[3], lo[2], 0x05040100u);
                e[2] = __builtin_amdgcn_perm(hi[1], hi[0], 0x05040100u);
                e[3] = __builtin_amdgcn_perm(hi[3], hi[2], 0x05040100u);
                o[0] = __builtin_amdgcn_perm(lo[1], lo[0], 0x07060302u);
                o[1] = __builtin_amdgcn_perm(lo[3], lo[2], 0x07060302u);
                o[2] = __builtin_amdgcn_perm(hi[1], hi[0], 0x07060302u);
                o[3] = __builtin_amdgcn_perm(hi[3], hi[2], 0x07060302u);
                fx[0][j] = __builtin_bit_cast(half8_t, e);
                fx[DD - 1][j] = __builtin_bit_cast(half8_t, o);
            }
        }
    };
    constexpr int K0 = TK / C::KSTEP;                  // MFMA sub-steps per slab
    constexpr int PER_K0 = DD * C::MT * C::NT;         // MFMAs per sub-step
    constexpr int STRIDE = (K0 * PER_K0) / C::L > 0 ? (K0 * PER_K0) / C::L : 1;  // MFMAs per load issued

    for (int it = 0; it < steps; ++it) {
        // slab `it` was requested ST-1 iterations ago; (ST-2)*L newer loads may stay in flight.
        // Near the end the ring holds repeats of the last slab, so the count stays constant.
        __builtin_amdgcn_s_waitcnt(vmcnt_imm(C::N_WAIT));
        KG_STAMP(4 + 4 * it);
        __syncthreads();  // slab `it` landed for every wave, and everyone left slab it-1
        KG_STAMP(5 + 4 * it);
        const CT *wb = (const CT *)(smem + (it % ST) * C::STAGE_BYTES);
        const CT *xb = (const CT *)(smem + (it % ST) * C::STAGE_BYTES + C::W_BYTES);
        // The L loads of slab it+ST-1 are spread between the MFMAs of this slab (the path into
        // LDS moves 64 bytes per clock and CU: issued in one burst it would stall the wave for
        // about half a slab), and the operands of sub-step k0+1 are read while k0 multiplies.
        const int nstep = min(it + ST - 1, steps - 1);
        const size_t w_off = (size_t)nstep * w_step, x_off = (size_t)nstep * x_step;
        const uint32_t dst = lds_base + ((it + ST - 1) % ST) * C::STAGE_BYTES + wave * 1024;
        frag_t fw[2][DD][C::MT], fx[2][DD][C::NT];
        load_frags(wb, xb, 0, fw[0], fx[0]);
        KG_STAMP(6 + 4 * it);
#pragma unroll
        for (int kk = 0; kk < K0; ++kk) {
            if (kk + 1 < K0) load_frags(wb, xb, (kk + 1) * C::KSTEP, fw[(kk + 1) & 1], fx[(kk + 1) & 1]);
#pragma unroll
            for (int dd = 0; dd < DD; ++dd)
#pragma unroll
                for (int i = 0; i < C::MT; ++i)
#pragma unroll
                    for (int j = 0; j < C::NT; ++j) {
                        acc[dd][i][j] = BS_LAST ? frag<CT>::mfma(fx[kk & 1][dd][j], fw[kk & 1][dd][i], acc[dd][i][j])
                                                : frag<CT>::mfma(fw[kk & 1][dd][i], fx[kk & 1][dd][j], acc[dd][i][j]);
                        const int m = kk * PER_K0 + (dd * C::MT + i) * C::NT + j;  // MFMA index in the slab
                        if ((m + 1) % STRIDE == 0 && m / STRIDE < C::L) {
                            const int q = m / STRIDE;  // load index
                            if (q < C::LW)
                                dma16(wptr[q < C::LW ? q : 0] + w_off, dst + q * (C::THREADS * 16));
                            else
                                dma16(xptr[q >= C::LW ? q - C::LW : 0] + x_off,
                                      dst + C::W_BYTES + (q - C::LW) * (C::THREADS * 16));
                            __builtin_amdgcn_sched_barrier(0);
                        }
                    }
        }
        // loads that did not get a slot above (fewer MFMAs than loads)
#pragma unroll
        for (int q = (K0 * PER_K0) / STRIDE; q < C::L; ++q) {
            if (q < C::LW)
                dma16(wptr[q < C::LW ? q : 0] + w_off, dst + q * (C::THREADS * 16));
            else
                dma16(xptr[q >= C::LW ? q - C::LW : 0] + x_off, dst + C::W_BYTES + (q - C::LW) * (C::THREADS * 16));
        }
    }
    KG_STAMP(2);
    __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));  // repeats of the last slab must land before LDS is released

    __syncthreads();  // every wave is done with the operand ring: LDS becomes the output tile
    // Epilogue: the accumulators are transposed through LDS so that global memory sees 16-byte
    // stores along the contiguous axis.  The MFMA rows run along that axis (bs_last: batch,
    // bs_first: outputs), so a lane holds 4 consecutive elements of it per 8-row group:
    //   bs_last : out[m][n..n+3]                       row = TN elements
    //   bs_first: out[n][(m..m+3) x d_i interleaved]   row = TM*DD elements
    // The tile is written in passes of as many rows as fit in the LDS of the ring.
    {
        constexpr int RC = (BS_LAST ? TN : TM * DD) + C::EPC;  // padded row, elements
        constexpr int LR = BS_LAST ? TM : TN;                   // rows of the whole tile
        constexpr int RPP_RAW = C::LDS_BYTES / (RC * C::ES) / 32 * 32;
        constexpr int RPP = RPP_RAW > LR ? LR : RPP_RAW;        // rows per pass (multiple of 32)
        constexpr int PASSES = (LR + RPP - 1) / RPP;
        constexpr int CPR = (RC - C::EPC) / C::EPC;             // 16-byte chunks per row
        static_assert(RPP >= 32, "output pass");
        TY *const out = (TY *)smem;
        const int l32 = lane & 31, lq = lane >> 5;
#pragma unroll
        for (int pass = 0; pass < PASSES; ++pass) {
            if (pass > 0) __syncthreads();
#pragma unroll
            for (int i = 0; i < C::MT; ++i)
#pragma unroll
                for (int j = 0; j < C::NT; ++j) {
                    const int mb = (wm * C::MT + i) * 32, nb = (wn * C::NT + j) * 32;
                    const int lrow = (BS_LAST ? mb : nb) + l32;      // row of the tile this lane writes
                    const int rcol = (BS_LAST ? nb : mb) + 4 * lq;  // + 8 * eg: 4 consecutive elements
                    if (lrow / RPP != pass) continue;               // uniform per wave (32-row tiles)
                    TY *dst = out + (lrow - pass * RPP) * RC;
#pragma unroll
                    for (int eg = 0; eg < 4; ++eg) {
                        if constexpr (sizeof(TY) == 4) {
                            float4_t v = {acc[0][i][j][4 * eg] * scale, acc[0][i][j][4 * eg + 1] * scale,
                                          acc[0][i][j][4 * eg + 2] * scale, acc[0][i][j][4 * eg + 3] * scale};
                            *(float4_t *)(dst + rcol + 8 * eg) = v;
                        } else if constexpr (DD == 1) {
                            half4_t v = {(half_t)(acc[0][i][j][4 * eg] * scale), (half_t)(acc[0][i][j][4 * eg + 1] * scale),
                                         (half_t)(acc[0][i][j][4 * eg + 2] * scale), (half_t)(acc[0][i][j][4 * eg + 3] * scale)};
                            *(half4_t *)(dst + rcol + 8 * eg) = v;
                        } else {
                            half8_t v;
#pragma unroll
                            for (int u = 0; u < 4; ++u) {
                                v[2 * u] = (half_t)(acc[0][i][j][4 * eg + u] * scale);
                                v[2 * u + 1] = (half_t)(acc[DD - 1][i][j][4 * eg + u] * scale);
                            }
                            *(half8_t *)(dst + (rcol + 8 * eg) * DD) = v;
                        }
                    }
                }
            __syncthreads();
            for (int q = tid; q < RPP * CPR; q += C::THREADS) {
                const int r = q / CPR, cc = (q % CPR) * C::EPC;
                const int row = pass * RPP + r;  // row of the tile
                if (row >= LR) break;
                const uint4_t v = *(const uint4_t *)(out + r * RC + cc);
                if constexpr (BS_LAST) {
                    const int n = n0 + cc;
                    if (n < batch)
                        *(uint4_t *)(y + ((size_t)(a_i * b + m0 + row) * d + d_i) * batch + n) = v;
                } else {
                    const int n = n0 + row;
                    if (n < batch)
                        *(uint4_t *)(y + (size_t)n * out_size + ((size_t)a_i * b + m0) * DD + cc) = v;
                }
            }
        }
    }
    KG_STAMP(3);
}

struct GemmInst {
    int combo, bs_last, dd, tm, tn, tk, threads, lds, epc;
    const void *fn;
};
// OCC_: waves per SIMD the register allocation must allow (2 lets two workgroups share a CU,
// so that one multiplies while the other stores its output tile)
#define GEMM_INST_O(COMBO_, CT_, BL_, DD_, TM_, TN_, TK_, WM_, WN_, ST_, OCC_)                        \
    {COMBO_, BL_, DD_, TM_, TN_, TK_, 64 * WM_ * WN_,                                                \
     GemmCfg<CT_, BL_, DD_, TM_, TN_, TK_, WM_, WN_, ST_>::LDS_BYTES,                                 \
     GemmCfg<CT_, BL_, DD_, TM_, TN_, TK_, WM_, WN_, ST_>::EPC,                                       \
     (const void *)ks_gemm_kernel<CT_, CT_, BL_, DD_, TM_, TN_, TK_, WM_, WN_, ST_, OCC_>}
#define GEMM_INST(COMBO_, CT_, BL_, DD_, TM_, TN_, TK_, WM_, WN_, ST_)                                \
    GEMM_INST_O(COMBO_, CT_, BL_, DD_, TM_, TN_, TK_, WM_, WN_, ST_, 1)
// The first instance that fits (and still yields >= 256 workgroups) is the default; the order
// comes from sweeps on (1,1536,384,2) fp16 and (1,768,192,2) fp32 at batch 25088.
const GemmInst gemm_insts[] = {
    // fp16, bs_first, d == 2
    GEMM_INST(1, half_t, false, 2, 256, 128, 32, 4, 2, 3),
    GEMM_INST(1, half_t, false, 2, 128, 256, 32, 2, 4, 3),
    GEMM_INST_O(1, half_t, false, 2, 128, 128, 32, 2, 2, 2, 2),
    GEMM_INST(1, half_t, false, 2, 128, 256, 32, 2, 2, 3),
    GEMM_INST(1, half_t, false, 2, 64, 256, 32, 1, 4, 3),
    // fp16, bs_last
    GEMM_INST(1, half_t, true, 1, 256, 256, 32, 2, 4, 4),
    GEMM_INST_O(1, half_t, true, 1, 128, 256, 32, 2, 2, 3, 2),
    GEMM_INST(1, half_t, true, 1, 256, 256, 32, 2, 2, 4),
    GEMM_INST(1, half_t, true, 1, 128, 128, 32, 2, 2, 4),
    // fp16, bs_first, d == 1
    GEMM_INST(1, half_t, false, 1, 256, 256, 32, 2, 4, 4),
    GEMM_INST_O(1, half_t, false, 1, 256, 128, 32, 2, 2, 3, 2),
    GEMM_INST(1, half_t, false, 1, 256, 256, 32, 2, 2, 4),
    GEMM_INST(1, half_t, false, 1, 128, 128, 32, 2, 2, 4),
    // fp32, bs_last
    GEMM_INST_O(0, float, true, 1, 128, 256, 16, 2, 2, 3, 2),
    GEMM_INST(0, float, true, 1, 128, 128, 16, 2, 2, 4),
    GEMM_INST(0, float, true, 1, 256, 256, 16, 2, 2, 4),
    GEMM_INST(0, float, true, 1, 64, 256, 16, 1, 4, 4),
};
constexpr int N_GEMM_INSTS = sizeof(gemm_insts) / sizeof(GemmInst);

bool gemm_fits(const GemmInst &t, const Problem &p, int combo)
{
    if (t.combo != combo || t.bs_last != p.bs_last) return false;
    if (p.b % t.tm || p.c % t.tk) return false;
    if (p.b % t.epc) return false;  // 16-byte weight vectors
    if (p.bs_last) {
        if (p.batch % t.epc || p.batch < t.epc) return false;
    } else {
        if (p.d != t.dd) return false;
        if (((int64_t)p.a * p.c * p.d) % t.epc || ((int64_t)p.c * p.d) % t.epc) return false;
        if (t.dd == 2 && (((int64_t)p.a * p.b * p.d) % 2)) return false;
    }
    return true;
}

}  // namespace

// variant: index into the instance table (-1: first that fits with enough workgroups)
int gemm_run(const Problem &p, int variant, bool launch, ksmm_tile *tile)
{
    const int combo = combo_of(p.x_dtype, p.w_dtype, p.y_dtype);
    int pick = -1;
    for (int i = 0; i < N_GEMM_INSTS; ++i) {
        if (variant >= 0 && variant != i) continue;
        const GemmInst &t = gemm_insts[i];
        if (!gemm_fits(t, p, combo)) continue;
        if (variant < 0) {
            // the big tiles only pay when they still fill the chip
            const int64_t groups = t.dd == 1 ? (int64_t)p.a * p.d : p.a;
            const int64_t wgs = groups * (p.b / t.tm) * ((p.batch + t.tn - 1) / t.tn);
            if (wgs < 256) continue;
        }
        pick = i;
        break;
    }
    if (pick < 0) return KSMM_ERR_BAD_ALGO;
    const GemmInst &t = gemm_insts[pick];
    const int m_tiles = p.b / t.tm;
    const int64_t n_tiles = (p.batch + t.tn - 1) / t.tn;
    const int64_t groups = t.dd == 1 ? (int64_t)p.a * p.d : p.a;
    const int64_t blocks = groups * m_tiles * n_tiles;
    const int64_t grid = (blocks + 7) / 8 * 8;
    if (grid > 0x7fffffffLL) return KSMM_ERR_TOO_LARGE;
    if (tile) {
        tile->algo = KSMM_ALGO_TILE;
        tile->variant = (4 << 24) | pick;
        tile->tile_m = t.tm;
        tile->tile_n = t.tn;
        tile->tile_k = t.tk;
        tile->tile_d = t.dd;
        tile->threads = t.threads;
        tile->lds_bytes = t.lds;
        tile->grid = grid;
    }
    if (!launch) return KSMM_OK;
    if (t.lds > 64 * 1024) {
        if (hipFuncSetAttribute(t.fn, hipFuncAttributeMaxDynamicSharedMemorySize, t.lds) != hipSuccess)
            return KSMM_ERR_LAUNCH;
    }
    int batch_i = (int)p.batch, n_tiles_i = (int)n_tiles, blocks_i = (int)blocks, m_tiles_i = m_tiles;
    void *args[] = {(void *)&p.x, (void *)&p.w, (void *)&p.y, &batch_i, (void *)&p.a, (void *)&p.b,
                    (void *)&p.c, (void *)&p.d, (void *)&p.scale, &m_tiles_i, &n_tiles_i, &blocks_i};
    hipError_t e = hipLaunchKernel(t.fn, dim3((unsigned)grid), dim3(t.threads), args, t.lds, p.stream);
    return e == hipSuccess ? KSMM_OK : KSMM_ERR_LAUNCH;
}

}  // namespace ksmm
