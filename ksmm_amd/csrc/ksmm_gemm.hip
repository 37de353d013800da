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
#include <type_traits>

#include "ksmm_mfma.h"


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


// the same with a uniform 64-bit base (SGPR pair) and a 32-bit per-lane byte offset
__device__ __forceinline__ void dma16s(const void *sbase, uint32_t voff, uint32_t lds_addr)
{
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                 :
                 : "v"(voff), "s"(sbase), "s"(lds_addr)
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
    static constexpr int PF = 4;  // L2 prefetch loads per thread (128-byte lines of the successor's input tile)
    static_assert(!BS_LAST || DD == 1, "DD > 1 is a batch-size-first variant");
    static_assert(ES == 2 || BS_LAST, "fp32 and e4m3 batch-size-first use other kernels");
    static_assert(TM % (32 * WM) == 0 && TN % (32 * WN) == 0 && TK % KSTEP == 0, "wave tiling");
    static_assert(W_CHUNKS % THREADS == 0 && X_CHUNKS % THREADS == 0, "every wave issues L loads per slab");
    static_assert(ES <= 2 ? (W_CPR == 8 || W_CPR % 16 == 0 || (ES == 1 && W_CPR == 4)) : W_CPR % 16 == 0, "weight swizzle group");
    static_assert(BS_LAST ? (ES <= 2 ? (X_CPR == 8 || X_CPR % 16 == 0) : X_CPR % 16 == 0) : (X_CPR == 4 || X_CPR == 8 || X_CPR % 16 == 0), "input swizzle group");
    static_assert(ST >= 2 && N_WAIT <= 63 && LDS_BYTES <= 160 * 1024, "ring");
    static_assert(DD * MT * NT * 16 <= 256, "accumulators");
};

// chunk swizzles (applied to the global address a lane fetches and by the operand reads)
// LDS has 64 banks of 4 bytes: a ds_read_b64 is served 32 lanes per clock and a ds_read_b128
// 16 lanes per clock, conflict-free when those lanes cover 256 bytes of distinct banks.
//  k-outer fp16 rows (CPR chunks of 16 bytes): the 32 lanes of a transpose load read 4 rows x
//  64 bytes -> XOR the 64-byte group index with row & 3 (rows of 128 bytes alternate bank
//  halves already: row / 2 & 1).
//  k-outer e4m3 rows: the 32 lanes of a transpose load read 8 rows x 32 bytes -> XOR the
//  32-byte group index with row & 7 (rows of 128 bytes: two rows per bank line, (row / 2) & 3;
//  rows of 64 bytes: four per bank line, (row / 4) & 1).
//  k-outer fp32: 2 rows x 128 bytes per ds_read_b32 wave -> XOR the 128-byte half with row & 1.
//  k-inner rows: 16 lanes read one chunk of 16 consecutive rows -> XOR the chunk so that the
//  rows sharing a 256-byte bank line differ (rows of 64, 128, >= 256 bytes).
template <typename CT, int CPR> __device__ __forceinline__ int swz_outer(int row)
{
    if (sizeof(CT) == 1) return CPR >= 16 ? 2 * (row & 7) : CPR == 8 ? 2 * ((row >> 1) & 3) : 2 * ((row >> 2) & 1);
    return sizeof(CT) == 2 ? (CPR >= 16 ? 4 * (row & 3) : 4 * ((row >> 1) & 1)) : 8 * (row & 1);
}
template <int CPR> __device__ __forceinline__ int swz_inner(int row)
{
    return CPR == 4 ? ((row >> 2) & 3) : CPR == 8 ? ((row >> 1) & 7) : (row & 15);
}

// k-outer operand (weights always, input for bs_last): S[k][idx], row of COLS elements.
// The address of a fragment is (per-lane byte offset, fixed for the kernel) + (stage base,
// uniform) + (k0 * row bytes, a compile-time constant that goes into the instruction's offset
// field): outer_off gives the first, outer_read takes the sum of the first two.
typedef __attribute__((address_space(3))) unsigned char *lds_bytes_t;
template <typename CT, int COLS> struct outer_frag;
template <int COLS> struct outer_frag<half_t, COLS> {
    __device__ static __forceinline__ uint32_t off(int idx0, int lane)
    {
        const int kq = lane >> 5, i16 = lane & 15, hs = (lane >> 4) & 1;
        const int row = 8 * kq + (i16 >> 2);  // + k0 (a multiple of 16): same row & 3
        const int chunk = (idx0 >> 3) + 2 * hs + ((i16 & 3) >> 1);
        return (uint32_t)(row * COLS * 2 + ((chunk ^ swz_outer<half_t, COLS / 8>(row)) << 4) + 8 * (i16 & 1));
    }
    __device__ static __forceinline__ half8_t read(uint32_t addr, int k0)
    {
        typedef short4_t __attribute__((address_space(3))) * lds_ptr;
        short4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(lds_bytes_t)(uintptr_t)(addr + k0 * COLS * 2));
        short4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(lds_bytes_t)(uintptr_t)(addr + (k0 + 4) * COLS * 2));
        typedef short short8_t __attribute__((ext_vector_type(8)));
        short8_t r = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
        return __builtin_bit_cast(half8_t, r);
    }
};
template <int COLS> struct outer_frag<fp8_t, COLS> {
    // ds_read_b64_tr_b8: 16 lanes address 8 rows x 16 bytes (lanes 2i, 2i+1: the two halves of
    // row i) and lane j receives column j, i.e. 8 consecutive k of one index
    __device__ static __forceinline__ uint32_t off(int idx0, int lane)
    {
        const int kq = lane >> 5, l16 = lane & 15, hs = (lane >> 4) & 1;
        const int row = 8 * kq + (l16 >> 1);  // + k0 (a multiple of 16): same row & 7
        const int chunk = (idx0 >> 4) + hs;
        return (uint32_t)(row * COLS + ((chunk ^ swz_outer<fp8_t, COLS / 16>(row)) << 4) + 8 * (l16 & 1));
    }
    __device__ static __forceinline__ long read(uint32_t addr, int k0)
    {
        typedef int int2_t __attribute__((ext_vector_type(2)));
        typedef int2_t __attribute__((address_space(3))) * lds_ptr;
        const int2_t r = __builtin_amdgcn_ds_read_tr8_b64_v2i32((lds_ptr)(lds_bytes_t)(uintptr_t)(addr + k0 * COLS));
        return __builtin_bit_cast(long, r);
    }
};
template <int COLS> struct outer_frag<float, COLS> {
    __device__ static __forceinline__ uint32_t off(int idx0, int lane)
    {
        const int row = lane >> 5, col = idx0 + (lane & 31);  // + k0 (even): same row & 1
        return (uint32_t)((row * COLS + ((((col >> 2) ^ (8 * (row & 1))) << 2) | (col & 3))) * 4);
    }
    __device__ static __forceinline__ float read(uint32_t addr, int k0)
    {
        typedef __attribute__((address_space(3))) float *lds_ptr;
        return *(lds_ptr)(lds_bytes_t)(uintptr_t)(addr + k0 * COLS * 4);
    }
};

template <typename CT, typename TY, bool BS_LAST, int DD, int TM, int TN, int TK, int WM, int WN, int ST, int OCC, bool KT, bool EPI>
__global__ __launch_bounds__(64 * WM * WN, OCC) void ks_gemm_kernel(const CT *__restrict__ x,
                                                              const CT *__restrict__ w,
                                                              TY *__restrict__ y, int batch, int a,
                                                              int b, int c, int d, Epi ep,
                                                              int m_tiles, int n_tiles, int blocks, int pf_dist)
{
    const float scale = ep.scale;
    // bias and activation live in an instantiation of their own: next to the accumulators their
    // registers would push the plain one into scratch memory
    constexpr bool has_epi = EPI;
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

    // ---- global addresses of the loads of one slab: uniform base + 32-bit per-lane offset ----
    // (the host checks that the offsets fit)
    const char *const wbase = (const char *)(w + ((size_t)(DD == 1 ? g : a_i * DD) * c) * b + m0);
    const char *const xbase = BS_LAST ? (const char *)(x + ((size_t)a_i * c * d + d_i) * batch + n0)
                                      : (const char *)(x + (size_t)n0 * in_size + (size_t)a_i * c * DD);
    // KT (bs_last): c need not be a multiple of TK.  The last slab then has rem < TK rows of its
    // own: the loads of the rows behind them are pointed at row rem-1 (valid memory, finite
    // whenever the data are), and the weight rows behind rem are cleared in LDS once they have
    // landed, so that they add nothing.
    static_assert(!KT || (BS_LAST && DD == 1), "K tails: batch-size-last only");
    const int steps = KT ? (c + TK - 1) / TK : c / TK;
    const int rem = KT ? c - (steps - 1) * TK : TK;  // rows of the last slab
    uint32_t wvoff[C::LW], xvoff[C::LX];
    uint32_t wvoff_t[KT ? C::LW : 1], xvoff_t[KT ? C::LX : 1];  // the same for the last slab
#pragma unroll
    for (int i = 0; i < C::LW; ++i) {
        const int q = tid + i * C::THREADS;
        const int dd = q / (TK * C::W_CPR), r = q % (TK * C::W_CPR);
        const int row = r / C::W_CPR, pc = r % C::W_CPR;
        const int col = (pc ^ swz_outer<CT, C::W_CPR>(row)) * C::EPC;
        wvoff[i] = (uint32_t)((((size_t)dd * c + row) * b + col) * C::ES);
        if constexpr (KT) wvoff_t[i] = (uint32_t)(((size_t)min(row, rem - 1) * b + col) * C::ES);
    }
#pragma unroll
    for (int i = 0; i < C::LX; ++i) {
        const int q = tid + i * C::THREADS;
        const int row = q / C::X_CPR, pc = q % C::X_CPR;
        if (BS_LAST) {
            const int col = (pc ^ swz_outer<CT, C::X_CPR>(row)) * C::EPC;
            xvoff[i] = (uint32_t)(((size_t)row * d * batch + min(col, batch - C::EPC - n0)) * C::ES);
            if constexpr (KT)
                xvoff_t[i] = (uint32_t)(((size_t)min(row, rem - 1) * d * batch + min(col, batch - C::EPC - n0)) * C::ES);
        } else {
            const int col = (pc ^ swz_inner<C::X_CPR>(row)) * C::EPC;
            xvoff[i] = (uint32_t)(((size_t)min(row, batch - 1 - n0) * in_size + col) * C::ES);
        }
    }
    const size_t w_step = (size_t)TK * b * C::ES;                                   // bytes per slab
    const size_t x_step = (BS_LAST ? (size_t)TK * d * batch : (size_t)TK * DD) * C::ES;
    const uint32_t lds_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char *)smem;
    auto issue = [&](int step, int stg) {
        const uint32_t dst = lds_base + stg * C::STAGE_BYTES + wave * 1024;
        const bool tail = KT && step == steps - 1;
#pragma unroll
        for (int i = 0; i < C::LW; ++i)
            dma16s(wbase + step * w_step, tail ? wvoff_t[KT ? i : 0] : wvoff[i], dst + i * (C::THREADS * 16));
#pragma unroll
        for (int i = 0; i < C::LX; ++i)
            dma16s(xbase + step * x_step, tail ? xvoff_t[KT ? i : 0] : xvoff[i], dst + C::W_BYTES + i * (C::THREADS * 16));
    };
    // clear this thread's chunks of the weight rows behind rem in stage stg (its own loads have
    // landed; the barrier that follows publishes the zeros with the rest)
    auto clear_tail = [&](int stg) {
#pragma unroll
        for (int i = 0; i < C::LW; ++i) {
            const int q = tid + i * C::THREADS;
            const int row = (q % (TK * C::W_CPR)) / C::W_CPR;
            if (row >= rem) {
                typedef __attribute__((address_space(3))) uint4_t *lds_ptr;
                *(lds_ptr)(lds_bytes_t)(uintptr_t)(lds_base + stg * C::STAGE_BYTES + q * 16) = uint4_t{0, 0, 0, 0};
            }
        }
    };

    // ---- per-lane byte offsets of the MFMA operands inside a stage (sub-step 0) --------------
    uint32_t woff[C::MT], xoff[C::NT];
#pragma unroll
    for (int i = 0; i < C::MT; ++i) woff[i] = outer_frag<CT, TM>::off((wm * C::MT + i) * 32, lane);
#pragma unroll
    for (int j = 0; j < C::NT; ++j) {
        const int idx0 = (wn * C::NT + j) * 32;
        if constexpr (BS_LAST) {
            xoff[j] = C::W_BYTES + outer_frag<CT, TN>::off(idx0, lane);
        } else {
            // k-inner rows of TK*DD elements; chunk (k0/8 + lane/32) (x 2 for the d_i pairs),
            // swizzled: the k0 part is XORed in when the operand is read
            const int row = idx0 + (lane & 31), lq = lane >> 5;
            xoff[j] = C::W_BYTES + row * (TK * DD * 2) + (((DD == 2 ? 2 * lq : lq) ^ swz_inner<C::X_CPR>(row)) << 4);
        }
    }

    float16_t acc[DD][C::MT][C::NT];
#pragma unroll
    for (int dd = 0; dd < DD; ++dd)
#pragma unroll
        for (int i = 0; i < C::MT; ++i)
#pragma unroll
            for (int j = 0; j < C::NT; ++j)
#pragma unroll
                for (int e = 0; e < 16; ++e) acc[dd][i][j][e] = 0.f;

    // L2 prefetch for the workgroup that will take this one's place: the input tile of logical
    // id lid + pf_dist (same XCD, pf_dist = workgroups resident per XCD), this workgroup's
    // share of its rows (the TM-tiles of one input tile split it).  One 4-byte load per
    // 128-byte line, result unused.
    // The loads are direct-to-LDS ones (no destination register to keep alive) into the last
    // ring stage: they are older than the loads of slab 0, so they have landed when the first
    // wait ends, before anything is requested into that stage.
    constexpr int PF = C::PF;
    if constexpr (BS_LAST) {
        const int flid = lid + pf_dist;
        if (pf_dist > 0 && flid < min(((int)blockIdx.x % 8 + 1) * per_xcd, blocks)) {
            const int f_mt = flid % m_tiles, f_rest = flid / m_tiles;
            const int f_nt = f_rest % n_tiles, f_g = f_rest / n_tiles;
            const int f_a = f_g / d, f_d = f_g - f_a * d, f_n0 = f_nt * TN;
            constexpr int LPR = TN * C::ES / 128;  // lines per row of the tile
            const int rows_per = (c + m_tiles - 1) / m_tiles;
            const int r_begin = f_mt * rows_per, r_end = min(c, r_begin + rows_per);
            const CT *fx = x + ((size_t)f_a * c * d + f_d) * batch + f_n0;
#pragma unroll
            for (int i = 0; i < PF; ++i) {
                const int q = tid + i * C::THREADS;
                const int r = r_begin + q / LPR, col = (q % LPR) * (128 / C::ES);
                if (r < r_end) {
                    const CT *ptr = fx + (size_t)r * d * batch + min(col, batch - 4 / C::ES - f_n0);
                    const uint32_t sink = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char *)smem +
                                          (ST - 1) * C::STAGE_BYTES + wave * 256;
                    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dword %0, off"
                                 :
                                 : "v"(ptr), "s"(sink)
                                 : "memory", "m0");
                }
            }
        }
    }
#pragma unroll
    for (int p = 0; p < ST - 1; ++p) issue(min(p, steps - 1), p);

    // MFMA operands of sub-step k0 of the slab whose operand addresses are wa[] / xa[].  Reading
    // them from LDS (read_frags) and making input operands of what was read (split_x) are separate
    // steps: for d == 2 the latter needs the data, and placed right behind the reads it would make
    // the wave wait out the LDS latency before it may issue the MFMAs that are already due.
    typedef typename frag<CT>::type frag_t;
    constexpr bool PAIRS = !BS_LAST && DD == 2;  // input rows hold (k, d_i) pairs
    // (16 waves leave 128 registers a lane: no room to keep pairs and operands side by side)
    constexpr bool LATE_SPLIT = PAIRS && C::THREADS <= 512;
    struct XPairs {
        uint4_t lo, hi;  // 16 consecutive halves = 8 (k, d_i) pairs; split early: the two operands
    };
    auto split_pairs = [](const uint4_t lo, const uint4_t hi, uint4_t &e, uint4_t &o) {
        e[0] = __builtin_amdgcn_perm(lo[1], lo[0], 0x05040100u);
        e[1] = __builtin_amdgcn_perm(lo[3], lo[2], 0x05040100u);
        e[2] = __builtin_amdgcn_perm(hi[1], hi[0], 0x05040100u);
        e[3] = __builtin_amdgcn_perm(hi[3], hi[2], 0x05040100u);
        o[0] = __builtin_amdgcn_perm(lo[1], lo[0], 0x07060302u);
        o[1] = __builtin_amdgcn_perm(lo[3], lo[2], 0x07060302u);
        o[2] = __builtin_amdgcn_perm(hi[1], hi[0], 0x07060302u);
        o[3] = __builtin_amdgcn_perm(hi[3], hi[2], 0x07060302u);
    };
    typedef typename std::conditional<PAIRS, XPairs, frag_t>::type xraw_t;
    auto read_frags = [&](const uint32_t(&wa)[C::MT], const uint32_t(&xa)[C::NT], int k0, frag_t(&fw)[DD][C::MT],
                          xraw_t(&xr)[C::NT]) {
#pragma unroll
        for (int dd = 0; dd < DD; ++dd)
#pragma unroll
            for (int i = 0; i < C::MT; ++i)
                fw[dd][i] = outer_frag<CT, TM>::read(wa[i] + dd * (TK * TM * C::ES), k0);
#pragma unroll
        for (int j = 0; j < C::NT; ++j) {
            if constexpr (BS_LAST) {
                xr[j] = outer_frag<CT, TN>::read(xa[j], k0);
            } else if constexpr (DD == 1) {
                typedef __attribute__((address_space(3))) half8_t *lds_ptr;
                xr[j] = *(lds_ptr)(lds_bytes_t)(uintptr_t)(xa[j] ^ ((k0 >> 3) << 4));
            } else {
                typedef __attribute__((address_space(3))) uint4_t *lds_ptr;
                const uint32_t pa = xa[j] ^ ((k0 >> 2) << 4);
                const uint4_t lo = *(lds_ptr)(lds_bytes_t)(uintptr_t)(pa);
                const uint4_t hi = *(lds_ptr)(lds_bytes_t)(uintptr_t)(pa ^ 16);
                if constexpr (LATE_SPLIT) {
                    xr[j].lo = lo;
                    xr[j].hi = hi;
                } else {
                    split_pairs(lo, hi, xr[j].lo, xr[j].hi);
                }
            }
        }
    };
    auto split_x = [&](const xraw_t(&xr)[C::NT], frag_t(&fx)[DD][C::NT]) {
#pragma unroll
        for (int j = 0; j < C::NT; ++j) {
            if constexpr (PAIRS) {
                // one operand per d_i
                uint4_t e = xr[j].lo, o = xr[j].hi;
                if constexpr (LATE_SPLIT) split_pairs(xr[j].lo, xr[j].hi, e, o);
                fx[0][j] = __builtin_bit_cast(half8_t, e);
                fx[DD - 1][j] = __builtin_bit_cast(half8_t, o);
            } else {
                fx[0][j] = xr[j];
            }
        }
    };
    constexpr int K0 = TK / C::KSTEP;                  // MFMA sub-steps per slab
    constexpr int PER_K0 = DD * C::MT * C::NT;         // MFMAs per sub-step
    static_assert(K0 >= 2 && K0 % 2 == 0, "operand double buffer alternates inside a slab");
    // The L loads of slab it+ST-1 are spread between the MFMAs of sub-steps 0..K0-2 of slab it
    // (the path into LDS moves 64 bytes per clock and CU: issued in one burst it would stall the
    // wave for about half a slab).  Before the MFMAs of the last sub-step every wave waits for
    // its loads of slab it+1 ((ST-2)*L newer ones may stay in flight; near the end the ring
    // holds repeats of the last slab, so the count stays constant), meets the others at a
    // barrier and requests the first operands of slab it+1, which arrive while the last
    // sub-step multiplies; operands of sub-step k0+1 are read while k0 multiplies.
    constexpr int SLOTS = (K0 - 1) * PER_K0;
    constexpr int STRIDE = SLOTS / C::L > 0 ? SLOTS / C::L : 1;  // MFMAs per load issued
    frag_t fw[2][DD][C::MT], fx[DD][C::NT];
    xraw_t xr[2][C::NT];
    uint32_t wa[C::MT], xa[C::NT];
    auto stage_addrs = [&](int stg) {
        const uint32_t base = lds_base + stg * C::STAGE_BYTES;
        // opaque to the compiler from here on, so that the k0 / d_i parts of an operand address
        // stay in the offset field of the LDS instructions instead of being re-added per read
#pragma unroll
        for (int i = 0; i < C::MT; ++i) {
            wa[i] = woff[i] + base;
            asm volatile("" : "+v"(wa[i]));
        }
#pragma unroll
        for (int j = 0; j < C::NT; ++j) {
            xa[j] = xoff[j] + base;
            asm volatile("" : "+v"(xa[j]));
        }
    };
    __builtin_amdgcn_s_waitcnt(vmcnt_imm(C::N_WAIT));
    if (KT && steps == 1 && rem < TK) clear_tail(0);
    __syncthreads();  // slab 0 landed for every wave
    stage_addrs(0);
    read_frags(wa, xa, 0, fw[0], xr[0]);

    for (int it = 0; it < steps; ++it) {
        const int nstep = min(it + ST - 1, steps - 1);
        const char *const wsrc = wbase + (size_t)nstep * w_step;
        const char *const xsrc = xbase + (size_t)nstep * x_step;
        const uint32_t dst = lds_base + ((it + ST - 1) % ST) * C::STAGE_BYTES + wave * 1024;
        const bool tail = KT && nstep == steps - 1;
        auto issue_one = [&](int q) {
            if (q < C::LW)
                dma16s(wsrc, tail ? wvoff_t[KT && q < C::LW ? q : 0] : wvoff[q < C::LW ? q : 0], dst + q * (C::THREADS * 16));
            else
                dma16s(xsrc, tail ? xvoff_t[KT && q >= C::LW ? q - C::LW : 0] : xvoff[q >= C::LW ? q - C::LW : 0],
                       dst + C::W_BYTES + (q - C::LW) * (C::THREADS * 16));
        };
#pragma unroll
        for (int kk = 0; kk < K0; ++kk) {
            if (kk + 1 < K0) {
                read_frags(wa, xa, (kk + 1) * C::KSTEP, fw[(kk + 1) & 1], xr[(kk + 1) & 1]);
            } else {
                __builtin_amdgcn_s_waitcnt(vmcnt_imm(C::N_WAIT));
                if (KT && it + 2 == steps && rem < TK) clear_tail((it + 1) % ST);
                __syncthreads();  // slab it+1 landed for every wave, and everyone left slab it
                if (it + 1 < steps) {
                    stage_addrs((it + 1) % ST);
                    read_frags(wa, xa, 0, fw[0], xr[0]);
                }
                __builtin_amdgcn_sched_barrier(0);  // requested before this sub-step multiplies
            }
            split_x(xr[kk & 1], fx);
#pragma unroll
            for (int dd = 0; dd < DD; ++dd)
#pragma unroll
                for (int i = 0; i < C::MT; ++i)
#pragma unroll
                    for (int j = 0; j < C::NT; ++j) {
                        acc[dd][i][j] = BS_LAST ? frag<CT>::mfma(fx[dd][j], fw[kk & 1][dd][i], acc[dd][i][j])
                                                : frag<CT>::mfma(fw[kk & 1][dd][i], fx[dd][j], acc[dd][i][j]);
                        const int m = kk * PER_K0 + (dd * C::MT + i) * C::NT + j;  // MFMA index in the slab
                        if (kk + 1 < K0 && (m + 1) % STRIDE == 0 && m / STRIDE < C::L) {
                            issue_one(m / STRIDE);
                            __builtin_amdgcn_sched_barrier(0);
                        }
                    }
            if (kk == K0 - 2) {
                // loads that did not get a slot above (fewer MFMAs than loads)
#pragma unroll
                for (int q = SLOTS / STRIDE; q < C::L; ++q) issue_one(q);
            }
        }
    }
    __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));  // repeats of the last slab must land before LDS is released

    __syncthreads();  // every wave is done with the operand ring: LDS becomes the output tile
    // Epilogue: the accumulators are transposed through LDS so that global memory sees 16-byte
    // stores along the contiguous axis.  The MFMA rows run along that axis (bs_last: batch,
    // bs_first: outputs), so a lane holds 4 consecutive elements of it per 8-row group:
    //   bs_last : out[m][n..n+3]                       row = TN elements
    //   bs_first: out[n][(m..m+3) x d_i interleaved]   row = TM*DD elements
    // The tile is written in passes of as many rows as fit in the LDS of the ring.
    {
        constexpr int OES = (int)sizeof(TY), OEPC = 16 / OES;  // output element, elements per 16 bytes
        constexpr int RC = (BS_LAST ? TN : TM * DD) + OEPC;     // padded row, elements
        constexpr int LR = BS_LAST ? TM : TN;                   // rows of the whole tile
        constexpr int RPP_RAW = C::LDS_BYTES / (RC * OES) / 32 * 32;
        constexpr int RPP = RPP_RAW > LR ? LR : RPP_RAW;        // rows per pass (multiple of 32)
        constexpr int PASSES = (LR + RPP - 1) / RPP;
        constexpr int CPR = (RC - OEPC) / OEPC;                 // 16-byte chunks per row
        static_assert(RPP >= 32, "output pass");
        TY *const out = (TY *)smem;
        const int l32 = lane & 31, lq = lane >> 5;
        // bias and activation act on the accumulators in place, before the tile is written out;
        // the passes below then store them as they are
        float st_scale = scale;
        if constexpr (has_epi) {
            const bool gelu = ep.act == KSMM_ACT_GELU;
#pragma unroll
            for (int i = 0; i < C::MT; ++i) {
                const int mb = (wm * C::MT + i) * 32;
                if constexpr (BS_LAST) {
                    // the lane's row is one output feature
                    const float bl = epi_bias<TY>(ep, ((size_t)a_i * b + m0 + mb + l32) * d + d_i);
#pragma unroll
                    for (int j = 0; j < C::NT; ++j)
#pragma unroll
                        for (int e = 0; e < 16; ++e) {
                            const float v = fmaf(acc[0][i][j][e], scale, bl);
                            acc[0][i][j][e] = gelu_if(gelu, v);
                        }
                } else {
                    // element u of group eg is output m0 + mb + 4*lq + 8*eg + u (x DD interleaved
                    // d_i): the lane's 4 * DD bias values of a group are consecutive, one vector load
                    static_assert(BS_LAST || sizeof(TY) == 2, "batch-size-first tiles write fp16");
                    typedef TY bias_v __attribute__((ext_vector_type(4 * DD)));
                    const size_t f0 = ((size_t)a_i * b + m0 + mb + 4 * lq) * DD;
#pragma unroll
                    for (int eg = 0; eg < 4; ++eg) {
                        bias_v bb = {};
                        if (ep.bias) bb = *(const bias_v *)((const TY *)ep.bias + f0 + 8 * eg * DD);
#pragma unroll
                        for (int j = 0; j < C::NT; ++j)
#pragma unroll
                            for (int u = 0; u < 4; ++u)
#pragma unroll
                                for (int dd = 0; dd < DD; ++dd) {
                                    const float v = fmaf(acc[dd][i][j][4 * eg + u], scale, (float)bb[u * DD + dd]);
                                    acc[dd][i][j][4 * eg + u] = gelu_if(gelu, v);
                                }
                    }
                }
            }
            st_scale = 1.f;
        }
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
                            float4_t v = {acc[0][i][j][4 * eg] * st_scale, acc[0][i][j][4 * eg + 1] * st_scale,
                                          acc[0][i][j][4 * eg + 2] * st_scale, acc[0][i][j][4 * eg + 3] * st_scale};
                            *(float4_t *)(dst + rcol + 8 * eg) = v;
                        } else if constexpr (DD == 1) {
                            half4_t v = {(half_t)(acc[0][i][j][4 * eg] * st_scale), (half_t)(acc[0][i][j][4 * eg + 1] * st_scale),
                                         (half_t)(acc[0][i][j][4 * eg + 2] * st_scale), (half_t)(acc[0][i][j][4 * eg + 3] * st_scale)};
                            *(half4_t *)(dst + rcol + 8 * eg) = v;
                        } else {
                            half8_t v;
#pragma unroll
                            for (int u = 0; u < 4; ++u) {
                                v[2 * u] = (half_t)(acc[0][i][j][4 * eg + u] * st_scale);
                                v[2 * u + 1] = (half_t)(acc[DD - 1][i][j][4 * eg + u] * st_scale);
                            }
                            *(half8_t *)(dst + (rcol + 8 * eg) * DD) = v;
                        }
                    }
                }
            __syncthreads();
            for (int q = tid; q < RPP * CPR; q += C::THREADS) {
                const int r = q / CPR, cc = (q % CPR) * OEPC;
                const int row = pass * RPP + r;  // row of the tile
                if (row >= LR) break;
                const uint4_t v = *(const uint4_t *)(out + r * RC + cc);
                if constexpr (BS_LAST) {
                    const int n = n0 + cc;
                    if (n < batch)
                        __builtin_nontemporal_store(v, (uint4_t *)(y + ((size_t)(a_i * b + m0 + row) * d + d_i) * batch + n));
                } else {
                    const int n = n0 + row;
                    // whole runs of TM*DD outputs per batch row: streaming stores
                    if (n < batch)
                        __builtin_nontemporal_store(v, (uint4_t *)(y + (size_t)n * out_size + ((size_t)a_i * b + m0) * DD + cc));
                }
            }
        }
    }
}


// ------------------------------------------------------------------------------------------
// Persistent form for fp16 batch-size-first blocks with d == 2: the same tile, ring and MFMA
// schedule as ks_gemm_kernel, with three differences that take the per-tile overheads out:
//  * a workgroup stays on its CU and walks through its tiles; the slab stream of the ring runs
//    on across tile boundaries, so the next tile's first slabs arrive while the current tile is
//    finished (no launch gap, no exposed first-slab latency);
//  * the lower half of the waves issues every direct-to-LDS load, so the other half never waits
//    on the vector-memory counter.  Operations of one wave complete in the order they were
//    issued: after a tile's output stores a loader's first wait also covers those stores, which
//    have had a slab's time to complete by then;
//  * the output tile leaves through the ring stage that has just been consumed (the other
//    stages already hold the next tile's slabs): every wave turns its 32x32 blocks around in a
//    private piece of it and stores whole 128-byte lines, without a workgroup barrier.
// All waves multiply and store their own part of the output.
template <typename CT, typename TY, int DD, int TM, int TN, int TK, int WM, int WN, int ST, int OCC, bool EPI, bool SP>
__global__ __launch_bounds__(64 * WM * WN, OCC) void ks_gemm_pbf_kernel(const CT *__restrict__ x,
                                                                const CT *__restrict__ w,
                                                                TY *__restrict__ y, int batch, int a,
                                                                int b, int c, int d, Epi ep,
                                                                int m_tiles, int n_tiles, int blocks)
{
    typedef GemmCfg<CT, false, DD, TM, TN, TK, WM, WN, ST> C;
    constexpr int NWAVES = WM * WN, LOADERS = 64 * (NWAVES / 2);      // loader threads (lower half)
    constexpr int LW = C::W_CHUNKS / LOADERS, LX = C::X_CHUNKS / LOADERS, L = LW + LX;
    constexpr int N_WAIT = (ST - 2) * L;
    static_assert(NWAVES % 2 == 0 && C::W_CHUNKS % LOADERS == 0 && C::X_CHUNKS % LOADERS == 0, "loader split");
    static_assert(ST >= 3 && N_WAIT <= 63, "ring");
    static_assert(sizeof(CT) == 2 && sizeof(TY) == 2, "fp16 only");
    static_assert(!SP || DD == 2, "the sparse-MFMA form is for (k, d_i) pairs");
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    const float scale = ep.scale;
    // bias and activation live in an instantiation of their own: next to the accumulators their
    // registers would push the plain one into scratch memory
    constexpr bool has_epi = EPI;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave / WN, wn = wave % WN;
    const bool loader = wave < NWAVES / 2;  // uniform per wave
    const size_t in_size = (size_t)a * c * d, out_size = (size_t)a * b * d;

    // ---- the tiles of this workgroup: XCD blockIdx % 8 owns a contiguous eighth of the logical
    // tile ids (TM-tile fastest, then batch tile, then a_i), its workgroup blockIdx / 8 takes
    // every slots-th one: the workgroups of an XCD work on neighbouring ids at any one time, so
    // the TM-tiles of one input tile share it through that XCD's L2
    const int per_xcd = (blocks + 7) / 8;
    const int slots = (int)gridDim.x / 8;  // the grid is a multiple of 8
    const int xcd_first = ((int)blockIdx.x % 8) * per_xcd;
    const int xcd_end = min(xcd_first + per_xcd, blocks);
    const int first = xcd_first + (int)blockIdx.x / 8;
    if (first >= xcd_end) return;
    const int my_tiles = (xcd_end - first + slots - 1) / slots;
    struct Tile {
        int m0, n0, a_i;
    };
    auto decode = [&](int t) {
        const int lid = first + t * slots;
        const int mt_id = lid % m_tiles, rest = lid / m_tiles;
        return Tile{mt_id * TM, (rest % n_tiles) * TN, rest / n_tiles};
    };

    // ---- load side (loader waves): a stream of slabs that runs ST-1 slabs ahead of the
    // multiplication, across tile boundaries.  uniform base + 32-bit per-lane offset
    const int steps = c / TK;
    const size_t w_step = (size_t)TK * b * C::ES, x_step = (size_t)TK * DD * C::ES;  // bytes per slab
    // Weight chunk i of a lane is LOADERS chunks = W_ROWS_PER rows further down than chunk i - 1,
    // in the same column and with the same swizzle (a multiple of 4 rows), and after LW_PER_DD
    // chunks it moves on to the next d_i: one per-lane offset, the rest are uniform additions.
    constexpr int W_ROWS_PER = LOADERS / C::W_CPR, LW_PER_DD = LW / DD;
    static_assert(LOADERS % C::W_CPR == 0 && W_ROWS_PER % 4 == 0 && LW % DD == 0 && W_ROWS_PER * LW_PER_DD == TK,
                  "uniform weight chunk strides");
    uint32_t wvoff0, xvoff[LX];
    {
        const int q = tid & (LOADERS - 1);
        const int row = q / C::W_CPR, pc = q % C::W_CPR;
        const int col = (pc ^ swz_outer<CT, C::W_CPR>(row)) * C::EPC;
        wvoff0 = (uint32_t)(((size_t)row * b + col) * C::ES);
    }
    const size_t w_chunk_step = (size_t)W_ROWS_PER * b * C::ES, w_dd_step = (size_t)c * b * C::ES;
    const char *i_w = nullptr, *i_x = nullptr;  // slab the load side is at
    int i_t = 0, i_k = 0;
    auto i_open = [&](int t) {
        const Tile q = decode(t);
        i_w = (const char *)(w + ((size_t)(q.a_i * DD) * c) * b + q.m0);
        i_x = (const char *)(x + (size_t)q.n0 * in_size + (size_t)q.a_i * c * DD);
        // the last batch tile repeats its last row instead of reading past the end
        int tid_ = tid & (LOADERS - 1);
        asm volatile("" : "+v"(tid_));
#pragma unroll
        for (int i = 0; i < LX; ++i) {
            const int qq = tid_ + i * LOADERS;
            const int row = qq / C::X_CPR, pc = qq % C::X_CPR;
            const int col = (pc ^ swz_inner<C::X_CPR>(row)) * C::EPC;
            xvoff[i] = (uint32_t)(((size_t)min(row, batch - 1 - q.n0) * in_size + col) * C::ES);
        }
    };
    // next slab of the stream; after the last one the load side stays there (the ring then
    // receives repeats of it, which keeps the number of loads per slab constant)
    auto i_advance = [&]() {
        if (i_k + 1 < steps) {
            ++i_k;
            i_w += w_step;
            i_x += x_step;
        } else if (i_t + 1 < my_tiles) {
            ++i_t;
            i_k = 0;
            i_open(i_t);
        }
    };
    const uint32_t lds_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char *)smem;
    auto issue_one = [&](const char *wsrc, const char *xsrc, uint32_t dst, int q) {
        // dst: stage base + this wave's kilobyte; chunk q of the lane
        if (q < LW)
            dma16s(wsrc + (q / LW_PER_DD) * w_dd_step + (q % LW_PER_DD) * w_chunk_step, wvoff0, dst + q * (LOADERS * 16));
        else
            dma16s(xsrc, xvoff[q >= LW ? q - LW : 0], dst + C::W_BYTES + (q - LW) * (LOADERS * 16));
    };

    // ---- per-lane byte offsets of the MFMA operands inside a stage (sub-step 0) --------------
    uint32_t woff[C::MT], xoff[C::NT];
#pragma unroll
    for (int i = 0; i < C::MT; ++i) woff[i] = outer_frag<CT, TM>::off((wm * C::MT + i) * 32, lane);
#pragma unroll
    for (int j = 0; j < C::NT; ++j) {
        const int row = (wn * C::NT + j) * 32 + (lane & 31), lq = lane >> 5;
        // (k, d_i) pairs: a lane's 16 halves are chunks 2 lq and 2 lq + 1 of the 4 chunks of a
        // sub-step; the sparse MFMA wants chunks lq and lq + 2 (see the multiplication below)
        xoff[j] = C::W_BYTES + row * (TK * DD * 2) + (((DD == 2 && !SP ? 2 * lq : lq) ^ swz_inner<C::X_CPR>(row)) << 4);
    }
    float16_t acc[DD][C::MT][C::NT];
    auto clear_acc = [&]() {
#pragma unroll
        for (int dd = 0; dd < DD; ++dd)
#pragma unroll
            for (int i = 0; i < C::MT; ++i)
#pragma unroll
                for (int j = 0; j < C::NT; ++j)
#pragma unroll
                    for (int e = 0; e < 16; ++e) acc[dd][i][j][e] = 0.f;
    };
    clear_acc();

    i_open(0);
#pragma unroll
    for (int p = 0; p < ST - 1; ++p) {
        if (loader) {
            const uint32_t dst = lds_base + p * C::STAGE_BYTES + wave * 1024;
#pragma unroll
            for (int q = 0; q < L; ++q) issue_one(i_w, i_x, dst, q);
        }
        i_advance();
    }

    // reading operands from LDS and splitting the (k, d_i) pairs of the input rows into one
    // operand per d_i are separate steps, as in ks_gemm_kernel
    typedef typename frag<CT>::type frag_t;
    struct XPairs {
        uint4_t lo, hi;
    };
    typedef typename std::conditional<DD == 2, XPairs, frag_t>::type xraw_t;  // d == 1: the operand itself
    auto read_frags = [&](const uint32_t(&wa)[C::MT], const uint32_t(&xa)[C::NT], int k0, frag_t(&fw)[DD][C::MT],
                          xraw_t(&xr)[C::NT]) {
#pragma unroll
        for (int dd = 0; dd < DD; ++dd)
#pragma unroll
            for (int i = 0; i < C::MT; ++i)
                fw[dd][i] = outer_frag<CT, TM>::read(wa[i] + dd * (TK * TM * C::ES), k0);
#pragma unroll
        for (int j = 0; j < C::NT; ++j) {
            if constexpr (DD == 2) {
                typedef __attribute__((address_space(3))) uint4_t *lds_ptr;
                const uint32_t pa = xa[j] ^ ((k0 >> 2) << 4);
                xr[j].lo = *(lds_ptr)(lds_bytes_t)(uintptr_t)(pa);
                xr[j].hi = *(lds_ptr)(lds_bytes_t)(uintptr_t)(pa ^ (SP ? 32 : 16));
            } else {
                typedef __attribute__((address_space(3))) half8_t *lds_ptr;
                xr[j] = *(lds_ptr)(lds_bytes_t)(uintptr_t)(xa[j] ^ ((k0 >> 3) << 4));
            }
        }
    };
    auto split_x = [&](const xraw_t(&xr)[C::NT], frag_t(&fx)[DD][C::NT]) {
#pragma unroll
        for (int j = 0; j < C::NT; ++j) {
            if constexpr (DD == 1) {
                fx[0][j] = xr[j];
            } else if constexpr (SP) {
                // nothing to split: the sparse MFMA takes the 16 interleaved halves as they are
            } else {
            const uint4_t lo = xr[j].lo, hi = xr[j].hi;
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
    constexpr int K0 = TK / C::KSTEP;           // MFMA sub-steps per slab
    constexpr int PER_K0 = DD * C::MT * C::NT;  // MFMAs per sub-step
    static_assert(K0 >= 2 && K0 % 2 == 0, "operand double buffer alternates inside a slab");
    constexpr int SLOTS = (K0 - 1) * PER_K0;
    constexpr int STRIDE = SLOTS / L > 0 ? SLOTS / L : 1;  // MFMAs per load issued (loader waves)
    frag_t fw[2][DD][C::MT], fx[DD][C::NT];
    xraw_t xr[2][C::NT];
    uint32_t wa[C::MT], xa[C::NT];
    auto stage_addrs = [&](int stg) {
        const uint32_t base = lds_base + stg * C::STAGE_BYTES;
#pragma unroll
        for (int i = 0; i < C::MT; ++i) {
            wa[i] = woff[i] + base;
            asm volatile("" : "+v"(wa[i]));
        }
#pragma unroll
        for (int j = 0; j < C::NT; ++j) {
            xa[j] = xoff[j] + base;
            asm volatile("" : "+v"(xa[j]));
        }
    };
    if (loader) __builtin_amdgcn_s_waitcnt(vmcnt_imm(N_WAIT));
    __syncthreads();  // slab 0 landed
    stage_addrs(0);
    read_frags(wa, xa, 0, fw[0], xr[0]);

    const int l32 = lane & 31, lq = lane >> 5;
    constexpr int OP = 128 + 16;  // bytes per row of a wave's output piece
    static_assert(NWAVES * 32 * OP <= C::STAGE_BYTES, "output pieces fit the consumed stage");
    // d == 1: a block row is 32 outputs = 64 bytes, so two neighbouring TM-blocks share a line
    constexpr int IP = DD == 2 ? 1 : 2;
    static_assert(C::MT % IP == 0, "TM-blocks pair up into whole lines");

    constexpr int TILE_STORES = (C::MT / IP) * C::NT * 4;  // stores of a wave per full tile
    static_assert(N_WAIT + TILE_STORES <= 63, "counter range");
    bool stores_behind = false;  // the previous tile issued exactly TILE_STORES stores (uniform)
    Tile cur = decode(0);
    int stg = 0;  // ring stage of the slab being multiplied
    for (int c_t = 0; c_t < my_tiles; ++c_t) {
        for (int c_k = 0; c_k < steps; ++c_k) {
            const char *const wsrc = i_w;
            const char *const xsrc = i_x;
            const int stg_fill = stg == 0 ? ST - 1 : stg - 1;  // stage of the slab ST-1 ahead
            const int stg_next = stg + 1 == ST ? 0 : stg + 1;
            const uint32_t dst = lds_base + stg_fill * C::STAGE_BYTES + wave * 1024;
#pragma unroll
            for (int kk = 0; kk < K0; ++kk) {
                if (kk + 1 < K0) {
                    read_frags(wa, xa, (kk + 1) * C::KSTEP, fw[(kk + 1) & 1], xr[(kk + 1) & 1]);
                } else {
                    if (loader) {
                        // behind the next slab's loads the counter holds the loads of the slab after
                        // it and, on the first slab of a tile, the previous tile's output stores
                        if (c_k == 0 && stores_behind)
                            __builtin_amdgcn_s_waitcnt(vmcnt_imm(N_WAIT + TILE_STORES));
                        else
                            __builtin_amdgcn_s_waitcnt(vmcnt_imm(N_WAIT));
                    }
                    __syncthreads();  // the next slab has landed, and everyone has left this one
                    // (at the end of a tile the next tile's first operands are read after its output
                    // has left: their registers are needed for that)
                    if (c_k + 1 < steps) {
                        stage_addrs(stg_next);
                        read_frags(wa, xa, 0, fw[0], xr[0]);
                    }
                    __builtin_amdgcn_sched_barrier(0);  // requested before this sub-step multiplies
                }
                split_x(xr[kk & 1], fx);
#pragma unroll
                for (int dd = 0; dd < DD; ++dd)
#pragma unroll
                    for (int i = 0; i < C::MT; ++i)
#pragma unroll
                        for (int j = 0; j < C::NT; ++j) {
                            if constexpr (SP) {
                                // Over the interleaved (k, d_i) axis of an input row (position
                                // P = 2 k + d_i, 32 positions per sub-step of 16 k) the weights of
                                // block d_i are 2:4 sparse: they sit at positions d_i and d_i + 2 of
                                // every four.  v_smfmac_f32_32x32x32_f16 takes 16 halves per lane of
                                // the dense operand and 8 of the compressed one; the index register
                                // names the positions (two bits per weight: 0,2 for d_i = 0 in its
                                // low half, 1,3 for d_i = 1 in its high half, chosen by the abid
                                // field).  Measured operand layout (lane half h = lane / 32): the
                                // dense operand's elements 0-7 are positions 8 h .. 8 h + 7 and its
                                // elements 8-15 positions 16 + 8 h .., the compressed operand's
                                // elements 0-3 go with positions 16 h .. 16 h + 7 and 4-7 with
                                // 16 h + 8 .. 16 h + 15, i.e. they are k = 8 h .. 8 h + 7 in order,
                                // exactly the lane's operand of the dense 32x32x16 MFMA; the input
                                // lane reads chunks h and h + 2 of the sub-step's four.
                                const half16_t xb = __builtin_bit_cast(half16_t, xr[kk & 1][j]);
                                if (dd == 0)
                                    acc[dd][i][j] = __builtin_amdgcn_smfmac_f32_32x32x32_f16(fw[kk & 1][dd][i], xb, acc[dd][i][j],
                                                                                           (int)0xDDDD8888u, 0, 0);
                                else
                                    acc[dd][i][j] = __builtin_amdgcn_smfmac_f32_32x32x32_f16(fw[kk & 1][dd][i], xb, acc[dd][i][j],
                                                                                           (int)0xDDDD8888u, 0, 1);
                            } else {
                                acc[dd][i][j] = frag<CT>::mfma(fw[kk & 1][dd][i], fx[dd][j], acc[dd][i][j]);
                            }
                            const int m = kk * PER_K0 + (dd * C::MT + i) * C::NT + j;  // MFMA index in the slab
                            if (kk + 1 < K0 && (m + 1) % STRIDE == 0 && m / STRIDE < L) {
                                if (loader) issue_one(wsrc, xsrc, dst, m / STRIDE);
                                __builtin_amdgcn_sched_barrier(0);
                            }
                        }
                if (kk == K0 - 2) {
                    // loads that did not get a slot above (fewer MFMAs than loads)
                    if (loader) {
#pragma unroll
                        for (int q = SLOTS / STRIDE; q < L; ++q) issue_one(wsrc, xsrc, dst, q);
                    }
                }
            }
            i_advance();
            if (c_k + 1 < steps) stg = stg_next;
        }
        // ---- the tile is complete.  Stage `stg` is consumed (every wave passed the barrier of its
        // last sub-step, so nobody reads it any more) and the other stages already hold slabs of
        // the next tile: each wave takes a private piece of it to turn its 32x32 blocks around.
        // In the accumulators a lane holds, per group eg, 4 outputs x 2 d_i of one batch row =
        // 16 of the row's 128 bytes; written like that a store touches 32 lines.  Through the
        // private piece (OP bytes per row: 16 lanes of a vector access fall on distinct banks)
        // eight neighbouring lanes get the eight pieces of a row: whole lines, 8 per store.
        // LDS accesses of one wave execute in order, so the piece needs no barrier.
        if constexpr (has_epi) {
#pragma unroll
            for (int i = 0; i < C::MT; ++i) {
                const size_t f0 = ((size_t)cur.a_i * b + cur.m0 + (wm * C::MT + i) * 32 + 4 * lq) * DD;
#pragma unroll
                for (int eg = 0; eg < 4; ++eg) {
                    // the lane's bias values of this group: (4 outputs) x (DD d_i), one vector load
                    typedef TY bias_v __attribute__((ext_vector_type(4 * DD)));
                    bias_v bb = {};
                    if (ep.bias) bb = *(const bias_v *)((const TY *)ep.bias + f0 + 8 * DD * eg);
#pragma unroll
                    for (int j = 0; j < C::NT; ++j)
#pragma unroll
                        for (int u = 0; u < 4; ++u)
#pragma unroll
                            for (int dd = 0; dd < DD; ++dd) {
                                const float v = fmaf(acc[dd][i][j][4 * eg + u], scale, (float)bb[DD * u + dd]);
                                acc[dd][i][j][4 * eg + u] = gelu_if(ep.act == KSMM_ACT_GELU, v);
                            }
                }
            }
        }
        const float st_scale = has_epi ? 1.f : scale;
        {
            unsigned char *const piece = smem + stg * C::STAGE_BYTES + wave * (32 * OP);
            unsigned char *const wr = piece + l32 * OP + (8 * DD) * lq;     // + 16 * DD * eg (+ 64 * second block)
            const unsigned char *const rd = piece + (lane >> 3) * OP + 16 * (lane & 7);  // + 8 * t rows
#pragma unroll
            for (int ip = 0; ip < C::MT / IP; ++ip)
#pragma unroll
                for (int j = 0; j < C::NT; ++j) {
                    const int i = ip * IP;
                    const int mb = (wm * C::MT + i) * 32, nb = (wn * C::NT + j) * 32;
#pragma unroll
                    for (int eg = 0; eg < 4; ++eg) {
                        if constexpr (DD == 2) {
                            half8_t v;
#pragma unroll
                            for (int u = 0; u < 4; ++u) {
                                v[2 * u] = (half_t)(acc[0][i][j][4 * eg + u] * st_scale);
                                v[2 * u + 1] = (half_t)(acc[DD - 1][i][j][4 * eg + u] * st_scale);
                            }
                            *(half8_t *)(wr + 32 * eg) = v;
                        } else {
#pragma unroll
                            for (int ii = 0; ii < IP; ++ii) {
                                const float16_t &ac = acc[0][i + ii][j];
                                const half4_t v = {(half_t)(ac[4 * eg] * st_scale), (half_t)(ac[4 * eg + 1] * st_scale),
                                                   (half_t)(ac[4 * eg + 2] * st_scale), (half_t)(ac[4 * eg + 3] * st_scale)};
                                *(half4_t *)(wr + 64 * ii + 16 * eg) = v;
                            }
                        }
                    }
                    __builtin_amdgcn_wave_barrier();
                    const int n = cur.n0 + nb + (lane >> 3);  // + 8 * t
                    TY *const dstp = y + (size_t)n * out_size + ((size_t)cur.a_i * b + cur.m0 + mb) * DD + 8 * (lane & 7);
#pragma unroll
                    for (int t = 0; t < 4; ++t) {
                        const uint4_t v = *(const uint4_t *)(rd + 8 * t * OP);
                        if (n + 8 * t < batch) __builtin_nontemporal_store(v, (uint4_t *)(dstp + (size_t)8 * t * out_size));
                    }
                    __builtin_amdgcn_wave_barrier();
                }
        }
        stores_behind = cur.n0 + TN <= batch;  // a ragged tile skips stores: then wait the safe way
        if (c_t + 1 < my_tiles) {
            __syncthreads();  // every private piece is read: the stage may receive slabs again
            clear_acc();
            cur = decode(c_t + 1);
            stg = stg + 1 == ST ? 0 : stg + 1;
            stage_addrs(stg);
            read_frags(wa, xa, 0, fw[0], xr[0]);
        }
    }
    if (loader) __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));  // repeats of the last slab must land before LDS is released
}

// ------------------------------------------------------------------------------------------
// Persistent form for batch-size-last blocks (fp32, fp16 and e4m3, any d): the scheme of
// ks_gemm_pbf_kernel with the operand roles of the batch-size-last tiles.  Both operands are
// k-outer, so every chunk of a loader lane is a whole number of rows further down than the one
// before it, with the same column and swizzle: one per-lane offset each for weights and input,
// the rest are uniform additions.  The accumulator rows run along the batch axis; a wave turns
// its blocks around in a piece of LDS of its own behind the ring (32 output rows x 128 bytes:
// two neighbouring 32-column blocks for fp16, one for fp32) and stores whole lines.  The pieces
// are private, so a tile switch needs no workgroup barrier: waves that finish their part of
// the tile early start on the next tile's first slab while the others still store.
template <typename CT, typename TY, int TM, int TN, int TK, int WM, int WN, int ST, int OCC, bool MTAIL, bool EPI>
__global__ __launch_bounds__(64 * WM * WN, OCC) void ks_gemm_pbl_kernel(const CT *__restrict__ x,
                                                                const CT *__restrict__ w,
                                                                TY *__restrict__ y, int batch, int a,
                                                                int b, int c, int d, Epi ep,
                                                                int m_tiles, int n_tiles, int blocks)
{
    typedef GemmCfg<CT, true, 1, TM, TN, TK, WM, WN, ST> C;
    constexpr int NWAVES = WM * WN, LOADERS = 64 * (NWAVES / 2);      // loader threads (lower half)
    constexpr int LW = C::W_CHUNKS / LOADERS, LX = C::X_CHUNKS / LOADERS, L = LW + LX;
    constexpr int N_WAIT = (ST - 2) * L;
    static_assert(NWAVES % 2 == 0 && C::W_CHUNKS % LOADERS == 0 && C::X_CHUNKS % LOADERS == 0, "loader split");
    static_assert(ST >= 3 && N_WAIT <= 63, "ring");
    static_assert(sizeof(CT) == sizeof(TY) || (sizeof(CT) == 1 && sizeof(TY) == 2), "fp32, fp16, e4m3 -> fp16");
    constexpr int OES = (int)sizeof(TY);
    constexpr int JP = OES == 2 ? 2 : 1;  // 32-column blocks per 128 bytes of an output row
    static_assert(C::NT % JP == 0, "blocks pair up into whole lines");
    constexpr int OP = 128 + 16;          // bytes per row of a wave's output piece
    constexpr int OUT_BASE = C::LDS_BYTES;  // the pieces follow the ring
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    const float scale = ep.scale;
    // bias and activation live in an instantiation of their own: next to the accumulators their
    // registers would push the plain one into scratch memory
    constexpr bool has_epi = EPI;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave / WN, wn = wave % WN;
    const bool loader = wave < NWAVES / 2;  // uniform per wave

    // ---- the tiles of this workgroup: XCD blockIdx % 8 owns a contiguous eighth of the logical
    // tile ids (TM-tile fastest, then batch tile, then the block a_i * d + d_i), its workgroup
    // blockIdx / 8 takes every slots-th one
    const int per_xcd = (blocks + 7) / 8;
    const int slots = (int)gridDim.x / 8;  // the grid is a multiple of 8
    const int xcd_first = ((int)blockIdx.x % 8) * per_xcd;
    const int xcd_end = min(xcd_first + per_xcd, blocks);
    const int first = xcd_first + (int)blockIdx.x / 8;
    if (first >= xcd_end) return;
    const int my_tiles = (xcd_end - first + slots - 1) / slots;
    struct Tile {
        int m0, n0, a_i, d_i;
    };
    auto decode = [&](int t) {
        const int lid = first + t * slots;
        const int mt_id = lid % m_tiles, rest = lid / m_tiles;
        const int g = rest / n_tiles, a_i = g / d;
        return Tile{mt_id * TM, (rest % n_tiles) * TN, a_i, g - a_i * d};
    };

    // ---- load side (loader waves): a stream of slabs that runs ST-1 slabs ahead of the
    // multiplication, across tile boundaries.  uniform base + 32-bit per-lane offset
    const int steps = c / TK;
    const size_t w_step = (size_t)TK * b * C::ES, x_step = (size_t)TK * d * batch * C::ES;  // bytes per slab
    constexpr int W_ROWS_PER = LOADERS / C::W_CPR, X_ROWS_PER = LOADERS / C::X_CPR;
    constexpr int SWZ_ROWS = C::ES == 1 ? 8 : C::ES == 2 ? 4 : 2;  // rows after which the chunk swizzle repeats
    static_assert(LOADERS % C::W_CPR == 0 && W_ROWS_PER % SWZ_ROWS == 0 && W_ROWS_PER * LW == TK, "uniform weight chunk strides");
    static_assert(LOADERS % C::X_CPR == 0 && X_ROWS_PER % SWZ_ROWS == 0 && X_ROWS_PER * LX == TK, "uniform input chunk strides");
    uint32_t wvoff0, xvoff0, xrow_off, wrow_off;
    int xcol, wcol;
    {
        const int q = tid & (LOADERS - 1);
        const int row = q / C::W_CPR, pc = q % C::W_CPR;
        wcol = (pc ^ swz_outer<CT, C::W_CPR>(row)) * C::EPC;
        wrow_off = (uint32_t)((size_t)row * b * C::ES);
        wvoff0 = wrow_off + (uint32_t)(wcol * C::ES);
        const int xrow = q / C::X_CPR, xpc = q % C::X_CPR;
        xcol = (xpc ^ swz_outer<CT, C::X_CPR>(xrow)) * C::EPC;
        xrow_off = (uint32_t)((size_t)xrow * d * batch * C::ES);
    }
    const size_t w_chunk_step = (size_t)W_ROWS_PER * b * C::ES, x_chunk_step = (size_t)X_ROWS_PER * d * batch * C::ES;
    const char *i_w = nullptr, *i_x = nullptr;  // slab the load side is at
    int i_t = 0, i_k = 0;
    auto i_open = [&](int t) {
        const Tile q = decode(t);
        i_w = (const char *)(w + ((size_t)(q.a_i * d + q.d_i) * c) * b + q.m0);
        i_x = (const char *)(x + ((size_t)q.a_i * c * d + q.d_i) * batch + q.n0);
        // the last batch tile repeats its last 16 bytes instead of reading past the end of a row
        xvoff0 = xrow_off + (uint32_t)(min(xcol, batch - C::EPC - q.n0) * C::ES);
        // MTAIL: so does a last TM-tile that reaches beyond b (its rows behind b are not stored)
        if constexpr (MTAIL) wvoff0 = wrow_off + (uint32_t)(min(wcol, b - C::EPC - q.m0) * C::ES);
    };
    // next slab of the stream; after the last one the load side stays there (the ring then
    // receives repeats of it, which keeps the number of loads per slab constant)
    auto i_advance = [&]() {
        if (i_k + 1 < steps) {
            ++i_k;
            i_w += w_step;
            i_x += x_step;
        } else if (i_t + 1 < my_tiles) {
            ++i_t;
            i_k = 0;
            i_open(i_t);
        }
    };
    const uint32_t lds_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char *)smem;
    auto issue_one = [&](const char *wsrc, const char *xsrc, uint32_t dst, int q) {
        // dst: stage base + this wave's kilobyte; chunk q of the lane
        if (q < LW)
            dma16s(wsrc + q * w_chunk_step, wvoff0, dst + q * (LOADERS * 16));
        else
            dma16s(xsrc + (q - LW) * x_chunk_step, xvoff0, dst + C::W_BYTES + (q - LW) * (LOADERS * 16));
    };

    // ---- per-lane byte offsets of the MFMA operands inside a stage (sub-step 0) --------------
    uint32_t woff[C::MT], xoff[C::NT];
#pragma unroll
    for (int i = 0; i < C::MT; ++i) woff[i] = outer_frag<CT, TM>::off((wm * C::MT + i) * 32, lane);
#pragma unroll
    for (int j = 0; j < C::NT; ++j) xoff[j] = C::W_BYTES + outer_frag<CT, TN>::off((wn * C::NT + j) * 32, lane);
    float16_t acc[C::MT][C::NT];
    auto clear_acc = [&]() {
#pragma unroll
        for (int i = 0; i < C::MT; ++i)
#pragma unroll
            for (int j = 0; j < C::NT; ++j)
#pragma unroll
                for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;
    };
    clear_acc();

    i_open(0);
#pragma unroll
    for (int p = 0; p < ST - 1; ++p) {
        if (loader) {
            const uint32_t dst = lds_base + p * C::STAGE_BYTES + wave * 1024;
#pragma unroll
            for (int q = 0; q < L; ++q) issue_one(i_w, i_x, dst, q);
        }
        i_advance();
    }

    typedef typename frag<CT>::type frag_t;
    auto read_frags = [&](const uint32_t(&wa)[C::MT], const uint32_t(&xa)[C::NT], int k0, frag_t(&fw)[C::MT],
                          frag_t(&fx)[C::NT]) {
#pragma unroll
        for (int i = 0; i < C::MT; ++i) fw[i] = outer_frag<CT, TM>::read(wa[i], k0);
#pragma unroll
        for (int j = 0; j < C::NT; ++j) fx[j] = outer_frag<CT, TN>::read(xa[j], k0);
    };
    constexpr int K0 = TK / C::KSTEP;      // MFMA sub-steps per slab
    constexpr int PER_K0 = C::MT * C::NT;  // MFMAs per sub-step
    static_assert(K0 >= 2 && K0 % 2 == 0, "operand double buffer alternates inside a slab");
    constexpr int SLOTS = (K0 - 1) * PER_K0;
    constexpr int STRIDE = SLOTS / L > 0 ? SLOTS / L : 1;  // MFMAs per load issued (loader waves)
    frag_t fw[2][C::MT], fx[2][C::NT];
    uint32_t wa[C::MT], xa[C::NT];
    auto stage_addrs = [&](int stg) {
        const uint32_t base = lds_base + stg * C::STAGE_BYTES;
#pragma unroll
        for (int i = 0; i < C::MT; ++i) {
            wa[i] = woff[i] + base;
            asm volatile("" : "+v"(wa[i]));
        }
#pragma unroll
        for (int j = 0; j < C::NT; ++j) {
            xa[j] = xoff[j] + base;
            asm volatile("" : "+v"(xa[j]));
        }
    };
    if (loader) __builtin_amdgcn_s_waitcnt(vmcnt_imm(N_WAIT));
    __syncthreads();  // slab 0 landed
    stage_addrs(0);
    read_frags(wa, xa, 0, fw[0], fx[0]);

    const int l32 = lane & 31, lq = lane >> 5;
    constexpr int TILE_STORES = C::MT * (C::NT / JP) * 4;  // stores of a wave per full tile
    static_assert(N_WAIT + TILE_STORES <= 63, "counter range");
    static_assert(OUT_BASE + NWAVES * 32 * OP <= 160 * 1024 / OCC, "ring and output pieces fit");
    unsigned char *const piece = smem + OUT_BASE + wave * (32 * OP);
    bool stores_behind = false;  // the previous tile issued exactly TILE_STORES stores (uniform)
    Tile cur = decode(0);
    int stg = 0;  // ring stage of the slab being multiplied
    for (int c_t = 0; c_t < my_tiles; ++c_t) {
        for (int c_k = 0; c_k < steps; ++c_k) {
            const char *const wsrc = i_w;
            const char *const xsrc = i_x;
            const int stg_fill = stg == 0 ? ST - 1 : stg - 1;  // stage of the slab ST-1 ahead
            const int stg_next = stg + 1 == ST ? 0 : stg + 1;
            const uint32_t dst = lds_base + stg_fill * C::STAGE_BYTES + wave * 1024;
#pragma unroll
            for (int kk = 0; kk < K0; ++kk) {
                if (kk + 1 < K0) {
                    read_frags(wa, xa, (kk + 1) * C::KSTEP, fw[(kk + 1) & 1], fx[(kk + 1) & 1]);
                } else {
                    if (loader) {
                        // behind the next slab's loads the counter holds the loads of the ST-2 slabs
                        // after it and, while the load of the next slab is older than the previous
                        // tile's output stores, those stores
                        if (c_k < ST - 2 && stores_behind)
                            __builtin_amdgcn_s_waitcnt(vmcnt_imm(N_WAIT + TILE_STORES));
                        else
                            __builtin_amdgcn_s_waitcnt(vmcnt_imm(N_WAIT));
                    }
                    __syncthreads();  // the next slab has landed, and everyone has left this one
                    // (at the end of a tile the next tile's first operands are read after its output
                    // has left: their registers are needed for that)
                    if (c_k + 1 < steps) {
                        stage_addrs(stg_next);
                        read_frags(wa, xa, 0, fw[0], fx[0]);
                    }
                    __builtin_amdgcn_sched_barrier(0);  // requested before this sub-step multiplies
                }
#pragma unroll
                for (int i = 0; i < C::MT; ++i)
#pragma unroll
                    for (int j = 0; j < C::NT; ++j) {
                        acc[i][j] = frag<CT>::mfma(fx[kk & 1][j], fw[kk & 1][i], acc[i][j]);
                        const int m = kk * PER_K0 + i * C::NT + j;  // MFMA index in the slab
                        if (kk + 1 < K0 && (m + 1) % STRIDE == 0 && m / STRIDE < L) {
                            if (loader) issue_one(wsrc, xsrc, dst, m / STRIDE);
                            __builtin_amdgcn_sched_barrier(0);
                        }
                    }
                if (kk == K0 - 2) {
                    // loads that did not get a slot above (fewer MFMAs than loads)
                    if (loader) {
#pragma unroll
                        for (int q = SLOTS / STRIDE; q < L; ++q) issue_one(wsrc, xsrc, dst, q);
                    }
                }
            }
            i_advance();
            if (c_k + 1 < steps) stg = stg_next;
        }
        // ---- the tile is complete.  In the accumulators a lane holds one output feature (row
        // l32 of the block) and, per group eg, 4 consecutive batch columns: written like that a
        // store touches 32 rows.  Through the wave's piece (OP bytes per row) eight neighbouring
        // lanes get the eight 16-byte parts of a row: whole lines, 8 rows per store.  LDS
        // accesses of one wave execute in order, so the piece needs no barrier.
        if constexpr (has_epi) {
            const bool gelu = ep.act == KSMM_ACT_GELU;
#pragma unroll
            for (int i = 0; i < C::MT; ++i) {
                const int mb = (wm * C::MT + i) * 32;
                const float bl = epi_bias<TY>(ep, ((size_t)cur.a_i * b + min(cur.m0 + mb + l32, b - 1)) * d + cur.d_i);
#pragma unroll
                for (int j = 0; j < C::NT; ++j)
#pragma unroll
                    for (int e = 0; e < 16; ++e) {
                        const float v = fmaf(acc[i][j][e], scale, bl);
                        acc[i][j][e] = gelu_if(gelu, v);
                    }
            }
        }
        const float st_scale = has_epi ? 1.f : scale;
        {
            unsigned char *const wr = piece + l32 * OP + (4 * OES) * lq;                  // + block, + 8 * OES * eg
            const unsigned char *const rd = piece + (lane >> 3) * OP + 16 * (lane & 7);  // + 8 * t rows
#pragma unroll
            for (int i = 0; i < C::MT; ++i)
#pragma unroll
                for (int jp = 0; jp < C::NT / JP; ++jp) {
                    const int mb = (wm * C::MT + i) * 32, nb = (wn * C::NT + jp * JP) * 32;
#pragma unroll
                    for (int jj = 0; jj < JP; ++jj)
#pragma unroll
                        for (int eg = 0; eg < 4; ++eg) {
                            const float16_t &ac = acc[i][jp * JP + jj];
                            if constexpr (OES == 4) {
                                const float4_t v = {ac[4 * eg] * st_scale, ac[4 * eg + 1] * st_scale,
                                                    ac[4 * eg + 2] * st_scale, ac[4 * eg + 3] * st_scale};
                                *(float4_t *)(wr + 32 * eg) = v;
                            } else {
                                const half4_t v = {(half_t)(ac[4 * eg] * st_scale), (half_t)(ac[4 * eg + 1] * st_scale),
                                                   (half_t)(ac[4 * eg + 2] * st_scale), (half_t)(ac[4 * eg + 3] * st_scale)};
                                *(half4_t *)(wr + 64 * jj + 16 * eg) = v;
                            }
                        }
                    __builtin_amdgcn_wave_barrier();
                    const int n = cur.n0 + nb + (16 / OES) * (lane & 7);
                    const int row = cur.m0 + mb + (lane >> 3);  // + 8 * t
                    TY *const dstp = y + (((size_t)cur.a_i * b + row) * d + cur.d_i) * batch + n;
#pragma unroll
                    for (int t = 0; t < 4; ++t) {
                        const uint4_t v = *(const uint4_t *)(rd + 8 * t * OP);
                        if (n < batch && (!MTAIL || row + 8 * t < b))
                            __builtin_nontemporal_store(v, (uint4_t *)(dstp + (size_t)8 * t * d * batch));
                    }
                    __builtin_amdgcn_wave_barrier();
                }
        }
        // a ragged tile skips stores: then wait the safe way
        stores_behind = cur.n0 + TN <= batch && (!MTAIL || cur.m0 + TM <= b);
        if (c_t + 1 < my_tiles) {
            clear_acc();
            cur = decode(c_t + 1);
            stg = stg + 1 == ST ? 0 : stg + 1;
            stage_addrs(stg);
            read_frags(wa, xa, 0, fw[0], fx[0]);
        }
    }
    if (loader) __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));  // repeats of the last slab must land before LDS is released
}

struct GemmInst {
    int combo, bs_last, dd, tm, tn, tk, threads, lds, epc;
    int ktail;  // takes c that is not a multiple of tk
    int wm;     // waves along the TM side
    int pers;   // persistent workgroups (per CU) with split memory roles (ks_gemm_pbf_kernel, ks_gemm_pbl_kernel)
    const void *fn[2];  // plain, with bias/activation
    int mtail;  // takes b that is not a multiple of tm (the last TM-tile is partly masked)
    int sp;     // d == 2 operands go to the 2:4 sparse MFMA as (k, d_i) pairs
};
// OCC_: waves per SIMD the register allocation must allow (2 lets two workgroups share a CU,
// so that one multiplies while the other stores its output tile)
#define GEMM_INST_K(COMBO_, CT_, TY_, BL_, DD_, TM_, TN_, TK_, WM_, WN_, ST_, OCC_, KT_)              \
    {COMBO_, BL_, DD_, TM_, TN_, TK_, 64 * WM_ * WN_,                                                \
     GemmCfg<CT_, BL_, DD_, TM_, TN_, TK_, WM_, WN_, ST_>::LDS_BYTES,                                 \
     GemmCfg<CT_, BL_, DD_, TM_, TN_, TK_, WM_, WN_, ST_>::EPC,                                       \
     KT_, WM_, 0, {(const void *)ks_gemm_kernel<CT_, TY_, BL_, DD_, TM_, TN_, TK_, WM_, WN_, ST_, OCC_, KT_, false>, \
                   (const void *)ks_gemm_kernel<CT_, TY_, BL_, DD_, TM_, TN_, TK_, WM_, WN_, ST_, OCC_, KT_, true>}}
#define GEMM_INST_PO(DD_, TM_, TN_, TK_, WM_, WN_, ST_, OCC_)                                          \
    {1, false, DD_, TM_, TN_, TK_, 64 * WM_ * WN_, GemmCfg<half_t, false, DD_, TM_, TN_, TK_, WM_, WN_, ST_>::LDS_BYTES, \
     8, 0, WM_, OCC_, {(const void *)ks_gemm_pbf_kernel<half_t, half_t, DD_, TM_, TN_, TK_, WM_, WN_, ST_, OCC_, false, false>, \
                       (const void *)ks_gemm_pbf_kernel<half_t, half_t, DD_, TM_, TN_, TK_, WM_, WN_, ST_, OCC_, true, false>}}
#define GEMM_INST_P(DD_, TM_, TN_, TK_, WM_, WN_, ST_) GEMM_INST_PO(DD_, TM_, TN_, TK_, WM_, WN_, ST_, 1)
// d == 2 through the 2:4 sparse MFMA (no operand split); `sp` tells the instances apart
#define GEMM_INST_PS(TM_, TN_, TK_, WM_, WN_, ST_, OCC_)                                               \
    {1, false, 2, TM_, TN_, TK_, 64 * WM_ * WN_, GemmCfg<half_t, false, 2, TM_, TN_, TK_, WM_, WN_, ST_>::LDS_BYTES, \
     8, 0, WM_, OCC_, {(const void *)ks_gemm_pbf_kernel<half_t, half_t, 2, TM_, TN_, TK_, WM_, WN_, ST_, OCC_, false, true>, \
                       (const void *)ks_gemm_pbf_kernel<half_t, half_t, 2, TM_, TN_, TK_, WM_, WN_, ST_, OCC_, true, true>}, 0, 1}
// OCC_: persistent workgroups per CU (4-wave tiles: two); MT_: partial last TM-tile
#define GEMM_INST_PLM(COMBO_, CT_, TY_, TM_, TN_, TK_, WM_, WN_, ST_, OCC_, MT_)                      \
    {COMBO_, true, 1, TM_, TN_, TK_, 64 * WM_ * WN_,                                                  \
     GemmCfg<CT_, true, 1, TM_, TN_, TK_, WM_, WN_, ST_>::LDS_BYTES + WM_ * WN_ * 32 * 144,           \
     GemmCfg<CT_, true, 1, TM_, TN_, TK_, WM_, WN_, ST_>::EPC, 0, WM_, OCC_,                          \
     {(const void *)ks_gemm_pbl_kernel<CT_, TY_, TM_, TN_, TK_, WM_, WN_, ST_, OCC_, MT_, false>,    \
      (const void *)ks_gemm_pbl_kernel<CT_, TY_, TM_, TN_, TK_, WM_, WN_, ST_, OCC_, MT_, true>}, MT_}
#define GEMM_INST_PL(COMBO_, CT_, TY_, TM_, TN_, TK_, WM_, WN_, ST_, OCC_)                            \
    GEMM_INST_PLM(COMBO_, CT_, TY_, TM_, TN_, TK_, WM_, WN_, ST_, OCC_, false)
#define GEMM_INST_T(COMBO_, CT_, TY_, BL_, DD_, TM_, TN_, TK_, WM_, WN_, ST_, OCC_)                   \
    GEMM_INST_K(COMBO_, CT_, TY_, BL_, DD_, TM_, TN_, TK_, WM_, WN_, ST_, OCC_, false)
#define GEMM_INST_O(COMBO_, CT_, BL_, DD_, TM_, TN_, TK_, WM_, WN_, ST_, OCC_)                        \
    GEMM_INST_T(COMBO_, CT_, CT_, BL_, DD_, TM_, TN_, TK_, WM_, WN_, ST_, OCC_)
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
    GEMM_INST(0, float, true, 1, 128, 128, 16, 2, 2, 4),
    GEMM_INST_O(0, float, true, 1, 128, 256, 16, 2, 2, 3, 2),
    GEMM_INST(0, float, true, 1, 256, 256, 16, 2, 2, 4),
    GEMM_INST(0, float, true, 1, 64, 256, 16, 1, 4, 4),
    // fp16, bs_first, d == 2: 4 waves with 128 x 64 (x 2 d_i) wave tiles: half the LDS operand
    // traffic per MFMA of the 8-wave tiles above
    GEMM_INST(1, half_t, false, 2, 256, 128, 32, 2, 2, 3),
    GEMM_INST(1, half_t, false, 2, 128, 256, 32, 1, 4, 3),
    // fp16, b a multiple of 64 only: last resort (variant -2), after the stream and k-loop tiles
    GEMM_INST(1, half_t, true, 1, 64, 256, 32, 1, 4, 3),
    GEMM_INST(1, half_t, false, 1, 64, 256, 32, 1, 4, 3),
    // e4m3 x e4m3 -> fp16, bs_last: the bytes go to LDS as they are and into the fp8 MFMA
    GEMM_INST_T(2, fp8_t, half_t, true, 1, 128, 256, 64, 2, 2, 3, 2),
    GEMM_INST_T(2, fp8_t, half_t, true, 1, 256, 256, 64, 2, 4, 4, 1),
    GEMM_INST_T(2, fp8_t, half_t, true, 1, 128, 128, 64, 2, 2, 4, 2),
    GEMM_INST_T(2, fp8_t, half_t, true, 1, 128, 256, 32, 2, 2, 4, 2),
    // bs_last, any c (partial last slab)
    GEMM_INST_K(1, half_t, half_t, true, 1, 128, 256, 32, 2, 2, 3, 2, true),
    GEMM_INST_K(1, half_t, half_t, true, 1, 64, 256, 32, 1, 4, 3, 1, true),
    GEMM_INST_K(0, float, float, true, 1, 128, 128, 16, 2, 2, 4, 1, true),
    GEMM_INST_K(0, float, float, true, 1, 64, 256, 16, 1, 4, 4, 1, true),
    GEMM_INST_K(2, fp8_t, half_t, true, 1, 128, 256, 32, 2, 2, 4, 2, true),
    // e4m3, b a multiple of 64 only
    GEMM_INST_T(2, fp8_t, half_t, true, 1, 64, 256, 64, 1, 4, 3, 2),
    GEMM_INST_K(2, fp8_t, half_t, true, 1, 64, 256, 64, 1, 4, 3, 2, true),
    // fp16, bs_first, d == 2: 16 waves on the 256 x 128 tile (4 per SIMD: more to issue from while
    // others wait at the slab barrier)
    GEMM_INST(1, half_t, false, 2, 256, 128, 32, 4, 4, 3),
    // fp16, bs_first, d == 2: persistent workgroups on the 2:4 sparse MFMA (the (k, d_i) pairs of an
    // input row go to the matrix cores as they are; listed ahead of the forms that split them, which
    // they beat by 3-4 %: (1,1536,384,2) at batch 25088 94.5 -> 90.9 us)
    GEMM_INST_PS(256, 128, 32, 4, 2, 3, 1),
    GEMM_INST_PS(128, 256, 32, 2, 4, 3, 1),
    // fp16, bs_first: persistent workgroups, loads and stores issued by different waves
    GEMM_INST_P(2, 256, 128, 32, 4, 2, 3),
    GEMM_INST_P(2, 128, 256, 32, 2, 4, 3),
    // persistent, bs_last
    GEMM_INST_PL(1, half_t, half_t, 256, 256, 32, 2, 4, 3, 1),
    GEMM_INST_PL(1, half_t, half_t, 128, 256, 32, 2, 4, 4, 1),
    GEMM_INST_PL(0, float, float, 128, 256, 16, 2, 4, 4, 1),
    GEMM_INST_PL(0, float, float, 256, 256, 16, 2, 4, 3, 1),
    GEMM_INST_PL(2, fp8_t, half_t, 256, 256, 64, 2, 4, 3, 1),
    GEMM_INST_PL(2, fp8_t, half_t, 128, 256, 64, 2, 4, 4, 1),
    // 4-wave tiles for b = 64, 192, ...: two persistent workgroups per CU
    GEMM_INST_PL(1, half_t, half_t, 64, 256, 32, 1, 4, 3, 2),
    GEMM_INST_PL(1, half_t, half_t, 64, 128, 32, 2, 2, 5, 2),
    GEMM_INST_PL(0, float, float, 64, 256, 16, 1, 4, 3, 2),
    GEMM_INST_PL(0, float, float, 64, 128, 16, 2, 2, 5, 2),
    // the same with a partly masked last TM-tile: b = 48, 80, 96, ... (variant -5 and the table)
    GEMM_INST_PLM(1, half_t, half_t, 64, 256, 32, 1, 4, 3, 2, true),
    GEMM_INST_PLM(1, half_t, half_t, 64, 128, 32, 2, 2, 5, 2, true),
    GEMM_INST_PLM(0, float, float, 64, 256, 16, 1, 4, 3, 2, true),
    GEMM_INST_PLM(0, float, float, 64, 128, 16, 2, 2, 5, 2, true),
    // fp16 bs_first d == 2: 4-wave tile, two persistent workgroups per CU (b = 64, 192, ...)
    GEMM_INST_PS(64, 128, 32, 1, 4, 3, 2),
    GEMM_INST_PO(2, 64, 128, 32, 1, 4, 3, 2),
    // fp16 bs_first d == 1: 4-wave tiles of 64 and 128 rows
    GEMM_INST_PO(1, 64, 256, 32, 1, 4, 3, 2),
    GEMM_INST_PO(1, 128, 256, 32, 2, 2, 3, 2),
    // e4m3: the 4-wave tiles, whole and masked
    GEMM_INST_PL(2, fp8_t, half_t, 64, 256, 64, 1, 4, 3, 2),
    GEMM_INST_PL(2, fp8_t, half_t, 64, 128, 64, 2, 2, 5, 2),
    GEMM_INST_PLM(2, fp8_t, half_t, 64, 256, 64, 1, 4, 3, 2, true),
    GEMM_INST_PLM(2, fp8_t, half_t, 64, 128, 64, 2, 2, 5, 2, true),
};
constexpr int GEMM_PF = 4;             // GemmCfg::PF
constexpr int N_GEMM_INSTS = sizeof(gemm_insts) / sizeof(GemmInst);

bool gemm_fits(const GemmInst &t, const Problem &p, int combo)
{
    if (t.combo != combo || t.bs_last != p.bs_last) return false;
    if ((p.b % t.tm && !t.mtail) || (p.c % t.tk && !t.ktail)) return false;
    if (p.b % t.epc) return false;  // 16-byte weight vectors
    if (p.bs_last) {
        if (p.batch % t.epc || p.batch < t.epc) return false;
    } else {
        if (p.d != t.dd) return false;
        if (((int64_t)p.a * p.c * p.d) % t.epc || ((int64_t)p.c * p.d) % t.epc) return false;
        if (t.dd == 2 && (((int64_t)p.a * p.b * p.d) % 2)) return false;
    }
    // per-lane byte offsets of the direct-to-LDS loads are 32-bit
    const int64_t es = 16 / t.epc, lim = 0xffffffffLL;
    if ((int64_t)t.dd * p.c * p.b * es >= lim) return false;
    if (p.bs_last ? ((int64_t)t.tk * p.d * p.batch + p.batch) * es >= lim
                  : ((int64_t)t.tn * p.a * p.c * p.d + (int64_t)p.c * p.d) * es >= lim)
        return false;
    return true;
}

}  // namespace

int gemm_inst_count() { return N_GEMM_INSTS; }

uint32_t gemm_inst_id(int i)
{
    if (i < 0 || i >= N_GEMM_INSTS) return 0;
    const GemmInst &t = gemm_insts[i];
    // threads and the LDS footprint stand for the wave grid and the ring depth
    const int v[13] = {t.combo, t.bs_last, t.dd, t.tm, t.tn, t.tk, t.threads, t.lds, t.ktail, t.wm, t.pers, t.mtail, t.sp};
    return inst_hash('G', v, t.sp ? 13 : t.mtail ? 12 : 11);  // (ids of the other instances predate the fields)
}

// variant: index into the instance table; -1: first that fits with enough workgroups to fill
// the chip (TM = 64 tiles only where nothing better exists); -4: the TM = 64 tiles, same
// condition; -5: the persistent tiles with a masked last TM-tile, for b beyond one tile and
// three tiles per persistent workgroup (they beat the k-loop tiles on 72 of 80 such patterns of
// the reference's list, up to 2x); -6: the 4-wave persistent batch-size-first tile; -2: first
// that fits
int gemm_run(const Problem &p, int variant, bool launch, ksmm_tile *tile)
{
    const int combo = combo_of(p.x_dtype, p.w_dtype, p.y_dtype);
    int pick = -1;
    for (int i = 0; i < N_GEMM_INSTS && variant == -6; ++i) {
        // -6: the 4-wave persistent batch-size-first tile (d == 2, b a multiple of 64) from half a
        // chip of tiles: 1.1-2.5x faster than the tile_bf and 64 x 256 GEMM tiles it
        // replaces ((1,192,192,2) 18.1 -> 12.5 us, (1,64,256,2) 21.5 -> 8.5, (2,320,64,2) 31.9 -> 17.2)
        const GemmInst &t = gemm_insts[i];
        if (!t.pers || t.bs_last || t.tm != 64 || !gemm_fits(t, p, combo)) continue;
        const int64_t tiles = (int64_t)p.a * (p.b / t.tm) * ((p.batch + t.tn - 1) / t.tn);
        if (tiles < 128) continue;  // (measured down to 196 tiles: still 2.5x)
        pick = i;
        break;
    }
    for (int i = 0; i < N_GEMM_INSTS && variant == -5; ++i) {
        const GemmInst &t = gemm_insts[i];
        if (!t.mtail || p.b <= t.tm || !gemm_fits(t, p, combo)) continue;
        const int64_t tiles = (int64_t)p.a * p.d * ((p.b + t.tm - 1) / t.tm) * ((p.batch + t.tn - 1) / t.tn);
        if (tiles < 3 * 256 * t.pers) continue;
        pick = i;
        break;
    }
    for (int i = 0; i < N_GEMM_INSTS && variant != -5 && variant != -6; ++i) {
        if (variant >= 0 && variant != i) continue;
        const GemmInst &t = gemm_insts[i];
        // TM = 64 tiles are a first choice only where nothing better exists: e4m3 (no stream
        // kernels) and partial K slabs; otherwise the stream and weight-stationary tiles come
        // first, then these (variant -4: 15-25 % faster than the k-loop tiles on 180 patterns
        // of the reference's list), then the k-loop tiles
        if (variant < 0 && (t.pers || t.mtail)) continue;  // taken below (persistent form of the pick) or by variant -5
        if (variant == -1 && t.tm < 128 && t.combo != 2 && !(t.ktail && p.c % t.tk)) continue;
        if (variant == -4 && t.tm >= 128) continue;  // -4: the TM = 64 tiles, after stream / weight-stationary
        // few K slabs: the 8-wave 256 x 256 tiles spend their time in prologue and epilogue; two
        // 4-wave workgroups per CU do better (measured on the (., 256, 64, .) fp16 patterns: 10 %)
        if (variant == -1 && t.threads == 512 && t.dd == 1 && p.c <= 128) continue;
        if (!gemm_fits(t, p, combo)) continue;
        if (variant == -1 || variant == -4) {
            // the big tiles only pay when they still fill the chip
            const int64_t groups = t.dd == 1 ? (int64_t)p.a * p.d : p.a;
            const int64_t wgs = groups * (p.b / t.tm) * ((p.batch + t.tn - 1) / t.tn);
            if (wgs < 256) continue;
        }
        pick = i;
        break;
    }
    if (pick < 0) return KSMM_ERR_BAD_ALGO;
    if (variant < 0 && variant > -5 && !gemm_insts[pick].pers) {
        // three or more tiles per CU: the persistent forms save the per-tile prologue and keep the
        // load stream running (8 % on (1,1536,384,2) fp16 batch-size-first at batch 25088 with the
        // tile of the pick; batch-size-last: 12 % with the first persistent tile that still
        // gives three tiles per CU, 5 % on fp32 (1,768,192,16))
        const GemmInst &o = gemm_insts[pick];
        for (int i = 0; i < N_GEMM_INSTS; ++i) {
            const GemmInst &q = gemm_insts[i];
            if (!q.pers || q.mtail || q.combo != o.combo || q.bs_last != o.bs_last || q.dd != o.dd) continue;
            if (!q.bs_last && (q.tm != o.tm || q.tk != o.tk || (q.tn != o.tn && q.tm > 64))) continue;
            if (!gemm_fits(q, p, combo)) continue;
            const int64_t groups = q.dd == 1 ? (int64_t)p.a * p.d : p.a;
            if (groups * (p.b / q.tm) * ((p.batch + q.tn - 1) / q.tn) < 3 * 256 * q.pers) continue;
            pick = i;
            break;
        }
    }
    const GemmInst &t = gemm_insts[pick];
    const int m_tiles = (p.b + t.tm - 1) / t.tm;
    const int64_t n_tiles = (p.batch + t.tn - 1) / t.tn;
    const int64_t groups = t.dd == 1 ? (int64_t)p.a * p.d : p.a;
    const int64_t blocks = groups * m_tiles * n_tiles;
    int64_t grid = (blocks + 7) / 8 * 8;
    if (t.pers && grid > 256 * t.pers) grid = 256 * t.pers;  // persistent workgroups: pers per CU
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
    Epi ep = epi_of(p);
    const void *fn = t.fn[ep.bias != nullptr || ep.act != KSMM_ACT_NONE];
    if (ensure_dynamic_lds(fn, t.lds) != KSMM_OK) return KSMM_ERR_LAUNCH;
    int batch_i = (int)p.batch, n_tiles_i = (int)n_tiles, blocks_i = (int)blocks, m_tiles_i = m_tiles;
    // L2 prefetch for the successor workgroup (bs_last): when the TM-tiles of an input tile can
    // cover it with PF lines per thread; distance = workgroups resident on an XCD (32 CUs)
    int pf_dist = 0;
    if (p.bs_last && m_tiles >= 2) {
        const int es = 16 / t.epc, resident = t.lds <= 80 * 1024 ? 64 : 32;  // workgroups per XCD
        const int64_t lines = ((int64_t)p.c + m_tiles - 1) / m_tiles * (t.tn * es / 128);
        // current and prefetched input tiles of an XCD must leave room in its 4 MB L2
        const int64_t in_l2 = 2 * (int64_t)p.c * t.tn * es * ((resident + m_tiles - 1) / m_tiles);
        if (lines <= (int64_t)GEMM_PF * t.threads && in_l2 <= (5 << 19)) pf_dist = resident;
    }
    if (t.pers) {
        void *pargs[] = {(void *)&p.x, (void *)&p.w, (void *)&p.y, &batch_i, (void *)&p.a, (void *)&p.b,
                         (void *)&p.c, (void *)&p.d, &ep, &m_tiles_i, &n_tiles_i, &blocks_i};
        hipError_t pe = hipLaunchKernel(fn, dim3((unsigned)grid), dim3(t.threads), pargs, t.lds, p.stream);
        return pe == hipSuccess ? KSMM_OK : KSMM_ERR_LAUNCH;
    }
    void *args[] = {(void *)&p.x, (void *)&p.w, (void *)&p.y, &batch_i, (void *)&p.a, (void *)&p.b,
                    (void *)&p.c, (void *)&p.d, &ep, &m_tiles_i, &n_tiles_i, &blocks_i, &pf_dist};
    hipError_t e = hipLaunchKernel(fn, dim3((unsigned)grid), dim3(t.threads), args, t.lds, p.stream);
    return e == hipSuccess ? KSMM_OK : KSMM_ERR_LAUNCH;
}

}  // namespace ksmm
