// "Stream" kernels of the tile family: the bandwidth-bound path for mid-sized b x c blocks.
//
// A persistent workgroup owns one (a_i, d_i) block and every wgs-th tile of batch columns.
// The b x c weight block is staged through LDS once and then lives in registers as MFMA
// operands.  Input tiles (the whole c extent x TN batch columns) are brought in with
// direct-to-LDS loads (global_load_lds_dwordx4: no staging registers), ST tiles deep, so that
// a CU keeps ~100 KB of HBM reads in flight: enough to cover the memory latency at 8 TB/s
// with one workgroup per CU.  The output tile is transposed through LDS and written with
// 16-byte stores along the contiguous axis.
//
// Direct-to-LDS loads write 64 consecutive 16-byte chunks per wave instruction, so tiles are
// stored without row padding; bank conflicts are avoided with an XOR swizzle of the chunk
// index by the row index instead (the swizzle is applied to the *global* address each lane
// fetches, and again by the MFMA operand reads).
//
// The loads are issued from inline assembly and tracked by hand: the kernel waits with
// s_waitcnt vmcnt(N) where N is the number of vector-memory instructions issued after the
// loads of the tile it is about to read (the counter retires in order).  The loop issues the
// same number of loads (L) and stores (S) per iteration in every wave, which makes N a
// compile-time constant.
//
// MFMA roles: the axis that is contiguous in the output runs along the MFMA *rows*, so that a
// lane holds 4 consecutive output elements and the LDS transpose takes 8/16-byte writes:
//   bs_last : A = X (rows = batch),   B = W (lanes = outputs)
//   bs_first: A = W (rows = outputs), B = X (lanes = batch)      (d == 1)
//
// Reference counterpart: kernel_bs_{first,last}_{float,half2,half4}
// (src/ksmm_py/layer/kronecker_sparse/template_kernels_float.cuh:85-491,
//  template_kernels_half.cuh:103-1092).
#include "ksmm_mfma.h"


namespace ksmm {

namespace {

// s_waitcnt immediate for gfx9-family encodings: vmcnt in bits [3:0] and [15:14], expcnt and
// lgkmcnt left at their maxima (no wait)
constexpr int vmcnt_imm(int n) { return (n & 15) | (7 << 4) | (15 << 8) | (((n >> 4) & 3) << 14); }

// one direct-to-LDS load: lane i of the wave writes its 16 bytes to lds_addr + 16 * i
__device__ __forceinline__ void dma16(const void *gptr, uint32_t lds_addr)
{
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off"
                 :
                 : "v"(gptr), "s"(lds_addr)
                 : "memory", "m0");
}

template <typename CT, typename TW, bool BS_LAST, int BB, int CC, int TN, int WM, int WN, int ST>
struct StreamCfg {
    static constexpr int THREADS = 64 * WM * WN;
    static constexpr int ES = (int)sizeof(CT);
    static constexpr int EPC = 16 / ES;  // elements per 16-byte chunk
    static constexpr int KSTEP = compute<CT>::KSTEP;
    static constexpr int MT = BB / WM / 32, NT = TN / WN / 32, KS = CC / KSTEP;
    // input stage: bs_last CC rows of TN elements (k-outer); bs_first TN rows of CC (k-inner)
    static constexpr int X_ROWS = BS_LAST ? CC : TN, X_COLS = BS_LAST ? TN : CC;
    static constexpr int X_CPR = X_COLS / EPC;
    static constexpr int X_CHUNKS = X_ROWS * X_CPR, L = X_CHUNKS / THREADS;
    static constexpr int X_STAGE_BYTES = X_CHUNKS * 16;
    // output tile: bs_last BB rows of TN; bs_first TN rows of BB; rows padded by one chunk
    static constexpr int O_ROWS = BS_LAST ? BB : TN, O_COLS = BS_LAST ? TN : BB;
    static constexpr int O_CPR = O_COLS / EPC, O_LD = O_COLS + EPC;
    static constexpr int O_CHUNKS = O_ROWS * O_CPR, S = O_CHUNKS / THREADS;
    static constexpr int O_BYTES = O_ROWS * O_LD * ES;
    static constexpr int LDW = pads<CT>::outer(BB);
    static constexpr int W_BYTES = CC * LDW * ES;
    static constexpr int W_EPV = stage<TW, CT>::EPV, W_VECS = CC * BB / W_EPV;
    // LDS map: [weight staging, later the output tile][ST input stages]; the stages do not
    // overlap the weight staging area, so the first input tiles are requested before the
    // weights are staged
    static constexpr int HEAD_BYTES = ((W_BYTES > O_BYTES ? W_BYTES : O_BYTES) + 1023) / 1024 * 1024;
    // behind the stages: the bias of the block's BB outputs as floats (zeros without a bias)
    static constexpr int BIAS_OFF = HEAD_BYTES + ST * X_STAGE_BYTES;
    static constexpr int LDS_BYTES = BIAS_OFF + BB * 4;
    static_assert(BB <= THREADS, "one bias value per thread");
    // vector-memory instructions issued after the loads of the tile being waited for
    static constexpr int N_SAFE = (ST - 1) * L;             // while fewer than ST-1 tiles were stored
    static constexpr int N_FULL = (ST - 1) * (L + S);       // steady state
    static_assert(BB % (32 * WM) == 0 && TN % (32 * WN) == 0 && CC % KSTEP == 0, "wave tiling");
    static_assert(X_CHUNKS % THREADS == 0 && O_CHUNKS % THREADS == 0, "every wave issues L loads and S stores");
    static_assert(X_CPR % (ES == 2 ? 8 : 16) == 0, "swizzle group");
    static_assert(N_FULL <= 63, "vmcnt range");
    static_assert(LDS_BYTES <= 160 * 1024, "LDS");
    static_assert(BB % W_EPV == 0, "weight vectors");
};

// Swizzle of the 16-byte chunk index inside a row (CPR chunks) of the input stage.  LDS has 64
// banks of 4 bytes; a ds_read_b64 is served 32 lanes per clock, a ds_read_b128 16 lanes:
//  k-outer fp16: the 32 lanes of a transpose load read 4 rows x 64 bytes -> the 64-byte group
//  index is XORed with row & 3 (rows of 128 bytes alternate bank halves already: row / 2 & 1);
//  k-outer fp32: a ds_read_b32 wave reads 2 rows x 128 bytes -> XOR the 128-byte half;
//  k-inner: 16 lanes read one chunk of 16 consecutive rows -> rows of 128 or 384 bytes
//  alternate bank halves, the chunk is XORed with row / 2; rows of 256 bytes with row & 15.
template <typename CT, bool BS_LAST, int CPR> __device__ __forceinline__ int swz(int row)
{
    if (BS_LAST) return sizeof(CT) == 2 ? (CPR >= 16 ? 4 * (row & 3) : 4 * ((row >> 1) & 1)) : 8 * (row & 1);
    return CPR % 16 == 0 ? (row & 15) : ((row >> 1) & 7);
}

// MFMA operand of the input from a swizzled stage
template <typename CT, bool BS_LAST, int X_COLS> struct xfrag;
template <int X_COLS> struct xfrag<half_t, true, X_COLS> {  // k-outer, transpose loads
    __device__ static __forceinline__ half8_t get(const half_t *s, int idx0, int k0, int lane)
    {
        const int kq = lane >> 5, i16 = lane & 15, hs = (lane >> 4) & 1;
        const int row = k0 + 8 * kq + (i16 >> 2);  // + 4 for the second load: same row & 3
        const int chunk = (idx0 >> 3) + 2 * hs + ((i16 & 3) >> 1);
        const int off = ((chunk ^ swz<half_t, true, X_COLS / 8>(row)) << 3) + 4 * (i16 & 1);
        typedef short4_t __attribute__((address_space(3))) * lds_ptr;
        const half_t *p = s + row * X_COLS + off;
        short4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(p));
        short4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(p + 4 * X_COLS));
        typedef short short8_t __attribute__((ext_vector_type(8)));
        short8_t r = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
        return __builtin_bit_cast(half8_t, r);
    }
};
template <int X_COLS> struct xfrag<half_t, false, X_COLS> {  // k-inner, 16-byte loads
    __device__ static __forceinline__ half8_t get(const half_t *s, int idx0, int k0, int lane)
    {
        const int row = idx0 + (lane & 31);
        const int chunk = (k0 >> 3) + (lane >> 5);
        return *(const half8_t *)(s + row * X_COLS + ((chunk ^ swz<half_t, false, X_COLS / 8>(row)) << 3));
    }
};
template <int X_COLS> struct xfrag<float, true, X_COLS> {  // k-outer, 4-byte loads
    __device__ static __forceinline__ float get(const float *s, int idx0, int k0, int lane)
    {
        const int row = k0 + (lane >> 5), col = idx0 + (lane & 31);
        return s[row * X_COLS + ((((col >> 2) ^ (8 * (row & 1))) << 2) | (col & 3))];
    }
};

template <typename CT, typename TW, typename TY, bool BS_LAST, int BB, int CC, int TN, int WM, int WN,
          int ST>
__global__ __launch_bounds__(64 * WM * WN) void ks_stream_kernel(const CT *__restrict__ x,
                                                                const TW *__restrict__ w,
                                                                TY *__restrict__ y, int batch, int a,
                                                                int d, Epi ep, int wgs_per_group)
{
    const float scale = ep.scale;
    const bool has_epi = ep.bias != nullptr || ep.act != KSMM_ACT_NONE;  // uniform
    typedef StreamCfg<CT, TW, BS_LAST, BB, CC, TN, WM, WN, ST> C;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    const int g = blockIdx.x / wgs_per_group;  // a_i * d + d_i
    const int s = blockIdx.x - g * wgs_per_group;
    // Tiles of TN batch columns (rows for bs_first), dealt round-robin over the workgroups of
    // the block: at any time the workgroups of a block work on neighbouring tiles, so the row
    // pieces in flight are contiguous in memory (and TN-aligned).
    const int n_tiles = (batch + TN - 1) / TN;
    if (s >= n_tiles) return;
    const int c_begin = s * TN, c_end = batch, step = wgs_per_group * TN;
    const int a_i = g / d, d_i = g - a_i * d;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave / WN, wn = wave % WN;
    const size_t in_size = (size_t)a * CC * d, out_size = (size_t)a * BB * d;

    // ---- direct-to-LDS loads of one input tile ---------------------------------------------
    const uint32_t lds_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char *)smem;
    const CT *xg = BS_LAST ? x + ((size_t)a_i * CC * d + d_i) * batch : x + (size_t)a_i * CC;
    const size_t x_kstride = (size_t)d * batch;
    // per-lane part of the global address of load i: fixed over tiles except for the column/row base
    size_t goff[C::L];  // element offset relative to (xg + tile base)
    int gcol[C::L];     // bs_last: column inside the tile; bs_first: row inside the tile
#pragma unroll
    for (int i = 0; i < C::L; ++i) {
        const int q = tid + i * C::THREADS;
        const int row = q / C::X_CPR, pc = q % C::X_CPR;
        const int col = (pc ^ swz<CT, BS_LAST, C::X_CPR>(row)) * C::EPC;  // logical column of this chunk
        if (BS_LAST) {
            goff[i] = (size_t)row * x_kstride;
            gcol[i] = col;
        } else {
            goff[i] = (size_t)col;
            gcol[i] = row;
        }
    }
    auto issue = [&](int n0, int stg) {
        const uint32_t dst = lds_base + C::HEAD_BYTES + stg * C::X_STAGE_BYTES + wave * 1024;
#pragma unroll
        for (int i = 0; i < C::L; ++i) {
            const CT *p;
            if (BS_LAST)
                p = xg + goff[i] + min(n0 + gcol[i], c_end - C::EPC);  // clamped: never past the share
            else
                p = xg + (size_t)min(n0 + gcol[i], c_end - 1) * in_size + goff[i];
            dma16(p, dst + i * (C::THREADS * 16));
        }
    };

    CT *const out = (CT *)smem;
    const int l32 = lane & 31, lq = lane >> 5;
    const int n_iters = (n_tiles - s + wgs_per_group - 1) / wgs_per_group;
    // ---- weights: global -> LDS (as stored, c x b, padded rows) -> registers ---------------
    // Their loads go out before the input tiles' so that they are not queued behind them; the
    // prologue tiles (ST-1 in flight; tiles past the end repeat the last one and are never
    // read) follow at once, and staging the weights overlaps with their flight.
    {
        CT *wl = (CT *)smem;
        const TW *wg = w + (size_t)g * CC * BB;
        // all loads first, then all LDS writes: one memory latency instead of one per vector
        constexpr int W_PER_T = (C::W_VECS + C::THREADS - 1) / C::THREADS;
        stage<TW, CT> r[W_PER_T];
#pragma unroll
        for (int i = 0; i < W_PER_T; ++i) {
            const int v = min(tid + i * C::THREADS, C::W_VECS - 1);
            r[i].load(wg + (size_t)(v / (BB / C::W_EPV)) * BB + (v % (BB / C::W_EPV)) * C::W_EPV);
        }
        const float bias_v = tid < BB ? epi_bias<TY>(ep, ((size_t)a_i * BB + tid) * d + d_i) : 0.f;
#pragma unroll
        for (int p = 0; p < ST - 1; ++p) issue(c_begin + min(p, n_iters - 1) * step, p);
        if (tid < BB) ((float *)(smem + C::BIAS_OFF))[tid] = bias_v;
#pragma unroll
        for (int i = 0; i < W_PER_T; ++i) {
            const int v = min(tid + i * C::THREADS, C::W_VECS - 1);
            r[i].store(wl + (v / (BB / C::W_EPV)) * C::LDW + (v % (BB / C::W_EPV)) * C::W_EPV);
        }
        __syncthreads();
    }
    typename frag<CT>::type wreg[C::MT][C::KS];
#pragma unroll
    for (int i = 0; i < C::MT; ++i)
#pragma unroll
        for (int ks = 0; ks < C::KS; ++ks)
            wreg[i][ks] = frag<CT>::k_outer((const CT *)smem, C::LDW, (wm * C::MT + i) * 32, ks * C::KSTEP, lane);
    __syncthreads();  // the staging area becomes the output tile from here on


    for (int it = 0; it < n_iters; ++it) {
        const int n0 = c_begin + it * step;
        const int n_stop = min(n0 + TN, c_end);  // columns (rows) this tile stores
        issue(c_begin + min(it + ST - 1, n_iters - 1) * step, (it + ST - 1) % ST);
        if (it >= ST - 1)
            __builtin_amdgcn_s_waitcnt(vmcnt_imm(C::N_FULL));
        else
            __builtin_amdgcn_s_waitcnt(vmcnt_imm(C::N_SAFE));
        __syncthreads();  // tile `it` has landed for every wave

        const CT *xb = (const CT *)(smem + C::HEAD_BYTES + (it % ST) * C::X_STAGE_BYTES);
        float16_t acc[C::MT][C::NT];
#pragma unroll
        for (int i = 0; i < C::MT; ++i)
#pragma unroll
            for (int j = 0; j < C::NT; ++j)
#pragma unroll
                for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;
        // all operand reads of the tile are issued before the first MFMA: with one wave per
        // SIMD nothing else would hide the LDS latency
        typename frag<CT>::type fx[C::KS][C::NT];
#pragma unroll
        for (int ks = 0; ks < C::KS; ++ks)
#pragma unroll
            for (int j = 0; j < C::NT; ++j)
                fx[ks][j] = xfrag<CT, BS_LAST, C::X_COLS>::get(xb, (wn * C::NT + j) * 32, ks * C::KSTEP, lane);
#pragma unroll
        for (int ks = 0; ks < C::KS; ++ks)
#pragma unroll
            for (int i = 0; i < C::MT; ++i)
#pragma unroll
                for (int j = 0; j < C::NT; ++j)
                    acc[i][j] = BS_LAST ? frag<CT>::mfma(fx[ks][j], wreg[i][ks], acc[i][j])
                                        : frag<CT>::mfma(wreg[i][ks], fx[ks][j], acc[i][j]);
        // ---- accumulators -> LDS output tile: out[lane index][4 consecutive row indices] ----
#pragma unroll
        for (int i = 0; i < C::MT; ++i)
#pragma unroll
            for (int j = 0; j < C::NT; ++j) {
                const int mb = (wm * C::MT + i) * 32, nb = (wn * C::NT + j) * 32;
                // bs_last: rows = batch, lanes = outputs -> out[m][n..n+3]
                // bs_first: rows = outputs, lanes = batch -> out[n][m..m+3]
                const int orow = (BS_LAST ? mb : nb) + l32;
                const int ocol0 = (BS_LAST ? nb : mb) + 4 * lq;
#pragma unroll
                for (int eg = 0; eg < 4; ++eg) {
                    CT *dst = out + orow * C::O_LD + ocol0 + 8 * eg;
                    if (has_epi) {
                        // output index of element u: bs_last the lane's row, bs_first 4 consecutive ones
                        const float *bs = (const float *)(smem + C::BIAS_OFF);
                        float v[4];
#pragma unroll
                        for (int u = 0; u < 4; ++u)
                            v[u] = epi_finish(ep, acc[i][j][4 * eg + u], BS_LAST ? bs[orow] : bs[ocol0 + 8 * eg + u]);
                        if constexpr (sizeof(CT) == 2)
                            *(half4_t *)dst = half4_t{(half_t)v[0], (half_t)v[1], (half_t)v[2], (half_t)v[3]};
                        else
                            *(float4_t *)dst = float4_t{v[0], v[1], v[2], v[3]};
                    } else if constexpr (sizeof(CT) == 2) {
                        half4_t hv = {(half_t)(acc[i][j][4 * eg] * scale), (half_t)(acc[i][j][4 * eg + 1] * scale),
                                      (half_t)(acc[i][j][4 * eg + 2] * scale), (half_t)(acc[i][j][4 * eg + 3] * scale)};
                        *(half4_t *)dst = hv;
                    } else {
                        float4_t fv = {acc[i][j][4 * eg] * scale, acc[i][j][4 * eg + 1] * scale,
                                       acc[i][j][4 * eg + 2] * scale, acc[i][j][4 * eg + 3] * scale};
                        *(float4_t *)dst = fv;
                    }
                }
            }
        __syncthreads();
        // ---- LDS output tile -> global, 16 bytes per lane along the contiguous axis --------
#pragma unroll
        for (int i = 0; i < C::S; ++i) {
            const int q = tid + i * C::THREADS;
            const int orow = q / C::O_CPR, oc = (q % C::O_CPR) * C::EPC;
            const uint4_t v = *(const uint4_t *)(out + orow * C::O_LD + oc);
            // the store is issued by every wave in every iteration (vmcnt bookkeeping); lanes
            // outside the share are masked off
            if (BS_LAST) {
                const int n = n0 + oc;
                TY *dst = y + ((size_t)(a_i * BB + orow) * d + d_i) * batch + min(n, c_end - C::EPC);
                if (n < n_stop) *(uint4_t *)dst = v;  // 128/256-byte row pieces: plain stores measured faster
            } else {
                const int n = n0 + orow;
                TY *dst = y + (size_t)min(n, c_end - 1) * out_size + (size_t)a_i * BB + oc;
                // whole rows of b outputs: streaming (nontemporal) stores measured faster
                if (n < n_stop) __builtin_nontemporal_store(v, (uint4_t *)dst);
            }
        }
    }
    // direct-to-LDS loads of the repeated last tile may still be in flight: they must land
    // before this workgroup's LDS is handed to another one
    __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));
}

struct StreamInst {
    int combo, bs_last, bb, cc, tn, threads, lds, epc;
    int per_cu;  // persistent workgroups per CU the heuristic launches; 0: only when forced
    int wm;      // waves along the output side
    const void *fn;
};
#define STREAM_INST(COMBO_, CT_, TW_, BL_, BB_, CC_, TN_, WM_, WN_, ST_, PER_CU_)                     \
    {COMBO_, BL_, BB_, CC_, TN_, 64 * WM_ * WN_,                                                     \
     StreamCfg<CT_, TW_, BL_, BB_, CC_, TN_, WM_, WN_, ST_>::LDS_BYTES,                               \
     StreamCfg<CT_, TW_, BL_, BB_, CC_, TN_, WM_, WN_, ST_>::EPC, PER_CU_, WM_,                       \
     (const void *)ks_stream_kernel<CT_, TW_, CT_, BL_, BB_, CC_, TN_, WM_, WN_, ST_>}
// The first instance that fits a problem is the default; the order and the workgroups-per-CU
// column come from sweeps at batch 25088 on MI355X.
#define STREAM_SET_H(COMBO_, TW_)                                                                     \
    STREAM_INST(COMBO_, half_t, TW_, true, 192, 192, 64, 2, 2, 3, 1),                                \
        STREAM_INST(COMBO_, half_t, TW_, false, 192, 192, 64, 2, 2, 3, 1),                           \
        STREAM_INST(COMBO_, half_t, TW_, true, 64, 64, 128, 1, 4, 3, 1),                             \
        STREAM_INST(COMBO_, half_t, TW_, false, 64, 64, 64, 1, 2, 3, 3),                             \
        STREAM_INST(COMBO_, half_t, TW_, true, 128, 128, 64, 2, 2, 4, 1),                            \
        STREAM_INST(COMBO_, half_t, TW_, false, 128, 128, 64, 2, 2, 4, 1),                           \
        STREAM_INST(COMBO_, half_t, TW_, true, 64, 64, 128, 1, 4, 5, 1),                             \
        STREAM_INST(COMBO_, half_t, TW_, false, 64, 64, 128, 1, 4, 5, 1),                            \
        STREAM_INST(COMBO_, half_t, TW_, true, 64, 64, 64, 1, 2, 6, 2),                              \
        STREAM_INST(COMBO_, half_t, TW_, false, 64, 64, 64, 1, 2, 6, 2),                             \
        STREAM_INST(COMBO_, half_t, TW_, false, 64, 64, 128, 1, 4, 3, 2),                            \
        STREAM_INST(COMBO_, half_t, TW_, true, 64, 64, 64, 1, 2, 3, 3)
const StreamInst stream_insts[] = {
    // 192 x 192 blocks on 12 waves (three per SIMD: operand reads, MFMAs and stores of different
    // waves overlap): batch-size-first (4,192,192,1) at batch 25088 16.7 us against 19.7 on 4
    // waves; batch-size-last gains nothing (forced or from the table only), nor do 6 waves
    STREAM_INST(1, half_t, half_t, false, 192, 192, 64, 6, 2, 3, 1),
    STREAM_INST(3, half_t, fp8_t, false, 192, 192, 64, 6, 2, 3, 1),
    STREAM_INST(1, half_t, half_t, true, 192, 192, 64, 6, 2, 3, 0),
    STREAM_INST(1, half_t, half_t, false, 192, 192, 64, 3, 2, 3, 0),
    STREAM_SET_H(1, half_t),
    STREAM_SET_H(3, fp8_t),
    // fp32: slower than the wave family on every block shape measured so far; forced use only
    STREAM_INST(0, float, float, true, 64, 64, 64, 1, 2, 4, 0),
    STREAM_INST(0, float, float, true, 64, 64, 128, 1, 4, 3, 0),
    STREAM_INST(0, float, float, true, 128, 128, 64, 2, 2, 2, 0),
    // more waves per block (forced or from the table)
    STREAM_INST(1, half_t, half_t, false, 128, 128, 64, 4, 2, 4, 0),
    STREAM_INST(1, half_t, half_t, true, 128, 128, 64, 4, 2, 4, 0),
    STREAM_INST(1, half_t, half_t, false, 64, 64, 64, 2, 2, 3, 0),
    STREAM_INST(1, half_t, half_t, true, 64, 64, 64, 2, 2, 3, 0),
    STREAM_INST(1, half_t, half_t, false, 64, 64, 128, 2, 4, 3, 0),
    STREAM_INST(1, half_t, half_t, true, 64, 64, 128, 2, 4, 3, 0),
};
constexpr int N_STREAM_INSTS = sizeof(stream_insts) / sizeof(StreamInst);

bool stream_fits(const StreamInst &t, const Problem &p, int combo)
{
    if (t.combo != combo || t.bs_last != p.bs_last) return false;
    if (p.b != t.bb || p.c != t.cc) return false;
    // every global access is a 16-byte vector along the contiguous axis
    if (p.bs_last) {
        if (p.batch % t.epc) return false;
    } else {
        if (p.d != 1) return false;
        if (((int64_t)p.a * p.c) % t.epc || ((int64_t)p.a * p.b) % t.epc) return false;
    }
    return true;
}

}  // namespace

int stream_inst_count() { return N_STREAM_INSTS; }

uint32_t stream_inst_id(int i)
{
    if (i < 0 || i >= N_STREAM_INSTS) return 0;
    const StreamInst &t = stream_insts[i];
    // threads and the LDS footprint stand for the wave grid and the number of stages
    const int v[8] = {t.combo, t.bs_last, t.bb, t.cc, t.tn, t.threads, t.lds, t.wm};
    return inst_hash('S', v, 8);
}

// variant: bits 0-6 instance (0x7f: first that fits), bits 7.. workgroups per group (0: heuristic)
int stream_run(const Problem &p, int variant, bool launch, ksmm_tile *tile)
{
    const int combo = combo_of(p.x_dtype, p.w_dtype, p.y_dtype);
    const int want = variant < 0 ? 0x7f : (variant & 0x7f);
    int64_t wgs = variant < 0 ? 0 : (variant >> 7);
    static_assert(N_STREAM_INSTS < 0x7f, "the variant's instance field must hold every index");
    if (want != 0x7f && want >= N_STREAM_INSTS) return KSMM_ERR_BAD_ALGO;
    int pick = -1;
    for (int i = 0; i < N_STREAM_INSTS; ++i) {
        if (want != 0x7f && want != i) continue;
        if (want == 0x7f && stream_insts[i].per_cu == 0) continue;
        if (stream_fits(stream_insts[i], p, combo)) {
            pick = i;
            break;
        }
    }
    if (pick < 0) return KSMM_ERR_BAD_ALGO;
    const StreamInst &t = stream_insts[pick];
    const int64_t groups = (int64_t)p.a * p.d;
    // bs_last shares are column ranges (multiples of the 16-byte vector), bs_first shares are rows
    if (wgs <= 0) {
        const int per_cu = t.per_cu > 0 ? t.per_cu : 1;
        wgs = (256 * per_cu + groups - 1) / groups;
    }
    if (wgs < 1) wgs = 1;
    const int64_t n_tiles = (p.batch + t.tn - 1) / t.tn;
    if (wgs > n_tiles) wgs = n_tiles;
    const int64_t grid = groups * wgs;
    if (grid > 0x7fffffffLL) return KSMM_ERR_TOO_LARGE;
    if (tile) {
        tile->algo = KSMM_ALGO_TILE;
        tile->variant = (2 << 24) | pick;
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
    int batch_i = (int)p.batch, wgs_i = (int)wgs;
    Epi ep = epi_of(p);
    void *args[] = {(void *)&p.x, (void *)&p.w, (void *)&p.y, &batch_i, (void *)&p.a, (void *)&p.d,
                    &ep, &wgs_i};
    hipError_t e = hipLaunchKernel(t.fn, dim3((unsigned)grid), dim3(t.threads), args, t.lds, p.stream);
    return e == hipSuccess ? KSMM_OK : KSMM_ERR_LAUNCH;
}

}  // namespace ksmm
