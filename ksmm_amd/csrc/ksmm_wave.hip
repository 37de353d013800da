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
#include <type_traits>

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
    template <bool NT> __device__ static __forceinline__ void load(const half_t *p, uint32_t (&o)[RAW])
    {
        if constexpr (VEC == 8) {
            uint4_t v = NT ? __builtin_nontemporal_load((const uint4_t *)p) : *(const uint4_t *)p;
            o[0] = v[0]; o[1] = v[1]; o[2] = v[2]; o[3] = v[3];
        } else {
            uint2_t v = NT ? __builtin_nontemporal_load((const uint2_t *)p) : *(const uint2_t *)p;
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
    template <bool NT> __device__ static __forceinline__ void load(const fp8_t *p, uint32_t (&o)[RAW])
    {
        if constexpr (VEC == 16) {
            uint4_t v = NT ? __builtin_nontemporal_load((const uint4_t *)p) : *(const uint4_t *)p;
            o[0] = v[0]; o[1] = v[1]; o[2] = v[2]; o[3] = v[3];
        } else {
            uint2_t v = NT ? __builtin_nontemporal_load((const uint2_t *)p) : *(const uint2_t *)p;
            o[0] = v[0]; o[1] = v[1];
        }
    }
    __device__ static __forceinline__ void unpack(const uint32_t (&in)[RAW], uint32_t (&o)[VEC / 2])
    {
#pragma unroll
        for (int i = 0; i < RAW; ++i) {
            o[2 * i] = __builtin_bit_cast(uint32_t, fp8x2_to_half2(in[i]));
            o[2 * i + 1] = __builtin_bit_cast(uint32_t, fp8x2_hi_to_half2(in[i]));
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
// EPI: the instance that also adds a bias and/or applies the activation (kept apart so that
// the plain instance's registers and loop body stay as they are).
template <int MT, int KS, int OCC, bool ROLL, bool EPI>
__global__ __launch_bounds__(256, OCC) void ks_wave_bl_f32(const float *__restrict__ x,
                                                     const float *__restrict__ w,
                                                     float *__restrict__ y, int batch, int a, int b,
                                                     int c, int d, Epi ep, int n_slabs,
                                                     int iters, int rr)
{
    const float scale = ep.scale;
    constexpr int VEC = 4, TN = 16 * VEC;
    const int lane = threadIdx.x & 63;
    const int q = lane >> 4, r = lane & 15;
    const int wpw = (int)(blockDim.x >> 6), wv = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    // A wave multiplies 16*MT output rows of a block: the whole block, or (b a multiple of that)
    // row group h of it, the groups of a block then reading the same input rows.
    const int m_split = b / (16 * MT);
    int gh, slab;
    if (m_split > 1 && wpw % m_split == 0) {
        // two or four row groups: the groups of a (block, share) are neighbouring waves of one
        // workgroup (one CU reads the rows once)
        const int unit = (int)blockIdx.x * (wpw / m_split) + wv / m_split;
        if (unit >= a * d * n_slabs) return;
        const int gb = unit / n_slabs;
        slab = unit - gb * n_slabs;
        gh = gb * m_split + wv % m_split;
    } else if (m_split % wpw) {
        const int wave = __builtin_amdgcn_readfirstlane(blockIdx.x * wpw + wv);
        gh = wave / n_slabs;
        slab = wave - gh * n_slabs;
    } else {
        // The row groups that read the same input rows at the same time (one block, one share of
        // the tiles) sit in workgroups whose indices are equal mod 8: one XCD, whose L2 then
        // fetches those rows once ((1,768,192,2) fp32 fetched 4.9x its input with the groups
        // spread over all XCDs).
        const int per_unit = m_split / wpw;  // workgroups per (block, share)
        const int slot = (int)(blockIdx.x >> 3), unit = (slot / per_unit) * 8 + (int)(blockIdx.x & 7);
        if (unit >= a * d * n_slabs) return;
        const int gb = unit / n_slabs;
        slab = unit - gb * n_slabs;
        gh = gb * m_split + (slot % per_unit) * wpw + wv;
    }
    const int g = gh / m_split;  // block index a_i * d + d_i
    if (g >= a * d) return;
    const int m_off = (gh - g * m_split) * (16 * MT);
    const int a_i = g / d, d_i = g - a_i * d;

    // weights -> A operands, once per wave
    float areg[MT][KS];
    {
        const float *wg = w + (size_t)g * c * b;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks)
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) areg[mt][ks] = wg[(4 * ks + q) * b + m_off + 16 * mt + r];
    }
    // Addressing: uniform (scalar) row base + one 32-bit per-lane byte offset, so that the
    // loads and stores need no per-row vector address registers.  The host checks that the
    // offsets fit in 32 bits.
    const size_t row_stride = (size_t)d * batch;  // elements between consecutive c_i (or b_i)
    const char *xg = (const char *)(x + ((size_t)a_i * c * d + d_i) * batch);
    char *yg = (char *)(y + (((size_t)a_i * b + m_off) * d + d_i) * batch);
    const uint32_t x_lane = (uint32_t)(q * row_stride) * 4u;      // + column offset
    const uint32_t y_lane = (uint32_t)(4 * q * row_stride) * 4u;  // + column offset
    // Tiles of one wave (all uniform): `regular` tiles at n_first, n_first + stride, ... and, in
    // the balanced mode, possibly one more at n_extra.
    //  rr == 0: `iters` consecutive tiles;  rr == 1: every n_slabs-th tile (the waves of a block
    //  then work on neighbouring tiles at any one time);
    //  rr == 2 (balanced): as rr == 1 for the full rounds; the tiles of the last, partial round go
    //  one each to wave 0 of every workgroup of the block, then to wave 1 of every workgroup, ...
    //  so that no workgroup (CU) gets more than its share rounded up.
    const int n_tiles_row = (batch + TN - 1) / TN;
    int stride, n_first, regular, n_extra = -1;
    if (rr == 2) {
        const int n_wg = n_slabs / wpw;
        const int full = n_tiles_row / n_slabs, rest = n_tiles_row - full * n_slabs;
        const int e = (slab % wpw) * n_wg + slab / wpw;
        stride = n_slabs * TN;
        n_first = slab * TN;
        regular = full;
        if (e < rest) n_extra = (full * n_slabs + e) * TN;
    } else if (rr == 1) {
        stride = n_slabs * TN;
        n_first = slab * TN;
        regular = n_first < batch ? (batch - n_first + stride - 1) / stride : 0;
    } else {
        stride = TN;
        n_first = slab * iters * TN;
        regular = n_first < batch ? min(iters, (batch - n_first + TN - 1) / TN) : 0;
    }
    const int count = regular + (n_extra >= 0 ? 1 : 0);
    const int last_vec = batch - VEC;
    if (count <= 0) return;
    auto tile_start = [&](int k) { return k < regular ? n_first + k * stride : n_extra; };  // k < count
    const int n_begin = tile_start(0);

    // Rolling register pipeline: xc[ks] holds input rows 4*ks + q of the current tile; as soon
    // as the MFMAs of step ks are issued the same registers are refilled with the next tile's
    // rows, so every load has a whole tile of matrix work to hide behind.  Columns past the
    // end are clamped to the last valid vector (batch % VEC == 0) and never stored.
    float4_t xc[KS];
    auto col_off = [&](int n0) { return (uint32_t)min(n0 + VEC * r, last_vec) * 4u; };
    {
        const uint32_t off = x_lane + col_off(n_begin);
#pragma unroll
        for (int ks = 0; ks < KS; ++ks)
            xc[ks] = *(const float4_t *)(xg + (size_t)(4 * ks) * row_stride * 4 + off);
    }
    // bias of the output rows this lane holds (16*mt + 4*q + i), once per wave
    float bv[EPI ? MT : 1][4];
    if constexpr (EPI) {
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int i = 0; i < 4; ++i)
                bv[mt][i] = epi_bias<float>(ep, ((size_t)a_i * b + m_off + 16 * mt + 4 * q + i) * d + d_i);
    }
    // Everything issued so far (weights, first tile) is complete before the loop, so that the
    // waits inside the loop only ever count that loop's own loads and stores.
    __builtin_amdgcn_s_waitcnt(0);
    // FULL tiles store without a predicate, which keeps the loop body free of branches; only a
    // wave's last tile can be the ragged one (batch not a multiple of the tile): it runs with
    // the predicate.
    auto do_tile = [&](int n0, int n_next, auto full) {
        // (the tile after the last one is the last one again: a cache hit that is not used)
        const uint32_t next_off = x_lane + col_off(n_next);
        float4_t acc[MT][VEC];
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int v = 0; v < VEC; ++v) acc[mt][v] = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
#pragma unroll
            for (int v = 0; v < VEC; ++v)
#pragma unroll
                for (int mt = 0; mt < MT; ++mt)
                    acc[mt][v] = __builtin_amdgcn_mfma_f32_16x16x4f32(areg[mt][ks], xc[ks][v],
                                                                      acc[mt][v], 0, 0, 0);
            if constexpr (ROLL) {
                xc[ks] = *(const float4_t *)(xg + (size_t)(4 * ks) * row_stride * 4 + next_off);
                __builtin_amdgcn_sched_barrier(0);  // keep the refill between the MFMA groups
            }
        }
        const int col = n0 + VEC * r;
        if (decltype(full)::value || col < batch) {
            const uint32_t off = y_lane + (uint32_t)col * 4u;
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    float4_t o;
                    if constexpr (EPI)
                        o = float4_t{epi_finish(ep, acc[mt][0][i], bv[mt][i]), epi_finish(ep, acc[mt][1][i], bv[mt][i]),
                                     epi_finish(ep, acc[mt][2][i], bv[mt][i]), epi_finish(ep, acc[mt][3][i], bv[mt][i])};
                    else
                        o = float4_t{acc[mt][0][i] * scale, acc[mt][1][i] * scale, acc[mt][2][i] * scale,
                                     acc[mt][3][i] * scale};
                    *(float4_t *)(yg + (size_t)(16 * mt + i) * row_stride * 4 + off) = o;
                }
        }
    };
    for (int k = 0; k + 1 < count; ++k) do_tile(tile_start(k), tile_start(k + 1), std::true_type{});
    const int n_fin = tile_start(count - 1);
    if (n_fin + TN <= batch)
        do_tile(n_fin, n_fin, std::true_type{});
    else
        do_tile(n_fin, n_fin, std::false_type{});
}

// ------------------------------------------------------------------------------------------
// fp32 "ring" form: the same wave-per-block design, with the input rows of the next tile
// arriving by direct-to-LDS loads (global_load_lds_dwordx4) instead of into registers.
//
// What bounds the register form is the number of bytes a CU keeps in flight: a wave owns one
// tile of staging registers next to the weight block and the accumulators, and a CU runs four
// such waves.  Here a wave owns a private piece of LDS of KS kilobytes, one per k-step: the load
// of k-step ks of the next tile is issued into slot ks as soon as the current tile has read
// that slot, and the lane that requested 16 bytes is the lane that reads them back
// (ds_read_b128 of its own 16 bytes: conflict-free, and no barrier, the waves stay
// independent).  The registers that held the staged tile now hold a second set of accumulators:
// the stores of tile t are issued one by one between the k-steps of tile t + 1 instead of in a
// burst behind it.  Up to eight such waves share a CU (LDS: KS KB per wave).
//
// Vector-memory operations of a wave complete in the order they were issued, and the counter
// behind s_waitcnt vmcnt(N) counts loads and stores alike: "the load of slot ks has landed" is
// "at most N operations younger than it are outstanding", with N the number of operations
// issued after it, which the loop structure fixes: per k-step one load (while there is a next
// tile) followed by that step's share of the previous tile's stores.  A count that is too
// small only waits longer, so the first two tiles of a wave (whose loads were not yet followed
// by a full tile of stores) use the count without stores.
// ------------------------------------------------------------------------------------------
constexpr int vmcnt_enc(int n)
{
    const int m = n > 63 ? 63 : n;
    return (m & 15) | (7 << 4) | (15 << 8) | (((m >> 4) & 3) << 14);
}

template <int I, int N, typename F> __device__ __forceinline__ void static_for(F &&f)
{
    if constexpr (I < N) {
        f(std::integral_constant<int, I>{});
        static_for<I + 1, N>(f);
    }
}

template <bool NT> __device__ __forceinline__ void ring_dma16(const void *sbase, uint32_t voff, uint32_t lds_addr)
{
    if constexpr (NT)
        asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1 nt"
                     :
                     : "v"(voff), "s"(sbase), "s"(lds_addr)
                     : "memory", "m0");
    else
        asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                     :
                     : "v"(voff), "s"(sbase), "s"(lds_addr)
                     : "memory", "m0");
}

// the lane's own 16 bytes of a slot, complete when the function returns
template <int OFF> __device__ __forceinline__ float4_t ring_read16(uint32_t lds_addr)
{
    float4_t v;
    asm volatile("ds_read_b128 %0, %1 offset:%2\n\ts_waitcnt lgkmcnt(0)" : "=v"(v) : "v"(lds_addr), "n"(OFF) : "memory");
    return v;
}

template <int MT, int KS, bool DEFER, bool NT, bool EPI>
__global__ __launch_bounds__(512, 1) void ks_wave_ring_f32(const float *__restrict__ x,
                                                            const float *__restrict__ w,
                                                            float *__restrict__ y, int batch, int a, int b,
                                                            int c, int d, Epi ep, int n_slabs,
                                                            int iters, int rr)
{
    (void)iters;
    (void)rr;
    extern __shared__ __attribute__((aligned(16))) unsigned char ring_smem[];
    const float scale = ep.scale;
    constexpr int VEC = 4, TN = 16 * VEC;
    constexpr int NST = 4 * MT;  // store instructions per tile (4 rows x 256 bytes each)
    static_assert(KS * 1024 + 1023 < 65536, "slot offsets are 16-bit immediates");
    const int lane = threadIdx.x & 63;
    const int q = lane >> 4, r = lane & 15;
    const int wave_in_wg = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int wpw = (int)(blockDim.x >> 6);
    const int m_split = b / (16 * MT);
    int gh, slab;
    if (m_split > 1 && wpw % m_split == 0) {
        // row groups of a (block, share): neighbouring waves of one workgroup
        const int unit = (int)blockIdx.x * (wpw / m_split) + wave_in_wg / m_split;
        if (unit >= a * d * n_slabs) return;
        const int gb = unit / n_slabs;
        slab = unit - gb * n_slabs;
        gh = gb * m_split + wave_in_wg % m_split;
    } else {
        const int wave = __builtin_amdgcn_readfirstlane(blockIdx.x * wpw + wave_in_wg);
        gh = wave / n_slabs;
        slab = wave - gh * n_slabs;
    }
    const int g = gh / m_split;  // block index a_i * d + d_i
    if (g >= a * d) return;
    const int m_off = (gh - g * m_split) * (16 * MT);
    const int a_i = g / d, d_i = g - a_i * d;
    // tiles of this wave: every n_slabs-th tile of the block's row of tiles, so that the waves of
    // a workgroup read neighbouring 256-byte pieces of the same rows at any one time
    const int n_tiles_row = (batch + TN - 1) / TN;
    const int count = slab < n_tiles_row ? (n_tiles_row - slab + n_slabs - 1) / n_slabs : 0;
    if (count <= 0) return;

    float areg[MT][KS];
    {
        const float *wg = w + (size_t)g * c * b;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks)
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) areg[mt][ks] = wg[(4 * ks + q) * b + m_off + 16 * mt + r];
    }
    const size_t row_stride = (size_t)d * batch;  // elements between consecutive c_i (or b_i)
    const char *const xg = (const char *)(x + ((size_t)a_i * c * d + d_i) * batch);
    char *const yg = (char *)(y + (((size_t)a_i * b + m_off) * d + d_i) * batch);
    const uint32_t x_lane = (uint32_t)(q * row_stride) * 4u;      // + column offset
    const uint32_t y_lane = (uint32_t)(4 * q * row_stride) * 4u;  // + column offset
    const size_t x_step = row_stride * 16;                        // bytes per k-step (4 rows)
    const int last_vec = batch - VEC;
    // Columns past the end are clamped to the last valid vector (batch % VEC == 0): such a lane
    // computes the outputs of that vector and stores them there, a second copy of the same values.
    auto col_off = [&](int k) { return (uint32_t)min((slab + k * n_slabs) * TN + VEC * r, last_vec) * 4u; };
    float bv[EPI ? MT : 1][4];
    if constexpr (EPI) {
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int i = 0; i < 4; ++i)
                bv[mt][i] = epi_bias<float>(ep, ((size_t)a_i * b + m_off + 16 * mt + 4 * q + i) * d + d_i);
    }
    const uint32_t lds_wave = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char *)ring_smem +
                              (uint32_t)wave_in_wg * (KS * 1024);
    const uint32_t lds_lane = lds_wave + (uint32_t)lane * 16u;
    __builtin_amdgcn_s_waitcnt(0);  // weights and bias are here: the counter starts clean
    {
        const uint32_t off = x_lane + col_off(0);
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) ring_dma16<NT>(xg + ks * x_step, off, lds_wave + ks * 1024);
    }
    auto store_one = [&](const float4_t(&acc)[MT][VEC], int s, uint32_t off) {
        const int mt = s >> 2, i = s & 3;
        float4_t o;
        if constexpr (EPI)
            o = float4_t{epi_finish(ep, acc[mt][0][i], bv[mt][i]), epi_finish(ep, acc[mt][1][i], bv[mt][i]),
                         epi_finish(ep, acc[mt][2][i], bv[mt][i]), epi_finish(ep, acc[mt][3][i], bv[mt][i])};
        else
            o = float4_t{acc[mt][0][i] * scale, acc[mt][1][i] * scale, acc[mt][2][i] * scale, acc[mt][3][i] * scale};
        float4_t *const dst = (float4_t *)(yg + (size_t)(16 * mt + i) * row_stride * 4 + off);
        if constexpr (NT)
            __builtin_nontemporal_store(o, dst);
        else
            *dst = o;
    };
    // One tile: k-step ks waits for slot ks, reads it, hands the slot to the next tile's load,
    // multiplies, and issues the stores of the previous tile that fall to this step.
    //  has_prev: `prev` holds a finished tile whose stores go out between the k-steps
    //  steady:   the tile before the previous one existed as well, so a full tile of stores was
    //            issued behind each load this tile waits for: exact counts
    //  has_next: there is a next tile to request
    auto do_tile = [&](float4_t(&cur)[MT][VEC], const float4_t(&prev)[MT][VEC], uint32_t next_off, uint32_t prev_off,
                       auto has_prev, auto steady, auto has_next) {
        constexpr bool HAS_PREV = decltype(has_prev)::value, STEADY = decltype(steady)::value,
                       HAS_NEXT = decltype(has_next)::value;
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int v = 0; v < VEC; ++v) cur[mt][v] = float4_t{0.f, 0.f, 0.f, 0.f};
        const uint32_t noff = x_lane + next_off;
        const uint32_t poff = y_lane + prev_off;
        static_for<0, KS>([&](auto ks_c) {
            constexpr int ks = decltype(ks_c)::value;
            // operations issued after the load of (this tile, ks): the loads of the later k-steps
            // of the tile it was issued in, the loads of the earlier k-steps of this tile, and in
            // the steady state one tile's worth of stores
            constexpr int after = (KS - 1 - ks) + (HAS_NEXT ? ks : 0) + (STEADY ? NST : 0);
            __builtin_amdgcn_s_waitcnt(vmcnt_enc(after));
            const float4_t xv = ring_read16<ks * 1024>(lds_lane);
            if constexpr (HAS_NEXT) ring_dma16<NT>(xg + ks * x_step, noff, lds_wave + ks * 1024);
#pragma unroll
            for (int v = 0; v < VEC; ++v)
#pragma unroll
                for (int mt = 0; mt < MT; ++mt)
                    cur[mt][v] = __builtin_amdgcn_mfma_f32_16x16x4f32(areg[mt][ks], xv[v], cur[mt][v], 0, 0, 0);
            if constexpr (HAS_PREV) {
                // stores s with s * KS / NST == ks: spread evenly over the k-steps
#pragma unroll
                for (int s = 0; s < NST; ++s)
                    if (s * KS / NST == ks) store_one(prev, s, poff);
            }
            __builtin_amdgcn_sched_barrier(0);
        });
    };
    auto flush = [&](const float4_t(&acc)[MT][VEC], uint32_t off) {
#pragma unroll
        for (int s = 0; s < NST; ++s) store_one(acc, s, y_lane + off);
    };
    float4_t acc_a[MT][VEC];
    const std::true_type yes{};
    const std::false_type no{};
    if constexpr (!DEFER) {
        // one set of accumulators (blocks whose weights leave no room for two): a tile's stores
        // follow its last k-step in a burst, so from the second tile on every load waited for
        // has a tile of stores behind it
        if (count == 1) {
            do_tile(acc_a, acc_a, 0u, 0u, no, no, no);
            flush(acc_a, col_off(0));
            return;
        }
        do_tile(acc_a, acc_a, col_off(1), 0u, no, no, yes);
        flush(acc_a, col_off(0));
        int k = 1;
        for (; k + 1 < count; ++k) {
            do_tile(acc_a, acc_a, col_off(k + 1), 0u, no, yes, yes);
            flush(acc_a, col_off(k));
        }
        do_tile(acc_a, acc_a, 0u, 0u, no, yes, no);
        flush(acc_a, col_off(k));
    } else {
    float4_t acc_b[MT][VEC];
    // tile k of the wave uses acc_a for even k, acc_b for odd k
    if (count == 1) {
        do_tile(acc_a, acc_b, 0u, 0u, no, no, no);
        flush(acc_a, col_off(0));
        return;
    }
    do_tile(acc_a, acc_b, col_off(1), 0u, no, no, yes);
    if (count == 2) {
        do_tile(acc_b, acc_a, 0u, col_off(0), yes, no, no);
        flush(acc_b, col_off(1));
        return;
    }
    do_tile(acc_b, acc_a, col_off(2), col_off(0), yes, no, yes);
    int k = 2;
    for (; k + 2 < count; k += 2) {
        do_tile(acc_a, acc_b, col_off(k + 1), col_off(k - 1), yes, yes, yes);
        do_tile(acc_b, acc_a, col_off(k + 2), col_off(k), yes, yes, yes);
    }
    if (count - k == 2) {
        do_tile(acc_a, acc_b, col_off(k + 1), col_off(k - 1), yes, yes, yes);
        do_tile(acc_b, acc_a, 0u, col_off(k), yes, yes, no);
        flush(acc_b, col_off(k + 1));
    } else {
        do_tile(acc_a, acc_b, 0u, col_off(k - 1), yes, yes, no);
        flush(acc_a, col_off(k));
    }
    }
}

// ------------------------------------------------------------------------------------------
// 16-bit MFMA path: x is fp16 or e4m3fn (decoded to fp16, exact), w is fp16 or e4m3fn,
// y is fp16.  MT = b / 16, KS = c / (4 * KL).  Each wave iteration covers 16 * VEC columns.
// ------------------------------------------------------------------------------------------
// NT: non-temporal loads of the input rows and stores of the output rows (streams that are not read
// again by this kernel: they need not stay in the caches)
template <typename TX, typename TW, int MT, int KS, int KL, int VEC, int OCC, bool ROLL, bool EPI, bool NT>
__global__ __launch_bounds__(256, OCC) void ks_wave_bl_h(const TX *__restrict__ x,
                                                   const TW *__restrict__ w,
                                                   half_t *__restrict__ y, int batch, int a, int b,
                                                   int c, int d, Epi ep, int n_slabs, int iters, int rr)
{
    const float scale = ep.scale;
    constexpr int TN = 16 * VEC, KSTEP = 4 * KL;
    typedef typename hvec<KL>::type frag_t;
    const int lane = threadIdx.x & 63;
    const int q = lane >> 4, r = lane & 15;
    const int wave = __builtin_amdgcn_readfirstlane(blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6));
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
    typedef row_io<TX, VEC> io;
    const size_t row_stride = (size_t)d * batch;
    const char *xg = (const char *)(x + ((size_t)a_i * c * d + d_i) * batch);
    char *yg = (char *)(y + ((size_t)a_i * b * d + d_i) * batch);
    const uint32_t x_lane = (uint32_t)(KL * q * row_stride) * (uint32_t)sizeof(TX);
    const uint32_t y_lane = (uint32_t)(4 * q * row_stride) * 2u;
    // this wave's tiles: see the fp32 kernel
    const int n_tiles_row = (batch + TN - 1) / TN;
    int stride, n_first, regular, n_extra = -1;
    if (rr == 2) {
        const int wpw = (int)(blockDim.x >> 6), n_wg = n_slabs / wpw;
        const int full = n_tiles_row / n_slabs, rest = n_tiles_row - full * n_slabs;
        const int e = (slab % wpw) * n_wg + slab / wpw;
        stride = n_slabs * TN;
        n_first = slab * TN;
        regular = full;
        if (e < rest) n_extra = (full * n_slabs + e) * TN;
    } else if (rr == 1) {
        stride = n_slabs * TN;
        n_first = slab * TN;
        regular = n_first < batch ? (batch - n_first + stride - 1) / stride : 0;
    } else {
        stride = TN;
        n_first = slab * iters * TN;
        regular = n_first < batch ? min(iters, (batch - n_first + TN - 1) / TN) : 0;
    }
    const int count = regular + (n_extra >= 0 ? 1 : 0);
    const int last_vec = batch - VEC;
    if (count <= 0) return;
    auto tile_start = [&](int k) { return k < regular ? n_first + k * stride : n_extra; };
    const int n_begin = tile_start(0);

    // Rolling register pipeline as in the fp32 kernel: raw[ks][jj] holds VEC packed columns of
    // input row KSTEP*ks + KL*q + jj; it is refilled for the next tile right after step ks.
    uint32_t raw[KS][KL][io::RAW];
    auto col_off = [&](int n0) { return (uint32_t)min(n0 + VEC * r, last_vec) * (uint32_t)sizeof(TX); };
    {
        const uint32_t off = x_lane + col_off(n_begin);
#pragma unroll
        for (int ks = 0; ks < KS; ++ks)
#pragma unroll
            for (int jj = 0; jj < KL; ++jj)
                io::template load<NT>((const TX *)(xg + (size_t)(KSTEP * ks + jj) * row_stride * sizeof(TX) + off),
                                      raw[ks][jj]);
    }
    float bv[EPI ? MT : 1][4];  // bias of the output rows this lane holds
    if constexpr (EPI) {
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int i = 0; i < 4; ++i)
                bv[mt][i] = epi_bias<half_t>(ep, ((size_t)a_i * b + 16 * mt + 4 * q + i) * d + d_i);
    }
    __builtin_amdgcn_s_waitcnt(0);
    auto do_tile = [&](int n0, int n_next, auto full) {
        const uint32_t next_off = x_lane + col_off(n_next);
        float4_t acc[MT][VEC];
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int v = 0; v < VEC; ++v) acc[mt][v] = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            uint32_t xh[KL][VEC / 2];  // fp16 pairs: columns (2i, 2i+1) of row jj
#pragma unroll
            for (int jj = 0; jj < KL; ++jj) io::unpack(raw[ks][jj], xh[jj]);
            if constexpr (ROLL) {
#pragma unroll
                for (int jj = 0; jj < KL; ++jj)
                    io::template load<NT>((const TX *)(xg + (size_t)(KSTEP * ks + jj) * row_stride * sizeof(TX) + next_off),
                                          raw[ks][jj]);
            }
#pragma unroll
            for (int v = 0; v < VEC; ++v) {
                // KL consecutive k of batch column VEC*r + v: in-register transpose
                uint32_t bw[KL / 2];
#pragma unroll
                for (int pp = 0; pp < KL / 2; ++pp)
                    bw[pp] = pick_pair(xh[2 * pp][v / 2], xh[2 * pp + 1][v / 2], v & 1);
                frag_t bf;
                if constexpr (KL == 8)
                    bf = __builtin_bit_cast(frag_t, uint4_t{bw[0], bw[1], bw[2], bw[3]});
                else
                    bf = __builtin_bit_cast(frag_t, uint2_t{bw[0], bw[1]});
#pragma unroll
                for (int mt = 0; mt < MT; ++mt)
                    acc[mt][v] = mfma16<KL>::run(areg[mt][ks], bf, acc[mt][v]);
            }
            if constexpr (ROLL) __builtin_amdgcn_sched_barrier(0);
        }
        const int col = n0 + VEC * r;
        if (decltype(full)::value || col < batch) {
            const uint32_t off = y_lane + (uint32_t)col * 2u;
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    half_t *dst = (half_t *)(yg + (size_t)(16 * mt + i) * row_stride * 2 + off);
                    constexpr int W = 8 < VEC ? 8 : VEC;  // halves per store (<= 16 bytes)
#pragma unroll
                    for (int v0 = 0; v0 < VEC; v0 += W) {
                        typename hvec<W>::type o;
#pragma unroll
                        for (int v = 0; v < W; ++v) {
                            if constexpr (EPI)
                                o[v] = (half_t)epi_finish(ep, acc[mt][v0 + v][i], bv[mt][i]);
                            else
                                o[v] = (half_t)(acc[mt][v0 + v][i] * scale);
                        }
                        if constexpr (NT)
                            __builtin_nontemporal_store(o, (typename hvec<W>::type *)(dst + v0));
                        else
                            *(typename hvec<W>::type *)(dst + v0) = o;
                    }
                }
        }
    };
    for (int k = 0; k + 1 < count; ++k) do_tile(tile_start(k), tile_start(k + 1), std::true_type{});
    const int n_fin = tile_start(count - 1);
    if (n_fin + TN <= batch)
        do_tile(n_fin, n_fin, std::true_type{});
    else
        do_tile(n_fin, n_fin, std::false_type{});
}

// ---- instance table ---------------------------------------------------------------------
struct WaveInst {
    int b, c, vec, kl, occ;
    // [0]: several tiles per wave, rolling register pipeline; [1]: one tile per wave (nothing is
    // reloaded); [2], [3]: the same with bias / activation
    const void *fn[4];
    int ring = 0;  // > 0: the ring form, with at most this many waves per workgroup (LDS: c / 4 KB each)
    int nt = 0;    // non-temporal loads of the input and stores of the output
    int pref = 0;  // the automatic choice looks at these first (measured faster than the older forms)
};

typedef void (*f32_fn)(const float *, const float *, float *, int, int, int, int, int, Epi, int, int, int);
template <typename TX, typename TW>
using h_fn = void (*)(const TX *, const TW *, half_t *, int, int, int, int, int, Epi, int, int, int);

// OCC_ = minimum waves per SIMD the register allocation must allow
#define F32_FN(B_, C_, OCC_, ROLL_, EPI_) (const void *)(f32_fn)ks_wave_bl_f32<B_ / 16, C_ / 4, OCC_, ROLL_, EPI_>
#define F32_INST(B_, C_, OCC_) \
    {B_, C_, 4, 1, OCC_, {F32_FN(B_, C_, OCC_, true, false), F32_FN(B_, C_, OCC_, false, false), \
                          F32_FN(B_, C_, OCC_, true, true), F32_FN(B_, C_, OCC_, false, true)}}
// DEFER_: a second set of accumulators, the stores of a tile spread over the next one
// NT_: non-temporal loads and stores (the `nt` field tells such instances apart)
#define F32_RING_FN(B_, C_, DEFER_, NT_, EPI_) (const void *)(f32_fn)ks_wave_ring_f32<B_ / 16, C_ / 4, DEFER_, NT_, EPI_>
#define F32_RING(B_, C_, DEFER_, NT_, WAVES_) \
    {B_, C_, 4, 1, DEFER_ ? 1 : 2, {F32_RING_FN(B_, C_, DEFER_, NT_, false), F32_RING_FN(B_, C_, DEFER_, NT_, false), \
                                    F32_RING_FN(B_, C_, DEFER_, NT_, true), F32_RING_FN(B_, C_, DEFER_, NT_, true)}, WAVES_, NT_, \
     (B_) == 48 && (C_) == 48 && NT_ && DEFER_}
const WaveInst f32_insts[] = {
    F32_INST(48, 48, 2), F32_INST(48, 48, 3), F32_INST(64, 64, 2), F32_INST(64, 64, 1),
    F32_INST(16, 16, 4), F32_INST(32, 32, 3), F32_INST(48, 192, 1),
    // also takes the two row groups of a 64 x 64 block (forced or from the table): half the
    // weight registers, three waves per SIMD; 6 % faster than the whole block per wave on
    // (6,64,64,1) at batch 25088 (groups of 16 rows were 15-40 % slower there and on 48 x 48)
    F32_INST(32, 64, 3),
    // ring form (input through a per-wave LDS ring, stores spread over the next tile)
    F32_RING(48, 48, true, false, 8), F32_RING(64, 64, false, false, 8), F32_RING(32, 64, true, false, 8),
    F32_RING(16, 16, true, false, 8), F32_RING(32, 32, true, false, 8), F32_RING(48, 48, false, false, 8),
    // the same with non-temporal loads and stores
    F32_RING(48, 48, true, true, 8), F32_RING(64, 64, false, true, 8), F32_RING(32, 64, true, true, 8),
    F32_RING(16, 16, true, true, 8), F32_RING(32, 32, true, true, 8),
};

#define H_FN(TX_, TW_, B_, C_, KL_, VEC_, OCC_, ROLL_, EPI_, NT_) \
    (const void *)(h_fn<TX_, TW_>)ks_wave_bl_h<TX_, TW_, B_ / 16, C_ / (4 * KL_), KL_, VEC_, OCC_, ROLL_, EPI_, NT_>
#define H_INST_N(TX_, TW_, B_, C_, KL_, VEC_, OCC_, NT_)                                                   \
    {B_, C_, VEC_, KL_, OCC_,                                                                              \
     {H_FN(TX_, TW_, B_, C_, KL_, VEC_, OCC_, true, false, NT_), H_FN(TX_, TW_, B_, C_, KL_, VEC_, OCC_, false, false, NT_), \
      H_FN(TX_, TW_, B_, C_, KL_, VEC_, OCC_, true, true, NT_), H_FN(TX_, TW_, B_, C_, KL_, VEC_, OCC_, false, true, NT_)}, 0, NT_, \
     NT_ && (B_) == 16 && sizeof(TX_) == 2}
#define H_INST(TX_, TW_, B_, C_, KL_, VEC_, OCC_) H_INST_N(TX_, TW_, B_, C_, KL_, VEC_, OCC_, false)
#define H_SET(TX_, TW_)                                                                      \
    H_INST(TX_, TW_, 64, 64, 8, 4, 2), H_INST(TX_, TW_, 64, 64, 8, 8, 2),                    \
        H_INST(TX_, TW_, 64, 64, 8, 8, 1), H_INST(TX_, TW_, 48, 48, 4, 4, 3),                \
        H_INST(TX_, TW_, 48, 48, 4, 8, 2), H_INST(TX_, TW_, 16, 16, 4, 8, 4),                \
        H_INST(TX_, TW_, 16, 16, 4, 4, 4), H_INST(TX_, TW_, 32, 32, 8, 8, 3),                \
        H_INST(TX_, TW_, 96, 96, 8, 4, 1), H_INST(TX_, TW_, 48, 192, 8, 4, 1),              \
        H_INST(TX_, TW_, 192, 48, 4, 4, 1),                                                 \
        H_INST_N(TX_, TW_, 16, 16, 4, 8, 4, true), H_INST_N(TX_, TW_, 16, 16, 4, 4, 4, true), \
        H_INST_N(TX_, TW_, 48, 48, 4, 8, 2, true), H_INST_N(TX_, TW_, 64, 64, 8, 8, 2, true), \
        H_INST_N(TX_, TW_, 32, 32, 8, 8, 3, true)
const WaveInst h_insts[] = {H_SET(half_t, half_t)};
const WaveInst hq_insts[] = {H_SET(half_t, fp8_t)};
const WaveInst q_insts[] = {
    H_INST(fp8_t, fp8_t, 64, 64, 8, 8, 2),  H_INST(fp8_t, fp8_t, 64, 64, 8, 8, 1),
    H_INST(fp8_t, fp8_t, 48, 48, 4, 8, 2),  H_INST(fp8_t, fp8_t, 16, 16, 4, 8, 4),
    H_INST(fp8_t, fp8_t, 16, 16, 4, 16, 3), H_INST(fp8_t, fp8_t, 32, 32, 8, 16, 2),
    H_INST(fp8_t, fp8_t, 32, 32, 8, 8, 3),  H_INST(fp8_t, fp8_t, 48, 192, 8, 8, 1),
    H_INST_N(fp8_t, fp8_t, 16, 16, 4, 8, 4, true), H_INST_N(fp8_t, fp8_t, 16, 16, 4, 16, 3, true),
    H_INST_N(fp8_t, fp8_t, 48, 48, 4, 8, 2, true), H_INST_N(fp8_t, fp8_t, 64, 64, 8, 8, 2, true),
    H_INST_N(fp8_t, fp8_t, 32, 32, 8, 16, 2, true),
};

const WaveInst *wave_table(int combo, int *n)
{
    switch (combo) {
    case 0: *n = sizeof(f32_insts) / sizeof(WaveInst); return f32_insts;
    case 1: *n = sizeof(h_insts) / sizeof(WaveInst); return h_insts;
    case 2: *n = sizeof(q_insts) / sizeof(WaveInst); return q_insts;
    case 3: *n = sizeof(hq_insts) / sizeof(WaveInst); return hq_insts;
    default: *n = 0; return nullptr;
    }
}

}  // namespace

int wave_inst_count(int combo)
{
    int n;
    wave_table(combo, &n);
    return n;
}

uint32_t wave_inst_id(int combo, int i)
{
    int n;
    const WaveInst *t = wave_table(combo, &n);
    if (i < 0 || i >= n) return 0;
    const int v[8] = {combo, t[i].b, t[i].c, t[i].vec, t[i].kl, t[i].occ, t[i].ring, t[i].nt};
    return inst_hash('W', v, t[i].nt ? 8 : t[i].ring ? 7 : 6);  // (ids of the older instances predate the fields)
}

int wave_run(const Problem &p, int variant, bool launch, ksmm_tile *tile)
{
    // batch-size-first: the register-stationary row kernel (variants >= 1000), d > 1 only
    if (!p.bs_last) return rows_bf_run(p, variant >= 1000 ? variant - 1000 : -1, launch, tile);
    const int combo = combo_of(p.x_dtype, p.w_dtype, p.y_dtype);
    int n_insts;
    const WaveInst *insts = wave_table(combo, &n_insts);
    if (!insts) return KSMM_ERR_BAD_DTYPE;
    // vector loads along the batch axis need every row start aligned to the vector
    // variant: bits 0-7 instance index (0xff: first that fits), bits 8-15 tiles per wave (0:
    // heuristic), bits 16-17 how tiles are dealt: 0 consecutive, 1 every n_slabs-th, 2 balanced
    // (bits 8-15 are then workgroups per block, 0: one round of workgroups over the chip);
    // -1: everything automatic
    const int want = variant < 0 ? 0xff : (variant & 0xff);
    int iters = variant < 0 ? 0 : ((variant >> 8) & 0xff);
    int rr = variant < 0 ? -1 : ((variant >> 16) & 3);
    if (rr == 3) return KSMM_ERR_BAD_ALGO;
    int pick = -1;
    // automatic choice: the preferred instances first, then the others in table order (ring and
    // non-temporal forms that are not marked preferred are taken only when forced or named by the
    // measured table)
    for (int pass = 0; pass < 2 && pick < 0; ++pass)
        for (int i = 0; i < n_insts; ++i) {
            // fp32: a forced instance also takes blocks whose b is a multiple of its rows (row groups)
            const bool rows_ok = insts[i].b == p.b || (combo == 0 && want == i && p.b % insts[i].b == 0);
            if (!rows_ok || insts[i].c != p.c) continue;
            if (p.batch % insts[i].vec) continue;
            if (want != 0xff && want != i) continue;
            if (want == 0xff && (pass == 0 ? !insts[i].pref : (insts[i].ring || insts[i].nt))) continue;
            pick = i;
            break;
        }
    if (pick < 0) return KSMM_ERR_BAD_ALGO;
    const WaveInst &in = insts[pick];
    // The per-lane byte offsets must fit in 32 bits.  The largest ones formed are row 3*KL of a
    // k-step plus one row of columns on the input side and row 12 of a 16-row output tile plus
    // one row of columns on the output side (rows are d*batch elements apart).
    {
        const int64_t db = (int64_t)p.d * p.batch;
        const int64_t x_max = (3 * in.kl * db + p.batch) * (int64_t)dtype_size(p.x_dtype);
        const int64_t y_max = (12 * db + p.batch) * (int64_t)dtype_size(p.y_dtype);
        if ((x_max > y_max ? x_max : y_max) >= 0xffffffffLL) return KSMM_ERR_BAD_ALGO;
    }
    const int tn = 16 * in.vec;
    const int64_t n_tiles = (p.batch + tn - 1) / tn;
    if (in.ring) {
        // Ring form: every wave takes every n_slabs-th tile of its block's row of tiles.  Bits
        // 18-21: waves per workgroup (0: four, one per SIMD; at most in.ring and what the LDS
        // holds, c / 4 KB per wave); tiles per wave (bits 8-15, 0: automatic): the smallest number
        // with which all workgroups are resident at once, one per CU.
        const int64_t groups = (int64_t)p.a * p.d * (p.b / in.b);
        const int ks = p.c / 4;
        int wmax = in.ring;
        if (wmax * ks > 160) wmax = 160 / ks;
        int wpw = variant < 0 ? 0 : ((variant >> 18) & 15);
        if (wpw > wmax || wmax < 1) return KSMM_ERR_BAD_ALGO;
        // (measured on (1,48,48,16) at batch 25088: one wave per SIMD, 7 tiles per wave, 224
        // workgroups 30.4 us; 7 or 8 waves per workgroup with 4 tiles each 31.1-31.3; workgroups
        // beyond one round 32-34)
        if (wpw == 0) wpw = wmax < 4 ? wmax : 4;
        if (iters == 0) {
            iters = 1;
            while (iters < 255 && groups * ((n_tiles + iters - 1) / iters) > 256 * (int64_t)wpw) ++iters;
        }
        const int64_t n_slabs = (n_tiles + iters - 1) / iters;
        const int64_t waves = groups * n_slabs;
        const int64_t blocks = (waves + wpw - 1) / wpw;
        if (blocks > 0x7fffffffLL) return KSMM_ERR_TOO_LARGE;
        const int lds = wpw * ks * 1024;
        if (tile) {
            tile->algo = KSMM_ALGO_WAVE;
            tile->variant = pick | (iters << 8) | (wpw << 18);
            tile->tile_m = in.b;
            tile->tile_n = tn;
            tile->tile_k = p.c;
            tile->tile_d = 1;
            tile->threads = 64 * wpw;
            tile->lds_bytes = lds;
            tile->grid = blocks;
        }
        if (!launch) return KSMM_OK;
        Epi ep = epi_of(p);
        const void *fn = in.fn[p.bias || p.act ? 2 : 0];
        if (ensure_dynamic_lds(fn, wmax * ks * 1024) != KSMM_OK) return KSMM_ERR_LAUNCH;
        int batch_i = (int)p.batch, n_slabs_i = (int)n_slabs, rr_i = 1;
        void *args[] = {(void *)&p.x, (void *)&p.w, (void *)&p.y, &batch_i, (void *)&p.a, (void *)&p.b,
                        (void *)&p.c, (void *)&p.d, &ep, &n_slabs_i, &iters, &rr_i};
        hipError_t e = hipLaunchKernel(fn, dim3((unsigned)blocks), dim3(64 * wpw), args, lds, p.stream);
        return e == hipSuccess ? KSMM_OK : KSMM_ERR_LAUNCH;
    }
    // Tiles per wave.  Small blocks (16x16, 32x32) have little matrix work per byte: one tile
    // per wave and many waves in flight measured best.  Larger blocks keep a SIMD's matrix pipe
    // busy for microseconds per tile; there a single round of workgroups (at most one per CU,
    // 4 waves each) with the rolling pipeline over several tiles is best, and a few workgroups
    // beyond 256 double the run time (two share a CU while the others have finished): take the
    // smallest count that fits one round.
    const int64_t groups = (int64_t)p.a * p.d * (p.b / in.b);  // blocks x row groups
    const int wpb = 4;
    // (Balanced dealing, rr == 2, keeps every CU within one tile of its share: (1,48,48,16) at
    // batch 25088 has 24.5 tiles per CU where 7 consecutive tiles per wave leave 32 CUs idle and
    // give the others 28.  Measured, it is 1-3 % slower than the consecutive split on that shape
    // and on (6,64,64,1): these kernels are not bound by the busiest CU.  It stays selectable.)
    if (rr < 0) rr = 0;
    int64_t n_slabs, blocks;
    int iters_field = 0;  // what the variant's bits 8-15 must hold to reproduce this launch
    if (rr == 2) {
        int64_t wgs_pb = iters > 0 ? iters : (256 / groups > 1 ? 256 / groups : 1);
        if (wgs_pb > 255) wgs_pb = 255;
        if (wgs_pb > (n_tiles + wpb - 1) / wpb) wgs_pb = (n_tiles + wpb - 1) / wpb;
        n_slabs = wpb * wgs_pb;
        blocks = groups * wgs_pb;
        iters_field = (int)(wgs_pb < 255 ? wgs_pb : 255);
        iters = 2;  // (several tiles per wave: the kernel with the rolling pipeline)
    } else {
        if (iters == 0) {
            iters = 1;
            if (in.b * p.c > 1024)
                while (iters < 255 && (groups * ((n_tiles + iters - 1) / iters) + wpb - 1) / wpb > 256) ++iters;
        }
        n_slabs = (n_tiles + iters - 1) / iters;
        blocks = (groups * n_slabs + wpb - 1) / wpb;
        iters_field = iters;
    }
    // row groups in multiples of the workgroup: the groups of a (block, share) get workgroup
    // indices that are equal mod 8 (see the kernel); the grid is padded to whole sets of 8
    const int64_t m_split = p.b / in.b;
    if (combo == 0 && !in.ring && m_split > wpb && m_split % wpb == 0)
        blocks = 8 * (m_split / wpb) * (((int64_t)p.a * p.d * n_slabs + 7) / 8);
    if (blocks > 0x7fffffffLL) return KSMM_ERR_TOO_LARGE;
    if (tile) {
        tile->algo = KSMM_ALGO_WAVE;
        tile->variant = pick | (iters_field << 8) | (rr << 16);
        tile->tile_m = in.b;
        tile->tile_n = tn;
        tile->tile_k = p.c;
        tile->tile_d = 1;
        tile->threads = 64 * wpb;
        tile->lds_bytes = 0;
        tile->grid = blocks;
    }
    if (!launch) return KSMM_OK;
    Epi ep = epi_of(p);
    void *args[] = {(void *)&p.x, (void *)&p.w, (void *)&p.y, nullptr, (void *)&p.a, (void *)&p.b,
                    (void *)&p.c, (void *)&p.d, &ep, nullptr, nullptr, &rr};
    int batch_i = (int)p.batch, n_slabs_i = (int)n_slabs;
    args[3] = &batch_i;
    args[9] = &n_slabs_i;
    args[10] = &iters;
    const void *fn = in.fn[(iters == 1 ? 1 : 0) + (p.bias || p.act ? 2 : 0)];
    hipError_t e = hipLaunchKernel(fn, dim3((unsigned)blocks), dim3(64 * wpb), args, 0, p.stream);
    return e == hipSuccess ? KSMM_OK : KSMM_ERR_LAUNCH;
}

}  // namespace ksmm
