// Fused factor chain for radix-16 butterflies: consecutive factors with b = c = 16 and
// power-of-two d applied to the same N = a*16*d <= 1024 features (batch-size-last), with the
// intermediates kept in LDS.
//
// A workgroup (16 waves) takes chunks of 64 batch columns, dealt round-robin over the grid.
//  The whole feature vector of the chunk (N rows x 64 columns, fp16) lives in LDS.
// Because every block is square, a block reads and writes the same 16 rows, so each factor is
// applied in place: wave w owns blocks w, w+8, ... of every factor, reads the 16 input rows of
// a block for all columns of the chunk, multiplies with v_mfma_f32_16x16x16_f16 (the 16x16
// weight block is stationary in registers for the life of the wave), and writes the 16 output
// rows back; after the last factor the rows go to global memory as whole 128-byte lines.  Only the
// chain input (e4m3fn or fp16) and the final fp16 output touch HBM: 77 MB instead of 283 MB for
// the 3-factor 1024-feature chain at batch 25088.
//
// LDS row = 128 bytes in four 32-byte slots of four 8-byte pieces; slots and pieces of a row are
// XOR-permuted by bits of the row number (lds_piece) so that both the transpose loads (4 rows per
// 16-lane group) and the accumulator stores (16 rows per 16-lane group) of a block with any
// power-of-two stride d are free of bank conflicts.  Piece p of slot s holds the 4 columns
// 32*(s/2) + 8*p + 4*(s%2) .. +3 of the chunk: sub-tile s of the MFMA then takes columns that
// make 8 consecutive columns (16 bytes of a global row) two pieces 32 bytes apart.  e4m3fn input is expanded to fp16 while it is staged.  The weights pass through the
// same LDS once, at the start, to be picked up in MFMA operand order by transpose loads.
//
// MFMA roles: A = X^T (rows = batch columns, k from ds_read_b64_tr_b16), B = W^T (lanes =
// outputs), so a lane holds 4 batch columns of one output row: 8-byte LDS writes.
//
// Reference counterpart: the Python loop over factors of KSLinear.forward_bs_last
// (src/ksmm_py/layer/kronecker_sparse/interface.py:269-291), one kernel launch and one HBM
// round trip of the intermediate per factor.
#include "ksmm_mfma.h"


namespace ksmm {

struct Chain16Args {
    const void *w[4];
    int log2d[4];
    float scale[4];
    const void *bias;  // of the last factor's outputs (fp16), or none
    int act;
};

namespace {

constexpr int CH_TN = 64;    // columns per chunk
constexpr int CH_ROW = 128;  // bytes per LDS row
constexpr int CH_THREADS = 1024, CH_WAVES = CH_THREADS / 64;  // 4 waves per SIMD: 128 registers each

// Byte offset of piece `piece` of slot `slot` in row `row`.  key = XOR of the 4-bit fields of the
// row number; the slot is XORed with the fold of key to two bits and the piece with key's upper
// two bits.  For rows r0 + i*d (d a power of two):
//  * i = 0..3   -> 4 different slots  (the 4 rows one 16-lane group of a transpose load reads),
//  * i = 0..15  -> 16 different (slot, piece) positions (the 16 rows the 16 lanes of one
//                  accumulator column group write), i.e. all 32 banks once.
// The map is linear over GF(2): lds_piece(r0 ^ r1, s, p) = lds_piece(r0, 0, 0) ^ lds_piece(r1, s, p).
__device__ __forceinline__ int lds_piece(int row, int slot, int piece)
{
    const int key = (row ^ (row >> 4) ^ (row >> 8)) & 15;
    return row * CH_ROW + (((slot ^ key ^ (key >> 2)) & 3) << 5) + ((piece ^ (key >> 2)) << 3);
}

typedef short4_t __attribute__((address_space(3))) * lds_tr_ptr;

// Four e4m3fn bytes -> four fp16 (hardware conversion, unit scale).
__device__ __forceinline__ half4_t fp8x4_to_half4(uint32_t v)
{
    const half2_t lo = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(v, 1.0f, false);
    const half2_t hi = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(v, 1.0f, true);
    return half4_t{lo[0], lo[1], hi[0], hi[1]};
}

// FULL: 1024 features (every wave has MAXB blocks per factor) and a batch that is a multiple of
// the chunk: no tile is ragged, so the chunk loop has no branches and the compiler's memory
// counters stay exact (a chunk's stores drain while the next chunk is staged and multiplied).
template <typename TX, typename TW, int NF, bool FULL>
__global__ __launch_bounds__(CH_THREADS) void ks_chain16_kernel(const TX *__restrict__ x, half_t *__restrict__ y,
                                                         Chain16Args args, int batch, int n_feat)
{
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    const int tid = threadIdx.x, lane = tid & 63, q = lane >> 4, r = lane & 15;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    // chunk c = columns 64c .. 64c+63; this workgroup takes chunks c0, c0 + gridDim.x, ...
    // An e4m3fn row piece of a chunk is 64 bytes, half a 128-byte line whose other half belongs
    // to the neighbouring chunk.  On a full grid (a multiple of 16 workgroups) the two chunks of a
    // line go to workgroups blockIdx.x and blockIdx.x + 8: same XCD (blockIdx.x % 8), same round,
    // same row order, so the second request meets the first in that XCD's L2 and the line comes
    // from HBM once.  Dealt to unrelated workgroups every line was fetched twice.
    int c0 = blockIdx.x;
    if (gridDim.x % 16 == 0) c0 = 2 * (8 * (c0 / 16) + c0 % 8) + (c0 / 8) % 2;
    const int c_begin = c0 * CH_TN, c_step = gridDim.x * CH_TN, c_end = batch;
    if (c_begin >= c_end) return;
    const int c_last = c_begin + ((c_end - 1 - c_begin) / c_step) * c_step;  // this workgroup's last chunk
    const int n_blocks = n_feat / 16;  // blocks per factor
    constexpr int MAXB = 64 / CH_WAVES;  // blocks per wave and factor (n_feat <= 1024)

    // ---- input staging: each thread carries 16-byte pieces of the next chunk in registers ----
    constexpr int X_ROWB = CH_TN * (int)sizeof(TX);      // input bytes per row and chunk
    constexpr int X_PPR = X_ROWB / 16;                   // 16-byte pieces per row
    constexpr int X_PER_T = 1024 * X_PPR / CH_THREADS;   // pieces per thread for 1024 rows
    uint4_t xreg[X_PER_T];
    // e4m3fn: a 16-lane group stages 4 rows x 4 pieces; rows u with bits 1 and 2 exchanged make
    // those 4 rows differ in the slot and in the piece permutation, so their 8-byte LDS writes
    // fall into different banks
    auto piece_row = [](int u) {
        return sizeof(TX) == 1 ? (u & ~6) | ((u & 2) << 1) | ((u & 4) >> 1) : u;
    };
    // `real` == false (uniform): nothing to fetch, every lane reads the same 16 bytes instead, so
    // that the instruction count stays the same without the traffic
    auto gload = [&](int n0, bool real) {
#pragma unroll
        for (int i = 0; i < X_PER_T; ++i) {
            const int p = tid + i * CH_THREADS, row = piece_row(p / X_PPR), pc = p % X_PPR;
            const int col = min(n0 + pc * (16 / (int)sizeof(TX)), c_end - 16 / (int)sizeof(TX));
            // rows past the end repeat the last one (loaded, never staged): no branch here
            const TX *src = x + (size_t)min(row, n_feat - 1) * batch + col;
            xreg[i] = *(const uint4_t *)(real ? src : x + c_begin);
        }
    };
    auto lstore = [&]() {
#pragma unroll
        for (int i = 0; i < X_PER_T; ++i) {
            const int p = tid + i * CH_THREADS, row = piece_row(p / X_PPR), pc = p % X_PPR;
            if (FULL || row < n_feat) {
                if constexpr (sizeof(TX) == 1) {
                    // e4m3fn: columns 16*pc .. +15 = pieces p0, p0+1 of slots 2t, 2t+1
                    const int off = lds_piece(row, 2 * (pc >> 1), 2 * (pc & 1));
                    *(half4_t *)(smem + off) = fp8x4_to_half4(xreg[i][0]);
                    *(half4_t *)(smem + (off ^ 32)) = fp8x4_to_half4(xreg[i][1]);
                    *(half4_t *)(smem + (off ^ 8)) = fp8x4_to_half4(xreg[i][2]);
                    *(half4_t *)(smem + (off ^ 40)) = fp8x4_to_half4(xreg[i][3]);
                } else {
                    // fp16: columns 8*pc .. +7 = piece pc%4 of slots 2t, 2t+1
                    const int off = lds_piece(row, 2 * (pc >> 2), pc & 3);
                    *(uint2_t *)(smem + off) = uint2_t{xreg[i][0], xreg[i][1]};
                    *(uint2_t *)(smem + (off ^ 32)) = uint2_t{xreg[i][2], xreg[i][3]};
                }
            }
        }
    };

    // ---- weights: staged through LDS as fp16 in kernel format (block g = a_i*d + d_i: element
    // (k, m) at (g*16 + k)*16 + m), then one transpose load per block gives the B operand:
    // lane (r = m, q) holds W[m][k = 4q..4q+3].  They stay in registers for the life of the wave.
    {
        constexpr int WV = 16 / (int)sizeof(TW);              // weights per 16-byte vector
        constexpr int W_PER_T = 1024 * 16 / WV / CH_THREADS;  // vectors per thread and factor
        const int n_vec = n_feat * 16 / WV;
        uint4_t wv[NF][W_PER_T];
#pragma unroll
        for (int f = 0; f < NF; ++f)
#pragma unroll
            for (int i = 0; i < W_PER_T; ++i) {
                const int v = min(tid + i * CH_THREADS, n_vec - 1);
                wv[f][i] = *((const uint4_t *)args.w[f] + v);
            }
        // the weights' loads go first and are waited for alone: staging them overlaps with the
        // flight of the (HBM-bound) first chunk
        __builtin_amdgcn_sched_barrier(0);
        gload(c_begin, true);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int f = 0; f < NF; ++f)
#pragma unroll
            for (int i = 0; i < W_PER_T; ++i) {
                const int v = tid + i * CH_THREADS;
                if (FULL || v < n_vec) {
                    unsigned char *dst = smem + ((size_t)f * n_feat * 16 + (size_t)v * WV) * 2;
                    if constexpr (sizeof(TW) == 1) {
#pragma unroll
                        for (int j = 0; j < 4; ++j) *(half4_t *)(dst + 8 * j) = fp8x4_to_half4(wv[f][i][j]);
                    } else {
                        *(uint4_t *)dst = wv[f][i];
                    }
                }
            }
    }
    __syncthreads();
    half4_t wreg[NF][MAXB];
#pragma unroll
    for (int f = 0; f < NF; ++f)
#pragma unroll
        for (int bi = 0; bi < MAXB; ++bi) {
            const int g = min(wave + CH_WAVES * bi, n_blocks - 1);
            const short4_t t = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                (lds_tr_ptr)(smem + ((size_t)f * n_feat * 16 + g * 256 + (4 * q + (r >> 2)) * 16) * 2 + ((r & 3) << 3)));
            wreg[f][bi] = __builtin_bit_cast(half4_t, t);
        }
    // per-lane parts of the LDS offsets: rows (4q + r/4)*d piece r%4 (A operand), row r*d piece q (D)
    int v_in[NF], v_out[NF];
#pragma unroll
    for (int f = 0; f < NF; ++f) {
        v_in[f] = lds_piece((4 * q + (r >> 2)) << args.log2d[f], 0, r & 3);
        v_out[f] = lds_piece(r << args.log2d[f], 0, q);
    }
    __syncthreads();

    for (int n0 = c_begin; n0 < c_end; n0 += c_step) {
        lstore();
        __syncthreads();
        if (FULL)
            gload(min(n0 + c_step, c_last), n0 + c_step < c_end);  // after the last chunk: a dummy request
        else if (n0 + c_step < c_end)
            gload(n0 + c_step, true);
        // an opaque zero: keeps the compiler from hoisting the per-block address arithmetic of
        // all NF x 8 blocks, and the addresses of the output pieces, out of this loop (it would
        // spill them)
        int opaque = 0;
        asm volatile("" : "+s"(opaque));
#pragma unroll
        for (int f = 0; f < NF; ++f) {
            const int ld = args.log2d[f];
            const float scale = args.scale[f];
            // first row of block g (scalar) and the A operand of its four sub-tiles
            auto block_row0 = [&](int g) { return ((g >> ld) << (ld + 4)) | (g & ((1 << ld) - 1)); };
            auto read_block = [&](int g, half4_t(&xa)[4]) {
                const int base = lds_piece(block_row0(g), 0, 0) ^ v_in[f];
#pragma unroll
                for (int s = 0; s < 4; ++s)
                    xa[s] = __builtin_bit_cast(
                        half4_t, __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_tr_ptr)(smem + (base ^ (s << 5)))));
            };
            half4_t xa[2][4];
            if (FULL || wave + opaque < n_blocks) read_block(wave + opaque, xa[0]);
#pragma unroll
            for (int bi = 0; bi < MAXB; ++bi) {
                const int g = wave + CH_WAVES * bi + opaque;
                if (!FULL && g >= n_blocks) break;  // uniform
                // the next block's rows are not this block's: read them before this block writes
                if (bi + 1 < MAXB && (FULL || g + CH_WAVES < n_blocks)) read_block(g + CH_WAVES, xa[(bi + 1) & 1]);
                float4_t acc[4];
#pragma unroll
                for (int s = 0; s < 4; ++s)
                    acc[s] = __builtin_amdgcn_mfma_f32_16x16x16f16(xa[bi & 1][s], wreg[f][bi],
                                                                   float4_t{0.f, 0.f, 0.f, 0.f}, 0, 0, 0);
                // D^T: lane (r = output m, q) holds the 4 columns of piece q of slot s
                half4_t o[4];
                const int row0 = block_row0(g);
                if (f + 1 == NF && (args.bias != nullptr || args.act != KSMM_ACT_NONE)) {
                    // the chain's epilogue: the lane's output row is row0 + r * d
                    const Epi ep{scale, args.act, args.bias};
                    const float bv = epi_bias<half_t>(ep, (size_t)(row0 + (r << ld)));
#pragma unroll
                    for (int s = 0; s < 4; ++s)
                        o[s] = half4_t{(half_t)epi_finish(ep, acc[s][0], bv), (half_t)epi_finish(ep, acc[s][1], bv),
                                       (half_t)epi_finish(ep, acc[s][2], bv), (half_t)epi_finish(ep, acc[s][3], bv)};
                } else {
#pragma unroll
                    for (int s = 0; s < 4; ++s)
                        o[s] = half4_t{(half_t)(acc[s][0] * scale), (half_t)(acc[s][1] * scale),
                                       (half_t)(acc[s][2] * scale), (half_t)(acc[s][3] * scale)};
                }
                // all inputs of the block are in registers: write its 16 output rows in place (the
                // last factor too: its rows leave for global memory from LDS, see below)
                const int obase = lds_piece(row0, 0, 0) ^ v_out[f];
#pragma unroll
                for (int s = 0; s < 4; ++s) *(half4_t *)(smem + (obase ^ (s << 5))) = o[s];
            }
            __syncthreads();
        }
        // ---- the chunk's result: N rows x 128 bytes, eight neighbouring lanes per row, so every
        // store instruction writes whole lines (straight from the accumulators a lane holds
        // 16 bytes of 16 different rows per 16-lane group: 64 separate pieces per instruction,
        // which took 2.5x the time of this detour through LDS).  In parts of OB pieces, to stay
        // within the registers the input prefetch leaves (a spilled prefetch would be reloaded
        // behind these stores and wait for them).
        constexpr int O_PER_T = 1024 * 8 / CH_THREADS;  // 16-byte pieces per thread for 1024 rows
        constexpr int OB = 2;
#pragma unroll
        for (int h = 0; h < O_PER_T / OB; ++h) {
            uint4_t v[OB];
#pragma unroll
            for (int i = 0; i < OB; ++i) {
                const int pp = tid + opaque + (h * OB + i) * CH_THREADS, row = pp >> 3, pc = pp & 7;
                const int off = lds_piece(FULL ? row : min(row, n_feat - 1), 2 * (pc >> 2), pc & 3);
                const uint2_t lo = *(const uint2_t *)(smem + off), hi = *(const uint2_t *)(smem + (off ^ 32));
                v[i] = uint4_t{lo[0], lo[1], hi[0], hi[1]};
            }
#pragma unroll
            for (int i = 0; i < OB; ++i) {
                const int pp = tid + opaque + (h * OB + i) * CH_THREADS, row = pp >> 3, pc = pp & 7;
                if (FULL || (row < n_feat && n0 + 8 * pc < c_end))
                    *(uint4_t *)(y + (size_t)row * batch + n0 + 8 * pc) = v[i];
            }
        }
        __syncthreads();  // the rows are read: the next chunk may be staged over them
    }
}

template <typename TX, typename TW> const void *chain16_fn(int nf, bool full)
{
    switch (nf) {
    case 2: return full ? (const void *)ks_chain16_kernel<TX, TW, 2, true> : (const void *)ks_chain16_kernel<TX, TW, 2, false>;
    case 3: return full ? (const void *)ks_chain16_kernel<TX, TW, 3, true> : (const void *)ks_chain16_kernel<TX, TW, 3, false>;
    case 4: return full ? (const void *)ks_chain16_kernel<TX, TW, 4, true> : (const void *)ks_chain16_kernel<TX, TW, 4, false>;
    default: return nullptr;
    }
}

}  // namespace

// Returns KSMM_ERR_BAD_ALGO when the chain is not a radix-16 butterfly this kernel takes.
int chain16_run(const ksmm_factor_desc *f, int n, const void *x, void *y, int64_t batch, int x_dtype,
                int y_dtype, int bs_last, bool launch, hipStream_t stream, const ksmm_epilogue *ep)
{
    if (!bs_last || n < 2 || n > 4 || y_dtype != KSMM_F16) return KSMM_ERR_BAD_ALGO;
    if (x_dtype != KSMM_FP8_E4M3 && x_dtype != KSMM_F16) return KSMM_ERR_BAD_ALGO;
    const int64_t n_feat = (int64_t)f[0].a * 16 * f[0].d;
    if (n_feat > 1024 || n_feat % 16) return KSMM_ERR_BAD_ALGO;
    for (int i = 0; i < n; ++i) {
        if (f[i].b != 16 || f[i].c != 16 || (int64_t)f[i].a * 16 * f[i].d != n_feat) return KSMM_ERR_BAD_ALGO;
        if (f[i].d & (f[i].d - 1)) return KSMM_ERR_BAD_ALGO;
        if (f[i].w_dtype != f[0].w_dtype) return KSMM_ERR_BAD_ALGO;
    }
    if (f[0].w_dtype != KSMM_FP8_E4M3 && f[0].w_dtype != KSMM_F16) return KSMM_ERR_BAD_ALGO;
    if (x_dtype == KSMM_FP8_E4M3 && f[0].w_dtype != KSMM_FP8_E4M3) return KSMM_ERR_BAD_ALGO;
    const int vec = x_dtype == KSMM_FP8_E4M3 ? 16 : 8;  // columns per 16-byte input vector
    if (batch % vec || batch % 8 || batch < 16) return KSMM_ERR_BAD_ALGO;
    if (((uintptr_t)x | (uintptr_t)y) & 15) return KSMM_ERR_BAD_ALGO;
    for (int i = 0; i < n; ++i)
        if ((uintptr_t)f[i].w & 15) return KSMM_ERR_BAD_ALGO;
    if (!launch) return KSMM_OK;
    // one persistent workgroup per CU
    const int64_t n_chunks = (batch + CH_TN - 1) / CH_TN;
    int64_t wgs = n_chunks < 256 ? n_chunks : 256;
    const bool full = n_feat == 1024 && batch % CH_TN == 0;
    const void *fn;
    if (x_dtype == KSMM_FP8_E4M3)
        fn = chain16_fn<fp8_t, fp8_t>(n, full);
    else if (f[0].w_dtype == KSMM_FP8_E4M3)
        fn = chain16_fn<half_t, fp8_t>(n, full);
    else
        fn = chain16_fn<half_t, half_t>(n, full);
    Chain16Args args;
    for (int i = 0; i < 4; ++i) {
        const int j = i < n ? i : n - 1;
        args.w[i] = f[j].w;
        args.log2d[i] = __builtin_ctz((unsigned)f[j].d);
        args.scale[i] = f[j].scale;
    }
    args.bias = ep ? ep->bias : nullptr;
    args.act = ep ? ep->act : KSMM_ACT_NONE;
    const int lds = (int)n_feat * CH_ROW;
    if (ensure_dynamic_lds(fn, lds) != KSMM_OK) return KSMM_ERR_LAUNCH;
    int batch_i = (int)batch, n_feat_i = (int)n_feat;
    void *kargs[] = {(void *)&x, (void *)&y, (void *)&args, &batch_i, &n_feat_i};
    hipError_t e = hipLaunchKernel(fn, dim3((unsigned)wgs), dim3(CH_THREADS), kargs, lds, stream);
    return e == hipSuccess ? KSMM_OK : KSMM_ERR_LAUNCH;
}

}  // namespace ksmm
