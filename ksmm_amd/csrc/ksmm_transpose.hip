// Layout change between batch-size-first (batch, features) and batch-size-last (features,
// batch): a plain 2-D transpose of 1-, 2- or 4-byte elements through a 64 x 64 LDS tile.
//
// It serves the batch-size-first factors with d > 1 that have no kernel of their own: in that
// layout the inputs of one block are d elements apart, which the MFMA operand loads cannot
// gather; the factor (or the whole chain) is run in batch-size-last layout between two
// transposes instead, on a workspace the caller provides.
//
// Global memory is read and written with 16-byte vectors (128-byte runs per row of a tile) when
// the sizes and addresses allow it, element by element otherwise.  The tile is kept in LDS with
// an odd stride in 4-byte words, so that the column reads of the store phase spread over the
// 64 banks.
//
// The same file holds the row re-pitch copy (rows cut or zero-filled to another length), which
// serves batch-size-last problems whose batch is not a multiple of the 16-byte vector: they run
// on a copy whose rows are padded to the vector, and the result is copied back.
//
// Reference counterpart: none as a kernel (the reference's batch-size-first kernels gather with
// strided scalar loads, template_kernels_float.cuh:156-161); KSLinear permutes activations with
// torch in its 'bmm' path (interface.py:213-267).
#include "ksmm_common.h"

namespace ksmm {

namespace {

constexpr int TT = 64;  // tile edge, elements

template <int ES> struct elem_of;
template <> struct elem_of<1> { typedef uint8_t type; };
template <> struct elem_of<2> { typedef uint16_t type; };
template <> struct elem_of<4> { typedef uint32_t type; };

// in: rows x cols, row-major with in_pitch elements per row; out: cols x rows with out_pitch
// elements per row.  VIN / VOUT: 16-byte vectors on that side (the pitch is a multiple of the
// vector there; a vector may reach past the last column into the padding of its row: what it
// reads there is never stored inside the matrix, what it writes there is never read).
template <int ES, bool VIN, bool VOUT>
__global__ __launch_bounds__(256) void ks_transpose_kernel(const void *__restrict__ in_, void *__restrict__ out_,
                                                          int rows, int cols, int tiles_c, int in_pitch,
                                                          int out_pitch)
{
    typedef typename elem_of<ES>::type T;
    constexpr int V = 16 / ES;             // elements per vector
    constexpr int LD = TT + 4 / ES;        // row stride in elements: an odd number of 4-byte words
    __shared__ __attribute__((aligned(16))) T tile[TT * LD + 8];
    const T *in = (const T *)in_;
    T *out = (T *)out_;
    const int tr = blockIdx.x / tiles_c, tc = blockIdx.x - tr * tiles_c;
    const int r0 = tr * TT, c0 = tc * TT;
    const int tid = threadIdx.x;

    // ---- load: tile[r][c] = in[r0 + r][c0 + c] ----
    if (VIN) {
        constexpr int VPR = TT / V;  // vectors per tile row
#pragma unroll
        for (int i = 0; i < TT * VPR / 256; ++i) {
            const int q = tid + i * 256, r = q / VPR, cv = (q % VPR) * V;
            if (r0 + r < rows && c0 + cv < cols) {  // in_pitch % V == 0: whole vectors
                const uint4_t v = *(const uint4_t *)(in + (size_t)(r0 + r) * in_pitch + c0 + cv);
                // 4-byte LDS writes (the odd stride leaves rows only 4-byte aligned)
                uint32_t *dst = (uint32_t *)(tile + r * LD + cv);
                dst[0] = v[0];
                dst[1] = v[1];
                dst[2] = v[2];
                dst[3] = v[3];
            }
        }
    } else {
        for (int q = tid; q < TT * TT; q += 256) {
            const int r = q / TT, c = q % TT;
            if (r0 + r < rows && c0 + c < cols) tile[r * LD + c] = in[(size_t)(r0 + r) * in_pitch + c0 + c];
        }
    }
    __syncthreads();
    // ---- store: out[c0 + c][r0 + r] = tile[r][c] ----
    if (VOUT) {
        constexpr int VPR = TT / V;
#pragma unroll
        for (int i = 0; i < TT * VPR / 256; ++i) {
            const int q = tid + i * 256, c = q / VPR, rv = (q % VPR) * V;
            if (c0 + c < cols && r0 + rv < rows) {  // out_pitch % V == 0
                T e[V];
#pragma unroll
                for (int j = 0; j < V; ++j) e[j] = tile[(rv + j) * LD + c];
                uint4_t v;
                if constexpr (ES == 4) {
                    v = uint4_t{e[0], e[1], e[2], e[3]};
                } else if constexpr (ES == 2) {
#pragma unroll
                    for (int j = 0; j < 4; ++j) v[j] = (uint32_t)e[2 * j] | ((uint32_t)e[2 * j + 1] << 16);
                } else {
#pragma unroll
                    for (int j = 0; j < 4; ++j)
                        v[j] = (uint32_t)e[4 * j] | ((uint32_t)e[4 * j + 1] << 8) | ((uint32_t)e[4 * j + 2] << 16) |
                               ((uint32_t)e[4 * j + 3] << 24);
                }
                *(uint4_t *)(out + (size_t)(c0 + c) * out_pitch + r0 + rv) = v;
            }
        }
    } else {
        for (int q = tid; q < TT * TT; q += 256) {
            const int c = q / TT, r = q % TT;
            if (r0 + r < rows && c0 + c < cols) out[(size_t)(c0 + c) * out_pitch + r0 + r] = tile[r * LD + c];
        }
    }
}

// the padding of every row of a pitched matrix: element q of the padding is column cols + q % pad
// of row q / pad
template <int ES>
__global__ __launch_bounds__(256) void ks_zero_pad_kernel(void *__restrict__ p_, int64_t total, int64_t pad, int64_t cols,
                                                         int64_t pitch)
{
    typedef typename elem_of<ES>::type T;
    const int64_t q = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (q >= total) return;
    const int64_t row = q / pad;
    ((T *)p_)[row * pitch + cols + (q - row * pad)] = 0;
}

template <int ES> const void *transpose_fn(bool vin, bool vout)
{
    if (vin && vout) return (const void *)ks_transpose_kernel<ES, true, true>;
    if (vin) return (const void *)ks_transpose_kernel<ES, true, false>;
    if (vout) return (const void *)ks_transpose_kernel<ES, false, true>;
    return (const void *)ks_transpose_kernel<ES, false, false>;
}

// out (rows x cols_out) <- in (rows x cols_in): the first min(cols_in, cols_out) columns of
// every row, zeros behind them.  A thread moves one 16-byte vector: aligned on the side whose
// row length is a multiple of the vector (VOUT: widening, VIN: narrowing), at element alignment
// on the other, element by element where the vector straddles the end of the row.
template <int ES, bool VIN, bool VOUT>
__global__ __launch_bounds__(256) void ks_repitch_kernel(const void *__restrict__ in_, void *__restrict__ out_,
                                                        int64_t rows, int cols_in, int cols_out, int vec_per_row)
{
    typedef typename elem_of<ES>::type T;
    constexpr int V = 16 / ES;
    const T *in = (const T *)in_;
    T *out = (T *)out_;
    const int64_t id = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int64_t r = id / vec_per_row;
    const int c0 = (int)(id - r * vec_per_row) * V;
    if (r >= rows) return;
    const T *src = in + r * cols_in + c0;
    T *dst = out + r * cols_out + c0;
    union {
        uint4_t v;
        T e[V];
    } u;
    u.v = uint4_t{0u, 0u, 0u, 0u};
    if (VIN) {  // cols_in % V == 0 and c0 < cols_out <= cols_in: a whole, aligned vector
        u.v = *(const uint4_t *)src;
    } else if (c0 + V <= cols_in) {
        // a whole vector at element alignment (global memory takes unaligned vector accesses)
        __builtin_memcpy(&u.v, src, 16);
    } else {
#pragma unroll
        for (int j = 0; j < V; ++j)
            if (c0 + j < cols_in) u.e[j] = src[j];
    }
    if (VOUT) {  // cols_out % V == 0
        *(uint4_t *)dst = u.v;
    } else if (c0 + V <= cols_out) {
        __builtin_memcpy(dst, &u.v, 16);
    } else {
#pragma unroll
        for (int j = 0; j < V; ++j)
            if (c0 + j < cols_out) dst[j] = u.e[j];
    }
}

template <int ES> const void *repitch_fn(bool vin, bool vout)
{
    if (vin && vout) return (const void *)ks_repitch_kernel<ES, true, true>;
    if (vin) return (const void *)ks_repitch_kernel<ES, true, false>;
    if (vout) return (const void *)ks_repitch_kernel<ES, false, true>;
    return (const void *)ks_repitch_kernel<ES, false, false>;
}

}  // namespace

// out (rows x cols_out) = the rows of in (rows x cols_in) cut or zero-filled to cols_out columns
int repitch_run(const void *in, void *out, int64_t rows, int64_t cols_in, int64_t cols_out, int elem_bytes,
                hipStream_t stream)
{
    if (rows < 1 || cols_in < 1 || cols_out < 1 || cols_in > 0x7fffffffLL || cols_out > 0x7fffffffLL)
        return KSMM_ERR_TOO_LARGE;
    const int v = 16 / elem_bytes;
    // threads cover the output's columns; input vectors only where those all lie inside the input
    const bool vin = cols_in % v == 0 && cols_out <= cols_in && ((uintptr_t)in & 15) == 0;
    const bool vout = cols_out % v == 0 && ((uintptr_t)out & 15) == 0;
    const int64_t vec_per_row = (cols_out + v - 1) / v;
    const int64_t blocks = (rows * vec_per_row + 255) / 256;
    if (blocks > 0x7fffffffLL) return KSMM_ERR_TOO_LARGE;
    const void *fn = elem_bytes == 4 ? repitch_fn<4>(vin, vout)
                                     : elem_bytes == 2 ? repitch_fn<2>(vin, vout) : repitch_fn<1>(vin, vout);
    int ci = (int)cols_in, co = (int)cols_out, vpr = (int)vec_per_row;
    void *args[] = {(void *)&in, (void *)&out, &rows, &ci, &co, &vpr};
    hipError_t e = hipLaunchKernel(fn, dim3((unsigned)blocks), dim3(256), args, 0, stream);
    return e == hipSuccess ? KSMM_OK : KSMM_ERR_LAUNCH;
}

// out (cols x rows, out_pitch elements per row) = transpose of in (rows x cols, in_pitch elements
// per row); elem_bytes in {1, 2, 4}; a pitch of 0 means the dense one
// zeros in columns [cols, pitch) of every row of a (rows x pitch) matrix of 1-, 2- or 4-byte elements
int zero_pad_run(void *p, int64_t rows, int64_t cols, int64_t pitch, int elem_bytes, hipStream_t stream)
{
    if (pitch <= cols) return KSMM_OK;
    const int64_t pad = pitch - cols, total = rows * pad;
    if ((total + 255) / 256 > 0x7fffffffLL) return KSMM_ERR_TOO_LARGE;
    const void *fn = elem_bytes == 4 ? (const void *)ks_zero_pad_kernel<4>
                                     : elem_bytes == 2 ? (const void *)ks_zero_pad_kernel<2> : (const void *)ks_zero_pad_kernel<1>;
    void *args[] = {(void *)&p, (void *)&total, (void *)&pad, (void *)&cols, (void *)&pitch};
    hipError_t e = hipLaunchKernel(fn, dim3((unsigned)((total + 255) / 256)), dim3(256), args, 0, stream);
    return e == hipSuccess ? KSMM_OK : KSMM_ERR_LAUNCH;
}

int transpose_run(const void *in, void *out, int64_t rows, int64_t cols, int elem_bytes, hipStream_t stream,
                  int64_t in_pitch, int64_t out_pitch)
{
    if (in_pitch == 0) in_pitch = cols;
    if (out_pitch == 0) out_pitch = rows;
    if (rows < 1 || cols < 1 || in_pitch < cols || out_pitch < rows || in_pitch > 0x7fffffffLL ||
        out_pitch > 0x7fffffffLL)
        return KSMM_ERR_TOO_LARGE;
    const int v = 16 / elem_bytes;
    const bool vin = in_pitch % v == 0 && ((uintptr_t)in & 15) == 0;
    const bool vout = out_pitch % v == 0 && ((uintptr_t)out & 15) == 0;
    const void *fn = elem_bytes == 4 ? transpose_fn<4>(vin, vout)
                                     : elem_bytes == 2 ? transpose_fn<2>(vin, vout) : transpose_fn<1>(vin, vout);
    const int64_t tiles_r = (rows + TT - 1) / TT, tiles_c = (cols + TT - 1) / TT;
    if (tiles_r * tiles_c > 0x7fffffffLL) return KSMM_ERR_TOO_LARGE;
    int rows_i = (int)rows, cols_i = (int)cols, tiles_c_i = (int)tiles_c, ip = (int)in_pitch, op = (int)out_pitch;
    void *args[] = {(void *)&in, (void *)&out, &rows_i, &cols_i, &tiles_c_i, &ip, &op};
    hipError_t e = hipLaunchKernel(fn, dim3((unsigned)(tiles_r * tiles_c)), dim3(256), args, 0, stream);
    return e == hipSuccess ? KSMM_OK : KSMM_ERR_LAUNCH;
}

}  // namespace ksmm
