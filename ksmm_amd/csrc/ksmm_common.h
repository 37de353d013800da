// Shared device/host helpers for the KS kernels (gfx950 only).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/ksmm_hip.h"

namespace ksmm {

typedef _Float16 half_t;
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef _Float16 half16_t __attribute__((ext_vector_type(16)));
typedef float float2_t __attribute__((ext_vector_type(2)));
typedef float float4_t __attribute__((ext_vector_type(4)));
typedef float float16_t __attribute__((ext_vector_type(16)));
typedef uint32_t uint2_t __attribute__((ext_vector_type(2)));
typedef uint32_t uint4_t __attribute__((ext_vector_type(4)));

struct fp8_t {  // OCP e4m3fn storage
    uint8_t bits;
};

// e4m3fn -> fp16 is exact: shift the 7 magnitude bits into the fp16 exponent/mantissa
// fields and rescale by 2^8 (the difference of the exponent biases, 15 - 7).  Sub-normals
// of e4m3fn land on fp16 sub-normals before the rescale, so they come out exact as well.
__device__ __forceinline__ half_t fp8_to_half(uint8_t v)
{
    uint16_t h = (uint16_t)(((uint16_t)(v & 0x80u) << 8) | ((uint16_t)(v & 0x7fu) << 7));
    return __builtin_bit_cast(half_t, h) * (half_t)256.0f;
}

// Two e4m3fn bytes (bits 0-7 and 8-15 of `v`) -> packed fp16 pair: the hardware conversion
// (v_cvt_scalef32_pk_f16_fp8 with unit scale; exact, every e4m3fn value is an fp16 value).
__device__ __forceinline__ half2_t fp8x2_to_half2(uint32_t v)
{
    return __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(v, 1.0f, false);
}
// the same for bits 16-23 and 24-31
__device__ __forceinline__ half2_t fp8x2_hi_to_half2(uint32_t v)
{
    return __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(v, 1.0f, true);
}

template <typename T> struct elem;
template <> struct elem<float> {
    static constexpr int dtype = KSMM_F32;
    __device__ static __forceinline__ float load(const float *p) { return *p; }
    __device__ static __forceinline__ void store(float *p, float v) { *p = v; }
};
template <> struct elem<half_t> {
    static constexpr int dtype = KSMM_F16;
    __device__ static __forceinline__ float load(const half_t *p) { return (float)*p; }
    __device__ static __forceinline__ void store(half_t *p, float v) { *p = (half_t)v; }
};
template <> struct elem<fp8_t> {
    static constexpr int dtype = KSMM_FP8_E4M3;
    __device__ static __forceinline__ float load(const fp8_t *p) { return (float)fp8_to_half(p->bits); }
};

static inline size_t dtype_size(int dt)
{
    return dt == KSMM_F32 ? 4 : dt == KSMM_F16 ? 2 : 1;
}

// One factor problem, as the launchers see it.
struct Problem {
    const void *x;
    const void *w;
    void *y;
    int64_t batch;
    int a, b, c, d;
    int x_dtype, w_dtype, y_dtype;
    int bs_last;
    float scale;
    hipStream_t stream;
    const void *bias = nullptr;  // one value of y's type per output feature, or none
    int act = KSMM_ACT_NONE;
};

// What a kernel does to an fp32 accumulator before rounding it to the output type:
// v = act(acc * scale + bias[output feature]).  Passed to the kernels by value.
struct Epi {
    float scale;
    int act;
    const void *bias;
};
static inline Epi epi_of(const Problem &p) { return Epi{p.scale, p.act, p.bias}; }

// GELU, erf form: x * Phi(x) = max(x, 0) - |x| * erfc(|x| / sqrt 2) / 2.  erfc by Abramowitz &
// Stegun 7.1.26 (|error| <= 1.5e-7, branch-free: one reciprocal, one exponential, a degree-4
// polynomial in t = 1 / (1 + p z)), far inside fp32 storage rounding of the result for the
// value range of activations.  The constants carry the factors the formula would multiply by:
// with z' = |x| sqrt(log2(e) / 2) the exponential is 2^(-z'^2), p is divided by sqrt(log2 e),
// and the polynomial's coefficients are halved: 12 vector instructions per value, two of them
// transcendental, which is what an epilogue with GELU costs next to the multiplications.
__device__ __forceinline__ float gelu_erf(float x)
{
    const float ax = fabsf(x);
    const float z = ax * 0.84932180028801907f;
    const float t = __builtin_amdgcn_rcpf(fmaf(0.2727374808792225f, z, 1.0f));
    float poly = fmaf(0.5307027145f, t, -0.7265760135f);
    poly = fmaf(poly, t, 0.7107068705f);
    poly = fmaf(poly, t, -0.142248368f);
    poly = fmaf(poly, t, 0.127414796f);
    const float tail = (poly * t) * __builtin_amdgcn_exp2f(-(z * z));  // erfc(|x| / sqrt 2) / 2
    return fmaf(-ax, tail, fmaxf(x, 0.f));
}

// GELU of v when `on` (uniform over the wave), v otherwise: a branch, never a select, so that a
// bias-only or plain epilogue does not pay for the GELU of every output (the empty asm keeps the
// compiler from computing both sides and choosing).
__device__ __forceinline__ float gelu_if(bool on, float v)
{
    if (on) {
        asm volatile("");
        v = gelu_erf(v);
    }
    return v;
}

template <typename TY> __device__ __forceinline__ float epi_bias(const Epi &e, size_t feature)
{
    return e.bias ? (float)((const TY *)e.bias)[feature] : 0.f;
}
__device__ __forceinline__ float epi_finish(const Epi &e, float acc, float bias_value)
{
    return gelu_if(e.act == KSMM_ACT_GELU, fmaf(acc, e.scale, bias_value));
}

// dtype combination index: 0 f32, 1 f16, 2 fp8*fp8->f16, 3 f16*fp8->f16, -1 unsupported
static inline int combo_of(int xd, int wd, int yd)
{
    if (xd == KSMM_F32 && wd == KSMM_F32 && yd == KSMM_F32) return 0;
    if (xd == KSMM_F16 && wd == KSMM_F16 && yd == KSMM_F16) return 1;
    if (xd == KSMM_FP8_E4M3 && wd == KSMM_FP8_E4M3 && yd == KSMM_F16) return 2;
    if (xd == KSMM_F16 && wd == KSMM_FP8_E4M3 && yd == KSMM_F16) return 3;
    return -1;
}

// Kernels that use more than 64 KB of dynamic LDS need their limit raised before the first
// launch.  Done once per (kernel, device): later calls only look the pair up.  Returns
// KSMM_OK or KSMM_ERR_LAUNCH.
int ensure_dynamic_lds(const void *fn, int bytes);

// Stable identity of a kernel instance: a hash of the numbers that describe it (family tag and
// template parameters), not of its position in an instance table.  The measured table names
// instances by these, so inserting or reordering instances cannot re-target its rows.
static inline uint32_t inst_hash(uint32_t tag, const int *v, int n)
{
    uint32_t h = 2166136261u ^ tag;
    for (int i = 0; i < n; ++i) {
        h ^= (uint32_t)v[i];
        h *= 16777619u;
        h ^= h >> 15;
    }
    return (h & 0x7fffffffu) | 1u;  // positive and never 0
}
// per (sub-)family: number of instances and the id of instance i (0 when i is out of range)
int wave_inst_count(int combo);
uint32_t wave_inst_id(int combo, int i);
int rows_inst_count();
uint32_t rows_inst_id(int i);
int stream_inst_count();
uint32_t stream_inst_id(int i);
int ktile_inst_count();
uint32_t ktile_inst_id(int i);
int ws_inst_count();
uint32_t ws_inst_id(int i);
int bf_inst_count();
uint32_t bf_inst_id(int i);
int gemm_inst_count();
uint32_t gemm_inst_id(int i);

// Launchers, one per kernel family.  Each fills `tile` and, when `launch` is true, enqueues
// the kernel on p.stream.  They return KSMM_ERR_BAD_ALGO when the family (or the requested
// variant) cannot run the problem.
int generic_run(const Problem &p, int variant, bool launch, ksmm_tile *tile);
int wave_run(const Problem &p, int variant, bool launch, ksmm_tile *tile);
int tile_run(const Problem &p, int variant, bool launch, ksmm_tile *tile);
int stream_run(const Problem &p, int variant, bool launch, ksmm_tile *tile);  // part of the tile family
int rows_bf_run(const Problem &p, int variant, bool launch, ksmm_tile *tile);  // part of the wave family
int gemm_run(const Problem &p, int variant, bool launch, ksmm_tile *tile);  // part of the tile family
int tile_bf_run(const Problem &p, int variant, bool launch, ksmm_tile *tile);  // part of the tile family

// Backward pass pieces (ksmm_backward.hip): blockwise transpose of a kernel-format weight, and the
// weight gradient (acc: fp32 scratch of wgrad_partial_floats() elements, one slice of a*b*c*d per
// batch split; kernel_used: 1 MFMA kernel, 0 tiled).
int block_transpose_run(const void *w, void *wt, int a, int b, int c, int d, int dtype, hipStream_t stream);
int64_t wgrad_partial_floats(int64_t batch, int a, int b, int c, int d, int dtype);
int wgrad_run(const void *dy, const void *x, void *dw, float *acc, int64_t batch, int a, int b, int c, int d,
              int dtype, int bs_last, float scale, hipStream_t stream, int *kernel_used);

// Fused radix-16 chain (intermediates in LDS); KSMM_ERR_BAD_ALGO when the chain does not qualify.
// out (cols x rows) = transpose of in (rows x cols); pitches in elements per row, 0 = dense
int transpose_run(const void *in, void *out, int64_t rows, int64_t cols, int elem_bytes, hipStream_t stream,
                  int64_t in_pitch = 0, int64_t out_pitch = 0);
// zeros in columns [cols, pitch) of every row of a (rows x pitch) matrix
int zero_pad_run(void *p, int64_t rows, int64_t cols, int64_t pitch, int elem_bytes, hipStream_t stream);
// out (rows x cols_out) = the rows of in (rows x cols_in) cut or zero-filled to cols_out columns
int repitch_run(const void *in, void *out, int64_t rows, int64_t cols_in, int64_t cols_out, int elem_bytes,
                hipStream_t stream);
int chain16_run(const ksmm_factor_desc *f, int n, const void *x, void *y, int64_t batch, int x_dtype,
                int y_dtype, int bs_last, bool launch, hipStream_t stream, const ksmm_epilogue *ep);

}  // namespace ksmm
