// MFMA building blocks shared by the LDS-staged kernel families (gfx950 only): register staging
// of 16-byte global vectors, MFMA operand fetch from LDS, LDS row paddings.
#pragma once
#include "ksmm_common.h"

namespace ksmm {

typedef short short4_t __attribute__((ext_vector_type(4)));

template <typename CT> struct compute;  // CT = element type held in LDS and fed to the MFMA
template <> struct compute<float> {
    static constexpr int KSTEP = 2;  // k per MFMA
};
template <> struct compute<half_t> {
    static constexpr int KSTEP = 16;
};
template <> struct compute<fp8_t> {  // e4m3 operands straight into the fp8 MFMA
    static constexpr int KSTEP = 16;
};

// 16 bytes of global memory -> EPV elements of CT, written to LDS contiguously;
// register-staged variant: load now, write to LDS later
template <typename TS, typename CT> struct stage;
template <> struct stage<float, float> {
    static constexpr int EPV = 4;
    uint4_t v;
    __device__ __forceinline__ void load(const float *g) { v = *(const uint4_t *)g; }
    __device__ __forceinline__ void store(float *l) const { *(uint4_t *)l = v; }
};
template <> struct stage<half_t, half_t> {
    static constexpr int EPV = 8;
    uint4_t v;
    __device__ __forceinline__ void load(const half_t *g) { v = *(const uint4_t *)g; }
    __device__ __forceinline__ void store(half_t *l) const { *(uint4_t *)l = v; }
};
template <> struct stage<fp8_t, half_t> {
    static constexpr int EPV = 16;
    uint4_t v;
    __device__ __forceinline__ void load(const fp8_t *g) { v = *(const uint4_t *)g; }
    __device__ __forceinline__ void store(half_t *l) const
    {
        uint4_t lo, hi;
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            lo[2 * i] = __builtin_bit_cast(uint32_t, fp8x2_to_half2(v[i]));
            lo[2 * i + 1] = __builtin_bit_cast(uint32_t, fp8x2_hi_to_half2(v[i]));
            hi[2 * i] = __builtin_bit_cast(uint32_t, fp8x2_to_half2(v[2 + i]));
            hi[2 * i + 1] = __builtin_bit_cast(uint32_t, fp8x2_hi_to_half2(v[2 + i]));
        }
        *(uint4_t *)l = lo;
        *(uint4_t *)(l + 8) = hi;
    }
};

// ---- MFMA fragment fetch from LDS ------------------------------------------------------------
// K-outer storage S[k][idx] (row stride ld elements): lane (i = lane % 32, kq = lane / 32)
template <typename CT> struct frag;
template <> struct frag<float> {
    typedef float type;
    __device__ static __forceinline__ float k_outer(const float *s, int ld, int idx0, int k0, int lane)
    {
        return s[(k0 + (lane >> 5)) * ld + idx0 + (lane & 31)];
    }
    __device__ static __forceinline__ float k_inner(const float *s, int ld, int idx0, int k0, int lane)
    {
        return s[(idx0 + (lane & 31)) * ld + k0 + (lane >> 5)];
    }
    __device__ static __forceinline__ float16_t mfma(float a, float b, float16_t c)
    {
        return __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0);
    }
};
template <> struct frag<half_t> {
    typedef half8_t type;
    __device__ static __forceinline__ half8_t k_outer(const half_t *s, int ld, int idx0, int k0, int lane)
    {
        // two transpose loads of 4 k each; a 16-lane group addresses 4 rows x 16 columns
        const int kq = lane >> 5, i16 = lane & 15, half_sel = (lane >> 4) & 1;
        const half_t *p = s + (k0 + 8 * kq + (i16 >> 2)) * ld + idx0 + 16 * half_sel + 4 * (i16 & 3);
        typedef short4_t __attribute__((address_space(3))) * lds_ptr;
        short4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(p));
        short4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(p + 4 * ld));
        typedef short short8_t __attribute__((ext_vector_type(8)));
        short8_t r = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
        return __builtin_bit_cast(half8_t, r);
    }
    // the operand of the 8-k step: k = k0 + 4 * (lane / 32) .. + 3 of column lane % 32
    __device__ static __forceinline__ half4_t k_outer4(const half_t *s, int ld, int idx0, int k0, int lane)
    {
        const int kq = lane >> 5, i16 = lane & 15, half_sel = (lane >> 4) & 1;
        const half_t *p = s + (k0 + 4 * kq + (i16 >> 2)) * ld + idx0 + 16 * half_sel + 4 * (i16 & 3);
        typedef short4_t __attribute__((address_space(3))) * lds_ptr;
        return __builtin_bit_cast(half4_t, __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(p)));
    }
    __device__ static __forceinline__ half8_t k_inner(const half_t *s, int ld, int idx0, int k0, int lane)
    {
        return *(const half8_t *)(s + (idx0 + (lane & 31)) * ld + k0 + 8 * (lane >> 5));
    }
    __device__ static __forceinline__ float16_t mfma(half8_t a, half8_t b, float16_t c)
    {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
    }
};

template <> struct frag<fp8_t> {
    typedef long type;  // 8 e4m3 values: k = 8 * (lane / 32) .. + 7 of row / column lane % 32
    __device__ static __forceinline__ float16_t mfma(long a, long b, float16_t c)
    {
        return __builtin_amdgcn_mfma_f32_32x32x16_fp8_fp8(a, b, c, 0, 0, 0);
    }
};

// LDS row paddings (elements): K-outer rows are read 32 consecutive elements at a time by
// two or four row groups, K-inner rows by 16-byte pieces of 32 different rows.
template <typename CT> struct pads;
template <> struct pads<float> {
    static constexpr int outer(int n) { return n + (((n % 64) == 32) ? 0 : ((96 - n % 64) % 64)); }
    static constexpr int inner(int k) { return k + 4; }
};
template <> struct pads<half_t> {
    static constexpr int outer(int n) { return n + ((((2 * n) % 128) == 32) ? 0 : (((160 - (2 * n) % 128) % 128) / 2)); }
    static constexpr int inner(int k) { return k + 8; }
};

}  // namespace ksmm
