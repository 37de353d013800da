/* CPU oracle for the Kronecker-sparse factor product, plain C.  TEST INFRASTRUCTURE ONLY:
 * nothing in the shipped library links or loads this file; tests, the smoke check and the
 * CPU-baseline leg of the benchmark do.
 *
 * Restates the CPU check of the reference's stand-alone harness
 * (src/ksmm_cu/src/template_sparse_mm.cu:813-842): for every batch row, every residue
 * m = j % d, every output j and every input k of the same super-block and residue,
 *     out[i][j] += in[i][k] * valuesT[sb*b*c*d + m*b*c + (k_in_sb/d)*b + j_in_sb/d]
 * with valuesT being the "kernel format" (a*d*c, b) of
 * src/ksmm_py/layer/kronecker_sparse/interface.py:65-69.  Unlike the harness, which
 * accumulates in the storage type, the sum is carried in double.
 *
 * Pinned by tests/test_oracle.py against the numpy five-loop definition.
 */
#include <stddef.h>

#define KS_ORACLE_BODY(TIN, TOUT)                                                         \
    if (a <= 0 || b <= 0 || c <= 0 || d <= 0 || nb < 0) return 1;                          \
    const long in_size = (long)a * c * d, out_size = (long)a * b * d;                      \
    _Pragma("omp parallel for schedule(static)")                                           \
    for (long j = 0; j < out_size; j++) {                                                  \
        const long sb = j / ((long)b * d);           /* super-block a_i            */      \
        const long j_in = j - sb * (long)b * d;      /* = b_i*d + d_i              */      \
        const long m = j_in % d, bi = j_in / d;                                            \
        const TIN *wcol = w + ((sb * d + m) * (long)c) * b + bi; /* stride b over c_i */   \
        for (long i = 0; i < nb; i++) {                                                    \
            double acc = 0.0;                                                              \
            for (long ci = 0; ci < c; ci++) {                                              \
                const long k = (sb * c + ci) * d + m;                                      \
                const double xv = bs_last ? (double)x[k * nb + i] : (double)x[i * in_size + k]; \
                acc += xv * (double)wcol[ci * b];                                          \
            }                                                                              \
            if (bs_last) y[j * nb + i] = (TOUT)acc; else y[i * out_size + j] = (TOUT)acc;  \
        }                                                                                  \
    }                                                                                      \
    return 0;

/* x: (a*c*d, nb) if bs_last else (nb, a*c*d); w: kernel format (a*d*c, b); y likewise. */
int ks_oracle_factor_f32(const float *x, const float *w, double *y, long nb, int a, int b,
                         int c, int d, int bs_last)
{
    KS_ORACLE_BODY(float, double)
}

int ks_oracle_factor_f64(const double *x, const double *w, double *y, long nb, int a, int b,
                         int c, int d, int bs_last)
{
    KS_ORACLE_BODY(double, double)
}
