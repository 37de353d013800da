// C ABI of libksmm_hip.so: argument checks, kernel-family dispatch, factor chains.
#include <string.h>

#include <atomic>

#include "ksmm_common.h"

using namespace ksmm;

namespace ksmm {

// (kernel, device) pairs whose dynamic-LDS limit has been raised: a fixed open-addressing set
// of atomics.  Insert-only and idempotent, so concurrent callers need no lock; it holds no
// caller-visible state (a lost race only repeats the attribute call).
int ensure_dynamic_lds(const void *fn, int bytes)
{
    if (bytes <= 64 * 1024) return KSMM_OK;
    constexpr unsigned SLOTS = 4096;  // far more than kernels x devices
    static std::atomic<uintptr_t> seen[SLOTS];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return KSMM_ERR_LAUNCH;
    const uintptr_t key = ((uintptr_t)fn << 8) ^ (uintptr_t)(dev + 1);
    unsigned h = (unsigned)((key * 0x9E3779B97F4A7C15ull) >> 40) % SLOTS;
    for (unsigned probe = 0; probe < SLOTS; ++probe, h = (h + 1) % SLOTS) {
        const uintptr_t cur = seen[h].load(std::memory_order_acquire);
        if (cur == key) return KSMM_OK;
        if (cur != 0) continue;
        // every instance declares its full ring; the limit never has to grow afterwards
        if (hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, bytes) != hipSuccess)
            return KSMM_ERR_LAUNCH;
        uintptr_t expected = 0;
        seen[h].compare_exchange_strong(expected, key, std::memory_order_release);
        return KSMM_OK;
    }
    // table full (cannot happen with the instance counts of this library): set it every time
    return hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, bytes) == hipSuccess
               ? KSMM_OK
               : KSMM_ERR_LAUNCH;
}

}  // namespace ksmm

// Scratch memory of ksmm_chain_forward_static: one fixed device array per GPU (each GPU that
// runs the library holds its own copy until the process ends).  In host code the name is only
// a handle for hipGetSymbolAddress (static_scratch below), never a device address.
constexpr int64_t KSMM_STATIC_SCRATCH_BYTES = 32ll << 20;
static __device__ __align__(256) unsigned char scratch[KSMM_STATIC_SCRATCH_BYTES];

namespace {

bool dtype_known(int dt) { return dt == KSMM_F32 || dt == KSMM_F16 || dt == KSMM_FP8_E4M3; }

int check_shape(int64_t batch, int a, int b, int c, int d, int xd, int wd, int yd)
{
    if (a < 1 || b < 1 || c < 1 || d < 1) return KSMM_ERR_BAD_PATTERN;
    if (batch < 1) return KSMM_ERR_BAD_BATCH;
    if (!dtype_known(xd) || !dtype_known(wd) || !dtype_known(yd)) return KSMM_ERR_BAD_DTYPE;
    if (combo_of(xd, wd, yd) < 0) return KSMM_ERR_BAD_DTYPE;
    const int64_t lim = 0x7fffffffLL;
    // products are checked step by step so that they cannot wrap
    int64_t acd = (int64_t)a * c;
    if (acd > lim) return KSMM_ERR_TOO_LARGE;
    acd *= d;
    int64_t abd = (int64_t)a * b;
    if (abd > lim) return KSMM_ERR_TOO_LARGE;
    abd *= d;
    if (acd > lim || abd > lim) return KSMM_ERR_TOO_LARGE;
    if (acd * batch > lim || abd * batch > lim) return KSMM_ERR_TOO_LARGE;
    int64_t nnz = (int64_t)a * b;
    nnz *= c;
    if (nnz > lim) return KSMM_ERR_TOO_LARGE;
    nnz *= d;
    if (nnz > lim) return KSMM_ERR_TOO_LARGE;
    return KSMM_OK;
}

// Measured choices for known patterns (the counterpart of the reference's *.best tables,
// src/ksmm_py/layer/kronecker_sparse/kernel.py:151-239): rows sorted by key.
// A row names its kernel by family, stable instance id (inst_hash of the instance's parameters)
// and a family-specific launch parameter, never by a position in an instance table.
struct TunedRow {
    int a, b, c, d, combo, bs_last, algo;
    uint32_t id;
    int param;
};
const TunedRow tuned_rows[] = {
#include "ksmm_tuned.inc"
    {0, 0, 0, 0, 0, 0, 0, 0, 0},  // sentinel: keeps the array non-empty
};

// (family, variant) <-> (family, instance id, parameter).  Variant layouts are those of
// ksmm_factor_forward_algo; `param` keeps what is not the instance: tiles per wave and tile
// order (wave), workgroups per a_i (row kernels), workgroups per block (stream, weight-stationary).
bool describe_variant(int algo, int variant, int combo, int bs_last, uint32_t *id, int *param)
{
    *param = 0;
    if (algo == KSMM_ALGO_GENERIC) {
        const int v[1] = {variant};
        *id = inst_hash('X', v, 1);
        return variant == 0 || variant == 1;
    }
    if (algo == KSMM_ALGO_WAVE) {
        if (bs_last) {
            if (variant < 0) return false;
            *id = wave_inst_id(combo, variant & 0xff);
            *param = variant >> 8;
        } else {
            if (variant < 1000) return false;
            *id = rows_inst_id((variant - 1000) & 0x3ff);
            *param = (variant - 1000) >> 10;
        }
        return *id != 0;
    }
    if (algo == KSMM_ALGO_TILE) {
        if (variant < 0) return false;
        const int sub = (variant >> 24) & 15, inst = variant & 0xff;
        *param = (variant >> 8) & 0xffff;
        switch (sub) {
        case 0: *id = ktile_inst_id(inst); break;
        case 1: *id = ws_inst_id(inst); break;
        case 2: *id = stream_inst_id(inst); break;
        case 3: *id = bf_inst_id(inst); break;
        case 4: *id = gemm_inst_id(inst); break;
        default: *id = 0;
        }
        return *id != 0;
    }
    return false;
}

template <typename F> int find_id(int n, uint32_t id, F id_of)
{
    for (int i = 0; i < n; ++i)
        if (id_of(i) == id) return i;
    return -1;
}

bool resolve_variant(int algo, uint32_t id, int param, int combo, int bs_last, int *variant)
{
    if (algo == KSMM_ALGO_GENERIC) {
        for (int v = 0; v <= 1; ++v) {
            const int a[1] = {v};
            if (inst_hash('X', a, 1) == id) return *variant = v, true;
        }
        return false;
    }
    if (algo == KSMM_ALGO_WAVE) {
        if (bs_last) {
            const int i = find_id(wave_inst_count(combo), id, [&](int k) { return wave_inst_id(combo, k); });
            return i >= 0 ? (*variant = i | (param << 8), true) : false;
        }
        const int i = find_id(rows_inst_count(), id, rows_inst_id);
        return i >= 0 ? (*variant = 1000 + (i | (param << 10)), true) : false;
    }
    if (algo == KSMM_ALGO_TILE) {
        int i, sub = 0;
        if ((i = find_id(ktile_inst_count(), id, ktile_inst_id)) >= 0) sub = 0;
        else if ((i = find_id(ws_inst_count(), id, ws_inst_id)) >= 0) sub = 1;
        else if ((i = find_id(stream_inst_count(), id, stream_inst_id)) >= 0) sub = 2;
        else if ((i = find_id(bf_inst_count(), id, bf_inst_id)) >= 0) sub = 3;
        else if ((i = find_id(gemm_inst_count(), id, gemm_inst_id)) >= 0) sub = 4;
        else return false;
        *variant = (sub << 24) | ((param & 0xffff) << 8) | i;
        return true;
    }
    return false;
}
constexpr int N_TUNED = (int)(sizeof(tuned_rows) / sizeof(TunedRow)) - 1;
constexpr int64_t TUNED_MIN_BATCH = 8192;  // the table was measured at batch 25088

int cmp_key(const TunedRow &r, const Problem &p, int combo)
{
    const int k[6] = {p.a, p.b, p.c, p.d, combo, p.bs_last};
    const int q[6] = {r.a, r.b, r.c, r.d, r.combo, r.bs_last};
    for (int i = 0; i < 6; ++i)
        if (q[i] != k[i]) return q[i] < k[i] ? -1 : 1;
    return 0;
}

const TunedRow *tuned_lookup(const Problem &p)
{
    const int combo = combo_of(p.x_dtype, p.w_dtype, p.y_dtype);
    int lo = 0, hi = N_TUNED - 1;
    while (lo <= hi) {
        const int mid = (lo + hi) / 2, c = cmp_key(tuned_rows[mid], p, combo);
        if (c == 0) return &tuned_rows[mid];
        if (c < 0)
            lo = mid + 1;
        else
            hi = mid - 1;
    }
    return nullptr;
}

// Family order for KSMM_ALGO_AUTO: the table inside each family decides whether it takes the
// problem; the generic family always does.
int dispatch(const Problem &p, int algo, int variant, bool launch, ksmm_tile *tile)
{
    switch (algo) {
    case KSMM_ALGO_GENERIC: return generic_run(p, variant, launch, tile);
    case KSMM_ALGO_WAVE: return wave_run(p, variant, launch, tile);
    case KSMM_ALGO_TILE: return tile_run(p, variant, launch, tile);
    case KSMM_ALGO_AUTO: {
        // variant -1: the tuned table first (large batches), then the heuristics below;
        // variant -3: heuristics only (what the tuner compares against)
        if (variant == -1 && p.batch >= TUNED_MIN_BATCH) {
            const TunedRow *row = tuned_lookup(p);
            int row_variant;
            if (row && row->algo != KSMM_ALGO_AUTO &&
                resolve_variant(row->algo, row->id, row->param, row->combo, row->bs_last, &row_variant)) {
                const int rc = dispatch(p, row->algo, row_variant, launch, tile);
                if (rc != KSMM_ERR_BAD_ALGO) return rc;
            }
        }
        // Table order from sweeps at batch 25088: batch-size-first 16-bit mid-sized blocks
        // (64x64 .. 192x192) go to the stream kernels of the tile family; batch-size-last blocks
        // the wave family has an instance for (up to 96x96), and fp32, go to the wave family,
        // larger 16-bit blocks to the stream kernels again (inside the tile family), the rest to
        // the GEMM and k-loop tiles; shapes none of them takes run on the generic kernel.
        int rc = KSMM_ERR_BAD_ALGO;
        if (p.x_dtype == KSMM_F16 && !p.bs_last) rc = stream_run(p, -1, launch, tile);
        if (rc != KSMM_ERR_BAD_ALGO) return rc;
        rc = wave_run(p, -1, launch, tile);
        if (rc != KSMM_ERR_BAD_ALGO) return rc;
        rc = tile_run(p, -1, launch, tile);
        if (rc != KSMM_ERR_BAD_ALGO) return rc;
        return generic_run(p, -1, launch, tile);
    }
    default: return KSMM_ERR_BAD_ALGO;
    }
}

// Rows of a batch-size-last workspace copy are padded to a multiple of 16 columns (the 16-byte
// vector of every type).
int64_t padded_batch(int64_t batch) { return (batch + 15) / 16 * 16; }

// A batch-size-first problem that only the generic kernel takes, while its batch-size-last
// twin has a real kernel: worth two transposes.  (The transposed copy has padded rows, so the
// twin runs at the padded batch.)
bool wants_transposed(const Problem &p)
{
    if (p.bs_last) return false;
    ksmm_tile t;
    memset(&t, 0, sizeof(t));
    if (dispatch(p, KSMM_ALGO_AUTO, -1, false, &t) != KSMM_OK || t.algo != KSMM_ALGO_GENERIC) return false;
    Problem q = p;
    q.bs_last = 1;
    q.batch = padded_batch(p.batch);
    // (a batch whose padded copies would pass the size limit stays on the kernel it has)
    if (check_shape(q.batch, p.a, p.b, p.c, p.d, p.x_dtype, p.w_dtype, p.y_dtype) != KSMM_OK) return false;
    memset(&t, 0, sizeof(t));
    // (the vector form of the generic kernel counts as a real kernel: variant 1)
    return dispatch(q, KSMM_ALGO_AUTO, -1, false, &t) == KSMM_OK && (t.algo != KSMM_ALGO_GENERIC || t.variant == 1);
}

// Batch-size-last rows are `batch` elements long: when that is not a multiple of the 16-byte
// vector only the one-thread-per-output kernel takes the problem.  With a workspace it runs on a
// copy whose rows are zero-filled to the next multiple of 16 columns (the vector of every type)
// and the result rows are cut back: two copies more, but on the kernel of the padded batch.
bool wants_padded(const Problem &p)
{
    if (!p.bs_last || p.batch % 16 == 0) return false;
    ksmm_tile t;
    memset(&t, 0, sizeof(t));
    if (dispatch(p, KSMM_ALGO_AUTO, -1, false, &t) != KSMM_OK || t.algo != KSMM_ALGO_GENERIC || t.variant == 1)
        return false;
    Problem q = p;
    q.batch = padded_batch(p.batch);
    if (check_shape(q.batch, p.a, p.b, p.c, p.d, p.x_dtype, p.w_dtype, p.y_dtype) != KSMM_OK) return false;
    memset(&t, 0, sizeof(t));
    return dispatch(q, KSMM_ALGO_AUTO, -1, false, &t) == KSMM_OK && (t.algo != KSMM_ALGO_GENERIC || t.variant == 1);
}

int64_t align256(int64_t v) { return (v + 255) / 256 * 256; }

// Bytes of the weight gradient's partial sums (at the batch as given and at the padded batch of the
// transposed copies: whichever is larger)
int64_t wgrad_partial_bytes(int64_t batch, int a, int b, int c, int d, int dtype)
{
    const int64_t p0 = wgrad_partial_floats(batch, a, b, c, d, dtype);
    const int64_t p1 = wgrad_partial_floats(padded_batch(batch), a, b, c, d, dtype);
    return align256((p0 > p1 ? p0 : p1) * 4);
}

// Bytes of the transposed copies of dY and X a batch-size-first weight gradient reduces (0: the
// problem is batch-size-last, or its padded copies would pass the size limit and the tiled
// kernel takes it as it is).
int64_t wgrad_transposed_bytes(int64_t batch, int a, int b, int c, int d, int dtype, int bs_last)
{
    if (bs_last) return 0;
    const int64_t bp = padded_batch(batch);
    if (check_shape(bp, a, b, c, d, dtype, dtype, dtype) != KSMM_OK) return 0;
    const int64_t es = (int64_t)dtype_size(dtype);
    return align256((int64_t)a * b * d * bp * es) + align256((int64_t)a * c * d * bp * es);
}

bool overlaps(const void *p, int64_t p_bytes, const void *q, int64_t q_bytes)
{
    const char *pb = (const char *)p, *qb = (const char *)q;
    return pb < qb + q_bytes && qb < pb + p_bytes;
}


int check_epilogue(const ksmm_epilogue *ep)
{
    if (!ep) return KSMM_OK;
    if (ep->act != KSMM_ACT_NONE && ep->act != KSMM_ACT_GELU) return KSMM_ERR_BAD_EPILOGUE;
    return KSMM_OK;
}

int factor_forward_impl(const void *x, const void *w, void *y, int64_t batch, int a, int b, int c, int d,
                        int x_dtype, int w_dtype, int y_dtype, int bs_last, float scale, int algo, int variant,
                        const ksmm_epilogue *ep, void *stream)
{
    int rc = check_shape(batch, a, b, c, d, x_dtype, w_dtype, y_dtype);
    if (rc != KSMM_OK) return rc;
    if ((rc = check_epilogue(ep)) != KSMM_OK) return rc;
    if (!x || !w || !y) return KSMM_ERR_NULL_POINTER;
    const int64_t xbytes = (int64_t)a * c * d * batch * (int64_t)dtype_size(x_dtype);
    const int64_t ybytes = (int64_t)a * b * d * batch * (int64_t)dtype_size(y_dtype);
    if (overlaps(x, xbytes, y, ybytes)) return KSMM_ERR_ALIAS;
    Problem p{x, w, y, batch, a, b, c, d, x_dtype, w_dtype, y_dtype, bs_last ? 1 : 0, scale,
              (hipStream_t)stream};
    if (ep) {
        p.bias = ep->bias;
        p.act = ep->act;
    }
    // Every kernel but the one-thread-per-output one moves 16-byte vectors: tensors that do not
    // start on a 16-byte boundary run on that kernel (a forced family refuses them).
    if ((((uintptr_t)x | (uintptr_t)w | (uintptr_t)y | (uintptr_t)p.bias) & 15) != 0) {
        if (algo != KSMM_ALGO_AUTO && !(algo == KSMM_ALGO_GENERIC && variant <= 0)) return KSMM_ERR_BAD_ALGO;
        return generic_run(p, 0, true, nullptr);
    }
    return dispatch(p, algo, variant, true, nullptr);
}

int factor_forward_ws_impl(const void *x, const void *w, void *y, int64_t batch, int a, int b, int c, int d,
                           int x_dtype, int w_dtype, int y_dtype, int bs_last, float scale,
                           const ksmm_epilogue *ep, void *workspace, int64_t workspace_bytes, void *stream)
{
    const int64_t need = ksmm_factor_workspace(batch, a, b, c, d, x_dtype, w_dtype, y_dtype, bs_last);
    if (need < 0) return (int)need;
    if (need == 0)
        return factor_forward_impl(x, w, y, batch, a, b, c, d, x_dtype, w_dtype, y_dtype, bs_last, scale,
                                   KSMM_ALGO_AUTO, -1, ep, stream);
    if (!x || !w || !y) return KSMM_ERR_NULL_POINTER;
    if (!workspace || workspace_bytes < need) return KSMM_ERR_WORKSPACE;
    const int64_t in_size = (int64_t)a * c * d, out_size = (int64_t)a * b * d;
    const int64_t xbytes = in_size * batch * (int64_t)dtype_size(x_dtype);
    const int64_t ybytes = out_size * batch * (int64_t)dtype_size(y_dtype);
    if (overlaps(x, xbytes, y, ybytes) || overlaps(workspace, need, x, xbytes) || overlaps(workspace, need, y, ybytes))
        return KSMM_ERR_ALIAS;
    if (((uintptr_t)workspace & 15) != 0) return KSMM_ERR_WORKSPACE;
    if (bs_last) {
        // rows padded to the vector (see wants_padded)
        const int64_t bp = padded_batch(batch);
        char *xp = (char *)workspace;
        char *yp = xp + align256(in_size * bp * (int64_t)dtype_size(x_dtype));
        int rc = repitch_run(x, xp, in_size, batch, bp, (int)dtype_size(x_dtype), (hipStream_t)stream);
        if (rc != KSMM_OK) return rc;
        rc = factor_forward_impl(xp, w, yp, bp, a, b, c, d, x_dtype, w_dtype, y_dtype, 1, scale, KSMM_ALGO_AUTO, -1,
                                 ep, stream);
        if (rc != KSMM_OK) return rc;
        return repitch_run(yp, y, out_size, bp, batch, (int)dtype_size(y_dtype), (hipStream_t)stream);
    }
    // transposed copies with rows of bp columns (bp = batch when that is a multiple of 16)
    const int64_t bp = padded_batch(batch);
    char *xt = (char *)workspace;
    char *yt = xt + align256(in_size * bp * (int64_t)dtype_size(x_dtype));
    int rc = transpose_run(x, xt, batch, in_size, (int)dtype_size(x_dtype), (hipStream_t)stream, 0, bp);
    if (rc != KSMM_OK) return rc;
    rc = factor_forward_impl(xt, w, yt, bp, a, b, c, d, x_dtype, w_dtype, y_dtype, 1, scale, KSMM_ALGO_AUTO, -1,
                             ep, stream);
    if (rc != KSMM_OK) return rc;
    return transpose_run(yt, y, out_size, batch, (int)dtype_size(y_dtype), (hipStream_t)stream, bp, 0);
}

int check_chain(const ksmm_factor_desc *f, int n, int64_t batch, int x_dtype, int y_dtype)
{
    if (!f) return KSMM_ERR_NULL_POINTER;
    if (n < 1 || n > KSMM_MAX_FACTORS) return KSMM_ERR_BAD_CHAIN;
    for (int i = 0; i < n; ++i) {
        // the first factor reads x_dtype, later ones read the intermediate type y_dtype
        int rc = check_shape(batch, f[i].a, f[i].b, f[i].c, f[i].d, i == 0 ? x_dtype : y_dtype,
                             f[i].w_dtype, y_dtype);
        if (rc != KSMM_OK) return rc;
        if (i > 0 && (int64_t)f[i].a * f[i].c * f[i].d != (int64_t)f[i - 1].a * f[i - 1].b * f[i - 1].d)
            return KSMM_ERR_CHAIN_MISMATCH;
    }
    return KSMM_OK;
}

// batch-size-first chain with at least one factor that needs the transposed route
bool chain_wants_transposed(const ksmm_factor_desc *f, int n, int64_t batch, int x_dtype, int y_dtype,
                            int bs_last)
{
    if (bs_last) return false;
    // a chain the fused kernel takes in batch-size-last layout: one pass over the data between two
    // transposes instead of one pass per factor
    if (chain16_run(f, n, nullptr, nullptr, padded_batch(batch), x_dtype, y_dtype, 1, false, nullptr, nullptr) == KSMM_OK)
        return true;
    for (int i = 0; i < n; ++i) {
        Problem p{nullptr, nullptr, nullptr, batch, f[i].a, f[i].b, f[i].c, f[i].d, i == 0 ? x_dtype : y_dtype,
                  f[i].w_dtype, y_dtype, 0, 1.f, nullptr};
        if (wants_transposed(p)) return true;
    }
    return false;
}

// batch-size-last chain whose batch is not a multiple of the vector, with at least one factor
// that has a real kernel at the padded batch
bool chain_wants_padded(const ksmm_factor_desc *f, int n, int64_t batch, int x_dtype, int y_dtype, int bs_last)
{
    if (!bs_last || batch % 16 == 0) return false;
    for (int i = 0; i < n; ++i) {
        Problem p{nullptr, nullptr, nullptr, batch, f[i].a, f[i].b, f[i].c, f[i].d, i == 0 ? x_dtype : y_dtype,
                  f[i].w_dtype, y_dtype, 1, 1.f, nullptr};
        if (wants_padded(p)) return true;
    }
    return false;
}

// The chain launcher behind ksmm_chain_forward, ksmm_chain_forward_ep and
// ksmm_chain_forward_static: `ep` (may be null) belongs to the last factor.
int chain_forward_impl(const ksmm_factor_desc *factors, int n_factors, const void *x, void *y, void *workspace,
                       int64_t workspace_bytes, int64_t batch, int x_dtype, int y_dtype, int bs_last, int fuse,
                       const ksmm_epilogue *ep, void *stream)
{
    int rc = check_chain(factors, n_factors, batch, x_dtype, y_dtype);
    if (rc != KSMM_OK) return rc;
    if ((rc = check_epilogue(ep)) != KSMM_OK) return rc;
    if (!x || !y) return KSMM_ERR_NULL_POINTER;
    for (int i = 0; i < n_factors; ++i)
        if (!factors[i].w) return KSMM_ERR_NULL_POINTER;
    const ksmm_factor_desc &last = factors[n_factors - 1];
    const int64_t in0 = (int64_t)factors[0].a * factors[0].c * factors[0].d;
    const int64_t out_n = (int64_t)last.a * last.b * last.d;
    const int64_t xbytes = in0 * batch * (int64_t)dtype_size(x_dtype);
    const int64_t ybytes = out_n * batch * (int64_t)dtype_size(y_dtype);
    if (overlaps(x, xbytes, y, ybytes)) return KSMM_ERR_ALIAS;
    if (workspace && workspace_bytes > 0) {
        if (overlaps(workspace, workspace_bytes, x, xbytes) || overlaps(workspace, workspace_bytes, y, ybytes))
            return KSMM_ERR_ALIAS;
        if (((uintptr_t)workspace & 15) != 0) return KSMM_ERR_WORKSPACE;
    }
    auto ep_of = [&](int i) { return i == n_factors - 1 ? ep : nullptr; };
    // The whole chain in batch-size-last layout on workspace buffers: input x0 (nb columns), two
    // ping-pong buffers of `one` bytes at pp; *result = where the last factor's output is.
    auto run_bs_last = [&](const void *x0, char *pp, int64_t one, int64_t nb, const void **result) -> int {
        int rc2 = KSMM_ERR_BAD_ALGO;
        if (fuse)
            rc2 = chain16_run(factors, n_factors, x0, pp, nb, x_dtype, y_dtype, 1, true, (hipStream_t)stream, ep);
        if (rc2 == KSMM_OK) {
            *result = pp;
            return KSMM_OK;
        }
        if (rc2 != KSMM_ERR_BAD_ALGO) return rc2;
        const void *cur = x0;
        int cur_dtype = x_dtype;
        for (int i = 0; i < n_factors; ++i) {
            void *dst = pp + (i & 1) * one;
            rc2 = factor_forward_impl(cur, factors[i].w, dst, nb, factors[i].a, factors[i].b, factors[i].c,
                                      factors[i].d, cur_dtype, factors[i].w_dtype, y_dtype, 1, factors[i].scale,
                                      KSMM_ALGO_AUTO, -1, ep_of(i), stream);
            if (rc2 != KSMM_OK) return rc2;
            cur = dst;
            cur_dtype = y_dtype;
        }
        *result = cur;
        return KSMM_OK;
    };
    if (chain_wants_transposed(factors, n_factors, batch, x_dtype, y_dtype, bs_last)) {
        // transpose once, run the whole chain in batch-size-last layout, transpose back
        // (a workspace below what ksmm_chain_workspace_layout() asks for is an error, as it is for
        // ksmm_factor_forward_ws: the factor-by-factor route would land on the one-thread-per-output
        // kernel without a word)
        const int64_t need_t = ksmm_chain_workspace_layout(factors, n_factors, batch, x_dtype, y_dtype, 0);
        if (!workspace || workspace_bytes < need_t) return KSMM_ERR_WORKSPACE;
        {
            const int64_t bp = padded_batch(batch);  // row length of the transposed copies
            const int64_t xt_bytes = align256(in0 * bp * (int64_t)dtype_size(x_dtype));
            char *xt = (char *)workspace;
            rc = transpose_run(x, xt, batch, in0, (int)dtype_size(x_dtype), (hipStream_t)stream, 0, bp);
            if (rc != KSMM_OK) return rc;
            const void *cur = nullptr;
            rc = run_bs_last(xt, xt + xt_bytes, (need_t - xt_bytes) / 2, bp, &cur);
            if (rc != KSMM_OK) return rc;
            return transpose_run(cur, y, out_n, batch, (int)dtype_size(y_dtype), (hipStream_t)stream, bp, 0);
        }
    } else if (chain_wants_padded(factors, n_factors, batch, x_dtype, y_dtype, bs_last)) {
        // pad the rows once, run the whole chain at the padded batch, cut the result rows back
        const int64_t need_p = ksmm_chain_workspace_layout(factors, n_factors, batch, x_dtype, y_dtype, 1);
        if (!workspace || workspace_bytes < need_p) return KSMM_ERR_WORKSPACE;
        {
            const int64_t bp = padded_batch(batch);
            const int64_t xp_bytes = align256(in0 * bp * (int64_t)dtype_size(x_dtype));
            char *xp = (char *)workspace;
            rc = repitch_run(x, xp, in0, batch, bp, (int)dtype_size(x_dtype), (hipStream_t)stream);
            if (rc != KSMM_OK) return rc;
            const void *cur = nullptr;
            rc = run_bs_last(xp, xp + xp_bytes, (need_p - xp_bytes) / 2, bp, &cur);
            if (rc != KSMM_OK) return rc;
            return repitch_run(cur, y, out_n, bp, batch, (int)dtype_size(y_dtype), (hipStream_t)stream);
        }
    }
    if (fuse) {
        // chains whose intermediates fit LDS run as one kernel (no workspace traffic)
        rc = chain16_run(factors, n_factors, x, y, batch, x_dtype, y_dtype, bs_last ? 1 : 0, true,
                         (hipStream_t)stream, ep);
        if (rc != KSMM_ERR_BAD_ALGO) return rc;
    }
    const int64_t need = ksmm_chain_workspace(factors, n_factors, batch, y_dtype);
    if (n_factors > 1 && (!workspace || workspace_bytes < need)) return KSMM_ERR_WORKSPACE;
    char *buf[2] = {(char *)workspace, (char *)workspace + need / 2};
    const void *cur = x;
    int cur_dtype = x_dtype;
    for (int i = 0; i < n_factors; ++i) {
        void *dst = (i == n_factors - 1) ? y : (void *)buf[i & 1];
        rc = factor_forward_impl(cur, factors[i].w, dst, batch, factors[i].a, factors[i].b, factors[i].c,
                                 factors[i].d, cur_dtype, factors[i].w_dtype, y_dtype, bs_last, factors[i].scale,
                                 KSMM_ALGO_AUTO, -1, ep_of(i), stream);
        if (rc != KSMM_OK) return rc;
        cur = dst;
        cur_dtype = y_dtype;
    }
    return KSMM_OK;
}

// ---- scratch of ksmm_chain_forward_static ---------------------------------------------------
// The device address of the array is asked for once per device, with that device current, and
// kept; kernels and copies only ever see that address.
constexpr int MAX_DEVICES = 64;
std::atomic<void *> scratch_ptr[MAX_DEVICES];

int static_scratch(void **out)
{
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= MAX_DEVICES) return KSMM_ERR_LAUNCH;
    void *ptr = scratch_ptr[dev].load(std::memory_order_acquire);
    if (!ptr) {
        if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)) != hipSuccess || !ptr) return KSMM_ERR_LAUNCH;
        scratch_ptr[dev].store(ptr, std::memory_order_release);  // racing callers store the same address
    }
    *out = ptr;
    return KSMM_OK;
}

}  // namespace

extern "C" {

int ksmm_version(void) { return KSMM_VERSION; }

const char *ksmm_strerror(int status)
{
    switch (status) {
    case KSMM_OK: return "ok";
    case KSMM_ERR_NULL_POINTER: return "null tensor pointer";
    case KSMM_ERR_BAD_PATTERN: return "pattern (a,b,c,d) must be four positive integers";
    case KSMM_ERR_BAD_BATCH: return "batch size must be positive";
    case KSMM_ERR_BAD_DTYPE: return "unsupported data type combination";
    case KSMM_ERR_TOO_LARGE: return "tensor too large (2^31 elements or more)";
    case KSMM_ERR_BAD_ALGO: return "kernel family/variant unknown or not applicable to this problem";
    case KSMM_ERR_LAUNCH: return "HIP kernel launch failed";
    case KSMM_ERR_CHAIN_MISMATCH: return "consecutive factors have incompatible sizes";
    case KSMM_ERR_WORKSPACE: return "workspace missing or too small";
    case KSMM_ERR_BAD_CHAIN: return "bad number of factors";
    case KSMM_ERR_ALIAS: return "output, input or workspace overlap";
    case KSMM_ERR_BAD_EPILOGUE: return "unknown activation in the epilogue";
    default: return "unknown ksmm status";
    }
}

int ksmm_validate(int64_t batch, int a, int b, int c, int d, int x_dtype, int w_dtype,
                  int y_dtype, int bs_last)
{
    (void)bs_last;
    return check_shape(batch, a, b, c, d, x_dtype, w_dtype, y_dtype);
}

int ksmm_query_tile(int64_t batch, int a, int b, int c, int d, int x_dtype, int w_dtype,
                    int y_dtype, int bs_last, int algo, ksmm_tile *out)
{
    if (!out) return KSMM_ERR_NULL_POINTER;
    int rc = check_shape(batch, a, b, c, d, x_dtype, w_dtype, y_dtype);
    if (rc != KSMM_OK) return rc;
    Problem p{nullptr, nullptr, nullptr, batch, a, b, c, d, x_dtype, w_dtype, y_dtype,
              bs_last ? 1 : 0, 1.f, nullptr};
    memset(out, 0, sizeof(*out));
    return dispatch(p, algo, -1, false, out);
}

int ksmm_query_tile_variant(int64_t batch, int a, int b, int c, int d, int x_dtype, int w_dtype,
                            int y_dtype, int bs_last, int algo, int variant, ksmm_tile *out)
{
    if (!out) return KSMM_ERR_NULL_POINTER;
    int rc = check_shape(batch, a, b, c, d, x_dtype, w_dtype, y_dtype);
    if (rc != KSMM_OK) return rc;
    Problem p{nullptr, nullptr, nullptr, batch, a, b, c, d, x_dtype, w_dtype, y_dtype,
              bs_last ? 1 : 0, 1.f, nullptr};
    memset(out, 0, sizeof(*out));
    return dispatch(p, algo, variant, false, out);
}

int ksmm_tuned_count(void) { return N_TUNED; }

int ksmm_tuned_row(int index, int row[10])
{
    if (!row) return KSMM_ERR_NULL_POINTER;
    if (index < 0 || index >= N_TUNED) return KSMM_ERR_BAD_ALGO;
    const TunedRow &r = tuned_rows[index];
    int variant = -1;  // the row's instance is gone from the library: the heuristics serve the pattern
    if (!resolve_variant(r.algo, r.id, r.param, r.combo, r.bs_last, &variant)) variant = -1;
    const int v[10] = {r.a, r.b, r.c, r.d, r.combo, r.bs_last, r.algo, (int)r.id, r.param, variant};
    for (int i = 0; i < 10; ++i) row[i] = v[i];
    return KSMM_OK;
}

int ksmm_variant_id(int algo, int variant, int x_dtype, int w_dtype, int y_dtype, int bs_last,
                    uint32_t *id, int *param)
{
    if (!id || !param) return KSMM_ERR_NULL_POINTER;
    const int combo = combo_of(x_dtype, w_dtype, y_dtype);
    if (combo < 0) return KSMM_ERR_BAD_DTYPE;
    return describe_variant(algo, variant, combo, bs_last ? 1 : 0, id, param) ? KSMM_OK : KSMM_ERR_BAD_ALGO;
}

int ksmm_variant_from_id(int algo, uint32_t id, int param, int x_dtype, int w_dtype, int y_dtype,
                         int bs_last, int *variant)
{
    if (!variant) return KSMM_ERR_NULL_POINTER;
    const int combo = combo_of(x_dtype, w_dtype, y_dtype);
    if (combo < 0) return KSMM_ERR_BAD_DTYPE;
    return resolve_variant(algo, id, param, combo, bs_last ? 1 : 0, variant) ? KSMM_OK : KSMM_ERR_BAD_ALGO;
}

int ksmm_factor_forward_algo(const void *x, const void *w, void *y, int64_t batch, int a,
                             int b, int c, int d, int x_dtype, int w_dtype, int y_dtype,
                             int bs_last, float scale, int algo, int variant, void *stream)
{
    return factor_forward_impl(x, w, y, batch, a, b, c, d, x_dtype, w_dtype, y_dtype, bs_last, scale, algo,
                               variant, nullptr, stream);
}

int ksmm_factor_forward(const void *x, const void *w, void *y, int64_t batch, int a, int b,
                        int c, int d, int x_dtype, int w_dtype, int y_dtype, int bs_last,
                        float scale, void *stream)
{
    return factor_forward_impl(x, w, y, batch, a, b, c, d, x_dtype, w_dtype, y_dtype, bs_last, scale,
                               KSMM_ALGO_AUTO, -1, nullptr, stream);
}

int64_t ksmm_factor_workspace(int64_t batch, int a, int b, int c, int d, int x_dtype, int w_dtype,
                              int y_dtype, int bs_last)
{
    int rc = check_shape(batch, a, b, c, d, x_dtype, w_dtype, y_dtype);
    if (rc != KSMM_OK) return rc;
    Problem p{nullptr, nullptr, nullptr, batch, a, b, c, d, x_dtype, w_dtype, y_dtype,
              bs_last ? 1 : 0, 1.f, nullptr};
    // both routes stage the input and the output: transposed, or with rows padded to the vector
    const int64_t nb = wants_transposed(p) || wants_padded(p) ? padded_batch(batch) : 0;
    if (nb == 0) return 0;
    return align256((int64_t)a * c * d * nb * (int64_t)dtype_size(x_dtype)) +
           align256((int64_t)a * b * d * nb * (int64_t)dtype_size(y_dtype));
}

int ksmm_factor_forward_ws(const void *x, const void *w, void *y, int64_t batch, int a, int b,
                           int c, int d, int x_dtype, int w_dtype, int y_dtype, int bs_last,
                           float scale, void *workspace, int64_t workspace_bytes, void *stream)
{
    return factor_forward_ws_impl(x, w, y, batch, a, b, c, d, x_dtype, w_dtype, y_dtype, bs_last, scale, nullptr,
                                  workspace, workspace_bytes, stream);
}

int ksmm_factor_forward_ep(const void *x, const void *w, void *y, int64_t batch, int a, int b,
                           int c, int d, int x_dtype, int w_dtype, int y_dtype, int bs_last,
                           float scale, const ksmm_epilogue *epilogue, void *workspace,
                           int64_t workspace_bytes, void *stream)
{
    return factor_forward_ws_impl(x, w, y, batch, a, b, c, d, x_dtype, w_dtype, y_dtype, bs_last, scale, epilogue,
                                  workspace, workspace_bytes, stream);
}

int64_t ksmm_chain_workspace(const ksmm_factor_desc *factors, int n_factors, int64_t batch,
                             int y_dtype)
{
    if (!factors) return KSMM_ERR_NULL_POINTER;
    if (n_factors < 1 || n_factors > KSMM_MAX_FACTORS) return KSMM_ERR_BAD_CHAIN;
    if (batch < 1) return KSMM_ERR_BAD_BATCH;
    if (!dtype_known(y_dtype)) return KSMM_ERR_BAD_DTYPE;
    int64_t widest = 0;
    for (int i = 0; i + 1 < n_factors; ++i) {
        if (factors[i].a < 1 || factors[i].b < 1 || factors[i].d < 1) return KSMM_ERR_BAD_PATTERN;
        int64_t o = (int64_t)factors[i].a * factors[i].b * factors[i].d;
        if (o > widest) widest = o;
    }
    // two buffers, each rounded up to 256 bytes so that both stay 256-byte aligned
    int64_t one = (widest * batch * (int64_t)dtype_size(y_dtype) + 255) / 256 * 256;
    return n_factors > 1 ? 2 * one : 0;
}

int64_t ksmm_chain_workspace_layout(const ksmm_factor_desc *factors, int n_factors, int64_t batch,
                                    int x_dtype, int y_dtype, int bs_last)
{
    int rc = check_chain(factors, n_factors, batch, x_dtype, y_dtype);
    if (rc != KSMM_OK) return rc;
    const int64_t nb = chain_wants_transposed(factors, n_factors, batch, x_dtype, y_dtype, bs_last) ||
                               chain_wants_padded(factors, n_factors, batch, x_dtype, y_dtype, bs_last)
                           ? padded_batch(batch) : 0;
    if (nb == 0) return ksmm_chain_workspace(factors, n_factors, batch, y_dtype);
    int64_t widest = 0;
    for (int i = 0; i < n_factors; ++i) {
        int64_t o = (int64_t)factors[i].a * factors[i].b * factors[i].d;
        if (o > widest) widest = o;
    }
    const int64_t in0 = (int64_t)factors[0].a * factors[0].c * factors[0].d;
    return align256(in0 * nb * (int64_t)dtype_size(x_dtype)) +
           2 * align256(widest * nb * (int64_t)dtype_size(y_dtype));
}

int ksmm_chain_forward(const ksmm_factor_desc *factors, int n_factors, const void *x, void *y,
                       void *workspace, int64_t workspace_bytes, int64_t batch, int x_dtype,
                       int y_dtype, int bs_last, int fuse, void *stream)
{
    return chain_forward_impl(factors, n_factors, x, y, workspace, workspace_bytes, batch, x_dtype, y_dtype,
                              bs_last, fuse, nullptr, stream);
}

int ksmm_chain_forward_ep(const ksmm_factor_desc *factors, int n_factors, const void *x, void *y,
                          void *workspace, int64_t workspace_bytes, int64_t batch, int x_dtype,
                          int y_dtype, int bs_last, int fuse, const ksmm_epilogue *epilogue,
                          void *stream)
{
    return chain_forward_impl(factors, n_factors, x, y, workspace, workspace_bytes, batch, x_dtype, y_dtype,
                              bs_last, fuse, epilogue, stream);
}

int64_t ksmm_factor_backward_workspace(int64_t batch, int a, int b, int c, int d, int dtype, int bs_last)
{
    int rc = check_shape(batch, a, b, c, d, dtype, dtype, dtype);
    if (rc != KSMM_OK) return rc;
    if (dtype != KSMM_F32 && dtype != KSMM_F16) return KSMM_ERR_BAD_DTYPE;
    const int64_t nnz = (int64_t)a * b * c * d;
    // transposed blocks (input gradient) | fp32 partial sums, one slice per batch split (weight
    // gradient) | what the forward kernels of the transposed factor ask for
    const int64_t fwd = ksmm_factor_workspace(batch, a, c, b, d, dtype, dtype, dtype, bs_last);
    if (fwd < 0) return fwd;
    return align256(nnz * (int64_t)dtype_size(dtype)) + wgrad_partial_bytes(batch, a, b, c, d, dtype) + align256(fwd) +
           wgrad_transposed_bytes(batch, a, b, c, d, dtype, bs_last);
}

int ksmm_factor_backward_input(const void *dy, const void *w, void *dx, int64_t batch, int a, int b,
                               int c, int d, int dtype, int bs_last, float scale, void *workspace,
                               int64_t workspace_bytes, void *stream)
{
    const int64_t need = ksmm_factor_backward_workspace(batch, a, b, c, d, dtype, bs_last);
    if (need < 0) return (int)need;
    if (!dy || !w || !dx) return KSMM_ERR_NULL_POINTER;
    if (!workspace || workspace_bytes < need || ((uintptr_t)workspace & 15) != 0) return KSMM_ERR_WORKSPACE;
    const int64_t nnz = (int64_t)a * b * c * d;
    char *wt = (char *)workspace;
    char *fwd_ws = wt + align256(nnz * (int64_t)dtype_size(dtype)) + wgrad_partial_bytes(batch, a, b, c, d, dtype);
    int rc = block_transpose_run(w, wt, a, b, c, d, dtype, (hipStream_t)stream);
    if (rc != KSMM_OK) return rc;
    // dX = K^T dY: the factor with pattern (a, c, b, d) and transposed blocks
    return factor_forward_ws_impl(dy, wt, dx, batch, a, c, b, d, dtype, dtype, dtype, bs_last, scale, nullptr, fwd_ws,
                                  workspace_bytes - (fwd_ws - wt), stream);
}

int ksmm_factor_backward_weight(const void *dy, const void *x, void *dw, int64_t batch, int a, int b,
                                int c, int d, int dtype, int bs_last, float scale, void *workspace,
                                int64_t workspace_bytes, void *stream)
{
    const int64_t need = ksmm_factor_backward_workspace(batch, a, b, c, d, dtype, bs_last);
    if (need < 0) return (int)need;
    if (!dy || !x || !dw) return KSMM_ERR_NULL_POINTER;
    if (!workspace || workspace_bytes < need || ((uintptr_t)workspace & 15) != 0) return KSMM_ERR_WORKSPACE;
    const int64_t nnz = (int64_t)a * b * c * d;
    float *acc = (float *)((char *)workspace + align256(nnz * (int64_t)dtype_size(dtype)));
    if (!bs_last && wgrad_transposed_bytes(batch, a, b, c, d, dtype, 0) > 0) {
        // Batch-size-first: the operands of one block are d elements apart along the features, and
        // the sum runs over the rows.  Both operands are transposed once into the workspace (rows
        // padded to 16 columns, the padding cleared) and the batch-size-last kernel reduces them.
        const int64_t es = (int64_t)dtype_size(dtype), bp = padded_batch(batch);
        const int64_t fwd = ksmm_factor_workspace(batch, a, c, b, d, dtype, dtype, dtype, 0);
        char *tdy = (char *)acc + wgrad_partial_bytes(batch, a, b, c, d, dtype) + align256(fwd);
        char *tx = tdy + align256((int64_t)a * b * d * bp * es);
        int rc = transpose_run(dy, tdy, batch, (int64_t)a * b * d, (int)es, (hipStream_t)stream, 0, bp);
        if (rc == KSMM_OK) rc = zero_pad_run(tdy, (int64_t)a * b * d, batch, bp, (int)es, (hipStream_t)stream);
        if (rc == KSMM_OK) rc = transpose_run(x, tx, batch, (int64_t)a * c * d, (int)es, (hipStream_t)stream, 0, bp);
        if (rc == KSMM_OK) rc = zero_pad_run(tx, (int64_t)a * c * d, batch, bp, (int)es, (hipStream_t)stream);
        if (rc != KSMM_OK) return rc;
        return wgrad_run(tdy, tx, dw, acc, bp, a, b, c, d, dtype, 1, scale, (hipStream_t)stream, nullptr);
    }
    return wgrad_run(dy, x, dw, acc, batch, a, b, c, d, dtype, bs_last ? 1 : 0, scale, (hipStream_t)stream, nullptr);
}

int64_t ksmm_static_scratch_bytes(void) { return KSMM_STATIC_SCRATCH_BYTES; }

int ksmm_chain_forward_static(const ksmm_factor_desc *factors, int n_factors, const void *x, void *y,
                              int64_t batch, int x_dtype, int y_dtype, int bs_last, int fuse,
                              const ksmm_epilogue *epilogue, void *stream)
{
    // what the chain would ask a caller to lend (0 when it needs no scratch at all)
    const int64_t need = ksmm_chain_workspace_layout(factors, n_factors, batch, x_dtype, y_dtype, bs_last);
    if (need < 0) return (int)need;
    if (need > KSMM_STATIC_SCRATCH_BYTES) return KSMM_ERR_WORKSPACE;
    void *buf = nullptr;
    if (need > 0) {
        const int rc = static_scratch(&buf);
        if (rc != KSMM_OK) return rc;
    }
    return chain_forward_impl(factors, n_factors, x, y, buf, need > 0 ? KSMM_STATIC_SCRATCH_BYTES : 0, batch,
                              x_dtype, y_dtype, bs_last, fuse, epilogue, stream);
}

}  // extern "C"
